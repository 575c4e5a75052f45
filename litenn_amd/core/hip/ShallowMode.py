class ShallowMode:
    """While at least one instance is entered, launches, copies and fills are
    skipped and no device memory is touched: shapes and the autograd graph
    still flow (counterpart of CLShallowMode.py:2-14)."""
    stack_count = 0

    def __enter__(self):
        ShallowMode.stack_count += 1
        return self

    def __exit__(self, *exc):
        ShallowMode.stack_count -= 1
        if ShallowMode.stack_count < 0:
            raise ValueError('Wrong stack_count.')

    @staticmethod
    def active():
        return ShallowMode.stack_count > 0
