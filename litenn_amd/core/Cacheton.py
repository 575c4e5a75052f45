class Cacheton:
    """Process-wide memo of plan objects keyed by (class, args, kwargs) and of
    named variables; everything is dropped by nn.cleanup()
    (same contract as Cacheton.py:1-51)."""
    cachetons = {}
    cachevars = {}

    @staticmethod
    def get(cls, *args, **kwargs):
        """The instance of cls built from these (hashable) arguments, built on
        first request."""
        per_class = Cacheton.cachetons.setdefault(cls, {})
        key = (args, tuple(kwargs.items()))
        try:
            return per_class[key]
        except KeyError:
            obj = per_class[key] = cls(*args, **kwargs)
            return obj

    @staticmethod
    def set_var(var_name, value):
        Cacheton.cachevars[var_name] = value

    @staticmethod
    def get_var(var_name):
        return Cacheton.cachevars.get(var_name, None)

    @staticmethod
    def _cleanup():
        Cacheton.cachetons = {}
        Cacheton.cachevars = {}
