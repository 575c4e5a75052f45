import litenn_amd as nn
from .ModuleBase import ModuleBase


class Module(ModuleBase):
    """Base class of layers and models (same user contract as Module.py:7-152):
    holds tensors / sub-modules / python values as attributes, is callable
    (-> forward), lists its trainable tensors, carries a training flag.

     saveables    names of attributes to save (None: every public one)
     trainables   names returned by trainables() (None: same as saveables)

    Calling Module.__init__ from a subclass is optional.
    """

    def __init__(self, saveables=None, trainables=None):
        super().__init__(saveables=saveables)
        self._trainables = trainables

    def forward(self, *args, **kwargs):
        raise NotImplementedError()

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def shallow_forward(self, *args, **kwargs):
        """forward() without launching kernels or allocating device memory;
        useful to learn output shapes."""
        with nn.devices._shallow_mode():
            return self.forward(*args, **kwargs)

    def is_training(self):
        return getattr(self, '_tr', False)

    def set_training(self, is_training):
        Module._spread_training(self, is_training)

    def trainables(self):
        """Tensors of this module and its sub-modules, for an Optimizer."""
        names = getattr(self, '_trainables', None)
        if names is None:
            names = getattr(self, '_saveables', None)
        out = []
        for var in vars(self):
            if names is not None:
                if var not in names:
                    continue
            elif var[0] == '_':
                continue
            Module._collect(getattr(self, var), out)
        return out

    @staticmethod
    def _collect(obj, out):
        if isinstance(obj, Module):
            out.extend(obj.trainables())
        elif isinstance(obj, nn.Tensor):
            out.append(obj)
        elif isinstance(obj, list):
            for el in obj:
                Module._collect(el, out)
        elif isinstance(obj, dict):
            for el in obj.values():
                Module._collect(el, out)

    @staticmethod
    def _spread_training(obj, flag):
        if isinstance(obj, Module):
            object.__setattr__(obj, '_tr', flag)
            for var in list(vars(obj)):
                if var in ('_parent_module_w', '_child_names'):
                    continue
                Module._spread_training(getattr(obj, var), flag)
        elif isinstance(obj, list):
            for el in obj:
                Module._spread_training(el, flag)
        elif isinstance(obj, dict):
            for el in obj.values():
                Module._spread_training(el, flag)
