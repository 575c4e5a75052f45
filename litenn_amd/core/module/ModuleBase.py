import logging
import pickle
import weakref
from pathlib import Path

import numpy as np

import litenn_amd as nn

log = logging.getLogger('litenn')


class ModuleBase:
    """Common base of Module and Optimizer: hierarchical names for child
    tensors / modules and a flat state dict for save / load
    (same behaviour as ModuleBase.py:9-199 and Saveable.py:24-42).

    Attributes whose name starts with '_' are ignored unless listed in
    `saveables`.
    """

    def __init__(self, saveables=None):
        self._saveables = saveables

    # ---- naming -------------------------------------------------------------
    def get_name(self, top_parent=None):
        parts, module = [], self
        while module is not None and module is not top_parent:
            parent = module._get_parent_module()
            parts.append(parent._get_child_name(module) if parent is not None else module.__class__.__name__)
            module = parent
        return '.'.join(reversed(parts))

    def _get_parent_module(self):
        ref = getattr(self, '_parent_module_w', None)
        return ref() if ref is not None else None

    def _get_child_names(self):
        names = getattr(self, '_child_names', None)
        if names is None:
            names = {}
            object.__setattr__(self, '_child_names', names)
        return names

    def _get_child_name(self, child):
        return self._get_child_names().get(id(child), None)

    def __setattr__(self, name, obj):
        object.__setattr__(self, name, obj)
        if name[0] == '_':
            saveables = getattr(self, '_saveables', None)
            if saveables is None or name not in saveables:
                return
        ModuleBase._adopt(self, obj, name)

    @staticmethod
    def _adopt(parent, obj, name):
        if isinstance(obj, (nn.Tensor, ModuleBase)):
            if isinstance(obj, nn.Tensor):
                if obj._is_reference():
                    raise Exception('You cannot assign Reference Tensor to the Module')
                if obj._is_produced_by_op():
                    raise Exception('You cannot assign Tensor produced by operator to the Module')
                if obj._parent_module_w is not None:
                    raise Exception(f'Tensor {obj.get_name()} is already assigned to the Module.')
            object.__setattr__(obj, '_parent_module_w', weakref.ref(parent))
            parent._get_child_names()[id(obj)] = name
        elif isinstance(obj, list):
            if len(obj) == 0:
                raise Exception(f"Empty list '{name}' set to {parent.__class__.__name__}: dynamic lists are not "
                                'allowed (use an _internal name for unsaved ones).')
            for i, el in enumerate(obj):
                ModuleBase._adopt(parent, el, f'{name}[{i}]')
        elif isinstance(obj, dict):
            if len(obj) == 0:
                raise Exception(f"Empty dict '{name}' set to {parent.__class__.__name__}: dynamic dicts are not "
                                'allowed (use an _internal name for unsaved ones).')
            for key, el in obj.items():
                ModuleBase._adopt(parent, el, f'{name}[{key}]')
        elif isinstance(obj, set):
            raise Exception('You cannot assign sets to the Module')

    # ---- state --------------------------------------------------------------
    def _state_items(self, prefix=''):
        """Yields (dotted name, owner, key, value) for every saveable leaf."""
        saveables = getattr(self, '_saveables', None)
        for var in list(vars(self)):
            if saveables is not None:
                if var not in saveables:
                    continue
            elif var[0] == '_':
                continue
            yield from ModuleBase._walk(self.__dict__, var, getattr(self, var), f'{prefix}{var}')

    @staticmethod
    def _walk(owner, key, obj, name):
        if isinstance(obj, ModuleBase):
            yield from obj._state_items(name + '.')
        elif isinstance(obj, (list, tuple)):
            yield (name + '__len', None, None, len(obj))
            for i, el in enumerate(obj):
                yield from ModuleBase._walk(obj, i, el, f'{name}[{i}]')
        elif isinstance(obj, dict):
            for k, el in obj.items():
                yield from ModuleBase._walk(obj, k, el, f'{name}[{k}]')
        elif isinstance(obj, (nn.Tensor, int, float, str, bool, np.ndarray)) or obj is None:
            yield (name, owner, key, obj)

    def dump_state(self):
        """{dotted name: ('np.ndarray', array) | ('python-var', value)}."""
        state = {}
        for name, owner, key, obj in self._state_items():
            if isinstance(obj, nn.Tensor):
                state[name] = ('np.ndarray', obj.np())
            elif owner is None:
                state[name] = ('python-var', obj)
            else:
                state[name] = ('python-var', obj)
        return state

    def load_state(self, state_dict):
        """Restore what matches; mismatches only warn."""
        for name, owner, key, obj in self._state_items():
            if owner is None:
                if name in state_dict and state_dict[name][1] != obj:
                    log.warning(f'{name}: saved length {state_dict[name][1]} != current {obj}')
                continue
            if name not in state_dict:
                log.warning(f'{name} is not found in the saved state')
                continue
            kind, value = state_dict[name]
            if isinstance(obj, nn.Tensor):
                if kind != 'np.ndarray' or tuple(value.shape) != tuple(obj.shape):
                    log.warning(f'{name}: saved value does not fit tensor shape {obj.shape}')
                    continue
                obj.set(value)
            else:
                owner[key] = value

    def save(self, filepath):
        Path(filepath).write_bytes(pickle.dumps(self.dump_state(), 4))

    def load(self, filepath):
        """Loads a file written by save().  Returns False if it does not exist."""
        p = Path(filepath)
        if not p.exists():
            return False
        self.load_state(pickle.loads(p.read_bytes()))
        return True
