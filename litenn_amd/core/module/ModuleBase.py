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
    # Layout of the flat state dict (what ModuleBase.py:131-199 writes, so files are interchangeable):
    #   tensor      '<owner path>.<attr>'          -> ('np.ndarray', array)        owner path relative to the saved
    #                                                                              module, '' for itself: '.kernel'
    #   int, float, complex, str (bool included)
    #               '<owner path>.<attr>' without a leading dot -> ('python-var', (class name, value))
    #   list        '<owner path>.<attr>__len' without a leading dot -> bare int; elements follow as '<attr>[i]'
    #   dict        elements as '<attr>[key]'; nothing for the dict itself
    # Tuples, None, arrays and anything else are not part of the state.
    def _visit_state(self, visit):
        """Calls visit(kind, name, obj, setter) for every saveable leaf under this module; for kind 'list' the
        return value says whether to descend into the elements."""
        top = self

        def walk(owner, obj, attr, setter):
            if isinstance(obj, ModuleBase):
                keep = getattr(obj, '_saveables', None)
                for var in list(vars(obj)):
                    if (var not in keep) if keep is not None else var[0] == '_':
                        continue
                    walk(obj, getattr(obj, var), var, lambda v, o=obj, n=var: setattr(o, n, v))
            elif isinstance(obj, nn.Tensor):
                visit('tensor', obj.get_name(top), obj, None)
            elif isinstance(obj, list):
                name = f'{owner.get_name(top)}.{attr}'.lstrip('.')
                if visit('list', name, obj, None):
                    for i, el in enumerate(obj):
                        walk(owner, el, f'{attr}[{i}]', lambda v, o=obj, k=i: o.__setitem__(k, v))
            elif isinstance(obj, dict):
                for k in list(obj):
                    walk(owner, obj[k], f'{attr}[{k}]', lambda v, o=obj, k=k: o.__setitem__(k, v))
            elif isinstance(obj, (int, float, complex, str)):
                visit('var', f'{owner.get_name(top)}.{attr}'.lstrip('.'), obj, setter)

        walk(None, self, None, None)

    def dump_state(self):
        """{name: ('np.ndarray', array) | ('python-var', (class name, value)) | list length}."""
        state = {}

        def visit(kind, name, obj, setter):
            if kind == 'tensor':
                state[name] = ('np.ndarray', obj.np())
            elif kind == 'list':
                state[name + '__len'] = len(obj)
            else:
                state[name] = ('python-var', (obj.__class__.__name__, obj))
            return True

        self._visit_state(visit)
        return state

    def load_state(self, state_dict):
        """Restores what matches by name, kind and shape / class; everything else only warns
        (ModuleBase.py:146-199).  A list whose saved length differs is skipped with all its elements."""
        def visit(kind, name, obj, setter):
            if kind == 'list':
                saved = state_dict.get(name + '__len', None)
                if saved is None or saved != len(obj):
                    log.warning(f'List {name} is not loaded, because length of list {len(obj)} != saved list len {saved}')
                    return False
                return True
            what = 'Tensor' if kind == 'tensor' else 'Variable'
            entry = state_dict.get(name, None)
            if entry is None:
                log.warning(f'{what} {name} is not loaded, because saved data is not found.')
                return True
            saved_kind, value = entry
            if kind == 'tensor':
                if saved_kind != 'np.ndarray':
                    log.warning(f'Tensor {name} is not loaded, because saved type is {saved_kind}, but must be np.ndarray')
                elif tuple(obj.shape) != value.shape:
                    log.warning(f'Tensor {name} is not loaded, because saved Tensor shape is {value.shape}, '
                                f'but must be {tuple(obj.shape)}')
                else:
                    obj.set(value)
            elif saved_kind != 'python-var':
                log.warning(f'Variable {name} is not loaded, because saved type is {saved_kind}, but must be python-var')
            else:
                class_name, value = value
                if class_name != obj.__class__.__name__:
                    log.warning(f'Variable {name} is not loaded, because saved class_name is {class_name}, '
                                f'but must be {obj.__class__.__name__}')
                else:
                    setter(value)
            return True

        self._visit_state(visit)

    def save(self, filepath):
        Path(filepath).write_bytes(pickle.dumps(self.dump_state(), 4))

    def load(self, filepath):
        """Loads a file written by save().  Returns False if it does not exist."""
        p = Path(filepath)
        if not p.exists():
            return False
        self.load_state(pickle.loads(p.read_bytes()))
        return True
