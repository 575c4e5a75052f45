import operator

import numpy as np

import litenn_amd as nn
import litenn_amd.core as nc

_seq = operator.methodcaller('_get_seq_id')

# Per-sweep state for gradient functions that share an intermediate result (the fused convolution epilogue forms
# its pre-activation gradient once for three gradient functions): a counter that identifies the running sweep
# (None outside one) and callbacks run when the gradient functions of the tensor being visited are done, so nothing
# computed from one sweep's gradients is reused by the next and nothing keeps gradient-sized tensors alive longer
# than their readers.
_sweep = {'id': 0, 'active': None, 'tensor_cleanups': []}


def current_sweep():
    """Identifier of the backward() call in progress, or None outside one."""
    return _sweep['active']


def after_gradfns_of_tensor(fn):
    """Call fn() once the gradient functions of the tensor the running backward() is visiting have all run (at once
    if no backward() is running): what they share - an intermediate formed by the first and read by the others -
    can be let go there instead of living until the sweep ends."""
    if _sweep['active'] is None:
        fn()
    else:
        _sweep['tensor_cleanups'].append(fn)


def _run_tensor_cleanups():
    fns, _sweep['tensor_cleanups'] = _sweep['tensor_cleanups'], []
    for fn in fns:
        fn()



def backward(loss, stop_grad=None, grad_for_non_trainables=False, keep_gradient_for_non_trainables=False):
    """Reverse-mode sweep (same observable behaviour as backward.py:8-158).

     loss        Tensor, list of Tensors, or {Tensor: np.ndarray initial gradient}
     stop_grad   None, Tensor or list of Tensors whose inputs are not visited
     grad_for_non_trainables
                 False: branches that reach no optimizer-attached tensor are
                 skipped, and gradients of non-attached tensors are dropped as
                 soon as they have been propagated.

    Tensors are visited in decreasing creation order; every registered
    gradient function adds into its input's gradient.
    """
    if _sweep['active'] is not None:
        raise Exception('backward() called from inside a gradient function')
    _sweep['id'] += 1
    _sweep['active'] = _sweep['id']
    try:
        _backward(loss, stop_grad, grad_for_non_trainables)
    finally:
        _run_tensor_cleanups()
        _sweep['active'] = None


def _backward(loss, stop_grad, grad_for_non_trainables):
    seeds = {}
    if isinstance(loss, dict):
        seeds = loss
        loss = list(loss.keys())
    elif not isinstance(loss, (tuple, list)):
        loss = [loss]
    if stop_grad is None:
        stop_grad = []
    elif not isinstance(stop_grad, (tuple, list)):
        stop_grad = [stop_grad]

    blocked = _untrainable_branches(loss) if not grad_for_non_trainables else {}
    for t in stop_grad:
        blocked[t._get_seq_id()] = []

    roots = [t for t in loss if t._get_seq_id() not in blocked]
    for t in roots:
        g = t.get_grad()
        fresh = all(not b.has_ptr() for b in g._get_buffers())   # still the implicit zeros: the seed may overwrite
        if t in seeds:
            if fresh and isinstance(seeds[t], np.ndarray) and seeds[t].size == g.shape.size:
                g.set(seeds[t])
            else:
                nc.op.add(g, nn.Tensor_from_value(seeds[t]), output_t=g)
        elif fresh:
            g.fill(1.0)
        else:
            nc.op.add_const(g, 1.0, output_t=g)

    pending = list({id(s): s for s in (t._get_top_reference_source() for t in roots)}.values())
    while pending:
        pending.sort(key=_seq)
        t = pending.pop()
        fns = t._get_gradfns()
        if fns is not None:
            for input_t, funcs in fns.items():
                if t._is_freezed() and input_t._is_trainable():
                    continue
                if input_t._get_seq_id() in blocked:
                    continue
                for func in funcs:
                    func(t, t.get_grad())
                src = input_t._get_top_reference_source()
                if not any(src is p for p in pending):
                    pending.append(src)
            _run_tensor_cleanups()
        if not grad_for_non_trainables and not t._is_trainable():
            t.free_grad()


def _untrainable_branches(loss):
    """seq-ids of tensors from which no optimizer-attached tensor is reachable
    (backward.py:48-99): walk inputs from the losses; whenever an attached
    tensor is met, unblock it and everything downstream of it."""
    blocked = {t._get_seq_id(): [] for t in loss}       # id -> ids of its consumers
    work = list(loss)
    while work:
        work.sort(key=_seq)
        t = work.pop()
        tid = t._get_seq_id()
        if t._is_trainable():
            stack = [tid]
            while stack:
                x = stack.pop()
                stack += blocked.pop(x, [])
            continue
        fns = t._get_gradfns()
        if fns is None:
            continue
        for input_t in fns:
            consumers = blocked.setdefault(input_t._get_seq_id(), [])
            if tid not in consumers:
                consumers.append(tid)
            src = input_t._get_top_reference_source()
            if not any(src is w for w in work):
                work.append(src)
    return blocked
