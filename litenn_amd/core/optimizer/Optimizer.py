import numpy as np

import litenn_amd as nn
import litenn_amd.core as nc


class Optimizer(nc.ModuleBase):
    """Base of optimizers (same contract as optimizer/Optimizer.py:36-204):
    marks its tensors trainable, keeps the iteration counter, applies
    clipnorm, then calls the subclass's _on_step().

     tensors_list   tensors to optimise (no references, gradients or op results)
     lr(0.001) lr_decay(0.0) clipnorm(0.0)
     lr_dropout(0.0)  fraction of elements whose learning rate is zero in a step: element gid of a tensor is
                      dropped where the counter hash of gid + seed, scaled to [0, 1], does not exceed it, with
                      a fresh host-drawn seed per update kernel (Optimizer.py:178-203)
    """

    def __init__(self, _tensors_list, lr=0.001, lr_decay=0.0, lr_dropout=0.0, clipnorm=0.0, saveables=None):
        if _tensors_list is None:
            raise ValueError('_tensors_list must be specified.')
        if not 0.0 <= lr_dropout <= 1.0:
            raise ValueError('lr_dropout must lie in [0, 1]')
        seen_ids, seen_names = set(), set()
        for t in _tensors_list:
            if id(t) in seen_ids:
                raise ValueError(f'Tensor {t.get_name()} has duplicate in a list.')
            if t.get_name() in seen_names:
                raise ValueError(f"Different tensors with the same name '{t.get_name()}'. If the same module class "
                                 'is used twice, derive two differently named subclasses.')
            seen_ids.add(id(t))
            seen_names.add(t.get_name())
        for t in _tensors_list:
            if t._is_reference():
                raise ValueError(f'Tensor {t.get_name()} is reference, and cannot be trained in optimizer.')
            if t._is_grad():
                raise ValueError(f'Tensor {t.get_name()} is gradient tensor, and cannot be trained in optimizer.')
            if t._is_trainable():
                raise ValueError(f'Tensor {t.get_name()} is already used by another optimizer.')
            if t._get_gradfns() is not None:
                raise Exception(f'Tensor {t.get_name()} is produced by operator and cannot be trained in optimizer.')
            t._set_trainable(True)
        self._tensors_list = _tensors_list
        self.lr, self.lr_decay, self.lr_dropout, self.clipnorm = lr, lr_decay, lr_dropout, clipnorm
        self.iteration = 0
        super().__init__((saveables or []) + ['iteration'])

    def get_trainable_tensors(self): return self._tensors_list
    def get_iteration(self): return self.iteration
    def set_iteration(self, iteration): self.iteration = iteration

    def zero_grad(self):
        for t in self._tensors_list:
            t.zero_grad()

    def print_no_grad(self):
        for t in self._tensors_list:
            if not t.has_grad():
                print(f'Tensor has no gradient : {t.get_name()}')

    def step(self, multi_gpu_step=False):
        """Update every tensor that has a gradient.  multi_gpu_step averages the
        tensors' values across the current devices through the host
        (Optimizer.py:149-153)."""
        if self.clipnorm != 0.0:
            sums = [nn.square(t.get_grad()).sum().np()[0] for t in self._tensors_list if t.has_grad()]
            l2norm = np.sqrt(np.sum(sums))
            if l2norm > self.clipnorm:
                mod = self.clipnorm / l2norm
                for t in self._tensors_list:
                    if t.has_grad():
                        nc.op.mul_const(t.get_grad(), mod, output_t=t.get_grad())
        self._on_step()
        if multi_gpu_step and len(nn.devices.get_current()) > 1:
            for t in self._tensors_list:
                t.set(np.mean([t.np(i) for i in range(t.np_count())], 0))
        self.iteration += 1

    def _on_step(self):
        raise NotImplementedError()

    def _kernel_seeds(self, count):
        """One seed per update kernel the reference would launch, drawn from numpy's global generator exactly as
        it does (Optimizer.py:178-182: np.random.randint(2147483648) per kernel.run, whether or not lr_dropout is on,
        so the generator's state stays in step with the reference's)."""
        return [int(np.random.randint(2147483648)) for _ in range(count)]

    def _current_lr(self):
        """lr / (1 + lr_decay * iteration)   (Optimizer.py:191-197)."""
        lr = np.float32(self.lr)
        if self.lr_decay != 0.0:
            lr = lr * np.float32(1.0 / (1.0 + self.lr_decay * self.iteration))
        return float(lr)
