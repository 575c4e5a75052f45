import litenn_amd as nn
from ..hip import api, launch, cached_permuted_copies, keep_permuted_copies
from .Optimizer import Optimizer


class SGD(Optimizer):
    """Stochastic gradient descent (same constructor as optimizer/SGD.py:29):
      acc = momentum*acc - lr*g
      v  += nesterov ? momentum*acc - lr*g : acc          (SGD.py:52,68-72)
    fused into one launch for all tensors."""

    def __init__(self, tensors_list, momentum=0.0, nesterov=False, lr=0.001, lr_decay=0.0, lr_dropout=0.0,
                 clipnorm=0.0):
        super().__init__(tensors_list, lr=lr, lr_decay=lr_decay, lr_dropout=lr_dropout, clipnorm=clipnorm,
                         saveables=['_accs'])
        self.momentum = momentum
        self.nesterov = nesterov
        self._accs = {t.get_name(): nn.Tensor_zeros_like(t) for t in self.get_trainable_tensors()}

    def _on_step(self):
        lr = self._current_lr()
        ts = [t for t in self.get_trainable_tensors() if t.has_grad()]
        if not ts:
            return
        k, ns = len(ts), [t.shape.size for t in ts]
        # every tensor's update in one launch per device: pointers arrive as (values, gradients, accumulators)
        grads, accs = [t.get_grad() for t in ts], [self._accs[t.get_name()] for t in ts]
        cached = cached_permuted_copies(ts)
        seeds = self._kernel_seeds(2 * k)     # per tensor: accumulator kernel, value kernel (SGD.py:76-83)
        if self.lr_dropout != 0.0:
            any_copy = any(c is not None for c in cached)
            cs, kks = [c[2] if c else 0 for c in cached], [c[3] if c else 0 for c in cached]
            lays = [c[4] if c else 0 for c in cached]

            def run(dev, *p):
                wps = p[3 * k:] if any_copy else None
                api.sgd_update_multi_lrd(dev, ns, p[:k], p[k:2 * k], p[2 * k:3 * k], self.momentum, lr, self.nesterov,
                                         self.lr_dropout, seeds, wps, cs if any_copy else None, kks if any_copy else None,
                                         lays if any_copy else None)
            launch(run, *ts, *grads, *accs, *([c[1] if c else None for c in cached] if any_copy else []))
            keep_permuted_copies(ts, cached)
        elif any(c is not None for c in cached):
            # convolution kernels whose permuted copy is cached: the update refreshes the copy in the same pass
            cs, kks = [c[2] if c else 0 for c in cached], [c[3] if c else 0 for c in cached]
            lays = [c[4] if c else 0 for c in cached]
            launch(lambda dev, *p: api.sgd_update_multi_wp(dev, ns, p[:k], p[k:2 * k], p[2 * k:3 * k], self.momentum, lr,
                                                           self.nesterov, p[3 * k:], cs, kks, lays),
                   *ts, *grads, *accs, *[c[1] if c else None for c in cached])
            keep_permuted_copies(ts, cached)
        else:
            launch(lambda dev, *p: api.sgd_update_multi(dev, ns, p[:k], p[k:2 * k], p[2 * k:], self.momentum, lr, self.nesterov),
                   *ts, *grads, *accs)
