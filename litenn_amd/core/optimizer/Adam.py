import litenn_amd as nn
from ..hip import api, launch, cached_permuted_copies, keep_permuted_copies
from .Optimizer import Optimizer


class Adam(Optimizer):
    """Adam as the reference defines it (same constructor as optimizer/Adam.py:29; no bias correction):
      m = beta_1*m + (1-beta_1)*g
      v = beta_2*v + (1-beta_2)*g*g
      t += -lr*m / (sqrt(v) + 1e-7)                     (Adam.py:43-72)
    fused into one launch per tensor (the reference runs three)."""

    def __init__(self, tensors_list, beta_1=0.9, beta_2=0.999, lr=0.001, lr_decay=0.0, lr_dropout=0.0, clipnorm=0.0):
        super().__init__(tensors_list, lr=lr, lr_decay=lr_decay, lr_dropout=lr_dropout, clipnorm=clipnorm,
                         saveables=['_ms', '_vs'])
        self.beta_1, self.beta_2 = beta_1, beta_2
        self._ms = {t.get_name(): nn.Tensor_zeros_like(t) for t in self.get_trainable_tensors()}
        self._vs = {t.get_name(): nn.Tensor_zeros_like(t) for t in self.get_trainable_tensors()}

    def _on_step(self):
        lr = self._current_lr()
        ts = [t for t in self.get_trainable_tensors() if t.has_grad()]
        if not ts:
            return
        k, ns = len(ts), [t.shape.size for t in ts]
        grads, ms, vs = [t.get_grad() for t in ts], [self._ms[t.get_name()] for t in ts], [self._vs[t.get_name()] for t in ts]
        cached = cached_permuted_copies(ts)
        seeds = self._kernel_seeds(k)     # one per tensor: the value kernel (Adam.py:76-86)
        if self.lr_dropout != 0.0:
            any_copy = any(c is not None for c in cached)
            cs, kks = [c[2] if c else 0 for c in cached], [c[3] if c else 0 for c in cached]
            lays = [c[4] if c else 0 for c in cached]

            def run(dev, *p):
                wps = p[4 * k:] if any_copy else None
                api.adam_update_multi_lrd(dev, ns, p[:k], p[k:2 * k], p[2 * k:3 * k], p[3 * k:4 * k], self.beta_1, self.beta_2,
                                          lr, self.lr_dropout, seeds, wps, cs if any_copy else None,
                                          kks if any_copy else None, lays if any_copy else None)
            launch(run, *ts, *grads, *ms, *vs, *([c[1] if c else None for c in cached] if any_copy else []))
            keep_permuted_copies(ts, cached)
        elif any(c is not None for c in cached):
            # convolution kernels whose permuted copy is cached: the update refreshes the copy in the same pass
            cs, kks = [c[2] if c else 0 for c in cached], [c[3] if c else 0 for c in cached]
            lays = [c[4] if c else 0 for c in cached]
            launch(lambda dev, *p: api.adam_update_multi_wp(dev, ns, p[:k], p[k:2 * k], p[2 * k:3 * k], p[3 * k:4 * k],
                                                            self.beta_1, self.beta_2, lr, p[4 * k:], cs, kks, lays),
                   *ts, *grads, *ms, *vs, *[c[1] if c else None for c in cached])
            keep_permuted_copies(ts, cached)
        else:
            launch(lambda dev, *p: api.adam_update_multi(dev, ns, p[:k], p[k:2 * k], p[2 * k:3 * k], p[3 * k:],
                                                         self.beta_1, self.beta_2, lr),
                   *ts, *grads, *ms, *vs)
