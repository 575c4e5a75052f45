import litenn_amd as nn
from ..hip import api, launch
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
        for t in self.get_trainable_tensors():
            if not t.has_grad():
                continue
            n = t.shape.size
            launch(lambda dev, v, g, m, s: api.adam_update(dev, n, v, g, m, s, self.beta_1, self.beta_2, lr),
                   t, t.get_grad(), self._ms[t.get_name()], self._vs[t.get_name()])
