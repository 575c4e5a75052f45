import litenn_amd as nn
from ..hip import api, launch
from .Optimizer import Optimizer


class SGD(Optimizer):
    """Stochastic gradient descent (same constructor as optimizer/SGD.py:29):
      acc = momentum*acc - lr*g
      v  += nesterov ? momentum*acc - lr*g : acc          (SGD.py:52,68-72)
    fused into one launch per tensor."""

    def __init__(self, tensors_list, momentum=0.0, nesterov=False, lr=0.001, lr_decay=0.0, lr_dropout=0.0,
                 clipnorm=0.0):
        super().__init__(tensors_list, lr=lr, lr_decay=lr_decay, lr_dropout=lr_dropout, clipnorm=clipnorm,
                         saveables=['_accs'])
        self.momentum = momentum
        self.nesterov = nesterov
        self._accs = {t.get_name(): nn.Tensor_zeros_like(t) for t in self.get_trainable_tensors()}

    def _on_step(self):
        lr = self._current_lr()
        for t in self.get_trainable_tensors():
            if not t.has_grad():
                continue
            acc_t = self._accs[t.get_name()]
            n = t.shape.size
            launch(lambda dev, v, g, a: api.sgd_update(dev, n, v, g, a, self.momentum, lr, self.nesterov),
                   t, t.get_grad(), acc_t)
