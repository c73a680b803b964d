"""``NLLLoss`` (``src/tortto/nn/modules/loss.py:38-46``)."""
from .. import functional as F
from .module import Module


class NLLLoss(Module):
    def __init__(self, weight=None, ignore_index=-100, reduction='mean'):
        super().__init__()
        self.weight = weight
        self.ignore_index = ignore_index
        self.reduction = reduction

    def forward(self, inpt, target):
        return F.nll_loss(inpt, target, weight=self.weight, ignore_index=self.ignore_index, reduction=self.reduction)
