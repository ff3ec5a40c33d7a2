"""``torch.nn`` modules whose forward and backward passes use the reproducible
operators -- the counterpart of RepDL's ``repdl/nn/{linear,conv,loss,batchnorm}.py``
module classes.  Each subclasses the PyTorch module it replaces, so parameters,
initialisation and ``state_dict`` layout are PyTorch's.
"""
from __future__ import annotations

import torch

from . import functional as F


class Linear(torch.nn.Linear):
    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return F.linear(input, self.weight, self.bias)


class Conv2d(torch.nn.Conv2d):
    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return F.conv2d(input, self.weight, self.bias, self.stride, self.padding, self.dilation, self.groups)


class CrossEntropyLoss(torch.nn.CrossEntropyLoss):
    def forward(self, input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        return F.cross_entropy(input, target, weight=self.weight, ignore_index=self.ignore_index,
                               reduction=self.reduction, label_smoothing=self.label_smoothing)


class _BatchNorm(torch.nn.modules.batchnorm._BatchNorm):
    """Batch statistics in training (or when no running statistics are tracked),
    running statistics otherwise (reference batchnorm.py:100-126)."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        self._check_input_dim(input)
        factor = 0.0 if self.momentum is None else self.momentum
        if self.training and self.track_running_stats and self.num_batches_tracked is not None:
            self.num_batches_tracked = self.num_batches_tracked + 1
            if self.momentum is None:
                factor = 1.0 / float(self.num_batches_tracked)
        use_batch = self.training or not self.track_running_stats
        return F.batch_norm(input, self.running_mean, self.running_var, self.weight, self.bias, use_batch,
                            factor, self.eps)


class BatchNorm1d(_BatchNorm):
    _check_input_dim = torch.nn.BatchNorm1d._check_input_dim


class BatchNorm2d(_BatchNorm):
    _check_input_dim = torch.nn.BatchNorm2d._check_input_dim
