"""RMSNormLayer with the constructor and numerics of sharktank/sharktank/layers/norm.py:18-41: statistics in
`dtype` (fp32), multiply by the weight in the weight's dtype, result cast back to the input dtype.  The three
steps run as one HIP kernel."""

import torch

from .. import _hip
from ..types import unbox_tensor
from .base import Theta, ThetaLayer

__all__ = ["RMSNormLayer"]


class RMSNormLayer(ThetaLayer):
    def __init__(self, theta: Theta, *, weight_name: str = "weight", epsilon: float = 1e-6, dtype: torch.dtype = torch.float32):
        super().__init__(theta)
        self.weight = self.theta_tensor(weight_name)
        self.epsilon = epsilon
        if dtype != torch.float32:
            raise NotImplementedError("RMSNormLayer: the kernel computes its statistics in float32")
        self.dtype = dtype

    def forward(self, x: torch.Tensor):
        return _hip.rms_norm(x, unbox_tensor(self.weight), self.epsilon)
