"""Layer base classes (mirror of sharktank/sharktank/layers/base.py:21-82, minus export/trace hooks)."""

import torch.nn as nn

from ..types import InferenceTensor, Theta

__all__ = ["BaseLayer", "ThetaLayer"]


class BaseLayer(nn.Module):
    pass


class ThetaLayer(BaseLayer):
    "Base class for layers that derive parameters from a Theta object."

    def __init__(self, theta: Theta):
        super().__init__()
        self.theta = theta

    def theta_tensor(self, name: str) -> InferenceTensor:
        return self.theta.tensor(name)
