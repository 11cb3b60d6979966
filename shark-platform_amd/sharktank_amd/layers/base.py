"""Layer base classes (mirror of sharktank/sharktank/layers/base.py:21-82: the tracing hooks and the theta accessor;
`sample_inputs`, which serves export, is not part of this path)."""

from typing import Dict

import torch
import torch.nn as nn

from ..types import InferenceTensor, Theta
from ..utils import debugging

__all__ = ["BaseLayer", "ThetaLayer"]


class BaseLayer(nn.Module):
    """Base class of the layers: forwards the tracing calls a model sprinkles over its forward to `utils.debugging`."""

    def trace_tensor(self, key: str, t: torch.Tensor, *, values: bool = True, golden: bool = False):
        debugging.trace_tensor(key, t, values=values, golden=golden)

    def trace_tensors(self, key: str, tensors: Dict[str, torch.Tensor], *, values: bool = True, golden: bool = False):
        debugging.trace_tensors(key, tensors, values=values, golden=golden)

    def trace_golden(self, key: str, t: torch.Tensor):
        debugging.trace_tensor(key, t, golden=True)

    def trace_goldens(self, key: str, tensors: Dict[str, torch.Tensor]):
        debugging.trace_tensors(key, tensors, golden=True)

    def assert_not_nan(self, *ts: torch.Tensor):
        """Raises if a tensor holds a NaN; only when `enable_nan_checks` is set (the check synchronises)."""
        if debugging.flags.enable_nan_checks:
            for t in ts:
                if torch.isnan(t).any():
                    raise AssertionError(f"Tensor contains nans! {t}")


class ThetaLayer(BaseLayer):
    "Base class for layers that derive parameters from a Theta object."

    def __init__(self, theta: Theta):
        super().__init__()
        self.theta = theta

    def theta_tensor(self, name: str) -> InferenceTensor:
        return self.theta.tensor(name)
