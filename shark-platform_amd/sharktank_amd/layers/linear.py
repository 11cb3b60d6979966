"""LinearLayer for the router gate (mirror of sharktank/sharktank/layers/linear.py:22-95 for the plain
weight (+ optional q_input fake-quant) case: y = matmul(x, weight.T))."""

from typing import Optional

import torch

from .. import ops
from ..types import QuantizedTensor, QuantizerTensor, unbox_tensor
from .base import Theta, ThetaLayer

__all__ = ["LinearLayer"]


class LinearLayer(ThetaLayer):
    def __init__(self, theta: Theta, *, weight_name: str = "weight", bias_name: str = "bias", fake_quant: bool = False):
        super().__init__(theta)
        self.weight = self.theta_tensor(weight_name)
        self.bias = None
        self.fake_quant = fake_quant
        if bias_name in self.theta.keys:
            self.bias = self.theta_tensor(bias_name)
        self.premul_input = theta.optional_tensor("premul_input")
        self.q_input: Optional[QuantizerTensor] = theta.optional_tensor("q_input")
        self.qdq_input = theta.optional_tensor("qdq_input")
        if self.q_input is not None and self.qdq_input is not None:
            raise AssertionError("LinearLayer cannot have both q_input and qdq_input")
        self.qdq_output = theta.optional_tensor("qdq_output")
        if self.premul_input is not None or self.qdq_input is not None or self.qdq_output is not None:
            raise NotImplementedError("LinearLayer: premul_input / qdq_input / qdq_output are outside the MoE path")

    def forward(self, x):
        if self.q_input is not None:
            x = self.q_input.quantize(x)
            x = x.unpack().dequant()
        y = ops.linear(x, self.weight, self.bias)
        if isinstance(y, QuantizedTensor):
            y = y.unpack().dequant()
        return y
