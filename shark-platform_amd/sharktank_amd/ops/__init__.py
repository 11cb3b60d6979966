"""`sharktank.ops`-compatible operator surface for the MoE path, backed by HIP kernels."""

from ._registry import *
from ._registry import _test_enable_last_op_dispatch, _test_get_last_op_dispatch
from .signatures import *
from . import hip_impls
from .hip_impls import device_weight, expert_dispatch, gather_experts
