from .base import BaseLayer, ThetaLayer
from .linear import LinearLayer
from .norm import RMSNormLayer
from .ffn_moe_block import PreGatherFFNMOE
from .mixture_of_experts_block import MoeBlock
