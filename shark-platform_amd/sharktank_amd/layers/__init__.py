from .base import BaseLayer, ThetaLayer
from .linear import LinearLayer
from .norm import RMSNormLayer
from .ffn_moe_block import FFNMOE, PreGatherFFNMOE, extract_ffn_layer
from .ffn_block import FFN
from .mixture_of_experts_block import MoeBlock
