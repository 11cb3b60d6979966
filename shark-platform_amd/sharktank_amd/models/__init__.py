from .moe_stack import MoeStack
