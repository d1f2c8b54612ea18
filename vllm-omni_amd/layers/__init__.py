from .adalayernorm import AdaLayerNorm
from .custom_op import CustomOp
from .rmsnorm import RMSNorm
from .rope import RotaryEmbedding

__all__ = ["AdaLayerNorm", "CustomOp", "RMSNorm", "RotaryEmbedding"]
