from .focused_la import FocusedLinearAttention
from .linfusion import GeneralizedLinearAttention
from .mlla import MambaLikeLinearAttention
from .polaformer import PolaLinearAttention
from .rala import RALALinearAttention

__all__ = [
    'GeneralizedLinearAttention',
    'FocusedLinearAttention',
    'MambaLikeLinearAttention',
    'PolaLinearAttention',
    'RALALinearAttention',
]
