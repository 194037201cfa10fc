"""Module-level mirrors of the reference's hot-path primitives with ``kernel_backend="hip"``."""

from .layers import LayerNorm, Linear, LinearNoBias  # noqa: F401
from .triangle_multiplication import (  # noqa: F401
    TriangleMultiplicationIncoming,
    TriangleMultiplicationOutgoing,
    hip_triangular_mult,
)
from .triangle_attention import (  # noqa: F401
    TriangleAttention,
    TriangleAttentionEndingNode,
    TriangleAttentionStartingNode,
    hip_triangular_attn,
)
