"""Mirrors of the reference's ``model/layers/folding`` modules on the hot path."""

from .attention_pair_bias import (  # noqa: F401
    AdaLN,
    CrossAttentionPairBias,
    PairBiasTiles,
    SelfAttentionPairBias,
    hip_attention_pair_bias,
    prepare_pair_bias,
)
from .transition import SwiGLU, Transition, hip_transition  # noqa: F401
