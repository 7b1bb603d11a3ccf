"""Causal linear attention for MI355X (gfx950): hand-written HIP kernels behind
the Python surface of ``flashlinear`` (flashlinear/__init__.py:1-2)."""

from .auto import LinearAttentionAuto
from .chunked import LinearAttentionChunked
from .feature import FeatureMapLinearAttention
from .linear_attn import LinearAttention
from .linear_attn_smallv_hd import LinearAttentionSmallVHD
from .normalised import LinearAttentionNormalised
from .poly import PolynomialLinearAttention

__all__ = ["LinearAttention", "LinearAttentionSmallVHD", "LinearAttentionChunked", "LinearAttentionAuto",
           "LinearAttentionNormalised",
           "PolynomialLinearAttention", "FeatureMapLinearAttention"]
