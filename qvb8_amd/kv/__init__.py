"""Banded KV cache: the per-channel affine codec and attention straight over its ids."""
from .codec import BandedKV, KVCertificateError, band_kv_heads, unband_kv_4d  # noqa: F401
from .fused_attn import QVLayout, attend, layout_from_segments, merge_lse, merge_lse_all  # noqa: F401
