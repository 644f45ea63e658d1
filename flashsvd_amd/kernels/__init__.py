"""Operator-level entry points under the names the FlashSVD runtime imports."""
from .densekv_reconstruct import (pack_qkv_shared_bases, reconstruct_qkv_token, reconstruct_qkv_token_shared,
                                  reconstruct_qkv_token_shared_hetero, reconstruct_qkv_token_shared_prepacked)
from .dual_split import *  # noqa: F401,F403
from .rope_attn import FlashSVDRoPEAttention, QKVFactors, apply_rotary_bmhd, rotate_half  # noqa: E402,F401
