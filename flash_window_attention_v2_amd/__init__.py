"""MI355X-native Swin V2 scaled-cosine window attention.

Same public names as the reference package `flash_win_attn_v2`
(flash_win_attn_v2/__init__.py:1-10), minus the torch.compile variant.
"""
from .win_attention_func import flash_win_attn_v2_func, win_attention_torch
from .flash_window_attention_v2 import FlashWindowAttentionV2

__all__ = ["flash_win_attn_v2_func", "win_attention_torch", "FlashWindowAttentionV2"]
