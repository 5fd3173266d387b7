"""MI355X-native Swin V2 scaled-cosine window attention.

Same public names as the reference package `flash_win_attn_v2`
(flash_win_attn_v2/__init__.py:1-10).
"""
from .win_attention_func import (flash_win_attn_v2_func, flash_win_attn_v2_grid_func, flash_win_attn_v2_qkvpacked_func,
                                 win_attention_torch, win_attention_torch_compile)
from .flash_window_attention_v2 import (FlashWindowAttentionV2, FlashWindowAttentionV2Grid,
                                         FlashWindowAttentionV2QKVPacked)
from .swin_transformer_v2 import WindowAttention, SwinTransformerV2

__all__ = ["flash_win_attn_v2_func", "flash_win_attn_v2_qkvpacked_func", "flash_win_attn_v2_grid_func",
           "win_attention_torch", "win_attention_torch_compile", "FlashWindowAttentionV2",
           "FlashWindowAttentionV2QKVPacked", "FlashWindowAttentionV2Grid",
           "WindowAttention", "SwinTransformerV2"]
