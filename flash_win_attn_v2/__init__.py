"""Import-name alias: `import flash_win_attn_v2` resolves to the gfx950 implementation, so code
written against the reference package (flash_win_attn_v2/__init__.py:1-10) runs unchanged.
The submodule names of the reference are aliased too."""
import sys

import flash_window_attention_v2_amd as _impl
from flash_window_attention_v2_amd import (FlashWindowAttentionV2, FlashWindowAttentionV2Grid,
                                           FlashWindowAttentionV2QKVPacked, SwinTransformerV2, WindowAttention,
                                           flash_win_attn_v2_func, flash_win_attn_v2_grid_func,
                                           flash_win_attn_v2_qkvpacked_func, win_attention_torch,
                                           win_attention_torch_compile)
from flash_window_attention_v2_amd import flash_window_attention_v2, kernels, swin_transformer_v2, win_attention_func

for _name in ("flash_window_attention_v2", "kernels", "swin_transformer_v2", "win_attention_func"):
    sys.modules[__name__ + "." + _name] = getattr(_impl, _name)

__all__ = _impl.__all__
