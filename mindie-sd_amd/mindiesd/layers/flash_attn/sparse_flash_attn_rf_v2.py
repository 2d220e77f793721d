"""Import-path alias: the reference keeps these functions in sparse_flash_attn_rf_v2.py."""
from .rainfusion import (avgpool, get_mask_index, get_blockwise_mask, rearrange_with_remaining,  # noqa: F401
                         inv_rearrange_with_remaining, do_tensor_rearrange_pooling, do_tensor_inv_rearrange,
                         do_tensor_pooling, rain_fusion_attention)
