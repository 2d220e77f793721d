"""Import-path alias: the reference keeps these functions in sparse_flash_attn_rf_v3.py."""
from .rainfusion import (_bsa_inv_rearrange, do_tensor_rearrange_only, rain_fusion_attention_v3,  # noqa: F401
                         bsa_sparse_attention_v3)
