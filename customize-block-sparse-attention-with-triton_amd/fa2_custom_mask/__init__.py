"""fa2_custom_mask: block-sparse FlashAttention-2 for AMD MI355X behind the reference's API.

Exports the names of the reference package (fa2_custom_mask/__init__.py:1-5) except the raw
Triton kernel objects, which have no counterpart here."""
from .fa2_custom_mask import (flash_attention_custom_mask, flash_attention_custom_mask_lse,
                              attention_forward_backward, build_groups_from_block_mask, _attention,
                              ForwardPlan, BackwardPlan, set_deterministic)
from .utils import is_hip, keep, reduce_dense_mask, block_mask_to_lists, TileLists
from .functional import (permute_qkv_triton, apply_head_wise_reorder, inv_permute_attn_triton,
                         apply_inv_reorder)

__all__ = [
    "flash_attention_custom_mask", "flash_attention_custom_mask_lse", "attention_forward_backward",
    "build_groups_from_block_mask", "is_hip", "keep", "reduce_dense_mask", "block_mask_to_lists",
    "TileLists", "ForwardPlan", "BackwardPlan", "set_deterministic", "permute_qkv_triton", "apply_head_wise_reorder", "inv_permute_attn_triton",
    "apply_inv_reorder",
]
