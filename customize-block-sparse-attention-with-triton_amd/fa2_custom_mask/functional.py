"""Head-wise token reorder wrappers, mirroring fa2_custom_mask/functional.py:5-84 of the
reference (same names, arguments, defaults and in-place write-back); the row gather itself
is the HIP kernel behind bsattn_reorder."""
import torch

from . import _ext

_PERMUTATIONS = [[0, 1, 2], [0, 2, 1], [1, 2, 0], [1, 0, 2], [2, 1, 0], [2, 0, 1]]       # functional.py:23-26
_PERMUTATIONS_INV = [[0, 1, 2], [0, 2, 1], [2, 0, 1], [1, 0, 2], [2, 1, 0], [1, 2, 0]]   # functional.py:69-76


def _launch(tensor, permute_orders, inv_permute_orders, F, H, W):
    if not tensor.is_cuda:
        raise RuntimeError("reorder needs a GPU tensor (there is no CPU path)")
    BS, N_head, N_token, D = tensor.shape
    assert N_token == F * H * W                                               # functional.py:7,48
    tensor = tensor.contiguous()
    orders = permute_orders.to(device=tensor.device, dtype=torch.int32).contiguous()
    inv = None
    if inv_permute_orders is not None:
        inv = inv_permute_orders.to(device=tensor.device, dtype=torch.int32).contiguous()
    output = torch.empty_like(tensor)                                         # functional.py:8,49
    rc = _ext.lib().bsattn_reorder(tensor.data_ptr(), output.data_ptr(), BS, N_head, F, H, W, D,
                                   tensor.element_size(), orders.data_ptr(),
                                   inv.data_ptr() if inv is not None else None,
                                   _ext.current_stream(tensor.device))
    _ext.check(rc, "bsattn_reorder")
    return output


def apply_head_wise_reorder(tensor, permute_orders, F, H, W):
    """functional.py:5-20: out[b,h,new_t,:] = tensor[b,h,t,:], new_t per head from permute_orders."""
    return _launch(tensor, permute_orders, None, F, H, W)


def apply_inv_reorder(tensor, permute_orders, inv_permute_orders, F, H, W):
    """functional.py:46-62: undo apply_head_wise_reorder."""
    return _launch(tensor, permute_orders, inv_permute_orders, F, H, W)


def permute_qkv_triton(query, key, value, permute_plan, i_block, F=13, H=30, W=45, n_text_tokens=226):
    """functional.py:22-43 (the name is kept for drop-in use; nothing here uses Triton)."""
    permutations = torch.tensor(_PERMUTATIONS, dtype=torch.int32, device=query.device)
    idx = permute_plan['permute'][i_block]                                    # :28
    permute_orders = permutations[idx]                                        # :29
    outs = []
    for x in (query, key, value):
        image = x[:, :, n_text_tokens:, :]                                    # :31-33
        outs.append(apply_head_wise_reorder(image.contiguous(), permute_orders, F, H, W))
    query[:, :, n_text_tokens:, :] = outs[0]                                  # :39-41
    key[:, :, n_text_tokens:, :] = outs[1]
    value[:, :, n_text_tokens:, :] = outs[2]
    return query, key, value


def inv_permute_attn_triton(attn_out, permute_plan, i_block, F=13, H=30, W=45, n_text_tokens=226):
    """functional.py:64-84."""
    permutations = torch.tensor(_PERMUTATIONS, dtype=torch.int32, device=attn_out.device)
    permutations_inv = torch.tensor(_PERMUTATIONS_INV, dtype=torch.int32, device=attn_out.device)
    idx = permute_plan['permute'][i_block]                                    # :78
    permute_orders = permutations[idx]
    inv_permute_orders = permutations_inv[idx]
    attn_image = attn_out[:, :, n_text_tokens:, :]                            # :81
    attn_image_out = apply_inv_reorder(attn_image.contiguous(), permute_orders, inv_permute_orders, F, H, W)
    attn_out[:, :, n_text_tokens:, :] = attn_image_out                        # :83
    return attn_out
