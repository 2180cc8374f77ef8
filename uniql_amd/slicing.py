"""Load-time slicing of packed W4A16 tensors on the GPU.

UniQL stores one full-size quantised model and cuts every layer down to the pruned size
when it is loaded (modeling/modeling_helpers.py:235-867).  The reference does this on the
CPU in numpy: unpack the Marlin layout, cut, pack again.  Here the same three steps run on
the device (uniql_w4a16_dequant's code output, a tensor slice, uniql_w4a16_pack), with the
reference's function names, argument order and results.
"""
from __future__ import annotations

import math

import torch

from . import ops

MIN_THREAD_N = 64      # quantize/quant_linear_layers.py: workspace = (size_n // 64) * 16 ints
MAX_PARALLEL = 16


def _pad_to(value: int, multiple: int) -> int:
    return (-value) % multiple


def slice_w4a16_up_gate_proj(weight, scale, workspace, hidden_size, intermediate_size,
                             reduced_intermediate_size, load_shape, num_bits=4, group_size=128):
    """Keeps the first `reduced_intermediate_size` output columns of an up/gate projection
    [hidden_size -> intermediate_size] (modeling_helpers.py:361-408).  The kept width is padded
    to a multiple of 256 with the neighbouring columns' codes and ZERO scales, as the reference
    does; the workspace shrinks with the width."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(hidden_size, group_size)
    pad_n = _pad_to(intermediate_size, 256)
    reduced_pad_n = _pad_to(reduced_intermediate_size, 256)
    assert load_shape[0] == weight.shape[0], "hidden_size dimension mismatch"
    size_k, size_n = hidden_size + pad_k, intermediate_size + pad_n
    keep = reduced_intermediate_size + reduced_pad_n
    assert size_n >= keep, "Reduced size shape exceeds recovered weight"
    codes, scales = ops.w4a16_unpack(weight, scale, size_n, size_k)
    cut_scales = scales[:, :keep].clone()
    cut_scales[:, reduced_intermediate_size:] = 0
    new_weight, new_scale = ops.w4a16_pack(codes[:, :keep], cut_scales)
    new_workspace = workspace[:(keep // MIN_THREAD_N) * MAX_PARALLEL].contiguous()
    return new_weight, new_scale, new_workspace


def slice_w4a16_down_proj(weight, scale, workspace, hidden_size, intermediate_size,
                          reduced_intermediate_size, load_shape, num_bits=4, group_size=128):
    """Keeps the first `reduced_intermediate_size` input rows of a down projection
    [intermediate_size -> hidden_size], rounded up to whole groups of 128
    (modeling_helpers.py:411-448); the scale rows of the kept groups are taken as they are."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(intermediate_size, group_size)
    reduced_pad_k = _pad_to(reduced_intermediate_size, group_size)
    pad_n = _pad_to(hidden_size, 256)
    assert load_shape[1] == weight.shape[1], "hidden_size dimension mismatch"
    size_k, size_n = intermediate_size + pad_k, hidden_size + pad_n
    keep = reduced_intermediate_size + reduced_pad_k
    assert size_k >= keep, "Reduced size shape exceeds recovered weight"
    # whole packed rows (16 K values each) are cut: no unpacking needed for a prefix of groups
    new_weight = weight[:keep // 16].contiguous()
    new_scale = scale[:int(math.ceil(reduced_intermediate_size / 128))].contiguous()
    return new_weight, new_scale, workspace


def _workspace_for(size_n: int, workspace):
    return workspace[:(size_n // MIN_THREAD_N) * MAX_PARALLEL].contiguous()


def _gather_columns(weight, scale, workspace, size_k, size_n, rows_real, cols: torch.Tensor, pad_n_new: int):
    """Unpacks [size_k, size_n], keeps the real K rows and the columns `cols`, pads the rows back
    to size_k with code 0 as the reference's torch.nn.functional.pad does, and packs with
    pad_n_new padding columns (code 0, scale 0)."""
    codes, scales = ops.w4a16_unpack(weight, scale, size_n, size_k)
    cut = codes[:rows_real][:, cols]
    if rows_real < size_k:
        cut = torch.cat([cut, cut.new_zeros(size_k - rows_real, cut.shape[1])], dim=0)
    new_weight, new_scale = ops.w4a16_pack(cut.contiguous(), scales[:, cols].contiguous(), pad_out=pad_n_new)
    return new_weight, new_scale, _workspace_for(cols.numel() + pad_n_new, workspace)


def _rope_half_columns(nheads, head_dim, reduced_head_dim, device):
    """Per head, the first reduced_head_dim/2 columns of each rotary half
    (modeling_helpers.py:481-486)."""
    half, hd_half = head_dim // 2, reduced_head_dim // 2
    d = torch.cat([torch.arange(hd_half, device=device), half + torch.arange(hd_half, device=device)])
    return (torch.arange(nheads, device=device)[:, None] * head_dim + d[None, :]).reshape(-1)


def _head_prefix(nheads, head_dim, reduced_head_dim, device):
    d = torch.arange(reduced_head_dim, device=device)
    return (torch.arange(nheads, device=device)[:, None] * head_dim + d[None, :]).reshape(-1)


def slice_w4a16_qk_proj(weight, bias, scale, workspace, hidden_size, nheads, head_dim, reduced_head_dim,
                        load_shape, num_bits=4, group_size=128):
    """Query/key projection [hidden_size -> nheads * head_dim]: every head keeps the first
    reduced_head_dim / 2 columns of each rotary half (modeling_helpers.py:451-530)."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(hidden_size, group_size)
    pad_n = _pad_to(nheads * head_dim, 256)
    reduced_pad_n = _pad_to(nheads * reduced_head_dim, 256)
    assert load_shape[0] == weight.shape[0], "hidden_size dimension mismatch"
    cols = _rope_half_columns(nheads, head_dim, reduced_head_dim, weight.device)
    new_weight, new_scale, new_workspace = _gather_columns(
        weight, scale, workspace, hidden_size + pad_k, nheads * head_dim + pad_n, hidden_size, cols, reduced_pad_n)
    new_bias = None if bias is None else bias[cols.to(bias.device)]
    return new_weight, new_bias, new_scale, new_workspace


def slice_w4a16_v_proj(weight, scale, workspace, hidden_size, nheads, head_dim, reduced_head_dim,
                       load_shape, num_bits=4, group_size=128):
    """Value projection: every head keeps its first reduced_head_dim columns
    (modeling_helpers.py:533-596)."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(hidden_size, group_size)
    pad_n = _pad_to(nheads * head_dim, 256)
    reduced_pad_n = _pad_to(nheads * reduced_head_dim, 256)
    assert load_shape[0] == weight.shape[0], "hidden_size dimension mismatch"
    cols = _head_prefix(nheads, head_dim, reduced_head_dim, weight.device)
    return _gather_columns(weight, scale, workspace, hidden_size + pad_k, nheads * head_dim + pad_n, hidden_size,
                           cols, reduced_pad_n)


def slice_w4a16_o_proj(weight, scale, workspace, hidden_size, nheads, head_dim, reduced_head_dim,
                       load_shape, num_bits=4, group_size=128):
    """Output projection [nheads * head_dim -> hidden_size]: the kept input rows do not line up
    with the groups of 128 any more, so the reference dequantises, keeps every head's first
    reduced_head_dim rows and quantises again (modeling_helpers.py:600-656); the same here with
    the device kernels (bit-exact fp16 weights out of uniql_w4a16_dequant, uniql_w4a16_quantize)."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(nheads * head_dim, group_size)
    pad_n = _pad_to(hidden_size, 256)
    assert load_shape[1] == weight.shape[1], "hidden_size dimension mismatch"
    size_k, size_n = nheads * head_dim + pad_k, hidden_size + pad_n
    w_full = ops.w4a16_dequant(weight, scale, size_n, size_k)              # fp16 (code - 8) * scale, [k, n]
    rows = _head_prefix(nheads, head_dim, reduced_head_dim, weight.device)
    kept = w_full[rows][:, :hidden_size]                                  # [nheads * reduced_head_dim, hidden]
    new_weight, new_scale = ops.w4a16_quantize(kept.t().contiguous(), None, pad_out=pad_n)
    return new_weight, new_scale, workspace


def slice_indices(indices, head_dim, reduced_head_dim):
    """modeling_helpers.py:659-663."""
    half, hd_half = head_dim // 2, reduced_head_dim // 2
    return torch.cat([indices[:, :hd_half], indices[:, half:half + hd_half]], dim=-1).to(torch.uint8)


def get_topk_head_indices(n_groups, num_heads, head_dim, topk_head_dim, device=None):
    """First topk_head_dim channels of every head (modeling_helpers.py:124-130; the grouping of
    heads does not change their order)."""
    return _head_prefix(num_heads, head_dim, topk_head_dim, device)


def get_topk_ssm_state_indices(n_groups, ssm_state_size, topk_ssm_state, device=None):
    """First topk_ssm_state states of every group (modeling_helpers.py:132-137)."""
    return _head_prefix(n_groups, ssm_state_size, topk_ssm_state, device)


def slice_w4a16_in_proj(weight, scale, workspace, hidden_size, n_groups, num_heads, intermediate_size,
                        ssm_state_size, load_intermediate_size, load_ssm_state_size, load_shape,
                        num_bits=4, group_size=128):
    """Mamba2 input projection [hidden -> z | x | B | C | dt]: z and x keep the first channels
    of every head, B and C the first states of every group, dt stays
    (modeling_helpers.py:665-757)."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    projection_size = 2 * intermediate_size + 2 * n_groups * ssm_state_size + num_heads
    reduced_projection_size = 2 * load_intermediate_size + 2 * n_groups * load_ssm_state_size + num_heads
    pad_k = _pad_to(hidden_size, group_size)
    pad_n = _pad_to(projection_size, 256)
    reduced_pad_n = _pad_to(reduced_projection_size, 256)
    assert load_shape[0] == weight.shape[0], "hidden_size dimension mismatch"
    dev = weight.device
    heads = get_topk_head_indices(n_groups, num_heads, intermediate_size // num_heads,
                                  load_intermediate_size // num_heads, dev)
    states = get_topk_ssm_state_indices(n_groups, ssm_state_size, load_ssm_state_size, dev)
    x_start = intermediate_size
    b_start = x_start + intermediate_size
    c_start = b_start + n_groups * ssm_state_size
    dt_start = c_start + n_groups * ssm_state_size
    cols = torch.cat([heads, x_start + heads, b_start + states, c_start + states,
                      torch.arange(dt_start, projection_size, device=dev)])
    return _gather_columns(weight, scale, workspace, hidden_size + pad_k, projection_size + pad_n, hidden_size,
                           cols, reduced_pad_n)


def slice_w4a16_out_proj(weight, scale, workspace, hidden_size, n_groups, num_heads, intermediate_size,
                         load_intermediate_size, load_shape, num_bits=4, group_size=128):
    """Mamba2 output projection [intermediate -> hidden]: dequantise, keep the first channels of
    every head, quantise again (modeling_helpers.py:809-867)."""
    assert num_bits == 4, "Only support 4-bit quantization for now"
    assert group_size == 128, "Only group_size 128 is supported on the device"
    pad_k = _pad_to(intermediate_size, group_size)
    pad_n = _pad_to(hidden_size, 256)
    assert load_shape[1] == weight.shape[1], "hidden_size dimension mismatch"
    w_full = ops.w4a16_dequant(weight, scale, hidden_size + pad_n, intermediate_size + pad_k)
    rows = get_topk_head_indices(n_groups, num_heads, intermediate_size // num_heads,
                                 load_intermediate_size // num_heads, weight.device)
    kept = w_full[rows][:, :hidden_size]
    new_weight, new_scale = ops.w4a16_quantize(kept.t().contiguous(), None, pad_out=pad_n)
    return new_weight, new_scale, workspace


def slice_conv1d(weight, bias, n_groups, num_heads, intermediate_size, ssm_state_size,
                 load_intermediate_size, load_ssm_state_size):
    """The matching cut of Mamba2's depthwise convolution over x | B | C
    (modeling_helpers.py:760-790)."""
    dev = weight.device
    heads = get_topk_head_indices(n_groups, num_heads, intermediate_size // num_heads,
                                  load_intermediate_size // num_heads, dev)
    states = get_topk_ssm_state_indices(n_groups, ssm_state_size, load_ssm_state_size, dev)
    b_start = intermediate_size
    c_start = b_start + n_groups * ssm_state_size
    idx = torch.cat([heads, b_start + states, c_start + states])
    return weight[idx].contiguous(), bias[idx].contiguous()


def slice_norm(weight, n_groups, num_heads, intermediate_size, load_intermediate_size):
    """modeling_helpers.py:793-800."""
    idx = get_topk_head_indices(n_groups, num_heads, intermediate_size // num_heads,
                                load_intermediate_size // num_heads, weight.device)
    return weight[idx].contiguous()


# ---------------------------------------------------------------------------------------------
# The walk over a model (modeling_helpers.py:235-358): for every decoder layer, the block that is a
# UniQL W4A16 MLP / attention / Mamba block gets the tensors of the full-size checkpoint
# (`loaded_model`, a name -> tensor dict) replaced by their cuts to the block's own sizes.
# `model` and `model_helper` are the reference's objects, used through the same attributes the
# reference uses (get_layers, *_w4a16_uniql_class_name, get_*_key, model.config, the blocks' sizes
# and the shapes of their packed weights); nothing else of them is touched.
def _replace(state, key, names, values):
    for name, value in zip(names, values):
        if value is not None:
            state[f"{key}.{name}"] = value


def _packed(state, key):
    return state[f"{key}.weight"], state[f"{key}.scale"], state[f"{key}.workspace"]


_WSW = ("weight", "scale", "workspace")
_WBSW = ("weight", "bias", "scale", "workspace")


def slice_quantized_weights(model, model_helper, loaded_model):
    cfg = model.config
    for layer_idx, layer in enumerate(model_helper.get_layers(model)):
        for _, block in layer.named_children():
            kind = block.__class__.__name__
            if kind == model_helper.mlp_w4a16_uniql_class_name:
                base = model_helper.get_mlp_key(layer_idx)
                sizes = (cfg.hidden_size, cfg.intermediate_size, block.intermediate_size)
                for proj in ("up_proj", "gate_proj"):  # models without a gate have no gate_proj tensors
                    key = f"{base}.{proj}"
                    if f"{key}.weight" in loaded_model:
                        _replace(loaded_model, key, _WSW, slice_w4a16_up_gate_proj(
                            *_packed(loaded_model, key), *sizes, getattr(block, proj).weight.shape))
                key = f"{base}.down_proj"
                _replace(loaded_model, key, _WSW, slice_w4a16_down_proj(
                    *_packed(loaded_model, key), *sizes, block.down_proj.weight.shape))
            elif kind == model_helper.attn_w4a16_uniql_class_name:
                base = model_helper.get_attn_key(layer_idx)
                head_dim = getattr(cfg, "head_dim", cfg.hidden_size // cfg.num_attention_heads)
                heads = {"q_proj": cfg.num_attention_heads, "k_proj": cfg.num_key_value_heads,
                         "v_proj": cfg.num_key_value_heads, "o_proj": cfg.num_attention_heads}
                for proj in ("q_proj", "k_proj"):
                    key = f"{base}.{proj}"
                    w, s, ws = _packed(loaded_model, key)
                    _replace(loaded_model, key, _WBSW, slice_w4a16_qk_proj(
                        w, loaded_model.get(f"{key}.bias"), s, ws, cfg.hidden_size, heads[proj], head_dim,
                        block.head_dim, getattr(block, proj).weight.shape))
                for proj, cut in (("v_proj", slice_w4a16_v_proj), ("o_proj", slice_w4a16_o_proj)):
                    key = f"{base}.{proj}"
                    _replace(loaded_model, key, _WSW, cut(*_packed(loaded_model, key), cfg.hidden_size, heads[proj],
                                                          head_dim, block.head_dim, getattr(block, proj).weight.shape))
                if f"{base}.indices" in loaded_model:
                    loaded_model[f"{base}.indices"] = slice_indices(loaded_model[f"{base}.indices"], head_dim,
                                                                    block.head_dim)
            elif kind == model_helper.mamba_w4a16_uniql_class_name:
                base = model_helper.get_mamba_key(layer_idx)
                full_inner = model_helper.get_mamba_full_intermediate_size
                full_state = model_helper.get_mamba_full_ssm_state_size
                key = f"{base}.in_proj"
                _replace(loaded_model, key, _WSW, slice_w4a16_in_proj(
                    *_packed(loaded_model, key), hidden_size=cfg.hidden_size, n_groups=block.n_groups,
                    num_heads=block.num_heads, intermediate_size=full_inner, ssm_state_size=full_state,
                    load_intermediate_size=block.intermediate_size, load_ssm_state_size=block.ssm_state_size,
                    load_shape=block.in_proj.weight.shape))
                key = f"{base}.conv1d"
                _replace(loaded_model, key, ("weight", "bias"), slice_conv1d(
                    loaded_model[f"{key}.weight"], loaded_model[f"{key}.bias"], block.n_groups, block.num_heads,
                    full_inner, full_state, block.intermediate_size, block.ssm_state_size))
                loaded_model[f"{base}.norm.weight"] = slice_norm(
                    loaded_model[f"{base}.norm.weight"], block.n_groups, block.num_heads, full_inner,
                    block.intermediate_size)
                key = f"{base}.out_proj"
                _replace(loaded_model, key, _WSW, slice_w4a16_out_proj(
                    *_packed(loaded_model, key), hidden_size=cfg.hidden_size, n_groups=block.n_groups,
                    num_heads=block.num_heads, intermediate_size=full_inner,
                    load_intermediate_size=block.intermediate_size, load_shape=block.out_proj.weight.shape))
    return loaded_model
