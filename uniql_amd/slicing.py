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
