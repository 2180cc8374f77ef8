"""Names of the reference's quantize/quantize_helpers.py, backed by the index
algebra in uniql_amd.layout.  Callers that slice packed checkpoints
(modeling/modeling_helpers.py:235-867 in the reference) use exactly these
functions, with these argument lists."""
from __future__ import annotations

import torch

from .. import layout

MARLIN_QQQ_TILE = 16
MARLIN_QQQ_MIN_THREAD_N = layout.MIN_THREAD_N
MARLIN_QQQ_MIN_THREAD_K = 128
MARLIN_QQQ_MAX_PARALLEL = layout.MAX_PARALLEL
GPTQ_MARLIN_TILE = 16
SUPPORTED_NUM_BITS = [4]
SUPPORTED_GROUP_SIZES = [-1, 128]


def get_pack_factor(num_bits: int) -> int:
    if 32 % num_bits:
        raise AssertionError(f"Unsupported num_bits = {num_bits}")
    return 32 // num_bits


def get_scale_perms():
    """(grouped, single-row) gather tables, derived from the transposes in layout."""
    grouped = layout.permute_scales(torch.arange(64).reshape(1, 64), 256, 64, 128).flatten().tolist()
    single = layout.permute_scales(torch.arange(32).reshape(1, 32), 128, 32, 128).flatten().tolist()
    return grouped, single


def get_w4a16_weight_perms() -> torch.Tensor:
    """The 1024-entry gather table of the 16x64 tile order, derived by packing an index
    ramp: entry 8 w + p is the tile-local position (16 columns x ... ) stored in nibble p of word w."""
    # tile-major value of element (k, n) inside one 16 x 64 row block: 256 (n/16) + 16 k + n%16
    k = torch.arange(16).reshape(16, 1)
    n = torch.arange(64).reshape(1, 64)
    pos = 256 * (n // 16) + 16 * k + (n % 16)                       # [16, 64], values 0..1023
    table = torch.empty(1024, dtype=torch.int64)
    # pack 4 bits at a time: three ramps of 4 bits would do, simpler to unpack positions directly
    for bit in range(0, 12, 4):
        codes = (pos >> bit) & 0xF
        words = layout.pack_codes(codes)                              # [1, 128]
        nib = (words.to(torch.int64).unsqueeze(-1) >> torch.arange(0, 32, 4)) & 0xF
        part = nib.reshape(-1)
        table = part << bit if bit == 0 else table | (part << bit)
    return table


def get_w4a16_permute_weights(q_w, size_k, size_n, num_bits, perm=None, group_size=128):
    assert num_bits == 4
    return layout.pack_codes(q_w.reshape(size_k, size_n))


def unpack_w4a16_permute_weights(q_packed, size_k, size_n, num_bits, perm=None, group_size=128):
    assert num_bits == 4
    return layout.unpack_codes(q_packed, size_k, size_n)


def w4a16_permute_scales(scale, size_k, size_n, group_size):
    return layout.permute_scales(scale, size_k, size_n, group_size)


def w4a16_unpermute_scales(permuted_scale, size_k, size_n, group_size):
    return layout.unpermute_scales(permuted_scale, size_k, size_n, group_size)


def get_fake_quantize_weights(w: torch.Tensor, num_bits: int, group_size: int = -1):
    assert num_bits == 4 and w.is_floating_point()
    if group_size == -1 or group_size >= w.shape[0]:
        raise NotImplementedError("per-column quantisation is not produced (see uniql_amd.layout.quantize_and_pack)")
    return layout.quantize_groupwise(w, group_size)


def w4a16_quantize(w: torch.Tensor, num_bits: int, group_size: int = -1, scale: torch.Tensor = None,
                   pad_out: int = 0):
    assert num_bits in SUPPORTED_NUM_BITS, f"Unsupported num_bits = {num_bits}"
    if group_size == -1:
        group_size = w.shape[0]
    w_ref, packed, s = layout.quantize_and_pack(w, group_size, scale, pad_out)
    return [w_ref, packed, s]
