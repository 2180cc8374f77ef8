"""Packed W4A16 tensor formats, written as index algebra.

The kernel format groups K in rows of 16 and N in chunks of 64.  Splitting the
indices into bit fields

    k = 16 r + 8 hi + 2 a + lo          (hi, lo in {0,1}; a in 0..3)
    n = 64 c + 16 j + 8 blk + c8        (j in 0..3; blk in {0,1}; c8 in 0..7)

the 32-bit word at packed[r, 128 c + 16 c8 + 4 a + j] stores code q[k, n] in the
nibble at bit 4 p with p = 4 lo + 2 blk + hi.  Packing is therefore one reshape,
one axis permutation and a shift-sum; no lookup table is needed.  (The table
form is quantize/quantize_helpers.py:37-50,66-84,144-165 of the reference; the
test-suite checks both forms against each other and against vectors produced by
the reference.)

All functions take and return torch tensors and run on whatever device the
input lives on.
"""
from __future__ import annotations

import torch

GROUP_SIZE = 128
TILE_K = 16
CHUNK_N = 64
PACK_FACTOR = 8
MIN_THREAD_N = 64      # granularity of the module's workspace buffer
MAX_PARALLEL = 16

_SHIFTS = torch.arange(0, 32, 4, dtype=torch.int64)


def pack_codes(q: torch.Tensor) -> torch.Tensor:
    """codes [K, N] in 0..15 (any integer dtype) -> int32 [K/16, 2N]."""
    k, n = q.shape
    if k % TILE_K or n % CHUNK_N:
        raise ValueError(f"pack_codes needs K % 16 == 0 and N % 64 == 0, got {k}x{n}")
    r, c = k // TILE_K, n // CHUNK_N
    #            r  hi a  lo c  j  blk c8
    v = q.reshape(r, 2, 4, 2, c, 4, 2, 8).to(torch.int64)
    #            r  c  c8 a  j  lo blk hi
    v = v.permute(0, 4, 7, 2, 5, 3, 6, 1).reshape(r, c * 128, 8)
    word = ((v & 0xF) << _SHIFTS.to(v.device)).sum(dim=-1)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)   # two's complement view
    return word.to(torch.int32).contiguous()


def unpack_codes(packed: torch.Tensor, size_k: int, size_n: int) -> torch.Tensor:
    """int32 [K/16, 2N] -> codes int32 [K, N]."""
    r, c = size_k // TILE_K, size_n // CHUNK_N
    if tuple(packed.shape) != (r, 2 * size_n):
        raise ValueError(f"packed shape {tuple(packed.shape)} does not match K={size_k}, N={size_n}")
    w = packed.to(torch.int64) & 0xFFFFFFFF
    v = (w.unsqueeze(-1) >> _SHIFTS.to(w.device)) & 0xF          # [r, 2N, p]
    #            r  c  c8 a  j  lo blk hi
    v = v.reshape(r, c, 8, 4, 4, 2, 2, 2)
    #            r  hi a  lo c  j  blk c8
    v = v.permute(0, 7, 3, 5, 1, 4, 6, 2).reshape(size_k, size_n)
    return v.to(torch.int32).contiguous()


def _is_grouped(size_k: int, group_size: int) -> bool:
    return group_size != -1 and group_size < size_k


def permute_scales(scale: torch.Tensor, size_k: int, size_n: int, group_size: int) -> torch.Tensor:
    """Natural-order scales [G, N] -> kernel order.

    Grouped: every 64-column block is an 8x8 transpose (position 8 i + j holds
    column i + 8 j).  One scale row: every 32-column block, seen as
    [hi(4), i(4), lo(2)], is stored as [i, hi, lo].
    (quantize_helpers.py:53-62,168-180)
    """
    if _is_grouped(size_k, group_size):
        if group_size != GROUP_SIZE:
            raise ValueError("only group size 128 is supported")
        out = scale.reshape(-1, 8, 8).transpose(1, 2)
    else:
        out = scale.reshape(-1, 4, 4, 2).permute(0, 2, 1, 3)
    return out.reshape(-1, size_n).contiguous()


def unpermute_scales(scale: torch.Tensor, size_k: int, size_n: int, group_size: int) -> torch.Tensor:
    """Inverse of permute_scales (quantize_helpers.py:244-275)."""
    if _is_grouped(size_k, group_size):
        out = scale.reshape(-1, 8, 8).transpose(1, 2)       # a transpose is its own inverse
    else:
        out = scale.reshape(-1, 4, 4, 2).permute(0, 2, 1, 3)  # swapping two axes too
    return out.reshape(-1, size_n).contiguous()


@torch.no_grad()
def quantize_groupwise(w: torch.Tensor, group_size: int = GROUP_SIZE):
    """Symmetric int4 codes with one scale per (group of 128 K, column).

    w: float [K, N].  Returns (w_ref [Kp, N], codes int32 [Kp, N], scale [Kp/g, N])
    with K zero-padded to a multiple of the group.  The arithmetic runs in w's
    dtype with the operation order of quantize_helpers.py:108-118, which is
    what decides ties and the all-zero-group case (0/0 = NaN, whose conversion to int32 gives
    INT_MIN on x86 and so code 0 after the clamp; with scale 0 the weight is -0.0 either way).
    """
    size_k, size_n = w.shape
    pad = (-size_k) % group_size
    if pad:
        w = torch.cat([w, w.new_zeros(pad, size_n)], dim=0)
    grp = w.view(-1, group_size, size_n)
    scale = grp.abs().amax(dim=1, keepdim=True)
    scale.mul_(2 / 15)
    codes = torch.round(grp / scale).int().add_(8).clamp_(0, 15)
    w_ref = (codes - 8) * scale
    return (w_ref.reshape(-1, size_n).contiguous(), codes.reshape(-1, size_n).contiguous(),
            scale.reshape(-1, size_n).contiguous())


@torch.no_grad()
def codes_from_scales(w: torch.Tensor, scale: torch.Tensor, group_size: int = GROUP_SIZE):
    """Codes of already fake-quantised weights given their group scales
    (the GPTQ hand-over, quantize_helpers.py:205-218)."""
    size_k, size_n = w.shape
    pad = (-size_k) % group_size
    if pad:
        w = torch.cat([w, w.new_zeros(pad, size_n)], dim=0)
    grp = w.view(-1, group_size, size_n)
    codes = (grp / scale.unsqueeze(1) + 8).round().int().clamp_(0, 15)
    return w.clone(), codes.reshape(-1, size_n).contiguous(), scale


@torch.no_grad()
def quantize_and_pack(w: torch.Tensor, group_size: int = GROUP_SIZE, scale: torch.Tensor | None = None,
                      pad_out: int = 0):
    """fp16 [K, N] -> (w_ref [Kp, Np], packed int32 [Kp/16, 2 Np], kernel-order scale [Kp/g, Np]).
    Mirrors w4a16_quantize (quantize_helpers.py:183-241) for group size 128."""
    size_k, _ = w.shape
    if group_size != GROUP_SIZE or size_k <= group_size:
        raise NotImplementedError(
            "per-column quantisation (in_features <= 128) is not produced: the reference packs its "
            "signed codes unmasked; only group size 128 is supported")
    if scale is None:
        w_ref, codes, scale = quantize_groupwise(w, group_size)
    else:
        w_ref, codes, scale = codes_from_scales(w, scale, group_size)
    if pad_out:
        zeros = lambda t: t.new_zeros(t.shape[0], pad_out)
        w_ref = torch.cat([w_ref, zeros(w_ref)], dim=1)
        codes = torch.cat([codes, zeros(codes)], dim=1)
        scale = torch.cat([scale, zeros(scale)], dim=1)
    kp, np_ = w_ref.shape
    return w_ref, pack_codes(codes), permute_scales(scale, kp, np_, group_size)


# ---- fusing layers that read the same input ---------------------------------------------
def concat_columns(weights, scales):
    """Packed tensors of layers with the same K, side by side along N: the packed words and the
    permuted scales of every 64-column block are contiguous, so this is a plain concatenation
    (every width must be a multiple of 64; the module pads to 256)."""
    for w, s in zip(weights, scales):
        if s.shape[1] % CHUNK_N or w.shape[1] != 2 * s.shape[1]:
            raise ValueError("every layer must be padded to a multiple of 64 columns")
    return torch.cat(list(weights), dim=1).contiguous(), torch.cat(list(scales), dim=1).contiguous()


def interleave_gate_up(gate_w, gate_s, up_w, up_s):
    """Gate and up projection interleaved in blocks of 64 columns (block 2c = columns 64c.. of
    gate, block 2c+1 = the same columns of up): the layout the kernels' silu(gate) * up
    epilogue reads.  Returns (packed int32 [K/16, 4 Np], scale fp16 [G, 2 Np])."""
    if gate_w.shape != up_w.shape or gate_s.shape != up_s.shape:
        raise ValueError("gate and up projections must have the same shape")
    rows, words = gate_w.shape
    groups, n_pad = gate_s.shape
    if n_pad % CHUNK_N or words != 2 * n_pad:
        raise ValueError("projections must be padded to a multiple of 64 columns")
    blocks = n_pad // CHUNK_N
    w = torch.stack((gate_w.view(rows, blocks, 2 * CHUNK_N), up_w.view(rows, blocks, 2 * CHUNK_N)), dim=2)
    s = torch.stack((gate_s.view(groups, blocks, CHUNK_N), up_s.view(groups, blocks, CHUNK_N)), dim=2)
    return w.reshape(rows, 2 * words).contiguous(), s.reshape(groups, 2 * n_pad).contiguous()


# ---- embedding table: one scale per row, 8 codes per word, nibble i <- element [0,2,4,6,1,3,5,7][i]
def pack_embedding_codes(codes: torch.Tensor) -> torch.Tensor:
    """codes [V, D] in 0..15 -> int32 [V, D/8] (quant_embedding_layers.py:39-43)."""
    v, d = codes.shape
    if d % PACK_FACTOR:
        raise ValueError("embedding_dim must be a multiple of 8")
    # element e = 2 pair + odd sits in nibble 4 odd + pair
    x = codes.reshape(v, d // 8, 4, 2).to(torch.int64) & 0xF
    x = x.transpose(2, 3).reshape(v, d // 8, 8)
    word = (x << _SHIFTS.to(x.device)).sum(dim=-1)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32).contiguous()


def unpack_embedding_codes(packed: torch.Tensor) -> torch.Tensor:
    v, words = packed.shape
    w = packed.to(torch.int64) & 0xFFFFFFFF
    x = (w.unsqueeze(-1) >> _SHIFTS.to(w.device)) & 0xF       # [v, words, nibble = 4 odd + pair]
    x = x.reshape(v, words, 2, 4).transpose(2, 3).reshape(v, words * 8)
    return x.to(torch.int32).contiguous()


@torch.no_grad()
def quantize_embedding(w: torch.Tensor):
    """[V, D] float -> (packed int32 [V, D/8], scales fp16 [V]); arithmetic in w's dtype
    (quant_embedding_layers.py:35-37)."""
    scales = w.abs().amax(dim=-1, keepdim=True) / 8
    codes = torch.round(w / scales + 8).clamp_(0, 15).to(torch.int32)
    return pack_embedding_codes(codes), scales.flatten().to(torch.float16)
