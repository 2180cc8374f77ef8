"""CPU oracle for UniQL's W4A16 hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, in numpy / CPU torch, what the reference computes on the
path  pack -> (GPU) dequant + matmul,  the per-row int4 embedding lookup and
the Walsh-Hadamard rotation.  It is the checker that tests/, the smoke test
and the `cpu_baseline` leg of bench.py compare the HIP kernels against.  It is
never imported by the `uniql_amd` package: the product path has no CPU
fallback.

Every function names the reference lines it follows (paths relative to the
reference checkout).

Pinning status (what proves each function right, besides reading):
  * weight permutation / pack / unpack ....... golden vectors produced by the
    reference's own quantize_helpers + an independent closed-form index map
    + bijection / round-trip properties
  * scale permutations ....................... golden vectors + closed form
  * group-128 quantiser (code selection) ..... golden vectors
  * dequant fp16_rn((q-8)*s) ................. closed form, exhaustive in tests
  * dequant + matmul ......................... brute-force loops on tiny shapes
  * embedding quantise/pack/lookup ........... hand-computed cases + brute force.  The
    reference module cannot be imported without its compiled extension, so
    `embedding_quantize`'s code selection is pinned by rows worked out by hand where the
    rounding steps decide: halves (round to even), sums that only tie after the fp16
    rounding of `w / scale + 8`, a quotient whose own fp16 rounding moves the code, the
    same rows in float32 (different codes), the clamp, and an all-zero row
    (tests/test_oracle_golden.py::test_embedding_quantize_rounding_ties_by_hand)
  * module forward with its fp16 roundings, SiLU-gated and squared-ReLU MLP fronts
    (linear_forward_fp16, silu_fp16, mlp_gate_up, relu2_fp16) ... torch's own fp16 CPU
    operators over all finite fp16 inputs / random tensors (the reference calls exactly
    those operators)
  * rotary embedding with gathered frequencies (rope_indices) ... the textbook complex
    rotation in float64 for identity indices, an independently permuted frequency table,
    norm preservation, and torch's fp16 CPU arithmetic for the order of the roundings
  * power-of-two Hadamard .................... scipy.linalg.hadamard, involution,
    Parseval.
  * composite Hadamard widths (12N/20N/28N/40N, `fwht_composite`) ... PARITY UNPINNED against
    the reference: its base matrices live in an un-vendored third-party package
    (Dao-AILab fast-hadamard-transform, commit unknown; submodule empty in the
    reference tree).  What is pinned is the mathematics: the matrices built here
    (Sloane's 12 x 12, Paley I over GF(19), Paley II over GF(13), the doubled 20) satisfy
    H H^T = n I, the transform equals x @ kron(H_base, H_P) in float64, and
    HadLinear's fused and lazy forms agree.
"""
from __future__ import annotations

import math

import numpy as np
import torch

TILE = 16          # quantize_helpers.py:13  (GPTQ_MARLIN_TILE)
PACK = 8           # quantize_helpers.py:31-34 with num_bits = 4
GROUP = 128        # quantize_helpers.py:16   (only 128 and -1 are supported)
MIN_THREAD_N = 64  # quantize_helpers.py:10
MAX_PARALLEL = 16  # quantize_helpers.py:12


# --------------------------------------------------------------------------
# a1: weight permutation table and the nibble packer
# --------------------------------------------------------------------------
def weight_perm_table() -> np.ndarray:
    """1024-entry gather table.  Follows quantize_helpers.py:144-165."""
    out = []
    for lane in range(32):
        eight = []
        col = lane // 4
        for block in (0, 1):
            for row in (2 * (lane % 4), 2 * (lane % 4) + 1,
                        2 * (lane % 4 + 4), 2 * (lane % 4 + 4) + 1):
                eight.append(16 * row + col + 8 * block)
        for j in range(4):
            out.extend(p + 256 * j for p in eight)
    table = np.asarray(out, dtype=np.int64)
    interleave = np.array([0, 2, 4, 6, 1, 3, 5, 7])
    return table.reshape(-1, 8)[:, interleave].ravel()


def scale_perm_tables():
    """(grouped, per-channel) scale gather tables.  quantize_helpers.py:53-62."""
    grouped = []
    for i in range(8):
        grouped.extend(i + 8 * j for j in range(8))
    single = []
    for i in range(4):
        single.extend(2 * i + j for j in (0, 1, 8, 9, 16, 17, 24, 25))
    return np.asarray(grouped), np.asarray(single)


def tile_and_permute(q: np.ndarray) -> np.ndarray:
    """[K, N] codes -> [K/16, 16 N] in kernel order.  quantize_helpers.py:37-50."""
    k, n = q.shape
    assert k % TILE == 0 and n % TILE == 0
    t = q.reshape(k // TILE, TILE, n // TILE, TILE).transpose(0, 2, 1, 3)
    t = t.reshape(k // TILE, n * TILE)
    perm = weight_perm_table()
    return t.reshape(-1, perm.size)[:, perm].reshape(t.shape)


def pack_weights(q: np.ndarray) -> np.ndarray:
    """[K, N] codes in 0..15 -> int32 [K/16, 2 N].  quantize_helpers.py:66-84."""
    t = tile_and_permute(np.asarray(q)).astype(np.uint32)
    packed = np.zeros((t.shape[0], t.shape[1] // PACK), dtype=np.uint32)
    for i in range(PACK):
        packed |= t[:, i::PACK] << np.uint32(4 * i)
    return packed.view(np.int32)


def unpack_weights(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """int32 [K/16, 2 N] -> [K, N] codes.  quantize_helpers.py:278-328."""
    u = np.ascontiguousarray(packed).view(np.uint32)
    assert u.shape == (size_k // TILE, size_n * TILE // PACK)
    t = np.zeros((u.shape[0], u.shape[1] * PACK), dtype=np.uint32)
    for i in range(PACK):
        t[:, i::PACK] = (u >> np.uint32(4 * i)) & np.uint32(0xF)
    perm = weight_perm_table()
    inv = np.empty_like(perm)
    inv[perm] = np.arange(perm.size)
    t = t.reshape(-1, perm.size)[:, inv].reshape(size_k // TILE, size_n * TILE)
    t = t.reshape(size_k // TILE, size_n // TILE, TILE, TILE).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(t.reshape(size_k, size_n)).astype(np.int32)


# --------------------------------------------------------------------------
# a2: scale permutation
# --------------------------------------------------------------------------
def _grouped(size_k: int, group_size: int) -> bool:
    # quantize_helpers.py:171 / :259
    return group_size < size_k and group_size != -1


def permute_scales(scale: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    """quantize_helpers.py:168-180."""
    grouped, single = scale_perm_tables()
    tab = grouped if _grouped(size_k, group_size) else single
    return np.ascontiguousarray(scale.reshape(-1, tab.size)[:, tab].reshape(-1, size_n))


def unpermute_scales(scale: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    """quantize_helpers.py:244-275."""
    grouped, single = scale_perm_tables()
    tab = grouped if _grouped(size_k, group_size) else single
    inv = np.argsort(tab)
    return np.ascontiguousarray(scale.reshape(-1, tab.size)[:, inv].reshape(-1, size_n))


# --------------------------------------------------------------------------
# a3: the group-128 symmetric quantiser (fp16 arithmetic on the CPU)
# --------------------------------------------------------------------------
@torch.no_grad()
def fake_quantize_grouped(w: torch.Tensor, group_size: int = GROUP):
    """fp16 [K, N] -> (w_ref fp16 [Kp, N], codes int32 [Kp, N], scale fp16 [Kp/g, N]).

    Follows quantize_helpers.py:87-121 (the per-group branch): the arithmetic
    is done by CPU torch in the tensor's own dtype, as the reference does.
    """
    size_k, size_n = w.shape
    assert group_size < size_k
    pad_k = (-size_k) % group_size
    if pad_k:
        w = torch.nn.functional.pad(w, (0, 0, 0, pad_k))
    g = w.reshape(-1, group_size, size_n)
    scale = g.abs().max(dim=1, keepdim=True)[0]
    scale *= 2 / 15
    q = torch.round(g / scale).int()      # NaN (0/0): INT_MIN on x86 (golden vectors), code 0 after the clamp
    q += 8
    q = torch.clamp(q, 0, 15)
    w_ref = (q - 8) * scale
    return (w_ref.reshape(-1, size_n).contiguous(),
            q.reshape(-1, size_n).contiguous(),
            scale.reshape(-1, size_n).contiguous())


@torch.no_grad()
def requantize_with_scales(w: torch.Tensor, scale: torch.Tensor, group_size: int = GROUP):
    """Codes for weights that were already fake-quantised with the given
    group scales (the GPTQ branch).  quantize_helpers.py:205-218."""
    size_k, size_n = w.shape
    pad_k = (-size_k) % group_size
    if pad_k:
        w = torch.nn.functional.pad(w, (0, 0, 0, pad_k))
    w_ref = w.clone()
    g = w.reshape(-1, group_size, size_n)
    q = ((g / scale.unsqueeze(1)) + 8).round().int()
    q = torch.clamp(q, 0, 15).reshape(size_k + pad_k, size_n).contiguous()
    return w_ref, q, scale


@torch.no_grad()
def w4a16_quantize(w: torch.Tensor, group_size: int = GROUP, scale: torch.Tensor | None = None,
                   pad_out: int = 0):
    """fp16 [K, N] -> (w_ref, packed int32 [Kp/16, 2 Np], permuted scale fp16 [Kp/g, Np]).

    Follows quantize_helpers.py:183-241 for the group-128 case.  The
    per-channel case (in_features <= 128) packs signed codes unmasked in the
    reference (quantize_helpers.py:123-135 with :75-80), which no supported
    model reaches; it is not restated.
    """
    size_k, size_n = w.shape
    assert group_size == GROUP and group_size < size_k
    if scale is None:
        w_ref, q, scale = fake_quantize_grouped(w, group_size)
    else:
        w_ref, q, scale = requantize_with_scales(w, scale, group_size)
    if pad_out:
        w_ref = torch.nn.functional.pad(w_ref, (0, pad_out))
        q = torch.nn.functional.pad(q, (0, pad_out))
        scale = torch.nn.functional.pad(scale, (0, pad_out))
    kp, np_ = w_ref.shape
    packed = torch.from_numpy(pack_weights(q.numpy()))
    s_perm = torch.from_numpy(permute_scales(scale.numpy(), kp, np_, group_size))
    return w_ref, packed, s_perm


# --------------------------------------------------------------------------
# a9: dequantisation, and the reference's CPU meaning of the linear layer
# --------------------------------------------------------------------------
def dequant_codes(q: np.ndarray, scale: np.ndarray, group_size: int = GROUP) -> np.ndarray:
    """codes [K, N], natural-order scale fp16 [K/g or 1, N] -> fp16 [K, N].

    w = fp16_rn(float(q - 8) * float(s)):  marlin_gemm_kernel.cuh:118-146 (the
    magic-number conversion yields q-8 exactly, then one fp16 multiply), equal
    to the CPU expression at quantize_helpers.py:118 and
    modeling/modeling_helpers.py:632-640.
    """
    k, n = q.shape
    s = np.asarray(scale, dtype=np.float16)
    if s.shape[0] == 1:
        s_full = np.broadcast_to(s, (k, n))
    else:
        s_full = np.repeat(s, group_size, axis=0)
    prod = (q.astype(np.float32) - 8.0) * s_full.astype(np.float32)   # exact in fp32
    return prod.astype(np.float16)


def dequant_packed(packed: np.ndarray, scale_perm: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Packed kernel-layout tensors -> dequantised fp16 [K, N]."""
    groups = scale_perm.shape[0]
    group_size = size_k // groups if groups > 1 else -1   # marlin_gemm_kernel.cuh:1008
    q = unpack_weights(packed, size_k, size_n)
    s = unpermute_scales(np.asarray(scale_perm), size_k, size_n,
                         group_size if group_size != -1 else size_k)
    return dequant_codes(q, s, group_size if group_size != -1 else size_k)


def gemm_fp32(x: np.ndarray, w_deq: np.ndarray) -> np.ndarray:
    """fp16 [M, K] x fp16 [K, N] -> float32 [M, N], accumulated in (at least)
    fp32.  The textbook product the kernel must match
    (marlin_gemm_kernel.cuh:443-462: fp16 operands, fp32 accumulate)."""
    xt = torch.from_numpy(np.ascontiguousarray(x)).to(torch.float32)
    wt = torch.from_numpy(np.ascontiguousarray(w_deq)).to(torch.float32)
    return torch.matmul(xt, wt).numpy()


def gemm_fp64(x: np.ndarray, w_deq: np.ndarray) -> np.ndarray:
    """Same product accumulated in float64 (the exact value up to 1e-13)."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w_deq, dtype=np.float64)


def linear_forward(x: np.ndarray, packed: np.ndarray, scale_perm: np.ndarray, *,
                   in_features: int, out_features: int, bias: np.ndarray | None = None,
                   exact: bool = False) -> np.ndarray:
    """What W4A16B16O16Linear.forward returns, before the final fp16 rounding.

    quant_linear_layers.py:91-116: flatten, zero-pad K, product, drop padded
    output columns, restore leading shape, add bias.
    Returns float32 (or float64 if exact) of shape (*x.shape[:-1], out_features).
    """
    size_k = packed.shape[0] * TILE
    size_n = packed.shape[1] * PACK // TILE
    lead = x.shape[:-1]
    x2 = np.asarray(x, dtype=np.float16).reshape(-1, x.shape[-1])
    assert x2.shape[1] == in_features
    if size_k != in_features:
        x2 = np.pad(x2, ((0, 0), (0, size_k - in_features)))
    w = dequant_packed(packed, scale_perm, size_k, size_n)
    y = gemm_fp64(x2, w) if exact else gemm_fp32(x2, w)
    y = y[:, :out_features].reshape(*lead, out_features)
    if bias is not None:
        y = y + np.asarray(bias, dtype=y.dtype)
    return y


def linear_forward_fp16(x: np.ndarray, packed: np.ndarray, scale_perm: np.ndarray, *, in_features: int,
                        out_features: int, bias: np.ndarray | None = None) -> np.ndarray:
    """The module's fp16 result with its roundings: the kernel's fp32-accumulated product is
    rounded to fp16 (marlin_gemm_kernel.cuh:560-606 writes halves), then `y + self.bias`
    (quant_linear_layers.py:113-114) adds two fp16 tensors and rounds again.  The float64
    product stands in for the fp32 accumulation (they differ by ~1e-6 relative)."""
    y = linear_forward(x, packed, scale_perm, in_features=in_features, out_features=out_features,
                       exact=True).astype(np.float16)
    if bias is not None:
        y = (y.astype(np.float32) + np.asarray(bias, dtype=np.float16).astype(np.float32)).astype(np.float16)
    return y


def silu_fp16(x: np.ndarray) -> np.ndarray:
    """torch.nn.SiLU on an fp16 tensor (ACT2FN["silu"], llama_qblocks.py:36): the value is
    computed in fp32 as x / (1 + exp(-x)) and rounded to fp16."""
    x32 = np.asarray(x, dtype=np.float16).astype(np.float32)
    with np.errstate(over="ignore"):
        return (x32 / (np.float32(1.0) + np.exp(-x32))).astype(np.float16)


def mlp_gate_up(gate16: np.ndarray, up16: np.ndarray) -> np.ndarray:
    """act_fn(gate_proj(x)) * up_proj(x) on the two layers' fp16 outputs
    (llama_qblocks.py:48-49): SiLU rounds to fp16, the product of two fp16 tensors rounds
    again."""
    a = silu_fp16(gate16).astype(np.float32)
    with np.errstate(over="ignore"):
        return (a * np.asarray(up16, dtype=np.float16).astype(np.float32)).astype(np.float16)


def relu2_fp16(y16: np.ndarray) -> np.ndarray:
    """act_fn(up_proj(x)) of the un-gated MLP with mlp_hidden_act = "relu2"
    (nemotron_h_qblocks.py:577,588; transformers' ReLUSquaredActivation: relu, then
    torch.square) on the layer's fp16 output: the exact square rounded once to fp16."""
    r = np.maximum(np.asarray(y16, dtype=np.float16).astype(np.float32), np.float32(0.0))
    with np.errstate(over="ignore"):
        return (r * r).astype(np.float16)


# --------------------------------------------------------------------------
# a10/a11: int4 embedding with one scale per vocabulary row
# --------------------------------------------------------------------------
EMB_INTERLEAVE = np.array([0, 2, 4, 6, 1, 3, 5, 7])   # quant_embedding_layers.py:33


@torch.no_grad()
def embedding_quantize(w: torch.Tensor):
    """[V, D] float -> (packed int32 [V, D/8], scales fp16 [V]).

    quant_embedding_layers.py:35-46: arithmetic in the weight's own dtype.
    """
    v, d = w.shape
    scales = w.abs().amax(dim=-1, keepdim=True) / 8
    q = torch.round((w / scales) + 8).clamp(0, 15)
    q = q.to(torch.int32).numpy().astype(np.uint32)
    q = q.reshape(v, -1, 8)[:, :, EMB_INTERLEAVE].reshape(v, -1)
    packed = np.zeros((v, d // PACK), dtype=np.uint32)
    for i in range(PACK):
        packed |= (q[:, i::PACK] & np.uint32(0xF)) << np.uint32(4 * i)
    return packed.view(np.int32), scales.flatten().to(torch.float16).numpy()


def embedding_unpack(packed: np.ndarray) -> np.ndarray:
    """int32 [V, D/8] -> codes [V, D] in natural element order (inverse of the
    interleaved packing at quant_embedding_layers.py:39-43)."""
    u = np.ascontiguousarray(packed).view(np.uint32)
    v, words = u.shape
    codes = np.zeros((v, words, 8), dtype=np.int32)
    for i in range(PACK):
        codes[:, :, EMB_INTERLEAVE[i]] = ((u >> np.uint32(4 * i)) & np.uint32(0xF)).astype(np.int32)
    return codes.reshape(v, words * 8)


def embedding_lookup(ids: np.ndarray, packed: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """out[..., :] = fp16_rn((code - 8) * scale[id]).
    quant_embedding_kernel.cuh:47-76 (conversion exact, one fp16 multiply) and
    :80-114 (one scale per token row, natural output order)."""
    ids = np.asarray(ids)
    rows = embedding_unpack(packed[ids.reshape(-1)])
    s = np.asarray(scales, dtype=np.float16)[ids.reshape(-1)].astype(np.float32)[:, None]
    out = ((rows.astype(np.float32) - 8.0) * s).astype(np.float16)
    return out.reshape(*ids.shape, rows.shape[1])


# --------------------------------------------------------------------------
# a12/a13: Walsh-Hadamard rotation
# --------------------------------------------------------------------------
def is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0     # hadamard_helpers.py:4-5


def had_variant(dim: int):
    """(base N, scale) chosen for a width.  hadamard_helpers.py:18-36."""
    scale = 1.0 / math.sqrt(dim)
    for base in (40, 28, 20, 12):
        if dim % base == 0 and is_pow2(dim // base):
            return base, scale
    assert is_pow2(dim), f"Invalid dim: {dim}. dim must be a power of 2."
    return 2, scale


def fwht(x: np.ndarray, scale: float, block: int | None = None,
         acc=np.float32) -> np.ndarray:
    """y = (x . H_block) * scale along the last axis, H the Sylvester
    (natural-order) Hadamard matrix, applied independently to consecutive
    `block`-wide pieces (block = whole width by default).  Internal arithmetic
    in `acc`, result rounded to x's dtype: the contract of
    fast_hadamard_transform(x, scale) as called at hadamard_helpers.py:35,45
    and quant_hadamard_layers.py:18.
    """
    dim = x.shape[-1]
    block = dim if block is None else block
    assert is_pow2(block) and dim % block == 0
    y = np.asarray(x).astype(acc).reshape(-1, dim // block, block).copy()
    h = 1
    while h < block:
        y = y.reshape(y.shape[0], y.shape[1], block // (2 * h), 2, h)
        a = y[:, :, :, 0, :].copy()
        b = y[:, :, :, 1, :].copy()
        y[:, :, :, 0, :] = a + b
        y[:, :, :, 1, :] = a - b
        y = y.reshape(y.shape[0], y.shape[1], block)
        h *= 2
    y = y * acc(scale)
    return y.reshape(x.shape).astype(x.dtype)


def _legendre(a: int, q: int) -> int:
    a %= q
    if a == 0:
        return 0
    return 1 if pow(a, (q - 1) // 2, q) == 1 else -1


def hadamard_base_matrix(base: int) -> np.ndarray:
    """The base x base Hadamard matrix behind fast_hadamard_transform_{base}N
    (hadamard_helpers.py:20-31).  The reference's own tables are not in its tree (parity
    unpinned); these are textbook constructions: 12 Sloane's "had.12" (first row + - ... -, the
    other rows cyclic shifts of + + - + - - - + + + - + behind a leading +), 20 Paley I over
    GF(19), 28 Paley II over GF(13), 40 the Sylvester doubling of the 20."""
    if base == 12:
        core = [1, -1, 1, -1, -1, -1, 1, 1, 1, -1, 1]
        h = np.ones((12, 12), dtype=np.int64)
        h[0, 1:] = -1
        for r in range(11):
            h[1 + r, 1:] = np.roll(core, r)
        return h
    if base == 20:
        q = 19
        jac = np.array([[_legendre(i - j, q) for j in range(q)] for i in range(q)], dtype=np.int64)
        s = np.zeros((q + 1, q + 1), dtype=np.int64)
        s[0, 1:] = 1
        s[1:, 0] = -1
        s[1:, 1:] = jac
        return s + np.eye(q + 1, dtype=np.int64)
    if base == 28:
        q = 13
        jac = np.array([[_legendre(i - j, q) for j in range(q)] for i in range(q)], dtype=np.int64)
        s = np.zeros((q + 1, q + 1), dtype=np.int64)
        s[0, 1:] = 1
        s[1:, 0] = 1
        s[1:, 1:] = jac
        eye = np.eye(q + 1, dtype=np.int64)
        return np.block([[s + eye, s - eye], [s - eye, -s - eye]])
    if base == 40:
        h20 = hadamard_base_matrix(20)
        return np.block([[h20, h20], [h20, -h20]])
    raise ValueError(f"no base matrix of order {base}")


def fwht_composite(x: np.ndarray, scale: float, base: int, acc=np.float32) -> np.ndarray:
    """y = (x . (H_base (x) H_P)) * scale along the last axis of width base * P: the P-point
    transform inside each of the `base` chunks, then the base matrix across the chunks, added in
    ascending chunk order; arithmetic in `acc`, one rounding to x's dtype.  The contract of
    fast_hadamard_transform_{12,20,28,40}N(x, scale) as called at hadamard_helpers.py:20-31,45."""
    dim = x.shape[-1]
    p = dim // base
    assert base * p == dim and is_pow2(p)
    z = fwht(np.asarray(x).astype(acc), 1.0, block=p, acc=acc).reshape(-1, base, p)
    h = hadamard_base_matrix(base)
    y = np.zeros_like(z)
    for c in range(base):
        total = np.zeros((z.shape[0], p), dtype=acc)
        for cp in range(base):
            total = total + (z[:, cp, :] if h[cp, c] > 0 else -z[:, cp, :])
        y[:, c, :] = total
    y = y * acc(scale)
    return y.reshape(x.shape).astype(x.dtype)


def hadamard_module_forward(x: np.ndarray, dim: int) -> np.ndarray:
    """Hadamard(dim).forward(x).  quant_hadamard_layers.py:5-21."""
    base, scale = had_variant(dim)
    if base != 2:
        return fwht_composite(x, scale, base)
    return fwht(x, scale)


def hadlinear_fused_weight(w: np.ndarray, input_transform: bool = True,
                           output_transform: bool = False) -> np.ndarray:
    """HadLinear.fuse_hadamard on W [Dout, Din].  quant_linear_layers.py:159-167."""
    w = np.asarray(w)
    if input_transform:
        w = fwht(w, 1.0 / math.sqrt(w.shape[1]))
    if output_transform:
        w = np.ascontiguousarray(fwht(np.ascontiguousarray(w.T), 1.0 / math.sqrt(w.shape[0])).T)
    return w


# --------------------------------------------------------------------------
# module buffer geometry (a4)
# --------------------------------------------------------------------------
def linear_geometry(in_features: int, out_features: int, group_size: int = GROUP):
    """Padded sizes and buffer shapes.  quant_linear_layers.py:13-48."""
    pad_out = (-out_features) % 256
    pad_in = (-in_features) % group_size
    size_n, size_k = out_features + pad_out, in_features + pad_in
    return dict(size_n=size_n, size_k=size_k, pad_in=pad_in, pad_out=pad_out,
                workspace=(size_n // MIN_THREAD_N) * MAX_PARALLEL,
                weight=(size_k // 16, size_n * 16 // 8),
                scale=(size_k // group_size, size_n))


# --------------------------------------------------------------------------
# rotary embedding with per-head gathered frequencies (pruned attention heads)
# --------------------------------------------------------------------------
def rope_indices(q: np.ndarray, k: np.ndarray, cos: np.ndarray, sin: np.ndarray, indices: np.ndarray):
    """apply_rotary_pos_emb_indices (modeling/llama/llama_rope.py:38-96) on fp16 arrays.

    q [b, hq, s, d], k [b, hk, s, d]; cos, sin [b or 1, s, D] (D = the unpruned head width);
    indices [hk, d] integer: which of the D table columns each kept column of a key/value head
    uses; query head h uses row h // (hq / hk) (repeat_interleave, :80).
    out = x * cos_g + rotate_half(x) * sin_g with every product and the sum rounded to fp16,
    as torch does for fp16 tensors (:94-95; rotate_half :4-8 negates the upper half exactly).
    """
    q = np.asarray(q, dtype=np.float16)
    k = np.asarray(k, dtype=np.float16)
    b, hq, s, d = q.shape
    hk = k.shape[1]
    assert indices.shape == (hk, d) and hq % hk == 0
    idx = np.asarray(indices, dtype=np.int64)
    cos = np.broadcast_to(np.asarray(cos, dtype=np.float16), (b, s, cos.shape[-1]))
    sin = np.broadcast_to(np.asarray(sin, dtype=np.float16), (b, s, sin.shape[-1]))

    def rotate(x, head_rows):
        # cos_g[b, h, s, j] = cos[b, s, idx[row(h), j]]
        cg = np.transpose(cos[:, :, idx[head_rows]], (0, 2, 1, 3)).astype(np.float32)
        sg = np.transpose(sin[:, :, idx[head_rows]], (0, 2, 1, 3)).astype(np.float32)
        half = d // 2
        rot = np.concatenate((-x[..., half:], x[..., :half]), axis=-1).astype(np.float32)
        a = (x.astype(np.float32) * cg).astype(np.float16)
        r = (rot * sg).astype(np.float16)
        return (a.astype(np.float32) + r.astype(np.float32)).astype(np.float16)

    return rotate(q, np.arange(hq) // (hq // hk)), rotate(k, np.arange(hk))
