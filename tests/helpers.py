"""Seeded synthetic problems (the benchmark's generator) and comparison rules."""
import numpy as np
import torch

from oracle import uniql_oracle as O

SEED = 1234


def make_linear_problem(m, k, n, seed=SEED, per_column=False):
    """codes U{0..15}, scales U[0.004, 0.02] fp16, activations N(0,1) fp16; packed by the oracle."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    groups = 1 if per_column else k // 128
    s = rng.uniform(0.004, 0.02, size=(groups, n)).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    packed = O.pack_weights(q)
    s_perm = O.permute_scales(s, k, n, k if groups == 1 else 128)
    return dict(q=q, s=s, x=x, packed=packed, s_perm=s_perm, m=m, k=k, n=n)


def to_gpu(p, dev):
    return (torch.from_numpy(p["x"]).to(dev), torch.from_numpy(p["packed"]).to(dev),
            torch.from_numpy(p["s_perm"]).to(dev))


def workspace_for(n, dev):
    return torch.zeros((n // 64) * 16, dtype=torch.int32, device=dev)


def reference_product(p, exact=False):
    w = O.dequant_codes(p["q"], p["s"], p["k"] if p["s"].shape[0] == 1 else 128)
    return O.gemm_fp64(p["x"], w) if exact else O.gemm_fp32(p["x"], w)


def unrounded_product(p, x=None):
    """x . ((q - 8) s) in float64 with the weights NOT rounded to fp16: what the streaming
    kernel computes (scale applied to each group's fp32 dot product) up to fp32 rounding."""
    k, n = p["k"], p["n"]
    group = k if p["s"].shape[0] == 1 else 128
    s_full = np.repeat(p["s"].astype(np.float64), group, axis=0)
    w = (p["q"].astype(np.float64) - 8.0) * s_full
    return (p["x"] if x is None else x).astype(np.float64) @ w


def check_fp32_result(y32, p, ref, m, x=None, forced_stream=False):
    """fp32 output against the float64 product.  The tiled kernel (m > 16) multiplies the
    reference's fp16-rounded weights: only fp32 accumulation error remains.  The streaming
    kernel (m <= 16) scales each group's dot product of raw codes: the same holds against the
    product with unrounded weights, and the distance to `ref` is the weights' rounding noise."""
    if m <= 16 or forced_stream:
        d = np.abs(y32 - unrounded_product(p, x)).max()
        assert d < 2e-4, d
        d = np.abs(y32 - ref).max()
        assert d < 1e-4 * np.sqrt(p["k"]), d   # ~ 2^-11 relative noise per weight, summed over K
    else:
        d = np.abs(y32 - ref).max()
        assert d < 2e-4, d


def fp16_half_ulp(ref):
    """Half the fp16 spacing at |ref| (normal range)."""
    a = np.maximum(np.abs(ref).astype(np.float64), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 11)


def check_layer_output(y16, ref, *, max_abs=1e-2, mean_rel=1e-3):
    """The path's tolerance: max-abs 1e-2 and mean relative 1e-3 against the
    fp32-accumulated reference.  An fp16 result cannot be closer to the reference than
    half an fp16 ulp of it (0.0078 once |y| >= 16, 0.0156 once |y| >= 32), so the absolute
    bound is max(1e-2, half ulp + 5e-3): the first term is the stated tolerance, the second
    the representation floor plus half the tolerance for the value before rounding (the
    streaming kernel does not round the scaled weights to fp16 as the reference does, which
    moves that value by up to about 4e-3 at K = 14336)."""
    y = np.asarray(y16, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    err = np.abs(y - ref)
    bound = np.maximum(max_abs, fp16_half_ulp(ref) + 0.5 * max_abs)
    assert (err <= bound).all(), f"max abs err {err.max():.4g} at |ref| {np.abs(ref).flat[err.argmax()]:.3g}"
    rel = err.sum() / np.abs(ref).sum()
    assert rel <= mean_rel, f"mean relative error {rel:.3g}"
    return err.max(), rel
