"""Seeded synthetic problems (the benchmark's generator) and comparison rules."""
import numpy as np
import torch

from oracle import uniql_oracle as O

SEED = 1234
# largest distance between the value a kernel holds before its final rounding and the reference
# (fp32 accumulation error up to K = 14336): asserted on fp32 outputs, used by check_layer_output
# only where the fp16 representation itself cannot meet 1e-2
PRE_ROUNDING_BOUND = 1e-4


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


def check_fp32_result(y32, p, ref, m, x=None, forced_stream=False):
    """fp32 output against the float64 product.  Both kernels multiply the reference's
    fp16-rounded weights exactly and accumulate in fp32: only the accumulation error remains
    (about 2^-24 sqrt(K) |y|)."""
    d = np.abs(y32 - ref).max()
    assert d < (2e-4 if p["k"] <= 4096 else PRE_ROUNDING_BOUND), d


def fp16_half_ulp(ref):
    """Half the fp16 spacing at |ref| (normal range)."""
    a = np.maximum(np.abs(ref).astype(np.float64), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 11)


# |ref| from which half an fp16 ulp alone exceeds the stated 1e-2 (spacing 2^-5 in [32, 64))
_FP16_FLOOR_FROM = 32.0


def check_layer_output(y16, ref, *, max_abs=1e-2, mean_rel=1e-3):
    """The path's tolerance: max-abs 1e-2 and mean relative 1e-3 against the fp32-accumulated
    reference.  The absolute bound is 1e-2 for every |ref| < 32.  From 32 on an fp16 result
    cannot be closer than half an fp16 ulp (0.0156 in [32, 64)); there the bound is that
    representation floor plus PRE_ROUNDING_BOUND for the value before rounding."""
    y = np.asarray(y16, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    err = np.abs(y - ref)
    bound = np.where(np.abs(ref) < _FP16_FLOOR_FROM, max_abs, fp16_half_ulp(ref) + PRE_ROUNDING_BOUND)
    assert (err <= bound).all(), f"max abs err {err.max():.4g} at |ref| {np.abs(ref).flat[err.argmax()]:.3g}"
    rel = err.sum() / np.abs(ref).sum()
    assert rel <= mean_rel, f"mean relative error {rel:.3g}"
    return err.max(), rel


def check_layer_output_torch(y16, ref64, *, max_abs=1e-2, mean_rel=1e-3):
    """check_layer_output on device tensors (for outputs too large to compare on the host):
    y16 fp16, ref64 float64, same shape."""
    import torch
    err = (y16.double() - ref64).abs()
    a = ref64.abs()
    half_ulp = torch.exp2(torch.floor(torch.log2(a.clamp_min(2.0 ** -14))) - 11)
    bound = torch.where(a < _FP16_FLOOR_FROM, torch.full_like(a, max_abs), half_ulp + PRE_ROUNDING_BOUND)
    worst = int((err - bound).argmax())
    assert bool((err <= bound).all()), \
        f"max abs err {float(err.max()):.4g}; worst excess at |ref| {float(a.flatten()[worst]):.3g}"
    rel = float(err.sum() / a.sum())
    assert rel <= mean_rel, f"mean relative error {rel:.3g}"
    return float(err.max()), rel
