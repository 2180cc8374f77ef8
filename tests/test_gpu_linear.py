"""GPU parity of the W4A16 linear path, through the C ABI (ops -> ctypes -> HIP)."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import (check_layer_output, make_linear_problem, reference_product, to_gpu,
                           check_fp32_result, workspace_for)

pytestmark = pytest.mark.gpu


def run_gemm(p, dev, **kw):
    from uniql_amd import ops
    x, b, s = to_gpu(p, dev)
    ws = workspace_for(p["n"], dev)
    y = ops.w4a16_gemm_ex(x, b, s, ws, p["m"], p["n"], p["k"], **kw)
    torch.cuda.synchronize()
    assert int(ws.abs().sum()) == 0, "workspace must stay zero"
    for buf in ops._accum_cache.values():
        assert int(buf.count_nonzero()) == 0, "accumulator words must be zero again after the call"
    return y.cpu().numpy()


# ------------------------------------------------------------------ bit-exact layer
@pytest.mark.parametrize("k,n", [(128, 128), (256, 256), (512, 384), (4096, 4096)])
def test_dequant_and_codes_bit_exact(gpu, k, n):
    from uniql_amd import ops
    p = make_linear_problem(1, k, n, seed=k + n)
    _, b, s = to_gpu(p, gpu)
    w, codes = ops.w4a16_dequant(b, s, n, k, want_codes=True)
    assert np.array_equal(codes.cpu().numpy().astype(np.int32), p["q"])
    want = O.dequant_codes(p["q"], p["s"])
    assert np.array_equal(w.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_dequant_every_code_times_every_scale(gpu):
    """16 codes x all 63488 finite fp16 scales (both signs, subnormals included)."""
    from uniql_amd import ops
    bits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    finite = bits[(bits & 0x7C00) != 0x7C00]
    n = 63488 // 128 * 128
    assert finite.size == 63488 and n == 63488
    s = finite.view(np.float16).reshape(1, n)
    k = 128
    q = np.tile(np.arange(16, dtype=np.int32)[:, None], (k // 16, n))
    packed = torch.from_numpy(O.pack_weights(q)).to(gpu)
    s_perm = torch.from_numpy(O.permute_scales(s, k, n, k)).to(gpu)
    w = ops.w4a16_dequant(packed, s_perm, n, k).cpu().numpy()
    want = O.dequant_codes(q, s, k)
    assert np.array_equal(w.view(np.uint16), want.view(np.uint16))


def test_dequant_golden_case(gpu, golden):
    from uniql_amd import ops
    b = torch.from_numpy(golden["A_packed"]).to(gpu)
    s = torch.from_numpy(golden["A_scale"]).to(gpu)
    w, codes = ops.w4a16_dequant(b, s, 256, 256, want_codes=True)
    assert np.array_equal(codes.cpu().numpy(), golden["A_codes"])
    assert np.array_equal(w.cpu().numpy().view(np.uint16), golden["A_w_ref"].view(np.uint16))


# ------------------------------------------------------------------ decode shapes
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 16])
@pytest.mark.parametrize("k,n", [(128, 128), (256, 256), (640, 384), (4096, 4096)])
def test_stream_kernel_small_m(gpu, m, k, n):
    p = make_linear_problem(m, k, n, seed=100 * m + k // 128 + n)
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True)
    check_fp32_result(y32, p, ref, m)
    y16 = run_gemm(p, gpu)
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    check_layer_output(y16, ref)


@pytest.mark.parametrize("k,n", [(4096, 6144), (4096, 28672), (14336, 4096)])
@pytest.mark.parametrize("m", [1, 8])
def test_stream_kernel_llama_shapes(gpu, m, k, n):
    p = make_linear_problem(m, k, n, seed=k + n + m)
    ref = reference_product(p)
    y16 = run_gemm(p, gpu)
    check_layer_output(y16, ref)


def _scales_across_the_expansion_ranges(groups, n, seed):
    """Scales inside the range of the streaming kernel's short expansion (2^-10 <= s < 2^-4, every
    binade, both ends), and outside it on every side: zero, subnormal, just below 2^-10, 2^-4 and
    above, large, negative."""
    rng = np.random.default_rng(seed)
    inside = np.concatenate([
        np.array([2.0 ** -10, 2.0 ** -4 - 2.0 ** -15, 0.004, 0.02, 0.0624], dtype=np.float16),
        (2.0 ** rng.uniform(-10, -4, size=64)).astype(np.float16)])
    inside = inside[(inside >= np.float16(2.0 ** -10)) & (inside < np.float16(2.0 ** -4))]
    outside = np.array([0.0, 6e-8, 2.0 ** -14, np.nextafter(np.float16(2.0 ** -10), np.float16(0)), 2.0 ** -4, 0.07,
                        0.5, 3.0, 1000.0, -0.01, -2.0 ** -12], dtype=np.float16)
    s = rng.choice(inside, size=(groups, n)).astype(np.float16)
    return s, outside, rng


def test_stream_kernel_reproduces_every_weight(gpu):
    """One-hot activation rows make every output element a single product 1 * w, exact in the
    matrix unit and in fp32: the streaming kernel's fp32 output must then BE the reference's
    fp16 weight fp16_rn((code - 8) * scale) (marlin_gemm_kernel.cuh:118-146), for all 16 codes,
    for scales over the whole range of the short expansion (both code positions of a packed
    word: the low one is held divided by 16 and multiplied back at the end) and for scales
    outside it, which take the long expansion (a wave switches when any of its lanes meets one)."""
    k, n, groups = 256, 256, 2
    s, outside, rng = _scales_across_the_expansion_ranges(groups, n, 11)
    # group 0: every column in range; group 1: out-of-range scales in a third of the columns
    cols = rng.choice(n, size=n // 3, replace=False)
    s[1, cols] = rng.choice(outside, size=cols.size)
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    q[:16] = np.arange(16)[:, None]          # every code in every column at least once per class of K row
    q[16:32] = np.arange(16)[::-1, None]
    w = O.dequant_codes(q, s, 128)
    p = dict(q=q, s=s, m=16, k=k, n=n, packed=O.pack_weights(q), s_perm=O.permute_scales(s, k, n, 128))
    for k0 in range(0, k, 16):
        x = np.zeros((16, k), dtype=np.float16)
        x[np.arange(16), k0 + np.arange(16)] = 1.0
        p["x"] = x
        y32 = run_gemm(p, gpu, out_f32=True)
        want = w[k0:k0 + 16].astype(np.float32)
        assert np.array_equal(y32, want), (k0, np.abs(y32 - want).max())


@pytest.mark.parametrize("m", [1, 6])
def test_scales_outside_the_short_expansion_range(gpu, m):
    """Random data with out-of-range scales sprinkled over groups and columns (so that some waves
    switch between the two expansions from one group to the next), with and without a K split."""
    k, n = 2048, 512
    p = make_linear_problem(m, k, n, seed=400 + m)
    s, outside, rng = _scales_across_the_expansion_ranges(k // 128, n, 12 + m)
    hit = rng.random(s.shape) < 0.02
    s[hit] = rng.choice(outside[np.abs(outside) <= 3.0], size=int(hit.sum()))
    s[5, :] = np.float16(0.25)               # a whole group outside
    p["s"] = s
    p["s_perm"] = O.permute_scales(s, k, n, 128)
    w = O.dequant_codes(p["q"], s, 128)
    ref = O.gemm_fp64(p["x"], w)
    budget = np.abs(p["x"].astype(np.float64)) @ np.abs(w.astype(np.float64))   # sum of |terms| per output
    for flags in (0, (8 << 8) | (4 << 16)):   # the default plan (K split) and one workgroup per strip
        y32 = run_gemm(p, gpu, out_f32=True, flags=flags)
        assert (np.abs(y32 - ref) <= 2.0 ** -20 * budget + 1e-30).all(), np.abs(y32 - ref).max()


def test_per_column_scales_outside_the_short_expansion_range(gpu):
    """One scale per column (a single scale row): a column outside the range sends its wave the long
    way in every group; one-hot rows again make the output the weights themselves."""
    k, n = 256, 256
    s, outside, rng = _scales_across_the_expansion_ranges(1, n, 21)
    cols = rng.choice(n, size=40, replace=False)
    s[0, cols] = rng.choice(outside, size=cols.size)
    q = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    w = O.dequant_codes(q, s, k)
    p = dict(q=q, s=s, m=16, k=k, n=n, packed=O.pack_weights(q), s_perm=O.permute_scales(s, k, n, k))
    for k0 in (0, 112, 240):
        x = np.zeros((16, k), dtype=np.float16)
        x[np.arange(16), k0 + np.arange(16)] = 1.0
        p["x"] = x
        y32 = run_gemm(p, gpu, out_f32=True)
        assert np.array_equal(y32, w[k0:k0 + 16].astype(np.float32)), k0


F_FORCE_SKINNY, F_FORCE_TILED = 2, 4


@pytest.mark.parametrize("m", [17, 33, 64, 65, 130])
def test_stream_kernel_forced_for_larger_m(gpu, m):
    """The streaming kernel walks larger M in slabs of 64 rows (not the default route)."""
    p = make_linear_problem(m, 512, 256, seed=m)
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True, flags=F_FORCE_SKINNY)
    check_fp32_result(y32, p, ref, m, forced_stream=True)
    check_layer_output(run_gemm(p, gpu, flags=F_FORCE_SKINNY), ref)


# ------------------------------------------------------------------ prefill shapes (tiled kernel)
@pytest.mark.parametrize("m", [17, 32, 33, 64, 65, 100, 128, 129, 256, 300])
@pytest.mark.parametrize("k,n", [(128, 128), (512, 256), (1408, 384)])
def test_tile_kernel_small_shapes(gpu, m, k, n):
    p = make_linear_problem(m, k, n, seed=7 * m + k + n)
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True)
    assert np.abs(y32 - ref).max() < 2e-4, np.abs(y32 - ref).max()
    y16 = run_gemm(p, gpu)
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    check_layer_output(y16, ref)


@pytest.mark.parametrize("m,k,n", [(256, 4096, 4096), (1024, 4096, 4096), (1024, 4096, 6144), (256, 14336, 4096)])
def test_tile_kernel_llama_shapes(gpu, m, k, n):
    p = make_linear_problem(m, k, n, seed=m + k + n)
    ref = reference_product(p)
    y16 = run_gemm(p, gpu)
    check_layer_output(y16, ref)


@pytest.mark.parametrize("m", [1, 5, 16])
def test_tile_kernel_forced_for_small_m(gpu, m):
    p = make_linear_problem(m, 640, 256, seed=m + 3)
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True, flags=F_FORCE_TILED)
    assert np.abs(y32 - ref).max() < 2e-4


@pytest.mark.parametrize("splits", [1, 2, 3, 11])
def test_tile_kernel_k_splits(gpu, splits):
    p = make_linear_problem(40, 1408, 256, seed=splits)        # 11 groups
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True, flags=splits << 8)
    assert np.abs(y32 - ref).max() < 2e-4
    again = run_gemm(p, gpu, out_f32=True, flags=splits << 8)
    assert np.array_equal(y32, again)                          # integer accumulation: order-independent


@pytest.mark.parametrize("m,k,n,splits,mt", [(1024, 1024, 4096, 4, 1), (1000, 1536, 2048, 3, 2), (257, 1536, 768, 3, 0),
                                             (300, 2048, 640, 4, 4), (200, 640, 1280, 3, 0), (300, 896, 1280, 2, 1),
                                             (200, 384, 1152, 3, 1)])
def test_tile_split_exchange_is_ordered(gpu, m, k, n, splits, mt):
    """K split over workgroups of the tiled kernel: partial tiles go through scratch memory and
    the last workgroup of a tile adds them.  The result must not depend on which workgroup that
    is, nor may it ever read a slot before it is complete: the same call many times over, with
    the scratch area dirtied in between, gives the same bits every time and the right values."""
    from uniql_amd import ops
    p = make_linear_problem(m, k, n, seed=m + k + n)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    flags = F_FORCE_TILED | (splits << 8) | (mt << 16)
    first = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True, flags=flags)
    assert np.abs(first.cpu().numpy() - reference_product(p, exact=True)).max() < 3e-4
    from uniql_amd import _capi
    _, scratch_bytes = ops._workspace(_capi.load(), m, n, k, k, 0, flags | _capi.F_OUT_F32)
    assert scratch_bytes > 0
    same = torch.ones((), dtype=torch.bool, device=gpu)
    for rep in range(300):  # up to 4096 workgroups per call: about a million tile exchanges in all
        # dirty the block the allocator will hand out as scratch area (same size, freed last): a
        # slot that is read before it is written then shows as NaN
        junk = torch.full((scratch_bytes,), 0xFF, dtype=torch.uint8, device=gpu)
        del junk
        again = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True, flags=flags)
        same &= (first == again).all()
    assert bool(same)


@pytest.mark.parametrize("mt", [1, 2])
@pytest.mark.parametrize("m,k,n", [(32, 256, 128), (100, 1024, 256), (256, 4096, 512), (64, 768, 128), (33, 640, 256)])
def test_tile_kernel_two_wave_quartets(gpu, m, k, n, mt):
    """eight waves per workgroup, the quartets taking alternate K groups (an odd number of
    groups, k = 640, falls back to one quartet)"""
    p = make_linear_problem(m, k, n, seed=m + k)
    ref = reference_product(p, exact=True)
    flags = (1 << 2) | (mt << 16) | (2 << 20)
    y32 = run_gemm(p, gpu, out_f32=True, flags=flags)
    check_fp32_result(y32, p, ref, 1000)
    y = run_gemm(p, gpu, flags=flags)
    check_layer_output(y, ref)
    # with K also split over workgroups (2 x 2 groups each at k = 1024)
    if k % 512 == 0:
        y32 = run_gemm(p, gpu, out_f32=True, flags=flags | (2 << 8))
        check_fp32_result(y32, p, ref, 1000)


def test_tile_kernel_per_column_and_stride(gpu):
    from uniql_amd import ops
    p = make_linear_problem(48, 384, 256, seed=21, per_column=True)
    ref = reference_product(p, exact=True)
    assert np.abs(run_gemm(p, gpu, out_f32=True) - ref).max() < 2e-4
    p = make_linear_problem(40, 256, 256, seed=22)
    x, b, s = to_gpu(p, gpu)
    big = torch.zeros(40, 512, dtype=torch.float16, device=gpu)
    big[:, :256] = x
    y = ops.w4a16_gemm_ex(big[:, :256], b, s, workspace_for(256, gpu), 40, 256, 256).cpu().numpy()
    check_layer_output(y, reference_product(p))


@pytest.mark.parametrize("upw", [1, 2, 4, 8])
def test_units_per_wave_override(gpu, upw):
    p = make_linear_problem(2, 1408, 256, seed=upw)     # 11 groups: ragged against 4*upw
    ref = reference_product(p, exact=True)
    y32 = run_gemm(p, gpu, out_f32=True, flags=upw << 8)
    check_fp32_result(y32, p, ref, 2)


def test_per_column_scales(gpu):
    for k in (128, 384):
        p = make_linear_problem(3, k, 256, seed=k, per_column=True)
        ref = reference_product(p, exact=True)
        y32 = run_gemm(p, gpu, out_f32=True)
        check_fp32_result(y32, p, ref, 3)


def test_deterministic_and_repeatable(gpu):
    p = make_linear_problem(4, 4096, 4096, seed=5)
    a = run_gemm(p, gpu)
    b = run_gemm(p, gpu)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


@pytest.mark.parametrize("m", [1, 3])
def test_nan_propagates_with_and_without_k_split(gpu, m):
    """A NaN activation makes its row NaN whether or not the launch splits K over workgroups
    (the partial sums then meet in the fixed-point accumulator words, which carry a NaN
    count); other rows are untouched, and the accumulator words are zero again afterwards."""
    p = make_linear_problem(m, 4096, 512, seed=90 + m)
    p["x"][m - 1, 1000] = np.nan
    split = run_gemm(p, gpu, out_f32=True)                        # 32 groups over several workgroups
    whole = run_gemm(p, gpu, out_f32=True, flags=(8 << 8) | (4 << 16))   # 4 waves x 8 groups: one workgroup per strip
    for y in (split, whole):
        assert np.isnan(y[m - 1]).all()
        assert np.isfinite(y[:m - 1]).all()
    assert np.array_equal(split[:m - 1], whole[:m - 1]) or np.abs(split[:m - 1] - whole[:m - 1]).max() < 1e-5
    y16 = run_gemm(p, gpu)
    assert np.isnan(y16[m - 1]).all()


def test_infinite_partial_sums_with_and_without_k_split(gpu):
    """What the header documents for partial sums beyond the accumulator words' range, pinned:
    an infinite activation gives an infinite fp16 result of the right sign with and without a K
    split (a partial sum clamped to +-2^18 is still beyond fp16's 65504); with fp32 output the
    launch that splits K shows the clamp (a finite value of at least 2^18) where the launch
    that does not split shows inf; +inf and -inf that meet from different workgroups cancel to
    a finite value when K is split and give NaN when it is not."""
    m, k, n = 2, 4096, 512
    p = make_linear_problem(m, k, n, seed=77)
    p["q"][:] = 15                      # every weight +7 s > 0: the sign of a column's sum is the activation's
    p["packed"] = O.pack_weights(p["q"])
    p["x"][:] = np.float16(0.001)
    p["x"][0, 100] = np.inf             # row 0: +inf in the first workgroup's K range
    p["x"][1, 100] = np.inf             # row 1: +inf there and -inf in the last workgroup's
    p["x"][1, 4000] = -np.inf
    whole_plan = (8 << 8) | (4 << 16)   # 4 waves x 8 groups: one workgroup per strip, no exchange
    y_split, y_whole = run_gemm(p, gpu), run_gemm(p, gpu, flags=whole_plan)
    for y in (y_split, y_whole):
        assert np.isposinf(y[0]).all()
    assert np.isnan(y_whole[1]).all()               # inf - inf inside one workgroup's fp32 sum
    assert np.isfinite(y_split[1]).all()            # the documented difference: clamped partial sums cancel
    f_split, f_whole = run_gemm(p, gpu, out_f32=True), run_gemm(p, gpu, out_f32=True, flags=whole_plan)
    assert np.isposinf(f_whole[0]).all()
    assert np.isfinite(f_split[0]).all() and (f_split[0] >= 2.0 ** 18).all()


def test_row_stride(gpu):
    """A may be a row-strided view (lda > k)."""
    from uniql_amd import ops
    p = make_linear_problem(4, 256, 256, seed=8)
    x, b, s = to_gpu(p, gpu)
    big = torch.zeros(4, 512, dtype=torch.float16, device=gpu)
    big[:, :256] = x
    y = ops.w4a16_gemm_ex(big[:, :256], b, s, workspace_for(256, gpu), 4, 256, 256).cpu().numpy()
    check_layer_output(y, reference_product(p))


@pytest.mark.parametrize("m,had_block", [(3, 256), (3, 128), (40, 128), (40, 512)])
def test_row_stride_with_rotation(gpu, m, had_block):
    """A row-strided view whose rows are rotated first (not the 128-block rotation fused into the
    streaming kernel, or any rotation ahead of the tiled kernel) gives the same bits as the
    contiguous input."""
    from uniql_amd import ops
    p = make_linear_problem(m, 1024, 256, seed=60 + m)
    x, b, s = to_gpu(p, gpu)
    big = torch.full((m, 1536), 3.0, dtype=torch.float16, device=gpu)
    big[:, :1024] = x
    kw = dict(had_block=had_block, had_scale=had_block ** -0.5)
    ws = workspace_for(256, gpu)
    want = ops.w4a16_gemm_ex(x, b, s, ws, m, 256, 1024, **kw)
    got = ops.w4a16_gemm_ex(big[:, :1024], b, s, ws, m, 256, 1024, **kw)
    assert torch.equal(want, got)
    xr = O.fwht(p["x"], had_block ** -0.5, block=had_block)
    check_layer_output(got.cpu().numpy(), O.gemm_fp64(xr, O.dequant_codes(p["q"], p["s"])))


# ------------------------------------------------------------------ fused rotation
@pytest.mark.parametrize("m", [1, 5, 16, 40, 200])
def test_fused_blockwise_hadamard(gpu, m):
    k, n = 1536, 256           # 12 blocks of 128: not a power of two overall
    p = make_linear_problem(m, k, n, seed=m + 40)
    xr = O.fwht(p["x"], 128 ** -0.5, block=128)          # fp16 result of the standalone rotation
    w = O.dequant_codes(p["q"], p["s"])
    ref = O.gemm_fp64(xr, w)
    y32 = run_gemm(p, gpu, out_f32=True, had_block=128, had_scale=128 ** -0.5)
    check_fp32_result(y32, p, ref, m, x=xr)
    check_layer_output(run_gemm(p, gpu, had_block=128, had_scale=128 ** -0.5), ref)


@pytest.mark.parametrize("had_block", [128, 2048])
def test_rotations_with_scales_outside_the_short_expansion_range(gpu, had_block):
    """The fused rotations (128-blocks while staging; whole rows in LDS) in front of units that
    take the long expansion and units that take the short one."""
    m, k, n = 3, 2048, 384
    p = make_linear_problem(m, k, n, seed=had_block)
    s, outside, rng = _scales_across_the_expansion_ranges(k // 128, n, had_block + 1)
    hit = rng.random(s.shape) < 0.03
    s[hit] = rng.choice(outside[np.abs(outside) <= 3.0], size=int(hit.sum()))
    p["s"], p["s_perm"] = s, O.permute_scales(s, k, n, 128)
    xr = O.fwht(p["x"], had_block ** -0.5, block=had_block)
    w = O.dequant_codes(p["q"], s, 128)
    ref = O.gemm_fp64(xr, w)
    budget = np.abs(xr.astype(np.float64)) @ np.abs(w.astype(np.float64))
    y32 = run_gemm(p, gpu, out_f32=True, had_block=had_block, had_scale=had_block ** -0.5)
    assert (np.abs(y32 - ref) <= 2.0 ** -20 * budget + 1e-30).all(), np.abs(y32 - ref).max()


@pytest.mark.parametrize("m", [1, 3])
def test_full_width_hadamard_prologue(gpu, m):
    k, n = 8192, 256
    p = make_linear_problem(m, k, n, seed=m + 80)
    xr = O.fwht(p["x"], k ** -0.5)
    ref = O.gemm_fp64(xr, O.dequant_codes(p["q"], p["s"]))
    y32 = run_gemm(p, gpu, out_f32=True, had_block=k, had_scale=k ** -0.5)
    check_fp32_result(y32, p, ref, m, x=xr)


@pytest.mark.parametrize("m,k,n", [(1, 8192, 4096), (2, 8192, 384), (1, 16384, 256), (4, 4096, 1024), (3, 2048, 640),
                                   (16, 1024, 256), (7, 256, 128), (2, 512, 4096)])
def test_full_row_rotation_inside_the_streaming_kernel(gpu, m, k, n):
    """Whole-row rotation (block = k) applied by every workgroup of the streaming kernel in LDS against the
    same call with the transform kernel run first into `temp` (UNIQL_F_SEPARATE_ROTATION): same butterfly
    order, same single fp16 rounding, so the outputs are identical; and against the oracle."""
    from uniql_amd import ops, _capi
    p = make_linear_problem(m, k, n, seed=m * 1000 + k)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    lib = _capi.load()
    import ctypes
    acc, tmp = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.uniql_w4a16_linear_workspace(m, n, k, k, k, 0, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert tmp.value == 0                                     # nothing goes through temporary memory
    assert lib.uniql_w4a16_linear_workspace(m, n, k, k, k, _capi.F_SEPARATE_ROTATION, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert tmp.value == (m * k * 2 + 255) // 256 * 256
    for out_f32 in (True, False):
        fused = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, had_block=k, had_scale=k ** -0.5, out_f32=out_f32)
        apart = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, had_block=k, had_scale=k ** -0.5, out_f32=out_f32,
                                  flags=_capi.F_SEPARATE_ROTATION)
        assert torch.equal(fused, apart)
    xr = O.fwht(p["x"], k ** -0.5)
    ref = O.gemm_fp64(xr, O.dequant_codes(p["q"], p["s"]))
    check_fp32_result(ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, had_block=k, had_scale=k ** -0.5, out_f32=True).cpu().numpy(),
                      p, ref, m, x=xr)
    check_layer_output(fused.cpu().numpy(), ref)


@pytest.mark.parametrize("m", [1, 5, 16, 40, 130])
def test_output_transpose(gpu, m):
    """the reference's output_transpose: D[n, m8], row index last, m rounded up to 8"""
    from uniql_amd import ops
    k, n = 512, 384
    p = make_linear_problem(m, k, n, seed=m)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    want = ops.w4a16o16_gemm(x, b, s, ws, m, n, k)
    got = ops.w4a16o16_gemm(x, b, s, ws, m, n, k, True)
    m8 = (m + 7) // 8 * 8
    assert tuple(got.shape) == (n, m8)
    assert torch.equal(got[:, :m], want.t())
    assert int(got[:, m:].abs().sum()) == 0


# ------------------------------------------------------------------ error paths
def test_errors(gpu):
    from uniql_amd import ops
    p = make_linear_problem(1, 256, 256)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(256, gpu)
    with pytest.raises(RuntimeError):
        ops.w4a16o16_gemm(x, b, s, ws[:2], 1, 256, 256, False, -1, -1, -1, 16)   # workspace too small
    with pytest.raises(RuntimeError):
        ops.w4a16o16_gemm(x.float(), b, s, ws, 1, 256, 256)               # dtype
    with pytest.raises(RuntimeError):
        ops.w4a16o16_gemm(x, b, s[:, :128].contiguous(), ws, 1, 256, 256)  # scale shape
    with pytest.raises(RuntimeError):
        ops.w4a16o16_gemm(x.cpu(), b, s, ws, 1, 256, 256)                 # no CPU path
    y = ops.w4a16o16_gemm(x[:0], b, s, ws, 0, 256, 256)
    assert tuple(y.shape) == (0, 256)


# ------------------------------------------------------------------ streams and graphs
def test_side_stream_and_graph_replay(gpu):
    """Every entry point only enqueues kernels on the stream it is given: the calls can be
    captured in a HIP graph and replayed, with eager work between the replays, and each replay
    gives the eager result again (the accumulator words return to zero after every call)."""
    from uniql_amd import ops
    problems = [make_linear_problem(1, 4096, 512, seed=301),      # streaming kernel, K split with atomics
                make_linear_problem(40, 1408, 256, seed=302),     # tiled kernel
                make_linear_problem(3, 1536, 256, seed=303)]      # streaming kernel with the fused rotation
    dev_in = [to_gpu(p, gpu) for p in problems]
    ws = [workspace_for(p["n"], gpu) for p in problems]

    bias = torch.linspace(-1, 1, 200, device=gpu).half()
    pair_bias = torch.linspace(-1, 1, 512, device=gpu).half()
    q0 = torch.randn(1, 70, 4, 16, generator=torch.Generator().manual_seed(5)).half().to(gpu)
    k0 = torch.randn(1, 70, 2, 16, generator=torch.Generator().manual_seed(6)).half().to(gpu)
    cos = torch.rand(1, 70, 16, generator=torch.Generator().manual_seed(7)).half().to(gpu)
    idx = torch.arange(16, dtype=torch.uint8, device=gpu).repeat(2, 1)
    table = (torch.randn(64, 128, generator=torch.Generator().manual_seed(8)) * 0.1).half().to(gpu)

    def run_all():
        outs = []
        for i, (p, (x, b, s)) in enumerate(zip(problems, dev_in)):
            kw = dict(had_block=128, had_scale=128 ** -0.5) if i == 2 else {}
            outs.append(ops.w4a16_gemm_ex(x, b, s, ws[i], p["m"], p["n"], p["k"], **kw))
        # the layer call with its epilogues: cut + bias (tiled kernel), gated pairs with K split over
        # workgroups (streaming kernel: the pair exchange through the accumulator words)
        x, b, s = dev_in[1]
        outs.append(ops.w4a16_linear(x[:, :1400], b, s, ws[1], 256, 1408, out_features=200, bias=bias))
        x, b, s = dev_in[0]
        outs.append(ops.w4a16_linear(x, b, s, ws[0], 512, 4096, silu_mul=True, bias=pair_bias))
        # rotary embedding (in place: work on copies), embedding-table quantiser
        q, k = q0.clone(), k0.clone()
        ops.rope_indices_(q, k, cos, cos, idx)
        outs += [q, k]
        outs += list(ops.w4_embedding_quantize(table))
        return outs

    eager = [y.clone() for y in run_all()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        on_side = [y.clone() for y in run_all()]                  # also sizes the side stream's accumulators
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for a, b in zip(eager, on_side):
        assert torch.equal(a, b)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run_all()
    for rep in range(3):
        for y in captured:
            y.fill_(float("nan")) if y.is_floating_point() else y.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, captured):
            assert torch.equal(a, b), f"replay {rep}"
        # eager work between the replays, on the same buffers' neighbours
        again = run_all()
        torch.cuda.synchronize()
        for a, b in zip(eager, again):
            assert torch.equal(a, b)
    for buf in ops._accum_cache.values():
        assert int(buf.count_nonzero()) == 0


def test_accumulator_cache_across_graphs_and_growth(gpu):
    """The Python layer caches the zero-in / zero-out accumulator words per stream.  Two hazards:
    a buffer allocated while a graph is being captured is only zero-filled when THAT graph
    replays, so a second graph (replayed first) and eager calls must not depend on it; and a
    buffer a graph has captured must stay allocated when a later, larger call replaces it."""
    from uniql_amd import ops
    ops.reset_accumulators()
    small = make_linear_problem(1, 4096, 512, seed=311)       # K split with atomics, small accumulator
    other = make_linear_problem(2, 2048, 256, seed=312)
    large = make_linear_problem(16, 1024, 8192, seed=313)     # 16 x 8192 words: beyond the cache's first size
    xs, bs, ss = to_gpu(small, gpu)
    xo, bo, so = to_gpu(other, gpu)
    xl, bl, sl = to_gpu(large, gpu)
    ws_s, ws_o, ws_l = (workspace_for(p["n"], gpu) for p in (small, other, large))

    def run_small():
        return ops.w4a16_gemm_ex(xs, bs, ss, ws_s, 1, 512, 4096)

    def run_other():
        return ops.w4a16_gemm_ex(xo, bo, so, ws_o, 2, 256, 2048)

    def run_large():
        return ops.w4a16_gemm_ex(xl, bl, sl, ws_l, 16, 8192, 1024)

    # first use of the capture stream happens inside the captures
    g1, g2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1):
        y1 = run_small()
    with torch.cuda.graph(g2):
        y2 = run_other()
    # dirty whatever the allocator hands out next, then replay the SECOND graph first
    junk = [torch.full((1 << 18,), -1, dtype=torch.int64, device=gpu) for _ in range(8)]
    del junk
    g2.replay()
    torch.cuda.synchronize()
    want_small, want_other, want_large = run_small().clone(), run_other().clone(), run_large().clone()
    assert torch.equal(y2, want_other)
    for rep in range(3):                                      # the recorded zero fills replay correctly too
        y1.fill_(float("nan"))
        y2.fill_(float("nan"))
        g1.replay()
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(y1, want_small) and torch.equal(y2, want_other), f"replay {rep}"
        assert torch.equal(run_small(), want_small)           # eager work between the replays

    # eager buffer captured by a graph, then outgrown by a larger call
    ops.reset_accumulators()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert torch.equal(run_small(), want_small)           # sizes the side stream's buffer eagerly
        g3 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g3, stream=side):
            y3 = run_small()
        before = ops._accum_cache[(side.device.index, side.cuda_stream)]
        assert torch.equal(run_large(), want_large)           # needs more words: the buffer is replaced
        assert ops._accum_cache[(side.device.index, side.cuda_stream)] is not before
        junk = [torch.full((1 << 16,), -1, dtype=torch.int64, device=gpu) for _ in range(16)]
        for rep in range(2):
            y3.fill_(float("nan"))
            g3.replay()
            side.synchronize()
            assert torch.equal(y3, want_small), f"replay {rep}"
        del junk
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ops.reset_accumulators()


@pytest.mark.parametrize("m", [1, 5, 40])
def test_lm_head_shape(gpu, m):
    """The models' last layer, 4096 -> 128256 (Llama-3.1's vocabulary; quantised like the other
    layers, quantize_model.py:126-143): 1002 column strips in one launch.  Too large for the CPU
    oracle in a test's time: the reference product is torch's fp32 matmul on the GPU with the
    weights from uniql_w4a16_dequant, which the tests above hold bit-exact against the oracle."""
    from uniql_amd import ops
    k, n = 4096, 128256
    g = torch.Generator(device=gpu).manual_seed(77 + m)
    b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), generator=g, device=gpu, dtype=torch.int64).to(torch.int32)
    s = (torch.rand(k // 128, n, generator=g, device=gpu) * 0.016 + 0.004).half()
    x = torch.randn(m, k, generator=g, device=gpu).half()
    ws = workspace_for(n, gpu)
    w = ops.w4a16_dequant(b, s, n, k)
    ref = (x.float() @ w.float()).cpu().numpy()
    del w
    y32 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True).cpu().numpy()
    assert np.abs(y32 - ref).max() < 5e-4
    y = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k)
    assert np.array_equal(y.cpu().numpy(), y32.astype(np.float16))
    check_layer_output(y.cpu().numpy(), ref)
