"""GPU parity of the 256 x 256 tile kernel (long prefill), forced through the tuning field of the
flags, against the oracle and against the 128-column kernel on the same calls."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import check_layer_output, make_linear_problem, reference_product, to_gpu, workspace_for
from tests.test_gpu_fused import assert_close16, deinterleave, gated_problem

pytestmark = pytest.mark.gpu

WIDE = 8 << 16      # "row tiles of 32 per workgroup" = 8: the 256 x 256 kernel
NARROW = 4 << 16    # the 128-column kernel with 128-row tiles


def run(p, dev, **kw):
    from uniql_amd import ops
    x, b, s = to_gpu(p, dev)
    y = ops.w4a16_gemm_ex(x, b, s, workspace_for(p["n"], dev), p["m"], p["n"], p["k"], **kw)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("m,k,n", [(256, 256, 256), (300, 512, 512), (257, 384, 768), (1000, 1024, 768), (513, 4096, 512),
                                   (17, 256, 256), (700, 1408, 256)])
def test_wide_kernel_against_the_oracle(gpu, m, k, n):
    """ragged M (rows past M inside the last tile), the shortest K (two groups), K groups that are
    not a power of two; fp32 output against the float64 product, fp16 output = its rounding"""
    p = make_linear_problem(m, k, n, seed=m + k + n)
    ref = reference_product(p, exact=True)
    y32 = run(p, gpu, out_f32=True, flags=WIDE)
    assert np.abs(y32 - ref).max() < 2e-4, np.abs(y32 - ref).max()
    y16 = run(p, gpu, flags=WIDE)
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    check_layer_output(y16, ref)
    assert np.array_equal(run(p, gpu, flags=WIDE), y16)  # same result from run to run
    # the 128-column kernel adds the same products in another order
    other = run(p, gpu, out_f32=True, flags=NARROW)
    assert np.abs(other - y32).max() < 1e-4


def test_wide_kernel_long_k(gpu):
    p = make_linear_problem(260, 14336, 256, seed=5)
    ref = reference_product(p, exact=True)
    y32 = run(p, gpu, out_f32=True, flags=WIDE)
    assert np.abs(y32 - ref).max() < 1e-4
    check_layer_output(run(p, gpu, flags=WIDE), ref)


def test_wide_kernel_strided_rows(gpu):
    from uniql_amd import ops
    p = make_linear_problem(300, 512, 256, seed=9)
    x, b, s = to_gpu(p, gpu)
    big = torch.zeros(300, 1024 + 8, dtype=torch.float16, device=gpu)
    big[:, 8:8 + 512] = x
    y = ops.w4a16_gemm_ex(big[:, 8:8 + 512], b, s, workspace_for(256, gpu), 300, 256, 512, flags=WIDE)
    want = ops.w4a16_gemm_ex(x, b, s, workspace_for(256, gpu), 300, 256, 512, flags=WIDE)
    assert torch.equal(y, want)
    check_layer_output(y.cpu().numpy(), reference_product(p))


@pytest.mark.parametrize("m", [256, 300])
@pytest.mark.parametrize("k,n,n_out", [(256, 256, 200), (640, 512, 512)])
def test_wide_kernel_cut_bias_residual_relu2(gpu, m, k, n, n_out):
    """the layer call's epilogues: bit-exact against the same kernel's plain product followed by
    torch's fp16 operations"""
    from uniql_amd import ops
    p = make_linear_problem(m, k, n, seed=m + k)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    gen = torch.Generator().manual_seed(m + n)
    bias = torch.randn(n_out, generator=gen).half().to(gpu)
    res = torch.randn(m, n_out, generator=gen).half().to(gpu)
    full = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, flags=WIDE)
    cut = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, flags=WIDE)
    assert torch.equal(cut, full[:, :n_out])
    biased = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, flags=WIDE)
    assert torch.equal(biased, full[:, :n_out] + bias)
    assert torch.equal(ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, residual=res, flags=WIDE),
                       res + biased)
    sq = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, relu2=True, flags=WIDE)
    assert torch.equal(sq, torch.relu(biased) ** 2)
    y32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, out_f32=True, flags=WIDE)
    full32 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True, flags=WIDE)
    assert torch.equal(y32, full32[:, :n_out] + bias.float())
    # into a column range of a wider buffer
    buf = torch.full((m, n_out + 40), 7.0, dtype=torch.float16, device=gpu)
    ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, out=buf[:, 16:16 + n_out], flags=WIDE)
    assert torch.equal(buf[:, 16:16 + n_out], cut)
    assert bool((buf[:, :16] == 7).all()) and bool((buf[:, 16 + n_out:] == 7).all())


@pytest.mark.parametrize("m", [256, 290])
def test_wide_kernel_transposed_output(gpu, m):
    from uniql_amd import ops
    p = make_linear_problem(m, 256, 256, seed=m)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(256, gpu)
    plain = ops.w4a16_gemm_ex(x, b, s, ws, m, 256, 256, flags=WIDE)
    t = ops.w4a16_gemm_ex(x, b, s, ws, m, 256, 256, transpose_out=True, flags=WIDE)
    assert torch.equal(t[:, :m], plain.t())


@pytest.mark.parametrize("m", [256, 300])
@pytest.mark.parametrize("k,width,n_out", [(256, 128, 128), (512, 256, 200)])
def test_wide_kernel_gated_pairs(gpu, m, k, width, n_out):
    from uniql_amd import ops
    g, u, w, s = gated_problem(m, k, width, seed=m + k)
    x = torch.from_numpy(g["x"]).to(gpu)
    w, s = w.to(gpu), s.to(gpu)
    ws = workspace_for(2 * width, gpu)
    both = ops.w4a16_gemm_ex(x, w, s, ws, m, 2 * width, k, flags=WIDE).cpu().numpy()
    g16, u16 = deinterleave(both, width)
    y = ops.w4a16_linear(x, w, s, ws, 2 * width, k, out_features=n_out, silu_mul=True, flags=WIDE)
    assert y.shape == (m, n_out)
    assert_close16(y.cpu().numpy(), O.mlp_gate_up(g16[:, :n_out], u16[:, :n_out]), ulps=2)
    bias = torch.from_numpy(np.random.default_rng(m).standard_normal(2 * n_out).astype(np.float16)).to(gpu)
    yb = ops.w4a16_linear(x, w, s, ws, 2 * width, k, out_features=n_out, silu_mul=True, bias=bias, flags=WIDE)
    bn = bias.cpu().numpy().astype(np.float32)
    gb = (g16[:, :n_out].astype(np.float32) + bn[:n_out]).astype(np.float16)
    ub = (u16[:, :n_out].astype(np.float32) + bn[n_out:]).astype(np.float16)
    assert_close16(yb.cpu().numpy(), O.mlp_gate_up(gb, ub), ulps=2)


def test_wide_kernel_behind_a_rotation_and_a_short_input(gpu):
    """the rotation and the zero padding of a short input run first, into the temporary buffer"""
    from uniql_amd import ops
    p = make_linear_problem(300, 512, 256, seed=31)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(256, gpu)
    for had in (128, 512):
        got = ops.w4a16_gemm_ex(x, b, s, ws, 300, 256, 512, had_block=had, had_scale=had ** -0.5, flags=WIDE)
        want = ops.w4a16_gemm_ex(ops.hadamard_blockwise(x, had ** -0.5, had), b, s, ws, 300, 256, 512, flags=WIDE)
        assert torch.equal(got, want)
    short = x[:, :456].contiguous()
    padded = torch.zeros_like(x)
    padded[:, :456] = short
    assert torch.equal(ops.w4a16_linear(short, b, s, ws, 256, 512, flags=WIDE),
                       ops.w4a16_gemm_ex(padded, b, s, ws, 300, 256, 512, flags=WIDE))


def test_wide_request_falls_back_where_the_kernel_cannot_run(gpu):
    """per-column scales, a width that is no multiple of 256, a single K group: the call is
    served by the 128-column kernel"""
    p = make_linear_problem(300, 384, 256, seed=3, per_column=True)
    assert np.abs(run(p, gpu, out_f32=True, flags=WIDE) - reference_product(p, exact=True)).max() < 2e-4
    p = make_linear_problem(300, 256, 384, seed=4)
    assert np.abs(run(p, gpu, out_f32=True, flags=WIDE) - reference_product(p, exact=True)).max() < 2e-4
    p = make_linear_problem(300, 128, 256, seed=5)
    assert np.abs(run(p, gpu, out_f32=True, flags=WIDE) - reference_product(p, exact=True)).max() < 2e-4


def test_wide_kernel_output_at_an_odd_address(gpu):
    """an output that is only 2-byte aligned takes the element-wise stores"""
    from uniql_amd import ops
    p = make_linear_problem(300, 256, 256, seed=23)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(256, gpu)
    want = ops.w4a16_linear(x, b, s, ws, 256, 256, flags=WIDE)
    flat = torch.zeros(300 * 256 + 8, dtype=torch.float16, device=gpu)
    out = flat[1:1 + 300 * 256].view(300, 256)
    ops.w4a16_linear(x, b, s, ws, 256, 256, out=out, flags=WIDE)
    assert torch.equal(out, want)
    assert float(flat[0]) == 0 and float(flat[-1]) == 0


def test_wide_request_with_a_row_stride_beyond_its_offsets(gpu):
    """256 rows of `lda` elements must fit 32-bit byte offsets; a larger stride (still fine for the
    128-column kernel) is served by that kernel"""
    from uniql_amd import ops
    p = make_linear_problem(260, 256, 256, seed=17)
    x, b, s = to_gpu(p, gpu)
    lda = (1 << 23) + 8
    big = torch.empty(260 * lda, dtype=torch.float16, device=gpu).view(260, lda)
    big[:, :256] = x
    y = ops.w4a16_gemm_ex(big[:, :256], b, s, workspace_for(256, gpu), 260, 256, 256, out_f32=True, flags=WIDE)
    assert np.abs(y.cpu().numpy() - reference_product(p, exact=True)).max() < 2e-4
    del big


def test_wide_kernel_in_a_graph(gpu):
    from uniql_amd import ops
    p = make_linear_problem(512, 512, 512, seed=12)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(512, gpu)
    eager = ops.w4a16_gemm_ex(x, b, s, ws, 512, 512, 512, flags=WIDE)
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.w4a16_gemm_ex(x, b, s, ws, 512, 512, 512, flags=WIDE)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out.copy_(ops.w4a16_gemm_ex(x, b, s, ws, 512, 512, 512, flags=WIDE))
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_wide_kernel_random_shapes(gpu):
    """600 seeded cases (rows 1..1100, K 256..2432 and a few long ones, 1..4 column blocks, strided
    rows, plain / cut + bias / residual / gated calls) against a float64 product of the bit-exact
    dequantised weights on the GPU; the hand-counted load pipeline has no shape it may miss"""
    from uniql_amd import ops
    import bench
    cache = {}
    for seed in range(600):
        rng = np.random.default_rng(seed)
        gen = torch.Generator(device=gpu).manual_seed(seed)
        k = 128 * int(rng.integers(2, 20)) if rng.integers(0, 6) else 128 * int(rng.integers(20, 120))
        n = 256 * int(rng.integers(1, 5))
        m = int(rng.integers(1, 1100))
        key = (k, n, seed % 3)
        if key not in cache:
            if len(cache) > 40:
                cache.clear()
            b, s = bench.make_weights(k, n, gpu, gen)
            cache[key] = (b, s, ops.w4a16_dequant(b, s, n, k).double())
        b, s, w = cache[key]
        lda = k + 8 * int(rng.integers(0, 5)) * int(rng.integers(0, 2))
        x = torch.randn((m, lda), device=gpu, generator=gen).half()[:, :k]
        ws = workspace_for(n, gpu)
        mode = int(rng.integers(0, 4))
        what = f"seed {seed}: m={m} k={k} n={n} lda={lda} mode={mode}"
        ref = x.double() @ w
        plain32 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True, flags=WIDE)
        assert float((plain32.double() - ref).abs().max()) < 3e-4, what
        plain16 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, flags=WIDE)
        assert torch.equal(plain16, plain32.half()), what
        if mode == 1:
            n_out = n - 8 * int(rng.integers(0, 20))
            bias = torch.randn(n_out, device=gpu, generator=gen).half()
            y = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, flags=WIDE)
            assert torch.equal(y, plain16[:, :n_out] + bias), what
        elif mode == 2:
            res = torch.randn((m, n), device=gpu, generator=gen).half()
            assert torch.equal(ops.w4a16_linear(x, b, s, ws, n, k, residual=res, flags=WIDE), res + plain16), what
        elif mode == 3:
            y = ops.w4a16_linear(x, b, s, ws, n, k, silu_mul=True, out_f32=True, flags=WIDE).double()
            v = ref.view(m, n // 128, 2, 64)
            g, u = v[:, :, 0].reshape(m, n // 2), v[:, :, 1].reshape(m, n // 2)
            want = g / (1 + torch.exp(-g)) * u
            assert float((y - want).abs().max()) < 1e-3 * max(1.0, float(want.abs().max())), what


@pytest.mark.parametrize("flags", [WIDE, NARROW])
def test_bias_and_residual_at_unaligned_addresses(gpu, flags):
    """bias and residual are read 16 bytes at a time where their addresses allow it: a bias that starts
    2 bytes off and a residual whose rows are 2 bytes off and an odd number of elements apart take
    the element loads and give the same result; so does the (gate, up) form with its second bias
    half at an odd offset"""
    from uniql_amd import ops
    m, k, n = 300, 256, 512
    p = make_linear_problem(m, k, n, seed=77)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    gen = torch.Generator().manual_seed(78)
    bias = torch.randn(n, generator=gen).half().to(gpu)
    res = torch.randn(m, n, generator=gen).half().to(gpu)
    want = ops.w4a16_linear(x, b, s, ws, n, k, bias=bias, residual=res, flags=flags)
    bias_off = torch.zeros(n + 8, dtype=torch.float16, device=gpu)
    bias_off[1:1 + n] = bias
    res_off = torch.zeros(m * (n + 3) + 8, dtype=torch.float16, device=gpu)
    res_view = res_off[1:1 + m * (n + 3)].view(m, n + 3)[:, :n]
    res_view.copy_(res)
    assert bias_off[1:1 + n].data_ptr() % 16 == 2 and res_view.stride(0) % 8 != 0
    got = ops.w4a16_linear(x, b, s, ws, n, k, bias=bias_off[1:1 + n], residual=res_view, flags=flags)
    assert torch.equal(got, want)
    # gated pairs: n / 2 outputs, bias = gate biases then up biases
    half = n // 2
    gbias = torch.randn(2 * half, generator=gen).half().to(gpu)
    want_g = ops.w4a16_linear(x, b, s, ws, n, k, bias=gbias, silu_mul=True, flags=flags)
    gb_off = torch.zeros(2 * half + 8, dtype=torch.float16, device=gpu)
    gb_off[3:3 + 2 * half] = gbias
    got_g = ops.w4a16_linear(x, b, s, ws, n, k, bias=gb_off[3:3 + 2 * half], silu_mul=True, flags=flags)
    assert torch.equal(got_g, want_g)
