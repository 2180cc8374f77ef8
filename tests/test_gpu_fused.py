"""GPU parity of the fused layer call (uniql_w4a16_linear): input padding, output cut, bias and
the SiLU-gated MLP front inside the kernels, against the unfused sequence and the oracle."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import check_layer_output, fp16_half_ulp, make_linear_problem, to_gpu, workspace_for

pytestmark = pytest.mark.gpu

F_FORCE_SKINNY, F_FORCE_TILED = 1 << 1, 1 << 2


def accumulators_are_zero():
    from uniql_amd import ops
    torch.cuda.synchronize()
    return all(int(buf.count_nonzero()) == 0 for buf in ops._accum_cache.values())


def assert_close16(got, want, *, ulps, floor=0.0, differing=5e-3):
    """fp16 arrays equal up to `ulps` fp16 steps at the larger magnitude (plus an absolute
    `floor` for values that are themselves rounding noise of a cancelling sum), and different
    at all in at most a `differing` share of the elements (at least 2 allowed)."""
    a, b = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    diff = np.abs(a - b)
    step = 2 * fp16_half_ulp(np.maximum(np.abs(a), np.abs(b)))
    bad = diff > floor + ulps * step
    assert not bad.any(), f"{bad.sum()} elements differ by more than {ulps} steps; worst {diff.max():.4g}"
    assert (diff > 0).sum() <= max(2, differing * diff.size), f"{(diff > 0).mean():.3g} of the elements differ"


@pytest.mark.parametrize("m", [1, 3, 16, 17, 100, 256])
@pytest.mark.parametrize("k,n,n_out", [(256, 256, 200), (640, 384, 384), (4096, 3584, 3456)])
def test_cut_and_bias_equal_the_unfused_sequence(gpu, m, k, n, n_out):
    """bit-exact: same kernels, the cut and the bias only move into the epilogue"""
    from uniql_amd import ops
    p = make_linear_problem(m, k, n, seed=m + k + n)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    full = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k)
    bias = torch.from_numpy(np.random.default_rng(5).standard_normal(n_out).astype(np.float16)).to(gpu)
    y = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out)
    assert y.shape == (m, n_out) and torch.equal(y, full[:, :n_out])
    yb = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias)
    assert torch.equal(yb, full[:, :n_out] + bias)
    # fp32 output: bias added without rounding
    y32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, out_f32=True)
    full32 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True)
    assert torch.equal(y32, full32[:, :n_out] + bias.float())
    assert accumulators_are_zero()
    # and against the oracle's module forward with its roundings
    want = O.linear_forward_fp16(p["x"], p["packed"], p["s_perm"], in_features=k, out_features=n_out,
                                 bias=bias.cpu().numpy())
    prod = O.linear_forward_fp16(p["x"], p["packed"], p["s_perm"], in_features=k, out_features=n_out)
    diff = np.abs(yb.cpu().numpy().astype(np.float64) - want.astype(np.float64))
    # a last-bit difference of the product (a step at the product's magnitude, two if the two
    # products sit on either side of a power of two) survives the bias add, whose own rounding
    # can add a step at the sum's magnitude
    step = 8 * fp16_half_ulp(np.maximum(np.abs(prod.astype(np.float64)), np.abs(want.astype(np.float64))))
    # both kernels multiply the reference's fp16-rounded weights: same roundings throughout
    assert (diff <= step).all() and (diff > 0).mean() < 5e-3


@pytest.mark.parametrize("m", [1, 3, 16, 17, 100, 256])
@pytest.mark.parametrize("k,n,n_out", [(256, 256, 200), (4096, 3584, 3456)])
def test_residual_add_equals_the_unfused_sequence(gpu, m, k, n, n_out):
    """the decoder layer's `residual + layer(x)`: bit-exact against torch's fp16 add of the layer's
    output, with and without a bias, also in place (D = residual)"""
    from uniql_amd import ops
    p = make_linear_problem(m, k, n, seed=m + k)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    gen = torch.Generator().manual_seed(m)
    res = torch.randn(m, n_out, generator=gen).half().to(gpu)
    bias = torch.randn(n_out, generator=gen).half().to(gpu)
    plain = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out)
    assert torch.equal(ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, residual=res), res + plain)
    biased = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias)
    assert torch.equal(ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias, residual=res), res + biased)
    # a residual that is a column range of a wider tensor, and the result written over it
    wide = torch.randn(m, n_out + 24, generator=gen).half().to(gpu)
    view = wide[:, 8:8 + n_out]
    want = view + plain
    ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, residual=view, out=view)
    assert torch.equal(view, want)
    y32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, residual=res, out_f32=True)
    p32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, out_f32=True)
    assert torch.equal(y32, p32 + res.float())
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out // 2, residual=res[:, :n_out // 2], silu_mul=True)
    assert accumulators_are_zero()


@pytest.mark.parametrize("m", [1, 5, 16, 40, 130])
@pytest.mark.parametrize("k_in", [200, 248, 136])
def test_input_padding_inside_the_call(gpu, m, k_in):
    from uniql_amd import ops
    k, n = 256, 256
    p = make_linear_problem(m, k, n, seed=m + k_in)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    x_short = x[:, :k_in].contiguous()
    x_pad = torch.nn.functional.pad(x_short, (0, k - k_in))
    want = ops.w4a16_gemm_ex(x_pad, b, s, ws, m, n, k)
    got = ops.w4a16_linear(x_short, b, s, ws, n, k)
    assert torch.equal(got, want)
    # a row stride larger than the width (a column range of a wider tensor)
    got2 = ops.w4a16_linear(x[:, :k_in], b, s, ws, n, k)
    assert torch.equal(got2, want)
    # padding combined with the rotation (fused for m <= 16, transform kernel otherwise)
    want_h = ops.w4a16_gemm_ex(x_pad, b, s, ws, m, n, k, had_block=128, had_scale=128 ** -0.5)
    got_h = ops.w4a16_linear(x_short, b, s, ws, n, k, had_block=128, had_scale=128 ** -0.5)
    assert torch.equal(got_h, want_h)
    want_h = ops.w4a16_gemm_ex(x_pad, b, s, ws, m, n, k, had_block=256, had_scale=1 / 16)
    got_h = ops.w4a16_linear(x_short, b, s, ws, n, k, had_block=256, had_scale=1 / 16)
    assert torch.equal(got_h, want_h)
    assert accumulators_are_zero()


def test_odd_input_width_falls_back_to_a_padded_copy(gpu):
    from uniql_amd import ops
    m, k, n, k_in = 4, 256, 128, 203
    p = make_linear_problem(m, k, n, seed=9)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    x_short = x[:, :k_in].contiguous()
    want = ops.w4a16_gemm_ex(torch.nn.functional.pad(x_short, (0, k - k_in)), b, s, ws, m, n, k)
    assert torch.equal(ops.w4a16_linear(x_short, b, s, ws, n, k), want)


@pytest.mark.parametrize("m", [1, 16, 64])
def test_output_into_a_column_range(gpu, m):
    """`out` may be a view with a larger row stride, aligned or not"""
    from uniql_amd import ops
    k, n, n_out = 384, 256, 200
    p = make_linear_problem(m, k, n, seed=m)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    want = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k)[:, :n_out]
    for width, off in ((512, 8), (515, 3)):
        big = torch.full((m, width), 7.0, dtype=torch.float16, device=gpu)
        ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, out=big[:, off:off + n_out])
        assert torch.equal(big[:, off:off + n_out], want)
        assert bool((big[:, :off] == 7).all()) and bool((big[:, off + n_out:] == 7).all())


def gated_problem(m, k, width, seed):
    """gate and up projections of `width` columns each and their interleaved packing"""
    from uniql_amd import layout
    g = make_linear_problem(m, k, width, seed=seed)
    u = make_linear_problem(m, k, width, seed=seed + 1)
    u["x"] = g["x"]
    w, s = layout.interleave_gate_up(torch.from_numpy(g["packed"]), torch.from_numpy(g["s_perm"]),
                                     torch.from_numpy(u["packed"]), torch.from_numpy(u["s_perm"]))
    return g, u, w, s


def deinterleave(y, width):
    """columns of the interleaved product -> (gate, up)"""
    m = y.shape[0]
    v = y.reshape(m, width // 64, 2, 64)
    return v[:, :, 0].reshape(m, width), v[:, :, 1].reshape(m, width)


@pytest.mark.parametrize("m", [1, 2, 7, 16, 17, 64, 200])
@pytest.mark.parametrize("k,width,n_out", [(256, 128, 128), (512, 256, 200), (4096, 1024, 1024), (1408, 512, 448)])
def test_gated_epilogue(gpu, m, k, width, n_out):
    from uniql_amd import ops
    g, u, w, s = gated_problem(m, k, width, seed=m + k)
    x = torch.from_numpy(g["x"]).to(gpu)
    w, s = w.to(gpu), s.to(gpu)
    ws = workspace_for(2 * width, gpu)
    # the interleaved tensor is a valid layer of width 2*width: its plain product holds the
    # gate and up outputs block by block, equal to the separate layers' outputs
    both = ops.w4a16_gemm_ex(x, w, s, ws, m, 2 * width, k).cpu().numpy()
    g16, u16 = deinterleave(both, width)
    for part, prob in ((g16, g), (u16, u)):
        ref = O.gemm_fp64(prob["x"], O.dequant_codes(prob["q"], prob["s"]))
        check_layer_output(part, ref)
    # fused: same sums, then the reference's roundings
    y = ops.w4a16_linear(x, w, s, ws, 2 * width, k, out_features=n_out, silu_mul=True)
    assert y.shape == (m, n_out)
    want = O.mlp_gate_up(g16[:, :n_out], u16[:, :n_out])
    # SiLU's exp may differ in the last fp32 bit from numpy's: rarely one fp16 step of the
    # activation, which the product can turn into two steps of the result
    assert_close16(y.cpu().numpy(), want, ulps=2)
    # with biases on both projections
    bias = torch.from_numpy(np.random.default_rng(m).standard_normal(2 * n_out).astype(np.float16)).to(gpu)
    yb = ops.w4a16_linear(x, w, s, ws, 2 * width, k, out_features=n_out, silu_mul=True, bias=bias)
    bn = bias.cpu().numpy().astype(np.float32)
    gb = (g16[:, :n_out].astype(np.float32) + bn[:n_out]).astype(np.float16)
    ub = (u16[:, :n_out].astype(np.float32) + bn[n_out:]).astype(np.float16)
    assert_close16(yb.cpu().numpy(), O.mlp_gate_up(gb, ub), ulps=2)
    # fp32 output: no intermediate rounding
    y32 = ops.w4a16_linear(x, w, s, ws, 2 * width, k, out_features=n_out, silu_mul=True, out_f32=True)
    both32 = ops.w4a16_gemm_ex(x, w, s, ws, m, 2 * width, k, out_f32=True).cpu().numpy().astype(np.float64)
    g32, u32 = deinterleave(both32, width)
    want32 = g32[:, :n_out] / (1 + np.exp(-g32[:, :n_out])) * u32[:, :n_out]
    assert np.abs(y32.cpu().numpy() - want32).max() < 1e-5 * max(1.0, np.abs(want32).max())
    assert accumulators_are_zero()


@pytest.mark.parametrize("m,flags", [(1, 1 << 8), (4, (8 << 16) | (1 << 8)), (16, 1 << 8),
                                     (40, F_FORCE_TILED | (3 << 8)), (40, F_FORCE_SKINNY), (5, F_FORCE_TILED | (2 << 8)),
                                     (130, F_FORCE_TILED | (4 << 8) | (1 << 16))])
def test_gated_epilogue_with_k_split_over_workgroups(gpu, m, flags):
    """forced plans: partial sums of the pair meet in the accumulator words"""
    from uniql_amd import ops
    k, width = 2048, 256
    g, u, w, s = gated_problem(m, k, width, seed=m)
    x = torch.from_numpy(g["x"]).to(gpu)
    w, s = w.to(gpu), s.to(gpu)
    ws = workspace_for(2 * width, gpu)
    both = ops.w4a16_gemm_ex(x, w, s, ws, m, 2 * width, k, flags=flags).cpu().numpy()
    g16, u16 = deinterleave(both, width)
    for rep in range(3):  # repeated: the words must be back at zero every time
        y = ops.w4a16_linear(x, w, s, ws, 2 * width, k, silu_mul=True, flags=flags)
        assert_close16(y.cpu().numpy(), O.mlp_gate_up(g16, u16), ulps=2)
        assert accumulators_are_zero()


def make_layer(in_f, out_f, bias, seed, dev):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    gen = torch.Generator().manual_seed(seed)
    lin = torch.nn.Linear(in_f, out_f, bias=bias).half()
    lin.weight.data = (torch.randn(out_f, in_f, generator=gen) * 0.05).half()
    if bias:
        lin.bias.data = torch.randn(out_f, generator=gen).half()
    return W4A16B16O16Linear.from_fp16(lin.to(dev))


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("in_f,widths", [(512, (512, 128, 128)), (4096, (3456, 1024, 1024)), (200, (300, 40))])
def test_fused_projection_module(gpu, in_f, widths, bias):
    from uniql_amd.quantize.fused_layers import W4A16FusedLinear
    layers = [make_layer(in_f, w, bias, 10 + i, gpu) for i, w in enumerate(widths)]
    fused = W4A16FusedLinear.from_linears(layers)
    gen = torch.Generator().manual_seed(3)
    for shape in [(1, in_f), (2, 3, in_f), (70, in_f)]:
        x = torch.randn(*shape, generator=gen).half().to(gpu)
        outs = fused(x)
        assert len(outs) == len(layers)
        for y, layer in zip(outs, layers):
            want = layer(x)
            assert y.shape == want.shape
            # a different grid may sum K in another order: at most the last bit of a few outputs
            # (a bias that cancels the product turns the product's last bit into many steps of
            # the small sum: absolute floor of one step at the products' magnitude)
            assert_close16(y.cpu().numpy(), want.cpu().numpy(), ulps=1, floor=8e-3 if bias else 1e-4,
                           differing=2e-2)


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("in_f,width", [(512, 256), (4096, 12160), (200, 300)])
def test_gate_up_module(gpu, in_f, width, bias):
    from uniql_amd.quantize.fused_layers import W4A16GateUpSiLU
    gate, up = make_layer(in_f, width, bias, 21, gpu), make_layer(in_f, width, bias, 22, gpu)
    fused = W4A16GateUpSiLU.from_linears(gate, up)
    gen = torch.Generator().manual_seed(4)
    for shape in [(1, in_f), (2, 3, in_f), (70, in_f)]:
        x = torch.randn(*shape, generator=gen).half().to(gpu)
        y = fused(x)
        g16, u16 = gate(x).cpu().numpy(), up(x).cpu().numpy()
        want = O.mlp_gate_up(g16, u16)
        assert y.shape == (*shape[:-1], width)
        # the gate/up sums may differ from the separate layers' in the last bit (other grid): one
        # step of g is up to |u| steps of g in the product, plus the roundings of SiLU and of the
        # product itself
        floor = 4e-2 if bias else 1e-4   # with a bias: one step of the un-biased products times |up|
        assert_close16(y.cpu().numpy(), want, ulps=8, floor=floor, differing=5e-2)
        # and torch's own operators on the GPU give the same
        t = torch.nn.functional.silu(gate(x)) * up(x)
        assert_close16(y.cpu().numpy(), t.cpu().numpy(), ulps=8, floor=floor, differing=5e-2)


@pytest.mark.parametrize("m", [1, 3, 16, 17, 100, 256])
@pytest.mark.parametrize("k,n,n_out,bias", [(256, 256, 200, True), (4096, 3584, 3456, False), (1408, 512, 512, True)])
def test_squared_relu_epilogue_equals_the_unfused_sequence(gpu, m, k, n, n_out, bias):
    """act_fn(up_proj(x)) with the squared ReLU: bit-exact against the activation applied to the
    layer's own output (torch's operators on the fp16 tensor, as the reference runs them), and
    against the oracle's restatement on the same outputs."""
    from transformers.activations import ACT2FN
    from uniql_amd import ops
    p = make_linear_problem(m, k, n, seed=m + k + n + 1)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(n, gpu)
    bias_t = torch.from_numpy(np.random.default_rng(6).standard_normal(n_out).astype(np.float16)).to(gpu) if bias else None
    plain = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias_t)
    got = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias_t, relu2=True)
    assert torch.equal(got, ACT2FN["relu2"](plain))
    assert np.array_equal(got.cpu().numpy().view(np.uint16), O.relu2_fp16(plain.cpu().numpy()).view(np.uint16))
    assert not torch.signbit(got).any()                               # negatives give +0, never -0
    # fp32 output: the activation of the unrounded sum
    plain32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias_t, out_f32=True)
    got32 = ops.w4a16_linear(x, b, s, ws, n, k, out_features=n_out, bias=bias_t, relu2=True, out_f32=True)
    assert torch.equal(got32, torch.square(torch.relu(plain32)))
    assert accumulators_are_zero()


def test_squared_relu_mlp_module(gpu):
    """The un-gated MLP of the squared-ReLU models: down_proj(act_fn(up_proj(x))) with the
    activation inside the first layer's call (nemotron_h_qblocks.py:588)."""
    from transformers.activations import ACT2FN
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    g = torch.Generator().manual_seed(9)
    up = torch.nn.Linear(512, 1408, bias=True).half()
    down = torch.nn.Linear(1408, 512, bias=False).half()
    for lin in (up, down):
        lin.weight.data = (torch.randn(lin.weight.shape, generator=g) * 0.05).half()
    up.bias.data = torch.randn(1408, generator=g).half()
    qup, qdown = W4A16B16O16Linear.from_fp16(up.to(gpu)), W4A16B16O16Linear.from_fp16(down.to(gpu))
    x = torch.randn(2, 5, 512, generator=g).half().to(gpu)
    want = qdown(ACT2FN["relu2"](qup(x)))
    got = qdown(qup(x, activation="relu2"))
    assert got.shape == (2, 5, 512) and torch.equal(got, want)
    with pytest.raises(ValueError):
        qup(x, activation="gelu")


def test_fused_call_errors(gpu):
    from uniql_amd import ops
    p = make_linear_problem(2, 256, 256)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(256, gpu)
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x[:, :100], b, s, ws, 256, 256)              # more than one group missing
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, out_features=300)
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, out_features=200, silu_mul=True)   # at most n/2 pairs
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, bias=torch.zeros(100, dtype=torch.float16, device=gpu))
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, out=torch.empty(2, 256, dtype=torch.float32, device=gpu))
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, out_features=128, silu_mul=True, relu2=True)
    with pytest.raises(RuntimeError):
        ops.w4a16_linear(x, b, s, ws, 256, 256, relu2=True, residual=torch.zeros(2, 256, dtype=torch.float16, device=gpu))
