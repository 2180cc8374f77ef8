"""The drop-in module classes on the GPU: buffers, from_fp16, forward semantics."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import check_layer_output

pytestmark = pytest.mark.gpu


def make_linear(in_f, out_f, bias, seed):
    g = torch.Generator().manual_seed(seed)
    lin = torch.nn.Linear(in_f, out_f, bias=bias).half()
    lin.weight.data = (torch.randn(out_f, in_f, generator=g) * 0.05).half()
    if bias:
        lin.bias.data = torch.randn(out_f, generator=g).half()
    return lin


@pytest.mark.parametrize("in_f,out_f,bias", [(256, 256, False), (200, 300, True), (4096, 3456, False),
                                             (3456, 4096, False)])
def test_linear_module_matches_oracle(gpu, in_f, out_f, bias):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    lin = make_linear(in_f, out_f, bias, in_f + out_f).to(gpu)
    q = W4A16B16O16Linear.from_fp16(lin)
    geo = O.linear_geometry(in_f, out_f)
    assert (q.size_k, q.size_n, q.pad_in, q.pad_out) == (geo["size_k"], geo["size_n"], geo["pad_in"], geo["pad_out"])
    assert tuple(q.weight.shape) == geo["weight"] and q.weight.dtype == torch.int32
    assert tuple(q.scale.shape) == geo["scale"] and q.scale.dtype == torch.float16
    assert q.workspace.numel() == geo["workspace"] and q.workspace.dtype == torch.int32
    assert set(q.state_dict()) == {"workspace", "weight", "scale"} | ({"bias"} if bias else set())
    # packed tensors equal the oracle's quantiser on the same weights
    _, o_packed, o_scale = O.w4a16_quantize(lin.weight.data.cpu().t().contiguous(), 128, None, geo["pad_out"])
    assert torch.equal(q.weight.cpu(), o_packed) and torch.equal(q.scale.cpu(), o_scale)
    g = torch.Generator().manual_seed(1)
    for shape in [(1, in_f), (2, 3, in_f), (70, in_f)]:
        x = torch.randn(*shape, generator=g).half()
        y = q(x.to(gpu))
        assert y.shape == (*shape[:-1], out_f) and y.dtype == torch.float16
        ref = O.linear_forward(x.numpy(), o_packed.numpy(), o_scale.numpy(), in_features=in_f,
                               out_features=out_f, exact=True)
        if bias:
            # the module adds the bias to the rounded fp16 product (quant_linear_layers.py:113-114)
            ref16 = ref.astype(np.float16)
            want = (torch.from_numpy(ref16) + lin.bias.data.cpu()).numpy()
            diff = np.abs(y.cpu().numpy().astype(np.float64) - want.astype(np.float64))
            assert diff.max() <= 2e-2
        else:
            check_layer_output(y.cpu().numpy(), ref)
    assert int(q.workspace.abs().sum()) == 0


def test_linear_module_empty_constructor_and_state_dict_roundtrip(gpu):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    lin = make_linear(384, 512, True, 2).to(gpu)
    src = W4A16B16O16Linear.from_fp16(lin)
    dst = W4A16B16O16Linear(384, 512, bias=True, device=gpu)
    dst.load_state_dict(src.state_dict(), strict=True)
    x = torch.randn(3, 384).half().to(gpu)
    assert torch.equal(src(x), dst(x))
    assert "W4A16B16O16Linear(in_features=384, out_features=512, bias=True)" == repr(dst)


def test_online_hadamard_extension(gpu):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    in_f, out_f = 1536, 256
    lin = make_linear(in_f, out_f, False, 3).to(gpu)
    q = W4A16B16O16Linear.from_fp16(lin).set_online_hadamard(128)
    x = torch.randn(2, in_f, generator=torch.Generator().manual_seed(2)).half()
    y = q(x.to(gpu)).cpu().numpy()
    xr = O.fwht(x.numpy(), 128 ** -0.5, block=128)
    ref = O.linear_forward(xr, q.weight.cpu().numpy(), q.scale.cpu().numpy(), in_features=in_f,
                           out_features=out_f, exact=True)
    check_layer_output(y, ref)


def test_hadlinear(gpu):
    from uniql_amd.quantize.quant_linear_layers import HadLinear
    lin = make_linear(256, 128, False, 4).to(gpu)
    x = torch.randn(5, 256, generator=torch.Generator().manual_seed(5)).half().to(gpu)
    lazy = HadLinear(lin, input_transform=True, output_transform=False, fuse_had=False)
    fused = HadLinear(lin, input_transform=True, output_transform=False, fuse_had=True)
    want_w = O.hadlinear_fused_weight(lin.weight.data.cpu().numpy(), True, False)
    assert np.array_equal(fused.weight.data.cpu().numpy().view(np.uint16), want_w.view(np.uint16))
    assert torch.equal(lazy(x), fused(x))
    # rotating the activation with the same matrix undoes the weight rotation
    from uniql_amd import ops
    xr = ops.fast_hadamard_transform(x, 256 ** -0.5)
    assert float((fused(xr).float() - lin(x).float()).abs().max()) < 2e-2
    both = HadLinear(lin, input_transform=True, output_transform=True, fuse_had=True)
    want_both = O.hadlinear_fused_weight(lin.weight.data.cpu().numpy(), True, True)
    assert np.array_equal(both.weight.data.cpu().numpy().view(np.uint16), want_both.view(np.uint16))


def test_extension_aliases_and_graph_capture(gpu):
    import uniql_amd
    uniql_amd.install_extension_aliases()
    import quant_embedding_cuda
    import quant_linear_cuda
    from tests.helpers import make_linear_problem, reference_product, to_gpu, workspace_for
    assert callable(quant_embedding_cuda.w4a16_embedding_lookup)
    p = make_linear_problem(1, 4096, 4096, seed=9)
    x, b, s = to_gpu(p, gpu)
    ws = workspace_for(4096, gpu)
    eager = quant_linear_cuda.w4a16o16_gemm(x, b, s, ws, 1, 4096, 4096, False, -1, -1, -1, 16)
    # the call allocates through torch's caching allocator and never synchronises: capturable
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            quant_linear_cuda.w4a16o16_gemm(x, b, s, ws, 1, 4096, 4096, False, -1, -1, -1, 16)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = quant_linear_cuda.w4a16o16_gemm(x, b, s, ws, 1, 4096, 4096, False, -1, -1, -1, 16)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
    check_layer_output(out.cpu().numpy(), reference_product(p))


def test_empty_inputs(gpu):
    """Zero tokens go through every module without a launch and give correctly shaped, empty
    results (a batch whose sequences have all finished, an empty id list)."""
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    from uniql_amd.quantize.quant_embedding_layers import W4O16Embedding
    from uniql_amd.quantize.quant_hadamard_layers import Hadamard
    from uniql_amd.quantize.fused_layers import W4A16FusedLinear, W4A16GateUpSiLU
    from uniql_amd import ops

    q = W4A16B16O16Linear.from_fp16(make_linear(200, 300, True, 3).to(gpu))
    for shape in [(0, 200), (2, 0, 200), (0, 5, 200)]:
        y = q(torch.empty(shape, dtype=torch.float16, device=gpu))
        assert y.shape == (*shape[:-1], 300) and y.dtype == torch.float16
    a = W4A16B16O16Linear.from_fp16(make_linear(256, 256, False, 4).to(gpu))
    b = W4A16B16O16Linear.from_fp16(make_linear(256, 512, False, 5).to(gpu))
    parts = W4A16FusedLinear.from_linears([a, b])(torch.empty(0, 256, dtype=torch.float16, device=gpu))
    assert [tuple(p.shape) for p in parts] == [(0, 256), (0, 512)]
    h = W4A16GateUpSiLU.from_linears(b, b)(torch.empty(3, 0, 256, dtype=torch.float16, device=gpu))
    assert h.shape == (3, 0, 512)

    emb = torch.nn.Embedding(64, 128).half().to(gpu)
    e = W4O16Embedding.from_fp16(emb)
    for shape in [(0,), (2, 0)]:
        out = e(torch.empty(shape, dtype=torch.int64, device=gpu))
        assert out.shape == (*shape, 128) and out.dtype == torch.float16

    assert Hadamard(256).to(gpu)(torch.empty(0, 256, dtype=torch.float16, device=gpu)).shape == (0, 256)

    qh = torch.empty(1, 0, 4, 64, dtype=torch.float16, device=gpu)
    kh = torch.empty(1, 0, 2, 64, dtype=torch.float16, device=gpu)
    cos = torch.empty(1, 0, 64, dtype=torch.float16, device=gpu)
    idx = torch.arange(32, device=gpu, dtype=torch.int32).repeat(2, 1)
    idx = torch.cat([idx, idx], dim=1).contiguous()
    ops.rope_indices_(qh, kh, cos, cos.clone(), idx)

    # the empty calls above leave later calls intact
    x = torch.randn(2, 200).half().to(gpu)
    assert torch.isfinite(q(x)).all()
    torch.cuda.synchronize()
