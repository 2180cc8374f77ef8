"""GPU parity of the int4 embedding gather and the Walsh-Hadamard transform (C ABI path)."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O

pytestmark = pytest.mark.gpu


def make_table(v, d, seed):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(v, d)).astype(np.int64)
    inter = O.EMB_INTERLEAVE
    words = np.zeros((v, d // 8), dtype=np.uint32)
    grouped = codes.reshape(v, d // 8, 8)[:, :, inter]
    for i in range(8):
        words |= (grouped[:, :, i].astype(np.uint32) & 15) << np.uint32(4 * i)
    scales = rng.uniform(0.004, 0.02, size=v).astype(np.float16)
    return words.view(np.int32), scales


@pytest.mark.parametrize("v,d,shape", [(64, 32, (5,)), (1000, 4096, (2, 7)), (50, 72, (3, 1)), (9, 8, (0,))])
def test_embedding_bit_exact(gpu, v, d, shape):
    from uniql_amd import ops
    packed, scales = make_table(v, d, v + d)
    rng = np.random.default_rng(1)
    ids = rng.integers(0, v, size=shape).astype(np.int64)
    out = ops.w4a16_embedding_lookup(torch.from_numpy(ids).to(gpu), torch.from_numpy(packed).to(gpu),
                                     torch.from_numpy(scales).to(gpu))
    want = O.embedding_lookup(ids, packed, scales)
    assert tuple(out.shape) == (*shape, d)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_embedding_scale_of_every_row_incl_the_last_of_an_odd_table(gpu):
    """The kernel reads a row's 16-bit scale as half of an aligned 32-bit word where that word lies
    inside the array, and as 16 bits otherwise: every id of an odd-sized and an even-sized table
    (the last row of the odd one has no such word), and a scales tensor that starts at an odd
    element of its storage (no 4-byte alignment)."""
    from uniql_amd import ops
    for v in (7, 8):
        packed, scales = make_table(v, 64, 40 + v)
        ids = np.arange(v, dtype=np.int64)
        want = O.embedding_lookup(ids, packed, scales)
        w = torch.from_numpy(packed).to(gpu)
        out = ops.w4a16_embedding_lookup(torch.from_numpy(ids).to(gpu), w, torch.from_numpy(scales).to(gpu))
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
        shifted = torch.zeros(v + 1, dtype=torch.float16, device=gpu)
        shifted[1:] = torch.from_numpy(scales).to(gpu)
        view = shifted[1:]
        assert view.data_ptr() % 4 == 2
        out = ops.w4a16_embedding_lookup(torch.from_numpy(ids).to(gpu), w, view)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_embedding_module_from_fp16(gpu):
    from uniql_amd.quantize.quant_embedding_layers import W4O16Embedding
    g = torch.Generator().manual_seed(3)
    emb = torch.nn.Embedding(300, 256).half()
    emb.weight.data = torch.randn(300, 256, generator=g).half()
    emb = emb.to(gpu)
    q = W4O16Embedding.from_fp16(emb)
    assert q.weight.dtype == torch.int32 and tuple(q.weight.shape) == (300, 32) and not q.weight.requires_grad
    assert q.scales.dtype == torch.float16 and tuple(q.scales.shape) == (300,)
    ids = torch.randint(0, 300, (4, 9), generator=g).to(gpu)
    out = q(ids)
    o_packed, o_scales = O.embedding_quantize(emb.weight.data.cpu())
    want = O.embedding_lookup(ids.cpu().numpy(), o_packed, o_scales)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # quantisation error of a symmetric 4-bit code: at most half a step (plus the clamp at +max)
    err = (out.float() - emb.weight.data[ids].float()).abs().amax(-1)
    step = q.scales[ids].float()
    assert bool((err <= step * 1.01).all())


def test_embedding_errors(gpu):
    from uniql_amd import ops
    packed, scales = make_table(16, 32, 0)
    w, s = torch.from_numpy(packed).to(gpu), torch.from_numpy(scales).to(gpu)
    ids = torch.zeros(3, dtype=torch.int64, device=gpu)
    with pytest.raises(RuntimeError):
        ops.w4a16_embedding_lookup(ids.int(), w, s)
    with pytest.raises(RuntimeError):
        ops.w4a16_embedding_lookup(ids, w.float(), s)
    with pytest.raises(RuntimeError):
        ops.w4a16_embedding_lookup(ids, w, s[:4])
    with pytest.raises(RuntimeError):
        ops.w4a16_embedding_lookup(ids.reshape(1, 1, 3), w, s)
    # ids outside the table give zeros (the reference would read out of bounds)
    bad = torch.tensor([0, 16, -1], dtype=torch.int64, device=gpu)
    out = ops.w4a16_embedding_lookup(bad, w, s)
    assert bool((out[1:] == 0).all()) and bool((out[0] != 0).any())


@pytest.mark.parametrize("dim", [2, 4, 8, 64, 128, 256, 1024, 4096, 8192, 32768])
def test_fwht_bit_exact_fp16(gpu, dim):
    """fp32 butterflies lowest bit first + one rounding: the oracle in fp32 is bit-identical."""
    from uniql_amd import ops
    rng = np.random.default_rng(dim)
    x = rng.standard_normal((3, dim)).astype(np.float16)
    y = ops.fast_hadamard_transform(torch.from_numpy(x).to(gpu), dim ** -0.5).cpu().numpy()
    want = O.fwht(x, dim ** -0.5)
    assert np.array_equal(y.view(np.uint16), want.view(np.uint16))


def test_fwht_blockwise_and_dtypes(gpu):
    from uniql_amd import ops
    rng = np.random.default_rng(6)
    x = rng.standard_normal((37, 1536)).astype(np.float16)       # 12 blocks of 128, 37 rows: ragged grid
    y = ops.hadamard_blockwise(torch.from_numpy(x).to(gpu), 128 ** -0.5, 128).cpu().numpy()
    assert np.array_equal(y.view(np.uint16), O.fwht(x, 128 ** -0.5, block=128).view(np.uint16))
    xf = rng.standard_normal((5, 2048)).astype(np.float32)
    yf = ops.fast_hadamard_transform(torch.from_numpy(xf).to(gpu), 2048 ** -0.5).cpu().numpy()
    assert np.array_equal(yf, O.fwht(xf, 2048 ** -0.5))
    xb = torch.from_numpy(xf).to(torch.bfloat16)
    yb = ops.fast_hadamard_transform(xb.to(gpu), 1.0).float().cpu().numpy()
    wantb = torch.from_numpy(O.fwht(xb.float().numpy(), 1.0)).to(torch.bfloat16).float().numpy()
    assert np.array_equal(yb, wantb)


def test_hadamard_module_and_involution(gpu):
    from uniql_amd.quantize.quant_hadamard_layers import Hadamard
    h = Hadamard(4096).to(gpu)
    assert h.N == 2 and abs(h.had_scale - 1 / 64) < 1e-12
    x = torch.randn(2, 3, 4096, generator=torch.Generator().manual_seed(0)).half().to(gpu)
    y = h(x)
    assert y.shape == x.shape and y.data_ptr() != x.data_ptr()
    want = O.hadamard_module_forward(x.cpu().numpy(), 4096)
    assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))
    back = h(y)
    assert float((back.float() - x.float()).abs().max()) < 5e-3
    with pytest.raises(AssertionError):
        Hadamard(12160)
    assert Hadamard(14336).N == 28 and Hadamard(3584).N == 28 and Hadamard(5120).N == 40


@pytest.mark.parametrize("dim", [12, 24, 1536, 20, 1280, 28, 3584, 14336, 40, 10240, 40960])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
def test_composite_hadamard_widths(gpu, dim, dtype):
    """fast_hadamard_transform_{12,20,28,40}N: bit for bit the oracle's fp32 arithmetic (same chunk
    transforms, same ascending sum over the base matrix, one rounding), and the module / helper
    pick the variant by width as the reference does.  The reference's own base matrices are not in
    its tree: parity with it is unpinned, the oracle pins the mathematics (tests/test_oracle_golden.py)."""
    from uniql_amd.quantize.hadamard_helpers import get_had_fn, had_transform
    fn, base, scale = get_had_fn(dim)
    assert base == O.had_variant(dim)[0] and base in (12, 20, 28, 40) and fn.__name__ == f"fast_hadamard_transform_{base}N"
    tdt = getattr(torch, dtype)
    x = torch.randn(3, dim, generator=torch.Generator().manual_seed(dim)).to(tdt)
    y = fn(x.to(gpu), scale)
    assert y.dtype == tdt and y.shape == x.shape
    if dtype == "bfloat16":     # numpy has no bfloat16: round the oracle's fp32 result with torch
        want32 = O.fwht_composite(x.float().numpy(), 1.0, base)
        want = (torch.from_numpy(want32) * torch.tensor(scale, dtype=torch.float32)).to(torch.bfloat16)
        assert torch.equal(y.cpu(), want)
    else:
        want = O.fwht_composite(x.numpy(), scale, base)
        assert np.array_equal(y.cpu().numpy().view(np.uint8), want.view(np.uint8))
    assert torch.equal(had_transform(x.to(gpu).view(3, 1, dim)).view(3, dim), y)


@pytest.mark.parametrize("din,dout", [(3584, 512), (1536, 14336), (1280, 640)])
def test_hadlinear_with_composite_widths(gpu, din, dout):
    """HadLinear on widths 28 * 128, 12 * 128, 28 * 512, 20 * 64, 20 * 32: rotating the input undoes the input-side
    rotation of the weight (H H^T = n I), the fused and the lazy form agree."""
    from uniql_amd.quantize.hadamard_helpers import get_had_fn
    from uniql_amd.quantize.quant_linear_layers import HadLinear
    g = torch.Generator().manual_seed(din + dout)
    lin = torch.nn.Linear(din, dout, bias=False).half().to(gpu)
    lin.weight.data = (torch.randn(dout, din, generator=g) * 0.05).half().to(gpu)
    x = torch.randn(4, din, generator=g).half().to(gpu)
    lazy = HadLinear(lin, input_transform=True, output_transform=True)
    fused = HadLinear(lin, input_transform=True, output_transform=True, fuse_had=True)
    fn_in, _, s_in = get_had_fn(din)
    fn_out, _, s_out = get_had_fn(dout)
    y_lazy, y_fused = lazy(fn_in(x, s_in)), fused(fn_in(x, s_in))
    assert float((y_lazy.float() - y_fused.float()).abs().max()) < 2e-2
    # y = (x H_in / sqrt(n)) (H_out^T W H_in / sqrt(n m))^T = (x W^T) H_out / sqrt(m): the plain product, output rotated
    want = fn_out(lin(x).float(), s_out)
    assert float((y_fused.float() - want).abs().max()) < 3e-2
