"""GPU parity at the exact sizes of the benchmark configurations: every Llama-3.1-8B linear at
M in {1, 2, 4, 8} (streaming kernel) and {256, 1024, 4096} (tiled kernel), the pruned Llama widths
(3456 / 12160, 128-block rotation fused ahead of down_proj), the Mamba2-8B block (in_proj
4096 -> 18560, 8192-point rotation + out_proj 8192 -> 4096, embedding 256000 x 4096 gathered for
2048 ids).

These matrices are too large for the CPU oracle in a test's time.  The reference product here is
torch's float64 matmul on the GPU over the weights uniql_w4a16_dequant returns, which
tests/test_gpu_linear.py holds bit-exact against the oracle (codes, every code x every scale); the
rotations come from the standalone transform kernel, bit-exact against the oracle in
tests/test_gpu_embedding_hadamard.py.  One CPU-oracle case per kernel stays in
tests/test_gpu_linear.py (test_stream_kernel_llama_shapes, test_tile_kernel_llama_shapes)."""
import numpy as np
import pytest
import torch

from oracle import uniql_oracle as O
from tests.helpers import PRE_ROUNDING_BOUND, check_layer_output_torch

pytestmark = pytest.mark.gpu

LLAMA = {"qkv": (4096, 6144), "o_proj": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}
# measured maxima of |fp32 result - float64 product of the fp16-rounded weights| are printed with -s
_seen = {}


def random_layer(k, n, dev, seed):
    """packed words (every nibble uniform in 0..15), permuted scales U[0.004, 0.02], workspace"""
    g = torch.Generator(device=dev).manual_seed(seed)
    b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), generator=g, device=dev, dtype=torch.int64).to(torch.int32)
    s = (torch.rand(k // 128, n, generator=g, device=dev) * 0.016 + 0.004).half()
    ws = torch.zeros((n // 64) * 16, dtype=torch.int32, device=dev)
    return b, s, ws, g


def reference64(x, b, s, n, k):
    from uniql_amd import ops
    w = ops.w4a16_dequant(b, s, n, k)          # fp16_rn((code - 8) * scale): the reference's weights
    return x.double() @ w.double()


def check_both_outputs(x, b, s, ws, m, n, k, ref, pre_bound, tag, **kw):
    """fp32 output (the value before the final rounding) within pre_bound of the float64 product,
    fp16 output = that value rounded once, and inside the path's tolerance."""
    from uniql_amd import ops
    y32 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, out_f32=True, **kw)
    d = float((y32.double() - ref).abs().max())
    _seen[tag] = max(_seen.get(tag, 0.0), d)
    print(f"{tag}: max |y32 - ref| = {d:.3e}")
    assert d < pre_bound, (tag, d)
    y16 = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, **kw)
    assert torch.equal(y16, y32.half())
    check_layer_output_torch(y16, ref)
    assert int(ws.count_nonzero()) == 0
    for buf in ops._accum_cache.values():
        assert int(buf.count_nonzero()) == 0


# ------------------------------------------------------------------ decode sweep
@pytest.mark.parametrize("m", [1, 2, 4, 8])
@pytest.mark.parametrize("name", list(LLAMA))
def test_decode_sweep_llama_shapes(gpu, name, m):
    """The streaming kernel expands every weight to the reference's fp16 value before the matrix
    unit: its value before the final rounding is the float64 product of those weights up to fp32
    accumulation error, on the real shapes, K = 14336 included."""
    k, n = LLAMA[name]
    b, s, ws, g = random_layer(k, n, gpu, seed=1000 + 10 * m + len(name))
    x = torch.randn(m, k, generator=g, device=gpu).half()
    ref = reference64(x, b, s, n, k)
    check_both_outputs(x, b, s, ws, m, n, k, ref, PRE_ROUNDING_BOUND, f"stream {name} m={m}")


# ------------------------------------------------------------------ prefill sweep
@pytest.mark.parametrize("m", [256, 1024, 4096])
@pytest.mark.parametrize("name", list(LLAMA))
def test_prefill_sweep_llama_shapes(gpu, name, m):
    """The tiled kernel multiplies the reference's fp16-rounded weights: only fp32 accumulation
    error separates its value before rounding from the float64 product."""
    k, n = LLAMA[name]
    b, s, ws, g = random_layer(k, n, gpu, seed=2000 + m + len(name))
    x = torch.randn(m, k, generator=g, device=gpu).half()
    ref = reference64(x, b, s, n, k)
    check_both_outputs(x, b, s, ws, m, n, k, ref, PRE_ROUNDING_BOUND, f"tile {name} m={m}")


# ------------------------------------------------------------------ pruned Llama, through the module
def pruned_module(in_f, out_f, dev, seed):
    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    layer = W4A16B16O16Linear(in_f, out_f, device=dev)
    b, s, _, g = random_layer(layer.size_k, layer.size_n, dev, seed)
    layer.weight.copy_(b)
    layer.scale.copy_(s)
    return layer, g


@pytest.mark.parametrize("m", [1, 1024])
@pytest.mark.parametrize("name,in_f,out_f,had", [("q", 4096, 3456, 0), ("o", 3456, 4096, 0),
                                                 ("gate_up", 4096, 24320, 0), ("down", 12160, 4096, 128)])
def test_pruned_llama_shapes(gpu, name, in_f, out_f, had, m):
    """Layer ratio 0.85: attention width 3456 (padded to 3584 output columns), MLP width 12160;
    down_proj rotates its input online in 128-wide blocks (fused into the streaming kernel at
    m = 1, a transform launch ahead of the tiled kernel at m = 1024)."""
    from uniql_amd import ops
    layer, g = pruned_module(in_f, out_f, gpu, seed=3000 + m + len(name))
    assert layer.size_n % 256 == 0 and layer.size_n - out_f == layer.pad_out
    if had:
        layer.set_online_hadamard(had)
    x = torch.randn(m, in_f, generator=g, device=gpu).half()
    xr = ops.hadamard_blockwise(x, had ** -0.5, had) if had else x
    ref = reference64(xr, layer.weight, layer.scale, layer.size_n, layer.size_k)[:, :out_f]
    y = layer(x)
    assert tuple(y.shape) == (m, out_f)
    check_layer_output_torch(y, ref)
    y32 = ops.w4a16_linear(x, layer.weight, layer.scale, layer.workspace, layer.size_n, layer.size_k,
                           out_features=out_f, had_block=had, had_scale=had ** -0.5 if had else 1.0, out_f32=True)
    d = float((y32.double() - ref).abs().max())
    print(f"pruned {name} m={m}: max |y32 - ref| = {d:.3e}")
    assert d < PRE_ROUNDING_BOUND


# ------------------------------------------------------------------ Mamba2-8B block
@pytest.mark.parametrize("m", [1, 2, 3, 16, 1024])
def test_mamba_in_proj(gpu, m):
    """4096 -> 18560 = 2 * 8192 + 2 * 8 * 128 + 128, padded to 18688 output columns (146 strips: at one and
    two rows the streaming kernel's plan of many one-group workgroups, from three rows on 8 waves)."""
    layer, g = pruned_module(4096, 18560, gpu, seed=4000 + m)
    assert layer.size_n == 18688 and tuple(layer.weight.shape) == (256, 37376)
    x = torch.randn(m, 4096, generator=g, device=gpu).half()
    ref = reference64(x, layer.weight, layer.scale, layer.size_n, layer.size_k)[:, :18560]
    y = layer(x)
    assert tuple(y.shape) == (m, 18560)
    check_layer_output_torch(y, ref)


@pytest.mark.parametrize("m", [1, 1024])
def test_mamba_out_proj_with_full_rotation(gpu, m):
    """8192-point Walsh-Hadamard over the whole row, then 8192 -> 4096.  The rotated activations
    of the reference come from the CPU oracle (fp32 butterflies, one fp16 rounding)."""
    k, n = 8192, 4096
    b, s, ws, g = random_layer(k, n, gpu, seed=4100 + m)
    x = torch.randn(m, k, generator=g, device=gpu).half()
    xr = torch.from_numpy(O.fwht(x.cpu().numpy(), k ** -0.5)).to(gpu)
    ref = reference64(xr, b, s, n, k)
    check_both_outputs(x, b, s, ws, m, n, k, ref, PRE_ROUNDING_BOUND, f"mamba out_proj m={m}",
                       had_block=k, had_scale=k ** -0.5)


def test_mamba_embedding_full_table(gpu):
    """256000 x 4096 table (500 MiB packed), 2048 ids drawn uniformly; the oracle expands only
    the gathered rows.  Bit-exact."""
    from uniql_amd import ops
    v, d, t = 256000, 4096, 2048
    g = torch.Generator(device=gpu).manual_seed(4200)
    table = torch.randint(-2 ** 31, 2 ** 31 - 1, (v, d // 8), generator=g, device=gpu, dtype=torch.int64).to(torch.int32)
    scales = (torch.rand(v, generator=g, device=gpu) * 0.016 + 0.004).half()
    ids = torch.randint(0, v, (t,), generator=g, device=gpu)
    ids[0], ids[1] = 0, v - 1                                   # both ends of the table
    out = ops.w4a16_embedding_lookup(ids, table, scales)
    assert tuple(out.shape) == (t, d)
    want = O.embedding_lookup(np.arange(t), table[ids].cpu().numpy(), scales[ids].cpu().numpy())
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
    out2 = ops.w4a16_embedding_lookup(ids.view(2, t // 2), table, scales)      # [B, S] ids
    assert torch.equal(out2.view(t, d), out)
