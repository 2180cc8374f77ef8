"""uniql_w4a16_gemm_static (the entry point that allocates nothing, scratch memory in the library's
own static device array) against uniql_w4a16_gemm with caller-provided buffers: same kernels,
so the outputs must be identical bit for bit; one case per kind of scratch use also against the
oracle.  Every case runs two calls in a row, the second with a smaller input, because the
static array keeps the first call's contents."""
import ctypes

import numpy as np
import pytest
import torch

from tests import helpers as H
from uniql_amd import _capi, ops

pytestmark = pytest.mark.gpu

F16_BYTES = 2


def run_pair(dev, m, k, n, *, had_block=0, flags=0, seed=H.SEED, oracle=False):
    p = H.make_linear_problem(m, k, n, seed=seed)
    x, b, s = H.to_gpu(p, dev)
    ws = H.workspace_for(n, dev)
    scale = had_block ** -0.5 if had_block else 1.0
    want = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k, had_block=had_block, had_scale=scale, flags=flags)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=dev)
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    got = ops.w4a16_gemm_static(x, b, s, ws, out, m, n, k, had_block=had_block, had_scale=scale, flags=flags)
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before   # torch allocated nothing either
    torch.cuda.synchronize()
    assert torch.equal(got, want), f"m={m} k={k} n={n} had={had_block} flags={flags:#x}"
    if oracle and not had_block:
        H.check_layer_output(got.cpu().numpy(), H.reference_product(p))
    return got


# (first call, smaller second call): every kind of scratch use
CASES = [
    # streaming kernel, K split over workgroups: 64-bit exchange words
    dict(a=(4, 4096, 4096), b=(1, 2048, 1024), kw={}),
    dict(a=(16, 14336, 4096), b=(3, 4096, 2048), kw={}),
    # tiled kernel with K splits: arrival counts + fp32 partial tiles in the temporary area
    dict(a=(64, 4096, 1024), b=(32, 2048, 512), kw=dict(flags=(4 << 8) | (1 << 16))),
    # full-width rotation through the temporary area, then the streaming kernel
    dict(a=(8, 8192, 1024), b=(2, 4096, 512), kw=dict(had_block_full=True)),
    # rotation + tiled kernel
    dict(a=(48, 2048, 512), b=(20, 1024, 256), kw=dict(had_block_full=True)),
    # no scratch at all (whole K per workgroup)
    dict(a=(256, 1024, 512), b=(100, 512, 256), kw={}),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c["a"])))
def test_static_scratch_matches_caller_buffers(gpu, case):
    kw = dict(case["kw"])
    full = kw.pop("had_block_full", False)
    for i, (m, k, n) in enumerate((case["a"], case["b"])):
        run_pair(gpu, m, k, n, had_block=k if full else 0, seed=H.SEED + i, oracle=True, **kw)


def test_alternating_kernels_share_the_array(gpu):
    """Partial tiles of the tiled kernel overwrite the temporary area, the streaming kernel's exchange
    words must still be zero afterwards, and the other way round."""
    for m, k, n, flags in ((64, 4096, 1024, (4 << 8) | (1 << 16)), (4, 4096, 4096, 0),
                           (32, 2048, 512, (2 << 8) | (1 << 16)), (1, 14336, 4096, 0), (2, 512, 256, 0)):
        run_pair(gpu, m, k, n, flags=flags)


def test_static_limit_is_reported(gpu):
    lib = _capi.load()
    assert lib.uniql_w4a16_gemm_static_limit(0) == 4 << 20
    assert lib.uniql_w4a16_gemm_static_limit(1) == 12 << 20
    assert lib.uniql_w4a16_gemm_static_limit(2) == 0
    # 16 rows x 65536 columns of 64-bit exchange words = 8 MiB > 4 MiB: refused before any launch
    fake = ctypes.c_void_p(0x10000)
    rc = lib.uniql_w4a16_gemm_static(fake, 4096, fake, fake, fake, None, 0, 16, 65536, 4096, 32, 0, 1.0, 0, None)
    assert rc == -7
    assert b"static" in lib.uniql_status_string(rc)
    # a rotated 1024 x 8192 input needs 16 MiB of temporary area > 12 MiB
    rc = lib.uniql_w4a16_gemm_static(fake, 8192, fake, fake, fake, None, 0, 1024, 4096, 8192, 64, 8192, 1.0, 0, None)
    assert rc == -7
    # argument errors of the product come back unchanged, nothing is enqueued
    assert lib.uniql_w4a16_gemm_static(fake, 4096, fake, fake, fake, None, 0, 1, 4096 + 64, 4096, 32, 0, 1.0, 0, None) == -2
    assert lib.uniql_w4a16_gemm_static(None, 4096, fake, fake, fake, None, 0, 1, 4096, 4096, 32, 0, 1.0, 0, None) == -1
    assert lib.uniql_w4a16_gemm_static(None, 4096, None, None, None, None, 0, 0, 4096, 4096, 32, 0, 1.0, 0, None) == 0
    torch.cuda.synchronize()


def test_static_entry_point_in_a_graph(gpu):
    """the callers it is for: a captured graph replays the call (its clearing of the exchange words
    is a kernel, not a memset) and every replay gives the eager result, with other calls on the
    array between the replays"""
    m, k, n = 4, 4096, 4096
    p = H.make_linear_problem(m, k, n, seed=H.SEED + 7)
    x, b, s = H.to_gpu(p, gpu)
    ws = H.workspace_for(n, gpu)
    want = ops.w4a16_gemm_ex(x, b, s, ws, m, n, k)
    out = torch.zeros((m, n), dtype=torch.float16, device=gpu)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.w4a16_gemm_static(x, b, s, ws, out, m, n, k)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.w4a16_gemm_static(x, b, s, ws, out, m, n, k)
    for i in range(4):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
        run_pair(gpu, 64, 4096, 1024, flags=(4 << 8) | (1 << 16))   # the tiled kernel's partial tiles in between
