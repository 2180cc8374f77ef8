"""Benchmark of the W4A16 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sweep [--sweep-json PATH]] [--no-cpu]

Default workload (the line the driver records): the decode sweep's M = 1 column,
"llama31_8b_decode_layer_m1": one step = the four W4A16 GEMVs of a Llama-3.1-8B
decoder layer at M = 1 (fused qkv 4096->6144, o_proj 4096->4096, fused gate_up
4096->28672, down_proj 14336->4096; group 128, fp16 scales, fp16 activations).
Inputs are synthetic (codes U{0..15}, scales U[0.004,0.02], x ~ N(0,1), seed 1234) and
resident in HBM before the timed region.  Successive steps use different weight
copies whose total size exceeds the 256 MB last-level cache, so the weights come
from HBM, not from cache.  Steps are replayed as HIP graphs of about 40 steps each, so
that launch overhead is the GPU's, not Python's, and replay boundaries are rare.

value = algorithmic bytes per step / time per step  (GB/s), algorithmic bytes of a
linear = K N / 2 + (K/128) N 2 + M K 2 + M N 2.  The same JSON line carries, under
"prefill_gemm_m1024", the other half of the metric: the four linears at M = 1024 through
the tiled MFMA kernels (TFLOP/s = 2 M K N / time, against 2.5 PFLOP/s dense fp16).

The line also carries, compactly (microseconds and the fraction of the bounding peak each), every
other size the metric is quoted on: "decode_sweep" (the four linears at M = 2, 4, 8 and the
model's last layer 4096 -> 128256 at M = 1), "prefill_sweep" (M = 256 and 4096), "pruned_llama"
(the four structured-pruned shapes at M = 1 and 1024, down_proj behind the fused 128-block
rotation), "mamba2" (in_proj, the 8192-point rotation + out_proj at M = 1 and 1024, the 4-bit
embedding gather of 2048 ids from 256000 x 4096), "secondary_kernels" (standalone transform,
rotary kernel), "library_fp16_gemm_m1024" (torch.matmul on the same weights dequantised
beforehand, same timing) and "mfma_only_loop" (what the matrix pipe alone sustains on such data),
"eager_us_per_call" (the module's forward without graphs, host cost included).

--sweep additionally prints (stderr) and writes (--sweep-json, default bench_sweep.json in the
working directory) the fused-layer comparisons: cache-resident decode, the MLP front with the
SiLU epilogue against the unfused sequence, a decoder layer's linears and glue as 5 against 12
launches, more transform and rotary sizes.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16
LLC_BYTES = 256 << 20
# HBM bytes per launch of the default workload (mean over the four linears) come from two
# rocprofv3 --pmc runs of this file, FETCH_SIZE and WRITE_SIZE, each scaled by the reading for a
# 128 MiB elementwise copy (--pmc-calibrate); the summary of those runs is a tracked file, and
# the figure is read from its "traffic_bytes_per_launch = N" line at run time, so it cannot
# outlive the profile it came from.
TRAFFIC_PROFILE = os.path.join("profiles", "w4a16_stream_kernel_llama31_8b_decode_layer_m1_hbm_traffic.txt")


def measured_traffic():
    """(bytes per launch or None, source)"""
    import re
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", f.read())
        return (int(m.group(1)) if m else None), TRAFFIC_PROFILE
    except OSError:
        return None, TRAFFIC_PROFILE

LLAMA_DECODE = [("qkv", 4096, 6144), ("o_proj", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]
PRUNED = [("q_pruned", 4096, 3584, 0), ("o_pruned", 3456, 4096, 0), ("gate_up_pruned", 4096, 24320, 0),
          ("down_pruned_had128", 12160, 4096, 128)]
MAMBA = [("mamba_in_proj", 4096, 18688, 0), ("mamba_out_proj_had8192", 8192, 4096, 8192)]


def linear_bytes(m, k, n):
    return k * n // 2 + (k // 128) * n * 2 + m * k * 2 + m * n * 2


def linear_flops(m, k, n):
    return 2 * m * k * n


# --------------------------------------------------------------------------------------
def make_weights(k, n, dev, gen):
    """Random packed tensors directly on the device: uniformly random 32-bit words are
    uniformly random int4 codes in every nibble of the packed layout."""
    import torch
    b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int64, device=dev, generator=gen).to(torch.int32)
    s = (torch.rand((k // 128, n), device=dev, generator=gen) * 0.016 + 0.004).to(torch.float16)
    return b, s


class Layer:
    """One linear shape with `copies` independent weight sets."""

    def __init__(self, name, k, n, m, copies, dev, gen, had_block=0):
        import torch
        self.name, self.k, self.n, self.m, self.had_block = name, k, n, m, had_block
        self.weights = [make_weights(k, n, dev, gen) for _ in range(copies)]
        self.x = torch.randn((m, k), device=dev, generator=gen).to(torch.float16)
        self.ws = torch.zeros((n // 64) * 16, dtype=torch.int32, device=dev)

    def run(self, i):
        from uniql_amd import ops
        b, s = self.weights[i % len(self.weights)]
        if self.had_block:
            return ops.w4a16_gemm_ex(self.x, b, s, self.ws, self.m, self.n, self.k, had_block=self.had_block,
                                     had_scale=self.had_block ** -0.5)
        return ops.w4a16o16_gemm(self.x, b, s, self.ws, self.m, self.n, self.k, False, -1, -1, -1, 16)


SETTLE_MS = 10.0   # untimed replays before every timed region, whatever --warmup says
GRAPH_STEPS = 40   # steps captured per HIP graph (a decode step of a 32-layer model replays more kernels than that)


def time_graphs(run_step, n_variants, steps, warmup):
    """Times exactly `steps` calls of run_step(i), i cycling over n_variants, as HIP graph
    replays: one graph holds a multiple of n_variants consecutive steps (about GRAPH_STEPS; a
    second, shorter graph the remainder), so the per-replay launch cost is shared by many
    kernels.  Returns (seconds per step from events on the launch stream, wall seconds per step)."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_variants):
            run_step(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    keep = []

    def capture(count):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(count):
                keep.append(run_step(i % n_variants))
        return g

    per_graph = n_variants * max(1, min(steps, GRAPH_STEPS) // n_variants)
    full = capture(per_graph)
    rest = capture(steps % per_graph) if steps % per_graph else None
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # untimed: the `warmup` steps asked for, and in any case SETTLE_MS of replays, because the clocks of a
    # chip that was idle need several milliseconds of load to settle (one replay is well under 1 ms)
    start.record()
    for _ in range(max(1, warmup // per_graph)):
        full.replay()
    stop.record()
    torch.cuda.synchronize()
    per_replay_ms = max(start.elapsed_time(stop) / max(1, warmup // per_graph), 1e-3)
    for _ in range(int(SETTLE_MS / per_replay_ms) + 1):
        full.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps // per_graph):
        full.replay()
    if rest is not None:
        rest.replay()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) * 1e-3 / steps, wall / steps


def copies_for(bytes_per_copy):
    return max(2, int(np.ceil(1.5 * LLC_BYTES / bytes_per_copy)) + 1)


# --------------------------------------------------------------------------------------
def cpu_baseline(budget_s=4.0):
    """The reference's CPU meaning of the layer (unpack -> un-permute -> (q-8)*s -> fp32 matmul),
    restated by the oracle, timed on this host: the four decoder-layer linears at M = 1 (the
    workload of `value`) and o_proj at M = 1024.  Every shape runs once untimed and then at least
    twice, as often as fits `budget_s` seconds (at most 5 times); the median is reported."""
    import torch

    from oracle import uniql_oracle as O
    rng = np.random.default_rng(1234)
    per_shape, tot_bytes, tot_sec = {}, 0, 0.0

    def one(name, m, k, n):
        packed = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(k // 16, 2 * n), dtype=np.int64).astype(np.int32)
        s_perm = rng.uniform(0.004, 0.02, size=(k // 128, n)).astype(np.float16)
        x = rng.standard_normal((m, k)).astype(np.float16)
        times, matmul = [], []
        O.gemm_fp32(x, O.dequant_packed(packed, s_perm, k, n))   # untimed: first-touch page faults, thread pool start
        while True:
            t0 = time.perf_counter()
            w = O.dequant_packed(packed, s_perm, k, n)
            t1 = time.perf_counter()
            O.gemm_fp32(x, w)
            t2 = time.perf_counter()
            times.append(t2 - t0)
            matmul.append(t2 - t1)
            if len(times) >= 5 or (len(times) >= 2 and sum(times) + times[-1] > budget_s):
                break
        sec = float(np.median(times))
        per_shape[f"{name}_m{m}"] = {"ms": round(sec * 1e3, 1), "matmul_ms": round(float(np.median(matmul)) * 1e3, 2),
                                     "runs": len(times), "gbs": round(linear_bytes(m, k, n) / sec / 1e9, 4)}
        return sec

    for name, k, n in LLAMA_DECODE:
        tot_sec += one(name, 1, k, n)
        tot_bytes += linear_bytes(1, k, n)
    one("o_proj", 1024, 4096, 4096)
    return {
        "value": round(tot_bytes / tot_sec / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "the four decoder-layer linears at M=1 (value = their bytes / their summed median times), plus o_proj at "
                  "M=1024; per call: unpack + un-permute + dequant (numpy, one thread) + fp32 matmul (torch, `cores` threads); "
                  f"host has {os.cpu_count()} cpus",
        "per_shape": per_shape,
    }


# --------------------------------------------------------------------------------------
def sweep(dev, gen, out_path):
    import torch

    from uniql_amd import ops
    rows = []

    def bench_linear(name, k, n, m, had_block=0, steps=200, copies=None):
        per = linear_bytes(m, k, n)
        if copies is None:
            copies = copies_for(k * n // 2) if m <= 64 else 2
        layer = Layer(name, k, n, m, copies, dev, gen, had_block)
        sec, _ = time_graphs(lambda i: layer.run(i), copies, steps, max(20, steps // 2))
        row = dict(op=name, m=m, k=k, n=n, had_block=had_block, us=sec * 1e6, gbs=per / sec / 1e9,
                   hbm_frac=per / sec / 1e9 / HBM_PEAK_GBS, tflops=linear_flops(m, k, n) / sec / 1e12,
                   mfma_frac=linear_flops(m, k, n) / sec / 1e12 / MFMA_F16_PEAK_TFLOPS)
        rows.append(row)
        print("%-24s M=%-5d K=%-6d N=%-6d %9.2f us %8.1f GB/s (%5.1f%% HBM) %8.1f TFLOP/s (%5.1f%% MFMA)" % (
            name, m, k, n, row["us"], row["gbs"], 100 * row["hbm_frac"], row["tflops"], 100 * row["mfma_frac"]),
            file=sys.stderr, flush=True)
        del layer
        torch.cuda.empty_cache()

    # the M = 1 launches over ONE copy of the weights: they stay in the 256 MB last-level cache
    # between steps, which a model of several GB never sees; reported beside the cold numbers only
    for name, k, n in LLAMA_DECODE:
        bench_linear(name + "_cache_resident", k, n, 1, copies=1)
    for name, n in (("lm_head_llama31", 128256), ("lm_head_mamba2", 256000)):
        for m in (1, 8):
            bench_linear(name, 4096, n, m, steps=60)

    for rows_x, dim, block in ((1, 8192, 8192), (1024, 8192, 8192), (1024, 12160 + 128, 128)):
        xs = [torch.randn((rows_x, dim), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
        sec, _ = time_graphs(lambda i: ops.hadamard_blockwise(xs[i], block ** -0.5, block), 4, 200, 20)
        per = rows_x * dim * 4
        rows.append(dict(op=f"fwht_block{block}", rows=rows_x, dim=dim, us=sec * 1e6, gbs=per / sec / 1e9))
        print("fwht rows=%d dim=%d block=%d: %.2f us %.1f GB/s" % (rows_x, dim, block, sec * 1e6, per / sec / 1e9),
              file=sys.stderr, flush=True)

    # MLP front act(gate(x)) * up(x): one launch with the epilogue against the product followed by
    # torch's silu and multiply (random words are random interleaved gate/up weights just as well)
    k, width = 4096, 14336
    for m in (1, 8, 1024):
        copies = copies_for(k * width) if m <= 64 else 2
        weights = [make_weights(k, 2 * width, dev, gen) for _ in range(copies)]
        x = torch.randn((m, k), device=dev, generator=gen).to(torch.float16)
        ws = torch.zeros((2 * width // 64) * 16, dtype=torch.int32, device=dev)

        def fused(i):
            b, sc = weights[i % copies]
            return ops.w4a16_linear(x, b, sc, ws, 2 * width, k, silu_mul=True)

        def unfused(i):
            b, sc = weights[i % copies]
            y = ops.w4a16_linear(x, b, sc, ws, 2 * width, k).view(m, width // 64, 2, 64)
            return torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]

        steps = 200 if m <= 64 else 100
        sec_f, _ = time_graphs(fused, copies, steps, 20)
        sec_u, _ = time_graphs(unfused, copies, steps, 20)
        per = linear_bytes(m, k, 2 * width) - m * width * 2   # half the output bytes
        rows.append(dict(op="gate_up_silu_mul", m=m, k=k, n=2 * width, us=sec_f * 1e6, us_unfused=sec_u * 1e6,
                         gbs=per / sec_f / 1e9, tflops=linear_flops(m, k, 2 * width) / sec_f / 1e12))
        print("gate_up + silu*mul M=%d: fused %.2f us (%.1f GB/s, %.1f TFLOP/s), product then torch ops %.2f us" % (
            m, sec_f * 1e6, per / sec_f / 1e9, linear_flops(m, k, 2 * width) / sec_f / 1e12, sec_u * 1e6),
            file=sys.stderr, flush=True)
        del weights
        torch.cuda.empty_cache()

    # The linears and glue of one Llama-3.1-8B decoder layer around attention, per token batch:
    # the reference's call sequence (q, k, v, rotary, o, residual add, gate, up, silu, multiply, down,
    # residual add: 12 launches, all on this build's kernels) against the fused one (qkv, rotary,
    # o + residual, gate/up with the SiLU epilogue, down + residual: 5 launches).  Attention itself
    # is left out of both.
    from uniql_amd import layout
    hid, nq, nkv, hd, inter = 4096, 32, 8, 128, 14336
    for m in (1, 8):
        copies = copies_for((hid * (nq + 2 * nkv) * hd + hid * hid + 3 * hid * inter) // 2)
        sets = []
        for _ in range(copies):
            w = {name: make_weights(k_, n_, dev, gen) for name, k_, n_ in (
                ("q", hid, nq * hd), ("k", hid, nkv * hd), ("v", hid, nkv * hd), ("o", nq * hd, hid),
                ("gate", hid, inter), ("up", hid, inter), ("down", inter, hid))}
            w["qkv"] = layout.concat_columns([w[n_][0] for n_ in "qkv"], [w[n_][1] for n_ in "qkv"])
            w["gate_up"] = layout.interleave_gate_up(*w["gate"], *w["up"])
            sets.append(w)
        x = torch.randn((m, hid), device=dev, generator=gen).to(torch.float16)
        attn = torch.randn((m, nq * hd), device=dev, generator=gen).to(torch.float16)
        cos = torch.rand((1, m, hd), device=dev, generator=gen).to(torch.float16)
        sin = torch.rand((1, m, hd), device=dev, generator=gen).to(torch.float16)
        idx = torch.arange(hd, device=dev).to(torch.uint8).repeat(nkv, 1)
        wsp = torch.zeros((2 * inter // 64) * 16, dtype=torch.int32, device=dev)

        def lin(w, xin, n_, k_, **kw):
            return ops.w4a16_linear(xin, w[0], w[1], wsp, n_, k_, **kw)

        def unfused(i):
            w = sets[i % copies]
            q = lin(w["q"], x, nq * hd, hid)
            k = lin(w["k"], x, nkv * hd, hid)
            v = lin(w["v"], x, nkv * hd, hid)
            ops.rope_indices_(q.view(1, m, nq, hd), k.view(1, m, nkv, hd), cos, sin, idx)
            o = x + lin(w["o"], attn, hid, nq * hd)
            h = torch.nn.functional.silu(lin(w["gate"], o, inter, hid)) * lin(w["up"], o, inter, hid)
            return o + lin(w["down"], h, hid, inter), v

        def fused(i):
            w = sets[i % copies]
            qkv = lin(w["qkv"], x, (nq + 2 * nkv) * hd, hid)
            q, k = qkv[:, :nq * hd], qkv[:, nq * hd:(nq + nkv) * hd]
            ops.rope_indices_(q.unflatten(1, (nq, hd)).unsqueeze(0), k.unflatten(1, (nkv, hd)).unsqueeze(0), cos, sin, idx)
            o = lin(w["o"], attn, hid, nq * hd, residual=x)
            h = lin(w["gate_up"], o, 2 * inter, hid, silu_mul=True)
            return lin(w["down"], h, hid, inter, residual=o), qkv

        sec_u, _ = time_graphs(unfused, copies, 200, 20)
        sec_f, _ = time_graphs(fused, copies, 200, 20)
        rows.append(dict(op="decoder_layer_linears_and_glue", m=m, us_fused=sec_f * 1e6, us_unfused=sec_u * 1e6,
                         launches_fused=5, launches_unfused=12))
        print("decoder layer (linears + rotary + MLP glue + residuals, no attention) M=%d: 5 launches %.2f us, 12 launches %.2f us"
              % (m, sec_f * 1e6, sec_u * 1e6), file=sys.stderr, flush=True)
        del sets
        torch.cuda.empty_cache()

    # rotary embedding with gathered frequencies, Llama-3.1-8B heads (32 query, 8 key/value)
    for rows_x, d in ((1, 128), (1024, 128), (1024, 108), (4096, 128)):
        qs = [torch.randn((1, rows_x, 32, d), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
        ks = [torch.randn((1, rows_x, 8, d), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
        cos = torch.rand((1, rows_x, 128), device=dev, generator=gen).to(torch.float16)
        sin = torch.rand((1, rows_x, 128), device=dev, generator=gen).to(torch.float16)
        half = torch.arange(d // 2, device=dev)
        idx = torch.cat((half, half + 64)).to(torch.uint8).repeat(8, 1)
        sec, _ = time_graphs(lambda i: ops.rope_indices_(qs[i], ks[i], cos, sin, idx), 4, 200, 20)
        per = rows_x * 40 * d * 2 * 2 + rows_x * 128 * 2 * 2
        rows.append(dict(op="rope_indices", rows=rows_x, head_dim=d, us=sec * 1e6, gbs=per / sec / 1e9))
        print("rope rows=%d head_dim=%d: %.2f us %.1f GB/s" % (rows_x, d, sec * 1e6, per / sec / 1e9),
              file=sys.stderr, flush=True)

    if os.path.dirname(out_path):
        os.makedirs(os.path.dirname(out_path), exist_ok=True)
    with open(out_path, "w") as f:
        json.dump(rows, f, indent=1)


def eager_cost(layer, dev, calls=1000):
    """The module's forward at M = 1 WITHOUT graphs: wall clock per call over `calls` back-to-back calls
    (host checks, ctypes, allocation and launch included; the GPU runs behind the host), beside the
    same kernel's time under graph replay.  The reference measures its TPOT both ways
    (profile_model.py:502-576)."""
    import torch

    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear
    mod = W4A16B16O16Linear(layer.k, layer.n, device=dev)
    mod.weight, mod.scale = layer.weights[0]
    x = layer.x
    for _ in range(300):
        mod(x)
    torch.cuda.synchronize()
    host, total = [], []
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(calls):
            mod(x)
        host.append(time.perf_counter() - t0)   # the host's share: the loop returns before the GPU has finished
        torch.cuda.synchronize()
        total.append(time.perf_counter() - t0)
    sec_k, _ = time_graphs(lambda i: mod(x), 1, 200, 40)
    return {"shape": f"{layer.name} {layer.k}x{layer.n} m=1", "calls": calls, "repeats": 3,
            "module_forward_host_us": round(float(np.median(host)) / calls * 1e6, 2),
            "module_forward_wall_us": round(float(np.median(total)) / calls * 1e6, 2),
            "same_call_graph_replay_us": round(sec_k * 1e6, 2),
            "wall_over_kernel": round(float(np.median(total)) / calls / sec_k, 2)}


def mfma_loop(dev, gen, iters=20000):
    """TFLOP/s of a loop of nothing but v_mfma_f32_32x32x16_f16 on all SIMDs (uniql_diag_mfma_loop),
    on N(0,1) operands and on zeros: the clock the chip settles at depends on the data."""
    import ctypes

    import torch

    from uniql_amd import _capi
    lib = _capi.load()
    out = torch.empty(256 * 256, dtype=torch.float32, device=dev)
    flops = 2.0 * 32 * 32 * 16 * 8 * iters * 1024
    res = {"what": "256 workgroups x 4 waves, 8 independent v_mfma_f32_32x32x16_f16 per loop iteration, no loads"}
    for label, ops_t in (("normal_data", torch.randn(512 * 8, device=dev, generator=gen).to(torch.float16)),
                         ("zeros", torch.zeros(512 * 8, dtype=torch.float16, device=dev))):
        stream = torch.cuda.current_stream().cuda_stream

        def launch():
            _capi.check(lib.uniql_diag_mfma_loop(ops_t.data_ptr(), out.data_ptr(), iters, stream), "uniql_diag_mfma_loop")
        for _ in range(3):
            launch()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(5):
            launch()
        b.record()
        torch.cuda.synchronize()
        sec = a.elapsed_time(b) * 1e-3 / 5
        res[label] = {"tflops": round(flops / sec / 1e12, 1), "frac_of_peak": round(flops / sec / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}
    return res


def embedding_gather(dev, gen):
    """[us, fraction of the HBM peak] of the 4-bit embedding gather: V = 256000, D = 4096, 2048 ids;
    bytes per token: D/2 codes + scale + id + 2 D output."""
    import torch

    from uniql_amd import ops
    v, d, t = 256000, 4096, 2048
    table_ = torch.randint(-2 ** 31, 2 ** 31 - 1, (v, d // 8), dtype=torch.int64, device=dev, generator=gen).to(torch.int32)
    scales = (torch.rand(v, device=dev, generator=gen) * 0.016 + 0.004).to(torch.float16)
    idsets = [torch.randint(0, v, (t,), device=dev, generator=gen) for _ in range(8)]
    sec, _ = time_graphs(lambda i: ops.w4a16_embedding_lookup(idsets[i], table_, scales), 8, 200, 20)
    per = t * (d // 2 + 2 + 8 + 2 * d)
    del table_
    torch.cuda.empty_cache()
    return [round(sec * 1e6, 2), round(per / sec / 1e9 / HBM_PEAK_GBS, 4)]


def secondary(dev, gen):
    """[us, fraction of the HBM peak] of the standalone transform (1024 rows of 8192; read + write)
    and of the rotary kernel (1024 tokens, 32 + 8 heads of 128; q and k read and written, cos/sin read)."""
    import torch

    from uniql_amd import ops
    out = {}
    xs = [torch.randn((1024, 8192), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
    sec, _ = time_graphs(lambda i: ops.hadamard_blockwise(xs[i], 8192 ** -0.5, 8192), 4, 200, 20)
    out["fwht_1024x8192"] = [round(sec * 1e6, 2), round(1024 * 8192 * 4 / sec / 1e9 / HBM_PEAK_GBS, 4)]
    del xs
    rows_x, d = 1024, 128
    qs = [torch.randn((1, rows_x, 32, d), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
    ks = [torch.randn((1, rows_x, 8, d), device=dev, generator=gen).to(torch.float16) for _ in range(4)]
    cos = torch.rand((1, rows_x, 128), device=dev, generator=gen).to(torch.float16)
    sin = torch.rand((1, rows_x, 128), device=dev, generator=gen).to(torch.float16)
    idx = torch.arange(d, device=dev).to(torch.uint8).repeat(8, 1)
    sec, _ = time_graphs(lambda i: ops.rope_indices_(qs[i], ks[i], cos, sin, idx), 4, 200, 20)
    per = rows_x * 40 * d * 2 * 2 + rows_x * 128 * 2 * 2
    out["rope_indices_1024_tokens"] = [round(sec * 1e6, 2), round(per / sec / 1e9 / HBM_PEAK_GBS, 4)]
    return out


# --------------------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--sweep", action="store_true")
    ap.add_argument("--sweep-json", default="bench_sweep.json", help="where --sweep writes its table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--sections", default="all",
                    help="comma-separated parts to run behind the headline step (default all): floor (per-linear product "
                         "and read-floor times, empty kernel, eager cost), decode_sweep, prefill (M = 1024, library GEMM, "
                         "MFMA-only loop), prefill_sweep, models (pruned Llama, Mamba2, embedding), secondary (transform, "
                         "rotary), or none.  Profiler runs name the parts whose kernels they summarise.")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="also launch three plain elementwise copies of 128 MiB (read 128 MiB, write 128 MiB each) "
                         "before the timed region: the known-size kernel a rocprofv3 --pmc run scales its "
                         "FETCH_SIZE / WRITE_SIZE readings by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(1234)

    if args.pmc_calibrate:
        src = torch.ones(64 << 20, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    from uniql_amd import ops
    known = ("floor", "decode_sweep", "prefill", "prefill_sweep", "models", "secondary")
    want = set(known) if args.sections == "all" else set(x for x in args.sections.split(",") if x and x != "none")
    if not want <= set(known):
        print(f"--sections: unknown part(s) {sorted(want - set(known))}; known: {known}", file=sys.stderr)
        sys.exit(2)

    m = 1
    step_bytes = sum(linear_bytes(m, k, n) for _, k, n in LLAMA_DECODE)
    weight_bytes = sum(k * n // 2 for _, k, n in LLAMA_DECODE)
    copies = copies_for(weight_bytes)
    layers = [Layer(name, k, n, m, copies, dev, gen) for name, k, n in LLAMA_DECODE]

    def run_step(i):
        return [layer.run(i) for layer in layers]

    sec_per_step, wall_per_step = time_graphs(run_step, copies, args.steps, args.warmup)
    launches = len(layers)
    gbs = step_bytes / sec_per_step / 1e9
    kernel_us = sec_per_step / launches * 1e6
    traffic, traffic_source = measured_traffic()
    result = {
        "metric": "W4A16 GEMV GB/s at M=1 (Llama-3.1-8B decoder-layer linears)", "value": round(gbs, 2),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 (int4 weights, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "llama31_8b_decode_layer_m1", "linears": [f"{n_}:{k}x{n}" for n_, k, n in LLAMA_DECODE],
                   "m": m, "group_size": 128, "weight_copies_rotated": copies, "launch": "hip_graph",
                   "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "wall_ms_per_step": round(wall_per_step * 1e3, 6)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "w4a16_stream_kernel<RC=1, HAD=0, WAVES, EXT=false> (all four launches of a step; WAVES = 8 for down_proj, 4 for the others)",
                     "launches_per_step": launches,
                     "avg_launch_us": round(kernel_us, 3), "bytes_per_launch": step_bytes // launches},
    }
    # what the memory system and the launch alone allow: the kernel that only reads the same bytes with the
    # same plan (uniql_w4a16_read_floor), per linear, beside the product kernel timed the same way
    floor = {}
    for layer in (layers if "floor" in want else []):
        def product(i, layer=layer):
            return layer.run(i)

        def reads(i, layer=layer):
            b, s = layer.weights[i % copies]
            ops.w4a16_read_floor(b, s, m, layer.n, layer.k)
        sec_k, _ = time_graphs(product, copies, 120, 40)
        sec_f, _ = time_graphs(reads, copies, 120, 40)
        floor[layer.name] = {"kernel_us": round(sec_k * 1e6, 2), "read_floor_us": round(sec_f * 1e6, 2),
                             "gbs": round(linear_bytes(m, layer.k, layer.n) / sec_k / 1e9, 1),
                             "hbm_frac": round(linear_bytes(m, layer.k, layer.n) / sec_k / 1e9 / HBM_PEAK_GBS, 4)}
    if "floor" in want:
        result["config"]["per_linear"] = floor
        result["config"]["read_floor_us_per_step"] = round(sum(v["read_floor_us"] for v in floor.values()), 2)
        # what one node of a replayed graph costs when its kernel does nothing (one workgroup fills 64 floats)
        tiny = torch.zeros(64, device=dev)
        sec_e, _ = time_graphs(lambda i: tiny.fill_(1.0), 1, 400, 40)
        result["config"]["empty_kernel_us_per_graph_node"] = round(sec_e * 1e6, 2)
        result["eager_us_per_call"] = eager_cost(layers[1], dev)
    del layers
    torch.cuda.empty_cache()

    def one_linear(name, k, n, rows, had_block=0, steps=None):
        """[us, fraction of the bounding peak]: HBM for up to 16 rows, dense fp16 MFMA beyond"""
        cps = copies_for(k * n // 2) if rows <= 64 else 2
        layer = Layer(name, k, n, rows, cps, dev, gen, had_block)
        sec, _ = time_graphs(lambda i: layer.run(i), cps, steps or (120 if rows <= 64 else 60), 40)
        del layer
        torch.cuda.empty_cache()
        if rows <= 16:
            return sec, linear_bytes(rows, k, n) / sec / 1e9 / HBM_PEAK_GBS
        return sec, linear_flops(rows, k, n) / sec / 1e12 / MFMA_F16_PEAK_TFLOPS

    def table(shapes, rows_list):
        out = {}
        for rows in rows_list:
            row, tot = {}, 0.0
            for name, k, n, *rest in shapes:
                sec, frac = one_linear(name, k, (n + 255) // 256 * 256, rows, rest[0] if rest else 0)
                row[name] = [round(sec * 1e6, 2), round(frac, 4)]
                tot += sec
            row["sum_us"] = round(tot * 1e6, 2)
            out[f"m{rows}"] = row
        return out

    # the decode sweep's other columns and the model's last layer (quantised like the rest,
    # quantize_model.py:126-143): [us, fraction of the HBM peak]
    if "decode_sweep" in want:
        result["decode_sweep"] = table(LLAMA_DECODE, (2, 4, 8))
        sec, frac = one_linear("lm_head", 4096, 128256, 1, steps=60)
        result["decode_sweep"]["lm_head_llama31_4096x128256_m1"] = [round(sec * 1e6, 2), round(frac, 4)]

    # second half of the metric: the same four linears at M = 1024 through the tiled MFMA kernels,
    # and beside them the library's fp16 GEMM on the same weights dequantised beforehand
    pm = 1024
    per_shape, tot_flops, tot_sec = {}, 0.0, 0.0
    lib_shape, lib_sec = {}, 0.0
    for name, k, n in (LLAMA_DECODE if "prefill" in want else []):
        layer = Layer(name, k, n, pm, 2, dev, gen)
        sec, _ = time_graphs(lambda i: layer.run(i), 2, 100, 40)
        fl = linear_flops(pm, k, n)
        per_shape[name] = {"us": round(sec * 1e6, 2), "tflops": round(fl / sec / 1e12, 1)}
        tot_flops += fl
        tot_sec += sec
        dense = [ops.w4a16_dequant(b, s_, n, k) for b, s_ in layer.weights]   # [k, n] fp16, natural order
        x = layer.x
        ref = torch.matmul(x, dense[0])
        err = (ref.float() - layer.run(0).float()).abs().max().item()
        sec_l, _ = time_graphs(lambda i: torch.matmul(x, dense[i % 2]), 2, 100, 40)
        lib_shape[name] = {"us": round(sec_l * 1e6, 2), "tflops": round(fl / sec_l / 1e12, 1),
                           "ours_over_library": round(sec_l / sec, 3), "max_abs_diff": round(err, 4)}
        lib_sec += sec_l
        del layer, dense
        torch.cuda.empty_cache()
    if "prefill" in want:
        result["prefill_gemm_m1024"] = {
            "metric": "W4A16 prefill GEMM TFLOP/s at M=1024 (same four linears)",
            "value": round(tot_flops / tot_sec / 1e12, 1),
            "unit": "TFLOP/s", "us_per_layer": round(tot_sec * 1e6, 2), "per_linear": per_shape,
            "roofline": {"bound": "mfma", "achieved": round(tot_flops / tot_sec / 1e12, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tot_flops / tot_sec / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                         "kernel": "w4a16_wide_kernel (256 x 256 tiles) for gate_up, w4a16_tile_kernel<MT> (MT = 4, or 2 "
                                   "for the 6144-wide qkv) for the other three"}}
        result["library_fp16_gemm_m1024"] = {
            "what": "torch.matmul(x[1024, k] fp16, w[k, n] fp16) on the same weights dequantised beforehand (its "
                    "dequantisation pass not counted), same graph timing",
            "value": round(tot_flops / lib_sec / 1e12, 1), "unit": "TFLOP/s", "us_per_layer": round(lib_sec * 1e6, 2),
            "frac_of_peak": round(tot_flops / lib_sec / 1e12 / MFMA_F16_PEAK_TFLOPS, 4), "per_linear": lib_shape}
        result["mfma_only_loop"] = mfma_loop(dev, gen)
    if "prefill_sweep" in want:
        # [us, fraction of the dense fp16 MFMA peak]
        result["prefill_sweep"] = table(LLAMA_DECODE, (256, 4096))
    if "models" in want:
        # configs[3]: structured-pruned Llama (widths padded to multiples of 256 as the module pads them);
        # down_proj behind the fused 128-block rotation.  configs[4]: the Mamba2 block.
        result["pruned_llama"] = table(PRUNED, (1, 1024))
        result["mamba2"] = table(MAMBA, (1, 1024))
        result["mamba2"]["embedding_256000x4096_2048ids"] = embedding_gather(dev, gen)
    if "secondary" in want:
        result["secondary_kernels"] = secondary(dev, gen)
        if "models" not in want:
            result["secondary_kernels"]["embedding_256000x4096_2048ids"] = embedding_gather(dev, gen)
    if args.sweep:
        sweep(dev, gen, args.sweep_json)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
