"""Extension-level operators: the functions the reference's compiled modules
export, with the same positional arguments, backed by the C ABI.

    w4a16o16_gemm           <- quant_linear_cuda          (csrc/linear/quant_linear.cpp:6-24)
    w4a16_embedding_lookup  <- quant_embedding_cuda       (csrc/embedding/quant_embedding.cpp:3-8)
    fast_hadamard_transform <- fast_hadamard_transform_cuda (quantize/hadamard_helpers.py:22-35)

Outputs are allocated with torch.empty on the input's device and kernels are
enqueued on torch's current stream, so calls are valid inside
torch.cuda.graph capture.  Errors surface as RuntimeError.
"""
from __future__ import annotations

import contextlib
import ctypes

import torch

from . import _capi

__all__ = [
    "w4a16o16_gemm", "w4a16_gemm_ex", "w4a16_gemm_static", "w4a16_linear", "prepare_linear", "linear_prepared",
    "w4a16_dequant", "w4a16_embedding_lookup",
    "fast_hadamard_transform", "hadamard_blockwise", "hadamard_composite", "composite_hadamard_variant",
    "w4a16_read_floor", "w4a16_quantize", "w4a16_pack", "w4a16_unpack", "w4_embedding_quantize", "rope_indices_",
]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_GUARD = contextlib.nullcontext()


def _device_guard(device: torch.device):
    """Makes `device` current for the allocations and the launch; free when it already is."""
    return _NO_GUARD if torch.cuda.current_device() == device.index else torch.cuda.device(device)


def _stream_ptr(device: torch.device) -> int:
    """The hipStream_t of torch's current stream on `device` (the raw accessor when this torch
    has it: the public one builds a Stream object on every call)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


# Zero-in / zero-out accumulator words of the split-K exchange, one buffer per
# (device, stream): kernels on one stream run in order, so they can share it; work on
# different streams may overlap and must not.
_accum_cache: dict = {}
# Buffers that were replaced by larger ones stay allocated: a captured graph may still hold
# their address, and memory handed back to the allocator would be reused under it.
_accum_retired: list = []
# Buffers born inside a graph capture, keyed by the capture as well: their zero fill is a node
# of that graph, so they are only known to be zero when that graph replays and serve nothing else.
# They are kept until reset_accumulators() (one buffer per capture that needed one; a capture on
# a stream that already ran an eager call uses that stream's eager buffer instead).
_accum_in_capture: dict = {}


def _capture_id(stream_ptr: int) -> int:
    out = ctypes.c_ulonglong(0)
    _capi.check(_capi.load().uniql_stream_capture_id(stream_ptr, ctypes.byref(out)), "uniql_stream_capture_id")
    return out.value


def _accumulator(device: torch.device, nbytes: int, stream: int | None = None) -> torch.Tensor:
    if stream is None:
        stream = _stream_ptr(device)
    key = (device.index, stream)
    buf = _accum_cache.get(key)
    if buf is not None and buf.numel() * 8 >= nbytes:
        return buf
    words = max(nbytes // 8, 1 << 16)
    capture = _capture_id(stream)
    if capture:
        ckey = (device.index, stream, capture)
        cbuf = _accum_in_capture.get(ckey)
        if cbuf is None or cbuf.numel() * 8 < nbytes:
            if cbuf is not None:
                _accum_retired.append(cbuf)
            # cleared by the library's own kernel, so that what the graph records is a kernel node
            # whatever this torch build's zero fill would have recorded
            cbuf = torch.empty(words, dtype=torch.int64, device=device)
            _capi.check(_capi.load().uniql_clear(cbuf.data_ptr(), words * 8, stream), "uniql_clear")
            _accum_in_capture[ckey] = cbuf
        return cbuf
    if buf is not None:
        _accum_retired.append(buf)
        words = max(words, 2 * buf.numel())  # geometric growth bounds what retirement keeps
    buf = torch.zeros(words, dtype=torch.int64, device=device)
    _accum_cache[key] = buf
    return buf


def reset_accumulators() -> None:
    """Drops the cached accumulator buffers (they are re-created zeroed).  Only needed
    after a kernel was aborted half-way, which can leave non-zero words behind.  Graphs
    captured before the call hold the old buffers' addresses and must be captured again."""
    _accum_cache.clear()
    _accum_retired.clear()
    _accum_in_capture.clear()


_workspace_cache: dict = {}


def _workspace(lib, m: int, n: int, k: int, k_in: int, had_block: int, flags: int):
    """(accum bytes, temp bytes) of one layer call with these flags: a pure function of its
    arguments, asked of the library once per distinct call shape."""
    key = (m, n, k, k_in, had_block, flags)
    hit = _workspace_cache.get(key)
    if hit is not None:
        return hit
    acc, tmp = ctypes.c_size_t(0), ctypes.c_size_t(0)
    _capi.check(lib.uniql_w4a16_linear_workspace(m, n, k, k_in, had_block, flags, ctypes.byref(acc), ctypes.byref(tmp)),
                "uniql_w4a16_linear_workspace")
    if len(_workspace_cache) > 4096:
        _workspace_cache.clear()
    _workspace_cache[key] = (acc.value, tmp.value)
    return acc.value, tmp.value


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor (this package has no CPU path)")


def w4a16_gemm_ex(A: torch.Tensor, B: torch.Tensor, s: torch.Tensor, workspace: torch.Tensor,
                  size_m: int, size_n: int, size_k: int, *, had_block: int = 0,
                  had_scale: float = 1.0, out_f32: bool = False, transpose_out: bool = False,
                  flags: int = 0) -> torch.Tensor:
    """D[m, n] = rotate(A)[m, k] . dequant(B)[k, n].  `had_block` 0 means no rotation.
    transpose_out: the result comes as [n, m8] with m8 = m rounded up to 8 (the reference's
    output_transpose layout, marlin_gemm_kernel.cuh:1023-1026); columns m.. are zero."""
    for t, name in ((A, "A"), (B, "B"), (s, "s"), (workspace, "workspace")):
        _require_gpu(t, name)
    if A.dtype != torch.float16 or s.dtype != torch.float16:
        raise RuntimeError("A and s must be float16")
    if B.dtype != torch.int32 or workspace.dtype != torch.int32:
        raise RuntimeError("B and workspace must be int32")
    if A.dim() != 2 or A.stride(1) != 1:
        raise RuntimeError("A must be 2-D with unit stride along K")
    if A.shape[0] != size_m or A.shape[1] != size_k:
        raise RuntimeError(f"A is {tuple(A.shape)}, expected ({size_m}, {size_k})")
    if not (B.is_contiguous() and s.is_contiguous() and workspace.is_contiguous()):
        raise RuntimeError("B, s and workspace must be contiguous")
    if tuple(B.shape) != (size_k // 16, 2 * size_n):
        raise RuntimeError(f"B is {tuple(B.shape)}, expected ({size_k // 16}, {2 * size_n})")
    if s.dim() != 2 or s.shape[1] != size_n:
        raise RuntimeError(f"s is {tuple(s.shape)}, expected (groups, {size_n})")
    groups = s.shape[0]
    # same test as the reference wrapper (marlin_gemm_kernel.cuh:1008-1010)
    if groups != 1 and (size_k // groups) * groups != size_k:
        raise RuntimeError(f"k={size_k} not compatible with {groups} groups.")
    lib = _capi.load()
    dev = A.device
    out_dtype = torch.float32 if out_f32 else torch.float16
    with _device_guard(dev):
        if transpose_out:
            D = torch.zeros((size_n, (size_m + 7) // 8 * 8), dtype=out_dtype, device=dev)
            flags |= _capi.F_TRANSPOSE_OUT
        else:
            D = torch.empty((size_m, size_n), dtype=out_dtype, device=dev)
        if out_f32:
            flags |= _capi.F_OUT_F32
        need_acc, need_tmp = _workspace(lib, size_m, size_n, size_k, size_k, had_block, flags)
        accum = _accumulator(dev, need_acc) if need_acc else None
        temp = torch.empty(need_tmp, dtype=torch.uint8, device=dev) if need_tmp else None
        lda = A.stride(0) if size_m > 1 else size_k
        code = lib.uniql_w4a16_gemm(
            A.data_ptr(), lda, B.data_ptr(), s.data_ptr(), D.data_ptr(),
            workspace.data_ptr(), workspace.numel(),
            accum.data_ptr() if accum is not None else None, accum.numel() * 8 if accum is not None else 0,
            temp.data_ptr() if temp is not None else None, need_tmp,
            size_m, size_n, size_k, groups, had_block, float(had_scale), flags, _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_gemm")
    return D


def w4a16_gemm_static(A: torch.Tensor, B: torch.Tensor, s: torch.Tensor, workspace: torch.Tensor, out: torch.Tensor,
                      size_m: int, size_n: int, size_k: int, *, had_block: int = 0, had_scale: float = 1.0,
                      flags: int = 0) -> torch.Tensor:
    """uniql_w4a16_gemm_static: the product into the caller's `out` with the library's own static
    scratch memory; neither this wrapper nor the call allocates anything.  Raises when the call's
    plan needs more scratch than the static buffer holds."""
    for t, name in ((A, "A"), (B, "B"), (s, "s"), (workspace, "workspace"), (out, "out")):
        _require_gpu(t, name)
    if A.dtype != torch.float16 or s.dtype != torch.float16 or B.dtype != torch.int32 or workspace.dtype != torch.int32:
        raise RuntimeError("A and s must be float16, B and workspace int32")
    want = torch.float32 if flags & _capi.F_OUT_F32 else torch.float16
    if out.dtype != want or not out.is_contiguous() or tuple(out.shape) != (size_m, size_n):
        raise RuntimeError(f"out must be a contiguous {want} tensor of shape ({size_m}, {size_n})")
    if flags & _capi.F_TRANSPOSE_OUT:
        raise RuntimeError("transposed output is not offered by this wrapper")
    if A.dim() != 2 or A.stride(1) != 1 or tuple(A.shape) != (size_m, size_k):
        raise RuntimeError(f"A must be ({size_m}, {size_k}) with unit stride along K")
    if not (B.is_contiguous() and s.is_contiguous()) or tuple(B.shape) != (size_k // 16, 2 * size_n) or \
            s.dim() != 2 or s.shape[1] != size_n:
        raise RuntimeError("B / s shapes do not match size_k, size_n")
    lib = _capi.load()
    dev = A.device
    with _device_guard(dev):
        code = lib.uniql_w4a16_gemm_static(
            A.data_ptr(), A.stride(0) if size_m > 1 else size_k, B.data_ptr(), s.data_ptr(), out.data_ptr(),
            workspace.data_ptr(), workspace.numel(), size_m, size_n, size_k, s.shape[0], had_block,
            float(had_scale), flags, _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_gemm_static")
    return out


class PreparedLinear:
    """What a layer call needs that does not change from call to call, validated once
    (prepare_linear): the packed tensors, their addresses and sizes, bias, rotation, epilogue.
    The tensors are held so that the addresses stay valid."""
    __slots__ = ("B", "s", "workspace", "bias", "b_ptr", "s_ptr", "ws_ptr", "ws_len", "bias_ptr", "size_n", "size_k",
                 "n_out", "groups", "had_block", "had_scale", "silu_mul", "dev", "needs")


def prepare_linear(B: torch.Tensor, s: torch.Tensor, workspace: torch.Tensor, size_n: int, size_k: int, *,
                   out_features: int | None = None, bias: torch.Tensor | None = None, silu_mul: bool = False,
                   had_block: int = 0, had_scale: float = 1.0) -> PreparedLinear:
    """Every check of w4a16_linear that concerns the layer and not the activations."""
    for t, name in ((B, "B"), (s, "s"), (workspace, "workspace")):
        _require_gpu(t, name)
    if s.dtype != torch.float16:
        raise RuntimeError("x and s must be float16")
    if B.dtype != torch.int32 or workspace.dtype != torch.int32:
        raise RuntimeError("B and workspace must be int32")
    if not (B.is_contiguous() and s.is_contiguous() and workspace.is_contiguous()):
        raise RuntimeError("B, s and workspace must be contiguous")
    if tuple(B.shape) != (size_k // 16, 2 * size_n) or s.dim() != 2 or s.shape[1] != size_n:
        raise RuntimeError("B / s shapes do not match size_k, size_n")
    n_max = size_n // 2 if silu_mul else size_n
    n_out = n_max if out_features is None else int(out_features)
    if not 0 < n_out <= n_max:
        raise RuntimeError(f"out_features={n_out} does not fit the packed width {n_max}")
    if bias is not None:
        _require_gpu(bias, "bias")
        if bias.dtype != torch.float16 or not bias.is_contiguous() or bias.numel() != (2 if silu_mul else 1) * n_out:
            raise RuntimeError("bias must be contiguous float16 with one entry per output column")
    p = PreparedLinear()
    p.B, p.s, p.workspace, p.bias = B, s, workspace, bias
    p.b_ptr, p.s_ptr, p.ws_ptr, p.ws_len = B.data_ptr(), s.data_ptr(), workspace.data_ptr(), workspace.numel()
    p.bias_ptr = bias.data_ptr() if bias is not None else None
    p.size_n, p.size_k, p.n_out, p.groups = int(size_n), int(size_k), n_out, s.shape[0]
    p.had_block, p.had_scale, p.silu_mul = int(had_block), float(had_scale), bool(silu_mul)
    p.dev = B.device
    p.needs = {}   # (m, k_in, flags) -> (accum bytes, temp bytes)
    return p


def linear_prepared(p: PreparedLinear, x: torch.Tensor, *, residual: torch.Tensor | None = None, relu2: bool = False,
                    out_f32: bool = False, out: torch.Tensor | None = None, flags: int = 0) -> torch.Tensor:
    """The per-call half of w4a16_linear: checks on the activations (and residual / out), the
    output's allocation, one call into the library."""
    if not x.is_cuda:
        raise RuntimeError("x must be a GPU tensor (this package has no CPU path)")
    if x.dtype != torch.float16:
        raise RuntimeError("x and s must be float16")
    if x.dim() != 2 or x.stride(1) != 1:
        raise RuntimeError("x must be 2-D with unit stride along K")
    m, k_in = x.shape
    size_k, n_out = p.size_k, p.n_out
    if not (size_k - 128 < k_in <= size_k):
        raise RuntimeError(f"x has {k_in} columns, the packed weights cover {size_k}")
    if p.silu_mul and relu2:
        raise RuntimeError("silu_mul and relu2 are different epilogues: choose one")
    res_ptr, ldr = None, 0
    if residual is not None:
        _require_gpu(residual, "residual")
        if p.silu_mul or relu2:
            raise RuntimeError("a residual cannot be combined with an activation epilogue")
        if residual.dtype != torch.float16 or tuple(residual.shape) != (m, n_out) or residual.stride(1) != 1:
            raise RuntimeError("residual must be float16 [m, out_features] with unit inner stride")
        res_ptr, ldr = residual.data_ptr(), (residual.stride(0) if m > 1 else n_out)
    x_ptr = x.data_ptr()
    if k_in % 8 or (m > 1 and x.stride(0) % 8) or x_ptr % 16:
        # rare: rows that cannot be read in 16-byte pieces are copied (and padded) here
        x = torch.nn.functional.pad(x, (0, size_k - k_in))
        k_in = size_k
        x_ptr = x.data_ptr()
    lib = _capi.load()
    dev = x.device
    out_dtype = torch.float32 if out_f32 else torch.float16
    with _device_guard(dev):
        if out is None:
            out = torch.empty((m, n_out), dtype=out_dtype, device=dev)
        elif out.dtype != out_dtype or tuple(out.shape) != (m, n_out) or out.stride(1) != 1 or out.device != dev:
            raise RuntimeError("out must be a [m, out_features] view with unit inner stride on x's device")
        if m == 0:
            return out
        if out_f32:
            flags |= _capi.F_OUT_F32
        key = (m, k_in, flags)
        need = p.needs.get(key)
        if need is None:
            need = p.needs[key] = _workspace(lib, m, p.size_n, size_k, k_in, p.had_block, flags)
        need_acc, need_tmp = need
        stream = _stream_ptr(dev)
        accum = _accumulator(dev, need_acc, stream) if need_acc else None
        temp = torch.empty(need_tmp, dtype=torch.uint8, device=dev) if need_tmp else None
        lda = x.stride(0) if m > 1 else max(k_in + (-k_in) % 8, 8)
        ldd = out.stride(0) if m > 1 else n_out
        code = lib.uniql_w4a16_linear(
            x_ptr, lda, k_in, p.b_ptr, p.s_ptr, p.bias_ptr, res_ptr, ldr,
            out.data_ptr(), ldd, n_out,
            _capi.EPI_SILU_MUL if p.silu_mul else (_capi.EPI_RELU2 if relu2 else _capi.EPI_NONE),
            p.ws_ptr, p.ws_len,
            accum.data_ptr() if accum is not None else None, accum.numel() * 8 if accum is not None else 0,
            temp.data_ptr() if temp is not None else None, need_tmp,
            m, p.size_n, size_k, p.groups, p.had_block, p.had_scale, flags, stream)
    if code:
        _capi.check(code, "uniql_w4a16_linear")
    return out


def w4a16_linear(x: torch.Tensor, B: torch.Tensor, s: torch.Tensor, workspace: torch.Tensor, size_n: int,
                 size_k: int, *, out_features: int | None = None, bias: torch.Tensor | None = None,
                 residual: torch.Tensor | None = None, silu_mul: bool = False, relu2: bool = False,
                 had_block: int = 0,
                 had_scale: float = 1.0, out_f32: bool = False, out: torch.Tensor | None = None,
                 flags: int = 0) -> torch.Tensor:
    """The layer's whole forward in one call (uniql_w4a16_linear): x [m, in_features] with
    in_features <= size_k (the kernel pads), product with the packed weights, only the first
    `out_features` columns stored, `bias` and then `residual` ([m, out_features], the decoder
    layer's `residual + layer(x)`) added with the reference's roundings.  With
    `silu_mul` the packed tensors hold a gate and an up projection interleaved in 64-column
    blocks (layout.interleave_gate_up) and the result is silu(gate) * up, [m, out_features].
    With `relu2` the result is relu(y)^2 of the (biased) output y, the un-gated MLP front of the
    squared-ReLU models.
    `out`: optional destination, a 2-D view with unit inner stride (for example a column range
    of a larger buffer).
    A caller that runs the same layer again and again validates it once with prepare_linear and
    calls linear_prepared (the module classes do): the checks on the packed tensors are about a
    third of this call's host time."""
    _require_gpu(x, "x")
    p = prepare_linear(B, s, workspace, size_n, size_k, out_features=out_features, bias=bias, silu_mul=silu_mul,
                       had_block=had_block, had_scale=had_scale)
    return linear_prepared(p, x, residual=residual, relu2=relu2, out_f32=out_f32, out=out, flags=flags)


def w4a16o16_gemm(A, B, s, workspace, size_m, size_n, size_k, output_transpose=False,
                  thread_k=-1, thread_n=-1, sms=-1, max_par=8):
    """Same call as the reference extension.  thread_k / thread_n / sms choose
    CUDA tile shapes there and are accepted and ignored; max_par only sizes the
    reference's lock array, the same check is applied to `workspace`."""
    if workspace.numel() < size_n // 128 * max_par:
        raise RuntimeError(f"workspace must be of size at least {size_n // 128 * max_par}.")
    return w4a16_gemm_ex(A, B, s, workspace, int(size_m), int(size_n), int(size_k),
                         transpose_out=bool(output_transpose))


def w4a16_dequant(B: torch.Tensor, s: torch.Tensor, size_n: int, size_k: int, want_codes: bool = False):
    """Natural-order dequantised weights fp16 [k, n] (and the raw codes uint8 [k, n])."""
    _require_gpu(B, "B")
    _require_gpu(s, "s")
    if B.dtype != torch.int32 or s.dtype != torch.float16 or not (B.is_contiguous() and s.is_contiguous()):
        raise RuntimeError("B must be contiguous int32 and s contiguous float16")
    if tuple(B.shape) != (size_k // 16, 2 * size_n) or s.dim() != 2 or s.shape[1] != size_n:
        raise RuntimeError("B / s shapes do not match size_k, size_n")
    lib = _capi.load()
    dev = B.device
    with _device_guard(dev):
        W = torch.empty((size_k, size_n), dtype=torch.float16, device=dev)
        codes = torch.empty((size_k, size_n), dtype=torch.uint8, device=dev) if want_codes else None
        code = lib.uniql_w4a16_dequant(B.data_ptr(), s.data_ptr(), W.data_ptr(),
                                       codes.data_ptr() if want_codes else None,
                                       size_n, size_k, s.shape[0], _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_dequant")
    return (W, codes) if want_codes else W


def w4a16_read_floor(B: torch.Tensor, s: torch.Tensor, size_m: int, size_n: int, size_k: int, flags: int = 0) -> None:
    """Measurement aid: enqueues the kernel that only reads what the streaming kernel reads for
    this shape (uniql_w4a16_read_floor), with the same plan.  Returns nothing."""
    _require_gpu(B, "B")
    _require_gpu(s, "s")
    if B.dtype != torch.int32 or s.dtype != torch.float16 or not (B.is_contiguous() and s.is_contiguous()):
        raise RuntimeError("B must be contiguous int32 and s contiguous float16")
    if tuple(B.shape) != (size_k // 16, 2 * size_n) or tuple(s.shape) != (size_k // 128, size_n):
        raise RuntimeError("B / s shapes do not match size_k, size_n (group-128 scales)")
    lib = _capi.load()
    dev = B.device
    with _device_guard(dev):
        need = lib.uniql_w4a16_read_floor_sink_bytes(size_m, size_n, size_k, flags)
        sink = torch.empty(max(need, 4), dtype=torch.uint8, device=dev)
        code = lib.uniql_w4a16_read_floor(B.data_ptr(), s.data_ptr(), sink.data_ptr(), sink.numel(), size_m, size_n,
                                          size_k, flags, _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_read_floor")


def w4a16_quantize(weight: torch.Tensor, given_scale: torch.Tensor | None = None, pad_out: int = 0):
    """Group-128 quantisation of an nn.Linear weight [out_features, in_features] (fp16, on the
    GPU) into (packed int32 [k_pad/16, 2 n_pad], permuted scale fp16 [k_pad/128, n_pad]), with the
    host arithmetic of the reference's from_fp16 / w4a16_quantize bit for bit.  given_scale:
    natural-order [k_pad/128, out_features] scales of already fake-quantised weights (GPTQ)."""
    _require_gpu(weight, "weight")
    if weight.dtype != torch.float16 or weight.dim() != 2 or weight.stride(1) != 1:
        raise RuntimeError("weight must be float16 [out_features, in_features] with unit inner stride")
    out_features, in_features = weight.shape
    k_pad = (in_features + 127) // 128 * 128
    n_pad = out_features + pad_out
    dev = weight.device
    if given_scale is not None:
        _require_gpu(given_scale, "given_scale")
        if given_scale.dtype != torch.float16 or tuple(given_scale.shape) != (k_pad // 128, out_features) \
                or not given_scale.is_contiguous():
            raise RuntimeError("given_scale must be contiguous float16 [k_pad/128, out_features]")
    lib = _capi.load()
    with _device_guard(dev):
        B = torch.empty((k_pad // 16, 2 * n_pad), dtype=torch.int32, device=dev)
        S = torch.empty((k_pad // 128, n_pad), dtype=torch.float16, device=dev)
        code = lib.uniql_w4a16_quantize(weight.data_ptr(), weight.stride(0),
                                        given_scale.data_ptr() if given_scale is not None else None,
                                        B.data_ptr(), S.data_ptr(), out_features, in_features, n_pad, k_pad,
                                        _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_quantize")
    return B, S


def w4a16_pack(codes: torch.Tensor, scales: torch.Tensor, pad_out: int = 0):
    """codes uint8 [k, n] and natural-order scales fp16 [k/128, n] -> (packed, permuted scale);
    the inverse of w4a16_unpack."""
    _require_gpu(codes, "codes")
    _require_gpu(scales, "scales")
    if codes.dtype != torch.uint8 or scales.dtype != torch.float16 or codes.dim() != 2:
        raise RuntimeError("codes must be uint8 [k, n] and scales float16 [k/128, n]")
    k, n = codes.shape
    if tuple(scales.shape) != (k // 128, n):
        raise RuntimeError("scales must be [k/128, n]")
    codes, scales = codes.contiguous(), scales.contiguous()
    n_pad = n + pad_out
    dev = codes.device
    lib = _capi.load()
    with _device_guard(dev):
        B = torch.empty((k // 16, 2 * n_pad), dtype=torch.int32, device=dev)
        S = torch.empty((k // 128, n_pad), dtype=torch.float16, device=dev)
        code = lib.uniql_w4a16_pack(codes.data_ptr(), scales.data_ptr(), B.data_ptr(), S.data_ptr(), n, k, n_pad,
                                    _stream_ptr(dev))
    _capi.check(code, "uniql_w4a16_pack")
    return B, S


def w4a16_unpack(B: torch.Tensor, s: torch.Tensor, size_n: int, size_k: int):
    """(codes uint8 [k, n], natural-order scales fp16 [k/128, n]) of a packed group-128 layer:
    what the reference's slicing code gets from unpack_w4a16_permute_weights and
    w4a16_unpermute_scales (quantize_helpers.py:244-328) on the CPU."""
    _, codes = w4a16_dequant(B, s, size_n, size_k, want_codes=True)
    n = torch.arange(size_n, device=B.device)
    pos = (n & ~63) + 8 * (n & 7) + ((n & 63) >> 3)
    return codes, s[:, pos].contiguous()


def w4a16_embedding_lookup(input: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """out[..., :] = (code - 8) * scale[id].  Checks follow quant_embedding_kernel.cuh:121-134."""
    if weight.dim() != 2:
        raise RuntimeError("weight must be 2-D")
    _require_gpu(weight, "weight")
    if weight.dtype != torch.int32:
        raise RuntimeError("weight's dtype must be int32")
    vocab, words = weight.shape
    dim = words * 8
    if scale.dim() != 1:
        raise RuntimeError("scale must be 1-D")
    _require_gpu(scale, "scale")
    if scale.dtype != torch.float16:
        raise RuntimeError("scale's dtype must be float16")
    if scale.numel() != vocab:
        raise RuntimeError("scale must have one entry per vocabulary row")
    if input.dim() not in (1, 2):
        raise RuntimeError("input must be a 1D or 2D tensor")
    _require_gpu(input, "input")
    if input.dtype != torch.int64:
        raise RuntimeError("input's dtype must be int64")
    lib = _capi.load()
    dev = input.device
    ids = input.contiguous()
    weight_c = weight.detach()
    if not weight_c.is_contiguous() or not scale.is_contiguous():
        raise RuntimeError("weight and scale must be contiguous")
    with _device_guard(dev):
        out = torch.empty((*ids.shape, dim), dtype=torch.float16, device=dev)
        code = lib.uniql_w4_embedding_lookup(ids.data_ptr(), ids.numel(), weight_c.data_ptr(), scale.data_ptr(),
                                             out.data_ptr(), vocab, dim, _stream_ptr(dev))
    _capi.check(code, "uniql_w4_embedding_lookup")
    return out


def w4_embedding_quantize(weight: torch.Tensor):
    """fp16 table [vocab, dim] on the GPU -> (packed int32 [vocab, dim/8], scales fp16 [vocab]) with the
    arithmetic of W4O16Embedding.from_fp16 (quant_embedding_layers.py:26-48) bit for bit."""
    _require_gpu(weight, "weight")
    if weight.dtype != torch.float16 or weight.dim() != 2 or weight.stride(1) != 1:
        raise RuntimeError("weight must be float16 [vocab, dim] with unit inner stride")
    vocab, dim = weight.shape
    if dim % 8 or weight.stride(0) % 8 or weight.data_ptr() % 16:
        raise RuntimeError("embedding_dim and the row stride must be multiples of 8")
    lib = _capi.load()
    dev = weight.device
    with _device_guard(dev):
        packed = torch.empty((vocab, dim // 8), dtype=torch.int32, device=dev)
        scales = torch.empty(vocab, dtype=torch.float16, device=dev)
        code = lib.uniql_w4_embedding_quantize(weight.data_ptr(), weight.stride(0) if vocab > 1 else dim,
                                               packed.data_ptr(), scales.data_ptr(), vocab, dim, _stream_ptr(dev))
    _capi.check(code, "uniql_w4_embedding_quantize")
    return packed, scales


def rope_indices_(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                  indices: torch.Tensor) -> None:
    """In-place rotary embedding with gathered frequencies on token-major tensors:
    q [batch, seq, n_q_heads, d], k [batch, seq, n_kv_heads, d] (last two axes contiguous, one row
    stride over batch and seq), cos / sin [1 or batch, seq, D], indices [n_kv_heads, d]
    (uint8, int32 or int64)."""
    for t, name in ((q, "q"), (k, "k"), (cos, "cos"), (sin, "sin"), (indices, "indices")):
        _require_gpu(t, name)
    if not (q.dtype == k.dtype == cos.dtype == sin.dtype == torch.float16):
        raise RuntimeError("q, k, cos and sin must be float16")
    if q.dim() != 4 or k.dim() != 4 or cos.dim() != 3 or sin.shape != cos.shape:
        raise RuntimeError("expected q, k [batch, seq, heads, d] and cos, sin [1 or batch, seq, D]")
    batch, seq, n_qh, d = q.shape
    n_kh = k.shape[2]
    if k.shape[0] != batch or k.shape[1] != seq or k.shape[3] != d:
        raise RuntimeError("q and k disagree on batch, sequence length or head width")
    if tuple(indices.shape) != (n_kh, d):
        raise RuntimeError(f"indices must be [{n_kh}, {d}]")
    index_bytes = {torch.uint8: 1, torch.int32: 4, torch.int64: 8}.get(indices.dtype)
    if index_bytes is None:
        raise RuntimeError("indices must be uint8, int32 or int64")
    if cos.shape[0] not in (1, batch) or cos.shape[1] != seq:
        raise RuntimeError("cos / sin must cover [1 or batch, seq]")

    def token_major(t, heads):
        ok = t.stride(3) == 1 and t.stride(2) == d and (batch == 1 or t.stride(0) == seq * t.stride(1))
        if not ok:
            raise RuntimeError("q / k must be token-major with contiguous heads (use .contiguous())")
        return t.stride(1) if seq > 1 else (t.stride(0) if batch > 1 else heads * d)

    q_stride, k_stride = token_major(q, n_qh), token_major(k, n_kh)
    if not (cos.is_contiguous() and sin.is_contiguous() and indices.is_contiguous()):
        raise RuntimeError("cos, sin and indices must be contiguous")
    lib = _capi.load()
    dev = q.device
    with _device_guard(dev):
        code = lib.uniql_rope_indices(q.data_ptr(), q_stride, k.data_ptr(), k_stride, cos.data_ptr(), sin.data_ptr(),
                                      cos.shape[2], indices.data_ptr(), index_bytes, batch * seq, seq, cos.shape[0],
                                      n_qh, n_kh, d, cos.shape[2], _stream_ptr(dev))
    _capi.check(code, "uniql_rope_indices")


def hadamard_blockwise(x: torch.Tensor, scale: float, block: int | None = None) -> torch.Tensor:
    """(x . H_block) * scale on consecutive block-wide pieces of the last axis; new tensor."""
    _require_gpu(x, "x")
    dim = x.shape[-1]
    block = dim if block is None else block
    dtypes = {torch.float16: _capi.DT_F16, torch.bfloat16: _capi.DT_BF16, torch.float32: _capi.DT_F32}
    if x.dtype not in dtypes:
        raise RuntimeError(f"hadamard transform supports float16 / bfloat16 / float32, got {x.dtype}")
    lib = _capi.load()
    xc = x.contiguous()
    dev = x.device
    with _device_guard(dev):
        y = torch.empty_like(xc)
        rows = xc.numel() // dim if dim else 0
        code = lib.uniql_fwht(xc.data_ptr(), y.data_ptr(), rows, dim, block, float(scale),
                              dtypes[x.dtype], _stream_ptr(dev))
    _capi.check(code, "uniql_fwht")
    return y


def fast_hadamard_transform(x: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Power-of-two Walsh-Hadamard transform along the last axis, times scale."""
    dim = x.shape[-1]
    if dim & (dim - 1):
        raise RuntimeError(f"fast_hadamard_transform needs a power-of-two width, got {dim}")
    return hadamard_blockwise(x, scale, dim)


def hadamard_composite(x: torch.Tensor, scale: float, base: int) -> torch.Tensor:
    """(x . (H_base (x) H_P)) * scale along the last axis of width base * P, P a power of two
    (uniql_fwht_composite); new tensor."""
    _require_gpu(x, "x")
    dim = x.shape[-1]
    dtypes = {torch.float16: _capi.DT_F16, torch.bfloat16: _capi.DT_BF16, torch.float32: _capi.DT_F32}
    if x.dtype not in dtypes:
        raise RuntimeError(f"hadamard transform supports float16 / bfloat16 / float32, got {x.dtype}")
    lib = _capi.load()
    xc = x.contiguous()
    dev = x.device
    with _device_guard(dev):
        y = torch.empty_like(xc)
        rows = xc.numel() // dim if dim else 0
        code = lib.uniql_fwht_composite(xc.data_ptr(), y.data_ptr(), rows, dim, base, float(scale),
                                        dtypes[x.dtype], _stream_ptr(dev))
    _capi.check(code, "uniql_fwht_composite")
    return y


class UnpinnedHadamardWarning(UserWarning):
    """The 12N / 20N / 28N / 40N transforms use this library's own base matrices."""


_composite_warned: set = set()


def _composite_notice(base: int) -> None:
    """The reference takes its 12 x 12, 20 x 20, 28 x 28 and 40 x 40 base matrices from a third-party
    extension that is not part of its tree (quantize/hadamard_helpers.py:20-31), so the ones used
    here (Sloane's 12, Paley 20 and 28, a doubled 20) are valid Hadamard matrices but not known
    to be the same ones.  A model whose weights were rotated offline by the reference at such a
    width would get a DIFFERENT online rotation here: finite, wrong outputs with no other sign.
    Hence a warning on the first use of every base, and UNIQL_AMD_COMPOSITE_HADAMARD=error to
    refuse instead (=quiet silences it for models rotated with this library on both sides)."""
    import os
    mode = os.environ.get("UNIQL_AMD_COMPOSITE_HADAMARD", "warn").lower()
    if mode == "error":
        raise NotImplementedError(
            f"fast_hadamard_transform_{base}N: base matrices not pinned to the reference's (UNIQL_AMD_COMPOSITE_HADAMARD=error)")
    if mode == "quiet" or base in _composite_warned:
        return
    _composite_warned.add(base)
    import warnings
    warnings.warn(
        f"fast_hadamard_transform_{base}N uses this library's own {base} x {base} Hadamard matrix, which is not known to "
        "equal the reference's: only use it where BOTH sides of a rotation (offline weights and online "
        "activations) come from this library.  UNIQL_AMD_COMPOSITE_HADAMARD=quiet silences this, =error refuses.",
        UnpinnedHadamardWarning, stacklevel=3)


def composite_hadamard_variant(base: int):
    """The transform fast_hadamard_transform_{base}N(x, scale) of the reference's extension, for widths
    base * 2^k (quantize/hadamard_helpers.py:20-31).  See _composite_notice for what is not pinned."""
    def _fn(x, scale=1.0):
        _composite_notice(base)
        return hadamard_composite(x, scale, base)
    _fn.__name__ = f"fast_hadamard_transform_{base}N"
    return _fn
