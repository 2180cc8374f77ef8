"""The shared library loads and exports exactly the functions the header declares
(no GPU needed: nothing is launched)."""
import ctypes
import os
import re

import pytest

from uniql_amd import _capi
from uniql_amd.build import LIB_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


HEADERS = ("uniql_amd.h", "uniql_amd_diag.h")


def header_text():
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in HEADERS)
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def header_functions():
    return set(re.findall(r"\b(uniql_[a-z0-9_]+)\s*\(", header_text()))


# C parameter / return types of the headers -> the ctypes type the binding must use
C_TO_CTYPES = {
    "int": ctypes.c_int, "unsigned": ctypes.c_uint, "float": ctypes.c_float, "int64_t": ctypes.c_int64,
    "size_t": ctypes.c_size_t, "const char*": ctypes.c_char_p,
    "unsigned long long*": ctypes.POINTER(ctypes.c_ulonglong), "size_t*": ctypes.POINTER(ctypes.c_size_t),
}


def c_type(decl: str, is_param: bool):
    """`const void* A` / `int64_t lda` / `size_t` -> ctypes type.  Every other pointer is passed as c_void_p."""
    decl = decl.strip()
    if is_param:  # drop the parameter's name
        decl = re.sub(r"\s*\b[A-Za-z_][A-Za-z0-9_]*$", "", decl) if not decl.endswith("*") else decl
    decl = re.sub(r"\s*\*", "*", decl).strip()
    if decl in C_TO_CTYPES:
        return C_TO_CTYPES[decl]
    assert decl.endswith("*"), f"unknown C type {decl!r}"
    return ctypes.c_void_p


def header_prototypes():
    """name -> (restype, [argtypes]) parsed from the declarations of the headers."""
    protos = {}
    for ret, name, params in re.findall(r"([A-Za-z_][A-Za-z0-9_ ]*?\**)\s*\b(uniql_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", header_text()):
        params = params.strip()
        args = [] if params in ("", "void") else [c_type(p, True) for p in params.split(",")]
        protos[name] = (c_type(ret, False), args)
    return protos


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB_PATH):
        from uniql_amd.build import build
        build(verbose=False)
    return _capi.load()


def test_header_and_binding_agree():
    assert header_functions() == set(_capi.SIGNATURES)


def test_binding_signatures_match_the_prototypes():
    """Return type, argument count and every argument's type of the ctypes table against the
    prototypes as the headers spell them."""
    protos = header_prototypes()
    assert set(protos) == set(_capi.SIGNATURES)
    for name, (res, args) in _capi.SIGNATURES.items():
        want_res, want_args = protos[name]
        assert res is want_res, f"{name}: return type {res} != {want_res}"
        assert len(args) == len(want_args), f"{name}: {len(args)} arguments bound, {len(want_args)} declared"
        for i, (got, want) in enumerate(zip(args, want_args)):
            assert got is want, f"{name}: argument {i} bound as {got}, declared as {want}"


def test_headers_compile_as_c_and_cxx(tmp_path):
    """Both headers are plain C99 and C++17 (the boundary a cgo / JNI / pybind binding would include)."""
    import shutil
    import subprocess
    src = '#include "uniql_amd_diag.h"\nint main(void) { return UNIQL_OK + UNIQL_F_FORCE_TILED * 0; }\n'
    for compiler, std, ext in (("gcc", "-std=c99", "c"), ("g++", "-std=c++17", "cpp")):
        if shutil.which(compiler) is None:
            pytest.skip(f"{compiler} not available")
        f = tmp_path / f"t.{ext}"
        f.write_text(src)
        subprocess.run([compiler, std, "-Wall", "-Werror", "-pedantic", "-fsyntax-only", f"-I{os.path.join(ROOT, 'include')}", str(f)],
                       check=True)


def test_every_declared_symbol_is_exported(lib):
    for name in header_functions():
        assert isinstance(getattr(lib, name), ctypes._CFuncPtr)


def test_host_only_entry_points(lib):
    assert lib.uniql_abi_version() == 1
    assert lib.uniql_status_string(0) == b"ok"
    assert b"NULL" in lib.uniql_status_string(-1)
    # streaming kernel: one 64-bit word per output element of a (<= 16 row) slab when K can be
    # split; tiled kernel: one word per output tile (far fewer); the answer covers both
    assert lib.uniql_w4a16_gemm_accum_bytes(1, 4096, 4096) == 4096 * 8
    assert lib.uniql_w4a16_gemm_accum_bytes(100, 4096, 4096) == 16 * 4096 * 8
    assert lib.uniql_w4a16_gemm_accum_bytes(4096, 4096, 4096) == 16 * 4096 * 8
    assert lib.uniql_w4a16_gemm_accum_bytes(1, 4096, 512) == 0
    assert lib.uniql_w4a16_gemm_temp_bytes(2, 4096, 8192, 8192) == 2 * 8192 * 2
    assert lib.uniql_w4a16_gemm_temp_bytes(2, 4096, 8192, 128) == 2 * 8192 * 2
    assert lib.uniql_w4a16_gemm_temp_bytes(2, 4096, 8192, 0) == 0
    import ctypes
    acc, tmp = ctypes.c_size_t(7), ctypes.c_size_t(7)
    ws = lib.uniql_w4a16_linear_workspace
    assert ws(1, 4096, 4096, 4096, 0, 0, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert (acc.value, tmp.value) == (4096 * 8, 0)                      # streaming kernel, K split with atomics
    assert ws(1024, 4096, 4096, 4096, 0, 0, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert (acc.value, tmp.value) == (0, 0)                             # tiled kernel, whole K per workgroup
    # tiled kernel forced to split K four ways with 128-row tiles: a count per tile, a partial tile per split
    forced = (4 << 8) | (4 << 16)
    assert ws(256, 4096, 4096, 4096, 0, forced, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert (acc.value, tmp.value) == (32 * 2 * 8, 4 * 256 * 4096 * 4)
    assert ws(256, 4096, 4096, 4000, 0, forced, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert tmp.value == 256 * 4096 * 2 + 4 * 256 * 4096 * 4             # + the zero-padded copy of the input
    assert ws(1, 4096 + 64, 4096, 4096, 0, 0, ctypes.byref(acc), ctypes.byref(tmp)) == -2
    assert ws(1, 4096, 4096, 4096, 0, 0, None, ctypes.byref(tmp)) == -1
    assert lib.uniql_stream_capture_id(None, None) == -1    # the result pointer is checked before any HIP call
    # the read-floor aid: one dword per wave of the streaming plan (o_proj at one row: 256 workgroups of 4 waves)
    assert lib.uniql_w4a16_read_floor_sink_bytes(1, 4096, 4096, 0) == 256 * 4 * 4
    assert lib.uniql_w4a16_read_floor_sink_bytes(1, 4096 + 64, 4096, 0) == 0
    assert lib.uniql_w4a16_read_floor(None, None, None, 0, 1, 4096, 4096 + 16, 0, None) == -2
    assert lib.uniql_w4a16_read_floor(None, None, None, 0, 1, 4096, 4096, 0, None) == -1


def test_static_entry_uses_the_needs_of_the_kernel_that_takes_the_call(lib):
    """uniql_w4a16_gemm_static sizes its scratch with the same decision as the launch: a prefill that
    the 256 x 256 kernel takes needs none (and passes the limit check whatever the 128-column
    kernel would have asked for), the same shape forced onto the 128-column kernel with K splits
    needs partial tiles beyond the static area and is refused before the pointers are looked at."""
    st = lib.uniql_w4a16_gemm_static
    acc, tmp = ctypes.c_size_t(0), ctypes.c_size_t(0)
    split4_tile128 = (4 << 8) | (4 << 16)     # four K splits, 128-row tiles of the 128-column kernel
    wide = 8 << 16                            # the 256 x 256 kernel
    m, n, k = 1024, 4096, 4096
    assert lib.uniql_w4a16_linear_workspace(m, n, k, k, 0, split4_tile128, ctypes.byref(acc), ctypes.byref(tmp)) == 0
    assert tmp.value == 4 * m * n * 4 > lib.uniql_w4a16_gemm_static_limit(1)
    assert st(None, k, None, None, None, None, 0, m, n, k, k // 128, 0, 1.0, split4_tile128, None) == -7
    assert st(None, k, None, None, None, None, 0, m, n, k, k // 128, 0, 1.0, wide, None) == -1      # no scratch needed: next check
    # per-column scales cannot take the 256 x 256 kernel: the call falls to the 128-column kernel's own plan
    assert st(None, k, None, None, None, None, 0, m, n, k, 1, 0, 1.0, wide, None) == -1
    # the default plan of a long, wide prefill: the 256 x 256 kernel, nothing to clear, nothing to refuse
    assert st(None, 4096, None, None, None, None, 0, 4096, 28672, 4096, 32, 0, 1.0, 0, None) == -1


def test_argument_checks_need_no_gpu(lib):
    """Shape errors are reported before anything touches the device."""
    f = lib.uniql_w4a16_gemm
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 1, 4096 + 64, 4096, 32, 0, 1.0, 0, None) == -2
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 1, 4096, 4096 + 16, 32, 0, 1.0, 0, None) == -2
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 1, 4096, 4096, 7, 0, 1.0, 0, None) == -2
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 1, 4096, 4096, 32, 0, 1.0, 8, None) == -1
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 1, 4096, 4096, 32, 0, 1.0, 0, None) == -1
    assert f(None, 4096, None, None, None, None, 0, None, 0, None, 0, 0, 4096, 4096, 32, 0, 1.0, 0, None) == 0
    g = lib.uniql_w4a16_linear
    args = dict(A=None, lda=4096, k_in=4096, B=None, S=None, bias=None, residual=None, ldr=0, D=None, ldd=4096,
                n_out=4096, epilogue=0,
                workspace=None, workspace_len=0, accum=None, accum_bytes=0, temp=None, temp_bytes=0, m=1, n=4096,
                k=4096, groups=32, had_block=0, had_scale=1.0, flags=0, stream=None)

    def call(**kw):
        return g(*{**args, **kw}.values())

    assert call() == -1                                  # shapes fine, pointers missing
    assert call(k_in=4096 - 128) == -2                   # a whole group of the input missing
    assert call(k_in=4095) == -2                         # not a multiple of 8
    assert call(n_out=4097) == -2
    assert call(epilogue=1, n_out=2049) == -2            # a gated call stores at most n/2 columns
    assert call(epilogue=1, n_out=2048, ldd=2048) == -1
    assert call(epilogue=2) == -1                        # squared ReLU: a known epilogue, pointers missing
    assert call(epilogue=3) == -5
    assert call(ldd=4095) == -2
    assert call(flags=8, ldd=0) == -2                    # transposed: ldd counts rows
    assert call(m=0) == 0
    # the tiled kernel addresses a tile's X rows with 32-bit byte offsets from the tile's first
    # row: a row stride of 2^24 elements or more is refused before anything is enqueued (the
    # pointers are never dereferenced: the shape check comes first)
    fake = ctypes.c_void_p(0x10000)
    assert call(A=fake, B=fake, S=fake, D=fake, m=17, n=128, k=128, k_in=128, groups=1, ldd=128, n_out=128,
                lda=1 << 24) == -2
    # the streaming kernel addresses a 16-row slab of activations with 32-bit byte offsets
    assert call(A=fake, B=fake, S=fake, D=fake, m=2, n=128, k=128, k_in=128, groups=1, ldd=128, n_out=128,
                lda=1 << 27) == -2
    assert lib.uniql_w4a16_linear_temp_bytes(3, 4096, 4096, 4000, 0) == 3 * 4096 * 2
    assert lib.uniql_w4a16_linear_temp_bytes(3, 4096, 4096, 4096, 0) == 0
    r = lib.uniql_rope_indices
    assert r(None, 4096, None, 1024, None, None, 128, None, 1, 4, 4, 1, 32, 8, 128, 128, None) == -1
    assert r(None, 4096, None, 1024, None, None, 128, None, 2, 4, 4, 1, 32, 8, 128, 128, None) == -5
    assert r(None, 4096, None, 1024, None, None, 128, None, 1, 4, 4, 1, 32, 5, 128, 128, None) == -2
    assert r(None, 4096, None, 1024, None, None, 128, None, 1, 5, 4, 1, 32, 8, 128, 128, None) == -2
    assert r(None, 4096, None, 1024, None, None, 128, None, 1, 4, 4, 1, 32, 8, 127, 128, None) == -2
    assert r(None, 4095, None, 1024, None, None, 128, None, 1, 4, 4, 1, 32, 8, 128, 128, None) == -2
    assert r(None, 4096, None, 1024, None, None, 128, None, 1, 0, 4, 1, 32, 8, 128, 128, None) == 0
    assert lib.uniql_w4_embedding_quantize(None, 64, None, None, 10, 60, None) == -2
    assert lib.uniql_w4_embedding_quantize(None, 64, None, None, 10, 64, None) == -1
    assert lib.uniql_w4_embedding_quantize(None, 64, None, None, 0, 64, None) == 0
    assert lib.uniql_fwht(None, None, 4, 96, 96, 1.0, 0, None) == -2
    assert lib.uniql_fwht(None, None, 4, 128, 128, 1.0, 7, None) == -5
    assert lib.uniql_w4_embedding_lookup(None, 5, None, None, None, 10, 12, None) == -2
    assert lib.uniql_w4_embedding_lookup(None, 0, None, None, None, 10, 64, None) == 0
