"""uniql_amd: MI355X (gfx950) kernels for UniQL's W4A16 hot path behind the
reference's module API.

    from uniql_amd.quantize.quant_linear_layers import W4A16B16O16Linear, HadLinear
    from uniql_amd.quantize.quant_embedding_layers import W4O16Embedding
    from uniql_amd.quantize.quant_hadamard_layers import Hadamard

`uniql_amd.ops` holds the extension-level functions with the reference's call
shapes; `uniql_amd.install_extension_aliases()` registers them under the
reference's extension module names so that unmodified reference files import
them.
"""
from __future__ import annotations

__version__ = "0.1.0"


def install_extension_aliases() -> None:
    """Makes `import quant_linear_cuda`, `import quant_embedding_cuda` and
    `import fast_hadamard_transform_cuda` resolve to the HIP-backed operators."""
    import sys
    import types

    from . import ops

    lin = types.ModuleType("quant_linear_cuda")
    lin.w4a16o16_gemm = ops.w4a16o16_gemm
    emb = types.ModuleType("quant_embedding_cuda")
    emb.w4a16_embedding_lookup = ops.w4a16_embedding_lookup
    had = types.ModuleType("fast_hadamard_transform_cuda")
    had.fast_hadamard_transform = ops.fast_hadamard_transform
    for n in (12, 20, 28, 40):
        setattr(had, f"fast_hadamard_transform_{n}N", ops.composite_hadamard_variant(n))
    sys.modules.setdefault("quant_linear_cuda", lin)
    sys.modules.setdefault("quant_embedding_cuda", emb)
    sys.modules.setdefault("fast_hadamard_transform_cuda", had)
