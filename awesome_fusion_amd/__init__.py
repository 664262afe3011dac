"""MI355X-native bfAintBGemm: bf16 activations x int8/int4 weights, fp32 accumulate, bf16 out.

The product is ``libbfaintb_gemm.so`` (hand-written HIP for gfx950 behind the C ABI declared in
``include/bfaintb_gemm.h``) and the C++ host driver under ``host/``.  This Python package is the
thin ctypes binding tests and the benchmark call through; it holds no arithmetic of its own and
has no CPU fallback: without the built library every call raises.
"""
from .gemm import (  # noqa: F401
    BfaintbError,
    Epilogue,
    PackedHeader,
    load_packed,
    save_packed,
    DECODE,
    PREFILL,
    PREFILL_128,
    PREFILL_256,
    AUTO,
    ACT_NONE,
    ACT_SILU_GATE,
    build_library,
    dequant,
    error_string,
    gemm,
    gemm_prepacked,
    gemm_reference,
    kernel_name,
    lib,
    prefill_tile,
    prepack,
    prepack_bytes,
    prepack_colmajor,
    prepacked_variant,
    prepacked_workspace_bytes,
    library_path,
    probe_read,
    split_k,
    unpack,
    variant,
    workspace_bytes,
    workspace_init,
)
