"""MI355X ternary linear-layer operators: a thin Python binding over the C-ABI library
`lib/libtllm_ternary.so` (hand-written HIP, gfx950). There is no CPU or PyTorch fallback:
every operator raises if the library is missing or a call is rejected."""
from .ops import (  # noqa: F401
    FileHeader,
    LinearPlan,
    SWIGLU_GATE,
    ModelFile,
    TllmError,
    add,
    copy_to_kv_cache,
    embedding_lookup,
    gemm_kernel,
    gemm_workspace_release,
    gemm_workspace_reserve,
    lib,
    lib_path,
    quantize_absmax_int8,
    read_stream,
    rmsnorm,
    rope,
    silu_mul,
    ternary_gemm,
    ternary_gemm_static,
    ternary_gemv,
    ternary_gemv_int8,
    ternarize_pack,
    write_synthetic_model,
)
