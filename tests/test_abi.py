"""Host-only checks of the drop-in boundary: every symbol include/tllm_ternary.h declares
is exported, the argument validation rejects bad calls without touching a GPU, and the
C++ interface compiles for the reference's call shapes."""
import ctypes as C
import os
import re
import subprocess

import pytest

import ternary_llm_amd as tl
from ternary_llm_amd import ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_exported():
    text = open(os.path.join(ROOT, "include", "tllm_ternary.h")).read()
    declared = set(re.findall(r"\b(tllm_[a-z0-9_]+)\s*\(", text))
    assert declared == set(ops.ABI_SYMBOLS)
    L = tl.lib()
    for name in declared:
        assert hasattr(L, name), name
    assert L.tllm_abi_version() == 1
    text = open(os.path.join(ROOT, "include", "tllm_model_file.h")).read()
    declared = set(re.findall(r"\b(tllm_[a-z0-9_]+)\s*\(", text))
    assert declared == set(ops.FILE_ABI_SYMBOLS)
    for name in declared:
        assert hasattr(L, name), name


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(ops, "_lib", None)
    monkeypatch.setattr(ops, "_LIB_PATH", "/nonexistent/libtllm_ternary.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.lib()


def _gemv(L, nz=0x1000, sg=0x2000, sc=0x3000, x=0x4000, y=0x5000, rows=4, cols=256, g=128):
    return L.tllm_ternary_gemv_f16(nz, sg, sc, x, y, rows, cols, g, None)


def test_validation_codes():
    L = tl.lib()
    assert _gemv(L, nz=None) == -1 and _gemv(L, y=None) == -1
    assert _gemv(L, rows=0) == -2 and _gemv(L, cols=0) == -2 and _gemv(L, cols=250) == -2
    assert _gemv(L, g=0) == -3 and _gemv(L, g=48) == -3
    assert _gemv(L, cols=160, g=128) == -3          # cols % group != 0: rejected, not truncated
    assert _gemv(L, x=0x4000, y=0x4010) == -5       # output inside the input
    assert _gemv(L, nz=0x1004) == -7 and _gemv(L, x=0x4002) == -7 and _gemv(L, y=0x5001) == -7
    assert L.tllm_ternary_gemm_f16(0x4000, 0x1000, 0x2000, 0x3000, 0x9000, 0, 4, 256, 128, None) == -2
    assert L.tllm_quantize_absmax_i8(None, 0x10, 0x20, 4, None) == -1
    assert L.tllm_quantize_absmax_i8(0x10, 0x20, 0x40, 0, None) == -2
    assert L.tllm_ternary_gemv_i8(0x1000, 0x2000, 0x3000, None, 1.0, 0x5000, 4, 256, 128, None) == -1
    assert L.tllm_ternary_gemv_i8_dscale(0x1000, 0x2000, 0x3000, 0x4000, None, 0x5000, 4, 256, 128, None) == -1
    assert L.tllm_rmsnorm_f16(None, 0x20, 0x30, None, None, 1, 8, 1e-5, None) == -1
    assert L.tllm_rmsnorm_f16(0x10, 0x20, 0x30, None, 0x40, 1, 8, 1e-5, None) == -1   # residual_out without residual
    assert L.tllm_rmsnorm_f16(0x10, 0x20, 0x30, None, None, 0, 8, 1e-5, None) == -2
    assert L.tllm_rmsnorm_f16(0x10, 0x20, 0x30, None, None, 1 << 20, 1 << 12, 1e-5, None) == -4
    assert L.tllm_silu_mul_f16(0x10, None, 0x30, 4, None) == -1
    assert L.tllm_silu_mul_f16(0x10, 0x20, 0x30, 0, None) == -2
    assert L.tllm_add_f16(0x10, None, 0x30, 4, None) == -1 and L.tllm_add_f16(0x10, 0x20, 0x30, 0, None) == -2
    assert L.tllm_rope_f16(None, 0x20, 1, 1, 8, 2, 64, 0, 10000.0, None) == -1
    assert L.tllm_rope_f16(0x10, 0x20, 1, 1, 8, 2, 63, 0, 10000.0, None) == -2      # odd head_dim
    assert L.tllm_rope_f16(0x10, 0x20, 1, 1, 8, 2, 64, -1, 10000.0, None) == -2     # negative position
    assert L.tllm_rope_f16(0x10, 0x20, 1, 1, 8, 2, 64, 0, 0.0, None) == -2          # theta must be positive
    assert L.tllm_rope_f16(0x12, 0x20, 1, 1, 8, 2, 64, 0, 10000.0, None) == -7      # pairs are read as 4-byte words
    assert L.tllm_embedding_lookup_f16(0x10, None, 0x30, 1, 8, None) == -1
    assert L.tllm_embedding_lookup_f16(0x10, 0x20, 0x30, 0, 8, None) == -2
    assert L.tllm_copy_to_kv_cache_f16(0x10, 0x20, None, 0x40, 1, 2, 64, 1, 0, 16, None) == -1
    assert L.tllm_copy_to_kv_cache_f16(0x10, 0x20, 0x30, 0x40, 1, 2, 64, 0, 0, 16, None) == -2
    assert L.tllm_copy_to_kv_cache_f16(0x10, 0x20, 0x30, 0x40, 1, 2, 64, 1, -1, 16, None) == -2
    h = C.c_void_p(0)
    assert L.tllm_linear_plan_create(C.byref(h), None, 1, 128) == -1
    arr = (ops._Problem * 1)(ops._Problem(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 4, 256, 17, 0))
    assert L.tllm_linear_plan_create(C.byref(h), arr, 1, 128) == -6   # batch > TLLM_MAX_PLAN_BATCH
    assert L.tllm_linear_plan_create(C.byref(h), arr, 0, 128) == -6
    assert L.tllm_linear_plan_create(C.byref(h), arr, 1, 64) == -3
    # SwiGLU pairs: the flagged gate needs an up problem right after it, same shape and input, batch 1
    P, GATE = ops._Problem, ops.SWIGLU_GATE
    gate = P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 1, GATE)
    for bad in ([gate],                                                             # nothing follows
                [gate, P(0x1000, 0x2000, 0x3000, 0x4000, 0, 32, 2048, 1, 0)],         # other shape
                [gate, P(0x1000, 0x2000, 0x3000, 0x5000, 0, 64, 2048, 1, 0)],         # other input
                [gate, P(0x1000, 0x2000, 0x3000, 0x4000, 0, 64, 2048, 1, GATE)],      # up flagged too
                [P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 2, GATE),
                 P(0x1000, 0x2000, 0x3000, 0x4000, 0, 64, 2048, 2, 0)],               # batch 2
                [P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 1, 4)],          # unknown flag
                [P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 2, ops.QUANTIZE_INPUT)]):  # quantised input: one row only
        arr = (P * len(bad))(*bad)
        assert L.tllm_linear_plan_create(C.byref(h), arr, len(bad), 128) == -6
    # RMSNorm prologue: batch 1, cols <= 16384, aligned weights, same weights on both halves of a pair
    def normed(problems, norms, eps=1e-5):
        arr = (P * len(problems))(*problems)
        ptrs = (C.c_void_p * len(problems))(*norms)
        return L.tllm_linear_plan_create_normed(C.byref(h), arr, ptrs, eps, len(problems), 128)
    one = P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 1, 0)
    assert L.tllm_linear_plan_create_normed(C.byref(h), (P * 1)(one), None, 1e-5, 1, 128) == -1
    assert normed([P(0x1000, 0x2000, 0x3000, 0x4000, 0x9000, 64, 2048, 2, 0)], [0x7000]) == -6
    assert normed([P(0x1000, 0x2000, 0x3000, 0x40000, 0x90000, 64, 32768, 1, 0)], [0x7000]) == -6
    assert normed([one], [0x7002]) == -7
    assert normed([one], [0x7000], eps=-1.0) == -6
    up_ = P(0x1000, 0x2000, 0x3000, 0x4000, 0, 64, 2048, 1, 0)
    assert normed([gate, up_], [0x7000, 0x8000]) == -6
    assert normed([gate, up_], [0x7000, None]) == -6
    # grouped GEMMs: host arrays of device pointers, 1 to TLLM_MAX_GEMM_GROUP matrices, outputs apart, groups of 128
    def grouped(nz=(0x10000,), sg=(0x20000,), sc=(0x30000,), out=(0x90000,), n=(256,), count=None, M=32, K=256, g=128, A=0x4000):
        k = len(n)
        ptrs = lambda v: (C.c_void_p * max(1, len(v)))(*v)
        return L.tllm_ternary_gemm_group_f16(A, ptrs(nz), ptrs(sg), ptrs(sc), ptrs(out), (C.c_int * max(1, k))(*n),
                                             k if count is None else count, M, K, g, None)
    assert L.tllm_ternary_gemm_group_f16(0x4000, None, None, None, None, None, 1, 32, 256, 128, None) == -1
    assert grouped(count=0) == -2 and grouped(count=5) == -2 and grouped(M=0) == -2
    assert grouped(nz=(None,)) == -1 and grouped(A=None) == -1
    assert grouped(g=64) == -3 and grouped(K=128) == -2                               # K = 128: not a shape of the row-split kernel
    assert grouped(nz=(0x10000, 0x10000), sg=(0x20000, 0x20000), sc=(0x30000, 0x30000), out=(0x90000, 0x90100), n=(256, 256)) == -5
    assert grouped(nz=(0x10004,)) == -7                                                 # mask planes in 16-byte pieces
    assert L.tllm_linear_plan_launch(None, None) == -6
    for code in range(-7, 1):
        assert L.tllm_error_string(code)
    with pytest.raises(tl.TllmError):
        ops.check(-2)


def test_cpp_dropin_call_shapes(tmp_path):
    exe = tmp_path / "dropin_calls"
    libdir = os.path.dirname(tl.lib_path())
    # a plain host C++ translation unit, as the reference's src/transformer.cpp is
    cmd = ["g++", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include",
           "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "dropin_calls.cpp"),
           "-L", libdir, "-ltllm_ternary", f"-Wl,-rpath,{libdir}", "-o", str(exe)]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "rejected=13" in out.stdout


def test_tuning_switches_round_trip():
    """The kernel-choice switches are plain values behind tllm_debug_set_tuning / tllm_debug_get_tuning (no
    environment reads on any call path): set, read back, restore; unknown names are rejected."""
    import ternary_llm_amd as tl
    for name, default in (("gemm_rowsplit", -1), ("stage_spin_limit", 0), ("batch_k_parts", 0), ("tall_max_batch", 4),
                          ("tall_min_share_milli", 1000), ("gemm_path", 0)):
        assert tl.get_tuning(name) == default, name
        with tl.tuning(**{name: 7}):
            assert tl.get_tuning(name) == 7
        assert tl.get_tuning(name) == default
    with pytest.raises(tl.TllmError):
        tl.set_tuning("no_such_switch", 1)


def test_kernel_choice_by_shape():
    """Host logic of the dispatcher (reference src/transformer.cpp:112-116: one token -> ternary_gemv, more ->
    ternary_gemm; here one entry point chooses among four kernels by shape, csrc/dispatch.hip). Asked through
    tllm_ternary_gemm_kernel, which touches no GPU (without one the cost model assumes the MI355X's 256 CUs)."""
    k = ops.gemm_kernel
    assert "gemv_mfma_kernel" in k(1, 4096, 4096) and "gemv_mfma_kernel" in k(1, 4096, 14336)
    for m in (2, 4, 16):
        assert "gemv_batch_kernel" in k(m, 4096, 4096)
    assert k(16, 4096, 14336) == "tllm::gemv_batch_kernel, K shared out"       # 64 blocks for 256 CUs: K is shared out
    assert k(16, 14336, 4096) == "tllm::gemv_batch_kernel"
    assert "gemm_ns_kernel<4, 1>" in k(512, 14336, 4096) and "gemm_ns_kernel<4, 1>" in k(512, 4096, 14336)
    assert k(2048, 14336, 4096) == "tllm::gemm_ns_kernel<4, 2>"                 # more tiles than CUs: two workgroups per CU
    assert "gemm_mfma_kernel" in k(100, 1000, 1536)                            # few rows: the four-wave kernel, K split
    assert k(1, 64, 96, 32)                                                    # any group size runs somewhere
    assert k(512, 4096, 4096, 64)
    for bad in ((0, 4096, 4096, 128), (4, 4096, 100, 128), (4, 4096, 4096, 48), (4, 4096, 160, 128)):
        assert k(*bad) == ""
    # the forced forms of the tests answer to their switch and leave it as it was
    before = ops.get_tuning("gemm_rowsplit")
    with ops.tuning(gemm_rowsplit=0):
        assert "gemm_mfma_kernel" in k(512, 14336, 4096)
    with ops.tuning(gemm_rowsplit=2):
        assert k(512, 14336, 4096) == "tllm::gemm_ns_kernel<4, 2>"
    assert ops.get_tuning("gemm_rowsplit") == before
