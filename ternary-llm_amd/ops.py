"""ctypes binding of include/tllm_ternary.h for torch device tensors.

The operator names and argument order mirror the reference's `namespace ternary`
(include/kernels.cuh:11-40): ternary_gemv, ternary_gemv_int8, quantize_absmax_int8,
ternary_gemm. Mask tensors are int32 (the uint32 bit patterns), fp16 tensors are
torch.float16. torch is used for device memory and streams only.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libtllm_ternary.so")
_lib = None

ABI_SYMBOLS = (
    "tllm_error_string", "tllm_abi_version", "tllm_ternary_gemv_f16", "tllm_ternary_gemv_i8",
    "tllm_ternary_gemv_i8_dscale", "tllm_quantize_absmax_i8", "tllm_ternary_gemm_f16",
    "tllm_linear_plan_create", "tllm_linear_plan_launch", "tllm_linear_plan_weight_bytes",
    "tllm_linear_plan_destroy",
)


class TllmError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"tllm error {code}: {text}")
        self.code = code


class _Problem(C.Structure):
    _fields_ = [("nonzero_masks", C.c_void_p), ("sign_masks", C.c_void_p), ("scales", C.c_void_p),
                ("input", C.c_void_p), ("output", C.c_void_p), ("rows", C.c_int32),
                ("cols", C.c_int32), ("batch", C.c_int32), ("reserved", C.c_int32)]


def lib_path():
    return _LIB_PATH


def lib():
    """Loads the HIP library; raises if it has not been built (no fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(f"{_LIB_PATH} is missing: build it with `python ternary-llm_amd/build.py` "
                           "(hipcc, gfx950). There is no CPU fallback.")
    L = C.CDLL(_LIB_PATH)
    vp, i, f = C.c_void_p, C.c_int, C.c_float
    L.tllm_error_string.restype = C.c_char_p
    L.tllm_error_string.argtypes = [i]
    L.tllm_abi_version.restype = i
    L.tllm_ternary_gemv_f16.argtypes = [vp, vp, vp, vp, vp, i, i, i, vp]
    L.tllm_ternary_gemv_i8.argtypes = [vp, vp, vp, vp, f, vp, i, i, i, vp]
    L.tllm_ternary_gemv_i8_dscale.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, vp]
    L.tllm_quantize_absmax_i8.argtypes = [vp, vp, vp, i, vp]
    L.tllm_ternary_gemm_f16.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, vp]
    L.tllm_linear_plan_create.argtypes = [C.POINTER(vp), C.POINTER(_Problem), i, i]
    L.tllm_linear_plan_launch.argtypes = [vp, vp]
    L.tllm_linear_plan_weight_bytes.argtypes = [vp]
    L.tllm_linear_plan_weight_bytes.restype = C.c_int64
    L.tllm_linear_plan_destroy.argtypes = [vp]
    L.tllm_linear_plan_destroy.restype = None
    _lib = L
    return L


def check(code):
    if code != 0:
        raise TllmError(code, lib().tllm_error_string(code).decode())


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream(stream):
    import torch
    if stream is None:
        stream = torch.cuda.current_stream()
    return C.c_void_p(stream.cuda_stream)


def ternary_gemv(nonzero_masks, sign_masks, scales, input, output, rows, cols, group_size=128,
                 stream=None):
    """y[rows] from packed W[rows, cols] and fp16 x[cols] (reference include/kernels.cuh:11-14)."""
    check(lib().tllm_ternary_gemv_f16(_ptr(nonzero_masks), _ptr(sign_masks), _ptr(scales),
                                      _ptr(input), _ptr(output), rows, cols, group_size,
                                      _stream(stream)))


def ternary_gemv_int8(nonzero_masks, sign_masks, weight_scales, input_int8, input_scale, output,
                      rows, cols, group_size=128, stream=None):
    """INT8-activation GEMV (reference include/kernels.cuh:19-24). `input_scale` is a Python
    float (passed by value like the reference) or a 1-element float32 device tensor."""
    L = lib()
    if isinstance(input_scale, (int, float)):
        code = L.tllm_ternary_gemv_i8(_ptr(nonzero_masks), _ptr(sign_masks), _ptr(weight_scales),
                                      _ptr(input_int8), float(input_scale), _ptr(output), rows,
                                      cols, group_size, _stream(stream))
    else:
        code = L.tllm_ternary_gemv_i8_dscale(_ptr(nonzero_masks), _ptr(sign_masks),
                                             _ptr(weight_scales), _ptr(input_int8),
                                             _ptr(input_scale), _ptr(output), rows, cols,
                                             group_size, _stream(stream))
    check(code)


def quantize_absmax_int8(input, output, scale, n, stream=None):
    """half[n] -> int8[n] + device float scale (reference include/kernels.cuh:30-32)."""
    check(lib().tllm_quantize_absmax_i8(_ptr(input), _ptr(output), _ptr(scale), n, _stream(stream)))


def ternary_gemm(A, nz_B, sign_B, scales_B, Cout, M, N, K, group_size=128, stream=None):
    """C[M,N] = A[M,K] @ W[N,K]^T (reference include/kernels.cuh:37-40)."""
    check(lib().tllm_ternary_gemm_f16(_ptr(A), _ptr(nz_B), _ptr(sign_B), _ptr(scales_B), _ptr(Cout),
                                      M, N, K, group_size, _stream(stream)))


class LinearPlan:
    """Several independent ternary linears issued as one launch."""

    def __init__(self, problems, group_size=128):
        """problems: iterable of (nz, sign, scales, input, output, rows, cols, batch)."""
        problems = list(problems)
        arr = (_Problem * max(len(problems), 1))()
        self._keep = problems  # keep the tensors alive as long as the plan
        for k, (nz, sg, sc, x, y, rows, cols, batch) in enumerate(problems):
            arr[k] = _Problem(nz.data_ptr(), sg.data_ptr(), sc.data_ptr(), x.data_ptr(),
                              y.data_ptr(), rows, cols, batch, 0)
        self._h = C.c_void_p(0)
        check(lib().tllm_linear_plan_create(C.byref(self._h), arr, len(problems), group_size))

    @property
    def weight_bytes(self):
        return int(lib().tllm_linear_plan_weight_bytes(self._h))

    def launch(self, stream=None):
        check(lib().tllm_linear_plan_launch(self._h, _stream(stream)))

    def close(self):
        if self._h:
            lib().tllm_linear_plan_destroy(self._h)
            self._h = C.c_void_p(0)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
