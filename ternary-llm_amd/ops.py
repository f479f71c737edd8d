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
    "tllm_linear_plan_destroy", "tllm_rmsnorm_f16", "tllm_silu_mul_f16", "tllm_linear_plan_create_normed", "tllm_linear_plan_create_i8",
    "tllm_add_f16", "tllm_rope_f16", "tllm_embedding_lookup_f16", "tllm_copy_to_kv_cache_f16",
    "tllm_linear_plan_kernel", "tllm_gemm_workspace_reserve", "tllm_gemm_workspace_release",
    "tllm_ternary_gemm_f16_static", "tllm_ternary_gemm_swiglu_f16", "tllm_ternary_gemm_group_f16", "tllm_read_stream", "tllm_ternary_gemm_kernel",
    "tllm_debug_set_tuning", "tllm_debug_get_tuning", "tllm_ternary_linear_int8_f16",
    "tllm_linear_plan_create_staged", "tllm_linear_plan_status",
)
# include/tllm_model_file.h
FILE_ABI_SYMBOLS = (
    "tllm_ternarize_pack_f32", "tllm_model_file_open", "tllm_model_file_close", "tllm_model_file_header",
    "tllm_model_file_linear_count", "tllm_model_file_linear", "tllm_model_file_pool_bytes",
    "tllm_model_file_upload", "tllm_model_file_problem", "tllm_model_file_write_synthetic",
)


class TllmError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"tllm error {code}: {text}")
        self.code = code


class _Problem(C.Structure):
    _fields_ = [("nonzero_masks", C.c_void_p), ("sign_masks", C.c_void_p), ("scales", C.c_void_p),
                ("input", C.c_void_p), ("output", C.c_void_p), ("rows", C.c_int32),
                ("cols", C.c_int32), ("batch", C.c_int32), ("flags", C.c_int32)]


class FileHeader(C.Structure):
    """The 256-byte .tllm header (include/tllm_model_file.h, reference include/format.h:20-37)."""
    _fields_ = [(n, C.c_uint32) for n in (
        "magic", "version", "arch", "vocab_size", "hidden_dim", "intermediate_dim", "n_layers", "n_heads",
        "n_kv_heads", "max_seq_len", "head_dim", "rope_theta_bits", "group_size", "rms_norm_eps_bits", "flags")] + \
        [("reserved", C.c_uint8 * (256 - 15 * 4))]


class FileLinear(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("nonzero_file", "sign_file", "scales_file",
                                           "nonzero_pool", "sign_pool", "scales_pool")] + \
        [(n, C.c_int32) for n in ("rows", "cols", "layer", "kind")]


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
    L.tllm_ternary_linear_int8_f16.argtypes = [vp, vp, vp, vp, vp, i, i, i, vp]
    L.tllm_ternary_gemv_i8_dscale.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, vp]
    L.tllm_quantize_absmax_i8.argtypes = [vp, vp, vp, i, vp]
    L.tllm_ternary_gemm_f16.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, vp]
    L.tllm_ternary_gemm_f16_static.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, vp]
    L.tllm_ternary_gemm_swiglu_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp]
    L.tllm_ternary_gemm_group_f16.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, vp]
    L.tllm_gemm_workspace_reserve.argtypes = [i, i, i, i, vp]
    L.tllm_read_stream.argtypes = [vp, C.c_size_t, vp, vp]
    L.tllm_gemm_workspace_release.argtypes = []
    L.tllm_debug_set_tuning.argtypes = [C.c_char_p, i]
    L.tllm_debug_get_tuning.argtypes = [C.c_char_p, C.POINTER(i)]
    L.tllm_gemm_workspace_release.restype = None
    L.tllm_linear_plan_create.argtypes = [C.POINTER(vp), C.POINTER(_Problem), i, i]
    L.tllm_linear_plan_create_normed.argtypes = [C.POINTER(vp), C.POINTER(_Problem), C.POINTER(vp), f, i, i]
    L.tllm_linear_plan_create_i8.argtypes = [C.POINTER(vp), C.POINTER(_Problem), C.POINTER(vp), i, i]
    L.tllm_linear_plan_create_staged.argtypes = [C.POINTER(vp), C.POINTER(_Problem), C.POINTER(vp), C.POINTER(vp),
                                                 C.POINTER(C.c_int32), f, i, i]
    L.tllm_linear_plan_status.argtypes = [vp]
    L.tllm_linear_plan_launch.argtypes = [vp, vp]
    L.tllm_linear_plan_weight_bytes.argtypes = [vp]
    L.tllm_linear_plan_weight_bytes.restype = C.c_int64
    L.tllm_linear_plan_destroy.argtypes = [vp]
    L.tllm_linear_plan_kernel.argtypes = [vp]
    L.tllm_linear_plan_kernel.restype = C.c_char_p
    L.tllm_ternary_gemm_kernel.argtypes = [i, i, i, i]
    L.tllm_ternary_gemm_kernel.restype = C.c_char_p
    L.tllm_linear_plan_destroy.restype = None
    L.tllm_rmsnorm_f16.argtypes = [vp, vp, vp, vp, vp, i, i, f, vp]
    L.tllm_silu_mul_f16.argtypes = [vp, vp, vp, i, vp]
    L.tllm_add_f16.argtypes = [vp, vp, vp, i, vp]
    L.tllm_rope_f16.argtypes = [vp, vp, i, i, i, i, i, i, f, vp]
    L.tllm_embedding_lookup_f16.argtypes = [vp, vp, vp, i, i, vp]
    L.tllm_copy_to_kv_cache_f16.argtypes = [vp, vp, vp, vp, i, i, i, i, i, i, vp]
    L.tllm_ternarize_pack_f32.argtypes = [vp, i, i, i, f, vp, vp, vp]
    L.tllm_model_file_open.argtypes = [C.c_char_p, C.POINTER(vp)]
    L.tllm_model_file_close.argtypes = [vp]
    L.tllm_model_file_close.restype = None
    L.tllm_model_file_header.argtypes = [vp, C.POINTER(FileHeader)]
    L.tllm_model_file_linear_count.argtypes = [vp]
    L.tllm_model_file_linear.argtypes = [vp, i, C.POINTER(FileLinear)]
    L.tllm_model_file_pool_bytes.argtypes = [vp]
    L.tllm_model_file_pool_bytes.restype = C.c_uint64
    L.tllm_model_file_upload.argtypes = [vp, vp, C.c_uint64, vp]
    L.tllm_model_file_problem.argtypes = [vp, i, vp, C.POINTER(_Problem)]
    L.tllm_model_file_write_synthetic.argtypes = [C.c_char_p, C.POINTER(FileHeader), C.c_uint64]
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


def ternary_linear_int8(nonzero_masks, sign_masks, weight_scales, input, output, rows, cols, group_size=128, stream=None):
    """The reference's INT8 linear (Transformer::ternary_linear_int8, src/transformer.cpp:126-143) in one launch:
    fp16 input, quantised inside the kernel; bit for bit quantize_absmax_int8 + ternary_gemv_int8."""
    check(lib().tllm_ternary_linear_int8_f16(_ptr(nonzero_masks), _ptr(sign_masks), _ptr(weight_scales), _ptr(input),
                                             _ptr(output), rows, cols, group_size, _stream(stream)))


def quantize_absmax_int8(input, output, scale, n, stream=None):
    """half[n] -> int8[n] + device float scale (reference include/kernels.cuh:30-32)."""
    check(lib().tllm_quantize_absmax_i8(_ptr(input), _ptr(output), _ptr(scale), n, _stream(stream)))


def ternary_gemm(A, nz_B, sign_B, scales_B, Cout, M, N, K, group_size=128, stream=None):
    """C[M,N] = A[M,K] @ W[N,K]^T (reference include/kernels.cuh:37-40)."""
    check(lib().tllm_ternary_gemm_f16(_ptr(A), _ptr(nz_B), _ptr(sign_B), _ptr(scales_B), _ptr(Cout),
                                      M, N, K, group_size, _stream(stream)))


def ternary_gemm_swiglu(A, nz_gate, sign_gate, scales_gate, nz_up, sign_up, scales_up, Cout, M, N, K, group_size=128, stream=None):
    """C[M,N] = silu(A @ gate^T) * (A @ up^T) in one launch: ternary_gemm on both matrices and silu_mul
    (reference src/transformer.cpp:264-286 at n_tokens > 1)."""
    check(lib().tllm_ternary_gemm_swiglu_f16(_ptr(A), _ptr(nz_gate), _ptr(sign_gate), _ptr(scales_gate), _ptr(nz_up),
                                             _ptr(sign_up), _ptr(scales_up), _ptr(Cout), M, N, K, group_size, _stream(stream)))


def ternary_gemm_group(A, weights, outputs, M, K, group_size=128, stream=None):
    """Several ternary_gemm calls on the same activations in one launch (the q/k/v projections of a prefill step,
    reference src/transformer.cpp:199-217 at n_tokens > 1). weights: [(nz, sign, scales), ...]; outputs: [C_i [M, N_i], ...]."""
    n = len(weights)
    arr = lambda vals: (C.c_void_p * n)(*[v.data_ptr() for v in vals])
    rows = (C.c_int * n)(*[int(o.shape[-1]) for o in outputs])
    check(lib().tllm_ternary_gemm_group_f16(_ptr(A), arr([w[0] for w in weights]), arr([w[1] for w in weights]),
                                            arr([w[2] for w in weights]), arr(outputs), rows, n, M, K, group_size, _stream(stream)))


def ternary_gemm_static(A, nz_B, sign_B, scales_B, Cout, M, N, K, group_size=128, stream=None):
    """ternary_gemm that never allocates: the split-K exchange uses the library's fixed device array."""
    check(lib().tllm_ternary_gemm_f16_static(_ptr(A), _ptr(nz_B), _ptr(sign_B), _ptr(scales_B), _ptr(Cout),
                                             M, N, K, group_size, _stream(stream)))


def read_stream(buf, stream=None):
    """Measurement aid: one read-only pass over a device tensor (the streaming ceiling of the GPU)."""
    check(lib().tllm_read_stream(_ptr(buf), buf.numel() * buf.element_size(), None, _stream(stream)))


def set_tuning(name, value):
    """Testing aid: sets one kernel-choice switch of the library (include/tllm_ternary.h, tllm_debug_set_tuning)."""
    check(lib().tllm_debug_set_tuning(name.encode(), int(value)))


def get_tuning(name):
    v = C.c_int(0)
    check(lib().tllm_debug_get_tuning(name.encode(), C.byref(v)))
    return v.value


class tuning:
    """with tuning(gemm_rowsplit=1, ...): the switches are set inside the block and put back afterwards."""

    def __init__(self, **kw):
        self.want = kw

    def __enter__(self):
        self.old = {k: get_tuning(k) for k in self.want}
        for k, v in self.want.items():
            set_tuning(k, v)
        return self

    def __exit__(self, *exc):
        for k, v in self.old.items():
            set_tuning(k, v)
        return False


def gemm_kernel(M, N, K, group_size=128):
    """Name of the kernel ternary_gemm runs for this shape on the current device."""
    return lib().tllm_ternary_gemm_kernel(M, N, K, group_size).decode()


def gemm_workspace_reserve(M, N, K, group_size=128, stream=None):
    """Creates the split-K workspace of the stream for this GEMM shape ahead of time (e.g. before graph capture)."""
    check(lib().tllm_gemm_workspace_reserve(M, N, K, group_size, _stream(stream)))


def gemm_workspace_release():
    """Frees every split-K workspace of the process (no GEMM may be in flight)."""
    lib().tllm_gemm_workspace_release()


def rmsnorm(input, weight, output, residual, residual_out, batch, dim, eps, stream=None):
    """RMSNorm with optional fused residual add (reference include/kernels.cuh:45-48)."""
    check(lib().tllm_rmsnorm_f16(_ptr(input), _ptr(weight), _ptr(output), _ptr(residual), _ptr(residual_out),
                                 batch, dim, float(eps), _stream(stream)))


def silu_mul(gate, up, output, size, stream=None):
    """SiLU(gate) * up (reference include/kernels.cuh:60-62)."""
    check(lib().tllm_silu_mul_f16(_ptr(gate), _ptr(up), _ptr(output), size, _stream(stream)))


def add(a, b, output, size, stream=None):
    """output = a + b in fp16 (reference include/kernels.cuh:64-66)."""
    check(lib().tllm_add_f16(_ptr(a), _ptr(b), _ptr(output), size, _stream(stream)))


def rope(q, k, batch, seq_len, n_heads, n_kv_heads, head_dim, start_pos, theta, stream=None):
    """Rotary position embedding of q and k in place (reference include/kernels.cuh:50-53)."""
    check(lib().tllm_rope_f16(_ptr(q), _ptr(k), batch, seq_len, n_heads, n_kv_heads, head_dim, start_pos, theta,
                              _stream(stream)))


def embedding_lookup(table, indices, output, n_tokens, dim, stream=None):
    """output[t] = table[indices[t]] (reference include/kernels.cuh:68-70); indices: int32 on the device."""
    check(lib().tllm_embedding_lookup_f16(_ptr(table), _ptr(indices), _ptr(output), n_tokens, dim, _stream(stream)))


def copy_to_kv_cache(k, v, k_cache, v_cache, batch, n_kv_heads, head_dim, seq_len, start_pos, max_seq_len,
                     stream=None):
    """New k/v rows into the caches at start_pos (reference include/kernels.cuh:72-76)."""
    check(lib().tllm_copy_to_kv_cache_f16(_ptr(k), _ptr(v), _ptr(k_cache), _ptr(v_cache), batch, n_kv_heads, head_dim,
                                          seq_len, start_pos, max_seq_len, _stream(stream)))


SWIGLU_GATE = 1  # TLLM_PROBLEM_SWIGLU_GATE
QUANTIZE_INPUT = 2  # TLLM_PROBLEM_QUANTIZE_INPUT


class LinearPlan:
    """Several independent ternary linears issued as one launch."""

    def __init__(self, problems, group_size=128, norm_weights=None, eps=1e-5, input_scales=None, stages=None,
                 residuals=None):
        """problems: iterable of (nz, sign, scales, input, output, rows, cols, batch[, flags]);
        flags = SWIGLU_GATE marks the gate of a pair whose up projection is the next problem
        (output may be None there): the pair stores silu(gate) * up in the gate's output."""
        problems = list(problems)
        arr = (_Problem * max(len(problems), 1))()
        self._keep = problems  # keep the tensors alive as long as the plan
        for k, prob in enumerate(problems):
            nz, sg, sc, x, y, rows, cols, batch = prob[:8]
            flags = prob[8] if len(prob) > 8 else 0
            arr[k] = _Problem(nz.data_ptr(), sg.data_ptr(), sc.data_ptr(), x.data_ptr(),
                              y.data_ptr() if y is not None else 0, rows, cols, batch, flags)
        self._h = C.c_void_p(0)
        if stages is not None:
            # dependent problems in one launch: stages[k] ascending; residuals[k] (or None) is added behind problem k's projection
            n = max(len(problems), 1)
            self._keep_norm = list(norm_weights) if norm_weights is not None else [None] * len(problems)
            self._keep_res = list(residuals) if residuals is not None else [None] * len(problems)
            nw = (C.c_void_p * n)(*[w.data_ptr() if w is not None else None for w in self._keep_norm])
            rs = (C.c_void_p * n)(*[r.data_ptr() if r is not None else None for r in self._keep_res])
            st = (C.c_int32 * n)(*[int(v) for v in stages])
            check(lib().tllm_linear_plan_create_staged(C.byref(self._h), arr, nw, rs, st, float(eps), len(problems), group_size))
        elif input_scales is not None:
            # int8 activations: every problem's input is an int8 tensor, input_scales[k] the float32 device tensor
            # that quantize_absmax_int8 wrote for it
            self._keep_scales = list(input_scales)
            ptrs = (C.c_void_p * max(len(problems), 1))(*[t.data_ptr() for t in self._keep_scales])
            check(lib().tllm_linear_plan_create_i8(C.byref(self._h), arr, ptrs, len(problems), group_size))
        elif norm_weights is None:
            check(lib().tllm_linear_plan_create(C.byref(self._h), arr, len(problems), group_size))
        else:
            # one fp16 weight tensor (or None) per problem: RMSNorm prologue on that problem's input
            self._keep_norm = list(norm_weights)
            ptrs = (C.c_void_p * max(len(problems), 1))(*[w.data_ptr() if w is not None else None
                                                         for w in self._keep_norm])
            check(lib().tllm_linear_plan_create_normed(C.byref(self._h), arr, ptrs, float(eps), len(problems),
                                                       group_size))

    @property
    def weight_bytes(self):
        return int(lib().tllm_linear_plan_weight_bytes(self._h))

    @property
    def kernel(self):
        """Name of the kernel a launch of this plan runs."""
        return lib().tllm_linear_plan_kernel(self._h).decode()

    def launch(self, stream=None):
        check(lib().tllm_linear_plan_launch(self._h, _stream(stream)))

    def status(self):
        """Staged plans: raises TllmError if a launch gave up waiting between two stages since the last call."""
        check(lib().tllm_linear_plan_status(self._h))

    def close(self):
        if self._h:
            lib().tllm_linear_plan_destroy(self._h)
            self._h = C.c_void_p(0)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def ternarize_pack(weight, group_size=128, threshold_factor=0.7):
    """Host: fp32 matrix [rows, cols] -> (nonzero uint32 [rows, cols/32], sign uint32, scales fp16
    [rows, cols/group]) as numpy arrays (reference ternarize/pack.py:41-101, 120-169)."""
    import numpy as np
    w = np.ascontiguousarray(weight, dtype=np.float32)
    rows, cols = w.shape
    nz = np.zeros((rows, max(cols // 32, 1)), np.uint32)
    sg = np.zeros_like(nz)
    sc = np.zeros((rows, max(cols // max(group_size, 1), 1)), np.uint16)
    check(lib().tllm_ternarize_pack_f32(w.ctypes.data, rows, cols, group_size, threshold_factor,
                                        nz.ctypes.data, sg.ctypes.data, sc.ctypes.data))
    return nz, sg, sc.view(np.float16)


def write_synthetic_model(path, seed=0, **dims):
    """Writes a synthetic .tllm file; dims are FileHeader fields (vocab_size, hidden_dim, ...)."""
    h = FileHeader()
    for k, v in dims.items():
        setattr(h, k, v)
    check(lib().tllm_model_file_write_synthetic(os.fsencode(path), C.byref(h), seed))


class ModelFile:
    """A .tllm file: header, the layout of its ternary linears, upload into one device pool."""

    def __init__(self, path):
        self._h = C.c_void_p(0)
        check(lib().tllm_model_file_open(os.fsencode(path), C.byref(self._h)))
        self.header = FileHeader()
        check(lib().tllm_model_file_header(self._h, C.byref(self.header)))
        self.linears = []
        for k in range(lib().tllm_model_file_linear_count(self._h)):
            fl = FileLinear()
            check(lib().tllm_model_file_linear(self._h, k, C.byref(fl)))
            self.linears.append(fl)
        self.pool_bytes = int(lib().tllm_model_file_pool_bytes(self._h))

    def upload(self, pool, stream=None):
        """pool: a uint8 device tensor of at least pool_bytes."""
        check(lib().tllm_model_file_upload(self._h, _ptr(pool), pool.numel(), _stream(stream)))

    def problem(self, index, pool):
        """(nz_ptr, sign_ptr, scales_ptr, rows, cols) of linear `index` inside `pool`."""
        pr = _Problem()
        check(lib().tllm_model_file_problem(self._h, index, _ptr(pool), C.byref(pr)))
        return pr.nonzero_masks, pr.sign_masks, pr.scales, pr.rows, pr.cols

    def close(self):
        if self._h:
            lib().tllm_model_file_close(self._h)
            self._h = C.c_void_p(0)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
