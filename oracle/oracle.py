"""ctypes binding of the CPU oracle (oracle/tllm_oracle.c). TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the cpu_baseline leg of bench.py import this
module; the shipped library never does. `build()` compiles the C file with gcc;
`load()` opens the built shared object and fails loudly if it is absent.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(_HERE, "tllm_oracle.c")
LIB = os.path.join(_HERE, "libtllm_oracle.so")

_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")


def build(force=True):
    """Compile the oracle with gcc (plain C, -O2, no fast-math so fp order is kept)."""
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(SRC):
        return LIB
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-o", LIB, SRC,
           "-lm", "-lpthread"]
    subprocess.run(cmd, check=True)
    return LIB


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB):
        raise RuntimeError(f"oracle library {LIB} is not built; run oracle.oracle.build()")
    L = C.CDLL(LIB)
    L.tllm_oracle_half_to_float.restype = C.c_float
    L.tllm_oracle_half_to_float.argtypes = [C.c_uint16]
    L.tllm_oracle_double_to_half.restype = C.c_uint16
    L.tllm_oracle_double_to_half.argtypes = [C.c_double]
    L.tllm_oracle_pack.argtypes = [_i8p, C.c_int, C.c_int, _u32p, _u32p]
    L.tllm_oracle_unpack.argtypes = [_u32p, _u32p, C.c_int, C.c_int, _i8p]
    L.tllm_oracle_gemv_f64.argtypes = [_u32p, _u32p, _u16p, _u16p, _f64p, C.c_int, C.c_int, C.c_int]
    L.tllm_oracle_gemv_hostloop.argtypes = [_u32p, _u32p, _f32p, _f32p, _f32p, C.c_int, C.c_int,
                                            C.c_int]
    L.tllm_oracle_gemv_hostloop_mt.argtypes = [_u32p, _u32p, _f32p, _f32p, _f32p, C.c_int, C.c_int,
                                               C.c_int, C.c_int]
    L.tllm_oracle_gemm_f64.argtypes = [_u16p, _u32p, _u32p, _u16p, _f64p, C.c_int, C.c_int, C.c_int,
                                       C.c_int]
    L.tllm_oracle_gemm_f32_elem.argtypes = [_u16p, _u32p, _u32p, _u16p, _f32p, C.c_int, C.c_int,
                                            C.c_int, C.c_int]
    L.tllm_oracle_quantize_i8.argtypes = [_u16p, _i8p, C.POINTER(C.c_float), C.c_int]
    L.tllm_oracle_gemv_i8_f64.argtypes = [_u32p, _u32p, _u16p, _i8p, C.c_float, _f64p, C.c_int,
                                          C.c_int, C.c_int]
    L.tllm_oracle_ternarize.argtypes = [_f32p, C.c_int64, C.c_int, C.c_float, _i8p, _u16p]
    L.tllm_oracle_rmsnorm_f64.argtypes = [_u16p, _u16p, C.c_void_p, C.c_void_p, _f64p, C.c_int, C.c_int,
                                          C.c_float]
    L.tllm_oracle_silu_mul_f64.argtypes = [_u16p, _u16p, _f64p, C.c_int]
    L.tllm_oracle_add_f64.argtypes = [_u16p, _u16p, _f64p, C.c_int]
    L.tllm_oracle_rope_f64.argtypes = [_u16p, _f64p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_double]
    L.tllm_oracle_rope_f32angle.argtypes = [_u16p, _u16p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    for f in ("add_f64", "rope_f64", "rmsnorm_f64", "silu_mul_f64", "pack", "unpack", "gemv_f64", "gemv_hostloop", "gemv_hostloop_mt", "gemm_f64",
              "gemm_f32_elem", "quantize_i8", "gemv_i8_f64", "ternarize"):
        getattr(L, "tllm_oracle_" + f).restype = None
    _lib = L
    return L


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def pack(w):
    """int8 {-1,0,1} [rows, cols] -> (nz, sign) uint32 [rows, cols/32]."""
    w = _c(w, np.int8)
    rows, cols = w.shape
    assert cols % 32 == 0
    nz = np.empty((rows, cols // 32), np.uint32)
    sg = np.empty_like(nz)
    load().tllm_oracle_pack(w, rows, cols, nz, sg)
    return nz, sg


def unpack(nz, sg):
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    rows, words = nz.shape
    w = np.empty((rows, words * 32), np.int8)
    load().tllm_oracle_unpack(nz, sg, rows, words * 32, w)
    return w


def gemv_f64(nz, sg, scales, x, group=128):
    """fp64 y[rows] from packed masks, fp16-bit scales [rows, cols/group] and fp16-bit x[cols]."""
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    rows, words = nz.shape
    y = np.empty(rows, np.float64)
    load().tllm_oracle_gemv_f64(nz, sg, _c(scales, np.uint16), _c(x, np.uint16), y, rows,
                                words * 32, group)
    return y


def gemv_hostloop(nz, sg, scales_f32, x_f32, group=128, threads=1):
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    rows, words = nz.shape
    y = np.empty(rows, np.float32)
    if threads <= 1:
        load().tllm_oracle_gemv_hostloop(nz, sg, _c(scales_f32, np.float32), _c(x_f32, np.float32),
                                         y, rows, words * 32, group)
    else:
        load().tllm_oracle_gemv_hostloop_mt(nz, sg, _c(scales_f32, np.float32),
                                            _c(x_f32, np.float32), y, rows, words * 32, group,
                                            threads)
    return y


def gemm_f64(A, nz, sg, scales, group=128):
    """fp64 C[M,N] from fp16-bit A[M,K] and the packed N x K weight."""
    A = _c(A, np.uint16)
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    M, K = A.shape
    N, words = nz.shape
    assert words * 32 == K
    Cm = np.empty((M, N), np.float64)
    load().tllm_oracle_gemm_f64(A, nz, sg, _c(scales, np.uint16), Cm, M, N, K, group)
    return Cm


def gemm_f32_elem(A, nz, sg, scales, group=128):
    A = _c(A, np.uint16)
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    M, K = A.shape
    N, _ = nz.shape
    Cm = np.empty((M, N), np.float32)
    load().tllm_oracle_gemm_f32_elem(A, nz, sg, _c(scales, np.uint16), Cm, M, N, K, group)
    return Cm


def quantize_i8(x):
    x = _c(x, np.uint16)
    q = np.empty(x.shape[0], np.int8)
    s = C.c_float(0.0)
    load().tllm_oracle_quantize_i8(x, q, C.byref(s), x.shape[0])
    return q, float(s.value)


def gemv_i8_f64(nz, sg, scales, xq, input_scale, group=128):
    nz, sg = _c(nz, np.uint32), _c(sg, np.uint32)
    rows, words = nz.shape
    y = np.empty(rows, np.float64)
    load().tllm_oracle_gemv_i8_f64(nz, sg, _c(scales, np.uint16), _c(xq, np.int8),
                                   float(input_scale), y, rows, words * 32, group)
    return y


def rmsnorm_f64(x, w, eps, residual=None, store_residual=False):
    """x, residual: fp16 bits [batch, dim]; w: fp16 bits [dim]. Returns (out f64, residual_out bits or None)."""
    x, w = _c(x, np.uint16), _c(w, np.uint16)
    batch, dim = x.shape
    out = np.empty((batch, dim), np.float64)
    res = _c(residual, np.uint16) if residual is not None else None
    ro = np.empty((batch, dim), np.uint16) if (store_residual and res is not None) else None
    load().tllm_oracle_rmsnorm_f64(x, w, res.ctypes.data if res is not None else None,
                                   ro.ctypes.data if ro is not None else None, out, batch, dim, float(eps))
    return out, ro


def silu_mul_f64(gate, up):
    gate, up = _c(gate, np.uint16).reshape(-1), _c(up, np.uint16).reshape(-1)
    out = np.empty(gate.size, np.float64)
    load().tllm_oracle_silu_mul_f64(gate, up, out, gate.size)
    return out


def add_f64(a, b):
    a, b = _c(a, np.uint16).reshape(-1), _c(b, np.uint16).reshape(-1)
    out = np.empty(a.size, np.float64)
    load().tllm_oracle_add_f64(a, b, out, a.size)
    return out


def rope_f64(x, batch, seq_len, heads, head_dim, start_pos, theta):
    """x: fp16 bits [batch, seq_len, heads, head_dim] -> rotated values, float64, same shape
    (reference kernels/rope.cu:22-80; q and k are rotated alike, each with its own head count)."""
    x = _c(x, np.uint16)
    assert x.size == batch * seq_len * heads * head_dim and head_dim % 2 == 0
    out = np.empty(x.size, np.float64)
    load().tllm_oracle_rope_f64(x.reshape(-1), out, batch, seq_len, heads, head_dim, start_pos, float(theta))
    return out.reshape(batch, seq_len, heads, head_dim)


def rope_f32angle(x, batch, seq_len, heads, head_dim, start_pos, theta):
    """The rotation in the reference's fp32 arithmetic (kernels/rope.cu:49-64): fp16 bits in, fp16 bits out."""
    x = _c(x, np.uint16)
    assert x.size == batch * seq_len * heads * head_dim and head_dim % 2 == 0
    out = np.empty(x.size, np.uint16)
    load().tllm_oracle_rope_f32angle(x.reshape(-1), out, batch, seq_len, heads, head_dim, start_pos, float(theta))
    return out.reshape(batch, seq_len, heads, head_dim)


def embedding_lookup(table, indices):
    """Rows of `table` picked by `indices` (reference kernels/elementwise.cu:54-89)."""
    return np.asarray(table)[np.asarray(indices, dtype=np.int64)]


def copy_to_kv_cache(k, v, k_cache, v_cache, start_pos):
    """Returns the caches [batch, n_kv_heads, max_seq_len, head_dim] after rows k, v
    [batch, seq_len, n_kv_heads, head_dim] went in at start_pos; positions past the cache are
    dropped (reference kernels/elementwise.cu:97-147)."""
    k_cache, v_cache = np.array(k_cache, copy=True), np.array(v_cache, copy=True)
    seq_len, max_seq = k.shape[1], k_cache.shape[2]
    n = max(0, min(seq_len, max_seq - start_pos))
    if n:
        k_cache[:, :, start_pos:start_pos + n, :] = np.transpose(np.asarray(k)[:, :n], (0, 2, 1, 3))
        v_cache[:, :, start_pos:start_pos + n, :] = np.transpose(np.asarray(v)[:, :n], (0, 2, 1, 3))
    return k_cache, v_cache


def ternarize(w, group=128, factor=0.7):
    w = _c(w, np.float32)
    flat = w.reshape(-1)
    assert flat.size % group == 0
    t = np.empty(flat.size, np.int8)
    s = np.empty(flat.size // group, np.uint16)
    load().tllm_oracle_ternarize(flat, flat.size, group, factor, t, s)
    return t.reshape(w.shape), s


def half_bits(a):
    """float array -> IEEE binary16 bit patterns (numpy's RNE conversion)."""
    return np.asarray(a, dtype=np.float16).view(np.uint16)


def half_values(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float64)


def error_report(got, ref):
    """The parity metric: max |got-ref| / max(|ref|, tau), tau = 2^-6 * rms(ref)."""
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    tau = rms / 64.0
    err = np.abs(got - ref)
    den = np.maximum(np.abs(ref), tau) if tau > 0 else np.ones_like(ref)
    small = np.abs(ref) < tau
    return {
        "max_rel": float(np.max(err / den)) if ref.size else 0.0,
        "normwise": float(np.max(err) / max(float(np.max(np.abs(ref))), 1e-300)) if ref.size else 0.0,
        "tau": tau,
        "n_small": int(np.count_nonzero(small)),
        "max_abs_small": float(np.max(err[small])) if small.any() else 0.0,
    }
