"""Pins the CPU oracle before anything is compared against it.

Each check is one a plausible mistake (wrong bit order, dropped scale, sign used
under a clear nz bit, transposed operand, wrong group index) would fail:
known-answer words from the reference's tests/test_packing.py:55-81, closed forms,
brute force over all ternary patterns, and a dense numpy float64 product built by
an independent unpacker (numpy unpackbits), not by the oracle's own loops.
"""
import itertools
import json
import math
import os

import numpy as np
import pytest

from tests import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ------------------------------------------------------------------ layout
def test_pack_known_answer_words(oracle):
    # tests/test_packing.py:55-81: row 0 has +1@0, -1@1, +1@31, -1@32, -1@63;
    # row 1 alternates +1/-1 over its first 32 columns.
    t = np.zeros((2, 64), np.int8)
    t[0, 0], t[0, 1], t[0, 31], t[0, 32], t[0, 63] = 1, -1, 1, -1, -1
    t[1, :32] = np.where(np.arange(32) % 2 == 0, 1, -1)
    nz, sg = oracle.pack(t)
    assert nz.shape == (2, 2) and sg.shape == (2, 2)
    assert nz[0, 0] == 0x80000003 and sg[0, 0] == 0x80000001
    assert nz[0, 1] == 0x80000001 and sg[0, 1] == 0x00000000
    assert nz[1, 0] == 0xFFFFFFFF and sg[1, 0] == 0x55555555
    assert nz[1, 1] == 0 and sg[1, 1] == 0
    np.testing.assert_array_equal(oracle.unpack(nz, sg), t)
    # the independent numpy packer agrees word for word
    nz2, sg2 = synth.pack_np(t)
    np.testing.assert_array_equal(nz, nz2)
    np.testing.assert_array_equal(sg, sg2)


def test_pack_roundtrip_random(oracle):
    rng = np.random.default_rng(123)
    w = synth.ternary_matrix(rng, 37, 416, 0.42)
    nz, sg = oracle.pack(w)
    np.testing.assert_array_equal(oracle.unpack(nz, sg), w)
    np.testing.assert_array_equal(synth.unpack_np(nz, sg), w)
    # single set bit: column 32*j+b <-> bit b of word j
    for col in (0, 1, 31, 32, 63, 64, 415):
        one = np.zeros((1, 416), np.int8)
        one[0, col] = -1
        n, s = oracle.pack(one)
        assert n[0, col // 32] == np.uint32(1 << (col % 32)) and n.sum() == n[0, col // 32]
        assert s.sum() == 0


def test_unpack_ignores_sign_under_zero(oracle):
    nz = np.array([[0x0000FFFF]], np.uint32)
    sg = np.array([[0xFFFF00FF]], np.uint32)
    w = oracle.unpack(nz, sg)[0]
    assert (w[:8] == 1).all() and (w[8:16] == -1).all() and (w[16:] == 0).all()


def test_half_conversions_exhaustive(oracle):
    L = oracle.load()
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    mine = np.array([L.tllm_oracle_half_to_float(int(b)) for b in bits], np.float32)
    finite = np.isfinite(vals)
    np.testing.assert_array_equal(mine[finite], vals[finite])
    assert np.isnan(mine[~finite & np.isnan(vals)]).all()
    # double -> half RNE against numpy, incl. ties, subnormals and overflow
    rng = np.random.default_rng(7)
    probe = np.concatenate([
        rng.standard_normal(4000) * 10.0 ** rng.integers(-9, 5, 4000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 5.96e-8, 2.98e-8, 2.9802322387695312e-08,
                  2.99e-8, 6.1e-5, 6.103515625e-05, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
                  1.0 + 2.0 ** -11 + 2.0 ** -30, -2049.0, 2051.0])])
    with np.errstate(over="ignore"):
        want = probe.astype(np.float16).view(np.uint16)
    got = np.array([L.tllm_oracle_double_to_half(float(v)) for v in probe], np.uint16)
    np.testing.assert_array_equal(got, want)


# -------------------------------------------------------------------- GEMV
@pytest.mark.parametrize("rows,cols,seed", [(8, 256, 1), (33, 384, 2), (64, 2048, 3)])
def test_gemv_f64_equals_dense_numpy(oracle, rows, cols, seed):
    nz, sg, s, x = synth.problem(seed, rows, cols, dontcare_sign=True)
    want = synth.dense_f64(nz, sg, s) @ x.astype(np.float64)
    got = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-13)


def test_gemv_closed_forms(oracle):
    rng = np.random.default_rng(11)
    cols = 512
    x = synth.acts_f16(rng, cols)
    xd = x.astype(np.float64)
    ones = np.full((1, cols // 128), 1.0, np.float16)
    full = np.full((1, cols // 32), 0xFFFFFFFF, np.uint32)
    zero = np.zeros_like(full)
    # all +1, s=1 -> sum(x); all -1 -> -sum(x); nz=0 -> exactly 0 whatever the sign words say
    assert oracle.gemv_f64(full, full, ones.view(np.uint16), x.view(np.uint16))[0] == pytest.approx(xd.sum(), rel=1e-13)
    assert oracle.gemv_f64(full, zero, ones.view(np.uint16), x.view(np.uint16))[0] == pytest.approx(-xd.sum(), rel=1e-13)
    assert oracle.gemv_f64(zero, full, ones.view(np.uint16), x.view(np.uint16))[0] == 0.0
    # one non-zero per row -> s[g(k)] * x[k]; distinct scale per group catches a wrong group index
    s = np.array([[0.5, 0.25, 2.0, 3.0]], np.float16)
    for k in (0, 127, 128, 200, 511):
        w = np.zeros((1, cols), np.int8)
        w[0, k] = -1
        nz, sg = synth.pack_np(w)
        got = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))[0]
        assert got == -float(s[0, k // 128]) * xd[k]


def test_gemv_invariants(oracle):
    nz, sg, s, x = synth.problem(5, 16, 640)
    su, xu = s.view(np.uint16), x.view(np.uint16)
    y = oracle.gemv_f64(nz, sg, su, xu)
    # sign antisymmetry: flipping every sign bit negates y
    np.testing.assert_allclose(oracle.gemv_f64(nz, ~sg, su, xu), -y, rtol=1e-13, atol=0)
    # don't-care sign bits under zero weights
    rng = np.random.default_rng(6)
    junk = rng.integers(0, 2**32, nz.shape, dtype=np.uint64).astype(np.uint32) & ~nz
    np.testing.assert_array_equal(oracle.gemv_f64(nz, sg | junk, su, xu), y)
    # row permutation equivariance
    perm = rng.permutation(16)
    np.testing.assert_array_equal(oracle.gemv_f64(nz[perm], sg[perm], s[perm].view(np.uint16), xu), y[perm])
    # linearity in x on exactly representable inputs: y(2x) = 2 y(x)
    x2 = (x.astype(np.float32) * 2).astype(np.float16)
    np.testing.assert_allclose(oracle.gemv_f64(nz, sg, su, x2.view(np.uint16)), 2 * y, rtol=1e-13)
    # per-group scale homogeneity: doubling one group's scale adds that group's contribution once more
    s2 = s.copy()
    s2[:, 2] = (s[:, 2].astype(np.float32) * 2).astype(np.float16)
    contrib = synth.dense_f64(nz, sg, s)[:, 256:384] @ x.astype(np.float64)[256:384]
    np.testing.assert_allclose(oracle.gemv_f64(nz, sg, s2.view(np.uint16), xu), y + contrib, rtol=1e-12, atol=1e-14)


def test_gemv_bruteforce_all_patterns(oracle):
    # all 3^4 patterns in one live nibble (columns 36..39 of a K=128 row), the rest zero
    x = np.zeros(128, np.float16)
    x[36:40] = np.array([1.5, -2.25, 0.375, 7.0], np.float16)
    s = np.array([[0.75]], np.float16)
    for pat in itertools.product((-1, 0, 1), repeat=4):
        w = np.zeros((1, 128), np.int8)
        w[0, 36:40] = pat
        nz, sg = synth.pack_np(w)
        want = 0.75 * sum(p * float(v) for p, v in zip(pat, x[36:40]))
        assert oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))[0] == want


def test_hostloop_matches_f64(oracle):
    nz, sg, s, x = synth.problem(9, 48, 1024, dontcare_sign=True)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    y1 = oracle.gemv_hostloop(nz, sg, s.astype(np.float32), x.astype(np.float32))
    y8 = oracle.gemv_hostloop(nz, sg, s.astype(np.float32), x.astype(np.float32), threads=5)
    np.testing.assert_array_equal(y1, y8)  # row split must not change a bit
    assert oracle.error_report(y1, ref)["max_rel"] < 2e-5
    # exact on integer data (no rounding anywhere): catches index/sign slips in the fp32 loop
    rng = np.random.default_rng(10)
    xi = rng.integers(-8, 9, 1024).astype(np.float32)
    si = rng.integers(1, 5, (48, 8)).astype(np.float32)
    want = (synth.unpack_np(nz, sg).astype(np.float64) * np.repeat(si, 128, axis=1)) @ xi
    np.testing.assert_array_equal(oracle.gemv_hostloop(nz, sg, si, xi).astype(np.float64), want)


def test_gemv_drops_tail_columns_like_reference(oracle):
    # kernels/ternary_gemv.cu:42 groups_per_row = cols / group_size: a trailing partial group is ignored
    nz, sg, s, x = synth.problem(12, 4, 160, group=32)
    s128 = s[:, :1].copy()
    got = oracle.gemv_f64(nz, sg, s128.view(np.uint16), x.view(np.uint16), group=128)
    want = (synth.unpack_np(nz, sg)[:, :128].astype(np.float64) * s128.astype(np.float64)) @ x[:128].astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-13)


# -------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("M,N,K", [(1, 8, 128), (5, 19, 384), (16, 32, 1024)])
def test_gemm_f64_rows_are_gemvs_and_dense(oracle, M, N, K):
    nz, sg, s, _ = synth.problem(20 + M, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M), M, K)
    Cm = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    want = A.astype(np.float64) @ synth.dense_f64(nz, sg, s).T
    np.testing.assert_allclose(Cm, want, rtol=1e-12, atol=1e-13)
    for m in range(M):
        np.testing.assert_allclose(Cm[m], oracle.gemv_f64(nz, sg, s.view(np.uint16), A[m].view(np.uint16)),
                                   rtol=1e-13, atol=1e-15)
    Ce = oracle.gemm_f32_elem(A.view(np.uint16), nz, sg, s.view(np.uint16))
    assert oracle.error_report(Ce, Cm)["max_rel"] < 5e-5


# --------------------------------------------------------------- INT8 pair
def test_quantize_closed_forms(oracle):
    q, sc = oracle.quantize_i8(np.zeros(64, np.float16).view(np.uint16))
    assert sc == 1.0 and not q.any()
    x = np.array([4.0, -4.0, 2.0, 0.0, 1.0], np.float16)
    q, sc = oracle.quantize_i8(x.view(np.uint16))
    assert sc == np.float32(4.0) / np.float32(127.0)
    assert q.tolist() == [127, -127, 64, 0, 32]  # 63.5 -> 64 and 31.75 -> 32
    # ties to even: absmax 127 makes x*inv == x exactly
    x = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float16)
    q, _ = oracle.quantize_i8(x.view(np.uint16))
    assert q.tolist() == [127, 0, 2, 2, 0, -2, -2]


def test_quantize_matches_numpy(oracle):
    rng = np.random.default_rng(31)
    x = synth.acts_f16(rng, 4096)
    q, sc = oracle.quantize_i8(x.view(np.uint16))
    xf = x.astype(np.float32)
    amax = np.abs(xf).max()
    inv = np.float32(127.0) / amax
    want = np.clip(np.rint(xf * inv), -127, 127).astype(np.int8)
    np.testing.assert_array_equal(q, want)
    assert sc == amax / np.float32(127.0)
    assert np.abs(q).max() == 127


def test_gemv_i8_exact_integer(oracle):
    nz, sg, s, _ = synth.problem(41, 24, 512, dontcare_sign=True)
    rng = np.random.default_rng(42)
    xq = rng.integers(-127, 128, 512).astype(np.int8)
    w = synth.unpack_np(nz, sg).astype(np.int64)
    gsum = (w * xq.astype(np.int64)).reshape(24, 4, 128).sum(axis=2)
    want = 0.0123 * (s.astype(np.float64) * gsum).sum(axis=1)
    got = oracle.gemv_i8_f64(nz, sg, s.view(np.uint16), xq, np.float32(0.0123))
    np.testing.assert_allclose(got, np.float64(np.float32(0.0123)) / 0.0123 * want, rtol=1e-12)


# ---------------------------------------------------------------- producer
def test_ternarize_degenerate_cases(oracle):
    # tests/test_packing.py:177-186: all-zero group -> all-zero ternary, scale 0
    t, s = oracle.ternarize(np.zeros((1, 128), np.float32))
    assert not t.any() and s[0] == 0
    # tests/test_packing.py:189-205: +-100 alternating -> all non-zero with matching signs
    w = np.full((1, 128), 100.0, np.float32)
    w[0, ::2] *= -1
    t, s = oracle.ternarize(w)
    np.testing.assert_array_equal(t[0], np.where(np.arange(128) % 2 == 0, -1, 1))
    assert s.view(np.float16)[0] == np.float16(100.0)


def test_ternarize_matches_numpy(oracle):
    rng = np.random.default_rng(42)
    w = rng.standard_normal((256, 128)).astype(np.float32)
    t, s = oracle.ternarize(w)
    assert set(np.unique(t).tolist()) <= {-1, 0, 1}
    assert s.shape == (256,)
    thr = 0.7 * np.abs(w).astype(np.float64).mean(axis=1, keepdims=True)
    margin = np.abs(np.abs(w) - thr) > 1e-5  # away from the threshold both evaluations agree
    want = np.where(w > thr, 1, np.where(w < -thr, -1, 0))
    np.testing.assert_array_equal(t[margin], want[margin])
    nzmean = (np.abs(w) * (t != 0)).sum(axis=1) / np.maximum((t != 0).sum(axis=1), 1)
    np.testing.assert_allclose(s.view(np.float16).astype(np.float64), nzmean, rtol=1.5e-3)


# ------------------------------------------------------------------ golden
def test_golden_fixtures(oracle):
    """Committed vectors (made by tests/golden/make_fixtures.py through the dense numpy
    route, not through the oracle) must be reproduced by the oracle."""
    names = sorted(f for f in os.listdir(GOLDEN) if f.startswith("gemv_") and f.endswith(".json"))
    assert names, "no golden fixtures committed"
    for name in names:
        with open(os.path.join(GOLDEN, name)) as f:
            fx = json.load(f)
        nz = np.array([int(v, 16) for v in fx["nz"]], np.uint32).reshape(fx["rows"], fx["cols"] // 32)
        sg = np.array([int(v, 16) for v in fx["sign"]], np.uint32).reshape(nz.shape)
        s = np.array([int(v, 16) for v in fx["scales"]], np.uint16).reshape(fx["rows"], -1)
        x = np.array([int(v, 16) for v in fx["x"]], np.uint16).reshape(fx["batch"], fx["cols"])
        y = np.array([float.fromhex(v) for v in fx["y_f64"]]).reshape(fx["batch"], fx["rows"])
        for b in range(fx["batch"]):
            got = oracle.gemv_f64(nz, sg, s, x[b], fx["group"])
            np.testing.assert_allclose(got, y[b], rtol=1e-12, atol=1e-14)
        got = oracle.gemm_f64(x, nz, sg, s, fx["group"])
        np.testing.assert_allclose(got, y, rtol=1e-12, atol=1e-14)


# ------------------------------------------------------------ element-wise
def test_rmsnorm_closed_forms(oracle):
    dim, eps = 384, float(np.float32(1e-5))   # eps travels as a C float
    ones = oracle.half_bits(np.ones(dim))
    # constant row c: every output is c / sqrt(c^2 + eps)
    for c in (0.5, -2.0, 3.0):
        out, _ = oracle.rmsnorm_f64(oracle.half_bits(np.full((1, dim), c)), ones, eps)
        np.testing.assert_allclose(out, c / np.sqrt(c * c + eps), rtol=1e-14)
    rng = np.random.default_rng(5)
    x = oracle.half_bits(rng.normal(0, 1.3, (3, dim)))
    # eps = 0, w = 1: the output has unit RMS; and scaling x by a power of two changes nothing
    out, _ = oracle.rmsnorm_f64(x, ones, 0.0)
    np.testing.assert_allclose(np.sqrt((out ** 2).mean(axis=1)), 1.0, rtol=1e-13)
    x4 = oracle.half_bits(oracle.half_values(x) * 4.0)
    out4, _ = oracle.rmsnorm_f64(x4, ones, 0.0)
    np.testing.assert_allclose(out4, out, rtol=1e-13)
    # the weight multiplies element-wise and is shared by the rows (not indexed by row)
    w = oracle.half_bits(rng.normal(1, 0.2, dim))
    outw, _ = oracle.rmsnorm_f64(x, w, eps)
    out1, _ = oracle.rmsnorm_f64(x, ones, eps)
    np.testing.assert_allclose(outw, out1 * oracle.half_values(w)[None, :], rtol=1e-13)
    # numpy restatement through the 2-norm: x * sqrt(dim) / sqrt(|x|^2 + dim*eps)
    xv = oracle.half_values(x)
    ref = xv * np.sqrt(dim) / np.sqrt(np.linalg.norm(xv, axis=1, keepdims=True) ** 2 + dim * eps)
    np.testing.assert_allclose(out1, ref, rtol=1e-13)


def test_rmsnorm_residual_path(oracle):
    dim, eps = 256, float(np.float32(1e-5))
    rng = np.random.default_rng(6)
    # values on a coarse grid: x + r is exact in fp16, so all three variants must coincide
    x = oracle.half_bits(rng.integers(-64, 64, (2, dim)) / 8.0)
    r = oracle.half_bits(rng.integers(-64, 64, (2, dim)) / 8.0)
    w = oracle.half_bits(rng.normal(1, 0.2, dim))
    summed = oracle.half_bits(oracle.half_values(x) + oracle.half_values(r))
    plain, _ = oracle.rmsnorm_f64(summed, w, eps)
    fused, ro = oracle.rmsnorm_f64(x, w, eps, residual=r, store_residual=True)
    nostore, none = oracle.rmsnorm_f64(x, w, eps, residual=r)
    assert none is None
    np.testing.assert_array_equal(ro, summed)
    np.testing.assert_allclose(fused, plain, rtol=1e-14)
    np.testing.assert_allclose(nostore, plain, rtol=1e-14)
    # inexact sums: the stored residual is the RNE fp16 of the fp32 sum; the statistic uses the
    # unrounded sum, the normalised value the rounded one
    x = oracle.half_bits(rng.normal(0, 1, (2, dim)))
    r = oracle.half_bits(rng.normal(0, 1, (2, dim)))
    t32 = oracle.half_values(x).astype(np.float32) + oracle.half_values(r).astype(np.float32)
    fused, ro = oracle.rmsnorm_f64(x, w, eps, residual=r, store_residual=True)
    np.testing.assert_array_equal(ro, t32.astype(np.float16).view(np.uint16))
    inv = 1.0 / np.sqrt((t32.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + eps)
    np.testing.assert_allclose(fused, oracle.half_values(ro) * inv * oracle.half_values(w), rtol=1e-13)
    nostore, _ = oracle.rmsnorm_f64(x, w, eps, residual=r)
    np.testing.assert_allclose(nostore, t32.astype(np.float64) * inv * oracle.half_values(w), rtol=1e-13)


def test_silu_mul_closed_forms(oracle):
    from scipy.special import expit
    rng = np.random.default_rng(7)
    g = rng.normal(0, 3, 1001).astype(np.float16)
    u = rng.normal(0, 1, 1001).astype(np.float16)
    one = np.ones_like(g)
    out = oracle.silu_mul_f64(g.view(np.uint16), u.view(np.uint16))
    gv, uv = g.astype(np.float64), u.astype(np.float64)
    np.testing.assert_allclose(out, gv * expit(gv) * uv, rtol=1e-13, atol=1e-300)
    # silu(0) = 0; silu(g) - silu(-g) = g; far right tail is the identity, far left tail vanishes
    assert oracle.silu_mul_f64(np.zeros(4, np.uint16), one[:4].view(np.uint16)).tolist() == [0.0] * 4
    sp = oracle.silu_mul_f64(g.view(np.uint16), one.view(np.uint16))
    sm = oracle.silu_mul_f64((-g).view(np.uint16), one.view(np.uint16))
    np.testing.assert_allclose(sp - sm, gv, rtol=1e-13, atol=1e-15)
    tail = oracle.silu_mul_f64(np.array([40.0, -40.0], np.float16).view(np.uint16),
                               np.array([2.0, 2.0], np.float16).view(np.uint16))
    assert tail[0] == pytest.approx(80.0, rel=1e-15) and abs(tail[1]) < 1e-15


def test_add_is_exact(oracle):
    rng = np.random.default_rng(11)
    a = rng.normal(0, 4, 2000).astype(np.float16)
    b = (rng.normal(0, 4, 2000) * 10.0 ** rng.integers(-6, 3, 2000)).astype(np.float16)
    out = oracle.add_f64(a.view(np.uint16), b.view(np.uint16))
    assert (out == a.astype(np.float64) + b.astype(np.float64)).all()
    # rounding the exact sum once is what an fp16 adder stores
    assert (oracle.half_bits(out) == (a + b).view(np.uint16)).all()


def test_rope_closed_forms(oracle):
    rng = np.random.default_rng(12)
    batch, seq, heads, hd = 2, 5, 3, 8
    x = rng.normal(0, 1, (batch, seq, heads, hd)).astype(np.float16)
    xv = x.astype(np.float64)
    # position 0: identity (only the first token of each batch entry when start_pos = 0)
    out = oracle.rope_f64(x.view(np.uint16), batch, seq, heads, hd, 0, 10000.0)
    assert (out[:, 0] == xv[:, 0]).all()
    # theta = 1: every pair turns by `pos` radians; (1, 0) -> (cos, sin) fixes sign and pair layout
    unit = np.zeros((1, 4, 1, 6), np.float16)
    unit[..., 0::2] = 1.0
    turned = oracle.rope_f64(unit.view(np.uint16), 1, 4, 1, 6, 3, 1.0)
    for s in range(4):
        for i in range(3):
            assert turned[0, s, 0, 2 * i] == pytest.approx(math.cos(3 + s), abs=1e-15)
            assert turned[0, s, 0, 2 * i + 1] == pytest.approx(math.sin(3 + s), abs=1e-15)
    # pair norms are preserved
    n_in = xv[..., 0::2] ** 2 + xv[..., 1::2] ** 2
    n_out = out[..., 0::2] ** 2 + out[..., 1::2] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-13)
    # start_pos shifts the sequence index: token s at start 7 == token 0 at start 7 + s
    a = oracle.rope_f64(x.view(np.uint16), batch, seq, heads, hd, 7, 500000.0)
    for s in range(seq):
        one = oracle.rope_f64(np.ascontiguousarray(x[:, s:s + 1]).view(np.uint16), batch, 1, heads, hd, 7 + s, 500000.0)
        assert (a[:, s:s + 1] == one).all()
    # complex-exponential restatement: (x0 + i x1) * exp(i * pos * theta^(-2i/hd))
    theta, start = 500000.0, 7
    pos = (start + np.arange(seq))[None, :, None, None]
    freq = theta ** (-2.0 * np.arange(hd // 2) / hd)
    z = (xv[..., 0::2] + 1j * xv[..., 1::2]) * np.exp(1j * pos * freq)
    np.testing.assert_allclose(a[..., 0::2], z.real, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(a[..., 1::2], z.imag, rtol=1e-12, atol=1e-14)


def test_embedding_and_kv_copy_index_arithmetic(oracle):
    rng = np.random.default_rng(13)
    table = rng.integers(0, 65536, (11, 6)).astype(np.uint16)
    idx = np.array([3, 0, 10, 3], np.int32)
    got = oracle.embedding_lookup(table, idx)
    for t, i in enumerate(idx):
        assert (got[t] == table[i]).all()
    batch, seq, heads, hd, max_seq = 2, 3, 2, 4, 6
    k = rng.integers(0, 65536, (batch, seq, heads, hd)).astype(np.uint16)
    v = rng.integers(0, 65536, (batch, seq, heads, hd)).astype(np.uint16)
    kc0 = rng.integers(0, 65536, (batch, heads, max_seq, hd)).astype(np.uint16)
    vc0 = rng.integers(0, 65536, (batch, heads, max_seq, hd)).astype(np.uint16)
    for start in (0, 2, 4, 5, 6):  # 4 and 5 run past the end of the cache, 6 is wholly outside
        kc, vc = oracle.copy_to_kv_cache(k, v, kc0, vc0, start)
        for b in range(batch):
            for h in range(heads):
                for p in range(max_seq):
                    s = p - start
                    inside = 0 <= s < seq
                    assert (kc[b, h, p] == (k[b, s, h] if inside else kc0[b, h, p])).all()
                    assert (vc[b, h, p] == (v[b, s, h] if inside else vc0[b, h, p])).all()


def test_rope_fp32_angle_restatement(oracle):
    """tllm_oracle_rope_f32angle restates the reference's fp32 arithmetic (kernels/rope.cu:49-64). Pinned by:
    position 0 is the identity (cos 0 = 1, sin 0 = 0: the fp16 inputs come back bit for bit); theta = 1 makes
    every frequency exactly 1, so the fp32 angle is exact for integer positions below 2^24 and the result must
    equal the exact-angle rotation up to fp32 sine/cosine and fp16 rounding; and in general it stays within
    pos * 2^-22 rad of the exact-angle rotation (the fp32 product pos * freq and powf are each good to an ulp)."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 4, 64)).astype(np.float16)
    xb = x.view(np.uint16)
    same = oracle.rope_f32angle(xb, 2, 3, 4, 64, 0, 10000.0)
    assert np.array_equal(same[:, 0], xb[:, 0])                      # tokens at position 0
    norm = np.sqrt((x.astype(np.float64).reshape(2, 3, 4, 32, 2) ** 2).sum(-1)).repeat(2, -1).reshape(x.shape)
    for pos, theta in ((1234, 1.0), (8191, 1.0), (1234, 10000.0), (8191, 500000.0), (100000, 500000.0)):
        exact = oracle.rope_f64(xb, 2, 3, 4, 64, pos, theta)
        ref32 = oracle.rope_f32angle(xb, 2, 3, 4, 64, pos, theta).view(np.float16).astype(np.float64)
        slack = (0.0 if theta == 1.0 else (pos + 2) * 2.0 ** -22) + 2.0 ** -10
        assert (np.abs(ref32 - exact) <= slack * norm + 1e-7).all(), (pos, theta, float(np.abs(ref32 - exact).max()))
