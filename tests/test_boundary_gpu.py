"""The drop-in boundary on the GPU: the C++ interface with real device buffers (the way the reference's own
callers and tests use it), and the places where a matrix-core kernel could part from the reference, pinned by
tests: where Inf / NaN activations go (only to the rows the reference poisons), the dynamic range of one activation
vector (outliers of any size), and how far the exact-angle RoPE is from the reference's fp32-angle arithmetic."""
import os
import struct
import subprocess

import numpy as np
import pytest

from tests import synth

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "bin", "dropin_device")


def build_dropin_device():
    """g++ + the HIP runtime API, a plain host translation unit (what src/transformer.cpp is). Built by
    __graft_entry__.build(); built here only if that binary is missing."""
    import ternary_llm_amd as tl
    libdir = os.path.dirname(tl.lib_path())
    os.makedirs(os.path.dirname(EXE), exist_ok=True)
    cmd = ["g++", "-std=c++17", "-O1", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "dropin_device.cpp"), "-L", libdir, "-ltllm_ternary", "-L", "/opt/rocm/lib", "-lamdhip64",
           f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib", "-o", EXE]
    subprocess.run(cmd, check=True, capture_output=True, text=True)


@pytest.fixture(scope="module")
def dev():
    import torch
    import ternary_llm_amd as tl
    assert torch.cuda.is_available(), "these tests need the MI355X"
    tl.lib()
    return torch, tl


def _up(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).cuda()


@pytest.mark.parametrize("rows,cols,M", [(300, 1536, 40), (4096, 4096, 7), (1000, 11008, 130)])
def test_cpp_interface_with_device_buffers(oracle, tmp_path, rows, cols, M):
    """ternary::ternary_gemv / ternary_gemm / quantize_absmax_int8 / ternary_gemv_int8 called from C++ through
    include/ternary_kernels.hpp on hipMalloc'ed buffers (reference tests/test_ternary_gemv.cu:122-161,
    src/transformer.cpp:102-142); outputs against the oracle; a call the reference would truncate silently is
    rejected and shows in ternary::last_error()."""
    if not os.path.exists(EXE):
        build_dropin_device()
    nz, sg, s, x = synth.problem(rows + cols + M, rows, cols, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M), M, cols)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(struct.pack("<3i", rows, cols, M))
        for a in (nz, sg, s.view(np.uint16), x.view(np.uint16), A.view(np.uint16)):
            f.write(np.ascontiguousarray(a).tobytes())
    run = subprocess.run([EXE, str(fin), str(fout)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    raw = open(fout, "rb").read()
    o = 0
    y = np.frombuffer(raw, np.float16, rows, o); o += 2 * rows
    Cm = np.frombuffer(raw, np.float16, M * rows, o).reshape(M, rows); o += 2 * M * rows
    q = np.frombuffer(raw, np.int8, cols, o); o += cols
    scale = np.frombuffer(raw, np.float32, 1, o)[0]; o += 4
    yi = np.frombuffer(raw, np.float16, rows, o); o += 2 * rows
    before, rejected = struct.unpack_from("<2i", raw, o)
    sb, xb = s.view(np.uint16), x.view(np.uint16)
    for name, got, ref in (("gemv", y, oracle.gemv_f64(nz, sg, sb, xb)),
                           ("gemm", Cm, oracle.gemm_f64(A.view(np.uint16), nz, sg, sb))):
        assert np.isfinite(got).all()
        rep = oracle.error_report(got.astype(np.float64), ref)
        assert rep["max_rel"] <= 1e-3, f"C++ {name}: {rep}"
    qo, so = oracle.quantize_i8(xb)
    assert np.array_equal(q, qo) and scale == so, "C++ quantize_absmax_int8 differs from the oracle"
    rep = oracle.error_report(yi.astype(np.float64), oracle.gemv_i8_f64(nz, sg, sb, qo, np.float32(so)))
    assert rep["max_rel"] <= 1e-3, f"C++ gemv_int8: {rep}"
    assert before == 0 and rejected == -3, (before, rejected)       # TLLM_ERR_BAD_GROUP, reported, not silent
    # the rejected call left the output untouched: y above was read before it, the int8 result after it is intact


def test_inf_nan_activations_reach_only_the_rows_the_reference_poisons(dev, oracle):
    """Reference kernels/ternary_gemv.cu:65-72 adds x[k] only where a weight bit is set: a NaN (or Inf) at column
    k reaches the rows with w[r, k] != 0 and no others. The decode kernels meet the activations in a matrix
    multiply, where 0 * NaN would be NaN for every row; they therefore keep non-finite (and outlier) activations
    out of the operand image and add them term by term to the rows that hold a weight on the column. Rows with
    a weight there are non-finite as in the reference; every other row is finite and keeps the 1e-3 bar against
    the evaluation without that column. The same for one activation row of a batch (2..16 rows)."""
    torch, tl = dev
    rows, cols, k = 512, 4096, 1000
    nz, sg, s, x = synth.problem(77, rows, cols)
    w = synth.unpack_np(nz, sg)
    hit = w[:, k] != 0
    assert 0.3 < (~hit).mean() < 0.55
    x0 = x.copy()
    x0[k] = 0
    ref0 = oracle.gemv_f64(nz, sg, s.view(np.uint16), x0.view(np.uint16))
    for bad in (np.float16(np.nan), np.float16(np.inf), np.float16(-np.inf)):
        xb = x.copy()
        xb[k] = bad
        y = torch.zeros(rows, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(_up(torch, nz), _up(torch, sg), _up(torch, s), _up(torch, xb), y, rows, cols, 128)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert (~np.isfinite(got[hit])).all(), "rows with a weight on the bad column must be non-finite (as in the reference)"
        if np.isinf(bad):   # the sign of the infinity follows the weight
            assert (np.sign(got[hit].astype(np.float64)) == np.sign(float(bad)) * w[hit, k]).all()
        assert np.isfinite(got[~hit]).all(), "rows without a weight on the bad column must stay finite (as in the reference)"
        rep = oracle.error_report(got[~hit].astype(np.float64), ref0[~hit])
        assert rep["max_rel"] <= 1e-3, rep
    for M, bad_row in ((4, 2), (16, 11), (3, 0)):
        A = synth.acts_f16(np.random.default_rng(3 + M), M, cols)
        A[bad_row, k] = np.float16(np.nan)
        Cm = torch.zeros((M, rows), dtype=torch.float16, device="cuda")
        tl.ternary_gemm(_up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s), Cm, M, rows, cols, 128)
        torch.cuda.synchronize()
        got = Cm.cpu().numpy()
        good = [m for m in range(M) if m != bad_row]
        assert np.isfinite(got[good]).all()
        assert (~np.isfinite(got[bad_row][hit])).all() and np.isfinite(got[bad_row][~hit]).all()
        A0 = A.copy()
        A0[bad_row, k] = 0
        ref = oracle.gemm_f64(A0.view(np.uint16), nz, sg, s.view(np.uint16))
        assert oracle.error_report(got[good].astype(np.float64), ref[good])["max_rel"] <= 1e-3
        assert oracle.error_report(got[bad_row][~hit].astype(np.float64), ref[bad_row][~hit])["max_rel"] <= 1e-3


@pytest.mark.parametrize("pos", [0, 1234, 8191])
def test_rope_distance_to_the_reference_fp32_angle(dev, oracle, pos):
    """tllm_rope_f16 forms the angle in fp64; the reference in fp32 (kernels/rope.cu:51-55), which leaves its angle
    off by up to about pos * 2^-23 rad. The kernel must stay within that distance (plus fp16 rounding of both
    results) of the reference's arithmetic, restated on the CPU: at position 0 the two agree bit for bit, at
    position 8191 they may differ by about 1e-3 of a pair's length."""
    torch, tl = dev
    batch, seq, heads, kv, hd, theta = 1, 3, 8, 2, 128, 500000.0
    rng = np.random.default_rng(pos)
    q = rng.standard_normal((batch, seq, heads, hd)).astype(np.float16)
    k = rng.standard_normal((batch, seq, kv, hd)).astype(np.float16)
    dq, dk = _up(torch, q.view(np.uint16).view(np.int16)).view(torch.float16), _up(torch, k.view(np.uint16).view(np.int16)).view(torch.float16)
    tl.rope(dq, dk, batch, seq, heads, kv, hd, pos, theta)
    torch.cuda.synchronize()
    for name, x, got, h in (("q", q, dq.cpu().numpy(), heads), ("k", k, dk.cpu().numpy(), kv)):
        ref32 = oracle.rope_f32angle(x.view(np.uint16), batch, seq, h, hd, pos, theta).view(np.float16)
        norm = np.sqrt((x.astype(np.float64).reshape(batch, seq, h, hd // 2, 2) ** 2).sum(-1)).repeat(2, -1).reshape(x.shape)
        diff = np.abs(got.astype(np.float64) - ref32.astype(np.float64))
        if pos == 0:
            assert np.array_equal(got[:, 0].view(np.uint16), ref32[:, 0].view(np.uint16)), name
        assert (diff <= ((pos + seq + 2) * 2.0 ** -22 + 2.0 ** -9) * norm + 1e-7).all(), (name, pos, float((diff / (norm + 1e-9)).max()))


def test_activation_dynamic_range_of_one_vector(dev, oracle):
    """The decode kernels (1 to 16 activation rows) feed the matrix cores the codes w + 1 in {0, 1, 2} and take the
    "+1" out again by subtracting the product of an all-zero weight row, both accumulated in fp32: what is in the
    operand image costs a row about 2^-21 of the largest magnitude of its 128-column group. Every group is
    normalised by itself, and an activation more than 2^8 times the typical magnitude of its group stays out of the
    image and is added term by term, as the reference adds it (kernels/ternary_gemv.cu:60-82): rows with a weight on
    an outlier column are dominated by it, rows without one must keep the 1e-3 bar against THEIR OWN magnitude
    whatever the outlier's size (2^8 ... 2^23 times the typical element checked here). The prefill GEMM (M > 16)
    decodes signed weights and is not affected."""
    torch, tl = dev
    rows, cols, k = 256, 4096, 77
    nz, sg, s, _ = synth.problem(901, rows, cols)
    w = synth.unpack_np(nz, sg)
    hit = w[:, k] != 0
    rng = np.random.default_rng(902)
    base = (rng.standard_normal(cols) * 2.0 ** -8).astype(np.float16)

    def errors(M, ratio_log2):
        A = np.tile(base, (M, 1))
        A[:, k] = np.float16(2.0 ** (ratio_log2 - 8))
        out = torch.zeros((M, rows), dtype=torch.float16, device="cuda")
        if M == 1:
            tl.ternary_gemv(_up(torch, nz), _up(torch, sg), _up(torch, s), _up(torch, A[0]), out, rows, cols, 128)
        else:
            tl.ternary_gemm(_up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s), out, M, rows, cols, 128)
        torch.cuda.synchronize()
        got = out.cpu().numpy().astype(np.float64)[M - 1]
        ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), A[M - 1].view(np.uint16))
        tau = np.sqrt(np.mean(ref[~hit] ** 2)) / 64.0          # floor from the rows WITHOUT the outlier
        rel = np.abs(got - ref) / np.maximum(np.abs(ref), tau)
        return rel[hit].max(), rel[~hit].max()

    for M in (1, 2, 4, 16, 64):
        for ratio in (7, 8, 9, 12, 16, 20, 23):
            with_outlier, without = errors(M, ratio)
            assert with_outlier <= 1e-3 and without <= 1e-3, (M, ratio, with_outlier, without)


def _outlier_case(seed, rows, cols, batch, n_out, ratio_log2):
    """Weights, activations with n_out outliers per activation row (magnitude 2^ratio_log2 times the typical element,
    random sign, random columns), the fp64 evaluation, and the error floor of the rows that hold no weight on any
    outlier column of their activation row."""
    nz, sg, s, _ = synth.problem(seed, rows, cols, dontcare_sign=True)
    w = synth.unpack_np(nz, sg)
    rng = np.random.default_rng(seed + 1)
    A = (rng.standard_normal((batch, cols)) * 2.0 ** -6).astype(np.float16)
    free = np.ones((batch, rows), bool)
    for b in range(batch):
        ks = rng.choice(cols, size=n_out, replace=False)
        A[b, ks] = (rng.choice([-1.0, 1.0], n_out) * 2.0 ** (ratio_log2 - 6)).astype(np.float16)
        free[b] = (w[:, ks] == 0).all(axis=1)
    return nz, sg, s, A, free


def _check_outliers(oracle, got, A, nz, sg, s, free, what):
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    for b in range(A.shape[0]):
        f = free[b]
        assert f.sum() >= 4, f"{what}: the case needs rows without a weight on any outlier column"
        tau = np.sqrt(np.mean(ref[b][f] ** 2)) / 64.0
        rel = np.abs(got[b] - ref[b]) / np.maximum(np.abs(ref[b]), tau)
        assert rel[f].max() <= 1e-3, (what, b, "rows without outliers", rel[f].max())
        assert oracle.error_report(got[b], ref[b])["max_rel"] <= 1e-3, (what, b)


@pytest.mark.parametrize("rows,cols,batch,n_out", [
    (300, 4096, 1, 3), (64, 28672, 1, 2),      # wide tiles: one segment, a row staged in segments
    (200, 14336, 3, 2), (130, 1152, 2, 1),     # tall tiles (plans of 2..4 rows run them; single calls: the batched kernel)
    (100, 8192, 16, 2), (520, 2048, 5, 3),     # the batched kernel
])
def test_outlier_activations_every_decode_path(dev, oracle, rows, cols, batch, n_out, tuned):
    """A few activations 2^14 times the typical one per activation row, on random columns: single calls (batch-1 kernel,
    batched kernel) and plans (wide tiles, tall tiles, batched kernel) keep the bar on the rows that hold no weight
    on them, and on all rows against the full evaluation."""
    torch, tl = dev
    nz, sg, s, A, free = _outlier_case(7000 + rows, rows, cols, batch, n_out, 14)
    dev_w = (_up(torch, nz), _up(torch, sg), _up(torch, s))
    out = torch.zeros((batch, rows), dtype=torch.float16, device="cuda")
    if batch == 1:
        tl.ternary_gemv(*dev_w, _up(torch, A[0]), out, rows, cols, 128)
    else:
        tl.ternary_gemm(_up(torch, A), *dev_w, out, batch, rows, cols, 128)
    torch.cuda.synchronize()
    _check_outliers(oracle, out.cpu().numpy().astype(np.float64), A, nz, sg, s, free, f"single call {rows}x{cols} b{batch}")
    tuned(tall_min_share_milli=0)          # small plans of 2..4 rows onto the tall tiles as well
    y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
    plan = tl.LinearPlan([(*dev_w, _up(torch, A), y, rows, cols, batch)])
    plan.launch()
    torch.cuda.synchronize()
    _check_outliers(oracle, y.cpu().numpy().astype(np.float64), A, nz, sg, s, free, f"plan {plan.kernel} {rows}x{cols} b{batch}")
    plan.close()


@pytest.mark.parametrize("batch", [1, 4, 16])
def test_more_outliers_than_the_list_holds(dev, oracle, batch):
    """100 elements per activation row at 2^11 times the typical magnitude: the list of a workgroup (64 entries in
    the batch-1 kernel, 128 for all activation rows together in the batched kernel) overflows, and the elements that
    find no room stay in the operand image. Nothing is lost or counted twice: every row stays within 4e-3 (an
    element inside the image costs the rows that hold no weight on it about 2^-21 of its magnitude; a hundred of
    them at this size are visible on the rows where they cancel), and the rows' own results are finite."""
    torch, tl = dev
    rows, cols = 192, 4096
    nz, sg, s, A, _ = _outlier_case(7100 + batch, rows, cols, batch, 100, 11)
    out = torch.zeros((batch, rows), dtype=torch.float16, device="cuda")
    if batch == 1:
        tl.ternary_gemv(_up(torch, nz), _up(torch, sg), _up(torch, s), _up(torch, A[0]), out, rows, cols, 128)
    else:
        tl.ternary_gemm(_up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s), out, batch, rows, cols, 128)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    rep = oracle.error_report(got, ref)
    assert rep["max_rel"] <= 4e-3, rep


def test_outliers_through_swiglu_pair_and_rmsnorm_prologue(dev, oracle):
    """The fused launches see the same list: a SwiGLU pair and an RMSNorm prologue on a vector with two huge channels
    give the bits of the separate operators (rmsnorm, two projections, silu_mul)."""
    torch, tl = dev
    rows, cols = 1024, 4096
    rng = np.random.default_rng(7200)
    x = (rng.standard_normal((1, cols)) * 0.5).astype(np.float16)
    x[0, [100, 3000]] = [900.0, -2500.0]
    wn = (rng.standard_normal(cols) * 0.1 + 1.0).astype(np.float16)
    g = synth.problem(7201, rows, cols, dontcare_sign=True)[:3]
    u = synth.problem(7202, rows, cols, dontcare_sign=True)[:3]
    dg, du = tuple(_up(torch, a) for a in g), tuple(_up(torch, a) for a in u)
    dx, dwn = _up(torch, x), _up(torch, wn)
    eps = 1e-5
    fused = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
    plan = tl.LinearPlan([(*dg, dx, fused, rows, cols, 1, tl.SWIGLU_GATE), (*du, dx, None, rows, cols, 1)],
                         norm_weights=[dwn, dwn], eps=eps)
    plan.launch()
    xn = torch.empty_like(dx)
    tl.rmsnorm(dx, dwn, xn, None, None, 1, cols, eps)
    yg = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
    yu = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
    tl.ternary_gemv(*dg, xn, yg, rows, cols, 128)
    tl.ternary_gemv(*du, xn, yu, rows, cols, 128)
    tl.silu_mul(yg, yu, yg, rows)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int16), yg.view(torch.int16))
    xn_h = xn.cpu().numpy()
    refg = oracle.gemv_f64(g[0], g[1], g[2].view(np.uint16), xn_h[0].view(np.uint16))
    tl.ternary_gemv(*dg, xn, yu, rows, cols, 128)
    torch.cuda.synchronize()
    assert oracle.error_report(yu.cpu().numpy().astype(np.float64)[0], refg)["max_rel"] <= 1e-3
    plan.close()
