"""GPU parity tests: every operator is called through the C ABI (ctypes -> libtllm_ternary.so)
and compared with the CPU oracle on the same seeded inputs.

Bar: max_i |y_i - ref_i| / max(|ref_i|, tau) <= 1e-3 with tau = 2^-6 * rms(ref), against the
fp64 evaluation of the same packed weights, fp16-rounded scales and activations; bit-exact
for the integer work (int8 quantisation).
"""
import json
import os

import numpy as np
import pytest

from tests import synth

pytestmark = pytest.mark.gpu

TOL = 1e-3
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def dev():
    import torch
    import ternary_llm_amd as tl
    assert torch.cuda.is_available(), "these tests need the MI355X"
    tl.lib()
    return torch, tl


def up(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    if a.dtype == np.uint16:
        a = a.view(np.float16)
    return torch.from_numpy(a).cuda()


def run_gemv(dev, nz, sg, s, x, group=128):
    torch, tl = dev
    rows, words = nz.shape
    y = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemv(up(torch, nz), up(torch, sg), up(torch, s), up(torch, x), y, rows, words * 32, group)
    torch.cuda.synchronize()
    return y.cpu().numpy().astype(np.float64)


def run_gemm(dev, A, nz, sg, s, group=128):
    torch, tl = dev
    N, words = nz.shape
    M = A.shape[0]
    Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemm(up(torch, A), up(torch, nz), up(torch, sg), up(torch, s), Cm, M, N, words * 32, group)
    torch.cuda.synchronize()
    return Cm.cpu().numpy().astype(np.float64)


def assert_close(oracle, got, ref, tol=TOL, what=""):
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    rep = oracle.error_report(got, ref)
    assert rep["max_rel"] <= tol, f"{what}: {rep}"


class gemm_forced:
    """Forces the GEMM kernel choice through the library's tuning switch (tllm_debug_set_tuning):
    gemm_forced(rowsplit=1) / (rowsplit=2) the row-split kernel in its eight-wave / four-wave form wherever the shape
    allows, gemm_forced(rowsplit=0) the four-wave kernel, gemm_forced() the library's own choice. The switch is put
    back on exit."""

    def __init__(self, rowsplit=-1):
        self.want = {"gemm_rowsplit": int(rowsplit)}

    def __enter__(self):
        import ternary_llm_amd as tl
        self.ctx = tl.tuning(**self.want)
        self.ctx.__enter__()
        return self

    def __exit__(self, *exc):
        return self.ctx.__exit__(*exc)


# -------------------------------------------------------------------- GEMV
@pytest.mark.parametrize("rows,cols,seed", [
    (2048, 2048, 101),    # benchmark configuration 1 (LLaMA-1B q_proj)
    (512, 2048, 102),     # 1B k/v_proj
    (2048, 8192, 103),    # 1B down_proj
    (1024, 4096, 104),    # 8B k/v_proj
    (256, 14336, 105),    # 8B down_proj row slice (K = 112 groups)
    (64, 28672, 106),     # 70B down_proj row slice (K = 224 groups)
])
def test_gemv_baseline_shapes(dev, oracle, rows, cols, seed):
    nz, sg, s, x = synth.problem(seed, rows, cols, dontcare_sign=True)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    assert_close(oracle, run_gemv(dev, nz, sg, s, x), ref, what=f"gemv {rows}x{cols}")


@pytest.mark.parametrize("rows,cols", [(1024, 1024), (4096, 4096), (4096, 11008)])
def test_gemv_reference_test_recipe(dev, oracle, rows, cols):
    """The data recipe of the reference's tests/test_ternary_gemv.cu:98-113: independent uniform
    random words for nz AND sign, scales U(-0.1,0.1) (negative allowed), x U(-1,1)."""
    rng = np.random.default_rng(rows + cols)
    nz = rng.integers(0, 2**32, (rows, cols // 32), dtype=np.uint64).astype(np.uint32)
    sg = rng.integers(0, 2**32, (rows, cols // 32), dtype=np.uint64).astype(np.uint32)
    s = rng.uniform(-0.1, 0.1, (rows, cols // 128)).astype(np.float16)
    x = rng.uniform(-1, 1, cols).astype(np.float16)
    got = run_gemv(dev, nz, sg, s, x)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    assert_close(oracle, got, ref, what=f"gemv ref-recipe {rows}x{cols}")
    # and the reference's own pass criterion against its fp32 host loop (tol 1e-2, rel-or-abs)
    loop = oracle.gemv_hostloop(nz, sg, s.astype(np.float32), x.astype(np.float32)).astype(np.float64)
    err = np.abs(got - loop)
    rel = np.where(np.abs(loop) > 1e-6, err / np.maximum(np.abs(loop), 1e-30), err)
    assert rel.max() < 1e-2 or err.max() < 1e-2


@pytest.mark.parametrize("rows,cols", [(1, 128), (3, 256), (17, 384), (100, 1152), (65, 640), (1, 4096), (15, 128),
                                       # wide tiles in units of 16 rows: row counts that end inside a tile,
                                       # a unit or a chunk, rows that are not whole slices of 2048 columns
                                       (16, 2048), (17, 2048), (33, 4096), (100, 2048), (70, 6144), (16, 14336),
                                       (50, 11008), (47, 2176), (49, 8192), (18433, 2048), (20000, 2048)])
def test_gemv_ragged_shapes(dev, oracle, rows, cols):
    nz, sg, s, x = synth.problem(rows * 7 + cols, rows, cols, dontcare_sign=True)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    assert_close(oracle, run_gemv(dev, nz, sg, s, x), ref, what=f"gemv {rows}x{cols}")


@pytest.mark.parametrize("rows,cols", [(64, 28672), (3000, 18432), (200, 16512), (96, 57344), (50, 36992),
                                       (2100, 28672), (16, 16384 + 2048), (20000, 18432)])
def test_gemv_rows_staged_in_segments(dev, oracle, rows, cols):
    """Rows longer than eight slices of 2048 columns: the operand image holds one segment of the row
    at a time (whole and ragged last slices, one and several tasks per workgroup, up to four segments)."""
    nz, sg, s, x = synth.problem(rows * 3 + cols, rows, cols, dontcare_sign=True)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    assert_close(oracle, run_gemv(dev, nz, sg, s, x), ref, what=f"gemv {rows}x{cols}")


def test_plan_mixing_segmented_and_short_rows(dev, oracle):
    """One plan with long rows (two and three segments), short rows and a SwiGLU pair over long rows;
    several tasks per problem, so segments are restaged between tasks of one problem."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    shapes = [(5000, 28672), (1024, 4096), (2500, 36864), (4096, 2048), (700, 18560)]
    problems, keep = [], []
    for rows, cols in shapes:
        w = _rand_weight(torch, gen, rows, cols)
        x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
        problems.append((*w, x, y, rows, cols, 1))
        keep.append((w, x, y))
    rows, cols = 3000, 20480
    g_w, u_w = _rand_weight(torch, gen, rows, cols), _rand_weight(torch, gen, rows, cols)
    xp = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
    fused = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
    problems += [(*g_w, xp, fused, rows, cols, 1, tl.SWIGLU_GATE), (*u_w, xp, None, rows, cols, 1)]
    plan = tl.LinearPlan(problems)
    for _ in range(2):  # the second launch finds the counters as the first one left them
        plan.launch()
    torch.cuda.synchronize()
    pick_rng = np.random.default_rng(5)
    for (w, x, y), (r, c) in zip(keep, shapes):
        single = torch.zeros(r, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(*w, x, single, r, c, 128)
        torch.cuda.synchronize()
        assert torch.isfinite(y).all()
        pick = pick_rng.integers(0, r, 96)
        ref = oracle.gemv_f64(w[0][pick].cpu().numpy().view(np.uint32), w[1][pick].cpu().numpy().view(np.uint32),
                              w[2][pick].cpu().numpy().view(np.uint16), x[0].cpu().numpy().view(np.uint16))
        assert_close(oracle, y[0][pick].cpu().numpy().astype(np.float64), ref, what=f"plan {r}x{c}")
        assert_close(oracle, single[pick].cpu().numpy().astype(np.float64), ref, what=f"single {r}x{c}")
    g = torch.zeros(rows, dtype=torch.float16, device="cuda")
    u = torch.zeros(rows, dtype=torch.float16, device="cuda")
    tl.ternary_gemv(*g_w, xp, g, rows, cols, 128)
    tl.ternary_gemv(*u_w, xp, u, rows, cols, 128)
    unfused = torch.empty_like(g)
    tl.silu_mul(g, u, unfused, rows)
    torch.cuda.synchronize()
    assert torch.equal(fused[0].view(torch.int16), unfused.view(torch.int16))
    plan.close()


def test_gemv_special_matrices(dev, oracle):
    rng = np.random.default_rng(5)
    cols = 1024
    x = synth.acts_f16(rng, cols)
    s = np.ones((4, cols // 128), np.float16)
    w = np.zeros((4, cols), np.int8)
    w[1], w[2] = 1, -1
    w[3, 777] = -1
    nz, sg = synth.pack_np(w)
    sg[0] = 0xFFFFFFFF  # sign bits under an all-zero row must not matter
    got = run_gemv(dev, nz, sg, s, x)
    xs = x.astype(np.float64).sum()
    assert got[0] == 0.0
    assert abs(got[1] - xs) <= 1e-3 * max(abs(xs), 1.0) and abs(got[2] + xs) <= 1e-3 * max(abs(xs), 1.0)
    assert got[3] == -float(x[777])
    # all-zero activations -> exactly zero
    nz, sg, s, _ = synth.problem(8, 32, 512)
    assert not run_gemv(dev, nz, sg, s, np.zeros(512, np.float16)).any()


def test_gemv_activation_range(dev, oracle):
    """Outliers and tiny activations (fp16 max-ish down to subnormals) keep the same bar."""
    nz, sg, s, x = synth.problem(77, 128, 2048, dontcare_sign=True)
    for scale_up, outlier in ((2.0 ** 13, 60000.0), (2.0 ** -12, 60000.0 * 2.0 ** -12), (2.0 ** -10, None)):
        xs = (x.astype(np.float64) * scale_up).astype(np.float16)
        if outlier is not None:
            xs[5] = np.float16(outlier)
        # keep the outputs inside fp16's normal range: tiny activations get larger weight scales
        ss = s if scale_up > 1 else (s.astype(np.float32) * 64).astype(np.float16)
        ref = oracle.gemv_f64(nz, sg, ss.view(np.uint16), xs.view(np.uint16))
        assert_close(oracle, run_gemv(dev, nz, sg, ss, xs), ref, what=f"gemv range x{scale_up}")


@pytest.mark.parametrize("group", [32, 64, 256])
def test_gemv_other_group_sizes(dev, oracle, group):
    nz, sg, s, x = synth.problem(group, 40, 1024, group=group)
    ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16), group)
    assert_close(oracle, run_gemv(dev, nz, sg, s, x, group), ref, what=f"gemv group {group}")


def test_gemv_sparsity_sweep(dev, oracle):
    for p0 in (0.0, 0.2, 0.7, 1.0):
        nz, sg, s, x = synth.problem(int(p0 * 10) + 300, 96, 4096, p_zero=p0, lo=0.005, hi=0.02)
        ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
        assert_close(oracle, run_gemv(dev, nz, sg, s, x), ref, what=f"gemv p0={p0}")


def _load_fixture(name):
    with open(os.path.join(GOLDEN, name)) as f:
        fx = json.load(f)
    nz = np.array([int(v, 16) for v in fx["nz"]], np.uint32).reshape(fx["rows"], fx["cols"] // 32)
    sg = np.array([int(v, 16) for v in fx["sign"]], np.uint32).reshape(nz.shape)
    s = np.array([int(v, 16) for v in fx["scales"]], np.uint16).reshape(fx["rows"], -1)
    x = np.array([int(v, 16) for v in fx["x"]], np.uint16).reshape(fx["batch"], fx["cols"])
    y = np.array([float.fromhex(v) for v in fx["y_f64"]]).reshape(fx["batch"], fx["rows"])
    return fx, nz, sg, s, x, y


def test_golden_fixtures_on_gpu(dev, oracle):
    for name in sorted(f for f in os.listdir(GOLDEN) if f.startswith("gemv_") and f.endswith(".json")):
        fx, nz, sg, s, x, y = _load_fixture(name)
        for b in range(fx["batch"]):
            assert_close(oracle, run_gemv(dev, nz, sg, s, x[b], fx["group"]), y[b], what=f"{name} gemv b{b}")
        assert_close(oracle, run_gemm(dev, x, nz, sg, s, fx["group"]), y, what=f"{name} gemm")


# -------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("M,N,K", [(2, 64, 256), (4, 1024, 4096), (5, 100, 1152), (16, 512, 2048),
                                   (33, 130, 640), (64, 256, 1024), (128, 384, 2048), (130, 200, 896),
                                   (130, 200, 2688), (300, 100, 3072), (257, 129, 5248)])  # K split unevenly
def test_gemm_vs_oracle(dev, oracle, M, N, K):
    nz, sg, s, _ = synth.problem(M * 1000 + N, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M + K), M, K)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    assert_close(oracle, run_gemm(dev, A, nz, sg, s), ref, what=f"gemm {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(600, 300, 640), (33, 128, 128), (257, 1000, 1152), (100, 129, 256), (512, 136, 384),
                                   (16, 64, 128), (1023, 260, 640)])  # K not a multiple of 512: these go to the GEMM kernels
def test_gemm_four_wave_kernel_edges(dev, oracle, M, N, K):
    """The four-wave kernel forced onto shapes with ragged edges: M not a multiple of 256 or of 32, N not a multiple
    of 128 or of 8 (the narrow store path), a single scale group, more tiles than CUs. Against the fp64 oracle, and
    against the library's own choice (the kernels differ only in the order of the fp32 additions)."""
    nz, sg, s, _ = synth.problem(M * 7 + N, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M + K + 5), M, K)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    with gemm_forced(rowsplit=0):
        got = run_gemm(dev, A, nz, sg, s)
    other = run_gemm(dev, A, nz, sg, s)
    assert_close(oracle, got, ref, what=f"four-wave gemm {M}x{N}x{K}")
    assert_close(oracle, other, ref, what=f"gemm as chosen {M}x{N}x{K}")
    assert_close(oracle, got, other, tol=2e-3, what=f"four-wave against the chosen kernel {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(600, 300, 640), (257, 1000, 1152), (512, 136, 384), (1023, 261, 896), (130, 200, 2688),
                                   (200, 301, 5248), (96, 17, 384)])
def test_gemm_row_split_kernel_last_half_block(dev, oracle, M, N, K):
    """K a multiple of 128 but not of 256: the row-split kernel runs the last 128 columns as a block whose upper mask
    words are zero. Scale rows then hold an odd number of groups (rows start on any halfword; 1023 x 261 and 96 x 17
    have an odd number of scales in all, which the four-wave kernel cannot fetch: the library then takes the row-split
    kernel by itself). Both forms, every output against the fp64 oracle, the last weight row and the last activation
    row included, and the same bits on every call."""
    torch, tl = dev
    nz, sg, s, _ = synth.problem(M * 3 + N + K, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M + K + 11), M, K)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    if (N * (K // 128)) % 2:
        assert "gemm_ns_kernel" in tl.gemm_kernel(M, N, K)
        assert_close(oracle, run_gemm(dev, A, nz, sg, s), ref, what=f"odd scale count, as chosen, {M}x{N}x{K}")
    for form in (1, 2):
        with gemm_forced(rowsplit=form):
            assert f"gemm_ns_kernel<4, {form}>" in tl.gemm_kernel(M, N, K)
            got = run_gemm(dev, A, nz, sg, s)
            again = run_gemm(dev, A, nz, sg, s)
        assert_close(oracle, got, ref, what=f"row-split gemm with a half block, form {form}, {M}x{N}x{K}")
        assert np.array_equal(got, again)


@pytest.mark.parametrize("M,N,K", [(600, 300, 768), (33, 130, 256), (257, 1000, 1280), (100, 129, 512), (1023, 260, 512),
                                   (128, 256, 256), (129, 257, 512), (16, 64, 256), (260, 300, 6144)])
def test_gemm_row_split_kernel_edges(dev, oracle, M, N, K):
    """The row-split kernel (chosen by itself for tall problems) forced onto shapes with ragged edges: M not a
    multiple of 128 or of 16, N not a multiple of 256 or of 8 (the narrow store path), a single block of 256 columns,
    tiles that are split along K (260 x 300 x 6144: six tiles in eight parts each). Against the fp64 oracle and against the
    four-wave kernel."""
    torch, tl = dev
    nz, sg, s, _ = synth.problem(M * 5 + N + K, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M + K + 9), M, K)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    with gemm_forced(rowsplit=0):
        other = run_gemm(dev, A, nz, sg, s)
    for form in (1, 2):  # eight waves with one weight fragment each / four waves with two
        with gemm_forced(rowsplit=form):
            name = tl.gemm_kernel(M, N, K)
            assert f"gemm_ns_kernel<4, {form}>" in name
            if K == 6144:  # six tiles on 256 CUs: the eight-wave form splits them along K
                assert ("K split" in name) == (form == 1)
            got = run_gemm(dev, A, nz, sg, s)
            again = run_gemm(dev, A, nz, sg, s)
        assert_close(oracle, got, ref, what=f"row-split gemm, form {form}, {M}x{N}x{K}")
        assert np.array_equal(got, again), "the row-split kernel must give the same bits on every call"
        assert_close(oracle, got, other, tol=2e-3, what=f"row-split form {form} against four-wave {M}x{N}x{K}")


@pytest.mark.parametrize("group,M", [(32, 3), (64, 20), (256, 5)])
def test_gemm_other_group_sizes(dev, oracle, group, M):
    """Group sizes the .tllm files do not use still give the reference's result (general kernel)."""
    nz, sg, s, _ = synth.problem(group + M, 72, 1024, group=group)
    A = synth.acts_f16(np.random.default_rng(group), M, 1024)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16), group)
    assert_close(oracle, run_gemm(dev, A, nz, sg, s, group), ref, what=f"gemm group {group}")


def test_gemm_prefill_shapes_sampled(dev, oracle):
    """8B gate/up and down shapes at M=16 and M=512; the oracle is evaluated on sampled output
    rows/columns (the full fp64 product would take minutes), every output is checked finite."""
    torch, tl = dev
    for (N, K) in ((14336, 4096), (4096, 14336)):
        nz, sg, s, _ = synth.problem(N + K, N, K)
        for M in (16, 512):
            A = synth.acts_f16(np.random.default_rng(M), M, K)
            got = run_gemm(dev, A, nz, sg, s)
            assert np.isfinite(got).all()
            rng = np.random.default_rng(M + N)
            ms = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
            ns = np.unique(np.concatenate([[0, N - 1], rng.integers(0, N, 300)]))
            ref = oracle.gemm_f64(A[ms].view(np.uint16), nz[ns], sg[ns], s[ns].view(np.uint16))
            assert_close(oracle, got[np.ix_(ms, ns)], ref, what=f"gemm {M}x{N}x{K}")


def test_gemm_rows_equal_gemv(dev, oracle):
    nz, sg, s, _ = synth.problem(61, 320, 1536)
    A = synth.acts_f16(np.random.default_rng(62), 7, 1536)
    Cm = run_gemm(dev, A, nz, sg, s)
    for m in range(7):
        yv = run_gemv(dev, nz, sg, s, A[m])
        ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), A[m].view(np.uint16))
        assert_close(oracle, Cm[m], ref, what=f"gemm row {m}")
        assert_close(oracle, yv, ref, what=f"gemv row {m}")


def test_gemm_split_k_repeatable_and_streams(dev, oracle):
    """Shapes with few weight tiles split K across workgroups (fp32 partial tiles exchanged through a
    per-stream workspace, summed in a fixed order): every repetition must give the same bits, the
    workspace must survive a change of shape, and two streams must not disturb each other."""
    torch, tl = dev
    cases = []
    for k, (M, N, K) in enumerate([(512, 1024, 4096), (130, 512, 2048), (512, 1024, 4096), (256, 256, 8192)]):
        nz, sg, s, _ = synth.problem(4000 + k, N, K)
        A = synth.acts_f16(np.random.default_rng(4100 + k), M, K)
        ref_rows = np.unique(np.random.default_rng(k).integers(0, M, 5))
        ref = oracle.gemm_f64(A[ref_rows].view(np.uint16), nz, sg, s.view(np.uint16))
        cases.append((M, N, K, up(torch, A), up(torch, nz), up(torch, sg), up(torch, s), ref_rows, ref))
    first = {}
    for rep in range(3):
        for k, (M, N, K, dA, dnz, dsg, ds, rows, ref) in enumerate(cases):
            Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            tl.ternary_gemm(dA, dnz, dsg, ds, Cm, M, N, K, 128)
            torch.cuda.synchronize()
            got = Cm.cpu().numpy()
            assert_close(oracle, got.astype(np.float64)[rows], ref, what=f"split-K {M}x{N}x{K} rep {rep}")
            if k in first:
                assert np.array_equal(got.view(np.uint16), first[k]), f"case {k} rep {rep}: bits changed"
            else:
                first[k] = got.view(np.uint16).copy()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for rep in range(4):
        for st, k in ((s1, 0), (s2, 3)):
            M, N, K, dA, dnz, dsg, ds, rows, ref = cases[k]
            Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            with torch.cuda.stream(st):
                tl.ternary_gemm(dA, dnz, dsg, ds, Cm, M, N, K, 128, stream=st)
            outs.append((k, Cm))
    torch.cuda.synchronize()
    for k, Cm in outs:
        assert np.array_equal(Cm.cpu().numpy().view(np.uint16), first[k]), f"two streams: case {k} differs"


# ---------------------------------------------------------- batched decode
@pytest.mark.parametrize("M,N,K", [(2, 16, 512), (3, 17, 512), (4, 4096, 14336 // 7), (4, 1000, 1536),
                                   (8, 300, 4096), (13, 255, 1024), (16, 256, 512), (16, 1031, 2048),
                                   (16, 64, 28672), (4, 512, 14336), (20, 272, 1024), (48, 100, 512)])
def test_batched_decode_vs_oracle(dev, oracle, M, N, K):
    """2..16 activation rows (and passes of 16 above that) on K a multiple of 512: block edges
    (N not a multiple of 16 or 256), long K, unused activation rows."""
    nz, sg, s, _ = synth.problem(M * 977 + N, N, K, dontcare_sign=True)
    A = synth.acts_f16(np.random.default_rng(M + K), M, K)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    assert_close(oracle, run_gemm(dev, A, nz, sg, s), ref, what=f"batched {M}x{N}x{K}")


def test_batched_decode_special_cases(dev, oracle):
    """Exact zeros for empty rows, rows of one kind, per-row activation ranges that differ by many
    orders of magnitude (every activation row and slice is normalised on its own), zero activation rows."""
    rng = np.random.default_rng(31)
    N, K, M = 96, 1024, 6
    w = synth.ternary_matrix(rng, N, K)
    w[0] = 0
    w[1] = 1
    w[2] = -1
    w[3, :] = 0
    w[3, 700] = -1
    nz, sg = synth.pack_np(w)
    s = synth.scales_f16(rng, N, K // 128, lo=1.0, hi=3.0)  # large scales: tiny activations still give normal fp16 outputs
    A = synth.acts_f16(rng, M, K).astype(np.float64)
    A[1] *= 1e-3
    A[2] *= 200.0
    A[3] = 0.0
    A[4, :512] = 0.0          # one all-zero slice
    A[5, 512:] *= 2.0 ** -10  # slices of very different magnitude in one row
    A = A.astype(np.float16)
    ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16))
    got = run_gemm(dev, A, nz, sg, s)
    assert np.all(got[:, 0] == 0.0) and np.all(got[3] == 0.0)
    for m in range(M):
        if m == 3:
            continue
        assert_close(oracle, got[m], ref[m], what=f"batched special row {m}")


def test_batched_plan_8b_layer_batch4_and_16(dev, oracle):
    """One LLaMA-3-8B-shaped layer (7 projections, rows cut to keep the oracle fast) as a plan at
    batch 2, 3, 4 and 16: sampled rows == oracle; at batch 16 the plan runs the kernel of the single
    call, so its output equals the single call's bit for bit, unless the single call shares out K among
    workgroups, which adds the fp32 sums in another order (up to 4 the plan takes the tall-tile kernel,
    which stages the 14336-column rows in segments)."""
    torch, tl = dev
    shapes = [(512, 4096), (128, 4096), (128, 4096), (512, 4096), (1800, 4096), (1800, 4096), (520, 14336)]
    for batch in (2, 3, 4, 16):
        probs, host = [], []
        for k, (rows, cols) in enumerate(shapes):
            nz, sg, s, _ = synth.problem(8100 + k, rows, cols)
            x = synth.acts_f16(np.random.default_rng(8200 + k + batch), batch, cols)
            y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
            probs.append((up(torch, nz), up(torch, sg), up(torch, s), up(torch, x), y, rows, cols, batch))
            host.append((nz, sg, s, x))
        plan = tl.LinearPlan(probs)
        for launch in range(2):
            for pr in probs:
                pr[4].fill_(float("nan"))
            plan.launch()
            torch.cuda.synchronize()
            for k, (pr, (nz, sg, s, x)) in enumerate(zip(probs, host)):
                got = pr[4].cpu().numpy()
                single = run_gemm(dev, x, nz, sg, s)
                if batch > 4 and "shared out" not in tl.gemm_kernel(batch, pr[5], pr[6]):
                    assert np.array_equal(got.astype(np.float64), single), f"batch {batch} problem {k}: plan != single call"
                rows_s = np.unique(np.random.default_rng(k).integers(0, nz.shape[0], 64))
                ref = oracle.gemm_f64(x.view(np.uint16), nz[rows_s], sg[rows_s], s[rows_s].view(np.uint16))
                assert_close(oracle, got.astype(np.float64)[:, rows_s], ref, what=f"batch {batch} problem {k}")
        plan.close()



@pytest.mark.parametrize("batch", [2, 3, 4])
def test_tall_tile_plan_with_batch_columns(dev, oracle, batch, tuned):
    """Plans of two to four activation rows on the tall-tile MFMA kernel (large plans take it by
    themselves; a small one is made to here): several batch columns in one operand image, rows of
    14336 and 36864 columns staged in segments, rows that are not whole slices, two launches."""
    torch, tl = dev
    tuned(tall_min_share_milli=0)
    shapes = [(700, 4096), (128, 4096), (1800, 4096), (520, 14336), (100, 36864), (300, 1152), (64, 512)]
    probs, host = [], []
    for k, (rows, cols) in enumerate(shapes):
        nz, sg, s, _ = synth.problem(9100 + k, rows, cols, dontcare_sign=True)
        x = synth.acts_f16(np.random.default_rng(9200 + k + batch), batch, cols)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((up(torch, nz), up(torch, sg), up(torch, s), up(torch, x), y, rows, cols, batch))
        host.append((nz, sg, s, x))
    plan = tl.LinearPlan(probs)
    assert plan.kernel == "tllm::gemv_mfma_kernel<Tall>"
    for launch in range(2):
        for pr in probs:
            pr[4].fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for k, (pr, (nz, sg, s, x)) in enumerate(zip(probs, host)):
            got = pr[4].cpu().numpy().astype(np.float64)
            rows_s = np.unique(np.random.default_rng(k).integers(0, nz.shape[0], 48))
            ref = oracle.gemm_f64(x.view(np.uint16), nz[rows_s], sg[rows_s], s[rows_s].view(np.uint16))
            assert np.isfinite(got).all()
            assert_close(oracle, got[:, rows_s], ref, what=f"tall plan batch {batch} problem {k}")
    plan.close()


def test_tall_tile_plan_in_fine_units(dev, oracle, tuned):
    """A plan of two activation rows sized so that the tall tiles run in units of 64 rows (a share
    per workgroup of more than 1.75 and less than 2 such units, i.e. less than one of the ordinary
    units of 128 rows): sampled rows against the oracle."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    batch, probs = 2, []
    for rows, cols in [(5600, 4096)] * 12 + [(9000, 14336)] * 6 + [(5600, 4096)] * 12:
        w = _rand_weight(torch, gen, rows, cols)
        x = torch.randn((batch, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((*w, x, y, rows, cols, batch))
    plan = tl.LinearPlan(probs)
    assert plan.kernel == "tllm::gemv_mfma_kernel<Tall, fine>", plan.kernel
    for launch in range(2):
        plan.launch()
    torch.cuda.synchronize()
    pick_rng = np.random.default_rng(7)
    for k in (0, 13, 16, 29):
        nz, sg, sc, x, y, rows, cols, b = probs[k]
        assert torch.isfinite(y).all()
        pick = pick_rng.integers(0, rows, 64)
        ref = oracle.gemm_f64(x.cpu().numpy().view(np.uint16), nz[pick].cpu().numpy().view(np.uint32),
                              sg[pick].cpu().numpy().view(np.uint32), sc[pick].cpu().numpy().view(np.uint16))
        assert_close(oracle, y[:, pick].cpu().numpy().astype(np.float64), ref, what=f"fine tall plan problem {k}")
    plan.close()


def test_tall_tile_plan_with_mixed_batch_sizes(dev, oracle, tuned):
    """One plan whose problems carry one to four activation rows each, on the tall-tile kernel: the
    segment length and the operand image depend on the problem's own batch size."""
    torch, tl = dev
    tuned(tall_min_share_milli=0)
    shapes = [(700, 4096, 1), (300, 14336, 3), (520, 8192, 4), (200, 36864, 2), (64, 512, 4), (900, 18432, 1)]
    probs, host = [], []
    for k, (rows, cols, batch) in enumerate(shapes):
        nz, sg, s, _ = synth.problem(9300 + k, rows, cols, dontcare_sign=True)
        x = synth.acts_f16(np.random.default_rng(9400 + k), batch, cols)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((up(torch, nz), up(torch, sg), up(torch, s), up(torch, x), y, rows, cols, batch))
        host.append((nz, sg, s, x))
    plan = tl.LinearPlan(probs)
    assert plan.kernel == "tllm::gemv_mfma_kernel<Tall>"
    for launch in range(2):
        plan.launch()
        torch.cuda.synchronize()
        for k, (pr, (nz, sg, s, x)) in enumerate(zip(probs, host)):
            got = pr[4].cpu().numpy().astype(np.float64)
            ref = oracle.gemm_f64(x.view(np.uint16), nz, sg, s.view(np.uint16))
            assert_close(oracle, got, ref, what=f"mixed-batch tall plan problem {k}")
    plan.close()


def test_tall_tile_plan_scales_on_any_halfword(dev, oracle, tuned):
    """The tall tiles fetch the four scales of a (row, slice) as one 8-byte load. The boundary asks
    for 2-byte alignment of a scale array only, and with an odd number of groups every second row
    starts on an odd halfword: arrays that begin one halfword past an aligned address, group counts
    of 9, 32 and 145, every output against the oracle."""
    torch, tl = dev
    tuned(tall_min_share_milli=0)
    batch = 3
    shapes = [(300, 1152), (520, 4096), (200, 18560), (64, 512)]
    probs, host = [], []
    for k, (rows, cols) in enumerate(shapes):
        nz, sg, s, _ = synth.problem(9500 + k, rows, cols, dontcare_sign=True)
        x = synth.acts_f16(np.random.default_rng(9600 + k), batch, cols)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        s_dev = up(torch, s)
        shifted = torch.zeros(s_dev.numel() + 1, dtype=s_dev.dtype, device="cuda")
        shifted[1:] = s_dev.reshape(-1)
        s_odd = shifted[1:].view(s_dev.shape)
        assert s_odd.data_ptr() % 4 == 2
        probs.append((up(torch, nz), up(torch, sg), s_odd, up(torch, x), y, rows, cols, batch))
        host.append((nz, sg, s, x, shifted))
    plan = tl.LinearPlan(probs)
    assert plan.kernel == "tllm::gemv_mfma_kernel<Tall>"
    plan.launch()
    torch.cuda.synchronize()
    for k, (pr, (nz, sg, s, x, _)) in enumerate(zip(probs, host)):
        got = pr[4].cpu().numpy().astype(np.float64)
        ref = oracle.gemm_f64(x.view(np.uint16), nz, sg, s.view(np.uint16))
        assert_close(oracle, got, ref, what=f"tall plan, shifted scales, problem {k}")
    plan.close()


# ------------------------------------------------------------- element-wise
def _half_out(oracle, ref):
    """fp16 rounding of an fp64 reference, as float64 (for a 1-ulp comparison)."""
    return np.asarray(ref, np.float64).astype(np.float16).astype(np.float64)


@pytest.mark.parametrize("batch,dim", [(1, 4096), (1, 2048), (3, 8192), (512, 4096), (2, 100), (1, 1), (5, 257),
                                       (2, 8), (3, 5120), (2, 8200)])
def test_rmsnorm_vs_oracle(dev, oracle, batch, dim):
    torch, tl = dev
    rng = np.random.default_rng(batch * 131 + dim)
    x = oracle.half_bits(rng.normal(0, 1.5, (batch, dim)))
    w = oracle.half_bits(rng.normal(1, 0.3, dim))
    eps = 1e-5
    ref, _ = oracle.rmsnorm_f64(x, w, eps)
    y = torch.full((batch, dim), float("nan"), dtype=torch.float16, device="cuda")
    tl.rmsnorm(up(torch, x), up(torch, w), y, None, None, batch, dim, eps)
    torch.cuda.synchronize()
    assert_close(oracle, y.cpu().numpy().astype(np.float64), ref, what=f"rmsnorm {batch}x{dim}")
    # in place, as a caller that normalises its own buffer would
    xin = up(torch, x)
    tl.rmsnorm(xin, up(torch, w), xin, None, None, batch, dim, eps)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(xin.cpu().numpy(), y.cpu().numpy())


@pytest.mark.parametrize("dim", [264, 2048, 4096, 6144, 16384])
@pytest.mark.parametrize("store", [False, True])
def test_rmsnorm_residual_vs_oracle(dev, oracle, store, dim):
    torch, tl = dev
    batch, eps = 7, 1e-6
    rng = np.random.default_rng(99 + dim)
    x = oracle.half_bits(rng.normal(0, 1, (batch, dim)))
    r = oracle.half_bits(rng.normal(0, 2, (batch, dim)))
    w = oracle.half_bits(rng.normal(1, 0.3, dim))
    ref, ro_ref = oracle.rmsnorm_f64(x, w, eps, residual=r, store_residual=store)
    y = torch.full((batch, dim), float("nan"), dtype=torch.float16, device="cuda")
    ro = torch.full((batch, dim), float("nan"), dtype=torch.float16, device="cuda") if store else None
    tl.rmsnorm(up(torch, x), up(torch, w), y, up(torch, r), ro, batch, dim, eps)
    torch.cuda.synchronize()
    assert_close(oracle, y.cpu().numpy().astype(np.float64), ref, what="rmsnorm+residual")
    if store:   # fp32 add then one fp16 rounding: bit-exact
        np.testing.assert_array_equal(ro.cpu().numpy().view(np.uint16), ro_ref)


def test_rmsnorm_closed_form_on_gpu(dev, oracle):
    torch, tl = dev
    dim = 4096
    x = torch.full((2, dim), 3.0, dtype=torch.float16, device="cuda")
    w = torch.ones(dim, dtype=torch.float16, device="cuda")
    y = torch.empty_like(x)
    tl.rmsnorm(x, w, y, None, None, 2, dim, 0.0)
    torch.cuda.synchronize()
    assert (y.cpu().numpy() == np.float16(1.0)).all()


@pytest.mark.parametrize("n", [1, 2, 255, 14336, 512 * 14336 + 1])
def test_silu_mul_vs_oracle(dev, oracle, n):
    torch, tl = dev
    rng = np.random.default_rng(n)
    g = oracle.half_bits(rng.normal(0, 3, n))
    u = oracle.half_bits(rng.normal(0, 1, n))
    ref = oracle.silu_mul_f64(g, u)
    gd, ud = up(torch, g), up(torch, u)
    out = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
    tl.silu_mul(gd, ud, out, n)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    assert_close(oracle, got, ref, what=f"silu_mul {n}")
    # the reference calls it in place on the gate buffer (src/transformer.cpp:285)
    tl.silu_mul(gd, ud, gd, n)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(gd.cpu().numpy(), out.cpu().numpy())
    if n > 2:   # buffers that start on an odd element (2-byte alignment only)
        gd = up(torch, g)
        out2 = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
        tl.silu_mul(gd[1:], ud[1:], out2[1:], n - 1)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out2.cpu().numpy()[1:], out.cpu().numpy()[1:])


def test_silu_mul_tails(dev, oracle):
    torch, tl = dev
    g = np.array([0.0, -0.0, 40.0, -40.0, 65504.0, -65504.0, 1.0], np.float16)
    u = np.array([5.0, 5.0, 2.0, 2.0, 1.0, 1.0, 1.0], np.float16)
    out = torch.full((7,), float("nan"), dtype=torch.float16, device="cuda")
    tl.silu_mul(up(torch, g), up(torch, u), out, 7)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    assert got[0] == 0 and got[1] == 0 and got[2] == 80.0 and got[3] == 0 and got[4] == 65504.0 and got[5] == 0
    assert got[6] == np.float64(np.float16(1.0 / (1.0 + np.exp(-1.0))))

@pytest.mark.parametrize("n", [1, 7, 8, 4096, 7 * 4096 + 3])
def test_add_bit_exact(dev, oracle, n):
    """fp16 residual add: equal, bit for bit, to the once-rounded exact sum; in place; odd start."""
    torch, tl = dev
    rng = np.random.default_rng(n)
    a = oracle.half_bits(rng.normal(0, 4, n))
    b = oracle.half_bits(rng.normal(0, 4, n) * 10.0 ** rng.integers(-6, 3, n))
    want = oracle.half_bits(oracle.add_f64(a, b))
    ad, bd = up(torch, a), up(torch, b)
    out = torch.zeros(n, dtype=torch.float16, device="cuda")
    tl.add(ad, bd, out, n)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), want)
    tl.add(ad, bd, ad, n)   # the reference adds into the residual buffer (src/transformer.cpp:253)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(ad.cpu().numpy().view(np.uint16), want)
    if n > 2:
        ad = up(torch, a)
        out2 = torch.zeros(n, dtype=torch.float16, device="cuda")
        tl.add(ad[1:], bd[1:], out2[1:], n - 1)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out2.cpu().numpy().view(np.uint16)[1:], want[1:])


@pytest.mark.parametrize("batch,seq,heads,kv_heads,hd,start,theta", [
    (1, 1, 32, 8, 128, 0, 500000.0),      # 8B decode step, first token
    (1, 1, 32, 8, 64, 1234, 500000.0),    # 1B decode step in mid-sequence
    (1, 1, 64, 8, 128, 8191, 500000.0),   # 70B decode at the end of an 8K context
    (1, 77, 32, 8, 128, 5, 10000.0),      # prefill of 77 tokens
    (2, 3, 2, 5, 6, 9, 10000.0),          # more kv heads than q heads, tiny head
])
def test_rope_vs_oracle(dev, oracle, batch, seq, heads, kv_heads, hd, start, theta):
    torch, tl = dev
    rng = np.random.default_rng(heads * hd + start)
    q = oracle.half_bits(rng.normal(0, 1, (batch, seq, heads, hd)))
    k = oracle.half_bits(rng.normal(0, 1, (batch, seq, kv_heads, hd)))
    ref_q = oracle.rope_f64(q, batch, seq, heads, hd, start, theta)
    ref_k = oracle.rope_f64(k, batch, seq, kv_heads, hd, start, theta)
    qd, kd = up(torch, q), up(torch, k)
    tl.rope(qd, kd, batch, seq, heads, kv_heads, hd, start, theta)
    torch.cuda.synchronize()
    got_q = qd.cpu().numpy().view(np.float16).astype(np.float64)
    got_k = kd.cpu().numpy().view(np.float16).astype(np.float64)
    # fp32 sine/cosine of the exactly formed angle and an fp32 rotation: 1e-3 of max(|ref|, tau) as
    # for the linears (a pair that rotates onto an axis leaves one small component)
    assert_close(oracle, got_q.reshape(-1), ref_q.reshape(-1), what="rope q")
    assert_close(oracle, got_k.reshape(-1), ref_k.reshape(-1), what="rope k")
    # tighter, normwise per pair: the rotation is good to fp16 rounding of the result
    err = np.hypot(got_q[..., 0::2] - ref_q[..., 0::2], got_q[..., 1::2] - ref_q[..., 1::2])
    nrm = np.hypot(ref_q[..., 0::2], ref_q[..., 1::2])
    assert (err <= 2.0 ** -10 * nrm + 1e-7).all()


def test_embedding_lookup_bit_exact(dev, oracle):
    torch, tl = dev
    rng = np.random.default_rng(3)
    for vocab, dim, n_tokens in ((1000, 2048, 1), (1000, 4096, 33), (50, 100, 7), (50, 8, 3)):
        table = rng.integers(0, 65536, (vocab, dim)).astype(np.uint16)
        idx = rng.integers(0, vocab, n_tokens).astype(np.int32)
        idx[0] = vocab - 1
        out = torch.zeros((n_tokens, dim), dtype=torch.float16, device="cuda")
        tl.embedding_lookup(up(torch, table), torch.from_numpy(idx).cuda(), out, n_tokens, dim)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), oracle.embedding_lookup(table, idx))


@pytest.mark.parametrize("batch,seq,heads,hd,start,max_seq", [
    (1, 1, 8, 128, 0, 64), (1, 1, 8, 64, 63, 64), (1, 40, 8, 128, 10, 64), (2, 5, 3, 6, 2, 8),
    (1, 10, 8, 128, 60, 64),   # runs past the end of the cache: the last 6 rows are dropped
    (1, 4, 2, 64, 64, 64),     # wholly outside: nothing is written
])
def test_copy_to_kv_cache_bit_exact(dev, oracle, batch, seq, heads, hd, start, max_seq):
    torch, tl = dev
    rng = np.random.default_rng(seq * 131 + start)
    k = rng.integers(0, 65536, (batch, seq, heads, hd)).astype(np.uint16)
    v = rng.integers(0, 65536, (batch, seq, heads, hd)).astype(np.uint16)
    kc = rng.integers(0, 65536, (batch, heads, max_seq, hd)).astype(np.uint16)
    vc = rng.integers(0, 65536, (batch, heads, max_seq, hd)).astype(np.uint16)
    want_k, want_v = oracle.copy_to_kv_cache(k, v, kc, vc, start)
    kcd, vcd = up(torch, kc), up(torch, vc)
    tl.copy_to_kv_cache(up(torch, k), up(torch, v), kcd, vcd, batch, heads, hd, seq, start, max_seq)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(kcd.cpu().numpy().view(np.uint16), want_k)
    np.testing.assert_array_equal(vcd.cpu().numpy().view(np.uint16), want_v)


# --------------------------------------------------------------- INT8 pair
@pytest.mark.parametrize("n", [1, 63, 2048, 4096, 14336, 28672])
def test_quantize_bit_exact(dev, oracle, n):
    torch, tl = dev
    rng = np.random.default_rng(n)
    x = synth.acts_f16(rng, n)
    if n > 8:
        x[3] = np.float16(0.5) * x[2]  # near-tie material
    q = torch.zeros(n, dtype=torch.int8, device="cuda")
    sc = torch.zeros(1, dtype=torch.float32, device="cuda")
    tl.quantize_absmax_int8(up(torch, x), q, sc, n)
    torch.cuda.synchronize()
    qo, so = oracle.quantize_i8(x.view(np.uint16))
    np.testing.assert_array_equal(q.cpu().numpy(), qo)
    assert sc.item() == so


def test_quantize_all_zero(dev, oracle):
    torch, tl = dev
    q = torch.ones(256, dtype=torch.int8, device="cuda")
    sc = torch.zeros(1, dtype=torch.float32, device="cuda")
    tl.quantize_absmax_int8(torch.zeros(256, dtype=torch.float16, device="cuda"), q, sc, 256)
    torch.cuda.synchronize()
    assert sc.item() == 1.0 and not q.cpu().numpy().any()


@pytest.mark.parametrize("rows,cols", [(1024, 1024), (4096, 4096), (300, 11008),
                                       (64, 28672), (96, 57344)])   # a whole long row in LDS; a row staged in segments
def test_gemv_int8(dev, oracle, rows, cols):
    torch, tl = dev
    nz, sg, s, x = synth.problem(rows + 3 * cols, rows, cols, dontcare_sign=True)
    d = [up(torch, a) for a in (nz, sg, s, x)]
    q = torch.zeros(cols, dtype=torch.int8, device="cuda")
    sc = torch.zeros(1, dtype=torch.float32, device="cuda")
    tl.quantize_absmax_int8(d[3], q, sc, cols)
    y1 = torch.zeros(rows, dtype=torch.float16, device="cuda")
    y2 = torch.zeros(rows, dtype=torch.float16, device="cuda")
    tl.ternary_gemv_int8(d[0], d[1], d[2], q, sc.item(), y1, rows, cols)   # host scale, as the reference
    tl.ternary_gemv_int8(d[0], d[1], d[2], q, sc, y2, rows, cols)          # device-resident scale
    torch.cuda.synchronize()
    ref = oracle.gemv_i8_f64(nz, sg, s.view(np.uint16), q.cpu().numpy(), np.float32(sc.item()))
    assert_close(oracle, y1.cpu().numpy().astype(np.float64), ref, what="gemv_i8")
    np.testing.assert_array_equal(y1.cpu().numpy(), y2.cpu().numpy())
    # against the fp16-activation oracle the reference's own int8 criterion applies
    # (tests/test_ternary_gemv.cu:270-271: max_rel < 5e-2 || max_abs < 5e-2)
    if cols > 11008:
        return   # the quantisation noise itself grows with sqrt(cols); the reference states the bound for its own sizes
    ref16 = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
    err = np.abs(y1.cpu().numpy().astype(np.float64) - ref16)
    rel = np.where(np.abs(ref16) > 1e-6, err / np.maximum(np.abs(ref16), 1e-30), err)
    assert rel.max() < 5e-2 or err.max() < 5e-2


# -------------------------------------------------------------------- plan
def test_linear_plan_matches_single_calls(dev, oracle):
    torch, tl = dev
    shapes = [(2048, 2048, 1), (512, 2048, 1), (512, 2048, 2), (100, 1152, 4), (8192, 2048, 1), (2048, 8192, 3), (1, 128, 1)]
    probs, refs = [], []
    for k, (rows, cols, batch) in enumerate(shapes):
        nz, sg, s, _ = synth.problem(900 + k, rows, cols, dontcare_sign=True)
        x = synth.acts_f16(np.random.default_rng(950 + k), batch, cols, unit_rms=True)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((up(torch, nz), up(torch, sg), up(torch, s), up(torch, x), y, rows, cols, batch))
        refs.append(oracle.gemm_f64(x.view(np.uint16), nz, sg, s.view(np.uint16)))
    plan = tl.LinearPlan(probs)
    want_bytes = sum(r * c // 32 * 8 + r * c // 128 * 2 for r, c, _ in shapes)
    assert plan.weight_bytes == want_bytes
    for _ in range(2):  # a second launch must give the same answer (no stale state)
        for p in probs:
            p[4].fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for p, ref, shp in zip(probs, refs, shapes):
            assert_close(oracle, p[4].cpu().numpy().astype(np.float64), ref, what=f"plan {shp}")
    plan.close()


def test_linear_plan_on_int8_activations(dev, oracle):
    """A plan whose problems read int8 activations and their device-resident scales (the reference's decode path,
    quantize_absmax_int8 + ternary_gemv_int8 per linear): every output must equal, bit for bit, what the single-call
    operator gives for that matrix, and agree with the oracle's integer arithmetic; a plan that mixes shapes the
    matrix-core kernel does not serve is rejected."""
    torch, tl = dev
    shapes = [(2048, 2048), (512, 2048), (2048, 8192), (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]
    probs, scales, refs = [], [], []
    for k, (rows, cols) in enumerate(shapes * 3):
        nz, sg, s, x = synth.problem(8100 + k, rows, cols, unit_rms=True)
        dx = up(torch, x)
        q = torch.zeros(cols, dtype=torch.int8, device="cuda")
        qs = torch.zeros(1, dtype=torch.float32, device="cuda")
        tl.quantize_absmax_int8(dx, q, qs, cols)
        y = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((up(torch, nz), up(torch, sg), up(torch, s), q, y, rows, cols, 1))
        scales.append(qs)
        torch.cuda.synchronize()
        if k < len(shapes):
            refs.append(oracle.gemv_i8_f64(nz, sg, s.view(np.uint16), q.cpu().numpy(), float(qs.item())))
    plan = tl.LinearPlan(probs, input_scales=scales)
    assert "gemv_mfma_kernel" in plan.kernel
    for launch in range(2):
        for p in probs:
            p[4].fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for k, (dnz, dsg, ds, q, y, rows, cols, _) in enumerate(probs):
            single = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
            tl.ternary_gemv_int8(dnz, dsg, ds, q, scales[k], single, rows, cols, 128)
            torch.cuda.synchronize()
            assert torch.equal(y[0], single), f"int8 plan, problem {k} ({rows}x{cols}), launch {launch}: differs from the single call"
            if k < len(shapes):
                assert_close(oracle, y[0].cpu().numpy().astype(np.float64), refs[k], what=f"int8 plan {rows}x{cols}")
    plan.close()
    # shorter rows (below the 2048 columns of the wide tiles): the plan runs the tall tiles, checked against the oracle
    tall, tall_scales, tall_refs = [], [], []
    for k, (rows, cols) in enumerate([(100, 1536), (64, 512), (300, 1152)]):
        nz, sg, s, x = synth.problem(8150 + k, rows, cols, unit_rms=True)
        q = torch.zeros(cols, dtype=torch.int8, device="cuda")
        qs = torch.zeros(1, dtype=torch.float32, device="cuda")
        tl.quantize_absmax_int8(up(torch, x), q, qs, cols)
        torch.cuda.synchronize()
        tall.append((up(torch, nz), up(torch, sg), up(torch, s), q, torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda"),
                     rows, cols, 1))
        tall_scales.append(qs)
        tall_refs.append(oracle.gemv_i8_f64(nz, sg, s.view(np.uint16), q.cpu().numpy(), float(qs.item())))
    plan = tl.LinearPlan(tall, input_scales=tall_scales)
    plan.launch()
    torch.cuda.synchronize()
    for p, ref in zip(tall, tall_refs):
        assert_close(oracle, p[4][0].cpu().numpy().astype(np.float64), ref, what=f"int8 plan, tall tiles, {p[5]}x{p[6]}")
    plan.close()
    # 384 columns are fewer than the matrix-core kernel takes: such a plan is refused, not run some other way
    nz, sg, s, x = synth.problem(8199, 64, 256 + 128, unit_rms=True)
    small = (up(torch, nz), up(torch, sg), up(torch, s), torch.zeros(384, dtype=torch.int8, device="cuda"),
             torch.zeros((1, 64), dtype=torch.float16, device="cuda"), 64, 384, 1)
    with pytest.raises(Exception):
        tl.LinearPlan([probs[0], small], input_scales=[scales[0], scales[0]])


def test_linear_plan_model_sweep_every_row(dev, oracle):
    """A LLaMA-1B-shaped sweep (8 layers x 7 matrices in one launch): every output row of every
    problem must equal what the single-call operator gives for that matrix (same kernel, fixed
    summation order: bit-identical), over several launches; layer 0 is checked against the oracle.
    Workgroups cross matrix boundaries mid-span here, which small plans do not exercise."""
    torch, tl = dev
    shapes = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (8192, 2048), (8192, 2048), (2048, 8192)]
    probs, host = [], []
    for layer in range(8):
        for k, (rows, cols) in enumerate(shapes):
            nz, sg, s, x = synth.problem(7000 + 10 * layer + k, rows, cols, unit_rms=True)
            y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
            probs.append((up(torch, nz), up(torch, sg), up(torch, s), up(torch, x.reshape(1, -1)), y, rows, cols, 1))
            host.append((nz, sg, s, x))
    singles = []
    for (dnz, dsg, ds, dx, _, rows, cols, _) in probs:
        y1 = torch.zeros(rows, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(dnz, dsg, ds, dx, y1, rows, cols, 128)
        singles.append(y1)
    torch.cuda.synchronize()
    for k in range(len(shapes)):
        nz, sg, s, x = host[k]
        ref = oracle.gemv_f64(nz, sg, s.view(np.uint16), x.view(np.uint16))
        assert_close(oracle, singles[k].cpu().numpy().astype(np.float64), ref, what=f"layer0 matrix {k}")
    plan = tl.LinearPlan(probs)
    for launch in range(4):
        for p in probs:
            p[4].fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for k, (p, y1) in enumerate(zip(probs, singles)):
            got = p[4][0].cpu().numpy()
            assert np.array_equal(got.view(np.uint16), y1.cpu().numpy().view(np.uint16)), \
                f"launch {launch} problem {k}: plan and single call differ"
    plan.close()


def _rand_weight(torch, gen, rows, cols):
    nz = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
    sg = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
    sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
    return nz, sg, sc


@pytest.mark.parametrize("rows,cols", [(14336, 4096), (8192, 2048), (100, 2048), (28672, 8192), (11008, 4096),
                                       (4100, 11008), (17, 2048), (20000, 2048)])
def test_swiglu_pair_vs_oracle_and_unfused(dev, oracle, rows, cols):
    """gate/up pair in one launch with the SiLU*mul epilogue: equal, bit for bit, to the two
    projections followed by the element-wise operator, and within tolerance of the fp64 evaluation
    silu(fp16(gate.x)) * fp16(up.x)."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(rows + cols)
    g_w, u_w = _rand_weight(torch, gen, rows, cols), _rand_weight(torch, gen, rows, cols)
    x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
    fused = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
    plan = tl.LinearPlan([(*g_w, x, fused, rows, cols, 1, tl.SWIGLU_GATE), (*u_w, x, None, rows, cols, 1)])
    plan.launch()
    torch.cuda.synchronize()
    g = torch.zeros(rows, dtype=torch.float16, device="cuda")
    u = torch.zeros(rows, dtype=torch.float16, device="cuda")
    tl.ternary_gemv(*g_w, x, g, rows, cols, 128)
    tl.ternary_gemv(*u_w, x, u, rows, cols, 128)
    unfused = torch.empty_like(g)
    tl.silu_mul(g, u, unfused, rows)
    torch.cuda.synchronize()
    assert torch.equal(fused[0].view(torch.int16), unfused.view(torch.int16))
    pick = np.random.default_rng(1).integers(0, rows, 128)
    xs = x[0].cpu().numpy().view(np.uint16)
    ref_g = oracle.gemv_f64(g_w[0][pick].cpu().numpy().view(np.uint32), g_w[1][pick].cpu().numpy().view(np.uint32),
                            g_w[2][pick].cpu().numpy().view(np.uint16), xs)
    ref_u = oracle.gemv_f64(u_w[0][pick].cpu().numpy().view(np.uint32), u_w[1][pick].cpu().numpy().view(np.uint32),
                            u_w[2][pick].cpu().numpy().view(np.uint16), xs)
    # the operator is defined on the fp16-rounded projections, as the reference's three launches are
    ref = oracle.silu_mul_f64(oracle.half_bits(ref_g), oracle.half_bits(ref_u))
    got = fused[0][pick].cpu().numpy().astype(np.float64)
    # a projection that lands on the other side of an fp16 rounding boundary moves the product by one
    # fp16 ulp of that factor: 2^-10 relative
    assert_close(oracle, got, ref, tol=2.5e-3, what=f"swiglu pair {rows}x{cols}")
    plan.close()


@pytest.mark.parametrize("cols,exact", [(4096, True), (2048, True), (8192, True), (16384, True), (11008, False)])
def test_rmsnorm_prologue_vs_unfused_and_oracle(dev, oracle, cols, exact):
    """q/k/v-like problems that read the residual stream through an RMSNorm prologue: equal to
    tllm_rmsnorm_f16 followed by the plain plan (bit for bit when cols is a multiple of 2048, where
    the sums are taken in the same order), and within tolerance of the fp64 evaluation."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(cols)
    x = (torch.randn((1, cols), device="cuda", generator=gen) * 3.0).to(torch.float16)
    wn = (torch.randn(cols, device="cuda", generator=gen) * 0.2 + 1.0).to(torch.float16)
    eps = 1e-5
    shapes = [(4096, cols), (1024, cols), (100, cols)]
    weights = [_rand_weight(torch, gen, r, c) for r, c in shapes]
    outs = [torch.full((1, r), float("nan"), dtype=torch.float16, device="cuda") for r, _ in shapes]
    fused = tl.LinearPlan([(*w, x, y, r, c, 1) for w, y, (r, c) in zip(weights, outs, shapes)],
                          norm_weights=[wn] * 3, eps=eps)
    fused.launch()
    xn = torch.empty_like(x)
    tl.rmsnorm(x, wn, xn, None, None, 1, cols, eps)
    ref_outs = [torch.zeros((1, r), dtype=torch.float16, device="cuda") for r, _ in shapes]
    plain = tl.LinearPlan([(*w, xn, y, r, c, 1) for w, y, (r, c) in zip(weights, ref_outs, shapes)])
    plain.launch()
    torch.cuda.synchronize()
    xn_ref, _ = oracle.rmsnorm_f64(x.cpu().numpy().view(np.uint16), wn.cpu().numpy().view(np.uint16), eps)
    xn_bits = oracle.half_bits(xn_ref[0])
    for w, y, yr, (r, c) in zip(weights, outs, ref_outs, shapes):
        if exact:
            assert torch.equal(y.view(torch.int16), yr.view(torch.int16)), f"{r}x{c}"
        pick = np.random.default_rng(r).integers(0, r, 64)
        ref = oracle.gemv_f64(w[0][pick].cpu().numpy().view(np.uint32), w[1][pick].cpu().numpy().view(np.uint32),
                              w[2][pick].cpu().numpy().view(np.uint16), xn_bits)
        # the normalised vector is rounded to fp16 before the product; where the fp32 statistic lands
        # on the other side of such a rounding, single elements of x' move by one fp16 ulp
        assert_close(oracle, y[0][pick].cpu().numpy().astype(np.float64), ref, tol=2e-3, what=f"normed {r}x{c}")
    fused.close()
    plain.close()


def test_rmsnorm_prologue_with_swiglu_pair(dev, oracle):
    """The FFN front half of a decoder layer in ONE launch: RMSNorm, gate and up projections, SiLU*mul
    (reference src/transformer.cpp:258-286: four launches). Equal to the four operators bit for bit."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31)
    h, ffn, eps = 4096, 14336, 1e-5
    x = (torch.randn((1, h), device="cuda", generator=gen) * 2.0).to(torch.float16)
    wn = (torch.randn(h, device="cuda", generator=gen) * 0.2 + 1.0).to(torch.float16)
    g_w, u_w = _rand_weight(torch, gen, ffn, h), _rand_weight(torch, gen, ffn, h)
    out = torch.full((1, ffn), float("nan"), dtype=torch.float16, device="cuda")
    plan = tl.LinearPlan([(*g_w, x, out, ffn, h, 1, tl.SWIGLU_GATE), (*u_w, x, None, ffn, h, 1)],
                         norm_weights=[wn, wn], eps=eps)
    for _ in range(2):
        out.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        xn = torch.empty_like(x)
        tl.rmsnorm(x, wn, xn, None, None, 1, h, eps)
        g = torch.zeros(ffn, dtype=torch.float16, device="cuda")
        u = torch.zeros(ffn, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(*g_w, xn, g, ffn, h, 128)
        tl.ternary_gemv(*u_w, xn, u, ffn, h, 128)
        want = torch.empty_like(g)
        tl.silu_mul(g, u, want, ffn)
        torch.cuda.synchronize()
        assert torch.equal(out[0].view(torch.int16), want.view(torch.int16))
    plan.close()


def test_swiglu_pairs_in_a_layer_sweep(dev, oracle):
    """Twelve 8B-shaped layers as one plan (q, k, v, o, the gate/up pair, down): large enough for the
    run-time pool, pairs in spans and in the pool alike; every output equals the separate calls."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    h, kv, ffn = 4096, 1024, 14336
    probs, expect = [], []
    for layer in range(12):
        x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
        xf = torch.randn((1, ffn), device="cuda", generator=gen).to(torch.float16)
        for rows, cols, xin in ((h, h, x), (kv, h, x), (kv, h, x), (h, h, x)):
            w = _rand_weight(torch, gen, rows, cols)
            y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
            probs.append((*w, xin, y, rows, cols, 1))
            e = torch.zeros(rows, dtype=torch.float16, device="cuda")
            tl.ternary_gemv(*w, xin, e, rows, cols, 128)
            expect.append((y, e))
        g_w, u_w = _rand_weight(torch, gen, ffn, h), _rand_weight(torch, gen, ffn, h)
        y = torch.zeros((1, ffn), dtype=torch.float16, device="cuda")
        probs.append((*g_w, x, y, ffn, h, 1, tl.SWIGLU_GATE))
        probs.append((*u_w, x, None, ffn, h, 1))
        g = torch.zeros(ffn, dtype=torch.float16, device="cuda")
        u = torch.zeros(ffn, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(*g_w, x, g, ffn, h, 128)
        tl.ternary_gemv(*u_w, x, u, ffn, h, 128)
        e = torch.empty_like(g)
        tl.silu_mul(g, u, e, ffn)
        expect.append((y, e))
        w = _rand_weight(torch, gen, h, ffn)
        y = torch.zeros((1, h), dtype=torch.float16, device="cuda")
        probs.append((*w, xf, y, h, ffn, 1))
        e = torch.zeros(h, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(*w, xf, e, h, ffn, 128)
        expect.append((y, e))
    torch.cuda.synchronize()
    plan = tl.LinearPlan(probs)
    for launch in range(3):
        for y, _ in expect:
            y.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for k, (y, e) in enumerate(expect):
            got, want = y[0].float(), e.float()
            # K = 14336: plan and single call may add a row's fp32 partial sums in a different
            # order; everything else is bit-identical
            if y.shape[1] == h and k % 6 == 5:
                assert torch.allclose(got, want, rtol=2e-3, atol=1e-4), f"launch {launch} output {k}"
            else:
                assert torch.equal(y[0].view(torch.int16), e.view(torch.int16)), f"launch {launch} output {k}"
    plan.close()


def test_linear_plan_large_sweep_shared_pool(dev, oracle):
    """A plan big enough (32 LLaMA-1B layers, 224 matrices) that part of it is dealt out at run time
    instead of belonging to a fixed span: whichever workgroup takes a piece, every output must equal
    the single-call result bit for bit, on every launch (the hand-out counters reset themselves)."""
    torch, tl = dev
    shapes = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (8192, 2048), (8192, 2048), (2048, 8192)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4242)
    probs = []
    for layer in range(32):
        for rows, cols in shapes:
            nz = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sg = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
            x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
            y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
            probs.append((nz, sg, sc, x, y, rows, cols, 1))
    singles = []
    for (nz, sg, sc, x, _, rows, cols, _) in probs:
        y1 = torch.zeros(rows, dtype=torch.float16, device="cuda")
        tl.ternary_gemv(nz, sg, sc, x, y1, rows, cols, 128)
        singles.append(y1)
    torch.cuda.synchronize()
    for k in (0, 55, 111):   # the single calls themselves, sampled rows against the oracle
        nz, sg, sc, x, _, rows, cols, _ = probs[k]
        pick = np.random.default_rng(k).integers(0, rows, 96)
        ref = oracle.gemv_f64(nz[pick].cpu().numpy().view(np.uint32), sg[pick].cpu().numpy().view(np.uint32),
                              sc[pick].cpu().numpy().view(np.uint16), x[0].cpu().numpy().view(np.uint16))
        assert_close(oracle, singles[k][pick].cpu().numpy().astype(np.float64), ref, what=f"single call {k}")
    plan = tl.LinearPlan(probs)
    for launch in range(3):
        for p in probs:
            p[4].fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        for k, (p, y1) in enumerate(zip(probs, singles)):
            assert torch.equal(p[4][0].view(torch.int16), y1.view(torch.int16)), \
                f"launch {launch} problem {k}: plan and single call differ"
    plan.close()


def test_large_plan_in_a_captured_graph(dev, oracle):
    """The same kind of plan recorded into a HIP graph: every replay (with eager work and
    synchronisation between replays) must reproduce the eager launch bit for bit. The kernel's own
    hand-out counters are reset by the kernel, not by a memset node."""
    torch, tl = dev
    shapes = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (8192, 2048), (8192, 2048), (2048, 8192)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(777)
    probs = []
    for layer in range(32):   # large enough for the run-time hand-out of its tail
        for rows, cols in shapes:
            nz = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sg = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
            x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
            y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
            probs.append((nz, sg, sc, x, y, rows, cols, 1))
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    eager = [p[4].clone() for p in probs]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plan.launch()          # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.launch()
    torch.cuda.synchronize()
    for replay in range(4):
        for p in probs:
            p[4].fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, (p, e) in enumerate(zip(probs, eager)):
            assert torch.equal(p[4].view(torch.int16), e.view(torch.int16)), f"replay {replay} problem {k}"
        if replay == 1:   # an eager launch between replays must not disturb the next replay
            plan.launch()
            torch.cuda.synchronize()
    plan.close()


def test_plan_launches_overlapping_on_two_streams(dev, oracle):
    """Launches of one large plan (its tail is handed out through device counters) issued on two streams so that
    they overlap in time: each launch has counters of its own, every launch must produce the bits of a launch
    that ran alone (all launches write the same values into the same outputs)."""
    torch, tl = dev
    shapes = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (8192, 2048), (8192, 2048), (2048, 8192)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(778)
    probs = []
    for layer in range(32):
        for rows, cols in shapes:
            nz = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sg = torch.randint(-2**31, 2**31 - 1, (rows, cols // 32), dtype=torch.int32, device="cuda", generator=gen)
            sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * 0.02 + 0.01).to(torch.float16)
            x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
            y = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
            probs.append((nz, sg, sc, x, y, rows, cols, 1))
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    alone = [p[4].clone() for p in probs]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for rep in range(3):
        for p in probs:
            p[4].fill_(float("nan"))
        torch.cuda.synchronize()
        for _ in range(5):
            plan.launch(stream=s1)
            plan.launch(stream=s2)
        torch.cuda.synchronize()
        for k, (p, a) in enumerate(zip(probs, alone)):
            assert torch.equal(p[4].view(torch.int16), a.view(torch.int16)), f"round {rep} problem {k}"
    plan.close()


def test_random_shapes_through_every_dispatch_path(dev, oracle):
    """Sixty seeded random (rows, cols, group, batch) problems against the oracle: whichever kernel the
    dispatcher picks (row-wave, tall, wide in 48- or 16-row units, batched decode, passes of it, the
    matrix-core GEMM with or without split K), the result has to be the same function of its inputs."""
    torch, tl = dev
    rng = np.random.default_rng(20240611)
    batches = [1, 1, 1, 2, 3, 4, 5, 8, 16, 17, 33, 70, 130]
    for case in range(60):
        group = int(rng.choice([128, 128, 128, 32, 64, 256]))
        cols = group * int(rng.integers(1, 1 + (6144 if case % 3 else 12288) // group))
        rows = int(rng.integers(1, 700 if case % 4 else 3000))
        batch = int(rng.choice(batches))
        nz, sg, s, _ = synth.problem(1000 + case, rows, cols, group=group, dontcare_sign=True)
        A = synth.acts_f16(rng, batch, cols)
        ref = oracle.gemm_f64(A.view(np.uint16), nz, sg, s.view(np.uint16), group)
        if batch == 1:
            got = run_gemv(dev, nz, sg, s, A[0], group)[None, :]
        else:
            got = run_gemm(dev, A, nz, sg, s, group)
        assert_close(oracle, got, ref, what=f"case {case}: rows {rows} cols {cols} group {group} batch {batch}")


# ---------------------------------------------- full-size, size-independent
def test_full_size_properties_8b(dev, oracle):
    """LLaMA-3-8B gate_proj (14336 x 4096) at full size: sampled rows against the oracle, plus
    properties that need no oracle: sign antisymmetry, exact zero for nz=0, power-of-two
    homogeneity in x (bit-exact), and row-slice consistency."""
    torch, tl = dev
    rows, cols = 14336, 4096
    nz, sg, s, x = synth.problem(8008, rows, cols)
    y = run_gemv(dev, nz, sg, s, x)
    pick = np.random.default_rng(1).integers(0, rows, 512)
    ref = oracle.gemv_f64(nz[pick], sg[pick], s[pick].view(np.uint16), x.view(np.uint16))
    assert_close(oracle, y[pick], ref, what="8B gate_proj sampled rows")
    # both sides are fp16-rounded, so they may sit one fp16 ulp (2^-10) apart
    assert oracle.error_report(run_gemv(dev, nz, ~sg, s, x), -y)["max_rel"] <= 2e-3
    assert not run_gemv(dev, np.zeros_like(nz), sg, s, x).any()
    x4 = (x.astype(np.float32) * 4).astype(np.float16)
    np.testing.assert_array_equal(run_gemv(dev, nz, sg, s, x4), 4 * y)
    np.testing.assert_array_equal(run_gemv(dev, nz[1000:1777], sg[1000:1777], s[1000:1777], x), y[1000:1777])


# ---------------------------------------------------------- benchmark configurations 4 and 5 at full size
def _device_problem(torch, rows, cols, p_zero, lo, hi, gen):
    """Seeded packed weights made on the device (the 70B matrices are too large to pack with numpy in
    test time): i.i.d. P(0) = p_zero, random sign bits also under zero weights, fp16 scales U[lo, hi]."""
    words = cols // 32
    pw = (torch.ones(32, dtype=torch.int64, device="cuda") << torch.arange(32, device="cuda"))
    nz = torch.empty((rows, words), dtype=torch.int32, device="cuda")
    step = max(1, (1 << 24) // cols)
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        v = ((torch.rand((r1 - r0, words, 32), device="cuda", generator=gen) >= p_zero).to(torch.int64) * pw).sum(dim=2)
        nz[r0:r1] = torch.where(v >= 2 ** 31, v - 2 ** 32, v).to(torch.int32)
    sg = torch.randint(-2 ** 31, 2 ** 31 - 1, (rows, words), dtype=torch.int32, device="cuda", generator=gen)
    sc = (torch.rand((rows, cols // 128), device="cuda", generator=gen) * (hi - lo) + lo).to(torch.float16)
    return nz, sg, sc


def _check_sampled(oracle, torch, A, nz, sg, sc, out, n_rows, n_cols, seed, what):
    """out[M, N] against the fp64 oracle on sampled activation rows x weight rows; everything finite."""
    assert bool(torch.isfinite(out).all()), f"{what}: non-finite output"
    M, N = out.shape
    rng = np.random.default_rng(seed)
    ms_ = np.unique(rng.integers(0, M, n_rows))
    ns_ = np.unique(np.concatenate([rng.integers(0, N, n_cols), [0, N - 1]]))
    ref = oracle.gemm_f64(A[ms_].cpu().numpy().view(np.uint16), nz[ns_].cpu().numpy().view(np.uint32),
                          sg[ns_].cpu().numpy().view(np.uint32), sc[ns_].cpu().numpy().view(np.uint16))
    full = out.float()
    tau = float(torch.sqrt(torch.mean(full * full)).item()) / 64.0
    got = out[ms_][:, ns_].cpu().numpy().astype(np.float64)
    rel = float((np.abs(got - ref) / np.maximum(np.abs(ref), tau)).max())
    assert rel <= TOL, f"{what}: max_rel {rel:.3e} (tau {tau:.3e})"


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("M", [16, 128, 512, 2048])
def test_cfg4_prefill_gemm_every_m(dev, oracle, M, N, K):
    """Benchmark configuration 4: X [M, K] N(0,1) against the LLaMA-3-8B gate/up (14336 x 4096) and down
    (4096 x 14336) matrices, every token count of the configuration. M = 2048 is the only case with eight
    256-row tiles; M = 128 runs the split-K path on both shapes."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(400 + M + N)
    nz, sg, sc = _device_problem(torch, N, K, 0.42, 0.01, 0.03, gen)
    A = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
    Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemm(A, nz, sg, sc, Cm, M, N, K, 128)
    torch.cuda.synchronize()
    _check_sampled(oracle, torch, A, nz, sg, sc, Cm, 6, 80, M + N, f"cfg4 M={M} {N}x{K}")


def _dense_weights(torch, nz, sg, sc):
    """fp32 [N, K] matrix of the packed weights (bit set in the sign plane: +scale, clear: -scale)."""
    rows, words = nz.shape
    sh = torch.arange(32, device="cuda", dtype=torch.int64)
    out = torch.empty((rows, words * 32), dtype=torch.float32, device="cuda")
    step = max(1, (1 << 23) // (words * 32))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        a = ((nz[r0:r1].to(torch.int64).unsqueeze(-1) >> sh) & 1).reshape(r1 - r0, -1)
        b = ((sg[r0:r1].to(torch.int64).unsqueeze(-1) >> sh) & 1).reshape(r1 - r0, -1)
        out[r0:r1] = (a * (2 * b - 1)).float() * sc[r0:r1].float().repeat_interleave(128, dim=1)
    return out


@pytest.mark.parametrize("M,N,K", [
    (1024, 4096, 14336),   # 256-row tiles, K split in two (128 tiles on 256 CUs)
    (640, 4096, 14336),    # the same with a ragged last tile of activation rows
    (512, 4096, 14336),    # 128-row tiles, K split
    (2048, 4096, 14336),   # 256-row tiles, no split
    (512, 1024, 4096),     # few tiles: K split eight ways
    (256, 256, 8192),
    (130, 512, 2048),
    (1024, 14336, 4096),
    (300, 2048, 2176),
])
def test_gemm_every_output_against_dense_product(dev, oracle, M, N, K):
    """Every element of C, not a sample: the packed weights are expanded to an fp32 matrix on the GPU and
    multiplied by the activations in fp32 (torch), which is itself checked against the fp64 oracle on sampled
    rows and columns. A fault confined to a few lanes and registers of one exchange step (1 output in 256)
    passes a sampled check more often than not; this test is the one that sees it. Each shape runs as the
    library chooses, with the row-split kernel forced in both its forms and with the four-wave kernels only."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7000 + M + N + K)
    nz, sg, sc = _device_problem(torch, N, K, 0.42, 0.01, 0.03, gen)
    A = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
    W = _dense_weights(torch, nz, sg, sc)
    ref = A.float() @ W.t()
    del W
    _check_sampled(oracle, torch, A, nz, sg, sc, ref, 4, 40, M + K, f"dense fp32 product {M}x{N}x{K}")
    tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
    for force in ({}, {"rowsplit": 1}, {"rowsplit": 2}, {"rowsplit": 0}):
        with gemm_forced(**force):
            for rep in range(2):
                Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
                tl.ternary_gemm(A, nz, sg, sc, Cm, M, N, K, 128)
                torch.cuda.synchronize()
                rel = (Cm.float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
                bad = int((~(rel <= TOL)).sum().item())
                assert bad == 0, (f"gemm {M}x{N}x{K} ({tl.gemm_kernel(M, N, K)}, forced={force}, repetition {rep}): "
                                  f"{bad} of {M * N} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}")


@pytest.mark.parametrize("M,N,K", [
    (512, 14336, 4096),   # the 8B FFN at a prefill of 512 tokens
    (200, 1000, 2048),    # ragged in M and N (N not a multiple of 8: the narrow store path)
    (130, 520, 2176),     # K = 128 (mod 256): a last half block; N a multiple of 8 only
    (1, 256, 384),        # a single activation row, the smallest K
    (2048, 2048, 2048),
])
def test_prefill_swiglu_pair_against_the_three_launches(dev, oracle, M, N, K):
    """tllm_ternary_gemm_swiglu_f16: gate GEMM, up GEMM and SiLU * up in one launch (reference
    src/transformer.cpp:264-286 at n_tokens > 1). Every output equals, bit for bit, what ternary_gemm on each matrix
    (forced to the four-wave row-split kernel, whose order of additions the pair kernel shares) followed by silu_mul
    stores; with the library's own choice of GEMM kernel for the separate launches the outputs agree to one rounding
    of either projection (2.5e-3 of the larger of |result| and a floor); and the gate projection inside the pair is
    within the bar of the fp32 product of the expanded weights (an up matrix of all-ones rows of weight makes the pair
    return silu(gate) * sum(x), which is checked directly)."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7700 + M + N + K)
    g_nz, g_sg, g_sc = _device_problem(torch, N, K, 0.42, 0.01, 0.03, gen)
    u_nz, u_sg, u_sc = _device_problem(torch, N, K, 0.42, 0.01, 0.03, gen)
    A = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
    f16 = dict(dtype=torch.float16, device="cuda")
    out = torch.full((M, N), float("nan"), **f16)
    tl.ternary_gemm_swiglu(A, g_nz, g_sg, g_sc, u_nz, u_sg, u_sc, out, M, N, K, 128)
    torch.cuda.synchronize()
    G, U = torch.zeros((M, N), **f16), torch.zeros((M, N), **f16)
    with gemm_forced(rowsplit=2):
        tl.ternary_gemm(A, g_nz, g_sg, g_sc, G, M, N, K, 128)
        tl.ternary_gemm(A, u_nz, u_sg, u_sc, U, M, N, K, 128)
    want = G.clone()
    tl.silu_mul(want, U, want, M * N)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16)), \
        f"{int((out.view(torch.int16) != want.view(torch.int16)).sum())} of {M * N} outputs differ from the three launches"
    # the library's own kernel choice for the separate launches: other order of additions, same results to a rounding
    tl.ternary_gemm(A, g_nz, g_sg, g_sc, G, M, N, K, 128)
    tl.ternary_gemm(A, u_nz, u_sg, u_sc, U, M, N, K, 128)
    tl.silu_mul(G, U, G, M * N)
    torch.cuda.synchronize()
    floor = float(torch.sqrt(torch.mean(G.float() ** 2)).item()) / 64.0
    rel = (out.float() - G.float()).abs() / torch.clamp(G.float().abs(), min=floor)
    assert float(rel.max()) <= 2.5e-3, f"max_rel {float(rel.max()):.3e} against the three launches as the library runs them"
    # against the fp32 product of the expanded weights
    Wg, Wu = _dense_weights(torch, g_nz, g_sg, g_sc), _dense_weights(torch, u_nz, u_sg, u_sc)
    g32 = (A.float() @ Wg.t()).half().float()
    u32 = (A.float() @ Wu.t()).half().float()
    ref = g32 / (1.0 + torch.exp(-g32)) * u32
    del Wg, Wu
    floor = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
    rel = (out.float() - ref).abs() / torch.clamp(ref.abs(), min=floor)
    assert float(rel.max()) <= 4e-3, f"max_rel {float(rel.max()):.3e} against silu(fp16(A gate^T)) * fp16(A up^T) in fp32"
    # twice the same bits
    again = torch.full((M, N), float("nan"), **f16)
    tl.ternary_gemm_swiglu(A, g_nz, g_sg, g_sc, u_nz, u_sg, u_sc, again, M, N, K, 128)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))


@pytest.mark.parametrize("M,K,Ns", [
    (512, 4096, (4096, 1024, 1024)),     # q, k, v of the 8B model at a prefill of 512 tokens
    (200, 2176, (520, 1000)),            # ragged everywhere; K = 128 (mod 256); an N that is not a multiple of 8
    (2048, 2048, (2048, 512, 512, 256)), # four matrices
    (96, 8192, (1024,)),                 # a group of one
])
def test_gemm_group_every_output(dev, oracle, M, K, Ns):
    """tllm_ternary_gemm_group_f16: several weight matrices on the same activations in one launch (the q/k/v
    projections of a prefill step, reference src/transformer.cpp:199-217 at n_tokens > 1). Every output of every
    matrix against the fp32 product of the expanded weights (sampled against the fp64 oracle); with the four-wave
    form forced (no tile is split along K) the bits equal those of the single calls forced the same way; repeated
    launches give the same bits."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7800 + M + K + sum(Ns))
    A = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
    ws = [_device_problem(torch, n, K, 0.42, 0.01, 0.03, gen) for n in Ns]
    f16 = dict(dtype=torch.float16, device="cuda")
    outs = [torch.full((M, n), float("nan"), **f16) for n in Ns]
    tl.ternary_gemm_group(A, ws, outs, M, K)
    torch.cuda.synchronize()
    first = [o.clone() for o in outs]
    for i, (n, w) in enumerate(zip(Ns, ws)):
        W = _dense_weights(torch, *w)
        ref = A.float() @ W.t()
        del W
        _check_sampled(oracle, torch, A, *w, ref, 3, 24, M + n, f"dense fp32 product of matrix {i}")
        tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
        rel = (outs[i].float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
        bad = int((~(rel <= TOL)).sum().item())
        assert bad == 0, f"matrix {i} ({M}x{n}x{K}): {bad} of {M * n} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}"
    for o in outs:
        o.fill_(float("nan"))
    tl.ternary_gemm_group(A, ws, outs, M, K)
    torch.cuda.synchronize()
    for a_, b_ in zip(outs, first):
        assert torch.equal(a_.view(torch.int16), b_.view(torch.int16))
    with gemm_forced(rowsplit=2):
        tl.ternary_gemm_group(A, ws, outs, M, K)
        compared = 0
        for n, w, o in zip(Ns, ws, outs):
            if "gemm_ns_kernel<4, 2>" not in tl.gemm_kernel(M, n, K):
                continue  # (a shape that the library streams through the batched kernel whatever is forced)
            compared += 1
            single = torch.zeros((M, n), **f16)
            tl.ternary_gemm(A, *w, single, M, n, K, 128)
            torch.cuda.synchronize()
            assert torch.equal(o.view(torch.int16), single.view(torch.int16)), f"matrix with {n} rows differs from its single call"
        assert compared or M < 128


def test_prefill_swiglu_pair_rejects_what_it_cannot_run(dev, oracle):
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7799)
    nz, sg, sc = _device_problem(torch, 256, 128, 0.42, 0.01, 0.03, gen)
    A = torch.randn((32, 128), device="cuda", generator=gen).to(torch.float16)
    out = torch.zeros((32, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(tl.TllmError) as err:       # K = 128: neither a multiple of 256 nor at least 384
        tl.ternary_gemm_swiglu(A, nz, sg, sc, nz, sg, sc, out, 32, 256, 128, 128)
    assert err.value.code == -2
    with pytest.raises(tl.TllmError) as err:       # group size other than 128
        tl.ternary_gemm_swiglu(A, nz, sg, sc, nz, sg, sc, out, 32, 256, 128, 64)
    assert err.value.code == -3
    with pytest.raises(tl.TllmError) as err:       # the output over the activations
        tl.ternary_gemm_swiglu(A, nz, sg, sc, nz, sg, sc, A, 32, 128, 128, 128)
    assert err.value.code < 0


@pytest.mark.parametrize("M,N,K", [
    (16, 4096, 14336),   # 64 blocks of 64 rows, four workgroups each
    (9, 1000, 4096),     # ragged last block, two parts of two steps
    (16, 192, 6144),     # three parts
    (5, 64, 28672),      # one block, eight parts
    (16, 320, 3584),     # an odd number of 512-column slices
    (24, 128, 8192),     # more than 16 activation rows: passes of the same launch, or the prefill kernel (the library's choice)
])
def test_batched_decode_k_shared_out_every_output(dev, oracle, M, N, K):
    """Few weight rows under a long K: the steps of a 64-row block are shared out among several workgroups, which
    exchange fp32 sums through the stream's workspace. Every output against the fp32 product of the expanded
    weights (itself sampled against the fp64 oracle); repeated calls give the same bits (the sums are added in part
    order whichever part arrives last); the entry point with the fixed exchange array gives the same bits; a
    captured graph without a reserved workspace (no exchange: one workgroup per block) stays within tolerance."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7300 + M + N + K)
    nz, sg, sc = _device_problem(torch, N, K, 0.42, 0.01, 0.03, gen)
    nz[N // 2] = 0  # a row without weights: exact zeros from every part
    A = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
    W = _dense_weights(torch, nz, sg, sc)
    ref = A.float() @ W.t()
    del W
    _check_sampled(oracle, torch, A, nz, sg, sc, ref, 4, 40, M + K, f"dense fp32 product {M}x{N}x{K}")
    if M <= 16:
        assert "K shared out" in tl.gemm_kernel(M, N, K)
    tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0

    def check(Cm, what):
        rel = (Cm.float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
        bad = int((~(rel <= TOL)).sum().item())
        assert bad == 0, f"{what} {M}x{N}x{K}: {bad} of {M * N} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}"
        assert bool((Cm[:, N // 2] == 0).all()), f"{what}: a row without weights must give exact zeros"

    outs = []
    for rep in range(3):
        Cm = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        tl.ternary_gemm(A, nz, sg, sc, Cm, M, N, K, 128)
        torch.cuda.synchronize()
        check(Cm, f"call {rep}")
        outs.append(Cm.view(torch.int16).clone())
    assert all(bool((o == outs[0]).all()) for o in outs[1:]), "repeated calls differ in bits"
    Cs = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemm_static(A, nz, sg, sc, Cs, M, N, K, 128)
    torch.cuda.synchronize()
    assert bool((Cs.view(torch.int16) == outs[0]).all()), "fixed exchange array: bits differ from the workspace's"
    # under capture on a stream that has no workspace nothing may be allocated: the launch takes no exchange
    st = torch.cuda.Stream()
    Cg = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(g, stream=st):
            tl.ternary_gemm(A, nz, sg, sc, Cg, M, N, K, 128, stream=st)
    torch.cuda.synchronize()
    for rep in range(2):
        Cg.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        check(Cg, f"graph replay {rep} without a workspace")
    # with a workspace reserved for the capture stream the captured launch shares out K like the eager one
    st2 = torch.cuda.Stream()
    tl.gemm_workspace_reserve(M, N, K, 128, stream=st2)
    Ch = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st2):
        with torch.cuda.graph(g2, stream=st2):
            tl.ternary_gemm(A, nz, sg, sc, Ch, M, N, K, 128, stream=st2)
    torch.cuda.synchronize()
    for rep in range(3):
        Ch.fill_(float("nan"))
        torch.cuda.synchronize()
        g2.replay()
        torch.cuda.synchronize()
        assert bool((Ch.view(torch.int16) == outs[0]).all()), f"graph replay {rep} with a reserved workspace: bits differ"


@pytest.mark.parametrize("batch", [1, 2, 4, 16])
def test_decode_plan_every_output_against_dense_product(dev, oracle, batch):
    """The decode kernels (one plan launch over the LLaMA-3-8B projections and a 70B-sized matrix pair) with
    every output row compared, not a sample, against the fp32 product of the expanded weights; the single-call
    entry points on the same operands must agree with the plan."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7100 + batch)
    shapes = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (28672, 8192), (8192, 28672), (1000, 1536)]
    probs, refs = [], []
    for rows, cols in shapes:
        nz, sg, sc = _device_problem(torch, rows, cols, 0.42, 0.01, 0.03, gen)
        x = torch.randn((batch, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        W = _dense_weights(torch, nz, sg, sc)
        refs.append(x.float() @ W.t())
        del W
        probs.append((nz, sg, sc, x, y, rows, cols, batch))
    _check_sampled(oracle, torch, probs[2][3], probs[2][0], probs[2][1], probs[2][2], refs[2], 2, 40, batch,
                   "dense fp32 product 14336x4096")
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    plan.close()
    for (nz, sg, sc, x, y, rows, cols, _), ref in zip(probs, refs):
        tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
        rel = (y.float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
        bad = int((~(rel <= TOL)).sum().item())
        assert bad == 0, f"plan {rows}x{cols} batch {batch}: {bad} of {batch * rows} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}"
        single = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        if batch == 1:
            tl.ternary_gemv(nz, sg, sc, x[0], single[0], rows, cols, 128)
        else:
            tl.ternary_gemm(x, nz, sg, sc, single, batch, rows, cols, 128)
        torch.cuda.synchronize()
        rel = (single.float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
        bad = int((~(rel <= TOL)).sum().item())
        assert bad == 0, f"single call {rows}x{cols} batch {batch}: {bad} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}"


LLAMA70B_LAYER = [(8192, 8192), (1024, 8192), (1024, 8192), (8192, 8192), (28672, 8192), (28672, 8192), (8192, 28672)]


@pytest.mark.parametrize("p_zero", [0.2, 0.42, 0.7])
@pytest.mark.parametrize("batch", [1, 16])
def test_cfg5_llama70b_layer_plan(dev, oracle, batch, p_zero):
    """Benchmark configuration 5: one full LLaMA-70B decoder layer (q, k, v, o, gate, up, down at hidden 8192,
    ffn 28672: 855.6 M weights) as one plan launch at batch 1 and batch 16, fp16 scales U[0.005, 0.02], zero
    fractions 0.2 / 0.42 / 0.7; sampled rows of every matrix against the oracle. The batch-16 matrices
    also go through the reference's own entry point for that case (ternary_gemm with M = 16)."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(int(500 + 100 * p_zero + batch))
    probs = []
    for rows, cols in LLAMA70B_LAYER:
        nz, sg, sc = _device_problem(torch, rows, cols, p_zero, 0.005, 0.02, gen)
        x = torch.randn((batch, cols), device="cuda", generator=gen).to(torch.float16)
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((nz, sg, sc, x, y, rows, cols, batch))
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    for k, (nz, sg, sc, x, y, rows, cols, _) in enumerate(probs):
        _check_sampled(oracle, torch, x, nz, sg, sc, y, 4, 48, 31 * k + batch, f"cfg5 {rows}x{cols} batch {batch} P0={p_zero}")
    plan.close()
    if batch == 16 and p_zero == 0.42:
        for k in (1, 4, 6):
            nz, sg, sc, x, y, rows, cols, _ = probs[k]
            Cm = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
            tl.ternary_gemm(x, nz, sg, sc, Cm, batch, rows, cols, 128)
            torch.cuda.synchronize()
            _check_sampled(oracle, torch, x, nz, sg, sc, Cm, 4, 48, k, f"cfg5 gemm entry {rows}x{cols} M=16")


def test_gemm_split_k_under_graph_capture(dev, oracle):
    """A GEMM whose shape splits K, captured into a HIP graph: with the workspace reserved beforehand the
    captured launch is the split one (bit-identical to the eager call); captured on a stream that has no
    workspace the call allocates nothing and runs without the split (same values within the bar). Every
    replay, with eager work between replays, gives the same bits."""
    torch, tl = dev
    M, N, K = 256, 1024, 4096
    nz, sg, s, _ = synth.problem(4300, N, K)
    A = synth.acts_f16(np.random.default_rng(4301), M, K)
    rows = np.unique(np.random.default_rng(1).integers(0, M, 6))
    ref = oracle.gemm_f64(A[rows].view(np.uint16), nz, sg, s.view(np.uint16))
    dA, dnz, dsg, ds = up(torch, A), up(torch, nz), up(torch, sg), up(torch, s)
    eager = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemm(dA, dnz, dsg, ds, eager, M, N, K, 128)
    torch.cuda.synchronize()
    assert_close(oracle, eager.cpu().numpy().astype(np.float64)[rows], ref, what="eager split-K")
    for reserve in (True, False):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            if reserve:
                tl.gemm_workspace_reserve(M, N, K, 128, stream=side)
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                tl.ternary_gemm(dA, dnz, dsg, ds, out, M, N, K, 128, stream=side)
        torch.cuda.synchronize()
        first = None
        for replay in range(3):
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = out.cpu().numpy()
            assert_close(oracle, got.astype(np.float64)[rows], ref, what=f"captured GEMM reserve={reserve} replay {replay}")
            if reserve:
                assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {replay}: differs from the eager split call"
            if first is None:
                first = got.view(np.uint16).copy()
            assert np.array_equal(got.view(np.uint16), first), f"reserve={reserve} replay {replay}: bits changed"
            if replay == 1:   # eager work between replays
                tl.ternary_gemm(dA, dnz, dsg, ds, eager, M, N, K, 128)
                torch.cuda.synchronize()
        del graph


def test_captured_split_gemm_survives_later_larger_shapes(dev, oracle):
    """A stream's exchange workspace never moves: a graph captured with a small split shape on a stream whose
    workspace was reserved for that shape, then eager calls on the same stream whose exchange is many times larger,
    then the graph again: every replay gives the bits of the eager small call."""
    torch, tl = dev
    small, large = (130, 256, 4096), (512, 1024, 14336)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    cases = {}
    for k, (M, N, K) in enumerate((small, large)):
        nz, sg, s, _ = synth.problem(9800 + k, N, K, dontcare_sign=True)
        A = synth.acts_f16(np.random.default_rng(9810 + k), M, K)
        cases[(M, N, K)] = (up(torch, A), up(torch, nz), up(torch, sg), up(torch, s), A, nz, sg, s)
    for shape in (small, large):
        assert "K split" in tl.gemm_kernel(*shape), f"{shape}: the test needs shapes that exchange partial sums"
    M, N, K = small
    dA, dnz, dsg, ds, A, nz, sg, s = cases[small]
    rows = np.unique(np.random.default_rng(2).integers(0, M, 6))
    ref = oracle.gemm_f64(A[rows].view(np.uint16), nz, sg, s.view(np.uint16))
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    eager = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        tl.gemm_workspace_reserve(M, N, K, 128, stream=side)
        tl.ternary_gemm(dA, dnz, dsg, ds, eager, M, N, K, 128, stream=side)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            tl.ternary_gemm(dA, dnz, dsg, ds, out, M, N, K, 128, stream=side)
    torch.cuda.synchronize()
    assert_close(oracle, eager.cpu().numpy().astype(np.float64)[rows], ref, what="eager small split")
    Ml, Nl, Kl = large
    lA, lnz, lsg, ls = cases[large][:4]
    big = torch.zeros((Ml, Nl), dtype=torch.float16, device="cuda")
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {replay}: differs from the eager call"
        with torch.cuda.stream(side):      # a larger exchange on the capture stream, and another reserve
            tl.ternary_gemm(lA, lnz, lsg, ls, big, Ml, Nl, Kl, 128, stream=side)
            tl.gemm_workspace_reserve(Ml, Nl, Kl, 128, stream=side)
        torch.cuda.synchronize()
    del graph


@pytest.mark.parametrize("cols", [4096, 8192])
def test_lm_head_shape_every_output(dev, oracle, cols):
    """The ternary output head of a .tllm model (reference src/transformer.cpp:308-311, src/model.cpp lm_head branch):
    128256 rows, far more than any projection. Batch 1 (single call and int8 pair), 4 and 16 activation rows, every
    output against the fp32 product of the expanded weights, which is itself checked against the fp64 oracle on
    samples."""
    torch, tl = dev
    rows = 128256
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8800 + cols)
    nz, sg, sc = _device_problem(torch, rows, cols, 0.42, 0.01, 0.03, gen)
    W = _dense_weights(torch, nz, sg, sc)
    for batch in (1, 4, 16):
        x = torch.randn((batch, cols), device="cuda", generator=gen).to(torch.float16)
        ref = x.float() @ W.t()
        y = torch.full((batch, rows), float("nan"), dtype=torch.float16, device="cuda")
        if batch == 1:
            tl.ternary_gemv(nz, sg, sc, x[0], y[0], rows, cols, 128)
        else:
            tl.ternary_gemm(x, nz, sg, sc, y, batch, rows, cols, 128)
        torch.cuda.synchronize()
        if batch == 1:
            _check_sampled(oracle, torch, x, nz, sg, sc, ref, 1, 48, cols, f"dense fp32 product {rows}x{cols}")
        tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
        rel = (y.float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
        bad = int((~(rel <= TOL)).sum().item())
        assert bad == 0, f"lm_head {rows}x{cols} batch {batch}: {bad} outputs beyond {TOL}, max_rel {float(rel.max()):.3e}"
        del ref, rel
    # the reference's decode path: quantise, then the int8 GEMV with the device-resident scale
    x = torch.randn((1, cols), device="cuda", generator=gen).to(torch.float16)
    q = torch.zeros(cols, dtype=torch.int8, device="cuda")
    qs = torch.zeros(1, dtype=torch.float32, device="cuda")
    yi = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
    tl.quantize_absmax_int8(x, q, qs, cols)
    tl.ternary_gemv_int8(nz, sg, sc, q, qs, yi[0], rows, cols, 128)
    torch.cuda.synchronize()
    ref = (q.float() * qs) @ W.t()
    tau = float(torch.sqrt(torch.mean(ref * ref)).item()) / 64.0
    rel = (yi[0].float() - ref).abs() / torch.clamp(ref.abs(), min=tau)
    assert float(rel.max()) <= TOL, f"lm_head int8 {rows}x{cols}: max_rel {float(rel.max()):.3e}"


@pytest.mark.parametrize("rows,cols,group", [(1024, 1024, 128), (4096, 4096, 128), (300, 11008, 128), (14336, 4096, 128),
                                             (4096, 14336, 128), (64, 28672, 128), (200, 36864, 128), (100, 256, 128),
                                             (50, 384, 64), (8, 128, 32)])
def test_fused_int8_linear_equals_the_pair(dev, oracle, rows, cols, group):
    """tllm_ternary_linear_int8_f16 (fp16 in, quantised inside the GEMV) stores the bits of quantize_absmax_int8 +
    ternary_gemv_int8 (reference src/transformer.cpp:126-143), on the matrix-core kernel (one segment, rows staged
    in segments) and on the general kernel (short rows, other group sizes); and stays within the bar of the
    oracle's integer arithmetic."""
    torch, tl = dev
    nz, sg, s, x = synth.problem(8300 + rows, rows, cols, group=group, dontcare_sign=True)
    x = (x.astype(np.float32) * 3.7).astype(np.float16)
    dnz, dsg, ds, dx = up(torch, nz), up(torch, sg), up(torch, s), up(torch, x)
    q = torch.zeros(cols, dtype=torch.int8, device="cuda")
    qs = torch.zeros(1, dtype=torch.float32, device="cuda")
    pair = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
    fused = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
    tl.quantize_absmax_int8(dx, q, qs, cols)
    tl.ternary_gemv_int8(dnz, dsg, ds, q, qs, pair, rows, cols, group)
    tl.ternary_linear_int8(dnz, dsg, ds, dx, fused, rows, cols, group)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int16), pair.view(torch.int16))
    qo, so = oracle.quantize_i8(x.view(np.uint16))
    ref = oracle.gemv_i8_f64(nz, sg, s.view(np.uint16), qo, np.float32(so), group)
    assert_close(oracle, fused.cpu().numpy().astype(np.float64), ref, what=f"fused int8 linear {rows}x{cols} g{group}")


def test_fused_int8_linear_special_inputs(dev, oracle):
    """All-zero activations (scale 1, outputs exactly 0), one non-zero element, and a plan of three problems that
    quantise their shared input themselves (the q/k/v group of a decode step) against the three pairs."""
    torch, tl = dev
    rows, cols = 512, 4096
    nz, sg, s, x = synth.problem(8400, rows, cols, dontcare_sign=True)
    dnz, dsg, ds = up(torch, nz), up(torch, sg), up(torch, s)
    y = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_linear_int8(dnz, dsg, ds, torch.zeros(cols, dtype=torch.float16, device="cuda"), y, rows, cols, 128)
    torch.cuda.synchronize()
    assert bool((y.view(torch.int16) == 0).all())
    one = np.zeros(cols, np.float16)
    one[1234] = np.float16(-0.37)
    tl.ternary_linear_int8(dnz, dsg, ds, up(torch, one), y, rows, cols, 128)
    torch.cuda.synchronize()
    w = synth.unpack_np(nz, sg)[:, 1234].astype(np.float64)
    amax = np.float32(abs(np.float16(-0.37)))                       # the element quantises to -127, the scale is amax / 127
    want = w * s[:, 1234 // 128].astype(np.float64) * -127.0 * float(amax / np.float32(127.0))
    np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want, rtol=1e-3, atol=0)
    shapes = [(4096, cols), (1024, cols), (1024, cols)]
    dx = up(torch, x)
    probs, pairs = [], []
    q = torch.zeros(cols, dtype=torch.int8, device="cuda")
    qs = torch.zeros(1, dtype=torch.float32, device="cuda")
    tl.quantize_absmax_int8(dx, q, qs, cols)
    for k, (r, c) in enumerate(shapes):
        a, b, sc_, _ = synth.problem(8410 + k, r, c, dontcare_sign=True)
        wdev = (up(torch, a), up(torch, b), up(torch, sc_))
        out = torch.full((1, r), float("nan"), dtype=torch.float16, device="cuda")
        probs.append((*wdev, dx.view(1, -1), out, r, c, 1, tl.QUANTIZE_INPUT))
        ref = torch.zeros(r, dtype=torch.float16, device="cuda")
        tl.ternary_gemv_int8(*wdev, q, qs, ref, r, c, 128)
        pairs.append(ref)
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    for pr, ref in zip(probs, pairs):
        assert torch.equal(pr[4][0].view(torch.int16), ref.view(torch.int16))
    plan.close()


@pytest.mark.parametrize("h,ffn,qd,kvd", [(4096, 14336, 4096, 1024), (2048, 8192, 2048, 512), (8192, 28672, 8192, 1024)])
def test_int8_decode_step_fusions_equal_the_reference_launches(dev, oracle, h, ffn, qd, kvd):
    """The reference's INT8 decode step (src/transformer.cpp:193-217 and 258-286): rmsnorm_forward, quantize_absmax_int8
    once, then the projections of the group on the shared int8 vector, then silu_mul_forward behind gate and up. As
    plans: the RMSNorm prologue, the quantisation inside the launch and the SwiGLU pair in ONE launch per group, with
    the bits of the separate launches; also the pair on an input that is quantised without a prologue."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(h + 7)
    f16 = dict(dtype=torch.float16, device="cuda")
    eps = 1e-5
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    x = (torch.randn((1, h), device="cuda", generator=gen) * 1.7).to(torch.float16)
    xn = torch.zeros((1, h), **f16)
    i8, i8s = torch.zeros(h, dtype=torch.int8, device="cuda"), torch.zeros(1, dtype=torch.float32, device="cuda")
    tl.rmsnorm(x, w["n2"], xn, None, None, 1, h, eps)
    tl.quantize_absmax_int8(xn, i8, i8s, h)
    g, u = torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16)
    tl.ternary_gemv_int8(*w["g"], i8, i8s, g, ffn, h, 128)
    tl.ternary_gemv_int8(*w["u"], i8, i8s, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    tl.rmsnorm(x, w["n1"], xn, None, None, 1, h, eps)
    tl.quantize_absmax_int8(xn, i8, i8s, h)
    want_qkv = []
    for name, r in (("q", qd), ("k", kvd), ("v", kvd)):
        o = torch.zeros((1, r), **f16)
        tl.ternary_gemv_int8(*w[name], i8, i8s, o, r, h, 128)
        want_qkv.append(o)
    act = torch.full((1, ffn), float("nan"), **f16)
    ffn_plan = tl.LinearPlan([(*w["g"], x, act, ffn, h, 1, tl.SWIGLU_GATE | tl.QUANTIZE_INPUT), (*w["u"], x, None, ffn, h, 1)],
                             norm_weights=[w["n2"], w["n2"]], eps=eps)
    outs = [torch.full((1, r), float("nan"), **f16) for r in (qd, kvd, kvd)]
    qkv_plan = tl.LinearPlan([(*w[name], x, o, r, h, 1, tl.QUANTIZE_INPUT) for name, o, r in zip("qkv", outs, (qd, kvd, kvd))],
                             norm_weights=[w["n1"]] * 3, eps=eps)
    for launch in range(2):
        ffn_plan.launch()
        qkv_plan.launch()
        torch.cuda.synchronize()
        assert torch.equal(act.view(torch.int16), g.view(torch.int16)), "RMSNorm + quantise + gate/up + SiLU * up"
        for name, got, ref in zip("qkv", outs, want_qkv):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"RMSNorm + quantise + {name}_proj"
    ffn_plan.close()
    qkv_plan.close()
    # the pair on a row that is quantised as it is (no prologue)
    tl.quantize_absmax_int8(x, i8, i8s, h)
    tl.ternary_gemv_int8(*w["g"], i8, i8s, g, ffn, h, 128)
    tl.ternary_gemv_int8(*w["u"], i8, i8s, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    act.fill_(float("nan"))
    plain = tl.LinearPlan([(*w["g"], x, act, ffn, h, 1, tl.SWIGLU_GATE | tl.QUANTIZE_INPUT), (*w["u"], x, None, ffn, h, 1)])
    plain.launch()
    torch.cuda.synchronize()
    assert torch.equal(act.view(torch.int16), g.view(torch.int16)), "quantise + gate/up + SiLU * up"
    plain.close()


def _chain_layer(torch, tl, gen, h, qd, kvd, ffn):
    """Random weights and norm vectors of one decoder layer (o, gate, up, down of this layer; q, k, v of the next)."""
    w = {name: _rand_weight(torch, gen, r, c) for name, (r, c) in
         dict(o=(h, qd), g=(ffn, h), u=(ffn, h), d=(h, ffn), q=(qd, h), k=(kvd, h), v=(kvd, h)).items()}
    w["n2"] = (torch.randn(h, device="cuda", generator=gen) * 0.1 + 1.0).to(torch.float16)
    w["n1"] = (torch.randn(h, device="cuda", generator=gen) * 0.1 + 1.0).to(torch.float16)
    return w


def _chain_separate(torch, tl, w, x, att, h, qd, kvd, ffn, eps):
    """The reference's launches (src/transformer.cpp:239-296 and 193-217 of the next layer), one operator call each."""
    f16 = dict(dtype=torch.float16, device="cuda")
    o, xn = torch.zeros((1, h), **f16), torch.zeros((1, h), **f16)
    g, u, d = torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    xs = x.clone()
    tl.ternary_gemv(*w["o"], att, o, h, qd, 128)
    tl.add(xs, o, xs, h)
    tl.rmsnorm(xs, w["n2"], xn, None, None, 1, h, eps)
    tl.ternary_gemv(*w["g"], xn, g, ffn, h, 128)
    tl.ternary_gemv(*w["u"], xn, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    tl.ternary_gemv(*w["d"], g, d, h, ffn, 128)
    tl.add(xs, d, xs, h)
    tl.rmsnorm(xs, w["n1"], xn, None, None, 1, h, eps)
    tl.ternary_gemv(*w["q"], xn, q, qd, h, 128)
    tl.ternary_gemv(*w["k"], xn, k, kvd, h, 128)
    tl.ternary_gemv(*w["v"], xn, v, kvd, h, 128)
    return xs, g, q, k, v


def _chain_staged(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps):
    probs = [(*w["o"], att, xs, h, qd, 1),
             (*w["g"], xs, hbuf, ffn, h, 1, tl.SWIGLU_GATE), (*w["u"], xs, None, ffn, h, 1),
             (*w["d"], hbuf, xs, h, ffn, 1),
             (*w["q"], xs, q, qd, h, 1), (*w["k"], xs, k, kvd, h, 1), (*w["v"], xs, v, kvd, h, 1)]
    norms = [None, w["n2"], w["n2"], None, w["n1"], w["n1"], w["n1"]]
    residuals = [xs, None, None, xs, None, None, None]
    return tl.LinearPlan(probs, norm_weights=norms, eps=eps, stages=[0, 1, 1, 2, 3, 3, 3], residuals=residuals)


def _chain_separate_int8(torch, tl, w, x, att, h, qd, kvd, ffn, eps):
    """The reference's INT8 decode launches (src/transformer.cpp:193-217, 244-296 with use_int8): every linear on the
    int8 quantisation of its input, the vectors shared inside a group."""
    f16 = dict(dtype=torch.float16, device="cuda")
    o, xn = torch.zeros((1, h), **f16), torch.zeros((1, h), **f16)
    g, u, d = torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    i8, i8s = torch.zeros(max(h, qd), dtype=torch.int8, device="cuda"), torch.zeros(1, dtype=torch.float32, device="cuda")
    xs = x.clone()
    tl.ternary_linear_int8(*w["o"], att, o, h, qd, 128)
    tl.add(xs, o, xs, h)
    tl.rmsnorm(xs, w["n2"], xn, None, None, 1, h, eps)
    tl.quantize_absmax_int8(xn, i8, i8s, h)
    tl.ternary_gemv_int8(*w["g"], i8, i8s, g, ffn, h, 128)
    tl.ternary_gemv_int8(*w["u"], i8, i8s, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    tl.ternary_linear_int8(*w["d"], g, d, h, ffn, 128)
    tl.add(xs, d, xs, h)
    tl.rmsnorm(xs, w["n1"], xn, None, None, 1, h, eps)
    tl.quantize_absmax_int8(xn, i8, i8s, h)
    tl.ternary_gemv_int8(*w["q"], i8, i8s, q, qd, h, 128)
    tl.ternary_gemv_int8(*w["k"], i8, i8s, k, kvd, h, 128)
    tl.ternary_gemv_int8(*w["v"], i8, i8s, v, kvd, h, 128)
    return xs, g, q, k, v


def _chain_staged_int8(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps):
    Q = tl.QUANTIZE_INPUT
    probs = [(*w["o"], att, xs, h, qd, 1, Q),
             (*w["g"], xs, hbuf, ffn, h, 1, tl.SWIGLU_GATE | Q), (*w["u"], xs, None, ffn, h, 1),
             (*w["d"], hbuf, xs, h, ffn, 1, Q),
             (*w["q"], xs, q, qd, h, 1, Q), (*w["k"], xs, k, kvd, h, 1, Q), (*w["v"], xs, v, kvd, h, 1, Q)]
    norms = [None, w["n2"], w["n2"], None, w["n1"], w["n1"], w["n1"]]
    residuals = [xs, None, None, xs, None, None, None]
    return tl.LinearPlan(probs, norm_weights=norms, eps=eps, stages=[0, 1, 1, 2, 3, 3, 3], residuals=residuals)


@pytest.mark.parametrize("handover", ["words", "barriers"])
@pytest.mark.parametrize("h,qd,kvd,ffn", [(4096, 4096, 1024, 14336), (2048, 2048, 512, 8192)])
def test_staged_int8_decode_layer_equals_the_reference_launches(dev, oracle, tuned, h, qd, kvd, ffn, handover):
    """The linear side of the reference's INT8 decode layer (fourteen launches and four copies of a scale to the host)
    as ONE launch: every input quantised inside the launch, behind the RMSNorm prologue where the reference normalises
    first. The residual stream, the FFN activation and q, k, v hold the bits of the separate launches."""
    torch, tl = dev
    tuned(stage_exchange=1 if handover == "words" else 0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(h + ffn + 1)
    eps = 1e-5
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    want = _chain_separate_int8(torch, tl, w, x, att, h, qd, kvd, ffn, eps)
    xs, hbuf = x.clone(), torch.full((1, ffn), float("nan"), **f16)
    q, k, v = torch.full((1, qd), float("nan"), **f16), torch.full((1, kvd), float("nan"), **f16), torch.full((1, kvd), float("nan"), **f16)
    plan = _chain_staged_int8(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps)
    assert ("tagged words" if handover == "words" else "barriers") in plan.kernel
    for launch in range(3):
        xs.copy_(x)
        for t in (hbuf, q, k, v):
            t.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        plan.status()
        for name, got, ref in zip(("residual stream", "silu(gate) * up", "q", "k", "v"), (xs, hbuf, q, k, v), want):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"launch {launch}: {name} differs from the separate launches"
    plan.close()


@pytest.mark.parametrize("handover", ["words", "barriers"])
@pytest.mark.parametrize("h,qd,kvd,ffn", [(4096, 4096, 1024, 14336), (2048, 2048, 512, 8192), (2048, 2304, 256, 5632)])
def test_staged_plan_equals_the_separate_launches(dev, oracle, tuned, h, qd, kvd, ffn, handover):
    """o_proj (+ residual) -> RMSNorm, gate/up, SiLU * up -> down_proj (+ residual) -> RMSNorm, q/k/v of the next
    layer as ONE launch with waits between the stages: the residual stream, the FFN activation and q, k, v hold the
    bits of the twelve separate launches, launch after launch; the projection rows are within the bar of the oracle.
    Both ways of handing results from stage to stage: tagged words that the next stage polls (the residual stream is
    updated in place twice, as the reference does), and barriers."""
    torch, tl = dev
    tuned(stage_exchange=1 if handover == "words" else 0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(h + ffn)
    eps = 1e-5
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    want = _chain_separate(torch, tl, w, x, att, h, qd, kvd, ffn, eps)
    xs, hbuf = x.clone(), torch.full((1, ffn), float("nan"), **f16)
    q, k, v = torch.full((1, qd), float("nan"), **f16), torch.full((1, kvd), float("nan"), **f16), torch.full((1, kvd), float("nan"), **f16)
    plan = _chain_staged(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps)
    assert "staged" in plan.kernel and ("tagged words" if handover == "words" else "barriers") in plan.kernel
    for launch in range(3):
        xs.copy_(x)
        for t in (hbuf, q, k, v):
            t.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        plan.status()
        for name, got, ref in zip(("residual stream", "silu(gate) * up", "q", "k", "v"), (xs, hbuf, q, k, v), want):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"launch {launch}: {name} differs from the separate launches"
    # the o_proj rows against the oracle: stream + projection, both fp16-rounded
    o_ref = oracle.gemv_f64(w["o"][0][:64].cpu().numpy().view(np.uint32), w["o"][1][:64].cpu().numpy().view(np.uint32),
                            w["o"][2][:64].cpu().numpy().view(np.uint16), att.cpu().numpy().view(np.uint16)[0])
    plan2 = tl.LinearPlan([(*w["o"], att, xs, h, qd, 1)], stages=[0], residuals=[xs])
    xs.copy_(x)
    plan2.launch()
    torch.cuda.synchronize()
    got = xs[0, :64].cpu().numpy().astype(np.float64) - x[0, :64].cpu().numpy().astype(np.float64)
    assert np.abs(got - o_ref).max() <= 2e-3 * max(1.0, np.abs(o_ref).max()) + np.abs(x[0, :64].cpu().numpy().astype(np.float64)).max() * 2.0 ** -10
    plan.close()
    plan2.close()


def test_staged_plan_whose_buffers_rule_out_tagged_words_waits_at_barriers(dev, oracle):
    """A stage that reads only PART of an earlier output (a view into it) cannot take it from the producer's tagged
    words; the plan then runs with barriers between its stages, and gives the bits of the separate launches. The same
    two problems on whole buffers run with tagged words."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    f16 = dict(dtype=torch.float16, device="cuda")
    wa, wb = _rand_weight(torch, gen, 4096, 2048), _rand_weight(torch, gen, 1024, 2048)
    wc = _rand_weight(torch, gen, 1024, 4096)
    x = torch.randn((1, 2048), device="cuda", generator=gen).to(torch.float16)
    ya, yb, yc = torch.zeros((1, 4096), **f16), torch.zeros((1, 1024), **f16), torch.zeros((1, 1024), **f16)
    tl.ternary_gemv(*wa, x, ya, 4096, 2048, 128)
    tl.ternary_gemv(*wb, ya[:, 2048:].contiguous(), yb, 1024, 2048, 128)
    tl.ternary_gemv(*wc, ya, yc, 1024, 4096, 128)
    want_a, want_b, want_c = ya.clone(), yb.clone(), yc.clone()
    part = ya[:, 2048:]                                  # the second half of the first stage's output, in place
    plan = tl.LinearPlan([(*wa, x, ya, 4096, 2048, 1), (*wb, part, yb, 1024, 2048, 1)], stages=[0, 1])
    assert "barriers" in plan.kernel
    whole = tl.LinearPlan([(*wa, x, ya, 4096, 2048, 1), (*wc, ya, yc, 1024, 4096, 1)], stages=[0, 1])
    assert "tagged words" in whole.kernel
    for launch in range(3):
        for t in (ya, yb, yc):
            t.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        plan.status()
        assert torch.equal(ya.view(torch.int16), want_a.view(torch.int16)) and torch.equal(yb.view(torch.int16), want_b.view(torch.int16))
        ya.fill_(float("nan"))
        whole.launch()
        torch.cuda.synchronize()
        whole.status()
        assert torch.equal(ya.view(torch.int16), want_a.view(torch.int16)) and torch.equal(yc.view(torch.int16), want_c.view(torch.int16))
    plan.close()
    whole.close()


@pytest.mark.parametrize("handover", ["words", "barriers"])
def test_staged_plan_in_a_captured_graph_and_on_a_second_stream(dev, oracle, tuned, handover):
    """The staged launch under graph capture (no allocation, counters that reset themselves, tags that every
    workgroup advances by itself): replays, with eager launches of the same plan on another stream between them, give
    the eager bits every time."""
    torch, tl = dev
    tuned(stage_exchange=1 if handover == "words" else 0)
    h, qd, kvd, ffn, eps = 2048, 2048, 512, 8192, 1e-5
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31)
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    want = _chain_separate(torch, tl, w, x, att, h, qd, kvd, ffn, eps)
    xs, hbuf = x.clone(), torch.zeros((1, ffn), **f16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    plan = _chain_staged(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        xs.copy_(x)
        plan.launch(stream=side)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            xs.copy_(x)
            plan.launch(stream=side)
    torch.cuda.synchronize()
    for replay in range(4):
        for t in (hbuf, q, k, v):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        plan.status()
        for name, got, ref in zip(("residual stream", "silu(gate) * up", "q", "k", "v"), (xs, hbuf, q, k, v), want):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"replay {replay}: {name}"
        xs.copy_(x)            # an eager launch between the replays
        plan.launch()
        torch.cuda.synchronize()
    del graph
    plan.close()


def test_staged_plan_of_int8_linears_and_of_long_rows(dev, oracle):
    """Inputs that the launch quantises itself (the reference's INT8 decode path, src/transformer.cpp:244-250 and
    288-296: o_proj and down_proj as ternary_linear_int8 with the residual add behind them) in a staged plan, with
    either way of handing results over; and rows too long to be staged from registers (the 70B down_proj, K = 28672,
    behind its gate/up pair), which make a staged plan wait at barriers and read the stage before with an invalidated
    cache. All give the bits of the separate launches."""
    torch, tl = dev
    gen = torch.Generator(device="cuda")
    gen.manual_seed(36)
    f16 = dict(dtype=torch.float16, device="cuda")
    # (1) o_proj(int8) + residual -> down-like projection (int8) + residual, 8B sizes
    h, mid = 4096, 14336
    wa, wb = _rand_weight(torch, gen, mid, h), _rand_weight(torch, gen, h, mid)
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    r1 = torch.randn((1, mid), device="cuda", generator=gen).to(torch.float16)
    r2 = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    ya, yb = torch.zeros((1, mid), **f16), torch.zeros((1, h), **f16)
    tl.ternary_linear_int8(*wa, x, ya, mid, h, 128)
    tl.add(r1, ya, ya, mid)
    tl.ternary_linear_int8(*wb, ya, yb, h, mid, 128)
    tl.add(r2, yb, yb, h)
    want_a, want_b = ya.clone(), yb.clone()
    for handover in ("tagged words", "barriers"):
        with tl.tuning(stage_exchange=1 if handover == "tagged words" else 0):
            plan = tl.LinearPlan([(*wa, x, ya, mid, h, 1, tl.QUANTIZE_INPUT), (*wb, ya, yb, h, mid, 1, tl.QUANTIZE_INPUT)],
                                 stages=[0, 1], residuals=[r1, r2])
        assert handover in plan.kernel
        for launch in range(3):
            ya.fill_(float("nan")); yb.fill_(float("nan"))
            plan.launch()
            torch.cuda.synchronize()
            plan.status()
            assert torch.equal(ya.view(torch.int16), want_a.view(torch.int16)), f"{handover}, launch {launch}: first stage"
            assert torch.equal(yb.view(torch.int16), want_b.view(torch.int16)), f"{handover}, launch {launch}: second stage"
        plan.close()
    # (2) 70B FFN: RMSNorm + gate/up pair 28672 x 8192 -> down_proj 8192 x 28672 + residual
    h, ffn, eps = 8192, 28672, 1e-5
    wg, wu, wd = _rand_weight(torch, gen, ffn, h), _rand_weight(torch, gen, ffn, h), _rand_weight(torch, gen, h, ffn)
    nw = (torch.randn(h, device="cuda", generator=gen) * 0.1 + 1.0).to(torch.float16)
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    xn, g, u, d = torch.zeros((1, h), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    tl.rmsnorm(x, nw, xn, None, None, 1, h, eps)
    tl.ternary_gemv(*wg, xn, g, ffn, h, 128)
    tl.ternary_gemv(*wu, xn, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    tl.ternary_gemv(*wd, g, d, h, ffn, 128)
    tl.add(x, d, d, h)
    act, out = torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    plan = tl.LinearPlan([(*wg, x, act, ffn, h, 1, tl.SWIGLU_GATE), (*wu, x, None, ffn, h, 1), (*wd, act, out, h, ffn, 1)],
                         norm_weights=[nw, nw, None], eps=eps, stages=[0, 0, 1], residuals=[None, None, x])
    assert "barriers" in plan.kernel
    for launch in range(2):
        act.fill_(float("nan")); out.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        plan.status()
        assert torch.equal(act.view(torch.int16), g.view(torch.int16)), f"launch {launch}: silu(gate) * up"
        assert torch.equal(out.view(torch.int16), d.view(torch.int16)), f"launch {launch}: stream after down_proj"
    plan.close()


def test_staged_plan_many_launches_back_to_back(dev, oracle):
    """Five hundred launches of one staged plan queued without a synchronisation between them (they take the plan's
    sixteen launch slots in turn; every launch reads its inputs from buffers no launch writes): the outputs of the last
    one, and of a launch in the middle that is copied out on the stream, are the bits of the separate launches."""
    torch, tl = dev
    h, qd, ffn, eps = 4096, 4096, 14336, 1e-5
    gen = torch.Generator(device="cuda")
    gen.manual_seed(35)
    w = _chain_layer(torch, tl, gen, h, qd, 1024, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    o, x1, xn = torch.zeros((1, h), **f16), torch.zeros((1, h), **f16), torch.zeros((1, h), **f16)
    g, u, d, x2 = torch.zeros((1, ffn), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16), torch.zeros((1, h), **f16)
    tl.ternary_gemv(*w["o"], att, o, h, qd, 128)
    tl.add(x, o, x1, h)
    tl.rmsnorm(x1, w["n2"], xn, None, None, 1, h, eps)
    tl.ternary_gemv(*w["g"], xn, g, ffn, h, 128)
    tl.ternary_gemv(*w["u"], xn, u, ffn, h, 128)
    tl.silu_mul(g, u, g, ffn)
    tl.ternary_gemv(*w["d"], g, d, h, ffn, 128)
    tl.add(x1, d, x2, h)
    s1, act, s2 = torch.zeros((1, h), **f16), torch.zeros((1, ffn), **f16), torch.zeros((1, h), **f16)
    plan = tl.LinearPlan([(*w["o"], att, s1, h, qd, 1), (*w["g"], s1, act, ffn, h, 1, tl.SWIGLU_GATE), (*w["u"], s1, None, ffn, h, 1),
                          (*w["d"], act, s2, h, ffn, 1)],
                         norm_weights=[None, w["n2"], w["n2"], None], eps=eps, stages=[0, 1, 1, 2], residuals=[x, None, None, s1])
    assert "tagged words" in plan.kernel
    middle = None
    for launch in range(500):
        plan.launch()
        if launch == 250:
            middle = (s1.clone(), act.clone(), s2.clone())
    torch.cuda.synchronize()
    plan.status()
    for tag, got in (("launch 250", middle), ("last launch", (s1, act, s2))):
        for name, a_, b_ in zip(("stream after o_proj", "silu(gate) * up", "stream after down_proj"), got, (x1, g, x2)):
            assert torch.equal(a_.view(torch.int16), b_.view(torch.int16)), f"{tag}: {name}"
    plan.close()


def test_staged_plan_tags_wrap_around(dev, oracle, tuned):
    """The tag of the words that hand results from stage to stage is the low 16 bits of a launch count. A plan created
    with that count just below the wrap is launched across it (more launches than launch slots times the distance to
    the wrap): every launch gives the bits of the separate launches."""
    torch, tl = dev
    tuned(stage_exchange=1, stage_epoch_start=65531)
    h, qd, kvd, ffn, eps = 2048, 2048, 512, 8192, 1e-5
    gen = torch.Generator(device="cuda")
    gen.manual_seed(33)
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    want = _chain_separate(torch, tl, w, x, att, h, qd, kvd, ffn, eps)
    xs, hbuf = x.clone(), torch.zeros((1, ffn), **f16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    plan = _chain_staged(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps)
    assert "tagged words" in plan.kernel
    for launch in range(16 * 8):          # sixteen launch slots, each crosses the wrap at its fifth launch
        xs.copy_(x)
        for t in (hbuf, q, k, v):
            t.fill_(float("nan"))
        plan.launch()
        torch.cuda.synchronize()
        plan.status()
        for name, got, ref in zip(("residual stream", "silu(gate) * up", "q", "k", "v"), (xs, hbuf, q, k, v), want):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"launch {launch}: {name}"
    plan.close()


@pytest.mark.parametrize("handover", ["words", "barriers"])
def test_staged_plan_wait_that_expires_is_reported(dev, oracle, tuned, handover):
    """A wait between two stages is bounded: with the bound forced down to one poll (tuning switch) the workgroups
    that arrive early give up, every workgroup ends normally, tllm_linear_plan_status reports the timeout once, and
    the next launch with the ordinary bound is complete and correct."""
    torch, tl = dev
    tuned(stage_exchange=1 if handover == "words" else 0)
    h, qd, kvd, ffn, eps = 2048, 2048, 512, 8192, 1e-5
    gen = torch.Generator(device="cuda")
    gen.manual_seed(32)
    w = _chain_layer(torch, tl, gen, h, qd, kvd, ffn)
    f16 = dict(dtype=torch.float16, device="cuda")
    x = torch.randn((1, h), device="cuda", generator=gen).to(torch.float16)
    att = torch.randn((1, qd), device="cuda", generator=gen).to(torch.float16)
    want = _chain_separate(torch, tl, w, x, att, h, qd, kvd, ffn, eps)
    xs, hbuf = x.clone(), torch.zeros((1, ffn), **f16)
    q, k, v = torch.zeros((1, qd), **f16), torch.zeros((1, kvd), **f16), torch.zeros((1, kvd), **f16)
    plan = _chain_staged(torch, tl, w, xs, att, hbuf, q, k, v, h, qd, kvd, ffn, eps)
    tl.set_tuning("stage_spin_limit", 1)
    try:
        plan.launch()
        torch.cuda.synchronize()
        with pytest.raises(tl.TllmError) as err:
            plan.status()
        assert err.value.code == -11
    finally:
        tl.set_tuning("stage_spin_limit", 0)
    plan.status()                       # cleared by the call that reported it
    xs.copy_(x)
    plan.launch()
    torch.cuda.synchronize()
    plan.status()
    for name, got, ref in zip(("residual stream", "silu(gate) * up", "q", "k", "v"), (xs, hbuf, q, k, v), want):
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), name
    plan.close()
