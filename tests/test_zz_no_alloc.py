"""tllm_ternary_gemm_f16_static: the GEMM entry point that allocates nothing (its split-K exchange lives in a fixed
device array of the library). Called through the C ABI and compared bit for bit with
tllm_ternary_gemm_f16 (same kernels, same split, same order of additions) and with the fp64 oracle, on two
calls in a row of which the second is smaller, on shapes that split K, and on shapes of the other routes."""
import numpy as np
import pytest

from tests import synth

pytestmark = pytest.mark.gpu


def _up(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).cuda()


def test_static_gemm_matches_the_allocating_entry_point(oracle):
    import torch
    import ternary_llm_amd as tl
    assert torch.cuda.is_available(), "needs the MI355X"
    L = tl.lib()
    # (M, N, K): two shapes that split K (the second smaller than the first), one with whole tiles only,
    # one decode-size batch (no GEMM kernel at all)
    shapes = [(512, 1024, 4096), (130, 512, 2048), (300, 4096, 1024), (8, 640, 1024)]
    cases = []
    for k, (M, N, K) in enumerate(shapes):
        nz, sg, s, _ = synth.problem(9100 + k, N, K, dontcare_sign=True)
        A = synth.acts_f16(np.random.default_rng(9200 + k), M, K)
        rows = np.unique(np.random.default_rng(k).integers(0, M, 5))
        ref = oracle.gemm_f64(A[rows].view(np.uint16), nz, sg, s.view(np.uint16))
        cases.append((M, N, K, _up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s), rows, ref))
    stream = torch.cuda.current_stream().cuda_stream

    def call(fn, case, out):
        M, N, K, dA, dnz, dsg, ds, _, _ = case
        code = fn(dA.data_ptr(), dnz.data_ptr(), dsg.data_ptr(), ds.data_ptr(), out.data_ptr(), M, N, K, 128, stream)
        assert code == 0, L.tllm_error_string(code).decode()

    for rep in range(2):   # the second round meets the array as the first one left it
        free_before = None
        for case in cases:
            M, N = case[0], case[1]
            got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            if rep == 1:
                torch.cuda.synchronize()
                free_before = torch.cuda.mem_get_info()[0]
            call(L.tllm_ternary_gemm_f16_static, case, got)
            if rep == 1:
                torch.cuda.synchronize()
                assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the free device memory"
            call(L.tllm_ternary_gemm_f16, case, want)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{case[:3]} round {rep}: differs from tllm_ternary_gemm_f16"
            rep_err = oracle.error_report(got.cpu().numpy().astype(np.float64)[case[7]], case[8])
            assert rep_err["max_rel"] <= 1e-3, f"{case[:3]} round {rep}: {rep_err}"
    # the row-split kernel's exchange slots live in the same fixed array: tiles split eight ways, then a smaller shape
    forced = tl.tuning(gemm_rowsplit=1)
    forced.__enter__()
    try:
        for k, (M, N, K) in enumerate([(260, 300, 6144), (130, 256, 4096)]):
            assert "K split" in tl.gemm_kernel(M, N, K)
            nz, sg, s, _ = synth.problem(9600 + k, N, K, dontcare_sign=True)
            A = synth.acts_f16(np.random.default_rng(9700 + k), M, K)
            rows = np.unique(np.random.default_rng(k).integers(0, M, 6))
            ref = oracle.gemm_f64(A[rows].view(np.uint16), nz, sg, s.view(np.uint16))
            case = (M, N, K, _up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s), None, None)
            got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            call(L.tllm_ternary_gemm_f16_static, case, got)
            call(L.tllm_ternary_gemm_f16, case, want)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"row-split kernel {M}x{N}x{K}: differs from tllm_ternary_gemm_f16"
            rep_err = oracle.error_report(got.cpu().numpy().astype(np.float64)[rows], ref)
            assert rep_err["max_rel"] <= 1e-3, f"row-split kernel {M}x{N}x{K}: {rep_err}"
    finally:
        forced.__exit__(None, None, None)
    # same argument checks as the allocating entry point
    M, N, K, dA, dnz, dsg, ds, _, _ = cases[0]
    out = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    assert L.tllm_ternary_gemm_f16_static(dA.data_ptr(), dnz.data_ptr(), dsg.data_ptr(), ds.data_ptr(), out.data_ptr(),
                                          0, N, K, 128, stream) == -2
    assert L.tllm_ternary_gemm_f16_static(dA.data_ptr(), dnz.data_ptr(), dsg.data_ptr(), None, out.data_ptr(),
                                          M, N, K, 128, stream) == -1
    assert b"fixed device scratch" in L.tllm_error_string(-10)


def test_static_gemm_in_a_captured_graph(oracle):
    """Captured without any preparation (nothing to reserve): replays equal the eager call bit for bit."""
    import torch
    import ternary_llm_amd as tl
    M, N, K = 256, 1024, 4096
    nz, sg, s, _ = synth.problem(9300, N, K)
    A = synth.acts_f16(np.random.default_rng(9301), M, K)
    dA, dnz, dsg, ds = _up(torch, A), _up(torch, nz), _up(torch, sg), _up(torch, s)
    eager = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tl.ternary_gemm_static(dA, dnz, dsg, ds, eager, M, N, K, 128)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            tl.ternary_gemm_static(dA, dnz, dsg, ds, out, M, N, K, 128, stream=side)
    torch.cuda.synchronize()
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {replay}"
        if replay == 0:
            tl.ternary_gemm_static(dA, dnz, dsg, ds, eager, M, N, K, 128)
            torch.cuda.synchronize()
