"""The GEMM entry point that allocates nothing (a81w41_gemm_repack_A81W41_fp32_static): the partial
tiles of its K split live in a file-scope device array of the library.  Checked through the C ABI
against the entry point it is a variant of, bit for bit, and against the oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(ora, synth, torch, M, N, K, seed):
    w4, s, o = synth.weight_files(N, K, seed)
    x = synth.activations(M, K, seed + 1, outliers=True)
    ba, bw = ora.quantize(x, True), ora.repack(w4, s, o, K, N, True)
    return torch.from_numpy(ba).cuda(), torch.from_numpy(bw).cuda(), ora.gemm_fp32(ba, bw, M, N, K)


def test_first_static_call_can_be_captured_and_allocates_nothing(pkg, ora, synth):
    """What the entry point is for: its very first call in the process, on a stream that has never been used, goes
    into a HIP graph under capture (the allocating entry point refuses that), the device's free memory does not
    move, and every replay returns the allocating entry point's bits."""
    import torch

    M, N, K = 322, 1024, 4096                       # splits K: partial tiles are parked
    a, b, want = _case(ora, synth, torch, M, N, K, 401)
    ref = pkg.ops.gemm_fp32(a, b, M, N, K)           # allocating entry point, eagerly, on the default stream
    got = torch.empty((M, N), dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream, capture_error_mode="thread_local"):
            pkg.ops.gemm_fp32(a, b, M, N, K, out=got, static_scratch=True)
        for rep in range(3):
            got.fill_(float("nan"))
            graph.replay()
            stream.synchronize()
            assert torch.equal(got, ref), rep
    # eager static calls on that stream, which has no scratch of its own (the allocating entry point would
    # now allocate 64 MiB for it): the device's free memory does not move
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(stream):
        for _ in range(2):
            pkg.ops.gemm_fp32(a, b, M, N, K, out=got, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(got, ref)
    g = got.cpu().numpy().astype(np.float64)
    assert np.max(np.linalg.norm(g - want, axis=1) / np.linalg.norm(want.astype(np.float64), axis=1)) <= 1e-4


def test_static_scratch_gemm_equals_the_allocating_entry_point(pkg, ora, synth):
    import torch

    L = pkg.capi.lib()
    # two calls in a row, the second smaller; then a shape without a K split and a few-row call.
    # (322, 1024, 4096) and (130, 136, 2048) split K (partial tiles parked in the static array).
    cases = [(322, 1024, 4096, 401), (130, 136, 2048, 403), (64, 64, 1024, 405), (5, 64, 256, 407), (322, 1024, 4096, 401)]
    assert L.a81w41_gemm_schedule_selfcheck(322, 1024, 4096, 1024, 256) > 0
    assert L.a81w41_gemm_schedule_selfcheck(130, 136, 2048, 1024, 256) > 0
    for M, N, K, seed in cases:
        a, b, want = _case(ora, synth, torch, M, N, K, seed)
        ref = pkg.ops.gemm_fp32(a, b, M, N, K)
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pkg.ops.gemm_fp32(a, b, M, N, K, out=got, static_scratch=True)
        torch.cuda.synchronize()
        assert torch.equal(got, ref), (M, N, K)
        g = got.cpu().numpy().astype(np.float64)
        err = np.max(np.linalg.norm(g - want, axis=1) / np.linalg.norm(want.astype(np.float64), axis=1))
        assert err <= 1e-4, (M, N, K, err)


def test_static_scratch_gemm_rejects_what_does_not_fit(pkg):
    import torch

    L = pkg.capi.lib()
    # a shape whose schedule on this device parks more partial tiles than the static array holds (on 256 CUs:
    # 700 rows, 704 tiles over K = 12288 cut in four = 2816 > 2048)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    N, K = 4096, 12288
    M = next((m for m in range(256, 4096, 4) if L.a81w41_gemm_schedule_selfcheck(m, N, K, 4 * cus, cus) > 2048), None)
    assert M is not None, "no shape on this device exceeds the static scratch"
    a = torch.zeros(M * (K // 64) * 80, dtype=torch.uint8, device="cuda")
    b = torch.zeros((N // 8) * (K // 64) * 384, dtype=torch.uint8, device="cuda")
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    st = L.a81w41_gemm_repack_A81W41_fp32_static(C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()), C.c_void_p(c.data_ptr()),
                                                 M, N, K, None)
    assert st == 1 and b"static scratch" in L.a81w41_last_error()
    # the allocating entry point takes the same call
    pkg.ops.gemm_fp32(a, b, M, N, K, out=c)
    torch.cuda.synchronize()
    assert float(c.abs().max()) == 0.0
