"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, validates arguments without touching a GPU, and its host-side
weight repack is byte-identical to the oracle's."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_exports_every_declared_symbol(pkg):
    L = pkg.capi.lib()
    header = open(os.path.join(ROOT, "include", "a81w41.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)   # declarations only, not prose
    declared = set(re.findall(r"\b(a81w41_[A-Za-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    for name in sorted(declared):
        assert hasattr(L, name), f"library lacks {name}"
    assert declared == set(pkg.capi.SIGNATURES), declared ^ set(pkg.capi.SIGNATURES)


def test_blob_sizes(pkg):
    L = pkg.capi.lib()
    assert L.a81w41_weight_blob_bytes(4096, 4096, 0) == 32768 * 320
    assert L.a81w41_weight_blob_bytes(4096, 4096, 1) == 32768 * 384
    assert L.a81w41_act_blob_bytes(4096, 0) == 64 * 72
    assert L.a81w41_act_blob_bytes(322 * 4096, 1) == 20608 * 80
    assert L.a81w41_weight_blob_bytes(4095, 4096, 0) == 0   # K % 64 != 0
    assert L.a81w41_act_blob_bytes(100, 0) == 0


@pytest.mark.parametrize("fp32", [False, True])
@pytest.mark.parametrize("N,K", [(8, 64), (24, 320), (1024, 4096)])
def test_host_repack_matches_oracle(pkg, ora, synth, fp32, N, K):
    w4, scale, offset = synth.weight_files(N, K, seed=61)
    scale = scale * np.float32(1.2345)      # not fp16-representable: exercises the rounding
    got = pkg.ops.repack_w81_weight(K, N, scale, offset, w4, fp32)
    assert np.array_equal(got, ora.repack(w4, scale, offset, K, N, fp32))


def test_argument_errors(pkg):
    L = pkg.capi.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data_as(C.c_void_p)
    assert L.a81w41_repack_w81_weight_fp16(100, 8, 32, p, p, p, p) == 1
    assert b"K % 64" in L.a81w41_last_error()
    assert L.a81w41_repack_w81_weight_fp16(64, 8, 16, p, p, p, p) == 1
    assert L.a81w41_repack_w81_weight_fp32(64, 8, 32, None, p, p, p) == 1
    assert L.a81w41_quantize_row_q8_1_repack_fp16(p, p, 100, None) == 1
    assert L.a81w41_quantize_row_q8_1_repack_fp16(p, p, 0, None) == 0      # empty input is a no-op
    assert L.a81w41_gemv_repack_A81W41_fp16(p, p, p, 1, 12, 64, None) == 1  # N % 8
    assert L.a81w41_gemm_repack_A81W41_fp32(p, p, p, 0, 8, 64, None) == 1   # M < 1
    h = C.c_void_p()
    assert L.a81w41_context_create(0, 64, C.byref(h)) == 1
    assert L.a81w41_linear_forward(None, p, 1, p, None) == 1
    assert L.a81w41_status_string(1) == b"invalid argument"


def test_no_gpu_is_reported_not_faked(pkg):
    """Without a device the compute entry points must fail loudly (no CPU path)."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    L = pkg.capi.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data_as(C.c_void_p)
    assert L.a81w41_quantize_row_q8_1_repack_fp32(p, p, 64, None) == 4
    assert L.a81w41_gemv_repack_A81W41_fp16(p, p, p, 1, 8, 64, None) == 4


def test_gemm_schedule_covers_every_tile_and_chunk_once(pkg):
    """The work list of the 64 x 64-tile kernel (persistent grid, last round cut along K): walked on the host for
    the shapes and row counts the layer sees and for odd ones, on the real chip size and on smaller ones.
    Every tile and every K chunk exactly once, tile numbering one-to-one, no partial tile shared."""
    L = pkg.capi.lib()
    shapes = [(4096, 4096), (4096, 1024), (4096, 12288), (12288, 4096), (4096, 6144), (4096, 24576),
              (512, 256), (4096, 8), (256, 4104), (64, 64), (1024, 40)]
    rows = [9, 33, 64, 65, 128, 322, 512, 640, 832, 1024, 2048, 4096]
    used_split = 0
    for K, N in shapes:
        for M in rows:
            for resident, cus in ((1024, 256), (512, 256), (768, 256), (16, 4), (3, 3)):
                got = L.a81w41_gemm_schedule_selfcheck(M, N, K, resident, cus)
                assert got >= 0, (M, N, K, resident, cus, got)
                assert got <= 4096
                used_split += got > 0
    assert used_split > 20      # the K split really is exercised
    assert L.a81w41_gemm_schedule_selfcheck(0, 64, 64, 1024, 256) < 0   # argument errors are negative too


def test_block_scaled_gemm_plan_covers_every_unit_once(pkg):
    """The layer object's M > 32 kernel cuts the (tile, 32-block) units of a launch into equal contiguous runs:
    walked on the host for the layer's shapes and odd ones, for several device sizes."""
    L = pkg.capi.lib()
    shapes = [(4096, 4096), (4096, 1024), (4096, 12288), (12288, 4096), (4096, 6144), (4096, 24576), (4096, 151936),
              (512, 256), (4096, 8), (256, 4104), (64, 64), (1024, 40)]
    shared = 0
    for K, N in shapes:
        for M in (33, 64, 65, 128, 129, 322, 512, 640, 1024, 2048, 4096):
            for slots in (512, 256, 8, 3, 1):
                got = L.a81w41_gemm_fp6_plan_selfcheck(M, N, K, slots)
                assert got >= 0, (M, N, K, slots, got)
                shared += got > 0
    assert shared > 50
    assert L.a81w41_gemm_fp6_plan_selfcheck(0, 64, 64, 512) < 0
