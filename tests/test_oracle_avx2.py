"""The AVX2+OpenMP CPU-baseline port must agree bit for bit with the scalar oracle, in every
integer-dot branch (maddubs, AVX-VNNI, AVX512-VNNI: lib.h:45-55) that this CPU can run."""
import ctypes as C

import numpy as np
import pytest

from oracle import ora as _ora_mod

BRANCHES = _ora_mod.avx_branches_supported() or ["avx2"]


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


@pytest.fixture(params=BRANCHES)
def avx(request, ora):
    return ora.avx(request.param)


def test_branch_names(ora):
    assert "avx2" in BRANCHES, "x86-64-v3 is the floor for the CPU baseline"
    for b in BRANCHES:
        assert b.replace("avx512vnni", "avx512-vnni").replace("avxvnni", "avx-vnni") in ora.avx(b).avx_dot_branch().decode()
    assert ora.avx() is ora.avx(BRANCHES[0])       # default = the branch the reference's #if chain would take


@pytest.mark.parametrize("fp32", [False, True])
def test_quantize(ora, avx, synth, fp32):
    x = synth.activations(9, 512, seed=51, outliers=True)
    x[2, :64] = 0
    want = ora.quantize(x, fp32)
    got = np.zeros_like(want)
    fn = avx.avx_quantize_row_q8_1_repack_fp32 if fp32 else avx.avx_quantize_row_q8_1_repack_fp16
    fn(_p(x), _p(got), x.size)
    assert np.array_equal(got, want)


def test_gemv(ora, avx, synth):
    N, K = 48, 1024
    w4, s, o = synth.weight_files(N, K, 52)
    bw = ora.repack(w4, s, o, K, N, False)
    ba = ora.quantize(synth.activations(1, K, 53), False)
    got = np.zeros(N, np.float32)
    avx.avx_gemv_repack_A81W41_fp16(_p(ba), _p(bw), _p(got), 1, N, K, 4)
    assert np.array_equal(got, ora.gemv_fp16(ba, bw, N, K))


@pytest.mark.parametrize("M", [1, 6, 7, 17])
def test_gemm(ora, avx, synth, M):
    N, K = 40, 512
    w4, s, o = synth.weight_files(N, K, 54)
    bw = ora.repack(w4, s, o, K, N, True)
    ba = ora.quantize(synth.activations(M, K, 55), True)
    got = np.zeros((M, N), np.float32)
    avx.avx_gemm_repack_A81W41_fp32(_p(ba), _p(bw), _p(got), M, N, K, 4)
    assert np.array_equal(got, ora.gemm_fp32(ba, bw, M, N, K))


@pytest.mark.parametrize("fp32", [False, True])
def test_quantize_when_127_over_amax_overflows(ora, avx, fp32):
    """amax below about 3.7e-37 makes 127/amax overflow to +inf (quantized_gemx_kernels.cc:735-737): x*id is
    then +-inf, or NaN where x is 0, and cvtps_epi32 returns 0x80000000 for all of them, which the two
    saturating packs turn into -128 while the int32 sum wraps (:747-780).  The x86 instructions of the port
    decide what comes out; the scalar oracle (and through it the GPU quantiser) has to produce those bytes."""
    x = np.zeros((4, 64), np.float32)
    tiny = np.float32(1e-38)                       # a normal fp32 for which 127 / amax = inf
    with np.errstate(over="ignore"):
        assert np.isinf(np.float32(127.0) / tiny)
    x[0, :32] = tiny * np.linspace(-1.0, 1.0, 32, dtype=np.float32)   # mixed signs
    x[0, 5] = 0.0                                  # a zero inside the block: 0 * inf = NaN
    x[0, 6] = -0.0
    x[0, 32:] = np.float32(3e-39)                  # fp32 subnormal amax
    x[0, 40] = 0.0
    x[1, :32] = 0.0
    x[1, 17] = np.float32(-2e-38)                  # a single element, the rest zeros
    x[1, 32:] = np.float32(1.0)                    # an ordinary block next to it
    x[2, :] = tiny
    x[2, ::2] *= np.float32(-1.0)
    x[3, :32] = np.float32(3.6e-37)                # just past the threshold: 127 / amax is finite
    x[3, 3] = 0.0
    x[3, 32:] = np.float32(3.8e-37)
    x[3, 35] = 0.0
    got = np.zeros_like(ora.quantize(x, fp32))
    fn = avx.avx_quantize_row_q8_1_repack_fp32 if fp32 else avx.avx_quantize_row_q8_1_repack_fp16
    fn(_p(x), _p(got), x.size)
    q = got.reshape(4, -1)[:, (16 if fp32 else 8):].view(np.int8)
    assert (q[0, :32] == -128).all() and (q[2] == -128).all()        # the x86 result this test is about
    assert (q[1, :32] == -128).all() and (q[1, 32:] == 127).all()
    assert np.array_equal(got, ora.quantize(x, fp32))
