"""Pins the oracle's activation quantizers (quantized_gemx_kernels.cc:693-911)
against the numpy closed form, textbook special cases and the dequantisation
error bound."""
import numpy as np
import pytest

from np_model import parse_act_blob, quantize_closed_form


@pytest.mark.parametrize("fp32", [False, True])
@pytest.mark.parametrize("outliers", [False, True])
def test_matches_closed_form(ora, synth, fp32, outliers):
    x = synth.activations(37, 1024, seed=21, outliers=outliers)
    x[3, 64:96] = 0.0                       # an all-zero block
    x[5, :32] *= np.float32(1e-30)          # tiny block, d is subnormal in fp16
    x[6, 32:64] *= np.float32(1e4)          # d overflows nothing but is large
    blob = ora.quantize(x, fp32)
    q, d, ss = parse_act_blob(blob, fp32)
    q0, d0, ss0 = quantize_closed_form(x)
    assert np.array_equal(q.reshape(-1, 32), q0)
    if fp32:
        assert np.array_equal(d.reshape(-1).view(np.uint32), d0.view(np.uint32))
        assert np.array_equal(ss.reshape(-1).view(np.uint32), ss0.view(np.uint32))
    else:
        # the fp16 scaled sum is rounded from the fp32 product with the *unrounded* d
        assert np.array_equal(d.reshape(-1), d0.astype(np.float16).astype(np.float32))
        assert np.array_equal(ss.reshape(-1), ss0.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("fp32", [False, True])
def test_special_cases(ora, fp32):
    x = np.zeros((4, 64), np.float32)
    x[1, 7] = 3.5            # single element -> q = +127 there, d = 3.5/127
    x[2, 40] = -2.0          # single negative element in the high block -> -127
    x[3, :] = 1.0            # constant block -> all 127, sum = 32*127
    q, d, ss = parse_act_blob(ora.quantize(x, fp32), fp32)
    assert not q[0].any() and not d[0].any() and not ss[0].any()
    assert q[1, 0, 7] == 127 and np.count_nonzero(q[1]) == 1
    assert q[2, 1, 8] == -127 and np.count_nonzero(q[2]) == 1
    assert (q[3] == 127).all()
    f = (lambda v: np.float32(v)) if fp32 else (lambda v: np.float32(np.float16(v)))
    assert d[1, 0] == f(np.float32(3.5) / np.float32(127))
    assert ss[1, 0] == f(np.float32(3.5) / np.float32(127) * np.float32(127))
    assert ss[2, 1] == f(np.float32(2.0) / np.float32(127) * np.float32(-127))
    assert ss[3, 0] == f(np.float32(1.0) / np.float32(127) * np.float32(32 * 127))


def test_invariants_and_error_bound(ora, synth):
    x = synth.activations(64, 4096, seed=22)
    q, d, ss = parse_act_blob(ora.quantize(x, True), True)
    q = q.reshape(-1, 32).astype(np.int32)
    d = d.reshape(-1)
    xb = x.reshape(-1, 32)
    assert np.abs(q).max() <= 127
    assert (np.abs(q).max(axis=1) == 127).all()          # amax element always maps to +-127
    # |x - d*q| <= d/2 up to fp32 rounding of x*id
    err = np.abs(xb.astype(np.float64) - d[:, None].astype(np.float64) * q)
    assert (err <= 0.5 * d[:, None] * (1 + 1e-5) + 1e-12).all()
    # sign symmetry and exact power-of-two scaling
    qn = parse_act_blob(ora.quantize(-x, True), True)[0]
    assert np.array_equal(qn.reshape(-1, 32), -q)
    q4, d4, ss4 = parse_act_blob(ora.quantize(x * np.float32(4.0), True), True)
    assert np.array_equal(q4.reshape(-1, 32), q)
    assert np.array_equal(d4.reshape(-1), d * np.float32(4.0))


def test_m_rows_are_independent(ora, synth):
    """forward() quantizes M*K floats in one call (QwenOperator.cc:100); rows must
    not interact because K % 64 == 0."""
    x = synth.activations(5, 256, seed=23)
    whole = ora.quantize(x, True).reshape(5, -1)
    for m in range(5):
        assert np.array_equal(whole[m], ora.quantize(x[m], True))


@pytest.mark.parametrize("fp32", [False, True])
def test_overflowing_inverse_scale_gives_the_x86_answer(ora, fp32):
    """amax < ~3.7e-37: 127/amax = +inf, every x*id is +-inf or (for x = 0) NaN, cvtps_epi32 answers
    0x80000000 for each of them, the saturating packs make that -128, and the int32 sum of 32 such values
    wraps to 0 (32 * -2^31 = 0 mod 2^32), so scaled_sum = d * 0 (quantized_gemx_kernels.cc:735-780).  The
    expected bytes are written out here; tests/test_oracle_avx2.py has the x86 instructions confirm them."""
    tiny = np.float32(1e-38)
    x = np.zeros((3, 64), np.float32)
    x[0, :32] = tiny * np.linspace(-1.0, 1.0, 32, dtype=np.float32)
    x[0, 5] = 0.0
    x[0, 32:] = np.float32(1.0)                       # ordinary neighbour in the same super-block
    x[1, 32:] = 0.0
    x[1, 32 + 9] = np.float32(-3e-39)                 # subnormal amax, every other element zero
    x[2, :32] = np.float32(3.8e-37)                   # just above the threshold: finite id, ordinary result
    x[2, 3] = 0.0
    q, d, ss = parse_act_blob(ora.quantize(x, fp32), fp32)
    f = (lambda v: np.float32(v)) if fp32 else (lambda v: np.float32(np.float16(v)))
    assert (q[0, 0] == -128).all() and ss[0, 0] == 0.0 and d[0, 0] == f(tiny / np.float32(127))
    assert (q[0, 1] == 127).all()
    assert (q[1, 1] == -128).all() and ss[1, 1] == 0.0
    assert not q[1, 0].any() and d[1, 0] == 0.0
    want = np.full(32, 127, np.int8)
    want[3] = 0
    assert np.array_equal(q[2, 0], want)
    assert ss[2, 0] == f(np.float32(3.8e-37) / np.float32(127) * np.float32(31 * 127))
