"""TEST INFRASTRUCTURE ONLY -- ctypes binding of the CPU oracle.

Importable from tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py``; the shipped package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liba81w41_oracle.so")


def build(force: bool = False) -> None:
    args = ["make", "-C", _HERE, "all"]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load(path):
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_lib = None
_avx = None

_vp, _i, _i64 = C.c_void_p, C.c_int, C.c_int64


def lib():
    global _lib
    if _lib is None:
        L = _load(_LIB)
        L.ora_fp32_to_fp16.argtypes = [C.c_float]
        L.ora_fp32_to_fp16.restype = C.c_uint16
        L.ora_fp16_to_fp32.argtypes = [C.c_uint16]
        L.ora_fp16_to_fp32.restype = C.c_float
        for name in ("ora_repack_w81_weight_fp16", "ora_repack_w81_weight_fp32"):
            getattr(L, name).argtypes = [_i, _i, _i, _vp, _vp, _vp, _vp]
            getattr(L, name).restype = None
        for name in ("ora_quantize_row_q8_1_repack_fp16", "ora_quantize_row_q8_1_repack_fp32"):
            getattr(L, name).argtypes = [_vp, _vp, _i64]
            getattr(L, name).restype = None
        for name in ("ora_gemv_repack_A81W41_fp16", "ora_gemm_repack_A81W41_fp32"):
            getattr(L, name).argtypes = [_vp, _vp, _vp, _i, _i, _i]
            getattr(L, name).restype = None
        L.ora_block_idot.argtypes = [_vp, _i, _vp, _i, _vp, _i, _i, _i]
        L.ora_block_idot.restype = None
        L.ora_linear_forward.argtypes = [_vp, _i, _i, _i, _vp, _vp, _vp, _vp]
        L.ora_linear_forward.restype = None
        L.ora_quantize_weight_q41.argtypes = [_vp, _i, _i, _vp, _vp, _vp]
        L.ora_quantize_weight_q41.restype = None
        L.ora_repack_w80_weight.argtypes = [_i, _i, _i, _vp, _vp, _vp]
        L.ora_repack_w80_weight.restype = None
        L.ora_quantize_row_q8_0_repack.argtypes = [_vp, _vp, _i64]
        L.ora_quantize_row_q8_0_repack.restype = None
        for name in ("ora_gemv_repack_A80W40", "ora_gemm_repack_A80W40"):
            getattr(L, name).argtypes = [_vp, _vp, _vp, _i, _i, _i]
            getattr(L, name).restype = None
        L.ora_block_idot_w80.argtypes = [_vp, _vp, _vp, _i, _i, _i]
        L.ora_block_idot_w80.restype = None
        L.ora_quantize_weight_q40.argtypes = [_vp, _i, _i, _vp, _vp]
        L.ora_quantize_weight_q40.restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_vp)


W_BLOCK = {False: 320, True: 384}
A_BLOCK = {False: 72, True: 80}


def repack(w4: np.ndarray, scale: np.ndarray, offset: np.ndarray, K: int, N: int, fp32: bool) -> np.ndarray:
    out = np.zeros(N * K // 512 * W_BLOCK[fp32], dtype=np.uint8)
    fn = lib().ora_repack_w81_weight_fp32 if fp32 else lib().ora_repack_w81_weight_fp16
    fn(K, N, 32, _p(out), _p(np.ascontiguousarray(scale, np.float32)),
       _p(np.ascontiguousarray(offset, np.float32)), _p(np.ascontiguousarray(w4, np.uint8)))
    return out


def quantize(x: np.ndarray, fp32: bool) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    k = x.size
    assert k % 64 == 0
    out = np.zeros(k // 64 * A_BLOCK[fp32], dtype=np.uint8)
    fn = lib().ora_quantize_row_q8_1_repack_fp32 if fp32 else lib().ora_quantize_row_q8_1_repack_fp16
    fn(_p(x), _p(out), k)
    return out


def gemv_fp16(a_blob: np.ndarray, b_blob: np.ndarray, N: int, K: int) -> np.ndarray:
    out = np.zeros(N, dtype=np.float32)
    lib().ora_gemv_repack_A81W41_fp16(_p(a_blob), _p(b_blob), _p(out), 1, N, K)
    return out


def gemm_fp32(a_blob: np.ndarray, b_blob: np.ndarray, M: int, N: int, K: int) -> np.ndarray:
    out = np.zeros((M, N), dtype=np.float32)
    lib().ora_gemm_repack_A81W41_fp32(_p(a_blob), _p(b_blob), _p(out), M, N, K)
    return out


def block_idot(a_blob, a_fp32: bool, b_blob, b_fp32: bool, M: int, N: int, K: int) -> np.ndarray:
    out = np.zeros((M, N, K // 32), dtype=np.int32)
    lib().ora_block_idot(_p(a_blob), int(a_fp32), _p(b_blob), int(b_fp32), _p(out), M, N, K)
    return out


def linear_forward(x: np.ndarray, b16: np.ndarray, b32: np.ndarray, N: int) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    M, K = x.shape
    scratch = np.zeros(M * K // 64 * 80, dtype=np.uint8)
    out = np.zeros((M, N), dtype=np.float32)
    lib().ora_linear_forward(_p(x), M, N, K, _p(b16), _p(b32), _p(scratch), _p(out))
    return out


def linear_forward_fast(x: np.ndarray, b16: np.ndarray, b32: np.ndarray, N: int, threads: int = 0) -> np.ndarray:
    """linear_forward through the AVX2+OpenMP port (bit-identical to the scalar functions, see
    tests/test_oracle_avx2.py): for full-size checks that the scalar oracle would take minutes for."""
    x = np.ascontiguousarray(x, np.float32)
    M, K = x.shape
    L = avx()
    threads = threads or L.avx_max_threads()
    out = np.zeros((M, N), dtype=np.float32)
    if M > 1:
        a = np.zeros(M * K // 64 * 80, dtype=np.uint8)
        L.avx_quantize_row_q8_1_repack_fp32(_p(x), _p(a), x.size)
        L.avx_gemm_repack_A81W41_fp32(_p(a), _p(b32), _p(out), M, N, K, threads)
    else:
        a = np.zeros(K // 64 * 72, dtype=np.uint8)
        L.avx_quantize_row_q8_1_repack_fp16(_p(x), _p(a), x.size)
        L.avx_gemv_repack_A81W41_fp16(_p(a), _p(b16), _p(out), 1, N, K, threads)
    return out


def quantize_weight_q41(w: np.ndarray):
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    w4 = np.zeros((N, K // 2), np.uint8)
    scale = np.zeros((N, K // 32), np.float32)
    offset = np.zeros((N, K // 32), np.float32)
    lib().ora_quantize_weight_q41(_p(w), N, K, _p(w4), _p(scale), _p(offset))
    return w4, scale, offset


# ------------------------------------------------------------------ A80W40 variant

FILL = 0xA5  # bytes the A80W40 writers must leave alone are pre-set to this


def repack_w80(w4: np.ndarray, scale: np.ndarray, K: int, N: int) -> np.ndarray:
    out = np.full(N * K // 512 * 320, FILL, dtype=np.uint8)
    lib().ora_repack_w80_weight(K, N, 32, _p(out), _p(np.ascontiguousarray(scale, np.float32)),
                                _p(np.ascontiguousarray(w4, np.uint8)))
    return out


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    assert x.size % 64 == 0
    out = np.full(x.size // 64 * 72, FILL, dtype=np.uint8)
    lib().ora_quantize_row_q8_0_repack(_p(x), _p(out), x.size)
    return out


def gemv_a80w40(a_blob: np.ndarray, b_blob: np.ndarray, N: int, K: int) -> np.ndarray:
    out = np.zeros(N, dtype=np.float32)
    lib().ora_gemv_repack_A80W40(_p(a_blob), _p(b_blob), _p(out), 1, N, K)
    return out


def gemm_a80w40(a_blob: np.ndarray, b_blob: np.ndarray, M: int, N: int, K: int) -> np.ndarray:
    out = np.zeros((M, N), dtype=np.float32)
    lib().ora_gemm_repack_A80W40(_p(a_blob), _p(b_blob), _p(out), M, N, K)
    return out


def block_idot_w80(a_blob, b_blob, M: int, N: int, K: int) -> np.ndarray:
    out = np.zeros((M, N, K // 32), dtype=np.int32)
    lib().ora_block_idot_w80(_p(a_blob), _p(b_blob), _p(out), M, N, K)
    return out


def quantize_weight_q40(w: np.ndarray):
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    w4 = np.zeros((N, K // 2), np.uint8)
    scale = np.zeros((N, K // 32), np.float32)
    lib().ora_quantize_weight_q40(_p(w), N, K, _p(w4), _p(scale))
    return w4, scale


# ------------------------------------------------------------------ AVX2 + OpenMP port (timed CPU baseline)

AVX_BRANCHES = {  # integer-dot branch of the reference's lib.h:45-55 -> (library, /proc/cpuinfo flags it needs)
    "avx512vnni": ("liba81w41_cpu_avx512vnni.so", {"avx512_vnni", "avx512vl", "avx512f", "avx2", "fma", "f16c"}),
    "avxvnni": ("liba81w41_cpu_avxvnni.so", {"avx_vnni", "avx2", "fma", "f16c"}),
    "avx2": ("liba81w41_cpu_avx2.so", {"avx2", "fma", "f16c"}),
}
_avx_libs = {}


def cpu_flags():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def avx_branches_supported():
    """Branches this host's CPU can run, best first (the order the reference's #if chain prefers)."""
    flags = cpu_flags()
    return [b for b, (_, need) in AVX_BRANCHES.items() if need <= flags]


def avx(branch=None):
    """The AVX2+OpenMP port; ``branch`` None = the best integer-dot branch this CPU supports."""
    global _avx
    if branch is None:
        if _avx is not None:
            return _avx
        sup = avx_branches_supported()
        if not sup:
            raise OSError("this CPU lacks AVX2/FMA/F16C: the CPU-baseline port cannot run here")
        _avx = avx(sup[0])
        return _avx
    if branch not in _avx_libs:
        L = _load(os.path.join(_HERE, AVX_BRANCHES[branch][0]))
        L.avx_dot_branch.restype = C.c_char_p
        _avx_libs[branch] = _bind_avx(L)
    return _avx_libs[branch]


def _bind_avx(L):
    if True:
        for name in ("avx_quantize_row_q8_1_repack_fp16", "avx_quantize_row_q8_1_repack_fp32"):
            getattr(L, name).argtypes = [_vp, _vp, _i64]
            getattr(L, name).restype = None
        for name in ("avx_gemv_repack_A81W41_fp16", "avx_gemm_repack_A81W41_fp32"):
            getattr(L, name).argtypes = [_vp, _vp, _vp, _i, _i, _i, _i]
            getattr(L, name).restype = None
        L.avx_max_threads.restype = _i
    return L
