"""Parity of the HIP path against the CPU oracle, through the C ABI.

Bars (from the workload definition): quantized activations and per-block int32
dots bit-exact; fp32 outputs within 1e-4 relative error normalised by the row
norm (TOL below)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-4


@pytest.fixture(scope="module")
def torch():
    import torch as t

    assert t.cuda.is_available()
    return t


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same_bytes(got, want):
    """Compact byte comparison (a failing array_equal would print megabytes)."""
    got, want = np.asarray(got).ravel(), np.asarray(want).ravel()
    if got.shape != want.shape:
        return f"shape {got.shape} vs {want.shape}"
    bad = np.flatnonzero(got != want)
    if bad.size == 0:
        return ""
    return f"{bad.size} of {got.size} differ; first at {bad[:8].tolist()}: got {got[bad[:8]].tolist()} want {want[bad[:8]].tolist()}"


def row_err(got, want):
    got = np.asarray(got, np.float64).reshape(want.shape)
    w = np.asarray(want, np.float64)
    return float(np.max(np.linalg.norm(got - w, axis=-1) / np.maximum(np.linalg.norm(w, axis=-1), 1e-30)))


# ------------------------------------------------------------------ quantizer: bit-exact

@pytest.mark.parametrize("fp32", [False, True])
@pytest.mark.parametrize("M,K", [(1, 64), (1, 4096), (3, 12288), (37, 1024), (322, 4096)])
def test_quantize_bit_exact(pkg, ora, synth, torch, fp32, M, K):
    x = synth.activations(M, K, seed=71, outliers=True)
    if M >= 3:
        x[1, 64:96] = 0.0                      # all-zero block: d = id = 0
        x[2, :32] *= np.float32(1e-30)         # fp16 scale underflows to a subnormal / zero
        x[0, 32:64] *= np.float32(3e3)
    got = pkg.ops.quantize(dev(torch, x), fp32).cpu().numpy()
    assert not same_bytes(got, ora.quantize(x, fp32))


def test_quantize_special_values(pkg, ora, torch):
    x = np.zeros((8, 64), np.float32)
    # 127/amax overflows: q = -128 everywhere, wrapped sum (pinned against x86 in tests/test_oracle_avx2.py)
    x[6, :32] = np.float32(1e-38) * np.linspace(-1.0, 1.0, 32, dtype=np.float32)
    x[6, 5] = 0.0
    x[6, 32:] = np.float32(3e-39)
    x[6, 40] = 0.0
    x[7, 17] = np.float32(-2e-38)
    x[7, 32:] = np.float32(3.8e-37)
    x[1, 7] = 3.5
    x[2, 40] = -2.0
    x[3, :] = 1.0
    x[4, :] = np.linspace(-1, 1, 64, dtype=np.float32)       # exact .5 ties after scaling
    x[5, :32] = np.float32(1e-42)                            # fp32 subnormal inputs
    x[5, 32:] = np.float32(3e38)
    for fp32 in (False, True):
        got = pkg.ops.quantize(dev(torch, x), fp32).cpu().numpy()
        assert not same_bytes(got, ora.quantize(x, fp32)), fp32


def test_quantize_unaligned_input(pkg, ora, synth, torch):
    x = synth.activations(1, 256 + 64, seed=72).ravel()
    xd = dev(torch, x)
    got = pkg.ops.quantize(xd[1:257], True).cpu().numpy()    # 4-byte aligned only
    assert not same_bytes(got, ora.quantize(x[1:257], True))


# ------------------------------------------------------------------ int32 block dots: bit-exact

@pytest.mark.parametrize("fp32", [False, True])
def test_block_idot_bit_exact(pkg, ora, synth, torch, fp32):
    M, N, K = (5, 40, 320) if fp32 else (1, 64, 1024)
    w4, s, o = synth.weight_files(N, K, 73)
    x = synth.activations(M, K, 74, outliers=True)
    bw = ora.repack(w4, s, o, K, N, fp32)
    ba = ora.quantize(x, fp32)
    got = pkg.ops.block_idot(dev(torch, ba), fp32, dev(torch, bw), fp32, M, N, K).cpu().numpy()
    assert not same_bytes(got, ora.block_idot(ba, fp32, bw, fp32, M, N, K))


# ------------------------------------------------------------------ GEMV (M = 1, fp16 params)

@pytest.mark.parametrize("N,K", [(8, 64), (8, 1024), (16, 1088), (40, 192), (256, 4096), (4096, 4096),
                                 (1024, 4096), (512, 12288),
                                 (16, 65536), (8, 106304)])     # rows that need more than 64 KiB of LDS, and the longest
def test_gemv_parity(pkg, ora, synth, torch, N, K):
    w4, s, o = synth.weight_files(N, K, 75)
    x = synth.activations(1, K, 76)
    bw = ora.repack(w4, s, o, K, N, False)
    ba = ora.quantize(x, False)
    got = pkg.ops.gemv_fp16(dev(torch, ba), dev(torch, bw), N, K).cpu().numpy()
    want = ora.gemv_fp16(ba, bw, N, K)
    assert row_err(got, want) <= TOL
    # far tighter than the bar in practice: only the fp32 summation order differs
    assert row_err(got, want) <= 5e-6


def test_random_shapes_through_the_layer(pkg, ora, synth, torch):
    """Forty seeded random (M, N, K): N any multiple of 8, K any multiple of 64, M from 1 to 300, through
    `Linear.forward` (the reference's M-dispatch) -- whichever kernel the shape lands on, same bar."""
    rng = np.random.default_rng(4242)
    for case in range(40):
        M = int(rng.choice([1, 1, 2, 3, 5, 8, 9, 17, 33, 64, 65, 127, 200, 300]))
        N = 8 * int(rng.integers(1, 160))
        K = 64 * int(rng.integers(1, 40))
        w4, s, o = synth.weight_files(N, K, 9000 + case)
        x = synth.activations(M, K, 9100 + case, outliers=bool(case & 1))
        got = pkg.ops.Linear.from_arrays(w4, s, o, N, K).forward(dev(torch, x)).cpu().numpy()
        fp32 = M > 1                                  # QwenOperator.cc:80-124: fp16 blocks + GEMV for one row
        ba, bw = ora.quantize(x, fp32), ora.repack(w4, s, o, K, N, fp32)
        want = ora.gemm_fp32(ba, bw, M, N, K) if fp32 else ora.gemv_fp16(ba, bw, N, K)
        assert row_err(got, want) <= 5e-6, (case, M, N, K)


def test_gemv_row_too_long_is_an_error(pkg, ora, synth, torch):
    N, K = 8, 106304 + 64
    bw = torch.zeros(N * K // 512 * 320, dtype=torch.uint8, device="cuda")
    ba = torch.zeros(K // 64 * 72, dtype=torch.uint8, device="cuda")
    with pytest.raises(pkg.capi.A81W41Error, match="max K = 106304"):
        pkg.ops.gemv_fp16(ba, bw, N, K)


def test_gemv_overwrites_and_is_deterministic(pkg, ora, synth, torch):
    N, K = 64, 4096
    w4, s, o = synth.weight_files(N, K, 77)
    bw = dev(torch, ora.repack(w4, s, o, K, N, False))
    ba = dev(torch, ora.quantize(synth.activations(1, K, 78), False))
    a = pkg.ops.gemv_fp16(ba, bw, N, K).cpu().numpy()
    b = pkg.ops.gemv_fp16(ba, bw, N, K).cpu().numpy()
    assert np.array_equal(a, b)


def test_gemv_extreme_codes(pkg, ora, torch):
    """codes 15 x q = -127 everywhere: block dots hit -60960, the int path must not wrap."""
    N, K = 16, 256
    w4 = np.full((N, K // 2), 0xFF, np.uint8)
    sc = np.full((N, K // 32), 0.01, np.float32)
    of = np.full((N, K // 32), -0.08, np.float32)
    bw = ora.repack(w4, sc, of, K, N, False)
    ba = ora.quantize(np.full((1, K), -1.0, np.float32), False)
    got = pkg.ops.gemv_fp16(dev(torch, ba), dev(torch, bw), N, K).cpu().numpy()
    assert row_err(got, ora.gemv_fp16(ba, bw, N, K)) <= TOL


# ------------------------------------------------------------------ GEMM (M > 1, fp32 params)

@pytest.mark.parametrize("M,N,K", [(2, 8, 64), (7, 40, 192), (33, 72, 320), (64, 64, 1024), (6, 256, 4096),
                                   (322, 96, 1024), (45, 32, 12288), (130, 136, 2048), (70, 520, 64),
                                   (65, 8, 128), (3, 16, 1088), (5, 4096, 4096), (8, 64, 12288), (4, 136, 12288),
                                   (8, 1024, 4096), (9, 64, 12288),
                                   # 9..32 rows on narrow layers: the one-row-panel kernel with register loads ...
                                   (9, 8, 64), (17, 136, 256), (32, 128, 4096), (31, 1000, 2048), (12, 4096, 4096),
                                   (32, 1024, 12288),
                                   # ... and with wave-private LDS stages on wide ones: ragged N, K not a multiple of
                                   # the ring or of the waves, shared K, more panels than workgroup slots
                                   (8, 4096, 12288), (7, 2056, 8192), (9, 8200, 64), (17, 9000, 320), (32, 8192, 1024), (20, 72000, 256), (25, 12288, 4096), (21, 1032, 320),
                                   # more tiles than workgroup slots (768): whole rounds plus a K-split partial
                                   # round, ragged rows and columns; 513..682 tiles: the two-per-CU schedule
                                   (256, 16384, 256), (322, 12288, 256), (1030, 4104, 256), (384, 24576, 512), (640, 4096, 256)])
def test_gemm_parity(pkg, ora, synth, torch, M, N, K):
    w4, s, o = synth.weight_files(N, K, 79)
    s = s * np.float32(1.0371)          # fp32 params that fp16 cannot hold
    x = synth.activations(M, K, 80, outliers=True)
    bw = ora.repack(w4, s, o, K, N, True)
    ba = ora.quantize(x, True)
    got = pkg.ops.gemm_fp32(dev(torch, ba), dev(torch, bw), M, N, K).cpu().numpy()
    want = ora.gemm_fp32(ba, bw, M, N, K)
    assert row_err(got, want) <= TOL
    assert row_err(got, want) <= 5e-6


def test_gemm_m1_matches_fp32_oracle_not_fp16(pkg, ora, synth, torch):
    """The GEMM entry point keeps fp32 parameters for any M, as the reference function does."""
    N, K = 64, 4096
    w4, s, o = synth.weight_files(N, K, 81)
    x = synth.activations(1, K, 82)
    bw = ora.repack(w4, s, o, K, N, True)
    ba = ora.quantize(x, True)
    got = pkg.ops.gemm_fp32(dev(torch, ba), dev(torch, bw), 1, N, K).cpu().numpy()
    assert row_err(got, ora.gemm_fp32(ba, bw, 1, N, K)) <= 5e-6


# ------------------------------------------------------------------ layer object: M-dispatch

@pytest.mark.parametrize("M", [1, 2, 13])
def test_linear_forward_dispatch(pkg, ora, synth, torch, M):
    N, K = 128, 1024
    w4, s, o = synth.weight_files(N, K, 83)
    layer = pkg.Linear.from_arrays(w4, s, o, N=N, K=K)
    b16 = ora.repack(w4, s, o, K, N, False)
    b32 = ora.repack(w4, s, o, K, N, True)
    x = synth.activations(M, K, 84)
    want = ora.linear_forward(x, b16, b32, N)
    got = layer.forward(dev(torch, x)).cpu().numpy()
    assert row_err(got, want) <= TOL
    got_h = layer.forward_host(x)
    assert np.array_equal(got_h, got)
    # the shared scratch holds this call's quantised activations, like the reference's buffer
    nbytes = M * K // 64 * (80 if M > 1 else 72)
    scratch = layer.ctx.activation_scratch(nbytes).cpu().numpy()
    assert not same_bytes(scratch, ora.quantize(x, fp32=(M > 1)))
    if M == 1:
        # the fp32-parameter result is ~1e-3 away: passing proves the fp16 path ran
        other = ora.gemm_fp32(ora.quantize(x, True), b32, 1, N, K)
        assert row_err(got, other) > 10 * row_err(got, want)


@pytest.mark.parametrize("N,K", [(8, 64), (4096, 4096), (24, 1088), (20000, 4096), (256, 12288)])
def test_linear_forward_m1_fused_prologue(pkg, ora, synth, torch, N, K):
    """M == 1 runs one kernel that quantises x itself; also more column groups than
    persistent workgroups (N = 20000 -> 2500 groups over 2048 workgroups)."""
    w4, s, o = synth.weight_files(N, K, 87)
    layer = pkg.Linear.from_blobs(ora.repack(w4, s, o, K, N, False), None, N, K)
    x = synth.activations(1, K, 88, outliers=True)
    got = layer.forward(dev(torch, x)).cpu().numpy()
    ba = ora.quantize(x, False)
    want = ora.gemv_fp16(ba, ora.repack(w4, s, o, K, N, False), N, K)
    assert row_err(got, want) <= 5e-6
    assert not same_bytes(layer.ctx.activation_scratch(K // 64 * 72).cpu().numpy(), ba)
    # x that is only 4-byte aligned takes the two-kernel path (quantiser, then GEMV): same numbers
    xd = dev(torch, np.concatenate([np.zeros(1, np.float32), x.ravel()]))[1:]
    assert xd.data_ptr() % 16 != 0
    got2 = layer.forward(xd).cpu().numpy()
    assert np.array_equal(got2.ravel(), got.ravel())


@pytest.mark.parametrize("M", [1, 5])
@pytest.mark.parametrize("Ns", [(512, 128, 128), (64, 8, 24, 40, 16)])
def test_forward_multi_equals_separate_calls(pkg, ora, synth, torch, M, Ns):
    """q/k/v-style fused call sites: one call (one launch for M == 1, two when more than
    four layers) must give exactly what separate forward calls give."""
    K = 1024
    layers = []
    for i, N in enumerate(Ns):
        w4, s, o = synth.weight_files(N, K, 90 + i)
        layers.append(pkg.Linear.from_arrays(w4, s, o, N=N, K=K))
    x = dev(torch, synth.activations(M, K, 95))
    sep = [l.forward(x).cpu().numpy() for l in layers]
    multi = [y.cpu().numpy() for y in pkg.Linear.forward_multi(layers, x)]
    for a, b in zip(sep, multi):
        assert np.array_equal(a, b)


def test_linear_load_from_files(pkg, ora, synth, torch, tmp_path):
    N, K = 64, 512
    w4, s, o = synth.weight_files(N, K, 85)
    d = str(tmp_path) + "/"
    w4.tofile(d + "weight_int4.bin")
    s.tofile(d + "scaling_factor_int4.bin")
    o.tofile(d + "offset_int4.bin")
    np.zeros((N, K // 32), np.int8).tofile(d + "zero_point_int4.bin")
    layer = pkg.Linear.load(d, N=N, K=K)
    x = synth.activations(3, K, 86)
    want = ora.linear_forward(x, ora.repack(w4, s, o, K, N, False), ora.repack(w4, s, o, K, N, True), N)
    assert row_err(layer.forward(dev(torch, x)).cpu().numpy(), want) <= TOL
    with pytest.raises(pkg.capi.A81W41Error):
        pkg.Linear.load(d + "missing/", N=N, K=K)


def test_cpp_host_mirror(pkg, ora, torch, tmp_path):
    """The C++ mirror of Qwen_Linear_with_bias_Int4 (host/QwenLinearInt4.hpp) driven by its
    self-check binary: same seeded layer rebuilt here, checksums compared with the oracle."""
    import os
    import re
    import subprocess

    exe = os.path.join(os.path.dirname(pkg.__file__), "host", "host_example")
    assert os.path.exists(exe), "build it with `make -C qwen3.ink.cpp_amd/host`"
    out = subprocess.run([exe, "--dir", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "file-loaded layer matches the array-built one" in out.stdout
    # replay the example's LCG
    state = [7]

    def lcg():
        state[0] = (state[0] * 1664525 + 1013904223) & 0xFFFFFFFF
        return state[0]

    N, K = 64, 256
    w4 = np.array([lcg() >> 24 for _ in range(N * K // 2)], np.uint8).reshape(N, K // 2)
    scale = np.zeros(N * K // 32, np.float32)
    for i in range(scale.size):
        scale[i] = np.float32(0.001) + np.float32(lcg() >> 20) * np.float32(1e-6)
    scale = scale.reshape(N, K // 32)
    offset = np.float32(-8.0) * scale
    b16 = ora.repack(w4, scale, offset, K, N, False)
    b32 = ora.repack(w4, scale, offset, K, N, True)
    sums = [float(v) for v in re.findall(r"checksum=(-?[0-9.]+)", out.stdout)]
    assert len(sums) == 2
    for M, got in zip((1, 3), sums):
        x = np.array([np.float32((lcg() >> 16) - 32768) / np.float32(16384.0) for _ in range(M * K)], np.float32)
        want = ora.linear_forward(x.reshape(M, K), b16, b32, N)
        assert abs(got - float(want.astype(np.float64).sum())) <= 1e-4 * float(np.abs(want).sum())


def test_gemm_scratch_is_left_clean_between_shapes(pkg, ora, synth, torch):
    """Calls with and without a K-split, of different sizes, one after the other on one device:
    each must match the oracle and repeat bit for bit (the split path's counters and partial
    tiles are shared per device and have to be back at rest after every launch)."""
    cases = [(322, 256, 1024), (64, 64, 1024), (33, 72, 320), (130, 136, 2048), (322, 256, 1024), (64, 64, 1024)]
    blobs = {}
    for rep in range(2):
        for (M, N, K) in cases:
            if (M, N, K) not in blobs:
                w4, s, o = synth.weight_files(N, K, 301 + N)
                x = synth.activations(M, K, 302 + M, outliers=True)
                ba, bw = ora.quantize(x, True), ora.repack(w4, s, o, K, N, True)
                blobs[(M, N, K)] = (dev(torch, ba), dev(torch, bw), ora.gemm_fp32(ba, bw, M, N, K), None)
            a, b, want, first = blobs[(M, N, K)]
            got = pkg.ops.gemm_fp32(a, b, M, N, K).cpu().numpy()
            assert row_err(got, want) <= TOL
            if first is None:
                blobs[(M, N, K)] = (a, b, want, got)
            else:
                assert np.array_equal(got, first)


def test_forward_m_gt_1_replays_from_a_hip_graph(pkg, ora, synth, torch):
    """The M > 1 forward (quantiser kernel + GEMM with its split-K scratch) captured into a HIP
    graph: every replay, with eager work between replays, equals the eager result."""
    M, N, K = 100, 512, 1024
    w4, s, o = synth.weight_files(N, K, 311)
    layer = pkg.Linear.from_arrays(w4, s, o, N, K)
    x = dev(torch, synth.activations(M, K, 312))
    eager = layer.forward(x).clone()
    y = torch.empty_like(eager)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        layer.forward(x, out=y)          # warm-up on the capture stream's side
    side.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        layer.forward(x, out=y)
    other = dev(torch, synth.activations(M, K, 313))
    for i in range(4):
        y.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)
        layer.forward(other)             # eager work between replays, same scratch
        torch.cuda.synchronize()


def test_gemm_calls_on_two_streams_do_not_share_partial_tiles(pkg, ora, synth, torch):
    """K-split GEMM launches that overlap in time on two streams (the free-standing entry point keeps one
    scratch per stream) and layer calls on two contexts (each owns its scratch): every result equals the
    one computed alone."""
    M, N, K = 322, 1024, 4096           # 96 tiles, K cut in four: partial tiles in use
    cases = []
    for seed in (501, 503):
        w4, s, o = synth.weight_files(N, K, seed)
        x = synth.activations(M, K, seed + 1, outliers=True)
        ba, bw = ora.quantize(x, True), ora.repack(w4, s, o, K, N, True)
        a, b = dev(torch, ba), dev(torch, bw)
        cases.append((a, b, pkg.ops.gemm_fp32(a, b, M, N, K).clone(), dev(torch, x), (w4, s, o)))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.empty((M, N), dtype=torch.float32, device="cuda") for _ in range(6)] for _ in range(2)]
    for i, st in enumerate(streams):        # first call on each stream creates its scratch
        with torch.cuda.stream(st):
            pkg.ops.gemm_fp32(cases[i][0], cases[i][1], M, N, K, out=outs[i][0])
    torch.cuda.synchronize()
    for r in range(6):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                pkg.ops.gemm_fp32(cases[i][0], cases[i][1], M, N, K, out=outs[i][r])
    torch.cuda.synchronize()
    for i in range(2):
        for r in range(6):
            assert torch.equal(outs[i][r], cases[i][2]), (i, r)
    # the same through two layer objects on two contexts
    layers = []
    for i in range(2):
        ctx = pkg.ops.Context(max_rows=M, max_cols=K)
        w4, s, o = cases[i][4]
        layers.append(pkg.Linear.from_arrays(w4, s, o, N=N, K=K, ctx=ctx))
    alone = [layers[i].forward(cases[i][3]).clone() for i in range(2)]
    torch.cuda.synchronize()
    for r in range(6):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                layers[i].forward(cases[i][3], out=outs[i][r])
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(alone[i], cases[i][2])
        for r in range(6):
            assert torch.equal(outs[i][r], alone[i]), (i, r)


@pytest.mark.parametrize("M,N,K", [(33, 8, 64), (40, 136, 256), (64, 64, 1024), (65, 1000, 2048), (128, 128, 4096),
                                   (130, 136, 2048), (322, 1024, 4096), (322, 256, 1024), (256, 16384, 256),
                                   (1030, 4104, 256), (640, 4096, 256), (384, 24576, 512), (100, 512, 12288)])
def test_layer_forward_block_scaled_kernel(pkg, ora, synth, torch, M, N, K):
    """The layer object's second M > 32 kernel, on the block-scaled fp6 matrix ops from its own operand
    formats (by default only for shapes where it is the faster one; forced here): ragged rows and columns
    (panels padded to 32), one tile shared by many workgroups, many tiles per workgroup, K from one 64-K
    super-block to 12288.  Same bars as the other kernels; the scratch still receives the reference's 80 B
    blocks; results repeat bit for bit."""
    w4, s, o = synth.weight_files(N, K, 601)
    s = s * np.float32(1.0371)          # fp32 params that fp16 cannot hold
    x = synth.activations(M, K, 602, outliers=True)
    ctx = pkg.ops.Context(max_rows=M, max_cols=K)
    layer = pkg.Linear.from_arrays(w4, s, o, N=N, K=K, ctx=ctx)
    layer.set_kernel("block_scaled")
    xd = dev(torch, x)
    got = layer.forward(xd).cpu().numpy()
    b16, b32 = ora.repack(w4, s, o, K, N, False), ora.repack(w4, s, o, K, N, True)
    want = ora.linear_forward_fast(x, b16, b32, N)
    assert row_err(got, want) <= TOL
    assert row_err(got, want) <= 3e-5      # the min terms run on 16-bit-significand pieces: below 2^-16 of a term
    qa = ctx.activation_scratch(M * K // 64 * 80).cpu().numpy()
    assert not same_bytes(qa, ora.quantize(x, True))
    assert np.array_equal(layer.forward(xd).cpu().numpy(), got)


def test_layer_kernel_choice_at_full_width(pkg, ora, synth, torch):
    """gate_proj of Qwen3-8B with the 322-row prompt of the reference's benchmark: by default the call runs on the
    block-scaled kernel (same bits as when forced), the int8 kernel stays selectable, both meet the bar."""
    M, N, K = 322, 12288, 4096
    w4, s, o = synth.weight_files(N, K, 611)
    x = synth.activations(M, K, 612, outliers=True)
    ctx = pkg.ops.Context(max_rows=M, max_cols=K)
    layer = pkg.Linear.from_arrays(w4, s, o, N=N, K=K, ctx=ctx)
    xd = dev(torch, x)
    auto = layer.forward(xd).cpu().numpy()
    layer.set_kernel("block_scaled")
    forced = layer.forward(xd).cpu().numpy()
    layer.set_kernel("int8")
    int8 = layer.forward(xd).cpu().numpy()
    layer.set_kernel("auto")
    assert np.array_equal(auto, forced)
    assert not np.array_equal(auto, int8)   # different summation trees
    b16, b32 = ora.repack(w4, s, o, K, N, False), ora.repack(w4, s, o, K, N, True)
    want = ora.linear_forward_fast(x, b16, b32, N)
    assert row_err(int8, want) <= TOL
    assert row_err(auto, want) <= 3e-5
    with pytest.raises(Exception):
        pkg.capi.check(pkg.capi.lib().a81w41_linear_set_kernel(layer.handle, 7))


def test_third_weight_copy_only_where_it_can_be_used(pkg, ora, synth, torch):
    """The block-scaled kernel's operand format (1 B per weight on top of the reference's two blobs) is built
    only for layers that a call their context admits can send to that kernel; the int8 choice frees it, the
    block-scaled choice builds it, and results are those of the int8 kernel to the path's bar either way."""
    K = 4096
    ctx = pkg.ops.Context(max_rows=512, max_cols=K)
    narrow_w = synth.weight_files(1024, K, 621)
    wide_w = synth.weight_files(12288, K, 622)
    narrow = pkg.Linear.from_arrays(*narrow_w, N=1024, K=K, ctx=ctx)     # k / v shape: never enough tiles at <= 512 rows
    wide = pkg.Linear.from_arrays(*wide_w, N=12288, K=K, ctx=ctx)        # gate shape: block-scaled from 256 rows on
    rb = narrow.resident_bytes()
    assert rb["block_scaled"] == 0 and rb["fp16_blob"] == 1024 * K * 5 // 8 and rb["fp32_blob"] == 1024 * K * 3 // 4
    assert wide.resident_bytes()["block_scaled"] == 12288 * K
    x = dev(torch, synth.activations(300, K, 623))
    base = narrow.forward(x).cpu().numpy()
    narrow.set_kernel("block_scaled")
    assert narrow.resident_bytes()["block_scaled"] == 1024 * K
    forced = narrow.forward(x).cpu().numpy()
    assert row_err(forced, base) <= 3e-5 and not np.array_equal(forced, base)
    narrow.set_kernel("int8")
    assert narrow.resident_bytes()["block_scaled"] == 0
    assert np.array_equal(narrow.forward(x).cpu().numpy(), base)
    wide.set_kernel("int8")
    assert wide.resident_bytes()["total"] == 12288 * K * 11 // 8
    wide.set_kernel("auto")
    assert wide.resident_bytes()["block_scaled"] == 12288 * K
    # a layer without an fp32-parameter blob (decode only) holds one copy
    only16 = pkg.Linear.from_blobs(ora.repack(*narrow_w, K, 1024, False), None, 1024, K, ctx)
    assert only16.resident_bytes() == {"total": 1024 * K * 5 // 8, "fp16_blob": 1024 * K * 5 // 8, "fp32_blob": 0, "block_scaled": 0}


def test_gemm_on_more_streams_than_scratches(pkg, ora, synth, torch):
    """The free-standing GEMM keeps one K-split scratch per stream, at most 16 per device: streams beyond that
    take over the least recently used scratch instead of failing.  20 fresh streams in turn, then the first
    again, all with the same bits."""
    M, N, K = 130, 136, 2048                       # splits K
    w4, s, o = synth.weight_files(N, K, 631)
    ba, bw = ora.quantize(synth.activations(M, K, 632), True), ora.repack(w4, s, o, K, N, True)
    a, b = dev(torch, ba), dev(torch, bw)
    ref = pkg.ops.gemm_fp32(a, b, M, N, K).clone()
    streams = [torch.cuda.Stream() for _ in range(20)]
    for st in streams + streams[:2]:
        with torch.cuda.stream(st):
            got = pkg.ops.gemm_fp32(a, b, M, N, K)
        st.synchronize()
        assert torch.equal(got, ref)


@pytest.mark.parametrize("M,N,K", [(2, 8, 64), (2, 12288, 4096), (3, 1024, 4096), (2, 4096, 6144), (6, 136, 1088), (8, 40, 1536),
                                   (4, 64, 3072), (3, 4096, 4160)])
def test_few_row_forward_quantises_in_its_prologue(pkg, ora, synth, torch, M, N, K):
    """Calls with few rows and M*K <= 12288 are one launch: every workgroup quantises the fp32 rows itself
    (quantize_row_q8_1_repack_fp32's arithmetic) on their way into LDS, workgroup 0 also writes the 80 B blocks
    to the scratch.  Scratch bit-exact, output the same bits as the contraction of the oracle-quantised rows by
    the same kernel without the prologue, all within the bar; shapes just above the limit take two launches."""
    w4, s, o = synth.weight_files(N, K, 641)
    s = s * np.float32(1.0371)
    x = synth.activations(M, K, 642, outliers=True)
    x[M - 1, :64] = 0.0                             # an all-zero block: d = 0, id = 0
    ctx = pkg.ops.Context(max_rows=8, max_cols=K)
    bw = ora.repack(w4, s, o, K, N, True)
    layer = pkg.Linear.from_blobs(None, bw, N, K, ctx)
    fused = M * K <= 12288
    assert layer.kernel_name(M).startswith("rows_fused" if fused else "rows ")
    got = layer.forward(dev(torch, x))
    ba = ora.quantize(x, True)
    assert np.array_equal(ctx.activation_scratch(M * K // 64 * 80).cpu().numpy(), ba)
    want = ora.gemm_fp32(ba, bw, M, N, K)
    assert row_err(got.cpu().numpy(), want) <= 5e-6
    # the same kernel without the prologue, on the quantised rows (the free-standing entry point)
    assert torch.equal(got, pkg.ops.gemm_fp32(dev(torch, ba), dev(torch, bw), M, N, K))


@pytest.mark.parametrize("N,K", [(4096, 4096), (12288, 4096), (4096, 12288), (4104, 4096), (2056, 320), (6144, 192)])
def test_9_to_32_rows_on_wide_layers_stage_their_rows_per_super_block(pkg, ora, synth, torch, N, K):
    """9 .. 32 rows on a layer wider than 2048 columns: the layer's quantiser launch also writes the 80 B blocks with
    the rows of a super-block next to each other, and the one-row-panel kernel stages them from there.  The scratch
    holds the oracle's blocks; the output has the bits of the free-standing entry point on those blocks (same
    kernel, rows staged from the reference's layout) and is within the bar; a call with fewer rows after one with
    more is not disturbed by the row slots the earlier call left behind."""
    w4, s, o = synth.weight_files(N, K, 661)
    s = s * np.float32(0.9371)
    bw = ora.repack(w4, s, o, K, N, True)
    ctx = pkg.ops.Context(max_rows=32, max_cols=K)
    layer = pkg.Linear.from_blobs(None, bw, N, K, ctx)
    for M in (32, 9, 17, 31):
        x = synth.activations(M, K, 662 + M, outliers=True)
        x[M - 1, 64:128] = 0.0                      # an all-zero block: d = 0, id = 0
        assert layer.kernel_name(M).startswith("rows32_staged")
        got = layer.forward(dev(torch, x))
        ba = ora.quantize(x, True)
        assert np.array_equal(ctx.activation_scratch(M * K // 64 * 80).cpu().numpy(), ba), M
        want = ora.gemm_fp32(ba, bw, M, N, K)
        assert row_err(got.cpu().numpy(), want) <= 5e-6, M
        assert torch.equal(got, pkg.ops.gemm_fp32(dev(torch, ba), dev(torch, bw), M, N, K)), M
        assert torch.equal(got, layer.forward(dev(torch, x))), M
