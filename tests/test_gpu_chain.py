"""Chains of overlapping launches (a81w41_context_chain_*): one-row calls that start while their predecessor
runs and wait for it inside the kernel.  A chained call must return the bits of the plain call, eagerly and
replayed from a captured graph; a wait that can never be satisfied must give up, leave the kernel running to
its end, and be reported by the host."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# (N, K) of a dependent chain: each layer's input is the previous layer's output.  Widths are chosen so that
# the launches have one and several rounds of column groups, 1 to 8 waves per group, and K/64 not a multiple of 16.
CHAIN = [(1024, 512), (4096, 1024), (576, 4096), (12288, 576), (4096, 12288), (1024, 4096), (512, 1024)]


@pytest.fixture(scope="module")
def layers(pkg, synth, ora):
    ctx = pkg.ops.Context(max_rows=4, max_cols=12288)
    out = []
    for i, (N, K) in enumerate(CHAIN):
        w4, scale, offset = synth.weight_files(N, K, 300 + i)
        out.append((pkg.ops.Linear.from_arrays(w4, scale, offset, N=N, K=K, ctx=ctx),
                    ora.repack(w4, scale, offset, K, N, fp32=False), N, K))
    return ctx, out


def _run(layers, x, chained, ctx):
    import torch

    ys = []
    if chained:
        ctx.chain_begin()
    try:
        for lin, _, _, _ in layers:
            x = lin.forward(x)
            ys.append(x)
    finally:
        if chained:
            ctx.chain_end()
    torch.cuda.synchronize()
    return [y.cpu().numpy() for y in ys]


def test_chained_calls_return_the_bits_of_plain_calls(pkg, synth, ora, layers):
    import torch

    ctx, ls = layers
    x = torch.from_numpy(synth.activations(1, CHAIN[0][1], seed=11)).cuda()
    plain = _run(ls, x, False, ctx)
    for rep in range(20):
        got = _run(ls, x, True, ctx)
        for i, (a, b) in enumerate(zip(plain, got)):
            assert np.array_equal(a, b), (rep, i)
    assert not ctx.chain_gave_up()
    # and the plain calls are the oracle's, link by link, from the GPU's own inputs
    xin = x.cpu().numpy()
    for (lin, b16, N, K), y in zip(ls, plain):
        want = ora.gemv_fp16(ora.quantize(xin, fp32=False), b16, N, K)
        assert np.linalg.norm(y - want) <= 1e-4 * np.linalg.norm(want)
        xin = y


def test_chain_replayed_from_a_graph(pkg, synth, layers):
    """The chain captured once (both of its streams) and replayed: every replay, with other work and
    synchronisations in between, returns the eager result -- the counters are back at zero after each run."""
    import torch

    ctx, ls = layers
    x = torch.from_numpy(synth.activations(1, CHAIN[0][1], seed=12)).cuda()
    plain = _run(ls, x, False, ctx)
    outs = [torch.empty(1, N, dtype=torch.float32, device="cuda") for N, _ in CHAIN]
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream, capture_error_mode="thread_local"):
            ctx.chain_begin()
            cur = x
            for (lin, _, _, _), o in zip(ls, outs):
                cur = lin.forward(cur, out=o)
            ctx.chain_end()
    for rep in range(6):
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, o) in enumerate(zip(plain, outs)):
            assert np.array_equal(a, o.cpu().numpy()), (rep, i)
        eager = _run(ls, x, rep % 2 == 0, ctx)  # the program's own eager work between the replays
        assert np.array_equal(eager[-1], plain[-1])
    assert not ctx.chain_gave_up()


def test_forward_multi_inside_a_chain(pkg, synth):
    import torch

    ctx = pkg.ops.Context(max_rows=4, max_cols=4096)
    K = 1024
    ls = []
    for i, N in enumerate((512, 128, 128)):
        w4, scale, offset = synth.weight_files(N, K, 340 + i)
        ls.append(pkg.ops.Linear.from_arrays(w4, scale, offset, N=N, K=K, ctx=ctx))
    x = torch.from_numpy(synth.activations(1, K, seed=13)).cuda()
    plain = [y.cpu().numpy() for y in pkg.ops.Linear.forward_multi(ls, x)]
    ctx.chain_begin()
    first = ls[0].forward(x)                       # a link in front, so that the grouped call has to wait
    got = pkg.ops.Linear.forward_multi(ls, x)
    ctx.chain_end()
    torch.cuda.synchronize()
    assert np.array_equal(first.cpu().numpy(), plain[0])
    for a, b in zip(plain, got):
        assert np.array_equal(a, b.cpu().numpy())
    assert not ctx.chain_gave_up()


def test_chain_rules_are_checked(pkg, synth, layers):
    import torch

    ctx, ls = layers
    x = torch.from_numpy(synth.activations(3, CHAIN[0][1], seed=14)).cuda()
    with pytest.raises(pkg.capi.A81W41Error):
        ctx.chain_end()                            # nothing open
    ctx.chain_begin()
    try:
        with pytest.raises(pkg.capi.A81W41Error):
            ctx.chain_begin()                      # already open
        with pytest.raises(pkg.capi.A81W41Error):
            ls[0][0].forward(x)                    # three rows
        with torch.cuda.stream(torch.cuda.Stream()):
            with pytest.raises(pkg.capi.A81W41Error):
                ls[0][0].forward(x[:1])            # another stream than the chain's
    finally:
        ctx.chain_end()
    torch.cuda.synchronize()
    assert not ctx.chain_gave_up()


def test_a_wait_that_cannot_be_satisfied_gives_up(pkg, synth, layers):
    """Forced from the host: the link waits on a counter nothing counts on, with a spin limit of 3 polls.  The
    kernel gives up, still runs to its end (its input is there, so even its output is right), the host reports
    it once, and the next chain works."""
    import torch

    ctx, ls = layers
    lin, _, N, K = ls[1]
    x = torch.from_numpy(synth.activations(1, K, seed=15)).cuda()
    want = lin.forward(x).cpu().numpy()
    y = torch.zeros(1, N, dtype=torch.float32, device="cuda")
    lib = pkg.capi.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    pkg.capi.check(lib.a81w41_context_chain_selfcheck_stuck_wait(lin.handle, C.c_void_p(x.data_ptr()),
                                                                 C.c_void_p(y.data_ptr()), 3, stream))
    torch.cuda.synchronize()
    assert ctx.chain_gave_up()
    assert not ctx.chain_gave_up()                 # reported once, then cleared
    assert np.array_equal(y.cpu().numpy(), want)
    x0 = torch.from_numpy(synth.activations(1, CHAIN[0][1], seed=11)).cuda()
    assert np.array_equal(_run(ls, x0, True, ctx)[-1], _run(ls, x0, False, ctx)[-1])
    assert not ctx.chain_gave_up()
