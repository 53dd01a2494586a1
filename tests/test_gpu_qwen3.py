"""The Qwen3 forward pass around the layer (a81w41_qwen3_*) against the numpy oracle on a tiny
seeded model: prefill, token-by-token decode, and greedy generation from the captured graph."""
import os

import numpy as np
import pytest

from oracle import qwen3_forward as qf
from tests.qwen3_fixture import TINY, build

pytestmark = pytest.mark.gpu

TOL = 5e-3   # logits, relative to their norm: fp32 summation orders + int8 re-quantisation of activations


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


@pytest.fixture(scope="module")
def models(pkg, synth, ora):
    gpu = pkg.Qwen3Model(**TINY)
    cpu = qf.Qwen3Oracle(**TINY)
    build(synth, ora, TINY, 900, gpu_model=gpu, oracle_model=cpu)
    return gpu, cpu


def test_prefill_then_decode_matches_oracle(models):
    gpu, cpu = models
    gpu.reset(); cpu.reset()
    prompt = [3, 99, 500, 7, 7, 123, 45, 256, 31, 8, 301, 2, 64]
    assert rel(gpu.forward(prompt), cpu.forward(prompt)) <= TOL
    for t in [17, 17, 400, 5, 111]:
        assert rel(gpu.forward([t]), cpu.forward([t])) <= TOL


@pytest.mark.parametrize("n_prompt", [1, 2, 5, 9, 40])
def test_prompt_lengths_cover_every_linear_kernel(models, n_prompt):
    """M = 1 (GEMV), 2..8 (few-row kernel), > 8 (matrix cores) all feed the same attention code."""
    gpu, cpu = models
    gpu.reset(); cpu.reset()
    ids = [(37 * i + 11) % TINY["vocab"] for i in range(n_prompt)]
    assert rel(gpu.forward(ids), cpu.forward(ids)) <= TOL


def test_greedy_generation_from_the_graph(models):
    gpu, cpu = models
    prompt = [9, 8, 7, 300, 301, 302, 5, 5, 5, 77, 140]
    n_new = 12
    gpu.reset()
    toks, t_pre, t_dec = gpu.generate_greedy(prompt, n_new)
    assert t_pre > 0 and t_dec > 0
    assert ((0 <= toks) & (toks < TINY["vocab"])).all()
    # teacher-forced check: at every step the token is the oracle's argmax, unless the oracle's
    # two best logits are closer than the parity tolerance
    cpu.reset()
    logits = cpu.forward(prompt)
    for i, tok in enumerate(toks):
        best = cpu.greedy(logits)
        if tok != best:
            gap = logits[best] - logits[tok]
            assert gap <= TOL * np.linalg.norm(logits), (i, tok, best, gap)
        if i + 1 < n_new:
            logits = cpu.forward([int(tok)])
    # a second run from scratch gives the same tokens, and eager decode agrees with the graph
    gpu.reset()
    toks2, _, _ = gpu.generate_greedy(prompt, n_new)
    assert np.array_equal(toks, toks2)
    gpu.reset()
    lg = gpu.forward(prompt)
    eager = []
    for i in range(n_new):
        eager.append(int(np.argmax(lg)))
        if i + 1 < n_new:
            lg = gpu.forward([eager[-1]])
    assert eager == [int(t) for t in toks]


def test_context_limits_are_errors(models, pkg):
    gpu, _ = models
    gpu.reset()
    with pytest.raises(pkg.capi.A81W41Error):
        gpu.forward(list(range(TINY["max_seq"] + 1)))
    with pytest.raises(pkg.capi.A81W41Error):
        gpu.generate_greedy([1, 2, 3], TINY["max_seq"])


def test_load_from_the_reference_directory_tree(models, pkg, synth, tmp_path):
    """a81w41_qwen3_load on a tree in the reference's layout (separate gate_proj / up_proj, fp32
    embedding, scaling.bin) gives the same model as setting the arrays one by one; with the
    oracle's cos/sin files in rotary_emb/ it still matches the oracle."""
    from tests.qwen3_fixture import arrays, write_reference_tree
    gpu, cpu = models
    a = arrays(synth, TINY, 900)
    prompt = [3, 99, 500, 7, 7, 123, 45, 256, 31, 8, 301]
    gpu.reset()
    want_prefill = gpu.forward(prompt)
    want_step = gpu.forward([17])
    root = str(tmp_path / "plain")
    write_reference_tree(root, a, TINY)
    loaded = pkg.Qwen3Model.load(root, **TINY)
    assert np.array_equal(loaded.forward(prompt), want_prefill)
    assert np.array_equal(loaded.forward([17]), want_step)
    root2 = str(tmp_path / "with_rotary")
    write_reference_tree(root2, a, TINY, rotary=(cpu.cos, cpu.sin))
    loaded2 = pkg.Qwen3Model.load(root2, **TINY)
    cpu.reset()
    assert rel(loaded2.forward(prompt), cpu.forward(prompt)) <= TOL
    # a missing file is an IO error, not a crash
    os.remove(os.path.join(root, "model", "layers", "layer1", "mlp", "up_proj", "offset_int4.bin"))
    with pytest.raises(pkg.capi.A81W41Error) as e:
        pkg.Qwen3Model.load(root, **TINY)
    assert e.value.status == 3


def test_cpp_model_mirror(models, pkg, synth, tmp_path):
    """host/QwenForCausalLM.hpp (the reference's Qwen3ForCausalLM interface) through the self-check
    binary: loads the tree, runs a 5-token prompt and one more token; argmax and logit sums match
    the Python-built model."""
    import re
    import subprocess
    from tests.qwen3_fixture import arrays, write_reference_tree
    gpu, _ = models
    root = str(tmp_path / "tree")
    write_reference_tree(root, arrays(synth, TINY, 900), TINY)
    exe = os.path.join(os.path.dirname(pkg.__file__), "host", "host_example")
    assert os.path.exists(exe), "build it with `make -C qwen3.ink.cpp_amd/host`"
    c = TINY
    out = subprocess.run([exe, "--model", root, str(c["n_layers"]), str(c["hidden"]), str(c["n_q_heads"]), str(c["n_kv_heads"]),
                          str(c["intermediate"]), str(c["vocab"]), str(c["max_seq"])], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    got = re.findall(r"pass (\d) argmax=(\d+) checksum=(-?[\d.]+)", out.stdout)
    assert len(got) == 2, out.stdout
    gpu.reset()
    for (_, am, cs), ids in zip(got, ([3, 99, 500, 7, 7], [17])):
        lg = gpu.forward(ids)
        assert int(am) == int(np.argmax(lg))
        assert abs(float(cs) - float(lg.astype(np.float64).sum())) <= 1e-3 * max(1.0, float(np.abs(lg).sum()))


def _logits_with_option(gpu, option, value, passes):
    """Logits of each pass on the same model with one test switch of a81w41_qwen3_set_option on."""
    gpu.set_option(option, value)
    try:
        gpu.reset()
        return np.stack([gpu.forward(ids) for ids in passes])
    finally:
        gpu.set_option(option, 0)
        gpu.reset()


def test_fused_prefill_is_bit_identical_to_separate_kernels(models):
    """With several rows the norms and SiLU*mul write quantised blocks directly; the blocks, and so the
    logits, must be the very bits of the separate norm / SiLU -> quantiser -> GEMM sequence, which the
    same model runs with the fusion switched off."""
    gpu, _ = models
    ids = [(53 * i + 7) % TINY["vocab"] for i in range(23)]
    gpu.reset()
    fused = gpu.forward(ids)
    assert np.array_equal(fused, _logits_with_option(gpu, "unfused", 1, [ids])[0])


def test_attention_quantised_output_is_bit_identical(models):
    """For one token the attention kernel writes o_proj's input as quantised blocks; with the switch on it
    writes fp32 and lets o_proj quantise it.  Same bits in, so same logits out, step after step."""
    gpu, _ = models
    passes = [[5, 6, 7, 300, 12, 99, 41], [17], [230], [8], [8]]
    gpu.reset()
    here = np.stack([gpu.forward(ids) for ids in passes])
    assert np.array_equal(here, _logits_with_option(gpu, "attn_fp32", 1, passes))


def test_chained_one_token_pass_is_bit_identical(models):
    """With the switch on, the one-token pass runs its linears and attention as a chain of overlapping launches
    instead of plain launches on one stream.  Same kernels' arithmetic in the same order: same logits, eagerly
    and from the captured graph, also with the attention's fp32 output and with a split context."""
    gpu, _ = models
    passes = [[5, 6, 7, 300, 12, 99, 41], [17], [230], [8], [8], [444], [1]]
    gpu.reset()
    here = np.stack([gpu.forward(ids) for ids in passes])
    assert np.array_equal(here, _logits_with_option(gpu, "chain", 1, passes))
    for opt, val in (("attn_fp32", 1), ("attention_split", 3)):
        gpu.set_option(opt, val)
        try:
            gpu.reset()
            a = np.stack([gpu.forward(ids) for ids in passes])
            assert np.array_equal(a, _logits_with_option(gpu, "chain", 1, passes)), opt
        finally:
            gpu.set_option(opt, 0)
    gpu.reset()
    toks, _, _ = gpu.generate_greedy(passes[0], 12)
    gpu.set_option("chain", 1)
    try:
        gpu.reset()
        chained, _, _ = gpu.generate_greedy(passes[0], 12)
    finally:
        gpu.set_option("chain", 0)
        gpu.reset()
    assert np.array_equal(toks, chained)
    assert not gpu.chain_gave_up()


def test_long_prompt_in_two_chunks(pkg, synth, ora):
    """150 tokens, then 45 more on top of the cached context: several query and key tiles of the
    matrix-core attention, the causal mask inside and across tiles, and a ragged last tile."""
    cfg = dict(TINY, max_seq=200)
    gpu, cpu = pkg.Qwen3Model(**cfg), qf.Qwen3Oracle(**cfg)
    build(synth, ora, cfg, 905, gpu_model=gpu, oracle_model=cpu)
    first = [(29 * i + 3) % cfg["vocab"] for i in range(150)]
    second = [(31 * i + 5) % cfg["vocab"] for i in range(45)]
    assert rel(gpu.forward(first), cpu.forward(first)) <= TOL
    assert rel(gpu.forward(second), cpu.forward(second)) <= TOL
    assert rel(gpu.forward([77]), cpu.forward([77])) <= TOL      # decode on top reads what the chunks cached


def test_gate_up_quantised_output_is_bit_identical(models):
    """For one token the gate|up launch writes silu(gate) * up as quantised blocks instead of its fp32
    outputs; with the switch on it keeps the fp32 outputs and down_proj's prologue does it.  Same bits."""
    gpu, _ = models
    passes = [[9, 450, 3, 3, 27, 81, 200, 11, 64], [100], [101], [7]]
    gpu.reset()
    here = np.stack([gpu.forward(ids) for ids in passes])
    assert np.array_equal(here, _logits_with_option(gpu, "no_pair", 1, passes))


def test_split_attention_for_one_token(models):
    """The one-token attention with every head's context cut into 4 shares (forced by the switch on this
    short context): same logits as the single-workgroup kernel up to the grouping of the sums."""
    gpu, cpu = models
    passes = [[(41 * i + 9) % TINY["vocab"] for i in range(37)], [17], [230], [8], [301]]
    gpu.reset(); cpu.reset()
    here = np.stack([gpu.forward(ids) for ids in passes])
    want = np.stack([cpu.forward(ids) for ids in passes])
    split = _logits_with_option(gpu, "attention_split", 4, passes)
    for a, b, c in zip(split, here, want):
        assert rel(a, c) <= TOL
        assert rel(a, b) <= 1e-3


def test_long_context_decode_picks_the_split(pkg, synth, ora):
    """700 cached tokens: the decode steps run the attention in three shares per head (chosen from the
    context length) and must still match the oracle; greedy generation replays it from the graph."""
    cfg = dict(TINY, max_seq=768)
    gpu, cpu = pkg.Qwen3Model(**cfg), qf.Qwen3Oracle(**cfg)
    build(synth, ora, cfg, 907, gpu_model=gpu, oracle_model=cpu)
    prompt = [(37 * i + 5) % cfg["vocab"] for i in range(700)]
    assert rel(gpu.forward(prompt), cpu.forward(prompt)) <= TOL
    for t in (3, 99, 255):
        assert rel(gpu.forward([t]), cpu.forward([t])) <= TOL
    gpu.reset()
    toks, _, _ = gpu.generate_greedy(prompt, 6)
    gpu.reset()
    again, _, _ = gpu.generate_greedy(prompt, 6)
    assert np.array_equal(toks, again)


def test_full_width_layer_against_the_oracle(pkg, synth, ora):
    """One layer at Qwen3-8B's real widths (hidden 4096, 32 / 8 heads, intermediate 12288; small
    vocabulary): the shapes whose launches differ from the tiny model's -- 16-wave GEMVs, the paired
    gate|up launch over 384 workgroups, the key-split schedules of the tile kernel, 4 query heads per
    KV head in both attention kernels -- against the numpy oracle, prompt and decode steps.

    The bar is wider than the tiny model's: every re-quantisation of a 4096- or 12288-wide row turns a
    relative difference eps of its input into about 2 * width * 50 * eps int8 codes that round the other
    way, each worth about 4e-4 of the next output's norm, so the 1e-5 by which the fp32 attention differs
    from the float64 one grows to a few 1e-3 at the logits (observed 0 .. 7e-3, the same to four digits
    for every fusion switch and attention variant: the GPU paths agree with each other far more closely
    than either does with the oracle).  A wrong index or operand gives errors of order 1."""
    cfg = dict(n_layers=1, hidden=4096, n_q_heads=32, n_kv_heads=8, intermediate=12288, vocab=1024, max_seq=64)
    gpu, cpu = pkg.Qwen3Model(**cfg), qf.Qwen3Oracle(**cfg)
    build(synth, ora, cfg, 911, gpu_model=gpu, oracle_model=cpu)
    wide_tol = 2e-2
    prompt = [(97 * i + 11) % cfg["vocab"] for i in range(11)]
    errs = [rel(gpu.forward(prompt), cpu.forward(prompt))]
    for t in (5, 1000, 77, 300):
        errs.append(rel(gpu.forward([t]), cpu.forward([t])))
    errs.append(rel(gpu.forward([1, 2, 3]), cpu.forward([1, 2, 3])))      # a few rows: the few-row kernels
    assert max(errs) <= wide_tol, errs
    assert sorted(errs)[len(errs) // 2] <= TOL, errs                       # and typically within the usual bar


@pytest.mark.parametrize("hidden,inter", [(1024, 3072), (2048, 6144)])
def test_one_token_pass_on_narrow_models(pkg, synth, ora, hidden, inter):
    """Qwen3-0.6B / 1.7B widths: short activation rows in wide workgroups (hidden 1024 would give the paired
    gate|up launch sixteen column groups per workgroup, more than its eight-group units allow).  Decode
    steps against the oracle, and the paired launch against the unpaired one bit for bit."""
    cfg = dict(n_layers=1, hidden=hidden, n_q_heads=16, n_kv_heads=8, intermediate=inter, vocab=512, max_seq=32)
    gpu, cpu = pkg.Qwen3Model(**cfg), qf.Qwen3Oracle(**cfg)
    build(synth, ora, cfg, 921, gpu_model=gpu, oracle_model=cpu)
    passes = [[3, 99, 500, 7], [17], [230], [8]]
    here = [gpu.forward(ids) for ids in passes]
    for got, ids in zip(here, passes):
        assert rel(got, cpu.forward(ids)) <= 2e-2
    assert np.array_equal(np.stack(here), _logits_with_option(gpu, "no_pair", 1, passes))
