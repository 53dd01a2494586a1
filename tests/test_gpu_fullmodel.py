"""The forward pass at Qwen3-8B's real size (36 layers, hidden 4096, 32 / 8 heads, intermediate 12288,
vocabulary 151 936), one seeded weight set per shape shared by the layers: a 322-token prompt and decode
steps.  End to end the model is checked through properties (the captured graph against eager passes, every
fusion against the separate kernels bit for bit, split against unsplit attention, repeatability); against
the oracle it is checked stage by stage on the activations the GPU itself produced in the last layer, so
that each kernel is held to its own bar instead of the chaotic end product of 36 re-quantising layers."""
import numpy as np
import pytest

from oracle import qwen3_forward as qf

pytestmark = pytest.mark.gpu

CFG = dict(n_layers=36, hidden=4096, n_q_heads=32, n_kv_heads=8, intermediate=12288, vocab=151936, max_seq=384)
N_PROMPT = 322


def row_rel(got, want):
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.max(np.linalg.norm(g - w, axis=-1) / np.maximum(np.linalg.norm(w, axis=-1), 1e-30)))


@pytest.fixture(scope="module")
def full(pkg, synth):
    ops = pkg.ops
    H, I, V = CFG["hidden"], CFG["intermediate"], CFG["vocab"]
    model = ops.Qwen3Model(**CFG)
    host = {"lin": [], "norm": None}
    dims = [((CFG["n_q_heads"] + 2 * CFG["n_kv_heads"]) * 128, H), (H, H), (2 * I, H), (H, I)]
    for which, (N, K) in enumerate(dims):
        w4, scale, offset = synth.weight_files(N, K, 7000 + which)
        b16 = ops.repack_w81_weight(K, N, scale, offset, w4, fp32=False)   # byte-equal to the oracle's repack
        b32 = ops.repack_w81_weight(K, N, scale, offset, w4, fp32=True)    # (tests/test_capi_host.py)
        for l in range(CFG["n_layers"]):
            model.set_linear_blobs(l, which, b16, b32)
        host["lin"].append((b16, b32, N, K))
    rng = np.random.default_rng(4242)
    # norm weights of alternating sign keep the seeded weights' common mode out of the residual stream,
    # so that greedy decoding does not settle on one token
    alt = np.where(np.arange(H) % 2 == 0, 1.0, -1.0)
    norms = []
    for l in range(CFG["n_layers"]):
        ws = []
        for which, n in enumerate([H, H, 128, 128]):
            w = 1.0 + 0.1 * rng.standard_normal(n)
            ws.append((w * alt if n == H else w).astype(np.float32))
            model.set_norm(l, which, ws[-1])
        norms.append(ws)
    host["norm"] = norms
    w4, scale, offset = synth.weight_files(V, H, 7100)
    host["lm_head"] = ops.repack_w81_weight(H, V, scale, offset, w4, fp32=False)
    model.set_linear_blobs(-1, 0, host["lm_head"], None)
    host["final_norm"] = ((1.0 + 0.1 * rng.standard_normal(H)) * alt).astype(np.float32)
    model.set_norm(-1, 0, host["final_norm"])
    emb = np.empty((V, H), np.float16)
    for r0 in range(0, V, 8192):
        r1 = min(V, r0 + 8192)
        emb[r0:r1] = (8.0 * rng.standard_normal((r1 - r0, H), dtype=np.float32)).astype(np.float16)
    model.set_embedding(emb)
    host["prompt"] = rng.integers(0, V, size=N_PROMPT).astype(np.int32)
    return model, host


def test_greedy_generation_graph_equals_eager_and_does_not_collapse(full):
    model, host = full
    n_new = 10
    model.reset()
    toks, t_pre, t_dec = model.generate_greedy(host["prompt"], n_new)      # decode steps replayed from one graph
    model.reset()
    again, _, _ = model.generate_greedy(host["prompt"], n_new)
    assert np.array_equal(toks, again)
    model.reset()
    logits = model.forward(host["prompt"])
    eager = []
    for _ in range(n_new):
        assert np.isfinite(logits).all()
        eager.append(int(np.argmax(logits)))
        logits = model.forward([eager[-1]])
    assert toks.tolist() == eager
    assert len(set(eager)) > n_new // 2, eager
    assert t_pre > 0 and t_dec > 0
    # the same generation with the decode steps as chains of overlapping launches
    model.set_option("chain", 1)
    try:
        model.reset()
        chained, _, _ = model.generate_greedy(host["prompt"], n_new)
    finally:
        model.set_option("chain", 0)
    assert np.array_equal(toks, chained)
    assert not model.chain_gave_up()


def _passes(model, host, option=None, value=1):
    if option:
        model.set_option(option, value)
    try:
        model.reset()
        out = [model.forward(host["prompt"])]
        for t in (17, 151935, 4000, 99):
            out.append(model.forward([t]))
        return np.stack(out)
    finally:
        if option:
            model.set_option(option, 0)


def test_fusions_are_bit_identical_at_full_size(full):
    """Prefill: norm / SiLU / attention epilogues writing quantised blocks; one token: add + norm in the GEMV
    prologues (incl. the 151 936-wide lm_head), attention writing o_proj's blocks, the paired gate|up launch."""
    model, host = full
    base = _passes(model, host)
    assert np.isfinite(base).all()
    # chain: the one-token pass as a chain of overlapping launches instead of plain launches on one stream
    for opt in ("attn_fp32", "no_pair", "chain"):
        assert np.array_equal(base, _passes(model, host, opt)), opt
    assert not model.chain_gave_up()
    # all separate kernels: the prompt pass has the same bits; the one-token passes then run the few-row vector
    # attention instead of the online-softmax kernel, which is another summation order
    unf = _passes(model, host, "unfused")
    assert np.array_equal(unf[0], base[0])
    assert row_rel(unf[1:], base[1:]) <= 2e-2
    vec = _passes(model, host, "vector_attention")          # prefill attention on the vector kernel
    assert row_rel(vec, base) <= 2e-2
    split = _passes(model, host, "attention_split", 4)      # 4 shares per head in the one-token attention
    assert np.array_equal(split[0], base[0])                # the prompt pass does not use it
    assert row_rel(split[1:], base[1:]) <= 2e-2
    assert np.median(np.linalg.norm(split[1:] - base[1:], axis=1) / np.linalg.norm(base[1:], axis=1)) <= 1e-2


@pytest.mark.parametrize("n_prompt", [20, 50])
def test_short_prompts_at_full_width(full, n_prompt):
    """Prompts of 9 .. 32 tokens send every layer-wide linear (4096 .. 24 576 columns) to the one-row-panel kernel with
    its LDS stages, 33 .. 64 tokens to the 64 x 64 tiles with a single row tile.  The fused pass (producers write the
    quantised blocks, the contraction stages its rows from the reference's layout) and the pass of separate kernels
    (the layer's own quantiser, rows staged from the per-super-block copy) give the same bits; a decode step on top
    of either agrees within the bar of the two attention kernels."""
    model, host = full
    prompt = host["prompt"][:n_prompt]

    def run():
        model.reset()
        first = model.forward(prompt).copy()
        return first, model.forward([int(np.argmax(first))]).copy()

    a0, a1 = run()
    assert np.isfinite(a0).all() and np.isfinite(a1).all()
    model.set_option("unfused", 1)
    try:
        b0, b1 = run()
    finally:
        model.set_option("unfused", 0)
    assert np.array_equal(a0, b0)
    assert row_rel(b1[None, :], a1[None, :]) <= 2e-2
    c0, _ = run()
    assert np.array_equal(a0, c0)       # repeatable


def test_last_layer_stage_by_stage_against_the_oracle(full, ora):
    """Unfused prompt pass, then each stage of layer 35 recomputed on the CPU from the GPU's own input to
    that stage (float64 numpy for attention / norm / SiLU, the AVX2 port -- bit-identical to the scalar oracle --
    for the quantised linears), so a stage's error is not amplified by the stages behind it."""
    model, host = full
    M, H, I, V = N_PROMPT, CFG["hidden"], CFG["intermediate"], CFG["vocab"]
    nq, nkv = CFG["n_q_heads"], CFG["n_kv_heads"]
    model.set_option("unfused", 1)
    try:
        model.reset()
        logits = model.forward(host["prompt"])
        qkv = model.read_buffer("qkv", M, (nq + 2 * nkv) * 128)
        attn = model.read_buffer("attention", M, nq * 128)
        gate_up = model.read_buffer("gate_up", M, 2 * I)
        act = model.read_buffer("act", M, I)
        down = model.read_buffer("block_out", M, H)
        resid = model.read_buffer("residual", M, H)
        normed = model.read_buffer("normed", M, H)
    finally:
        model.set_option("unfused", 0)
    # attention (QwenAttention.cc:84-122,150-195): the buffer holds q normalised and rotated, k and v as
    # projected; keys are normalised, rotated and rounded to binary16 on their way into the cache
    q = qkv[:, :nq * 128].reshape(M, nq, 128).astype(np.float64)
    cos, sin = qf.rope_tables(CFG["max_seq"], 1e6)
    k = qf.rmsnorm(qkv[:, nq * 128:(nq + nkv) * 128].reshape(M, nkv, 128), host["norm"][-1][3], 1e-6)
    k = qf.rotate_half_apply(k, cos[:M, None, :], sin[:M, None, :]).astype(np.float16).astype(np.float64)
    v = qkv[:, (nq + nkv) * 128:].reshape(M, nkv, 128).astype(np.float16).astype(np.float64)
    want = np.empty((M, nq, 128))
    causal = np.tril(np.ones((M, M), bool))
    for h in range(nq):
        s = (q[:, h] @ k[:, h // (nq // nkv)].T) / np.sqrt(128.0)
        want[:, h] = qf.softmax_rows(np.where(causal, s, -np.inf)) @ v[:, h // (nq // nkv)]
    # the worst of 322 x 32 head rows, each relative to its own 128-vector (rows whose weighted values cancel
    # down to a small vector set it: 5e-5 on this data; all rows together agree to 2e-5 of the token row's norm)
    assert row_rel(attn.reshape(M, nq, 128), want) <= 1e-4
    assert row_rel(attn, want.reshape(M, nq * 128)) <= 2e-5
    # SiLU * mul (QwenOperator.cc:697-713)
    g64, u64 = gate_up[:, :I].astype(np.float64), gate_up[:, I:].astype(np.float64)
    assert row_rel(act, g64 / (1.0 + np.exp(-g64)) * u64) <= 2e-6
    # down projection of that very input: quantiser + M = 322 GEMM at K = 12288
    b16, b32, N, K = host["lin"][3]
    assert row_rel(down, ora.linear_forward_fast(act, b16, b32, N)) <= 1e-4
    # final add + RMSNorm: the residual stream ends finite, the norm is the float64 one
    assert np.isfinite(resid).all()
    x64 = resid.astype(np.float64)
    want_n = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * host["final_norm"].astype(np.float64)
    assert row_rel(normed, want_n) <= 2e-6
    # lm_head over the whole vocabulary on the last row (fp16-parameter quantiser + GEMV)
    want_l = ora.linear_forward_fast(normed[M - 1:M], host["lm_head"], np.zeros(1, np.uint8), V)[0]
    assert row_rel(logits[None], want_l[None]) <= 1e-4

    # one token on top, unfused: the separate norm writes `normed` row 0 and lm_head's own quantiser reads it
    model.set_option("unfused", 1)
    try:
        unf = model.forward([1234])
        h0 = model.read_buffer("normed", 1, H)
    finally:
        model.set_option("unfused", 0)
    assert row_rel(unf[None], ora.linear_forward_fast(h0, host["lm_head"], np.zeros(1, np.uint8), V)) <= 1e-4
    # the same token through the fused pass: add + norm run in the prologue of the 151 936-wide GEMV, on the
    # pending block output and the residual row the pass leaves behind; recompute that prologue in fp32
    model.reset()
    model.forward(host["prompt"])
    fused = model.forward([1234])
    x = model.read_buffer("residual", 1, H) + model.read_buffer("block_out", 1, H)
    inv = np.float32(1.0 / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-6))
    h_fused = (x * inv) * host["final_norm"]
    assert row_rel(fused[None], ora.linear_forward_fast(h_fused, host["lm_head"], np.zeros(1, np.uint8), V)) <= 1e-4
