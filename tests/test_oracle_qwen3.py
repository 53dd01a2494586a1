"""Pins the numpy restatement of the Qwen3 forward pass (oracle/qwen3_forward.py) through
properties its mathematics fixes; a dropped term, a wrong sign or a transposed operand fails
at least one of them.  No GPU."""
import numpy as np
import pytest

from oracle import qwen3_forward as qf
from tests.qwen3_fixture import TINY, build


def test_rmsnorm_gives_unit_rms_and_scales_with_weight():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(5, 256)).astype(np.float32) * 7
    y = qf.rmsnorm(x, np.ones(256, np.float32), 0.0)
    assert np.allclose(np.sqrt((y.astype(np.float64) ** 2).mean(-1)), 1.0, atol=1e-6)
    w = rng.normal(size=256).astype(np.float32)
    assert np.allclose(qf.rmsnorm(x, w, 0.0), y * w, rtol=1e-6, atol=1e-7)
    # eps enters under the root: a zero row stays zero instead of becoming NaN
    assert np.array_equal(qf.rmsnorm(np.zeros((1, 8), np.float32), np.ones(8, np.float32), 1e-6), np.zeros((1, 8), np.float32))
    # and a constant row c gives c / sqrt(c^2 + eps)
    assert np.allclose(qf.rmsnorm(np.full((1, 8), 2.0, np.float32), np.ones(8, np.float32), 5.0), 2.0 / 3.0)


def test_rotation_is_a_rotation_with_the_relative_position_property():
    cos, sin = qf.rope_tables(64, 1e6)
    # table values: pair (j, j+64) shares the angle pos * theta^(-2j/128)
    assert np.allclose(cos[3, 5], np.cos(3 * 1e6 ** (-10 / 128)), atol=1e-7)
    assert np.array_equal(cos[:, :64], cos[:, 64:]) and np.array_equal(sin[:, :64], sin[:, 64:])
    rng = np.random.default_rng(2)
    q, k = rng.normal(size=128).astype(np.float32), rng.normal(size=128).astype(np.float32)
    # position 0 is the identity
    assert np.allclose(qf.rotate_half_apply(q, cos[0], sin[0]), q)
    # norms are preserved, and <R_m q, R_n k> depends on m - n only
    dots = {}
    for m, n in [(7, 3), (24, 20), (40, 36), (9, 3)]:
        qm, kn = qf.rotate_half_apply(q, cos[m], sin[m]), qf.rotate_half_apply(k, cos[n], sin[n])
        assert np.isclose(np.linalg.norm(qm), np.linalg.norm(q), rtol=1e-5)
        dots[(m, n)] = float(qm.astype(np.float64) @ kn.astype(np.float64))
    assert np.isclose(dots[(7, 3)], dots[(24, 20)], rtol=1e-4, atol=1e-4)
    assert np.isclose(dots[(7, 3)], dots[(40, 36)], rtol=1e-4, atol=1e-4)
    assert not np.isclose(dots[(7, 3)], dots[(9, 3)], rtol=1e-3)
    # the sign convention: a unit vector on axis j turns towards axis j + 64 by the angle
    e = np.zeros(128, np.float32); e[5] = 1
    r = qf.rotate_half_apply(e, cos[2], sin[2])
    assert np.isclose(r[5], cos[2, 5]) and np.isclose(r[69], sin[2, 5])


def test_softmax_and_silu_closed_forms():
    s = np.array([[0.0, np.log(3.0), -np.inf]])
    assert np.allclose(qf.softmax_rows(s), [[0.25, 0.75, 0.0]])
    assert np.allclose(qf.softmax_rows(s + 1000.0), [[0.25, 0.75, 0.0]])      # shift invariance, no overflow
    g = np.array([0.0, 1.0, -1.0, 20.0], np.float32)
    want = g / (1 + np.exp(-g.astype(np.float64)))
    assert np.allclose(qf.silu_mul(g, np.full(4, 2.0, np.float32)), 2 * want, rtol=1e-6)


@pytest.fixture(scope="module")
def tiny(synth, ora):
    m = qf.Qwen3Oracle(**TINY)
    build(synth, ora, TINY, 900, oracle_model=m)
    return m


def test_single_token_context_returns_its_value(tiny, ora):
    """With one key the softmax is 1: attention output of the first token is its V (as stored,
    fp16), repeated for every query head of the KV group."""
    tiny.reset()
    tiny.forward([17])
    l = 0
    v0 = tiny.v[l][0, 0].astype(np.float32)
    # recompute layer 0 up to the attention output by hand
    x = tiny.embedding[[17]].astype(np.float32)
    h = qf.rmsnorm(x, tiny.norm[l][0], tiny.eps)
    qkv = ora.linear_forward(h, *tiny.lin[l][0][:2], tiny.lin[l][0][2])
    v_direct = qkv[0, (TINY["n_q_heads"] + TINY["n_kv_heads"]) * 128:].astype(np.float16).astype(np.float32)
    assert np.array_equal(v0, v_direct)


def test_prompt_in_one_pass_equals_token_by_token(tiny):
    """Causality + cache bookkeeping: logits after a 9-token prompt are the same whether the
    prompt goes in as one M = 9 pass, as 4 + 5, or (up to the M == 1 / M > 1 kernel difference of
    the quantized layer, ~1e-3) one token at a time."""
    ids = [3, 99, 500, 7, 7, 123, 45, 256, 31]
    tiny.reset(); a = tiny.forward(ids)
    tiny.reset(); tiny.forward(ids[:4]); b = tiny.forward(ids[4:])
    # rows of an M > 1 pass are independent in the linears, and the first pass only adds cache
    # rows: the last row's logits differ only through the M == 1 lm_head input, which is equal
    assert np.allclose(a, b, rtol=0, atol=2e-3 * np.abs(a).max())
    tiny.reset()
    for t in ids:
        c = tiny.forward([t])
    assert np.linalg.norm(a - c) <= 3e-2 * np.linalg.norm(a)
    # a different earlier token changes the result (the context is really used) ...
    tiny.reset(); d = tiny.forward([4] + ids[1:])
    assert np.linalg.norm(a - d) > 1e-2 * np.linalg.norm(a)
    # ... the same token repeated gives the same logits at every position (all keys and values
    # are equal, so every softmax average is that one value) ...
    tiny.reset(); e1 = tiny.forward([11]); e2 = tiny.forward([11])
    assert np.allclose(e1, e2, rtol=0, atol=1e-5 * np.abs(e1).max())
    # ... and order matters
    tiny.reset(); f1 = tiny.forward([5, 11, 12])
    tiny.reset(); f2 = tiny.forward([11, 5, 12])
    assert np.linalg.norm(f1 - f2) > 1e-3 * np.linalg.norm(f1)


def test_full_width_logits_are_sensitive_to_1e_5_in_the_attention(synth, ora, monkeypatch):
    """Why the GPU test of a full-width layer has a wider bar than the tiny model's: perturb the
    oracle's own softmax weights by 1e-5 (what fp32 attention differs from float64 by) and the logits of
    a 4096-wide layer move by some 1e-3 of their norm, because each re-quantisation of a wide row rounds
    dozens of int8 codes the other way.  The effect is bounded well below the wide bar (2e-2)."""
    cfg = dict(n_layers=1, hidden=4096, n_q_heads=32, n_kv_heads=8, intermediate=12288, vocab=1024, max_seq=64)
    a, b = qf.Qwen3Oracle(**cfg), qf.Qwen3Oracle(**cfg)
    build(synth, ora, cfg, 911, oracle_model=a)
    build(synth, ora, cfg, 911, oracle_model=b)
    exact = qf.softmax_rows
    rng = np.random.default_rng(0)
    noisy = lambda s: exact(s) * (1.0 + 1e-5 * rng.standard_normal(s.shape))
    prompt = [(97 * i + 11) % cfg["vocab"] for i in range(11)]
    errs = []
    for ids in (prompt, [5], [1000]):
        ya = a.forward(ids)
        monkeypatch.setattr(qf, "softmax_rows", noisy)
        yb = b.forward(ids)
        monkeypatch.setattr(qf, "softmax_rows", exact)
        errs.append(float(np.linalg.norm(yb.astype(np.float64) - ya) / np.linalg.norm(ya.astype(np.float64))))
    assert max(errs) > 1e-4, errs          # far more than the 1e-5 that went in
    assert max(errs) < 2e-2, errs



def test_cost_of_the_fp16_cache_and_embedding(synth, ora, capsys):
    """The build keeps the KV cache and the embedding table in binary16; the reference keeps both in
    fp32 (QwenAttention.cc:13-16, ops/embedding.cc:13-26).  The oracle in the reference's storage mode
    against the oracle in the build's: what the two narrowings move at the logits (tiny model, prompt and
    decode steps).  The fast (AVX2 port) linears give the same logits as the scalar ones, bit for bit."""
    def make(kv_dtype, emb_fp32, fast=False):
        m = qf.Qwen3Oracle(**TINY, kv_dtype=kv_dtype, fast_linear=fast)
        build(synth, ora, TINY, 900, oracle_model=m)
        # one fp32 table for both: the build's mode sees it rounded to binary16
        table = (np.float32(1.0) + synth.standard_normal(TINY["vocab"] * TINY["hidden"], 31)).reshape(
            TINY["vocab"], TINY["hidden"]).astype(np.float32)
        m.embedding = table if emb_fp32 else table.astype(np.float16)
        return m

    ours, ref, fast = make(np.float16, False), make(np.float32, True), make(np.float16, False, fast=True)
    passes = [[3, 99, 500, 7, 7, 123, 45, 256, 31, 8, 301], [17], [400], [5]]
    worst = 0.0
    for ids in passes:
        a, b, c = ours.forward(ids), ref.forward(ids), fast.forward(ids)
        assert np.array_equal(a, c)
        worst = max(worst, float(np.linalg.norm(a - b) / np.linalg.norm(b)))
    with capsys.disabled():
        print(f"\n[fp16 KV cache + fp16 embedding vs fp32 storage: logits move by at most {worst:.2e} of their norm]")
    assert 0.0 < worst <= 2e-2
