"""CPU restatement of the reference's Qwen3 forward pass around the quantized linear layer.

TEST INFRASTRUCTURE ONLY: tests/, __graft_entry__.smoke() and bench.py's checker legs may
import this; the product never does.

Follows, in numpy:
  Qwen3ForCausalLM::forward      qwen3/src/qwen/QwenForCausalLM.cc:11-60   (lm_head on the last token)
  Qwen3Model::forward            qwen3/src/qwen/QwenDecoder.cc:53-141      (embedding, causal mask :6-21, final norm)
  Qwen3DecoderLayer::forward     qwen3/src/qwen/QwenDecoderLayer.cc:39-118
  Qwen3Attention::forward        qwen3/src/qwen/QwenAttention.cc:52-208    (fused qkv :78-83, q/k norm :84-89)
  Qwen3RMSNorm::forward          qwen3/src/qwen/QwenOperator.cc:24-53
  RotaryPosEmb::apply            qwen3/src/ops/RotaryPosEmb.cc:6-78        (rotate-half)
  Qwen3SiLuMul                   qwen3/src/qwen/QwenOperator.cc:697-713
  sample_token_greedy            qwen3/src/qwen/Pipeline.cc:54-62          (first maximum)
Every linear is oracle.ora.linear_forward, the C restatement of the A81W41 layer with the
reference's dispatch on M.  Deliberate differences from the reference, shared with the GPU
build: the KV cache holds IEEE binary16 values (the reference's holds fp32, QwenAttention.cc:13-16),
the embedding table is given as binary16 (the reference's is fp32, ops/embedding.cc:13-26), gate_proj
and up_proj are one 2*intermediate-wide linear (gate rows first), the cos/sin tables are computed
here (theta given) instead of loaded from rotary_emb files.  kv_dtype=np.float32 together with an
fp32 embedding table gives the reference's own storage choices; tests/test_oracle_qwen3.py measures
what the two narrowings cost at the logits.

Pinned by tests/test_oracle_qwen3.py through properties the mathematics fixes (RMS of a
normalised row, norm preservation and relative-position property of the rotation, softmax
rows, a single-key context returning V, causality: a prompt processed in one pass equals the
same tokens fed one by one).
"""
from __future__ import annotations

import numpy as np

from . import ora

HEAD_DIM = 128


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """QwenOperator.cc:36-48: x / sqrt(mean(x^2) + eps) * w over the last axis."""
    x = x.astype(np.float32)
    var = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    inv = (1.0 / np.sqrt(var + eps)).astype(np.float32)
    return ((x * inv) * w.astype(np.float32)).astype(np.float32)


def rope_tables(max_seq: int, theta: float):
    """cos/sin [max_seq][128]; angle(pos, j) = pos * theta^(-2 (j mod 64) / 128)."""
    j = np.arange(HEAD_DIM) % (HEAD_DIM // 2)
    inv_freq = np.power(float(theta), -2.0 * j / HEAD_DIM)
    ang = np.arange(max_seq, dtype=np.float64)[:, None] * inv_freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def rotate_half_apply(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """RotaryPosEmb.cc:31-52: x*cos + cat(-x2, x1)*sin; x [..., 128], cos/sin broadcastable."""
    half = HEAD_DIM // 2
    rot = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
    return (x * cos + rot * sin).astype(np.float32)


def softmax_rows(s: np.ndarray) -> np.ndarray:
    s = s.astype(np.float64)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def silu_mul(g: np.ndarray, u: np.ndarray) -> np.ndarray:
    g64 = g.astype(np.float64)
    return ((g64 * (1.0 / (1.0 + np.exp(-g64)))).astype(np.float32) * u.astype(np.float32)).astype(np.float32)


class Qwen3Oracle:
    def __init__(self, n_layers, hidden, n_q_heads, n_kv_heads, intermediate, vocab, max_seq,
                 rope_theta=1e6, rms_eps=1e-6, kv_dtype=np.float16, fast_linear=False):
        self.kv_dtype = kv_dtype          # np.float32: the reference's cache
        self.fast_linear = fast_linear    # linears through the AVX2 port (same bits, for full-size models)
        self.L, self.H, self.nq, self.nkv, self.I, self.V, self.S = n_layers, hidden, n_q_heads, n_kv_heads, intermediate, vocab, max_seq
        self.eps = rms_eps
        self.cos, self.sin = rope_tables(max_seq, rope_theta)
        self.lin = [[None] * 4 for _ in range(n_layers)]     # (b16, b32, N)
        self.norm = [[None] * 4 for _ in range(n_layers)]
        self.lm_head = None
        self.final_norm = None
        self.embedding = None
        self.reset()

    def reset(self):
        self.pos = 0
        self.k = np.zeros((self.L, self.nkv, self.S, HEAD_DIM), self.kv_dtype)
        self.v = np.zeros((self.L, self.nkv, self.S, HEAD_DIM), self.kv_dtype)

    def _linear(self, x, entry):
        b16, b32, N = entry
        if b32 is None:
            b32 = np.zeros(1, np.uint8)   # never read: only M == 1 calls go here
            assert x.shape[0] == 1
        return (ora.linear_forward_fast if self.fast_linear else ora.linear_forward)(x, b16, b32, N)

    def forward(self, ids) -> np.ndarray:
        ids = np.asarray(ids, np.int64)
        M, p0 = len(ids), self.pos
        assert p0 + M <= self.S
        x = self.embedding[ids].astype(np.float32)                       # [M][H]
        scale = np.float32(1.0 / np.sqrt(np.float32(HEAD_DIM)))
        qd, kd = self.nq * HEAD_DIM, self.nkv * HEAD_DIM
        group = self.nq // self.nkv
        for l in range(self.L):
            h = rmsnorm(x, self.norm[l][0], self.eps)
            qkv = self._linear(h, self.lin[l][0])
            q = qkv[:, :qd].reshape(M, self.nq, HEAD_DIM)
            k = qkv[:, qd:qd + kd].reshape(M, self.nkv, HEAD_DIM)
            v = qkv[:, qd + kd:].reshape(M, self.nkv, HEAD_DIM)
            q = rmsnorm(q, self.norm[l][2], self.eps)
            k = rmsnorm(k, self.norm[l][3], self.eps)
            cos, sin = self.cos[p0:p0 + M, None, :], self.sin[p0:p0 + M, None, :]
            q = rotate_half_apply(q, cos, sin)
            k = rotate_half_apply(k, cos, sin)
            self.k[l][:, p0:p0 + M] = k.transpose(1, 0, 2).astype(self.kv_dtype)
            self.v[l][:, p0:p0 + M] = v.transpose(1, 0, 2).astype(self.kv_dtype)
            attn = np.zeros((M, self.nq, HEAD_DIM), np.float32)
            for hq in range(self.nq):
                K = self.k[l][hq // group, :p0 + M].astype(np.float64)   # [T][128]
                Vv = self.v[l][hq // group, :p0 + M].astype(np.float64)
                s = (q[:, hq].astype(np.float64) @ K.T) * float(scale)   # [M][T]
                t = np.arange(p0 + M)[None, :]
                s = np.where(t <= (p0 + np.arange(M))[:, None], s, -np.inf)   # QwenDecoder.cc:14-18
                attn[:, hq] = (softmax_rows(s) @ Vv).astype(np.float32)
            o = self._linear(attn.reshape(M, qd), self.lin[l][1])
            x = (x + o).astype(np.float32)
            h = rmsnorm(x, self.norm[l][1], self.eps)
            gu = self._linear(h, self.lin[l][2])
            act = silu_mul(gu[:, :self.I], gu[:, self.I:])
            x = (x + self._linear(act, self.lin[l][3])).astype(np.float32)
        h = rmsnorm(x, self.final_norm, self.eps)
        self.pos += M
        return self._linear(h[M - 1:M], self.lm_head)[0]

    @staticmethod
    def greedy(logits: np.ndarray) -> int:
        return int(np.argmax(logits))      # first maximum, like std::max_element
