"""Host-side mirror of the reference's linear-layer interface on top of the C ABI.

``Linear`` plays the role of ``Qwen_Linear_with_bias_Int4`` (QwenOperator.h:86-231):
constructed from the four-file weight layout (or arrays in that layout), its
``forward`` takes activations ``[M][K]`` and returns ``[M][N]`` with the
reference's M-dispatch.  The free functions mirror the reference's free
functions one to one (QwenOperator.h:83-84, 277-278, 293-304).  torch is used
only to own device memory and to name the stream.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi


def _torch():
    import torch

    return torch


def _stream():
    return C.c_void_p(_torch().cuda.current_stream().cuda_stream)


def _np_ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def _dev_ptr(t):
    """Device address of a CUDA tensor, or of a raw int address (e.g. a layer's weight blob)."""
    if isinstance(t, int):
        return C.c_void_p(t)
    assert t.is_cuda and t.is_contiguous()
    return C.c_void_p(t.data_ptr())


# ---------------------------------------------------------------- load time (host)

def repack_w81_weight(K: int, N: int, scale: np.ndarray, offset: np.ndarray, w4: np.ndarray,
                      fp32: bool) -> np.ndarray:
    """repack_w81_weight_fp16 / _fp32: file layout -> 320 B / 384 B blocks (host bytes)."""
    L = capi.lib()
    out = np.zeros(L.a81w41_weight_blob_bytes(K, N, int(fp32)), dtype=np.uint8)
    fn = L.a81w41_repack_w81_weight_fp32 if fp32 else L.a81w41_repack_w81_weight_fp16
    capi.check(fn(K, N, 32, _np_ptr(out), _np_ptr(np.ascontiguousarray(scale, np.float32)),
                  _np_ptr(np.ascontiguousarray(offset, np.float32)),
                  _np_ptr(np.ascontiguousarray(w4, np.uint8))))
    return out


def quantize_weight_q41(w: np.ndarray):
    """quantize_row_q41_tinyml: fp32 [N][K] -> (weight_int4 [N][K/2], scale [N][K/32], offset [N][K/32])."""
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    w4 = np.zeros((N, K // 2), np.uint8)
    scale = np.zeros((N, K // 32), np.float32)
    offset = np.zeros((N, K // 32), np.float32)
    capi.check(capi.lib().a81w41_quantize_weight_q41(_np_ptr(w), N, K, _np_ptr(w4), _np_ptr(scale), _np_ptr(offset)))
    return w4, scale, offset


# ---------------------------------------------------------------- device kernels

def quantize(x, fp32: bool):
    """quantize_row_q8_1_repack_fp16 / _fp32 on a CUDA float32 tensor -> uint8 blob tensor."""
    torch = _torch()
    L = capi.lib()
    x = x.contiguous()
    k = x.numel()
    out = torch.empty(L.a81w41_act_blob_bytes(k, int(fp32)), dtype=torch.uint8, device=x.device)
    fn = L.a81w41_quantize_row_q8_1_repack_fp32 if fp32 else L.a81w41_quantize_row_q8_1_repack_fp16
    capi.check(fn(_dev_ptr(x), _dev_ptr(out), k, _stream()))
    return out


def gemv_fp16(a_blob, b_blob, N: int, K: int, M: int = 1, out=None):
    """gemv_repack_A81W41_fp16; ``b_blob`` is a uint8 CUDA tensor or a raw device address."""
    torch = _torch()
    if out is None:
        out = torch.empty(N, dtype=torch.float32, device=a_blob.device)
    capi.check(capi.lib().a81w41_gemv_repack_A81W41_fp16(_dev_ptr(a_blob), _dev_ptr(b_blob), _dev_ptr(out),
                                                         M, N, K, _stream()))
    return out


def gemm_fp32(a_blob, b_blob, M: int, N: int, K: int, out=None, static_scratch: bool = False):
    """gemm_repack_A81W41_fp32; ``b_blob`` is a uint8 CUDA tensor or a raw device address.
    ``static_scratch``: the entry point that allocates nothing (``..._fp32_static``)."""
    torch = _torch()
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a_blob.device)
    fn = capi.lib().a81w41_gemm_repack_A81W41_fp32_static if static_scratch else capi.lib().a81w41_gemm_repack_A81W41_fp32
    capi.check(fn(_dev_ptr(a_blob), _dev_ptr(b_blob), _dev_ptr(out), M, N, K, _stream()))
    return out


def block_idot(a_blob, a_fp32: bool, b_blob, b_fp32: bool, M: int, N: int, K: int):
    torch = _torch()
    out = torch.empty((M, N, K // 32), dtype=torch.int32, device=a_blob.device)
    capi.check(capi.lib().a81w41_block_idot(_dev_ptr(a_blob), int(a_fp32), _dev_ptr(b_blob), int(b_fp32),
                                            _dev_ptr(out), M, N, K, _stream()))
    return out


# ---------------------------------------------------------------- the A80W40 variant

def repack_w80_weight(K: int, N: int, scale: np.ndarray, w4: np.ndarray, fill: int = 0) -> np.ndarray:
    """repack_w80_weight: file layout -> 320 B blocks whose min fields keep the ``fill`` byte."""
    L = capi.lib()
    out = np.full(L.a81w41_weight_blob_bytes(K, N, 0), fill, dtype=np.uint8)
    capi.check(L.a81w41_repack_w80_weight(K, N, 32, _np_ptr(out), _np_ptr(np.ascontiguousarray(scale, np.float32)),
                                          _np_ptr(np.ascontiguousarray(w4, np.uint8))))
    return out


def quantize_weight_q40(w: np.ndarray):
    """quantize_row_q40_tinyml: fp32 [N][K] -> (weight_int4 [N][K/2], scale [N][K/32])."""
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    w4 = np.zeros((N, K // 2), np.uint8)
    scale = np.zeros((N, K // 32), np.float32)
    capi.check(capi.lib().a81w41_quantize_weight_q40(_np_ptr(w), N, K, _np_ptr(w4), _np_ptr(scale)))
    return w4, scale


def quantize_q8_0(x, out=None):
    """quantize_row_q8_0_repack on a CUDA float32 tensor -> 72 B blocks (sum fields of ``out`` untouched)."""
    torch = _torch()
    L = capi.lib()
    x = x.contiguous()
    k = x.numel()
    if out is None:
        out = torch.zeros(L.a81w41_act_blob_bytes(k, 0), dtype=torch.uint8, device=x.device)
    capi.check(L.a81w41_quantize_row_q8_0_repack(_dev_ptr(x), _dev_ptr(out), k, _stream()))
    return out


def gemv_a80w40(a_blob, b_blob, N: int, K: int, M: int = 1, out=None):
    """gemv_repack_A80W40."""
    torch = _torch()
    if out is None:
        out = torch.empty(N, dtype=torch.float32, device=a_blob.device)
    capi.check(capi.lib().a81w41_gemv_repack_A80W40(_dev_ptr(a_blob), _dev_ptr(b_blob), _dev_ptr(out), M, N, K, _stream()))
    return out


def gemm_a80w40(a_blob, b_blob, M: int, N: int, K: int, out=None, workspace=None):
    """gemm_repack_A80W40; ``workspace`` (uint8 CUDA tensor) is allocated if not given."""
    torch = _torch()
    L = capi.lib()
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a_blob.device)
    if workspace is None:
        workspace = torch.empty(L.a81w41_gemm_repack_A80W40_workspace_bytes(M, N, K), dtype=torch.uint8, device=a_blob.device)
    capi.check(L.a81w41_gemm_repack_A80W40(_dev_ptr(a_blob), _dev_ptr(b_blob), _dev_ptr(out), M, N, K,
                                           _dev_ptr(workspace), workspace.numel(), _stream()))
    return out


def block_idot_a80w40(a_blob, b_blob, M: int, N: int, K: int):
    torch = _torch()
    out = torch.empty((M, N, K // 32), dtype=torch.int32, device=a_blob.device)
    capi.check(capi.lib().a81w41_block_idot_A80W40(_dev_ptr(a_blob), _dev_ptr(b_blob), _dev_ptr(out), M, N, K, _stream()))
    return out


def attention(q, k_cache, v_cache, pos: int, n_q: int, n_kv: int, scale: float, variant: int = 0):
    """Parity hook a81w41_qwen3_attention: q [M][n_q*128] fp32, caches [n_kv][max_seq][128] fp16 (CUDA tensors)."""
    torch = _torch()
    M, max_seq = q.shape[0], k_cache.shape[1]
    out = torch.empty((M, n_q * 128), dtype=torch.float32, device=q.device)
    pos_dev = torch.tensor([pos], dtype=torch.int32, device=q.device)
    capi.check(capi.lib().a81w41_qwen3_attention(_dev_ptr(q), q.shape[1], _dev_ptr(k_cache), _dev_ptr(v_cache),
                                                 _dev_ptr(pos_dev), _dev_ptr(out), out.shape[1], M, n_q, n_kv, max_seq,
                                                 scale, variant, _stream()))
    return out


def attention_one_token(qkv, q_w, k_w, cos, sin, k_cache, v_cache, pos: int, n_q: int, n_kv: int, eps: float, scale: float,
                        splits: int = 1):
    """Parity hook a81w41_qwen3_attention_one_token: q/k norm + RoPE + cache append + attention for the token
    whose fused row is qkv; appends to k_cache / v_cache [n_kv][max_seq][128] fp16 in place (CUDA tensors)."""
    torch = _torch()
    out = torch.empty(n_q * 128, dtype=torch.float32, device=qkv.device)
    pos_dev = torch.tensor([pos], dtype=torch.int32, device=qkv.device)
    capi.check(capi.lib().a81w41_qwen3_attention_one_token(
        _dev_ptr(qkv), n_q, n_kv, _dev_ptr(q_w), _dev_ptr(k_w), _dev_ptr(cos), _dev_ptr(sin), _dev_ptr(pos_dev),
        _dev_ptr(k_cache), _dev_ptr(v_cache), _dev_ptr(out), k_cache.shape[1], eps, scale, splits, _stream()))
    return out


# ---------------------------------------------------------------- layer objects

class Context:
    """ModelContext (QwenOperator.h:34-43): the activation scratch shared by all layers."""

    def __init__(self, max_rows: int = 4096, max_cols: int = 12288):
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_context_create(max_rows, max_cols, C.byref(h)))
        self.handle = h

    def activation_scratch(self, nbytes: int):
        """Copy of the first ``nbytes`` of the scratch: the last forward's quantised activations."""
        torch = _torch()
        out = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        src = capi.lib().a81w41_context_activation_scratch_dev(self.handle)
        torch.cuda.current_stream().synchronize()
        import ctypes

        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        rc = hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(src), nbytes, 3)  # device to device
        if rc != 0:
            raise RuntimeError(f"hipMemcpy failed with {rc}")
        return out

    def chain_begin(self):
        """Until ``chain_end`` the one-row forward calls of this context's layers (on the current stream) are
        links of a chain of overlapping launches (``a81w41_context_chain_begin``)."""
        capi.check(capi.lib().a81w41_context_chain_begin(self.handle, _stream()))

    def chain_end(self):
        capi.check(capi.lib().a81w41_context_chain_end(self.handle))

    def chain_gave_up(self) -> bool:
        """Synchronises; whether an in-kernel wait of a chain gave up since the last call (and clears it)."""
        flag = C.c_int(0)
        capi.check(capi.lib().a81w41_context_chain_status(self.handle, C.byref(flag)))
        return bool(flag.value)

    def chain_set_spin_limit(self, polls: int):
        capi.check(capi.lib().a81w41_context_chain_set_spin_limit(self.handle, int(polls)))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h and capi is not None:  # module globals are gone at interpreter shutdown
            capi.lib().a81w41_context_destroy(h)


_default_ctx = None


def default_context() -> Context:
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context()
    return _default_ctx


class Linear:
    """Qwen_Linear_with_bias_Int4: holds both repacked weight blobs on the device."""

    def __init__(self, handle, ctx: Context, N: int, K: int):
        self.handle, self.ctx, self.N, self.K = handle, ctx, N, K

    @classmethod
    def from_arrays(cls, w4, scale, offset, N: int, K: int, ctx: Context | None = None) -> "Linear":
        ctx = ctx or default_context()
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_linear_create(
            ctx.handle, N, K, _np_ptr(np.ascontiguousarray(w4, np.uint8)),
            _np_ptr(np.ascontiguousarray(scale, np.float32)),
            _np_ptr(np.ascontiguousarray(offset, np.float32)), C.byref(h)))
        return cls(h, ctx, N, K)

    @classmethod
    def from_blobs(cls, blob16, blob32, N: int, K: int, ctx: Context | None = None) -> "Linear":
        ctx = ctx or default_context()
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_linear_create_from_blobs(
            ctx.handle, N, K, _np_ptr(blob16) if blob16 is not None else None,
            _np_ptr(blob32) if blob32 is not None else None, C.byref(h)))
        return cls(h, ctx, N, K)

    @classmethod
    def load(cls, path: str, N: int, K: int, ctx: Context | None = None) -> "Linear":
        """The reference constructor: (ctx, path, 1, N, K) reading the .bin files under ``path``."""
        ctx = ctx or default_context()
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_linear_load(ctx.handle, path.encode(), 1, N, K, C.byref(h)))
        return cls(h, ctx, N, K)

    KERNELS = {"auto": 0, "int8": 1, "block_scaled": 2}

    def set_kernel(self, choice: str) -> None:
        """Which kernel M > 32 calls contract on: "auto" (by shape, the default), "int8", "block_scaled"."""
        capi.check(capi.lib().a81w41_linear_set_kernel(self.handle, self.KERNELS[choice]))

    def forward(self, x, out=None):
        """x: CUDA float32 [M][K] (or [1][M][K]) -> [M][N]; enqueues on the current stream."""
        torch = _torch()
        x = x.contiguous()
        M = x.numel() // self.K
        if out is None:
            out = torch.empty(x.shape[:-1] + (self.N,), dtype=torch.float32, device=x.device)
        capi.check(capi.lib().a81w41_linear_forward(self.handle, _dev_ptr(x), M, _dev_ptr(out), _stream()))
        return out

    def kernel_name(self, M: int) -> str:
        """Which kernel a forward call of M rows runs on (``a81w41_linear_kernel_name``)."""
        return capi.lib().a81w41_linear_kernel_name(self.handle, int(M)).decode()

    def resident_bytes(self) -> dict:
        """Device bytes of the layer's weight copies (``a81w41_linear_resident_bytes``)."""
        a, b, c = C.c_size_t(), C.c_size_t(), C.c_size_t()
        total = capi.lib().a81w41_linear_resident_bytes(self.handle, C.byref(a), C.byref(b), C.byref(c))
        return {"total": int(total), "fp16_blob": a.value, "fp32_blob": b.value, "block_scaled": c.value}

    def forward_quantized(self, a_blob, M: int, out=None):
        """Rows already quantised (CUDA uint8, M*K/64 blocks of 80 B) -> [M][N] (``a81w41_linear_forward_quantized``)."""
        torch = _torch()
        if out is None:
            out = torch.empty((M, self.N), dtype=torch.float32, device=a_blob.device)
        capi.check(capi.lib().a81w41_linear_forward_quantized(self.handle, _dev_ptr(a_blob), M, _dev_ptr(out), _stream()))
        return out

    def forward_host(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)
        M = x.size // self.K
        out = np.empty(x.shape[:-1] + (self.N,), np.float32)
        capi.check(capi.lib().a81w41_linear_forward_host(self.handle, _np_ptr(x), M, _np_ptr(out)))
        return out

    @staticmethod
    def forward_multi(layers, x, outs=None):
        """[layer(x) for layer in layers] in one call (one launch for M == 1): q/k/v, gate/up."""
        torch = _torch()
        x = x.contiguous()
        M = x.numel() // layers[0].K
        if outs is None:
            outs = [torch.empty(x.shape[:-1] + (l.N,), dtype=torch.float32, device=x.device) for l in layers]
        n = len(layers)
        hs = (C.c_void_p * n)(*[l.handle.value for l in layers])
        ys = (C.c_void_p * n)(*[o.data_ptr() for o in outs])
        capi.check(capi.lib().a81w41_linear_forward_multi(n, hs, _dev_ptr(x), M, ys, _stream()))
        return outs

    @property
    def weight_fp16_ptr(self) -> int:
        return capi.lib().a81w41_linear_weight_fp16_dev(self.handle)

    @property
    def weight_fp32_ptr(self) -> int:
        return capi.lib().a81w41_linear_weight_fp32_dev(self.handle)

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h and capi is not None:
            capi.lib().a81w41_linear_destroy(h)


class Qwen3Model:
    """The Qwen3 forward pass around the layer (``a81w41_qwen3_*``): host arrays in, token ids
    and logits out.  Weights are set per layer; ``which`` follows the C ABI (linears: 0 qkv,
    1 o, 2 gate_up, 3 down; norms: 0 input, 1 post-attention, 2 q, 3 k; layer -1: lm_head /
    final norm)."""

    def __init__(self, n_layers, hidden, n_q_heads, n_kv_heads, intermediate, vocab, max_seq,
                 rope_theta=1e6, rms_eps=1e-6):
        self.cfg = capi.Qwen3Config(n_layers, hidden, n_q_heads, n_kv_heads, intermediate, vocab, max_seq,
                                    rope_theta, rms_eps)
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_qwen3_create(C.byref(self.cfg), C.byref(h)))
        self.handle = h

    @classmethod
    def load(cls, root: str, **cfg) -> "Qwen3Model":
        """Read the reference's weight directory tree (``a81w41_qwen3_load``)."""
        self = cls.__new__(cls)
        self.cfg = capi.Qwen3Config(cfg["n_layers"], cfg["hidden"], cfg["n_q_heads"], cfg["n_kv_heads"],
                                    cfg["intermediate"], cfg["vocab"], cfg["max_seq"], cfg.get("rope_theta", 1e6),
                                    cfg.get("rms_eps", 1e-6))
        h = C.c_void_p()
        capi.check(capi.lib().a81w41_qwen3_load(root.encode(), C.byref(self.cfg), C.byref(h)))
        self.handle = h
        return self

    def set_linear(self, layer, which, w4, scale, offset):
        w4, scale, offset = (np.ascontiguousarray(w4, np.uint8), np.ascontiguousarray(scale, np.float32),
                             np.ascontiguousarray(offset, np.float32))
        capi.check(capi.lib().a81w41_qwen3_set_linear(self.handle, layer, which, w4.ctypes.data, scale.ctypes.data,
                                                      offset.ctypes.data))

    def set_linear_blobs(self, layer, which, blob16, blob32):
        p16 = np.ascontiguousarray(blob16).ctypes.data if blob16 is not None else None
        p32 = np.ascontiguousarray(blob32).ctypes.data if blob32 is not None else None
        capi.check(capi.lib().a81w41_qwen3_set_linear_blobs(self.handle, layer, which, p16, p32))

    def set_norm(self, layer, which, w):
        w = np.ascontiguousarray(w, np.float32)
        capi.check(capi.lib().a81w41_qwen3_set_norm(self.handle, layer, which, w.ctypes.data))

    def set_embedding(self, table_fp16):
        t = np.ascontiguousarray(table_fp16, np.float16)
        assert t.shape == (self.cfg.vocab, self.cfg.hidden)
        capi.check(capi.lib().a81w41_qwen3_set_embedding(self.handle, t.ctypes.data))

    OPTIONS = {"unfused": 0, "attn_fp32": 1, "no_pair": 2, "vector_attention": 3, "attention_split": 4, "chain": 5,
               "chain_spin_limit": 6}

    def set_option(self, name: str, value: int):
        """Test switch of ``a81w41_qwen3_set_option`` (see include/a81w41.h)."""
        capi.check(capi.lib().a81w41_qwen3_set_option(self.handle, self.OPTIONS[name], int(value)))

    def chain_gave_up(self) -> bool:
        """Synchronises; whether a wait inside a chained one-token pass gave up since the last call (and clears it)."""
        flag = C.c_int(0)
        capi.check(capi.lib().a81w41_qwen3_chain_status(self.handle, C.byref(flag)))
        return bool(flag.value)

    def resident_bytes(self) -> dict:
        """Device bytes the model holds, by kind (``a81w41_qwen3_resident_bytes``)."""
        a, b, c, d = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        total = capi.lib().a81w41_qwen3_resident_bytes(self.handle, C.byref(a), C.byref(b), C.byref(c), C.byref(d))
        return {"total": int(total), "linear_weights": a.value, "other_weights": b.value, "kv_cache": c.value, "buffers": d.value}

    BUFFERS = {"residual": 0, "normed": 1, "qkv": 2, "attention": 3, "block_out": 4, "gate_up": 5, "act": 6, "logits": 7}

    def read_buffer(self, name: str, rows: int, cols: int) -> np.ndarray:
        """Parity hook ``a81w41_qwen3_read_buffer``: the first rows x cols floats of an activation buffer."""
        out = np.empty((rows, cols), np.float32)
        capi.check(capi.lib().a81w41_qwen3_read_buffer(self.handle, self.BUFFERS[name], out.ctypes.data, out.size))
        return out

    def reset(self):
        capi.check(capi.lib().a81w41_qwen3_reset(self.handle))

    def forward(self, token_ids):
        """New tokens on top of the cached context -> logits of the last one (numpy fp32 [vocab])."""
        ids = np.ascontiguousarray(token_ids, np.int32)
        logits = np.empty(self.cfg.vocab, np.float32)
        capi.check(capi.lib().a81w41_qwen3_forward(self.handle, ids.ctypes.data, len(ids), logits.ctypes.data))
        return logits

    def generate_greedy(self, prompt, n_new):
        """-> (n_new token ids, prefill ms, decode ms)"""
        ids = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(n_new, np.int32)
        t_pre, t_dec = C.c_double(), C.c_double()
        capi.check(capi.lib().a81w41_qwen3_generate_greedy(self.handle, ids.ctypes.data, len(ids), n_new,
                                                           out.ctypes.data, C.byref(t_pre), C.byref(t_dec)))
        return out, t_pre.value, t_dec.value

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h and capi is not None:
            capi.lib().a81w41_qwen3_destroy(h)
