// Host side of the Qwen3 forward pass: owns weights, KV cache and activation buffers, and
// issues the kernels of one pass in the reference's order (QwenDecoderLayer.cc:39-118,
// QwenAttention.cc:52-208, QwenDecoder.cc:53-141, QwenForCausalLM.cc:11-60).
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <new>
#include <string>
#include <vector>

#include "../../include/a81w41.h"
#include "a81w41_kernels.h"

namespace {

int fail(int status, const char* fmt, ...) {
    char buf[400];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    return a81w41::report_failure(status, buf);
}

#define Q_HIP(expr)                                                                  \
    do {                                                                             \
        hipError_t _e = (expr);                                                      \
        if (_e != hipSuccess) return fail(A81W41_ERR_HIP, "%s: %s", #expr, hipGetErrorString(_e)); \
    } while (0)
#define Q_TRY(expr)              \
    do {                         \
        int _st = (expr);        \
        if (_st) return _st;     \
    } while (0)

constexpr int kHeadDim = 128;

struct LayerWeights {
    a81w41_linear* lin[4] = {nullptr, nullptr, nullptr, nullptr};  // qkv, o, gate_up, down
    float* norm[4] = {nullptr, nullptr, nullptr, nullptr};         // input, post-attention, q, k
    void* k_cache = nullptr;                                       // fp16 [n_kv][max_seq][128]
    void* v_cache = nullptr;
};

}  // namespace

struct a81w41_qwen3 {
    a81w41_qwen3_config cfg{};
    a81w41_context* ctx = nullptr;
    std::vector<LayerWeights> layers;
    a81w41_linear* lm_head = nullptr;
    float* final_norm = nullptr;
    void* embedding = nullptr;  // fp16 [vocab][hidden]
    float *cos_t = nullptr, *sin_t = nullptr;
    // activations, sized for max_seq rows
    float *x = nullptr, *x2 = nullptr, *h = nullptr, *qkv = nullptr, *attn = nullptr, *o = nullptr, *gate_up = nullptr, *act = nullptr;
    float* logits = nullptr;
    int *ids = nullptr, *pos = nullptr, *step = nullptr, *history = nullptr;
    int history_len = 0;
    int host_pos = 0;
    int plan_ctx = 0;              // longest context the passes being enqueued will see (picks the attention's key split)
    float* attn_part = nullptr;    // split attention: n_q * kAttentionMaxSplits * 132 floats
    unsigned* attn_arrive = nullptr;  // ... and n_q arrival counters, zero between launches
    float attn_scale = 0.f;  // 1/sqrt(128) unless a scaling.bin said otherwise
    hipStream_t stream = nullptr;
    int cu_count = 0;  // of the device the model lives on
    // Switches of a81w41_qwen3_set_option: each keeps a fusion off (or fixes the attention's key split) so
    // that tests can compare the fused pass with the separate kernels bit for bit.
    bool opt_unfused = false, opt_attn_fp32 = false, opt_no_pair = false, opt_vector_attention = false, opt_chain = false;
    unsigned opt_spin_limit = 0;  // 0: the chain's default
    int opt_attention_split = 0;
    int qkv_dim() const { return (cfg.n_q_heads + 2 * cfg.n_kv_heads) * kHeadDim; }
};

namespace {

int linear_dims(const a81w41_qwen3* m, int layer, int which, int& N, int& K) {
    const a81w41_qwen3_config& c = m->cfg;
    if (layer == -1) {
        N = c.vocab;
        K = c.hidden;
        return 0;
    }
    if (layer < 0 || layer >= c.n_layers || which < 0 || which > 3)
        return fail(A81W41_ERR_INVALID_ARG, "no linear %d in layer %d", which, layer);
    switch (which) {
        case 0: N = m->qkv_dim(); K = c.hidden; break;
        case 1: N = c.hidden; K = c.n_q_heads * kHeadDim; break;
        case 2: N = 2 * c.intermediate; K = c.hidden; break;
        default: N = c.hidden; K = c.intermediate; break;
    }
    return 0;
}

a81w41_linear** linear_slot(a81w41_qwen3* m, int layer, int which) {
    return layer == -1 ? &m->lm_head : &m->layers[layer].lin[which];
}

int ready(const a81w41_qwen3* m) {
    if (!m->lm_head || !m->final_norm || !m->embedding) return fail(A81W41_ERR_INVALID_ARG, "lm_head, final norm or embedding not set");
    for (size_t l = 0; l < m->layers.size(); l++)
        for (int w = 0; w < 4; w++)
            if (!m->layers[l].lin[w] || !m->layers[l].norm[w])
                return fail(A81W41_ERR_INVALID_ARG, "layer %zu: linear or norm %d not set", l, w);
    return 0;
}

// One pass over M new tokens whose ids are in m->ids; leaves the last token's logits in
// m->logits and advances the device position by M.  Enqueues only.
int enqueue_pass_one_token(a81w41_qwen3* m, hipStream_t s);
bool one_token_pass_usable(const a81w41_qwen3* m);
bool prefill_fusion_usable(const a81w41_qwen3* m);

int enqueue_pass(a81w41_qwen3* m, int M, hipStream_t s) {
    if (M == 1 && one_token_pass_usable(m)) return enqueue_pass_one_token(m, s);
    const a81w41_qwen3_config& c = m->cfg;
    const int qkv_dim = m->qkv_dim(), q_dim = c.n_q_heads * kHeadDim;
    const float scale = m->attn_scale;  // scaling.bin, QwenAttention.cc:44-46
    Q_HIP(a81w41::launch_embed_rows(m->ids, m->embedding, m->x, M, c.hidden, c.vocab, s));
    const float* pending = nullptr;  // output of the previous sub-block, not yet added to the residual stream x
    // Several rows: the norms and SiLU*mul write the quantised blocks of their result straight into the
    // context's scratch, and the matrix-core contraction reads them from there -- the same blocks the
    // linear's own quantiser would produce from the fp32 rows, which therefore never go to memory.
    const bool quant_fused = M > 1 && prefill_fusion_usable(m);
    void* scratch = a81w41_context_activation_scratch_dev(m->ctx);
    const a81w41::GemmScratch& gws = a81w41::context_gemm_scratch(m->ctx);
    // the contraction of rows that sit in the scratch as 80 B blocks: where the layer picks the block-scaled
    // kernel, that one takes them in its own operand format
    auto gemm_from_scratch = [&](a81w41_linear* lin, float* out, int N, int K) -> hipError_t {
        if (a81w41::linear_block_scaled(lin, M)) {
            void* a6 = a81w41::context_a6_scratch(m->ctx);
            if (hipError_t e = a81w41::launch_a80_to_a6(scratch, a6, M, K, s); e != hipSuccess) return e;
            return a81w41::launch_gemm_fp6(a6, a81w41::linear_w6(lin), out, M, N, K, gws, s);
        }
        return a81w41::launch_gemm_fp32(scratch, a81w41_linear_weight_fp32_dev(lin), out, M, N, K, gws, s);
    };
    const bool attn_blocks = !m->opt_vector_attention && a81w41::attention_prefill_fits(M, c.n_q_heads, c.n_kv_heads);
    for (int l = 0; l < c.n_layers; l++) {
        LayerWeights& L = m->layers[l];
        const float* norm_in = pending ? pending : m->x;
        const float* norm_res = pending ? m->x : nullptr;
        if (quant_fused) {
            Q_HIP(a81w41::launch_add_rmsnorm_quant(norm_in, norm_res, L.norm[0], m->x, scratch, M, c.hidden, c.rms_eps, s));
            Q_HIP(gemm_from_scratch(L.lin[0], m->qkv, qkv_dim, c.hidden));
        } else {
            Q_HIP(a81w41::launch_add_rmsnorm(norm_in, norm_res, L.norm[0], m->x, m->h, M, c.hidden, c.rms_eps, s));
            Q_TRY(a81w41_linear_forward(L.lin[0], m->h, M, m->qkv, s));
        }
        Q_HIP(a81w41::launch_qk_norm_rope_cache(m->qkv, qkv_dim, M, c.n_q_heads, c.n_kv_heads, L.norm[2], L.norm[3],
                                                m->cos_t, m->sin_t, m->pos, L.k_cache, L.v_cache, c.max_seq, c.rms_eps, s));
        if (quant_fused && attn_blocks) {  // the matrix-core attention hands o_proj its input as quantised blocks
            Q_HIP(a81w41::launch_attention_prefill(m->qkv, qkv_dim, L.k_cache, L.v_cache, m->pos, nullptr, q_dim, M, c.n_q_heads,
                                                   c.n_kv_heads, c.max_seq, scale, s, scratch));
            Q_HIP(gemm_from_scratch(L.lin[1], m->o, c.hidden, q_dim));
        } else {
            Q_HIP(a81w41::launch_attention(m->qkv, qkv_dim, L.k_cache, L.v_cache, m->pos, m->attn, q_dim, M, c.n_q_heads,
                                           c.n_kv_heads, c.max_seq, scale, s, m->opt_vector_attention ? 1 : 0));
            Q_TRY(a81w41_linear_forward(L.lin[1], m->attn, M, m->o, s));
        }
        if (quant_fused) {
            Q_HIP(a81w41::launch_add_rmsnorm_quant(m->o, m->x, L.norm[1], m->x, scratch, M, c.hidden, c.rms_eps, s));
            Q_HIP(gemm_from_scratch(L.lin[2], m->gate_up, 2 * c.intermediate, c.hidden));
            Q_HIP(a81w41::launch_silu_mul_quant(m->gate_up, scratch, M, c.intermediate, s));
            Q_HIP(gemm_from_scratch(L.lin[3], m->o, c.hidden, c.intermediate));
        } else {
            Q_HIP(a81w41::launch_add_rmsnorm(m->o, m->x, L.norm[1], m->x, m->h, M, c.hidden, c.rms_eps, s));
            Q_TRY(a81w41_linear_forward(L.lin[2], m->h, M, m->gate_up, s));
            Q_HIP(a81w41::launch_silu_mul(m->gate_up, m->act, M, c.intermediate, s));
            Q_TRY(a81w41_linear_forward(L.lin[3], m->act, M, m->o, s));
        }
        pending = m->o;
    }
    Q_HIP(a81w41::launch_add_rmsnorm(pending ? pending : m->x, pending ? m->x : nullptr, m->final_norm, m->x, m->h, M,
                                     c.hidden, c.rms_eps, s));
    // lm_head on the last token only (QwenForCausalLM.cc:43-46)
    Q_TRY(a81w41_linear_forward(m->lm_head, m->h + (size_t)(M - 1) * c.hidden, 1, m->logits, s));
    Q_HIP(a81w41::launch_advance(m->pos, M, s));
    return 0;
}

// The same pass for one token with the elementwise work folded into the neighbouring kernels, five
// launches per layer: every add + RMSNorm runs inside the GEMV that consumes it (qkv, gate_up,
// lm_head); the q/k norm, rotation and cache append run inside the attention kernel, which hands
// o_proj its input as quantised blocks; gate_up hands down_proj silu(gate) * up as quantised
// blocks.  The residual row alternates between x and x2, because a prologue's workgroup 0 writes
// the new residual while the other workgroups still read the old one.
// q/k norm + rotation + cache append + attention for the one new token, in one workgroup per head or,
// for long contexts, in `splits` workgroups per head.
int attention_step(a81w41_qwen3* m, LayerWeights& L, float* out, void* q_out, int splits, float scale, hipStream_t s,
                   const a81w41::ChainLink* link) {
    const a81w41_qwen3_config& c = m->cfg;
    if (splits <= 1)
        Q_HIP(a81w41::launch_attention_one_token(m->qkv, c.n_q_heads, c.n_kv_heads, L.norm[2], L.norm[3], m->cos_t, m->sin_t,
                                                 m->pos, L.k_cache, L.v_cache, out, q_out, c.max_seq, c.rms_eps, scale, s, link));
    else
        Q_HIP(a81w41::launch_attention_one_token_split(m->qkv, c.n_q_heads, c.n_kv_heads, L.norm[2], L.norm[3], m->cos_t,
                                                       m->sin_t, m->pos, L.k_cache, L.v_cache, out, q_out, m->attn_part,
                                                       m->attn_arrive, splits, c.max_seq, c.rms_eps, scale, s, link));
    return 0;
}

int enqueue_pass_one_token(a81w41_qwen3* m, hipStream_t s) {
    const a81w41_qwen3_config& c = m->cfg;
    const int qkv_dim = m->qkv_dim();
    const float scale = m->attn_scale;
    void* scratch = a81w41_context_activation_scratch_dev(m->ctx);
    // test switches (a81w41_qwen3_set_option): attention output as fp32 through o_proj's own quantiser (same
    // bits); gate_up writes fp32 and down_proj's prologue does SiLU * mul and the quantising (same bits)
    const bool attn_fp32 = m->opt_attn_fp32, no_pair = m->opt_no_pair || !a81w41::gemv_pair_fits(2 * c.intermediate, c.hidden);
    // Key split of the attention: one workgroup per head, or several shares per head for long contexts.
    const int env_split = m->opt_attention_split;
    // measured (32 query heads, 64 decode steps after the prompt): one share up to about 560 keys, three up
    // to 1280, four up to 2560, then one per 512 keys
    const int ctx = m->plan_ctx;
    int splits = ctx <= 560 ? 1 : ctx <= 1280 ? 3 : ctx <= 2560 ? 4 : (ctx + 511) / 512;
    // ... but no more workgroups than the chip has CUs (a second round of them would cost more than longer shares)
    const int fit = m->cu_count / c.n_q_heads;
    if (splits > fit) splits = fit;
    if (env_split > 0) splits = env_split;
    splits = splits < 1 ? 1 : (splits > a81w41::kAttentionMaxSplits ? a81w41::kAttentionMaxSplits : splits);
    Q_HIP(a81w41::launch_embed_rows(m->ids, m->embedding, m->o, 1, c.hidden, c.vocab, s));  // pending = the embedding
    // The linears and the attention of the pass are one dependent chain (QwenDecoderLayer.cc:39-105).  As links of
    // an overlapping chain each of them starts while its predecessor runs and requests its first weight blocks
    // (or cache rows) before it waits for it; same kernels' arithmetic, same bits.
    a81w41::ChainState* chain = nullptr;
    if (m->opt_chain && !no_pair && a81w41::gemv_chain_fits(c.hidden, true) && a81w41::gemv_chain_fits(c.intermediate, false) &&
        a81w41::gemv_chain_fits(c.n_q_heads * kHeadDim, false))
        chain = a81w41::context_chain(m->ctx);
    if (chain) {
        chain->spin_limit = m->opt_spin_limit ? m->opt_spin_limit : a81w41::ChainState{}.spin_limit;
        Q_HIP(a81w41::chain_begin(chain, s));
    }
    struct CloseOnExit {  // a failed launch must not leave the chain open (and the side stream forked)
        a81w41::ChainState* c;
        ~CloseOnExit() {
            if (c && c->open) (void)a81w41::chain_end(c);
        }
    } close_on_exit{chain};
    // every launch of the chained pass: the link and stream it gets, and the workgroups the next link waits for
    hipStream_t ls = s;
    a81w41::ChainLink link;
    unsigned grid = 0;
    auto next_link = [&]() { link = a81w41::chain_next(chain, &ls); };
    const float* res_in = nullptr;
    for (int l = 0; l < c.n_layers; l++) {
        LayerWeights& L = m->layers[l];
        a81w41::GemvPrologue p0;
        p0.res_in = res_in;
        p0.res_out = m->x2;
        p0.norm_w = L.norm[0];
        p0.eps = c.rms_eps;
        if (chain) {
            next_link();
            Q_HIP(a81w41::launch_gemv_chain_add_norm(m->o, p0, scratch, a81w41_linear_weight_fp16_dev(L.lin[0]), m->qkv, qkv_dim,
                                                     c.hidden, link, chain->cus, &grid, ls));
            a81w41::chain_launched(chain, grid);
            next_link();
            Q_TRY(attention_step(m, L, attn_fp32 ? m->attn : nullptr, attn_fp32 ? nullptr : scratch, splits, scale, ls, &link));
            a81w41::chain_launched(chain, (unsigned)(c.n_q_heads * splits));
            next_link();
            if (attn_fp32) {
                const void* B = a81w41_linear_weight_fp16_dev(L.lin[1]);
                Q_HIP(a81w41::launch_gemv_chain_fused(m->attn, scratch, 1, &B, &m->o, &c.hidden, c.n_q_heads * kHeadDim, link,
                                                      chain->cus, &grid, ls));
            } else {
                Q_HIP(a81w41::launch_gemv_chain_blob(scratch, a81w41_linear_weight_fp16_dev(L.lin[1]), m->o, c.hidden,
                                                     c.n_q_heads * kHeadDim, link, chain->cus, &grid, ls));
            }
            a81w41::chain_launched(chain, grid);
        } else {
            Q_HIP(a81w41::launch_gemv_add_norm(m->o, p0, scratch, a81w41_linear_weight_fp16_dev(L.lin[0]), m->qkv, qkv_dim,
                                               c.hidden, s));
            if (attn_fp32) {
                Q_TRY(attention_step(m, L, m->attn, nullptr, splits, scale, s, nullptr));
                Q_TRY(a81w41_linear_forward(L.lin[1], m->attn, 1, m->o, s));
            } else {  // the attention kernel hands o_proj its input already quantised
                Q_TRY(attention_step(m, L, nullptr, scratch, splits, scale, s, nullptr));
                Q_HIP(a81w41::launch_gemv_fp16(scratch, a81w41_linear_weight_fp16_dev(L.lin[1]), m->o, c.hidden,
                                               c.n_q_heads * kHeadDim, s));
            }
        }
        a81w41::GemvPrologue p1;
        p1.res_in = m->x2;
        p1.res_out = m->x;
        p1.norm_w = L.norm[1];
        p1.eps = c.rms_eps;
        if (chain) {  // gate_up writes silu(gate) * up as quantised blocks: down_proj's input, ready to contract
            p1.pair_out = static_cast<uint8_t*>(scratch);
            next_link();
            Q_HIP(a81w41::launch_gemv_chain_add_norm_silu_pair(m->o, p1, a81w41_linear_weight_fp16_dev(L.lin[2]),
                                                               2 * c.intermediate, c.hidden, link, chain->cus, &grid, ls));
            a81w41::chain_launched(chain, grid);
            next_link();
            Q_HIP(a81w41::launch_gemv_chain_blob(scratch, a81w41_linear_weight_fp16_dev(L.lin[3]), m->o, c.hidden, c.intermediate,
                                                 link, chain->cus, &grid, ls));
            a81w41::chain_launched(chain, grid);
        } else if (no_pair) {
            Q_HIP(a81w41::launch_gemv_add_norm(m->o, p1, scratch, a81w41_linear_weight_fp16_dev(L.lin[2]), m->gate_up,
                                               2 * c.intermediate, c.hidden, s));
            Q_HIP(a81w41::launch_gemv_silu_mul(m->gate_up, scratch, a81w41_linear_weight_fp16_dev(L.lin[3]), m->o, c.hidden,
                                               c.intermediate, s));
        } else {  // gate_up writes silu(gate) * up as quantised blocks: down_proj's input, ready to contract
            p1.pair_out = static_cast<uint8_t*>(scratch);
            Q_HIP(a81w41::launch_gemv_add_norm_silu_pair(m->o, p1, a81w41_linear_weight_fp16_dev(L.lin[2]), 2 * c.intermediate,
                                                         c.hidden, s));
            Q_HIP(a81w41::launch_gemv_fp16(scratch, a81w41_linear_weight_fp16_dev(L.lin[3]), m->o, c.hidden, c.intermediate, s));
        }
        res_in = m->x;
    }
    a81w41::GemvPrologue pf;
    pf.res_in = res_in;
    pf.res_out = m->x2;
    pf.norm_w = m->final_norm;
    pf.eps = c.rms_eps;
    if (chain) {
        next_link();
        Q_HIP(a81w41::launch_gemv_chain_add_norm(m->o, pf, scratch, a81w41_linear_weight_fp16_dev(m->lm_head), m->logits, c.vocab,
                                                 c.hidden, link, chain->cus, &grid, ls));
        a81w41::chain_launched(chain, grid);
        Q_HIP(a81w41::chain_end(chain));
    } else {
        Q_HIP(a81w41::launch_gemv_add_norm(m->o, pf, scratch, a81w41_linear_weight_fp16_dev(m->lm_head), m->logits, c.vocab,
                                           c.hidden, s));
    }
    Q_HIP(a81w41::launch_advance(m->pos, 1, s));
    return 0;
}

bool prefill_fusion_usable(const a81w41_qwen3* m) {
    if (m->opt_unfused) return false;
    for (const LayerWeights& L : m->layers)
        for (int w = 0; w < 4; w++)
            if (!a81w41_linear_weight_fp32_dev(L.lin[w])) return false;
    return true;
}

bool one_token_pass_usable(const a81w41_qwen3* m) {
    if (m->opt_unfused || !a81w41::gemv_add_norm_fits(m->cfg.hidden)) return false;
    if (a81w41::gemv_lds_bytes(m->cfg.intermediate) > a81w41::kLdsLimitBytes) return false;
    for (const LayerWeights& L : m->layers)
        for (int w = 0; w < 4; w++)
            if (!a81w41_linear_weight_fp16_dev(L.lin[w])) return false;
    return a81w41_linear_weight_fp16_dev(m->lm_head) != nullptr;
}

// After a synchronisation: did an in-kernel wait of a chained pass give up?  (Clears the condition.)
int check_chain(a81w41_qwen3* m) {
    a81w41::ChainState* chain = a81w41::context_chain(m->ctx);
    if (!chain || chain->open) return 0;
    bool gave_up = false;
    Q_HIP(a81w41::chain_status(chain, &gave_up));
    if (gave_up)
        return fail(A81W41_ERR_HIP, "a wait inside the chained one-token pass gave up: the results of that pass are invalid "
                                    "(is the GPU shared with other work?)");
    return 0;
}

template <typename T>
int dev_alloc(T** p, size_t count) {
    Q_HIP(hipMalloc(reinterpret_cast<void**>(p), count * sizeof(T)));
    return 0;
}

}  // namespace

extern "C" {

int a81w41_qwen3_create(const a81w41_qwen3_config* cfg, a81w41_qwen3** out) {
    if (!cfg || !out) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    *out = nullptr;
    const a81w41_qwen3_config& c = *cfg;
    if (c.n_layers < 1 || c.n_q_heads < 1 || c.n_kv_heads < 1 || c.n_q_heads % c.n_kv_heads || c.hidden < 64 ||
        c.hidden % 64 || c.intermediate < 64 || c.intermediate % 64 || c.vocab < 8 || c.vocab % 8 || c.max_seq < 1 ||
        c.max_seq > 8192 || !(c.rope_theta > 0.f) || !(c.rms_eps >= 0.f))
        return fail(A81W41_ERR_INVALID_ARG, "bad model configuration (hidden, intermediate multiples of 64; vocab of 8; "
                                            "max_seq <= 8192; n_q_heads a multiple of n_kv_heads)");
    // on any failure below the half-built model is torn down by its regular destructor
    std::unique_ptr<a81w41_qwen3, void (*)(a81w41_qwen3*)> m(new (std::nothrow) a81w41_qwen3, a81w41_qwen3_destroy);
    if (!m) return fail(A81W41_ERR_HIP, "out of host memory");
    m->cfg = c;
    m->attn_scale = 1.0f / std::sqrt((float)kHeadDim);
    {
        int dev = 0;
        Q_HIP(hipGetDevice(&dev));
        Q_HIP(hipDeviceGetAttribute(&m->cu_count, hipDeviceAttributeMultiprocessorCount, dev));
        if (m->cu_count < 1) return fail(A81W41_ERR_HIP, "device reports no compute units");
    }
    const int max_cols = c.hidden > c.intermediate ? c.hidden : c.intermediate;
    const int q_dim = c.n_q_heads * kHeadDim;
    Q_TRY(a81w41_context_create(c.max_seq, max_cols > q_dim ? max_cols : q_dim, &m->ctx));
    m->layers.resize(c.n_layers);
    const size_t cache_elems = (size_t)c.n_kv_heads * c.max_seq * kHeadDim;
    for (auto& L : m->layers) {
        Q_HIP(hipMalloc(&L.k_cache, cache_elems * 2));
        Q_HIP(hipMalloc(&L.v_cache, cache_elems * 2));
        Q_HIP(hipMemset(L.k_cache, 0, cache_elems * 2));
        Q_HIP(hipMemset(L.v_cache, 0, cache_elems * 2));
    }
    const size_t rows = c.max_seq;
    Q_TRY(dev_alloc(&m->x, rows * c.hidden));
    Q_TRY(dev_alloc(&m->x2, (size_t)c.hidden));  // second residual row of the one-token pass
    Q_TRY(dev_alloc(&m->h, rows * c.hidden));
    Q_TRY(dev_alloc(&m->qkv, rows * m->qkv_dim()));
    Q_TRY(dev_alloc(&m->attn, rows * q_dim));
    Q_TRY(dev_alloc(&m->o, rows * c.hidden));
    Q_TRY(dev_alloc(&m->gate_up, rows * 2 * c.intermediate));
    Q_TRY(dev_alloc(&m->act, rows * c.intermediate));
    Q_TRY(dev_alloc(&m->logits, (size_t)c.vocab));
    Q_TRY(dev_alloc(&m->attn_part, (size_t)c.n_q_heads * a81w41::kAttentionMaxSplits * 132));
    Q_TRY(dev_alloc(&m->attn_arrive, (size_t)c.n_q_heads));
    Q_HIP(hipMemset(m->attn_arrive, 0, (size_t)c.n_q_heads * sizeof(unsigned)));
    Q_TRY(dev_alloc(&m->ids, rows));
    Q_TRY(dev_alloc(&m->pos, 1));
    Q_TRY(dev_alloc(&m->step, 1));
    m->history_len = 8192;
    Q_TRY(dev_alloc(&m->history, (size_t)m->history_len));
    Q_HIP(hipMemset(m->pos, 0, sizeof(int)));
    Q_HIP(hipMemset(m->step, 0, sizeof(int)));
    Q_HIP(hipMemset(m->ids, 0, rows * sizeof(int)));
    // rotate-half tables: angle(pos, j) = pos * theta^(-2 (j mod 64) / 128), both halves alike
    std::vector<float> cs((size_t)c.max_seq * kHeadDim), sn(cs.size());
    for (int p = 0; p < c.max_seq; p++)
        for (int j = 0; j < kHeadDim; j++) {
            const double inv_freq = std::pow((double)c.rope_theta, -2.0 * (j % (kHeadDim / 2)) / (double)kHeadDim);
            const double a = (double)p * inv_freq;
            cs[(size_t)p * kHeadDim + j] = (float)std::cos(a);
            sn[(size_t)p * kHeadDim + j] = (float)std::sin(a);
        }
    Q_TRY(dev_alloc(&m->cos_t, cs.size()));
    Q_TRY(dev_alloc(&m->sin_t, sn.size()));
    Q_HIP(hipMemcpy(m->cos_t, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
    Q_HIP(hipMemcpy(m->sin_t, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
    Q_HIP(hipStreamCreate(&m->stream));
    *out = m.release();
    return A81W41_OK;
}

void a81w41_qwen3_destroy(a81w41_qwen3* m) {
    if (!m) return;
    if (m->stream) (void)hipStreamSynchronize(m->stream);
    for (auto& L : m->layers) {
        for (int w = 0; w < 4; w++) {
            a81w41_linear_destroy(L.lin[w]);
            (void)hipFree(L.norm[w]);
        }
        (void)hipFree(L.k_cache);
        (void)hipFree(L.v_cache);
    }
    a81w41_linear_destroy(m->lm_head);
    void* bufs[] = {m->final_norm, m->embedding, m->cos_t, m->sin_t, m->x, m->x2, m->h, m->qkv, m->attn, m->o,
                    m->gate_up, m->act, m->logits, m->ids, m->pos, m->step, m->history, m->attn_part, m->attn_arrive};
    for (void* b : bufs) (void)hipFree(b);
    if (m->stream) (void)hipStreamDestroy(m->stream);
    a81w41_context_destroy(m->ctx);
    delete m;
}

int a81w41_qwen3_set_linear(a81w41_qwen3* m, int layer, int which, const uint8_t* weight_int4, const float* scale,
                            const float* offset) {
    if (!m) return fail(A81W41_ERR_INVALID_ARG, "null model");
    int N, K;
    Q_TRY(linear_dims(m, layer, which, N, K));
    a81w41_linear** slot = linear_slot(m, layer, which);
    a81w41_linear* fresh = nullptr;
    Q_TRY(a81w41_linear_create(m->ctx, N, K, weight_int4, scale, offset, &fresh));
    a81w41_linear_destroy(*slot);
    *slot = fresh;
    return A81W41_OK;
}

int a81w41_qwen3_set_linear_blobs(a81w41_qwen3* m, int layer, int which, const void* blob_fp16, const void* blob_fp32) {
    if (!m) return fail(A81W41_ERR_INVALID_ARG, "null model");
    int N, K;
    Q_TRY(linear_dims(m, layer, which, N, K));
    a81w41_linear** slot = linear_slot(m, layer, which);
    a81w41_linear* fresh = nullptr;
    Q_TRY(a81w41_linear_create_from_blobs(m->ctx, N, K, blob_fp16, blob_fp32, &fresh));
    a81w41_linear_destroy(*slot);
    *slot = fresh;
    return A81W41_OK;
}

int a81w41_qwen3_set_norm(a81w41_qwen3* m, int layer, int which, const float* weight) {
    if (!m || !weight) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    float** slot;
    size_t n;
    if (layer == -1) {
        slot = &m->final_norm;
        n = m->cfg.hidden;
    } else {
        if (layer < 0 || layer >= m->cfg.n_layers || which < 0 || which > 3)
            return fail(A81W41_ERR_INVALID_ARG, "no norm %d in layer %d", which, layer);
        slot = &m->layers[layer].norm[which];
        n = which < 2 ? (size_t)m->cfg.hidden : (size_t)kHeadDim;
    }
    if (!*slot) Q_TRY(dev_alloc(slot, n));
    Q_HIP(hipMemcpy(*slot, weight, n * 4, hipMemcpyHostToDevice));
    return A81W41_OK;
}

int a81w41_qwen3_set_embedding(a81w41_qwen3* m, const uint16_t* table_fp16) {
    if (!m || !table_fp16) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    const size_t bytes = (size_t)m->cfg.vocab * m->cfg.hidden * 2;
    if (!m->embedding) Q_HIP(hipMalloc(&m->embedding, bytes));
    Q_HIP(hipMemcpy(m->embedding, table_fp16, bytes, hipMemcpyHostToDevice));
    return A81W41_OK;
}

int a81w41_qwen3_set_option(a81w41_qwen3* m, int option, int value) {
    if (!m) return fail(A81W41_ERR_INVALID_ARG, "null model");
    switch (option) {
        case A81W41_QWEN3_OPT_UNFUSED: m->opt_unfused = value != 0; break;
        case A81W41_QWEN3_OPT_ATTN_FP32: m->opt_attn_fp32 = value != 0; break;
        case A81W41_QWEN3_OPT_NO_PAIR: m->opt_no_pair = value != 0; break;
        case A81W41_QWEN3_OPT_VECTOR_ATTENTION: m->opt_vector_attention = value != 0; break;
        case A81W41_QWEN3_OPT_CHAIN: m->opt_chain = value != 0; break;
        case A81W41_QWEN3_OPT_CHAIN_SPIN_LIMIT:
            if (value < 0) return fail(A81W41_ERR_INVALID_ARG, "spin limit must be >= 0 (0: default)");
            m->opt_spin_limit = (unsigned)value;
            break;
        case A81W41_QWEN3_OPT_ATTENTION_SPLIT:
            if (value < 0 || value > a81w41::kAttentionMaxSplits)
                return fail(A81W41_ERR_INVALID_ARG, "attention split must be 0 (automatic) .. %d", a81w41::kAttentionMaxSplits);
            m->opt_attention_split = value;
            break;
        default: return fail(A81W41_ERR_INVALID_ARG, "unknown option %d", option);
    }
    return A81W41_OK;
}

size_t a81w41_qwen3_resident_bytes(const a81w41_qwen3* m, size_t* linear_weights, size_t* other_weights, size_t* kv_cache,
                                   size_t* buffers) {
    if (!m) return 0;
    const a81w41_qwen3_config& c = m->cfg;
    size_t lin = 0, other = 0;
    for (const LayerWeights& L : m->layers) {
        for (int w = 0; w < 4; w++) {
            lin += a81w41_linear_resident_bytes(L.lin[w], nullptr, nullptr, nullptr);
            if (L.norm[w]) other += (size_t)(w < 2 ? c.hidden : kHeadDim) * sizeof(float);
        }
    }
    lin += a81w41_linear_resident_bytes(m->lm_head, nullptr, nullptr, nullptr);
    if (m->final_norm) other += (size_t)c.hidden * sizeof(float);
    if (m->embedding) other += (size_t)c.vocab * c.hidden * 2;
    other += 2 * (size_t)c.max_seq * kHeadDim * sizeof(float);  // rotation tables
    const size_t kv = 2 * (size_t)c.n_layers * c.n_kv_heads * c.max_seq * kHeadDim * 2;
    const size_t rows = c.max_seq;
    size_t buf = (rows * c.hidden * 3 + (size_t)c.hidden + rows * m->qkv_dim() + rows * c.n_q_heads * kHeadDim +
                  rows * 3 * c.intermediate + (size_t)c.vocab) * sizeof(float);
    buf += (size_t)c.n_q_heads * a81w41::kAttentionMaxSplits * 132 * sizeof(float) + (size_t)c.n_q_heads * sizeof(unsigned);
    buf += (rows + 2 + (size_t)m->history_len) * sizeof(int);
    buf += a81w41::context_resident_bytes(m->ctx);
    if (linear_weights) *linear_weights = lin;
    if (other_weights) *other_weights = other;
    if (kv_cache) *kv_cache = kv;
    if (buffers) *buffers = buf;
    return lin + other + kv + buf;
}

int a81w41_qwen3_chain_status(a81w41_qwen3* m, int* gave_up) {
    if (!m || !gave_up) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    Q_HIP(hipStreamSynchronize(m->stream));
    return a81w41_context_chain_status(m->ctx, gave_up);
}

int a81w41_qwen3_read_buffer(a81w41_qwen3* m, int which, float* host_out, size_t count) {
    if (!m || !host_out) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    const a81w41_qwen3_config& c = m->cfg;
    const size_t rows = c.max_seq;
    const float* src = nullptr;
    size_t have = 0;
    switch (which) {
        case A81W41_QWEN3_BUF_RESIDUAL: src = m->x; have = rows * c.hidden; break;
        case A81W41_QWEN3_BUF_NORMED: src = m->h; have = rows * c.hidden; break;
        case A81W41_QWEN3_BUF_QKV: src = m->qkv; have = rows * m->qkv_dim(); break;
        case A81W41_QWEN3_BUF_ATTENTION: src = m->attn; have = rows * c.n_q_heads * kHeadDim; break;
        case A81W41_QWEN3_BUF_BLOCK_OUT: src = m->o; have = rows * c.hidden; break;
        case A81W41_QWEN3_BUF_GATE_UP: src = m->gate_up; have = rows * 2 * c.intermediate; break;
        case A81W41_QWEN3_BUF_ACT: src = m->act; have = rows * c.intermediate; break;
        case A81W41_QWEN3_BUF_LOGITS: src = m->logits; have = c.vocab; break;
        default: return fail(A81W41_ERR_INVALID_ARG, "unknown buffer %d", which);
    }
    if (count > have) return fail(A81W41_ERR_INVALID_ARG, "buffer %d holds %zu floats, %zu asked for", which, have, count);
    Q_HIP(hipStreamSynchronize(m->stream));
    Q_HIP(hipMemcpy(host_out, src, count * sizeof(float), hipMemcpyDeviceToHost));
    return A81W41_OK;
}

int a81w41_qwen3_reset(a81w41_qwen3* m) {
    if (!m) return fail(A81W41_ERR_INVALID_ARG, "null model");
    Q_HIP(hipStreamSynchronize(m->stream));
    Q_HIP(hipMemset(m->pos, 0, sizeof(int)));
    Q_HIP(hipMemset(m->step, 0, sizeof(int)));
    m->host_pos = 0;
    return A81W41_OK;
}

int a81w41_qwen3_forward(a81w41_qwen3* m, const int* token_ids, int n_tokens, float* logits_host) {
    if (!m || !token_ids) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    Q_TRY(ready(m));
    if (n_tokens < 1 || m->host_pos + n_tokens > m->cfg.max_seq)
        return fail(A81W41_ERR_INVALID_ARG, "%d tokens on top of %d do not fit max_seq %d", n_tokens, m->host_pos, m->cfg.max_seq);
    Q_HIP(hipMemcpy(m->ids, token_ids, (size_t)n_tokens * sizeof(int), hipMemcpyHostToDevice));
    m->plan_ctx = m->host_pos + n_tokens;
    Q_TRY(enqueue_pass(m, n_tokens, m->stream));
    Q_HIP(hipStreamSynchronize(m->stream));
    m->host_pos += n_tokens;
    Q_TRY(check_chain(m));
    if (logits_host) Q_HIP(hipMemcpy(logits_host, m->logits, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost));
    return A81W41_OK;
}

int a81w41_qwen3_attention(const float* q_dev, int q_row_stride, const void* k_cache_dev, const void* v_cache_dev,
                           const int* pos_dev, float* out_dev, int out_row_stride, int M, int n_q, int n_kv, int max_seq,
                           float scale, int variant, void* stream) {
    if (!q_dev || !k_cache_dev || !v_cache_dev || !pos_dev || !out_dev) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    if (M < 1 || n_kv < 1 || n_q < n_kv || n_q % n_kv || max_seq < 1 || max_seq > 8192 || q_row_stride < n_q * kHeadDim ||
        out_row_stride < n_q * kHeadDim || q_row_stride % 4 || out_row_stride % 4 || variant < 0 || variant > 6)
        return fail(A81W41_ERR_INVALID_ARG, "bad attention shape");
    if ((reinterpret_cast<uintptr_t>(q_dev) | reinterpret_cast<uintptr_t>(out_dev) | reinterpret_cast<uintptr_t>(k_cache_dev) |
         reinterpret_cast<uintptr_t>(v_cache_dev)) & 15)
        return fail(A81W41_ERR_INVALID_ARG, "attention buffers must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (variant >= 2) {
        const int heads = variant == 2 ? 0 : 1 << (variant - 3);  // 3..6: 1, 2, 4, 8 heads per workgroup
        if (!a81w41::attention_prefill_fits(M, n_q, n_kv) || (heads && (n_q / n_kv) % heads))
            return fail(A81W41_ERR_INVALID_ARG,
                        "the matrix-core attention needs M > 8, n_q / n_kv in {1, 2, 4, 8} and a divisor of it as heads per workgroup");
        Q_HIP(a81w41::launch_attention_prefill(q_dev, q_row_stride, k_cache_dev, v_cache_dev, pos_dev, out_dev, out_row_stride, M,
                                               n_q, n_kv, max_seq, scale, s, nullptr, heads));
    } else {
        Q_HIP(a81w41::launch_attention(q_dev, q_row_stride, k_cache_dev, v_cache_dev, pos_dev, out_dev, out_row_stride, M, n_q, n_kv,
                                       max_seq, scale, s, variant));
    }
    return A81W41_OK;
}

int a81w41_qwen3_attention_one_token(const float* qkv_dev, int n_q, int n_kv, const float* q_w_dev, const float* k_w_dev,
                                     const float* cos_dev, const float* sin_dev, const int* pos_dev, void* k_cache_dev,
                                     void* v_cache_dev, float* out_dev, int max_seq, float eps, float scale, int splits,
                                     void* stream) {
    if (!qkv_dev || !q_w_dev || !k_w_dev || !cos_dev || !sin_dev || !pos_dev || !k_cache_dev || !v_cache_dev || !out_dev)
        return fail(A81W41_ERR_INVALID_ARG, "null argument");
    if (n_kv < 1 || n_q < n_kv || n_q % n_kv || max_seq < 1 || max_seq > 8192 || splits < 1 ||
        splits > a81w41::kAttentionMaxSplits)
        return fail(A81W41_ERR_INVALID_ARG, "bad attention shape");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (splits == 1) {
        Q_HIP(a81w41::launch_attention_one_token(qkv_dev, n_q, n_kv, q_w_dev, k_w_dev, cos_dev, sin_dev, pos_dev, k_cache_dev,
                                                 v_cache_dev, out_dev, nullptr, max_seq, eps, scale, s));
        return A81W41_OK;
    }
    float* part = nullptr;
    unsigned* arrive = nullptr;
    Q_HIP(hipMalloc(&part, (size_t)n_q * splits * 132 * sizeof(float)));
    hipError_t e = hipMalloc(&arrive, (size_t)n_q * sizeof(unsigned));
    if (e == hipSuccess) e = hipMemsetAsync(arrive, 0, (size_t)n_q * sizeof(unsigned), s);
    if (e == hipSuccess)
        e = a81w41::launch_attention_one_token_split(qkv_dev, n_q, n_kv, q_w_dev, k_w_dev, cos_dev, sin_dev, pos_dev, k_cache_dev,
                                                     v_cache_dev, out_dev, nullptr, part, arrive, splits, max_seq, eps, scale, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(part);
    (void)hipFree(arrive);
    Q_HIP(e);
    return A81W41_OK;
}

int a81w41_qwen3_generate_greedy(a81w41_qwen3* m, const int* prompt, int n_prompt, int n_new, int* out_tokens,
                                 double* prefill_ms, double* decode_ms) {
    if (!m || !prompt || !out_tokens) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    Q_TRY(ready(m));
    if (n_prompt < 1 || n_new < 1 || n_new > m->history_len || m->host_pos + n_prompt + n_new - 1 > m->cfg.max_seq)
        return fail(A81W41_ERR_INVALID_ARG, "prompt of %d and %d new tokens on top of %d do not fit max_seq %d", n_prompt,
                    n_new, m->host_pos, m->cfg.max_seq);
    hipStream_t s = m->stream;
    // events and graph objects are released on every way out of this function
    struct Scoped {
        hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        ~Scoped() {
            for (hipEvent_t e : ev)
                if (e) (void)hipEventDestroy(e);
            if (exec) (void)hipGraphExecDestroy(exec);
            if (graph) (void)hipGraphDestroy(graph);
        }
    } own;
    for (hipEvent_t& e : own.ev) Q_HIP(hipEventCreate(&e));
    const hipEvent_t e0 = own.ev[0], e1 = own.ev[1], e2 = own.ev[2], e3 = own.ev[3];
    Q_HIP(hipMemcpy(m->ids, prompt, (size_t)n_prompt * sizeof(int), hipMemcpyHostToDevice));
    Q_HIP(hipMemset(m->step, 0, sizeof(int)));
    Q_HIP(hipEventRecord(e0, s));
    m->plan_ctx = m->host_pos + n_prompt + n_new - 1;  // also what the decode steps captured below will reach
    Q_TRY(enqueue_pass(m, n_prompt, s));
    // first new token: argmax of the prompt's logits; it becomes the next pass's input id
    Q_HIP(a81w41::launch_argmax_token(m->logits, m->cfg.vocab, m->ids, m->history, m->history_len, m->step, s));
    Q_HIP(hipEventRecord(e1, s));
    Q_HIP(hipStreamSynchronize(s));
    m->host_pos += n_prompt;

    const int n_steps = n_new - 1;
    if (n_steps > 0) {
        // one decode step = a pass over the single id in ids[0] + argmax; captured once, replayed
        hipGraph_t& graph = own.graph;
        hipGraphExec_t& exec = own.exec;
        bool captured = false;
        if (hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal) == hipSuccess) {
            int st = enqueue_pass(m, 1, s);
            if (st == 0 && a81w41::launch_argmax_token(m->logits, m->cfg.vocab, m->ids, m->history, m->history_len, m->step, s) != hipSuccess)
                st = 1;
            const hipError_t ee = hipStreamEndCapture(s, &graph);
            if (st == 0 && ee == hipSuccess && graph && hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess)
                captured = true;
        }
        (void)hipGetLastError();
        Q_HIP(hipEventRecord(e3, s));
        for (int i = 0; i < n_steps; i++) {
            if (captured) {
                Q_HIP(hipGraphLaunch(exec, s));
            } else {
                Q_TRY(enqueue_pass(m, 1, s));
                Q_HIP(a81w41::launch_argmax_token(m->logits, m->cfg.vocab, m->ids, m->history, m->history_len, m->step, s));
            }
        }
        Q_HIP(hipEventRecord(e2, s));
        Q_HIP(hipStreamSynchronize(s));
        m->host_pos += n_steps;
    } else {
        Q_HIP(hipEventRecord(e2, s));
        Q_HIP(hipStreamSynchronize(s));
    }
    float ms01 = 0.f, ms12 = 0.f;
    Q_HIP(hipEventElapsedTime(&ms01, e0, e1));
    if (n_steps > 0) Q_HIP(hipEventElapsedTime(&ms12, e3, e2));
    if (prefill_ms) *prefill_ms = ms01;
    if (decode_ms) *decode_ms = ms12;
    Q_TRY(check_chain(m));
    Q_HIP(hipMemcpy(out_tokens, m->history, (size_t)n_new * sizeof(int), hipMemcpyDeviceToHost));
    return A81W41_OK;
}

}  // extern "C"

namespace {

int read_exact(const std::string& name, void* dst, size_t bytes) {
    FILE* f = fopen(name.c_str(), "rb");
    if (!f) return fail(A81W41_ERR_IO, "cannot open %s", name.c_str());
    const size_t got = fread(dst, 1, bytes, f);
    fclose(f);
    if (got != bytes) return fail(A81W41_ERR_IO, "%s: expected %zu bytes, read %zu", name.c_str(), bytes, got);
    return A81W41_OK;
}

bool file_exists(const std::string& name) {
    FILE* f = fopen(name.c_str(), "rb");
    if (f) fclose(f);
    return f != nullptr;
}

struct LinearFiles {
    std::vector<uint8_t> w4;
    std::vector<float> scale, offset;
};

// <dir>/weight_int4.bin, scaling_factor_int4.bin, offset_int4.bin (QwenOperator.h:137-140), appended to f
int append_linear_files(const std::string& dir, int N, int K, LinearFiles& f) {
    const size_t w0 = f.w4.size(), s0 = f.scale.size();
    f.w4.resize(w0 + (size_t)N * K / 2);
    f.scale.resize(s0 + (size_t)N * K / 32);
    f.offset.resize(s0 + (size_t)N * K / 32);
    Q_TRY(read_exact(dir + "/weight_int4.bin", f.w4.data() + w0, (size_t)N * K / 2));
    Q_TRY(read_exact(dir + "/scaling_factor_int4.bin", f.scale.data() + s0, (size_t)N * K / 32 * 4));
    Q_TRY(read_exact(dir + "/offset_int4.bin", f.offset.data() + s0, (size_t)N * K / 32 * 4));
    return 0;
}

int load_norm(a81w41_qwen3* m, int layer, int which, const std::string& file, size_t n) {
    std::vector<float> w(n);
    Q_TRY(read_exact(file, w.data(), n * 4));
    return a81w41_qwen3_set_norm(m, layer, which, w.data());
}

int load_into(a81w41_qwen3* m, const std::string& root) {
    const a81w41_qwen3_config& c = m->cfg;
    const int q_dim = c.n_q_heads * kHeadDim, qkv_dim = m->qkv_dim();
    const std::string model = root + "/model";
    for (int l = 0; l < c.n_layers; l++) {
        const std::string lp = model + "/layers/layer" + std::to_string(l);
        {
            LinearFiles f;
            Q_TRY(append_linear_files(lp + "/self_attn/qkv_proj", qkv_dim, c.hidden, f));
            Q_TRY(a81w41_qwen3_set_linear(m, l, 0, f.w4.data(), f.scale.data(), f.offset.data()));
        }
        {
            LinearFiles f;
            Q_TRY(append_linear_files(lp + "/self_attn/o_proj", c.hidden, q_dim, f));
            Q_TRY(a81w41_qwen3_set_linear(m, l, 1, f.w4.data(), f.scale.data(), f.offset.data()));
        }
        {   // gate rows, then up rows: one linear of 2*intermediate outputs
            LinearFiles f;
            Q_TRY(append_linear_files(lp + "/mlp/gate_proj", c.intermediate, c.hidden, f));
            Q_TRY(append_linear_files(lp + "/mlp/up_proj", c.intermediate, c.hidden, f));
            Q_TRY(a81w41_qwen3_set_linear(m, l, 2, f.w4.data(), f.scale.data(), f.offset.data()));
        }
        {
            LinearFiles f;
            Q_TRY(append_linear_files(lp + "/mlp/down_proj", c.hidden, c.intermediate, f));
            Q_TRY(a81w41_qwen3_set_linear(m, l, 3, f.w4.data(), f.scale.data(), f.offset.data()));
        }
        Q_TRY(load_norm(m, l, 0, lp + "/input_layernorm/weight.bin", c.hidden));
        Q_TRY(load_norm(m, l, 1, lp + "/post_attention_layernorm/weight.bin", c.hidden));
        Q_TRY(load_norm(m, l, 2, lp + "/self_attn/q_norm/weight.bin", kHeadDim));
        Q_TRY(load_norm(m, l, 3, lp + "/self_attn/k_norm/weight.bin", kHeadDim));
        if (l == 0 && file_exists(lp + "/self_attn/scaling.bin")) Q_TRY(read_exact(lp + "/self_attn/scaling.bin", &m->attn_scale, 4));
    }
    {
        LinearFiles f;
        Q_TRY(append_linear_files(root + "/lm_head", c.vocab, c.hidden, f));
        Q_TRY(a81w41_qwen3_set_linear(m, -1, 0, f.w4.data(), f.scale.data(), f.offset.data()));
    }
    Q_TRY(load_norm(m, -1, 0, model + "/norm/weight.bin", c.hidden));
    {   // fp32 table on disk (ops/embedding.cc:7-9), fp16 in HBM
        const size_t n = (size_t)c.vocab * c.hidden;
        std::vector<float> t(n);
        Q_TRY(read_exact(model + "/embed_tokens/weight.bin", t.data(), n * 4));
        std::vector<uint16_t> hbits(n);
        for (size_t i = 0; i < n; i++) hbits[i] = a81w41::float_to_half_bits(t[i]);
        Q_TRY(a81w41_qwen3_set_embedding(m, hbits.data()));
    }
    // the reference's precomputed tables (include/ops/RotaryPosEmb.h:8-14) replace the computed ones
    const std::string rp = model + "/rotary_emb";
    if (file_exists(rp + "/cos_cached.bin") && file_exists(rp + "/sin_cached.bin")) {
        const size_t n = (size_t)c.max_seq * kHeadDim;
        std::vector<float> cs(n), sn(n);
        Q_TRY(read_exact(rp + "/cos_cached.bin", cs.data(), n * 4));
        Q_TRY(read_exact(rp + "/sin_cached.bin", sn.data(), n * 4));
        Q_HIP(hipMemcpy(m->cos_t, cs.data(), n * 4, hipMemcpyHostToDevice));
        Q_HIP(hipMemcpy(m->sin_t, sn.data(), n * 4, hipMemcpyHostToDevice));
    }
    return 0;
}

}  // namespace

extern "C" int a81w41_qwen3_load(const char* root, const a81w41_qwen3_config* cfg, a81w41_qwen3** out) {
    if (!root || !out) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    *out = nullptr;
    a81w41_qwen3* m = nullptr;
    Q_TRY(a81w41_qwen3_create(cfg, &m));
    const int st = load_into(m, std::string(root));
    if (st) {
        a81w41_qwen3_destroy(m);
        return st;
    }
    *out = m;
    return A81W41_OK;
}
