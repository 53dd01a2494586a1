// The non-quantised operators around the A81W41 linears in the Qwen3 forward pass, written for
// one token stream on one GPU.  Activations are fp32 row-major, the KV cache is fp16
// [kv_head][max_seq][128], the embedding table fp16.  Positions come from device memory
// (pos_dev[0] = number of tokens already in the cache), so a captured decode step can be
// replayed unchanged.  Every index that depends on device data is clamped into its array.
//
// What each kernel restates:
//   embed_rows              Embedding::forward                 src/ops/embedding.cc:13-26
//   add_rmsnorm             add + Qwen3RMSNorm::forward        QwenOperator.cc:24-53, 715-722
//   qk_norm_rope_cache      per-head RMSNorm, rotate-half RoPE, KV-cache append
//                                                            QwenAttention.cc:78-122, ops/RotaryPosEmb.cc:6-78
//   attention               QK^T * scale, causal mask, softmax, PV (GQA)   QwenAttention.cc:150-195
//   silu_mul                Qwen3SiLuMul                       QwenOperator.cc:697-713
//   add_rmsnorm / silu_mul with q_out: the same, followed in the same thread by the fp32-parameter
//                           activation quantiser of the linear that consumes the row
//                           (quantize_row_q8_1_repack_fp32, quantized_gemx_kernels.cc:803-911), so the
//                           fp32 row never goes to memory; the blocks are bit-identical to quantising it
//   argmax_token            sample_token_greedy (first maximum)  Pipeline.cc:54-62
#include "a81w41_kernels.h"
#include "quantize_common.h"

#include <hip/hip_fp16.h>

#include <cstdlib>

namespace a81w41 {
namespace {

constexpr int kHeadDim = 128;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// block-wide sum over THREADS threads; red: THREADS/64 floats of LDS
template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < THREADS / 64; w++) s += red[w];
    return s;
}

// float4 number j of a row-major fp32 array -> its place in the array's 80 B blocks.  The 8 lanes of
// an aligned group must hold the 8 float4 of one 32-block (consecutive j, all 8 lanes active).
__device__ __forceinline__ void store_quantized_float4(uint8_t* __restrict__ blob, long long j, float4 v) {
    const Quant4 qz = quantize_float4_of_block32(v);
    uint8_t* blk = blob + (j >> 4) * kABlock32;
    const int h = (int)(j >> 3) & 1, p = (int)j & 7;
    *reinterpret_cast<uint32_t*>(blk + 16 + 32 * h + 4 * p) = qz.packed;
    if (p == 0) {
        float* par = reinterpret_cast<float*>(blk);
        par[h] = qz.d;
        par[2 + h] = qz.ssum;
    }
}

__global__ __launch_bounds__(256) void embed_rows_kernel(const int* __restrict__ ids, const __half* __restrict__ table,
                                                       float* __restrict__ out, int hidden, int vocab) {
    const int m = blockIdx.x;
    const int id = min(max(ids[m], 0), vocab - 1);
    // hidden is a multiple of 64 and the table 16-byte aligned: eight halves per load, two float4 per store
    const uint4* row = reinterpret_cast<const uint4*>(table + (size_t)id * hidden);
    float4* dst = reinterpret_cast<float4*>(out + (size_t)m * hidden);
    for (int j = threadIdx.x; j < (hidden >> 3); j += 256) {
        const uint4 u = row[j];
        const __half2* h2 = reinterpret_cast<const __half2*>(&u);
        const float2 a = __half22float2(h2[0]), b = __half22float2(h2[1]), c = __half22float2(h2[2]), d = __half22float2(h2[3]);
        dst[2 * j] = make_float4(a.x, a.y, b.x, b.y);
        dst[2 * j + 1] = make_float4(c.x, c.y, d.x, d.y);
    }
}

// res_out = x + res_in (res_in may be null: res_out = x); norm_out = res_out / sqrt(mean(res_out^2) + eps) * w
// (res_out may be the same buffer as x or res_in: every element is read and written by one thread).
// One workgroup per row; a thread keeps up to 4 float4 of the row in registers (hidden <= 16 * THREADS),
// longer rows are re-read from res_out.  With QUANT the normalised row is written as 80 B blocks to
// q_out instead of as floats to norm_out.
template <int THREADS, bool QUANT>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_kernel(const float* x, const float* res_in, const float* __restrict__ w,
                                                            float* res_out, float* __restrict__ norm_out,
                                                            uint8_t* __restrict__ q_out, int hidden, float eps) {
    __shared__ float red[THREADS / 64];
    const size_t base = (size_t)blockIdx.x * hidden;
    const int n4 = hidden >> 2;  // hidden is a multiple of 64
    const float4* x4 = reinterpret_cast<const float4*>(x + base);
    const float4* r4 = res_in ? reinterpret_cast<const float4*>(res_in + base) : nullptr;
    float4* o4 = reinterpret_cast<float4*>(res_out + base);
    float4 keep[4];
    float ss = 0.f;
    auto add_in = [&](int j) {
        float4 v = x4[j];
        if (r4 != nullptr) {
            const float4 r = r4[j];
            v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
        }
        o4[j] = v;
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        return v;
    };
#pragma unroll
    for (int slot = 0; slot < 4; slot++) {
        const int j = threadIdx.x + slot * THREADS;
        keep[slot] = j < n4 ? add_in(j) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int j = threadIdx.x + 4 * THREADS; j < n4; j += THREADS) (void)add_in(j);
    const float total = block_sum<THREADS>(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4* n4p = QUANT ? nullptr : reinterpret_cast<float4*>(norm_out + base);
    auto scale_out = [&](int j, float4 v) {
        const float4 g = w4[j];
        const float4 n = make_float4((v.x * inv) * g.x, (v.y * inv) * g.y, (v.z * inv) * g.z, (v.w * inv) * g.w);
        if (QUANT)  // j < n4 holds for whole groups of 8 lanes: n4 is a multiple of 16
            store_quantized_float4(q_out, (long long)blockIdx.x * n4 + j, n);
        else
            n4p[j] = n;
    };
#pragma unroll
    for (int slot = 0; slot < 4; slot++) {
        const int j = threadIdx.x + slot * THREADS;
        if (j < n4) scale_out(j, keep[slot]);
    }
    for (int j = threadIdx.x + 4 * THREADS; j < n4; j += THREADS) scale_out(j, o4[j]);
}

// One wave per (token, head).  Heads 0..n_q-1 are query heads (normalised and rotated in place),
// then n_kv key heads (normalised, rotated, stored fp16 at the token's position) and n_kv value
// heads (stored fp16).  Lane l owns dimensions l and l + 64, the two partners of rotate-half.
__global__ __launch_bounds__(64) void qk_norm_rope_cache_kernel(float* __restrict__ qkv, int row_stride, int n_q, int n_kv,
                                                              const float* __restrict__ q_w, const float* __restrict__ k_w,
                                                              const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                              const int* __restrict__ pos_dev, __half* __restrict__ k_cache,
                                                              __half* __restrict__ v_cache, int max_seq, float eps) {
    const int m = blockIdx.x, head = blockIdx.y, l = threadIdx.x;
    const int pos = min(pos_dev[0] + m, max_seq - 1);
    float* src = qkv + (size_t)m * row_stride + (size_t)head * kHeadDim;
    const float x0 = src[l], x1 = src[l + 64];
    if (head >= n_q + n_kv) {  // value head
        __half* dst = v_cache + ((size_t)(head - n_q - n_kv) * max_seq + pos) * kHeadDim;
        dst[l] = __float2half_rn(x0);
        dst[l + 64] = __float2half_rn(x1);
        return;
    }
    const float* w = head < n_q ? q_w : k_w;
    const float inv = 1.0f / sqrtf(wave_sum(x0 * x0 + x1 * x1) / (float)kHeadDim + eps);
    const float n0 = (x0 * inv) * w[l], n1 = (x1 * inv) * w[l + 64];
    const float* c = cos_t + (size_t)pos * kHeadDim;
    const float* s = sin_t + (size_t)pos * kHeadDim;
    const float r0 = n0 * c[l] + (-n1) * s[l];
    const float r1 = n1 * c[l + 64] + n0 * s[l + 64];
    if (head < n_q) {
        src[l] = r0;
        src[l + 64] = r1;
    } else {
        __half* dst = k_cache + ((size_t)(head - n_q) * max_seq + pos) * kHeadDim;
        dst[l] = __float2half_rn(r0);
        dst[l + 64] = __float2half_rn(r1);
    }
}

// ---- attention ------------------------------------------------------------------------------
// Sixteen lanes share a cache row (lane sub = lane % 16 owns dimensions 8*sub..8*sub+7, one
// 16-byte load), so a wave-wide load covers four consecutive rows = 1 KiB contiguous; a wave
// takes rows 4*wave + lane/16, + 4*waves, ... with four loads in flight.

// Rows of the key / value cache a lane of the one-token kernels requests ahead (rows 64 apart: 4 = the
// first 256 of a head; 8 measured equal or slower).
constexpr int kRowsAhead = 4;

// Workgroup barrier that orders LDS traffic only: every LDS access this wave has issued is done, global
// loads stay in flight (__syncthreads() would wait for them too: one counter covers loads and stores).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt = 0; vector-memory and export counters left alone
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// The first R of a lane's rows (key0, key0 + 4*kWaves, ...), requested ahead of their use; rows past
// the end repeat the last one (n_rows = 0: row 0, which is inside the cache and never used).
template <int kWaves, int R>
__device__ __forceinline__ void load_first_rows(const uint4* __restrict__ R4, int n_rows, int key0, uint4 (&u)[R]) {
    const int last = max(n_rows - 1, 0);
#pragma unroll
    for (int i = 0; i < R; i++) u[i] = R4[(size_t)min(key0 + i * 4 * kWaves, last) * 16];
}

// One batch of R rows: scores[key] = scale * <q, row>, running maximum over the rows below n_rows.
template <int kWaves, int R>
__device__ __forceinline__ void score_batch(const uint4 (&u)[R], int key0, int n_rows, const float (&qv)[8], float scale,
                                            float* scores, int sub, float& local_max) {
#pragma unroll
    for (int i = 0; i < R; i++) {
        const int key = key0 + i * 4 * kWaves;
        const __half2* h2 = reinterpret_cast<const __half2*>(&u[i]);
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float2 f = __half22float2(h2[e]);
            dot = fmaf(qv[2 * e], f.x, dot);
            dot = fmaf(qv[2 * e + 1], f.y, dot);
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
        dot *= scale;
        if (key < n_rows) {
            if (sub == 0) scores[key] = dot;
            local_max = fmaxf(local_max, dot);
        }
    }
}

// scores[r] = scale * <q, K[r]> for r < n_rows; returns the maximum over the rows this lane saw.
template <int kWaves>
__device__ __forceinline__ float score_rows(const uint4* __restrict__ K4, int n_rows, const float (&qv)[8], float scale,
                                            float* scores, int wave, int grp, int sub) {
    constexpr int kRowsPerPass = 4 * kWaves;
    float local_max = -3.402823466e38f;
    for (int key0 = 4 * wave + grp; key0 < n_rows; key0 += 4 * kRowsPerPass) {
        uint4 u[4];
#pragma unroll
        for (int i = 0; i < 4; i++) u[i] = K4[(size_t)min(key0 + i * kRowsPerPass, n_rows - 1) * 16];
        score_batch<kWaves, 4>(u, key0, n_rows, qv, scale, scores, sub, local_max);
    }
    return local_max;
}

// One batch of R rows: acc[e] += p[key] * row[8*sub + e].
template <int kWaves, int R>
__device__ __forceinline__ void weigh_batch(const uint4 (&u)[R], int key0, int n_rows, const float* p, float (&acc)[8]) {
#pragma unroll
    for (int i = 0; i < R; i++) {
        const int key = key0 + i * 4 * kWaves;
        const float w = key < n_rows ? p[key] : 0.f;
        const __half2* h2 = reinterpret_cast<const __half2*>(&u[i]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float2 f = __half22float2(h2[e]);
            acc[2 * e] = fmaf(w, f.x, acc[2 * e]);
            acc[2 * e + 1] = fmaf(w, f.y, acc[2 * e + 1]);
        }
    }
}

// acc[e] += sum over this lane's rows of p[r] * V[r][8*sub + e]
template <int kWaves>
__device__ __forceinline__ void weigh_rows(const uint4* __restrict__ V4, int n_rows, const float* p, float (&acc)[8], int wave,
                                           int grp) {
    constexpr int kRowsPerPass = 4 * kWaves;
    for (int key0 = 4 * wave + grp; key0 < n_rows; key0 += 4 * kRowsPerPass) {
        uint4 u[4];
#pragma unroll
        for (int i = 0; i < 4; i++) u[i] = V4[(size_t)min(key0 + i * kRowsPerPass, n_rows - 1) * 16];
        weigh_batch<kWaves, 4>(u, key0, n_rows, p, acc);
    }
}

// Sum acc over the four row groups of the wave, park the wave's row in part[wave][128].
__device__ __forceinline__ void park_wave_row(float (&acc)[8], float* part, int wave, int grp, int sub) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        acc[e] += __shfl_xor(acc[e], 16, 64);
        acc[e] += __shfl_xor(acc[e], 32, 64);
    }
    if (grp == 0) {
        float4* dst = reinterpret_cast<float4*>(part + wave * kHeadDim + 8 * sub);
        dst[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        dst[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
}

// One workgroup of THREADS threads per (query head, token).  Keys 0..pos (pos = tokens before
// this call + token index) of the head's KV group, all already in the cache.  Scores live in
// LDS (max_seq floats); partial rows of the waves are summed through LDS in wave order.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void attention_kernel(const float* __restrict__ q, int q_row_stride,
                                                          const __half* __restrict__ k_cache, const __half* __restrict__ v_cache,
                                                          const int* __restrict__ pos_dev, float* __restrict__ out, int out_row_stride,
                                                          int n_q, int n_kv, int max_seq, float scale) {
    constexpr int kWaves = THREADS / 64;
    extern __shared__ float sm[];  // [0, kWaves*128): PV partials; then max_seq scores
    __shared__ float red[kWaves];
    float* part = sm;
    float* scores = sm + kWaves * kHeadDim;
    const int head = blockIdx.x, m = blockIdx.y, t = threadIdx.x;
    const int wave = t >> 6, lane = t & 63, sub = lane & 15, grp = lane >> 4;
    const int n_keys = min(pos_dev[0] + m, max_seq - 1) + 1;
    const int kvh = head / (n_q / n_kv);
    const uint4* K4 = reinterpret_cast<const uint4*>(k_cache + (size_t)kvh * max_seq * kHeadDim) + sub;  // row r: K4[16 r]
    const uint4* V4 = reinterpret_cast<const uint4*>(v_cache + (size_t)kvh * max_seq * kHeadDim) + sub;
    float qv[8];
    {
        const float4* q4 = reinterpret_cast<const float4*>(q + (size_t)m * q_row_stride + (size_t)head * kHeadDim + 8 * sub);
        const float4 a = q4[0], b = q4[1];
        qv[0] = a.x; qv[1] = a.y; qv[2] = a.z; qv[3] = a.w;
        qv[4] = b.x; qv[5] = b.y; qv[6] = b.z; qv[7] = b.w;
    }
    float local_max = wave_max(score_rows<kWaves>(K4, n_keys, qv, scale, scores, wave, grp, sub));
    if (lane == 0) red[wave] = local_max;
    __syncthreads();  // also publishes the scores
    float mx = red[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) mx = fmaxf(mx, red[w]);
    __syncthreads();
    float local_sum = 0.f;
    for (int key = t; key < n_keys; key += THREADS) {
        const float e = expf(scores[key] - mx);
        scores[key] = e;
        local_sum += e;
    }
    local_sum = wave_sum(local_sum);
    if (lane == 0) red[wave] = local_sum;
    __syncthreads();  // also publishes the exponentials
    float denom = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) denom += red[w];

    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
    weigh_rows<kWaves>(V4, n_keys, scores, acc, wave, grp);
    park_wave_row(acc, part, wave, grp, sub);
    __syncthreads();
    if (t < kHeadDim) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) s += part[w * kHeadDim + t];
        out[(size_t)m * out_row_stride + (size_t)head * kHeadDim + t] = s / denom;
    }
}

// ---- one-token attention, wave-local: every group of 16 lanes keeps a running (maximum, sum of
// exponentials, weighted values) over its own cache rows, so that no score ever goes through LDS and the
// waves meet once, at the end.  exp is v_exp_f32 on x * log2(e) (relative error about |x| * 2^-24), as
// in the matrix-core kernel.
struct RunningSoftmax {
    float m, l;      // the same in the 16 lanes of a group
    float acc[8];    // this lane's 8 head dimensions
};

__device__ __forceinline__ float exp_fast(float x) { return __expf(x); }

// One batch of R rows this group holds keys and values of (rows key0, key0 + 4*kWaves, ...; rows at or
// past n_rows do not count).
template <int kWaves, int R>
__device__ __forceinline__ void attend_batch(RunningSoftmax& st, const uint4 (&kq)[R], const uint4 (&vq)[R], int key0, int n_rows,
                                             const float (&qv)[8], float scale) {
    float sc[R];
    float bm = -3.402823466e38f;
#pragma unroll
    for (int i = 0; i < R; i++) {
        const __half2* h2 = reinterpret_cast<const __half2*>(&kq[i]);
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float2 f = __half22float2(h2[e]);
            dot = fmaf(qv[2 * e], f.x, dot);
            dot = fmaf(qv[2 * e + 1], f.y, dot);
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
        sc[i] = dot * scale;
        if (key0 + i * 4 * kWaves < n_rows) bm = fmaxf(bm, sc[i]);
    }
    const float m_new = fmaxf(st.m, bm);
    const float corr = exp_fast(st.m - m_new);  // 0 when nothing came before (m = -3.4e38), 1 when the batch is empty
    st.l *= corr;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] *= corr;
#pragma unroll
    for (int i = 0; i < R; i++) {
        const float p = key0 + i * 4 * kWaves < n_rows ? exp_fast(sc[i] - m_new) : 0.f;
        st.l += p;
        const __half2* h2 = reinterpret_cast<const __half2*>(&vq[i]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float2 f = __half22float2(h2[e]);
            st.acc[2 * e] = fmaf(p, f.x, st.acc[2 * e]);
            st.acc[2 * e + 1] = fmaf(p, f.y, st.acc[2 * e + 1]);
        }
    }
    st.m = m_new;
}

// All cached rows of this group: the first R come in k_first / v_first (requested ahead), the rest in
// batches of 4.
template <int kWaves, int R>
__device__ __forceinline__ void attend_rows(RunningSoftmax& st, const uint4* __restrict__ K4, const uint4* __restrict__ V4,
                                            int n_rows, const float (&qv)[8], float scale, int wave, int grp,
                                            const uint4 (&k_first)[R], const uint4 (&v_first)[R]) {
    constexpr int kRowsPerPass = 4 * kWaves;
    int key0 = 4 * wave + grp;
    if (key0 < n_rows) attend_batch<kWaves, R>(st, k_first, v_first, key0, n_rows, qv, scale);
    for (key0 += R * kRowsPerPass; key0 < n_rows; key0 += 4 * kRowsPerPass) {
        uint4 kq[4], vq[4];
#pragma unroll
        for (int i = 0; i < 4; i++) kq[i] = K4[(size_t)min(key0 + i * kRowsPerPass, n_rows - 1) * 16];
#pragma unroll
        for (int i = 0; i < 4; i++) vq[i] = V4[(size_t)min(key0 + i * kRowsPerPass, n_rows - 1) * 16];
        attend_batch<kWaves, 4>(st, kq, vq, key0, n_rows, qv, scale);
    }
}

// The new token itself (key and value in LDS, fp16-rounded): one more row for the group that calls this.
__device__ __forceinline__ void attend_new_token(RunningSoftmax& st, const float* k_new, const float* v_new, const float (&qv)[8],
                                                 float scale, int sub) {
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) dot = fmaf(qv[e], k_new[8 * sub + e], dot);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
    dot *= scale;
    const float m_new = fmaxf(st.m, dot);
    const float corr = exp_fast(st.m - m_new), p = exp_fast(dot - m_new);
    st.l = st.l * corr + p;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = fmaf(p, v_new[8 * sub + e], st.acc[e] * corr);
    st.m = m_new;
}

// Fold the four groups of a wave (lanes 16 and 32 apart), park the wave's (maximum, sum, 128 values) in
// LDS: wm[wave], wl[wave], part[wave][128].
__device__ __forceinline__ void park_wave_state(RunningSoftmax& st, float* part, float* wm, float* wl, int wave, int lane,
                                                int grp, int sub) {
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
        const float m_o = __shfl_xor(st.m, off, 64), l_o = __shfl_xor(st.l, off, 64);
        const float m_new = fmaxf(st.m, m_o);
        const float a = exp_fast(st.m - m_new), b = exp_fast(m_o - m_new);
        st.l = st.l * a + l_o * b;
#pragma unroll
        for (int e = 0; e < 8; e++) st.acc[e] = st.acc[e] * a + __shfl_xor(st.acc[e], off, 64) * b;
        st.m = m_new;
    }
    if (grp == 0) {
        float4* dst = reinterpret_cast<float4*>(part + wave * kHeadDim + 8 * sub);
        dst[0] = make_float4(st.acc[0], st.acc[1], st.acc[2], st.acc[3]);
        dst[1] = make_float4(st.acc[4], st.acc[5], st.acc[6], st.acc[7]);
    }
    if (lane == 0) {
        wm[wave] = st.m;
        wl[wave] = st.l;
    }
}

// Thread t < 128 folds the waves' parked states in wave order: maximum, sum and value t of the whole.
template <int kWaves>
__device__ __forceinline__ void fold_waves(const float* part, const float* wm, const float* wl, int t, float& m_all, float& l_all,
                                           float& o_all) {
    m_all = wm[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) m_all = fmaxf(m_all, wm[w]);
    l_all = 0.f, o_all = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
        const float f = exp_fast(wm[w] - m_all);
        l_all = fmaf(wl[w], f, l_all);
        o_all = fmaf(part[w * kHeadDim + t], f, o_all);
    }
}

// The same for one new token, with qk_norm_rope_cache folded in: wave 0 normalises and rotates
// the head's query, wave 1 the KV group's new key, wave 2 takes the new value; key and value are
// rounded to fp16 as the cache holds them, used from LDS as the last row of the context, and
// written to the cache by the first query head of the group only.  Rows 0..pos-1 come from the
// cache, so no workgroup reads what another one writes.
// CHAIN: the launch is a link of a chain of overlapping launches (chain.h): the norm weights, the rotation and
// the first cached rows are requested first, then the workgroup waits for the launch that writes qkv, reads the
// new token's row with agent-scope loads, and its outputs leave with agent-scope stores before it signals.
template <bool CHAIN>
__global__ __launch_bounds__(1024) void attention_one_token_kernel(const float* __restrict__ qkv, int n_q, int n_kv,
                                                                 const float* __restrict__ q_w, const float* __restrict__ k_w,
                                                                 const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                 const int* __restrict__ pos_dev, __half* __restrict__ k_cache,
                                                                 __half* __restrict__ v_cache, float* __restrict__ out,
                                                                 uint8_t* __restrict__ q_out, int max_seq, float eps,
                                                                 float scale, const ChainLink link) {
    constexpr int kWaves = 16;
    extern __shared__ float sm[];  // [0, kWaves*128): the waves' weighted values; 3*128: q, new key, new value
    __shared__ float wm[kWaves], wl[kWaves];
    float* part = sm;
    float* q_s = sm + kWaves * kHeadDim;
    float* k_new = q_s + kHeadDim;
    float* v_new = k_new + kHeadDim;
    const int head = blockIdx.x, t = threadIdx.x;
    const int wave = t >> 6, lane = t & 63, sub = lane & 15, grp = lane >> 4;
    const int pos = min(pos_dev[0], max_seq - 1);  // rows 0..pos-1 are cached, row pos is the new token
    const int group = n_q / n_kv, kvh = head / group;
    const bool writer = head == kvh * group;
    const uint4* K4 = reinterpret_cast<const uint4*>(k_cache + (size_t)kvh * max_seq * kHeadDim) + sub;
    const uint4* V4 = reinterpret_cast<const uint4*>(v_cache + (size_t)kvh * max_seq * kHeadDim) + sub;
    // The loads of the prepare step go first (the vector-memory counter retires in order), then every
    // lane requests its first cached key rows, whose round trip then overlaps the prepare step; the
    // barriers from here to the weighting step order LDS only, so requested rows stay in flight.
    float x0 = 0.f, x1 = 0.f, w0 = 0.f, w1 = 0.f, c0 = 0.f, c1 = 0.f, s0 = 0.f, s1 = 0.f;
    const float* src = nullptr;
    if (wave < 3) {
        const int src_head = wave == 0 ? head : (wave == 1 ? n_q + kvh : n_q + n_kv + kvh);
        src = qkv + (size_t)src_head * kHeadDim;
        if (!CHAIN) {
            x0 = src[lane];
            x1 = src[lane + 64];
        }
        if (wave < 2) {
            const float* w = wave == 0 ? q_w : k_w;
            const float* c = cos_t + (size_t)pos * kHeadDim;
            const float* sn = sin_t + (size_t)pos * kHeadDim;
            w0 = w[lane], w1 = w[lane + 64];
            c0 = c[lane], c1 = c[lane + 64];
            s0 = sn[lane], s1 = sn[lane + 64];
        }
    }
    uint4 k_first[kRowsAhead], v_first[kRowsAhead];
    load_first_rows<kWaves, kRowsAhead>(K4, pos, 4 * wave + grp, k_first);
    load_first_rows<kWaves, kRowsAhead>(V4, pos, 4 * wave + grp, v_first);
    if (CHAIN) {
        __builtin_amdgcn_sched_barrier(0);
        chain_wait(link);
        if (wave < 3) {
            x0 = load_agent(src + lane);
            x1 = load_agent(src + lane + 64);
        }
    }
    if (wave == 2) {
        const __half h0 = __float2half_rn(x0), h1 = __float2half_rn(x1);
        v_new[lane] = __half2float(h0);
        v_new[lane + 64] = __half2float(h1);
        if (writer) {
            __half* dst = v_cache + ((size_t)kvh * max_seq + pos) * kHeadDim;
            dst[lane] = h0;
            dst[lane + 64] = h1;
        }
    } else if (wave < 2) {
        const float inv = 1.0f / sqrtf(wave_sum(x0 * x0 + x1 * x1) / (float)kHeadDim + eps);
        const float n0 = (x0 * inv) * w0, n1 = (x1 * inv) * w1;
        const float r0 = n0 * c0 + (-n1) * s0;
        const float r1 = n1 * c1 + n0 * s1;
        if (wave == 0) {
            q_s[lane] = r0;
            q_s[lane + 64] = r1;
        } else {
            const __half h0 = __float2half_rn(r0), h1 = __float2half_rn(r1);
            k_new[lane] = __half2float(h0);
            k_new[lane + 64] = __half2float(h1);
            if (writer) {
                __half* dst = k_cache + ((size_t)kvh * max_seq + pos) * kHeadDim;
                dst[lane] = h0;
                dst[lane + 64] = h1;
            }
        }
    }
    lds_barrier();
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; e++) qv[e] = q_s[8 * sub + e];
    RunningSoftmax st;
    st.m = -3.402823466e38f, st.l = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = 0.f;
    attend_rows<kWaves, kRowsAhead>(st, K4, V4, pos, qv, scale, wave, grp, k_first, v_first);
    if (wave == kWaves - 1 && grp == 3) attend_new_token(st, k_new, v_new, qv, scale, sub);
    park_wave_state(st, part, wm, wl, wave, lane, grp, sub);
    lds_barrier();
    if (t < kHeadDim) {
        float m_all, l_all, o_all;
        fold_waves<kWaves>(part, wm, wl, t, m_all, l_all, o_all);
        const float val = o_all / l_all;
        // the head's 128 outputs are four whole 32-blocks of the row: with q_out they go out as the
        // quantised blocks the next linear's quantiser would make of them
        if (q_out != nullptr)
            store_quantized_value_fp16<CHAIN>(q_out, head * kHeadDim + t, val);
        else if (CHAIN)
            store_agent(out + (size_t)head * kHeadDim + t, val);
        else
            out[(size_t)head * kHeadDim + t] = val;
    }
    if (CHAIN) chain_signal(link, gridDim.x);
}

// The same step for long contexts: S workgroups per query head, workgroup (head, s) takes the cached
// rows [s*chunk, (s+1)*chunk) and the last one also the new token.  Each leaves its maximum, its sum of
// exponentials and its unnormalised weighted values in `partials` ([head][s][132]: maximum, sum, 2 pad,
// 128 values); the last workgroup of a head to arrive (counter in `arrivals`, left at zero again) merges
// the S shares in order s = 0..S-1, so the result does not depend on who is last.  Partials and counters
// are accessed with agent-scope relaxed atomics only (coherent across the XCDs' L2s on their own) and
// ordered by waiting for the stores and by the workgroup barriers.
constexpr int kSplitStride = 132;
template <bool CHAIN>
__global__ __launch_bounds__(1024) void attention_one_token_split_kernel(
    const float* __restrict__ qkv, int n_q, int n_kv, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ pos_dev,
    __half* __restrict__ k_cache, __half* __restrict__ v_cache, float* __restrict__ out, uint8_t* __restrict__ q_out,
    float* __restrict__ partials, unsigned* __restrict__ arrivals, int max_seq, float eps, float scale, const ChainLink link) {
    constexpr int kWaves = 16;
    extern __shared__ float sm[];  // [0, kWaves*128): the waves' weighted values; 3*128: q, new key, new value
    __shared__ float wm[kWaves], wl[kWaves];
    __shared__ unsigned s_arrived;
    float* part = sm;
    float* q_s = sm + kWaves * kHeadDim;
    float* k_new = q_s + kHeadDim;
    float* v_new = k_new + kHeadDim;
    const int head = blockIdx.x, split = blockIdx.y, S = gridDim.y, t = threadIdx.x;
    const int wave = t >> 6, lane = t & 63, sub = lane & 15, grp = lane >> 4;
    const int pos = min(pos_dev[0], max_seq - 1);  // rows 0..pos-1 are cached, row pos is the new token
    const int chunk = (pos + S - 1) / S;
    const int k0 = min(split * chunk, pos), n = min(k0 + chunk, pos) - k0;  // this share: cached rows k0 .. k0+n-1
    const bool own = split == S - 1;                                        // ... and the new token
    const int group = n_q / n_kv, kvh = head / group;
    const bool writer = own && head == kvh * group;
    const uint4* K4 = reinterpret_cast<const uint4*>(k_cache + ((size_t)kvh * max_seq + k0) * kHeadDim) + sub;
    const uint4* V4 = reinterpret_cast<const uint4*>(v_cache + ((size_t)kvh * max_seq + k0) * kHeadDim) + sub;
    // as in the one-workgroup kernel: prepare loads, then the first key rows, LDS-only barriers up to the weighting
    const bool prepares = wave == 0 || (own && wave < 3);
    float x0 = 0.f, x1 = 0.f, w0 = 0.f, w1 = 0.f, c0 = 0.f, c1 = 0.f, s0 = 0.f, s1 = 0.f;
    const float* src = nullptr;
    if (prepares) {
        const int src_head = wave == 0 ? head : (wave == 1 ? n_q + kvh : n_q + n_kv + kvh);
        src = qkv + (size_t)src_head * kHeadDim;
        if (!CHAIN) {
            x0 = src[lane];
            x1 = src[lane + 64];
        }
        if (wave < 2) {
            const float* w = wave == 0 ? q_w : k_w;
            const float* c = cos_t + (size_t)pos * kHeadDim;
            const float* sn = sin_t + (size_t)pos * kHeadDim;
            w0 = w[lane], w1 = w[lane + 64];
            c0 = c[lane], c1 = c[lane + 64];
            s0 = sn[lane], s1 = sn[lane + 64];
        }
    }
    uint4 k_first[kRowsAhead], v_first[kRowsAhead];
    load_first_rows<kWaves, kRowsAhead>(K4, n, 4 * wave + grp, k_first);
    load_first_rows<kWaves, kRowsAhead>(V4, n, 4 * wave + grp, v_first);
    if (CHAIN) {
        __builtin_amdgcn_sched_barrier(0);
        chain_wait(link);
        if (prepares) {
            x0 = load_agent(src + lane);
            x1 = load_agent(src + lane + 64);
        }
    }
    if (prepares && wave == 2) {
        const __half h0 = __float2half_rn(x0), h1 = __float2half_rn(x1);
        v_new[lane] = __half2float(h0);
        v_new[lane + 64] = __half2float(h1);
        if (writer) {
            __half* dst = v_cache + ((size_t)kvh * max_seq + pos) * kHeadDim;
            dst[lane] = h0;
            dst[lane + 64] = h1;
        }
    } else if (prepares) {
        const float inv = 1.0f / sqrtf(wave_sum(x0 * x0 + x1 * x1) / (float)kHeadDim + eps);
        const float n0 = (x0 * inv) * w0, n1 = (x1 * inv) * w1;
        const float r0 = n0 * c0 + (-n1) * s0;
        const float r1 = n1 * c1 + n0 * s1;
        if (wave == 0) {
            q_s[lane] = r0;
            q_s[lane + 64] = r1;
        } else {
            const __half h0 = __float2half_rn(r0), h1 = __float2half_rn(r1);
            k_new[lane] = __half2float(h0);
            k_new[lane + 64] = __half2float(h1);
            if (writer) {
                __half* dst = k_cache + ((size_t)kvh * max_seq + pos) * kHeadDim;
                dst[lane] = h0;
                dst[lane + 64] = h1;
            }
        }
    }
    lds_barrier();
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; e++) qv[e] = q_s[8 * sub + e];
    RunningSoftmax st;
    st.m = -3.402823466e38f, st.l = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = 0.f;
    attend_rows<kWaves, kRowsAhead>(st, K4, V4, n, qv, scale, wave, grp, k_first, v_first);
    if (own && wave == kWaves - 1 && grp == 3) attend_new_token(st, k_new, v_new, qv, scale, sub);
    park_wave_state(st, part, wm, wl, wave, lane, grp, sub);
    lds_barrier();
    float* mine = partials + ((size_t)head * S + split) * kSplitStride;
    if (t < kHeadDim) {  // an empty share: maximum -3.4e38, sum 0 -- its weight in the merge is exp(-huge) = 0
        float m_all, l_all, o_all;
        fold_waves<kWaves>(part, wm, wl, t, m_all, l_all, o_all);
        __hip_atomic_store(mine + 4 + t, o_all, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t == 0) {
            __hip_atomic_store(mine, m_all, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(mine + 1, l_all, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
    __syncthreads();
    if (t == 0) s_arrived = atomicAdd(&arrivals[head], 1u);
    __syncthreads();
    if (s_arrived != (unsigned)(S - 1)) {
        if (CHAIN) chain_signal(link, gridDim.x * gridDim.y);
        return;
    }
    if (t < kHeadDim) {
        const float* base = partials + (size_t)head * S * kSplitStride;
        float m_all = -3.402823466e38f;
        for (int j = 0; j < S; j++)
            m_all = fmaxf(m_all, __hip_atomic_load(base + j * kSplitStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        float l_all = 0.f, o_all = 0.f;
        for (int j = 0; j < S; j++) {
            const float f = exp_fast(__hip_atomic_load(base + j * kSplitStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - m_all);
            l_all = fmaf(__hip_atomic_load(base + j * kSplitStride + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), f, l_all);
            o_all = fmaf(__hip_atomic_load(base + j * kSplitStride + 4 + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), f, o_all);
        }
        const float val = o_all / l_all;
        if (q_out != nullptr)
            store_quantized_value_fp16<CHAIN>(q_out, head * kHeadDim + t, val);
        else if (CHAIN)
            store_agent(out + (size_t)head * kHeadDim + t, val);
        else
            out[(size_t)head * kHeadDim + t] = val;
    }
    if (t == 0) __hip_atomic_store(&arrivals[head], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    if (CHAIN) chain_signal(link, gridDim.x * gridDim.y);
}

// out[m][j] = silu(gate_up[m][j]) * gate_up[m][inter + j]
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate_up, float* __restrict__ out, int inter,
                                                     long long total) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long long m = i / inter;
    const int j = (int)(i - m * inter);
    const float g = gate_up[m * 2 * inter + j], u = gate_up[m * 2 * inter + inter + j];
    out[i] = (g * (1.0f / (1.0f + expf(-g)))) * u;
}

// The same product, four per thread, written as the 80 B blocks of the [M][inter] result.
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(const float4* __restrict__ gate_up, uint8_t* __restrict__ q_out,
                                                           int inter4, long long total4) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total4) return;  // total4 is a multiple of 16: whole groups of 8 lanes leave together
    const long long m = i / inter4;
    const int j = (int)(i - m * inter4);
    const float4 g = gate_up[m * 2 * inter4 + j], u = gate_up[m * 2 * inter4 + inter4 + j];
    float4 v;
    v.x = (g.x * (1.0f / (1.0f + expf(-g.x)))) * u.x;
    v.y = (g.y * (1.0f / (1.0f + expf(-g.y)))) * u.y;
    v.z = (g.z * (1.0f / (1.0f + expf(-g.z)))) * u.z;
    v.w = (g.w * (1.0f / (1.0f + expf(-g.w)))) * u.w;
    store_quantized_float4(q_out, i, v);
}

// First index of the maximum of logits[0..n); written to next_id[0] and to history[*step], then
// the step counter and the position advance (the token just consumed is now in the cache).
__global__ __launch_bounds__(1024) void argmax_token_kernel(const float* __restrict__ logits, int n, int* __restrict__ next_id,
                                                          int* __restrict__ history, int history_len, int* __restrict__ step_dev) {
    __shared__ float best_v[1024];
    __shared__ int best_i[1024];
    const int t = threadIdx.x;
    float bv = -3.402823466e38f;
    int bi = 0x7fffffff;
    // n is a multiple of 8 and logits 16-byte aligned: scan float4s, four in flight
    const float4* l4 = reinterpret_cast<const float4*>(logits);
    const int n4 = n >> 2;
    for (int j0 = t; j0 < n4; j0 += 4 * 1024) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = j0 + u * 1024;
            v[u] = j < n4 ? l4[j] : make_float4(-3.402823466e38f, -3.402823466e38f, -3.402823466e38f, -3.402823466e38f);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = 4 * (j0 + u * 1024);  // indices rise within a thread, so '>' keeps the first maximum
            const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (e[k] > bv) {
                    bv = e[k];
                    bi = i + k;
                }
        }
    }
    best_v[t] = bv;
    best_i[t] = bi;
    __syncthreads();
    for (int s = 512; s > 0; s >>= 1) {
        if (t < s) {
            const float ov = best_v[t + s];
            const int oi = best_i[t + s];
            if (ov > best_v[t] || (ov == best_v[t] && oi < best_i[t])) {
                best_v[t] = ov;
                best_i[t] = oi;
            }
        }
        __syncthreads();
    }
    if (t == 0) {
        const int id = best_i[0] == 0x7fffffff ? 0 : best_i[0];
        next_id[0] = id;
        const int st = step_dev[0];
        if (st >= 0 && st < history_len) history[st] = id;
        step_dev[0] = st + 1;
    }
}

__global__ void advance_kernel(int* __restrict__ pos_dev, int by) {
    if (threadIdx.x == 0 && blockIdx.x == 0) pos_dev[0] += by;
}

}  // namespace

hipError_t launch_embed_rows(const int* ids, const void* table_fp16, float* out, int M, int hidden, int vocab, hipStream_t s) {
    hipLaunchKernelGGL(embed_rows_kernel, dim3(M), dim3(256), 0, s, ids, static_cast<const __half*>(table_fp16), out, hidden, vocab);
    return hipGetLastError();
}

hipError_t launch_add_rmsnorm(const float* x, const float* res_in, const float* w, float* res_out, float* norm_out, int M,
                              int hidden, float eps, hipStream_t s) {
    // few rows: one wide workgroup per row, the row's latency is all there is to hide
    if (M <= 16)
        hipLaunchKernelGGL((add_rmsnorm_kernel<1024, false>), dim3(M), dim3(1024), 0, s, x, res_in, w, res_out, norm_out, nullptr,
                           hidden, eps);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<256, false>), dim3(M), dim3(256), 0, s, x, res_in, w, res_out, norm_out, nullptr,
                           hidden, eps);
    return hipGetLastError();
}

hipError_t launch_add_rmsnorm_quant(const float* x, const float* res_in, const float* w, float* res_out, void* q_out, int M,
                                    int hidden, float eps, hipStream_t s) {
    uint8_t* q = static_cast<uint8_t*>(q_out);
    if (M <= 16)
        hipLaunchKernelGGL((add_rmsnorm_kernel<1024, true>), dim3(M), dim3(1024), 0, s, x, res_in, w, res_out, nullptr, q, hidden, eps);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<256, true>), dim3(M), dim3(256), 0, s, x, res_in, w, res_out, nullptr, q, hidden, eps);
    return hipGetLastError();
}

hipError_t launch_qk_norm_rope_cache(float* qkv, int row_stride, int M, int n_q, int n_kv, const float* q_w, const float* k_w,
                                     const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache, void* v_cache,
                                     int max_seq, float eps, hipStream_t s) {
    hipLaunchKernelGGL(qk_norm_rope_cache_kernel, dim3(M, n_q + 2 * n_kv), dim3(64), 0, s, qkv, row_stride, n_q, n_kv, q_w, k_w,
                       cos_t, sin_t, pos_dev, static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), max_seq, eps);
    return hipGetLastError();
}

size_t attention_lds_bytes(int max_seq, int threads) {
    return (size_t)((threads / 64) * kHeadDim + max_seq) * sizeof(float);
}

hipError_t launch_attention(const float* q, int q_row_stride, const void* k_cache, const void* v_cache, const int* pos_dev,
                            float* out, int out_row_stride, int M, int n_q, int n_kv, int max_seq, float scale, hipStream_t s,
                            int variant) {
    static const bool vector_only = tuning_env("A81W41_ATTENTION_VECTOR") != nullptr;  // measurement aid (tuning builds)
    if (variant == 0 && !vector_only && attention_prefill_fits(M, n_q, n_kv))
        return launch_attention_prefill(q, q_row_stride, k_cache, v_cache, pos_dev, out, out_row_stride, M, n_q, n_kv, max_seq,
                                        scale, s);
    // few tokens: the context of one head is all the parallelism there is, so use wide workgroups
    if (M <= 8) {
        hipLaunchKernelGGL(attention_kernel<1024>, dim3(n_q, M), dim3(1024), attention_lds_bytes(max_seq, 1024), s, q,
                           q_row_stride, static_cast<const __half*>(k_cache), static_cast<const __half*>(v_cache), pos_dev,
                           out, out_row_stride, n_q, n_kv, max_seq, scale);
    } else {
        hipLaunchKernelGGL(attention_kernel<256>, dim3(n_q, M), dim3(256), attention_lds_bytes(max_seq, 256), s, q,
                           q_row_stride, static_cast<const __half*>(k_cache), static_cast<const __half*>(v_cache), pos_dev,
                           out, out_row_stride, n_q, n_kv, max_seq, scale);
    }
    return hipGetLastError();
}

hipError_t launch_attention_one_token(const float* qkv, int n_q, int n_kv, const float* q_w, const float* k_w,
                                      const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache, void* v_cache,
                                      float* out, void* q_out, int max_seq, float eps, float scale, hipStream_t s,
                                      const ChainLink* link) {
    const size_t lds = (size_t)(16 * kHeadDim + 3 * kHeadDim) * sizeof(float);
    if (link)
        hipLaunchKernelGGL(attention_one_token_kernel<true>, dim3(n_q), dim3(1024), lds, s, qkv, n_q, n_kv, q_w, k_w, cos_t, sin_t,
                           pos_dev, static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), out,
                           static_cast<uint8_t*>(q_out), max_seq, eps, scale, *link);
    else
        hipLaunchKernelGGL(attention_one_token_kernel<false>, dim3(n_q), dim3(1024), lds, s, qkv, n_q, n_kv, q_w, k_w, cos_t, sin_t,
                           pos_dev, static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), out,
                           static_cast<uint8_t*>(q_out), max_seq, eps, scale, ChainLink{});
    return hipGetLastError();
}

hipError_t launch_attention_one_token_split(const float* qkv, int n_q, int n_kv, const float* q_w, const float* k_w,
                                            const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache,
                                            void* v_cache, float* out, void* q_out, float* partials, unsigned* arrivals,
                                            int splits, int max_seq, float eps, float scale, hipStream_t s,
                                            const ChainLink* link) {
    const size_t lds = (size_t)(16 * kHeadDim + 3 * kHeadDim) * sizeof(float);
    if (link)
        hipLaunchKernelGGL(attention_one_token_split_kernel<true>, dim3(n_q, splits), dim3(1024), lds, s, qkv, n_q, n_kv, q_w, k_w,
                           cos_t, sin_t, pos_dev, static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), out,
                           static_cast<uint8_t*>(q_out), partials, arrivals, max_seq, eps, scale, *link);
    else
        hipLaunchKernelGGL(attention_one_token_split_kernel<false>, dim3(n_q, splits), dim3(1024), lds, s, qkv, n_q, n_kv, q_w, k_w,
                           cos_t, sin_t, pos_dev, static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), out,
                           static_cast<uint8_t*>(q_out), partials, arrivals, max_seq, eps, scale, ChainLink{});
    return hipGetLastError();
}

hipError_t launch_silu_mul(const float* gate_up, float* out, int M, int inter, hipStream_t s) {
    const long long total = (long long)M * inter;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gate_up, out, inter, total);
    return hipGetLastError();
}

hipError_t launch_silu_mul_quant(const float* gate_up, void* q_out, int M, int inter, hipStream_t s) {
    const long long total4 = (long long)M * (inter / 4);
    hipLaunchKernelGGL(silu_mul_quant_kernel, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, s,
                       reinterpret_cast<const float4*>(gate_up), static_cast<uint8_t*>(q_out), inter / 4, total4);
    return hipGetLastError();
}

hipError_t launch_argmax_token(const float* logits, int n, int* next_id, int* history, int history_len, int* step_dev,
                               hipStream_t s) {
    hipLaunchKernelGGL(argmax_token_kernel, dim3(1), dim3(1024), 0, s, logits, n, next_id, history, history_len, step_dev);
    return hipGetLastError();
}

hipError_t launch_advance(int* pos_dev, int by, hipStream_t s) {
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, s, pos_dev, by);
    return hipGetLastError();
}

}  // namespace a81w41
