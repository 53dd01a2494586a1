// Causal GQA attention for many new tokens at once (the prompt pass) on the matrix cores:
// QK^T * scale, causal mask, softmax, PV (QwenAttention.cc:150-195) over the fp16 KV cache.
//
// One workgroup per (tile of 32 query tokens, KV head) with G x S waves: the G query heads of the
// KV group share every staged key / value tile, and the key tiles of a head are dealt round-robin
// to S waves, which shortens the serial walk over the context S times.  Each wave keeps the
// running-maximum ("online") softmax of its share in fp32; the S shares are merged at the end.
//
// Both products are computed transposed, so that a lane owns one query token:
//   S^T = K Q^T      A = key tile (row = key, k = head dim), B = Q^T (column = query)
//   O^T = V^T P^T    A = V^T (row = head dim, k = key),     B = P^T (column = query)
// with v_mfma_f32_32x32x16_f16, whose result registers of lane (query q, half kh) hold rows
// 8g + 4kh + i (g, i = 0..3).  A row's maximum and sum are therefore in-lane reductions over 16
// registers plus one exchange with lane q of the other half, and the rescaling factor of the
// running output is a per-lane scalar.  The same registers feed the second product directly:
// its contraction index may run over the keys in any order as long as V^T uses the same one,
// so the value tile is staged transposed in LDS in exactly the order the P registers have.
//
// The cache holds fp16, which the matrix cores take as it is.  The fp32 queries and
// probabilities are split into two fp16 terms (x = hi + lo, |lo| <= 2^-11 |hi|) and multiplied
// in two instructions, which keeps about 22 significant bits: the result matches the fp32
// vector kernels of the short-prompt path to rounding noise.
//
// Output: fp32 rows, or (q_out) the rows' 80 B quantised blocks for the linear that follows
// (quantize_row_q8_1_repack_fp32, quantized_gemx_kernels.cc:803-911).  A lane holds 16 of the 32
// values of each of its row's four 32-blocks per head and the lane of the other half the other 16,
// so the block maximum and sum are in-lane reductions plus one exchange; the bits equal those of
// quantising the fp32 rows.
#include "a81w41_kernels.h"

#include <cstdlib>
#include "quantize_common.h"

#include <hip/hip_fp16.h>

namespace a81w41 {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kHeadDim = 128;
constexpr int kTile = 32;         // query tokens per workgroup, keys per step
constexpr int kKStride = 272;     // bytes per key row of the staged key tile (256 + 16: conflict-free 16-byte reads)
// Bytes per head-dim row of the transposed value tile (32 keys * 2 + 8).  18 words: the rows 8 apart that
// the lanes of a wave write together fall into alternating halves of the 32 banks, and the 8-byte operand
// reads of 32 consecutive rows cover every bank once.
constexpr int kVStride = 72;
constexpr int kTileLdsBytes = kTile * kKStride + kHeadDim * kVStride;  // one key tile + one transposed value tile
constexpr int kMergeSlotBytes = 64 * 64 * 4;                           // one wave's 128 x 32 fp32 output
constexpr float kLowest = -3.0e38f;

// Position of key `key` (0..31 inside the tile) along the contraction index of the second product:
// register v = 4g + i of half kh holds key 8g + 4kh + i; chunk c = g >> 1 takes registers 8c..8c+7.
__device__ __forceinline__ int value_slot(int key) {
    const int g = key >> 3, kh = (key >> 2) & 1, i = key & 3;
    return ((g >> 1) * 2 + kh) * 8 + 4 * (g & 1) + i;
}

__device__ __forceinline__ void split_fp16(const float (&x)[8], v8h& hi, v8h& lo) {
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const _Float16 h = (_Float16)x[t];
        hi[t] = h;
        lo[t] = (_Float16)(x[t] - (float)h);
    }
}

// exp for the softmax weights: v_exp_f32 on x * log2(e), relative error about |x| * 2^-24.
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

// G = query heads per KV head, S = key splits: wave (h, sp) = (wave % G, wave / G) owns query head
// kvh*G + h and every S-th key tile starting at sp.  A round stages S consecutive key / value
// tiles; at the end the S partial (maximum, sum, output) triples of a head are merged through LDS.
template <int G, int S>
__global__ __launch_bounds__(64 * G * S) void attention_prefill_kernel(const float* __restrict__ q, int q_row_stride,
                                                                      const __half* __restrict__ k_cache,
                                                                      const __half* __restrict__ v_cache,
                                                                      const int* __restrict__ pos_dev, float* __restrict__ out,
                                                                      int out_row_stride, uint8_t* __restrict__ q_out, int n_q,
                                                                      int M, int max_seq, float scale) {
    constexpr int kThreads = 64 * G * S;
    constexpr int kKPieces = S * kTile * 16;       // 16-byte pieces (key, 8 head dims) of the S staged key tiles
    constexpr int kKItems = kKPieces / kThreads;
    constexpr int kVPieces = S * (kTile / 2) * 16; // (pair of adjacent keys, 8 head dims) of the S value tiles
    constexpr int kVItems = (kVPieces + kThreads - 1) / kThreads;
    static_assert(kKItems * kThreads == kKPieces, "key tile pieces must divide over the workgroup");
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, kh = lane >> 5;
    const int h = wave % G, sp = wave / G;
    // gridDim.z workgroups share a KV head when its group of query heads is larger than G
    const int kvh = blockIdx.y, head = kvh * (n_q / (int)gridDim.y) + (int)blockIdx.z * G + h;
    const int m0 = blockIdx.x * kTile;
    const int pos0 = pos_dev[0];
    const int m_last = min(m0 + kTile, M) - 1;                  // last real token of the tile
    const int n_keys = min(pos0 + m_last, max_seq - 1) + 1;     // keys the tile's last token sees
    const int n_tiles = (n_keys + kTile - 1) / kTile;
    const int n_rounds = (n_tiles + S - 1) / S;
    const int m = m0 + r;                                       // this lane's query token
    const int last_key = min(pos0 + min(m, m_last), n_keys - 1);  // it sees keys 0..last_key
    const uint8_t* k_lds = lds + sp * kTileLdsBytes;            // this wave's tile of the round
    const uint8_t* v_lds = k_lds + kTile * kKStride;

    // this lane's query row as B operands: step d covers head dims 16d + 8kh .. + 7
    v8h q_hi[8], q_lo[8];
    {
        const float* row = q + (size_t)min(m, M - 1) * q_row_stride + (size_t)head * kHeadDim + 8 * kh;
#pragma unroll
        for (int d = 0; d < 8; d++) {
            const float4 a = *reinterpret_cast<const float4*>(row + 16 * d);
            const float4 b = *reinterpret_cast<const float4*>(row + 16 * d + 4);
            const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            split_fp16(x, q_hi[d], q_lo[d]);
        }
    }

    const __half* k_base = k_cache + (size_t)kvh * max_seq * kHeadDim;
    const __half* v_base = v_cache + (size_t)kvh * max_seq * kHeadDim;
    uint4 k_reg[kKItems], v_reg[kVItems][2];
    auto fetch = [&](int round) {  // rows past the context repeat the last one (they are masked)
        const int key0 = round * S * kTile;
#pragma unroll
        for (int it = 0; it < kKItems; it++) {
            const int piece = tid + it * kThreads, key = piece >> 4, sub = piece & 15;  // key: 0 .. 32 S - 1
            k_reg[it] = *reinterpret_cast<const uint4*>(k_base + (size_t)min(key0 + key, n_keys - 1) * kHeadDim + 8 * sub);
        }
#pragma unroll
        for (int it = 0; it < kVItems; it++) {
            const int piece = tid + it * kThreads;
            if (piece < kVPieces) {
                const int tl = piece >> 8, sub = (piece >> 4) & 15, pair = piece & 15;
#pragma unroll
                for (int j = 0; j < 2; j++)
                    v_reg[it][j] = *reinterpret_cast<const uint4*>(
                        v_base + (size_t)min(key0 + tl * kTile + 2 * pair + j, n_keys - 1) * kHeadDim + 8 * sub);
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int it = 0; it < kKItems; it++) {
            const int piece = tid + it * kThreads, tl = piece >> 9, key = (piece >> 4) & 31, sub = piece & 15;
            *reinterpret_cast<uint4*>(lds + tl * kTileLdsBytes + key * kKStride + 16 * sub) = k_reg[it];
        }
#pragma unroll
        for (int it = 0; it < kVItems; it++) {
            const int piece = tid + it * kThreads;
            if (piece < kVPieces) {  // keys 2 pair and 2 pair + 1 sit next to each other along the contraction index
                const int tl = piece >> 8, sub = (piece >> 4) & 15, pair = piece & 15;
                const uint32_t a[4] = {v_reg[it][0].x, v_reg[it][0].y, v_reg[it][0].z, v_reg[it][0].w};
                const uint32_t b[4] = {v_reg[it][1].x, v_reg[it][1].y, v_reg[it][1].z, v_reg[it][1].w};
                uint8_t* col = lds + tl * kTileLdsBytes + kTile * kKStride + (8 * sub) * kVStride + 2 * value_slot(2 * pair);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint32_t lo = (a[e >> 1] >> (16 * (e & 1))) & 0xffffu, hi = (b[e >> 1] >> (16 * (e & 1))) & 0xffffu;
                    *reinterpret_cast<uint32_t*>(col + e * kVStride) = lo | (hi << 16);
                }
            }
        }
    };

    v16f o_acc[4];
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int v = 0; v < 16; v++) o_acc[b][v] = 0.f;
    float m_run = kLowest, l_run = 0.f;

    fetch(0);
    for (int round = 0; round < n_rounds; round++) {  // uniform over the workgroup
        __syncthreads();  // every wave is done with the previous round's tiles
        stage();
        __syncthreads();
        if (round + 1 < n_rounds) fetch(round + 1);
        const int tile = round * S + sp;
        if (tile >= n_tiles) continue;  // uniform over the wave; the barriers are outside

        v16f s_acc;
#pragma unroll
        for (int v = 0; v < 16; v++) s_acc[v] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; d++) {
            const v8h a = *reinterpret_cast<const v8h*>(k_lds + r * kKStride + 32 * d + 16 * kh);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, q_hi[d], s_acc, 0, 0, 0);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, q_lo[d], s_acc, 0, 0, 0);
        }

        float sc[16];
        float t_max = kLowest;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int key = tile * kTile + 8 * (v >> 2) + 4 * kh + (v & 3);
            sc[v] = key <= last_key ? s_acc[v] * scale : kLowest;
            t_max = fmaxf(t_max, sc[v]);
        }
        t_max = fmaxf(t_max, __shfl_xor(t_max, 32, 64));
        const float m_new = fmaxf(m_run, t_max);
        // a token that sees none of this tile's keys and none before it (only possible in a wave
        // whose first tile is not tile 0) keeps m_new = kLowest: its weights must still be 0
        const float alpha = fast_exp(m_run - m_new);
        float p[16];
        float p_sum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            p[v] = sc[v] > kLowest ? fast_exp(sc[v] - m_new) : 0.f;
            p_sum += p[v];
        }
        p_sum += __shfl_xor(p_sum, 32, 64);
        l_run = l_run * alpha + p_sum;
        m_run = m_new;
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) o_acc[b][v] *= alpha;

        v8h p_hi[2], p_lo[2];
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const float x[8] = {p[8 * c], p[8 * c + 1], p[8 * c + 2], p[8 * c + 3],
                                p[8 * c + 4], p[8 * c + 5], p[8 * c + 6], p[8 * c + 7]};
            split_fp16(x, p_hi[c], p_lo[c]);
        }
#pragma unroll
        for (int b = 0; b < 4; b++) {
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const uint8_t* src = v_lds + (32 * b + r) * kVStride + (2 * c + kh) * 16;  // 8-byte aligned
                const uint2 a0 = *reinterpret_cast<const uint2*>(src), a1 = *reinterpret_cast<const uint2*>(src + 8);
                const uint4 a4 = make_uint4(a0.x, a0.y, a1.x, a1.y);
                const v8h a = __builtin_bit_cast(v8h, a4);
                o_acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, p_hi[c], o_acc[b], 0, 0, 0);
                o_acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, p_lo[c], o_acc[b], 0, 0, 0);
            }
        }
    }

    // ---- merge the S partial results of each head ------------------------------------------------
    // LDS now holds: the outputs being handed over (one 16 KiB slot per sending wave), then the
    // running maxima and sums of all waves.
    float* stat = reinterpret_cast<float*>(lds + kMergeSlotBytes * G * (S / 2 > 0 ? S / 2 : 1));
    __syncthreads();  // the staged tiles are dead
    if (kh == 0) {
        stat[(sp * G + h) * 32 + r] = m_run;
        stat[(S * G + sp * G + h) * 32 + r] = l_run;
    }
    __syncthreads();
    float m_fin = kLowest;
#pragma unroll
    for (int j = 0; j < S; j++) m_fin = fmaxf(m_fin, stat[(j * G + h) * 32 + r]);  // finite: tile 0 holds key 0
    float l_tot = 0.f;
#pragma unroll
    for (int j = 0; j < S; j++)
        l_tot += stat[(S * G + j * G + h) * 32 + r] * fast_exp(stat[(j * G + h) * 32 + r] - m_fin);
    const float f = fast_exp(m_run - m_fin);  // 0 for a wave that had no visible key
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int v = 0; v < 16; v++) o_acc[b][v] *= f;
#pragma unroll
    for (int stride = S / 2; stride >= 1; stride >>= 1) {  // sp in [stride, 2 stride) hands over to sp - stride
        float4* slot = reinterpret_cast<float4*>(lds + (size_t)((sp % stride) * G + h) * kMergeSlotBytes);
        if (sp >= stride && sp < 2 * stride) {
#pragma unroll
            for (int b = 0; b < 4; b++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    slot[(4 * b + g) * 64 + lane] =
                        make_float4(o_acc[b][4 * g], o_acc[b][4 * g + 1], o_acc[b][4 * g + 2], o_acc[b][4 * g + 3]);
        }
        __syncthreads();
        if (sp < stride) {
#pragma unroll
            for (int b = 0; b < 4; b++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 t = slot[(4 * b + g) * 64 + lane];
                    o_acc[b][4 * g] += t.x;
                    o_acc[b][4 * g + 1] += t.y;
                    o_acc[b][4 * g + 2] += t.z;
                    o_acc[b][4 * g + 3] += t.w;
                }
        }
        __syncthreads();
    }

    if (sp != 0) return;  // whole waves
    const float inv = 1.0f / l_tot;
    if (q_out == nullptr) {
        if (m <= m_last) {
            float* dst = out + (size_t)m * out_row_stride + (size_t)head * kHeadDim + 4 * kh;
#pragma unroll
            for (int b = 0; b < 4; b++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    *reinterpret_cast<float4*>(dst + 32 * b + 8 * g) =
                        make_float4(o_acc[b][4 * g] * inv, o_acc[b][4 * g + 1] * inv, o_acc[b][4 * g + 2] * inv,
                                    o_acc[b][4 * g + 3] * inv);
        }
        return;
    }
    // 32-block b of this head: values 8g + 4kh + i (g, i = 0..3) here, the rest in lane ^ 32.  All lanes
    // take part in the exchanges; rows past the last token store nothing.
#pragma unroll
    for (int b = 0; b < 4; b++) {
        float val[16];
        float amax = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            val[v] = o_acc[b][v] * inv;
            amax = fmaxf(amax, fabsf(val[v]));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const float d = amax / 127.f;                           // the quantiser's arithmetic, step by step
        const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
        unsigned sum = 0;
        uint32_t word[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            word[g] = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int r_ = rne_i32(val[4 * g + i] * id);
                sum += (unsigned)r_;
                word[g] |= (uint32_t)(sat8(r_) & 0xff) << (8 * i);
            }
        }
        sum += (unsigned)__shfl_xor((int)sum, 32, 64);
        if (m <= m_last) {
            uint8_t* blk = q_out + ((size_t)m * (2 * n_q) + 2 * head + (b >> 1)) * kABlock32;
            const int h2 = b & 1;
#pragma unroll
            for (int g = 0; g < 4; g++) *reinterpret_cast<uint32_t*>(blk + 16 + 32 * h2 + 8 * g + 4 * kh) = word[g];
            if (kh == 0) {
                float* par = reinterpret_cast<float*>(blk);
                par[h2] = d;
                par[2 + h2] = __fmul_rn(d, (float)(int)sum);
            }
        }
    }
}

template <int G, int S>
constexpr size_t prefill_lds_bytes() {
    constexpr size_t staging = (size_t)S * kTileLdsBytes;
    constexpr size_t merge = (size_t)kMergeSlotBytes * G * (S / 2 > 0 ? S / 2 : 1) + (size_t)2 * S * G * 32 * sizeof(float);
    return staging > merge ? staging : merge;
}

template <int G, int S>
hipError_t launch_prefill(dim3 grid, const float* q, int q_row_stride, const __half* kc, const __half* vc, const int* pos_dev,
                          float* out, int out_row_stride, uint8_t* q_out, int n_q, int M, int max_seq, float scale,
                          hipStream_t s) {
    constexpr size_t lds = prefill_lds_bytes<G, S>();
    static_assert(lds <= (size_t)kLdsLimitBytes, "attention tile buffers exceed the LDS of a CU");
    if (lds > 64 * 1024) {  // a kernel gets 64 KiB of dynamic LDS without asking
        const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<G, S>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (attr != hipSuccess) return attr;
    }
    hipLaunchKernelGGL((attention_prefill_kernel<G, S>), grid, dim3(64 * G * S), lds, s, q, q_row_stride, kc, vc, pos_dev, out,
                       out_row_stride, q_out, n_q, M, max_seq, scale);
    return hipGetLastError();
}

}  // namespace

bool attention_prefill_fits(int M, int n_q, int n_kv) {
    if (M <= 8 || n_kv < 1 || n_q % n_kv) return false;
    const int g = n_q / n_kv;
    return g == 1 || g == 2 || g == 4 || g == 8;
}

hipError_t launch_attention_prefill(const float* q, int q_row_stride, const void* k_cache, const void* v_cache,
                                    const int* pos_dev, float* out, int out_row_stride, int M, int n_q, int n_kv, int max_seq,
                                    float scale, hipStream_t s, void* q_out, int heads_per_workgroup) {
    const int tiles = (M + kTile - 1) / kTile, group = n_q / n_kv;
    uint8_t* qo = static_cast<uint8_t*>(q_out);
    const __half* kc = static_cast<const __half*>(k_cache);
    const __half* vc = static_cast<const __half*>(v_cache);
    // G heads x S key splits per workgroup, at most 8 waves: a wave needs about 220 registers per
    // lane (64 for its query, 64 for its output), which rules out four waves per SIMD.  The whole
    // group in one workgroup shares each staged tile among the most heads; with few query tiles that
    // leaves most of the chip idle (322 tokens, 8 KV heads: 88 workgroups), so the group is then cut
    // into workgroups of fewer heads and more key splits until there are at least 128 (322 tokens: 23.6 -> 21.2 us
    // with two heads per workgroup; one head per workgroup: 32.6 us, and 10.2 against 11.3 us at 64 tokens).
    // A81W41_ATTENTION_HEADS=<G> fixes the heads per workgroup (measurement aid, tuning builds only).
    static const int env_g = tuning_env_int("A81W41_ATTENTION_HEADS");
    int g = group;
    while (g > 1 && tiles * n_kv * (group / g) < 128) g >>= 1;
    if (env_g > 0 && env_g <= group && group % env_g == 0) g = env_g;
    if (heads_per_workgroup > 0) {
        if (heads_per_workgroup > group || group % heads_per_workgroup) return hipErrorInvalidValue;
        g = heads_per_workgroup;
    }
    const dim3 grid(tiles, n_kv, group / g);
    switch (g) {
        case 1: return launch_prefill<1, 4>(grid, q, q_row_stride, kc, vc, pos_dev, out, out_row_stride, qo, n_q, M, max_seq, scale, s);
        case 2: return launch_prefill<2, 4>(grid, q, q_row_stride, kc, vc, pos_dev, out, out_row_stride, qo, n_q, M, max_seq, scale, s);
        case 4: return launch_prefill<4, 2>(grid, q, q_row_stride, kc, vc, pos_dev, out, out_row_stride, qo, n_q, M, max_seq, scale, s);
        case 8: return launch_prefill<8, 1>(grid, q, q_row_stride, kc, vc, pos_dev, out, out_row_stride, qo, n_q, M, max_seq, scale, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace a81w41
