// M = 1 contraction: C[0..N) = quantised activation row (fp16 params) x int4
// weights (320 B blocks, fp16 params).  HBM-bound: every weight byte is read
// exactly once, with 128-bit loads.
//
// Work split.  A column group g (8 columns) owns K/64 consecutive 320 B blocks.
// Workgroups are persistent and stage the activation row in LDS once.  The
// waves of a workgroup form slots of WPG waves; per iteration each slot takes
// one column group (slot s of workgroup b: groups b*slots+s, +grid*slots, ...)
// and wave w of the slot takes steps w, w+WPG, ... of 16 consecutive blocks
// (5 KiB contiguous) each.  Inside a wave, 4 lanes share a block:
//   lane = 4*blk + sub,  h = sub & 1 (columns 4h..4h+3),  pp = sub >> 1
// and the lane reads the 16-byte chunks of packs p = pp, pp+2, pp+4, pp+6 that
// hold its four columns -- so each wave-wide load instruction touches 16 runs of
// 64 contiguous, 64-byte aligned bytes.  The loads of the next step (or of the
// next group's first step) are issued before the current step is consumed.
// The lane accumulates its four packs with v_dot4_i32_i8 into exact int32
// partial block dots (low and high 32-block, 4 columns), one DPP add merges the
// two pp lanes, and lane (h, pp) then applies the scale / min epilogue for
// 32-block lh = pp with the reference's operations:
//   acc = fma(float(idot), fl(dA*dW), acc);  acc = fma(mW, sA, acc)
// (quantized_gemx_kernels.cc:181-188).  fp32 partial sums are reduced across
// lanes, then across the waves in a fixed order (deterministic output).
//
// Activation row in LDS: either copied from a 72 B-block blob, or quantised on
// the fly from fp32 by every workgroup (fused prologue; workgroup 0 also writes
// the blob out so the caller's scratch holds what the reference's would).  The
// fp32 row is x itself, or silu(gate)*up of a [2K] gate|up row (Qwen3SiLuMul,
// QwenOperator.cc:697-713), or rmsnorm(x + residual)*w (add + Qwen3RMSNorm,
// QwenOperator.cc:24-53,715-722; workgroup 0 also writes the new residual),
// which saves the separate elementwise launch in front of a decode-step linear.
//
// Paired output (prologue id 5, add + norm in front): the matrix is a gate|up pair (N = 2 I) and the
// launch does not write its N outputs but the quantised blocks of silu(gate) * up, the next linear's
// input (Qwen3SiLuMul + quantize_row_q8_1_repack_fp16).  Workgroup u owns 32-block u of that row:
// its iterations take the four gate groups 4u..4u+3, then the four up groups, park the 64 sums in
// LDS, and 32 lanes finish the block.
//
// The A80W40 variant (gemv_repack_A80W40, quantized_gemx_kernels.cc:39-109) shares the
// kernel: same blocks, codes read as code - 8, no min term.  The lane subtracts eight
// times the sum of the activation bytes it dotted, which keeps the block dots exact,
// and never touches the min / scaled-sum fields (that variant's writers leave them unset).
#include "gemv_common.h"

#include <cstdio>
#include <cstdlib>

namespace a81w41 {
namespace {

using namespace gemv;

// Argument order: the leading pointer and integers are handed over in scalar registers at dispatch
// (kernel-argument preloading, switched on in the Makefile; it stops at the first struct), so the row
// can be requested before the load of the remaining arguments has come back (0.2-0.3 us per launch).
template <int PRO, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void gemv_a81w41_fp16_kernel(const void* __restrict__ A_or_x, int nb_n,
                                                                     int nb_k, int wpg_log2,
                                                                     uint8_t* __restrict__ a_out,
                                                                     const GemvBatch bt,
                                                                     const GemvPrologue pro) {
    extern __shared__ __align__(16) uint32_t lds[];  // nb_k*24 words of activations, then 2*kWaves*32 floats
    constexpr int kThreads = 64 * kWaves;
    constexpr bool kA80 = PRO == kProBlobA80;
    constexpr bool kFromBlob = PRO == kProBlob || PRO == kProBlobA80;
    constexpr bool kPair = PRO == kProAddNormPair;
    constexpr bool kAddNorm = PRO == kProAddNorm || PRO == kProAddNormPair;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 3, pp = sub >> 1;
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    const int wpg = 1 << wpg_log2;                 // waves per column group
    const int slots = kWaves >> wpg_log2;          // column groups in flight per workgroup
    const int slot = wave >> wpg_log2, wig = wave & (wpg - 1);
    const int spw = (n_steps + wpg - 1) >> wpg_log2;  // steps per wave per group
    const int blk_in_step = lane >> 2;
    const int g_stride = gridDim.x * slots;

    // Work items of this wave: item i -> group (blockIdx.x*slots + slot) + (i / spw) * g_stride,
    // step wig + (i % spw) * wpg.
    int gb = blockIdx.x * slots;  // slot 0's group: the loop bound, uniform over the workgroup
    int g = gb + slot, si = 0;
    BlockLoads cur;
    // The vector-memory counter retires in order: a wait for a load also waits for everything requested
    // before it.  So the activation loads of the prologue go first and the first weight blocks right
    // behind them (the scheduling barriers pin that order); the prologue then runs on the activations
    // while the weights are still on their way.
    auto request_first_weights = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        // every wave of the workgroup has requested its part of the row before any of them requests weights:
        // the CU's memory path serves requests in the order they come, and a late wave's row request behind
        // 16 waves' weight blocks held the whole workgroup at the barrier after the prologue
        __builtin_amdgcn_s_barrier();
        const int blk = wig * kBlocksPerStep + blk_in_step;
        const int pg = kPair ? pair_group(min(g, nb_n - 1), g_stride, slots, nb_n) : g;
        load_block<!kA80>(cur, locate(bt, pg, nb_k).B + (size_t)blk * kWBlock16, sub, g < nb_n && blk < nb_k);
        __builtin_amdgcn_sched_barrier(0);
    };

    // Activation prologue.  All global loads of a chunk are issued before the first
    // is consumed, so the prologue costs about one memory round trip, not one per element.
    constexpr int kChunk = 4;
    if (!kFromBlob) {
        const float4* x4 = reinterpret_cast<const float4*>(A_or_x);
        const int n_vec = 16 * nb_k;
        for (int base = 0; base < n_vec; base += kChunk * kThreads) {
            float4 v[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_vec) ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            float4 up[PRO == kProSiluMul ? kChunk : 1];  // kProSiluMul: x4 is the gate half of a [2K] row, the up half follows it
            float4 g[kAddNorm ? kChunk : 1], rr[kAddNorm ? kChunk : 1];  // norm weights and residual, requested with the row
            if (PRO == kProSiluMul) {
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    const int i = base + u * kThreads + tid;
                    up[PRO == kProSiluMul ? u : 0] = (i < n_vec) ? x4[n_vec + i] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            if (kAddNorm) {
                const float4* r4 = reinterpret_cast<const float4*>(pro.res_in);
                const float4* w4 = reinterpret_cast<const float4*>(pro.norm_w);
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    const int i = base + u * kThreads + tid;
                    g[kAddNorm ? u : 0] = (i < n_vec) ? w4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                    rr[kAddNorm ? u : 0] = (i < n_vec && r4 != nullptr) ? r4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            if (base == 0) request_first_weights();
            if (PRO == kProSiluMul) {
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    if (base + u * kThreads >= n_vec) break;  // empty slice (uniform)
                    const float4 p = up[PRO == kProSiluMul ? u : 0];
                    v[u].x = (v[u].x * (1.0f / (1.0f + expf(-v[u].x)))) * p.x;
                    v[u].y = (v[u].y * (1.0f / (1.0f + expf(-v[u].y)))) * p.y;
                    v[u].z = (v[u].z * (1.0f / (1.0f + expf(-v[u].z)))) * p.z;
                    v[u].w = (v[u].w * (1.0f / (1.0f + expf(-v[u].w)))) * p.w;
                }
            }
            if (kAddNorm) {  // the whole row is in this one chunk (the launcher checks)
                const bool has_res = pro.res_in != nullptr;
                float4* o4 = reinterpret_cast<float4*>(pro.res_out);
                // sum of squares in an order that does not depend on the workgroup's width: per float4, then over
                // each aligned group of 64 float4 (a wave's slice), then over the groups by the same tree
                float ss[kChunk];
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    const int i = base + u * kThreads + tid;
                    ss[u] = 0.f;
                    if (i < n_vec) {
                        if (has_res) {
                            const float4 r = rr[kAddNorm ? u : 0];
                            v[u].x += r.x; v[u].y += r.y; v[u].z += r.z; v[u].w += r.w;
                        }
                        if (blockIdx.x == 0) o4[i] = v[u];
                        ss[u] = v[u].x * v[u].x + v[u].y * v[u].y + v[u].z * v[u].z + v[u].w * v[u].w;
                    }
                }
                float* part = reinterpret_cast<float*>(lds + nb_k * kLdsWordsPerSb);  // the reduction area, idle now
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    if (base + u * kThreads >= n_vec) break;  // empty slice (uniform over the workgroup)
                    ss[u] = wave_sum_fixed_order(ss[u]);
                    if (lane == 0) part[u * kWaves + wave] = ss[u];
                }
                lds_barrier();
                sum_groups_fixed_order(part, (n_vec + 63) / 64, wave, lane);
                lds_barrier();
                const float total = part[64];
                const float inv = 1.0f / sqrtf(total / (float)(64 * nb_k) + pro.eps);
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    const int i = base + u * kThreads + tid;
                    if (i < n_vec)
                        v[u] = make_float4((v[u].x * inv) * g[kAddNorm ? u : 0].x, (v[u].y * inv) * g[kAddNorm ? u : 0].y,
                                           (v[u].z * inv) * g[kAddNorm ? u : 0].z, (v[u].w * inv) * g[kAddNorm ? u : 0].w);
                }
            }
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                // wide workgroups cover a short row with fewer than kChunk slices: skip the empty ones
                // (uniform over the workgroup; an empty slice costs the quantiser's two divisions)
                if (base + u * kThreads >= n_vec) break;
                const int i = base + u * kThreads + tid;
                const bool valid = i < n_vec;  // uniform over each aligned group of 8 lanes
                const Quant4 qz = quantize_float4_of_block32(v[u]);
                if (valid) {
                    const int b32 = i >> 3, p = i & 7, sb = b32 >> 1, lh = b32 & 1;
                    const uint16_t d16 = f32_to_f16_bits(qz.d), s16 = f32_to_f16_bits(qz.ssum);
                    uint32_t* dst = lds + sb * kLdsWordsPerSb;
                    dst[lds_q_word(lh, p)] = qz.packed;
                    if (p == 0) {
                        dst[12 * lh + 8] = __float_as_uint(f16_bits_to_f32(d16));
                        dst[12 * lh + 9] = __float_as_uint(f16_bits_to_f32(s16));
                    }
                    if (a_out != nullptr && blockIdx.x == 0) {
                        uint8_t* ob = a_out + (size_t)sb * kABlock16;
                        *reinterpret_cast<uint32_t*>(ob + 8 + 32 * lh + 4 * p) = qz.packed;
                        if (p == 0) {
                            reinterpret_cast<uint16_t*>(ob)[lh] = d16;
                            reinterpret_cast<uint16_t*>(ob)[2 + lh] = s16;
                        }
                    }
                }
            }
        }
    } else {
        // nine 8-byte words per 72 B block -> 24-word LDS image.
        const uint2* A64 = reinterpret_cast<const uint2*>(A_or_x);
        const int n_w = 9 * nb_k;
        for (int base = 0; base < n_w; base += kChunk * kThreads) {
            uint2 v[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_w) ? A64[i] : make_uint2(0, 0);
            }
            if (base == 0) request_first_weights();
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                if (i < n_w) {
                    const int sb = i / 9, w = i - sb * 9;
                    uint32_t* dst = lds + sb * kLdsWordsPerSb;
                    if (w == 0) {  // s_low | s_high, scaled_sum_low | scaled_sum_high
                        dst[8] = __float_as_uint(f16_bits_to_f32(v[u].x & 0xffff));
                        dst[12 + 8] = __float_as_uint(f16_bits_to_f32(v[u].x >> 16));
                        dst[9] = __float_as_uint(f16_bits_to_f32(v[u].y & 0xffff));
                        dst[12 + 9] = __float_as_uint(f16_bits_to_f32(v[u].y >> 16));
                    } else {
                        const int qi = 2 * (w - 1);  // q words qi, qi+1: same 32-block, packs p, p+1
                        dst[lds_q_word(qi >> 3, qi & 7)] = v[u].x;
                        dst[lds_q_word(qi >> 3, (qi & 7) + 1)] = v[u].y;
                    }
                }
            }
        }
    }
    lds_barrier();  // the activation image is complete; the first weight blocks may still be on their way

    float* red = reinterpret_cast<float*>(lds + nb_k * kLdsWordsPerSb);
    float* pair_vals = red + 2 * kMaxWaves * 32;  // 64 floats behind the reduction area
    int parity = 0;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    while (gb < nb_n) {  // gb, si advance identically in every wave: uniform over the workgroup
        const int step = wig + si * wpg;
        const int blk = step * kBlocksPerStep + blk_in_step;
        const bool valid = blk < nb_k;
        // next work item of this wave
        int ng = g, nsi = si + 1;
        if (nsi == spw) {
            nsi = 0;
            ng = g + g_stride;
        }
        BlockLoads nxt;
        {
            const int nblk = (wig + nsi * wpg) * kBlocksPerStep + blk_in_step;
            const int png = kPair ? pair_group(min(ng, nb_n - 1), g_stride, slots, nb_n) : ng;
            load_block<!kA80>(nxt, locate(bt, png, nb_k).B + (size_t)nblk * kWBlock16, sub, ng < nb_n && nblk < nb_k);
        }

        consume_block<kA80>(cur, lds + (valid ? blk : 0) * kLdsWordsPerSb + 12 * pp, pp, acc);
        cur = nxt;

        if (nsi == 0) {  // group finished (uniform over the workgroup)
            sum_rows_of_16(acc);
            float* r = red + parity * (kWaves * 32);
            if ((lane & 15) < 2) {
                float4* dst = reinterpret_cast<float4*>(r + wave * 32 + (lane >> 4) * 8 + 4 * (lane & 1));
                *dst = make_float4(acc[0], acc[1], acc[2], acc[3]);
            }
            lds_barrier();  // not __syncthreads(): the next item's weight blocks stay in flight
            if (tid < 8 * slots) {  // thread (s, col) sums slot s's waves and rows in order and stores
                const int s_ = tid >> 3, col = tid & 7;
                const int gs = gb + s_;
                const float* rs = r + (s_ << wpg_log2) * 32 + col;
                float v = 0.f;
                for (int w = 0; w < 4 * wpg; w++) v += rs[w * 8];
                if (kPair) {  // sum w*8 + col of the workgroup's 64: gate 0..31, up 32..63
                    pair_vals[((gb / g_stride) * slots + s_) * 8 + col] = v;
                } else if (gs < nb_n) {
                    locate(bt, gs, nb_k).C[col] = v;
                }
            }
            parity ^= 1;  // this buffer is rewritten only after the next group's barrier
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] = 0.f;
            gb += g_stride;
        }
        g = ng;
        si = nsi;
    }
    if (kPair) {
        __syncthreads();  // the 64 sums are in LDS
        if (tid < 32) {
            const float gt = pair_vals[tid], up = pair_vals[32 + tid];
            const float act = (gt * (1.0f / (1.0f + expf(-gt)))) * up;  // Qwen3SiLuMul, QwenOperator.cc:697-713
            store_quantized_value_fp16(pro.pair_out, blockIdx.x * 32 + tid, act);
        }
    }
}

}  // namespace

int gemv_lds_bytes(int K) { return ((K / 64) * kLdsWordsPerSb + 2 * kMaxWaves * 32 + 64) * (int)sizeof(uint32_t); }

int gemv_max_k() { return (kLdsLimitBytes - gemv_lds_bytes(0)) / ((int)sizeof(uint32_t) * kLdsWordsPerSb) * 64; }

namespace {

struct GemvTune {
    int waves, max_grid, wpg;  // workgroup width, persistent-grid cap, waves per column group (0 = auto)
};

// Workgroup width and persistent-grid cap.  In tuning builds A81W41_GEMV_TUNE="waves,grid,wpg" overrides
// the table (measurement aid; waves must be 4, 8 or 16).
GemvTune pick_tune(int nb_n, int nb_k) {
    static const GemvTune env = [] {
        GemvTune t{0, 0, 0};
        if (const char* e = tuning_env("A81W41_GEMV_TUNE")) sscanf(e, "%d,%d,%d", &t.waves, &t.max_grid, &t.wpg);
        return t;
    }();
    if (env.waves == 4 || env.waves == 8 || env.waves == 16)
        return {env.waves, env.max_grid > 0 ? env.max_grid : kGemvMaxGrid, env.wpg};
    // Measured on MI355X: few column groups -> narrow workgroups so every CU gets one;
    // long K -> wide workgroups (the activation row is staged per workgroup).
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    if (nb_n <= 256) return {4, kGemvMaxGrid, 0};
    if (n_steps <= 4) {
        // K = 4096 class.  N = 4096 and 12288: 8 waves, 512 workgroups.  Measured exceptions:
        // 6144 (q+k+v in one linear) is 7 % faster with 16-wave workgroups, the vocabulary-sized head
        // 3 % with two waves per column group.
        if (nb_n > 512 && nb_n <= 1024) return {16, 256, 0};
        if (nb_n > 2048 && nb_n <= 4096) return {8, 768, 0};  // 24576 (gate+up in one launch): one even round, 8 % faster
        if (nb_n > 16384) return {8, 512, 2};
        return {8, 512, 0};
    }
    return {16, 256, 0};
}

}  // namespace

// Waves per column group of a launch over nb_n groups of nb_k blocks: a power of two, at most the workgroup
// width and the number of 16-block steps.  It fixes the order in which a column's partial sums are added.
int gemv_waves_per_group_log2(int nb_n, int nb_k, bool paired_output) {
    const GemvTune t = pick_tune(nb_n, nb_k);
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    int wpg_log2 = 0;
    const int want = t.wpg > 0 ? t.wpg : n_steps;
    while ((2 << wpg_log2) <= want && (2 << wpg_log2) <= t.waves) wpg_log2++;
    // paired output: a workgroup walks its eight groups in 8 / slots rounds, so at most eight groups at a time
    // (short rows in wide workgroups -- hidden 1024 with 16 waves -- would otherwise have sixteen)
    if (paired_output)
        while ((t.waves >> wpg_log2) > 8) wpg_log2++;
    return wpg_log2;
}

namespace {

template <int PRO>
hipError_t launch(const void* a_or_x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs,
                  const int* Ns, int K, const GemvPrologue& pro, hipStream_t s) {
    const int nb_k = K / 64;
    GemvBatch bt;
    int nb_n = 0;
    for (int j = 0; j < kGemvMaxBatch; j++) {
        const int jj = j < n_mat ? j : n_mat - 1;
        bt.B[j] = static_cast<const uint8_t*>(Bs[jj]);
        bt.C[j] = Cs[jj];
        if (j < n_mat) nb_n += Ns[j] / 8;
        bt.end[j] = nb_n;
    }
    const GemvTune t = pick_tune(nb_n, nb_k);
    // the add + norm prologue holds the whole row in one chunk of 4 float4 per thread
    if ((PRO == kProAddNorm || PRO == kProAddNormPair) && 16 * nb_k > 4 * 64 * t.waves) return hipErrorInvalidValue;
    const int wpg_log2 = gemv_waves_per_group_log2(nb_n, nb_k, PRO == kProAddNormPair);
    const int slots = t.waves >> wpg_log2;
    const int wgs = (nb_n + slots - 1) / slots;
    int grid = wgs < t.max_grid ? wgs : t.max_grid;
    if (PRO == kProAddNormPair) {  // one workgroup per 32-block of the paired output
        if (n_mat != 1 || nb_n % 8 || pro.pair_out == nullptr) return hipErrorInvalidValue;
        grid = nb_n / 8;
    }
    uint8_t* ao = static_cast<uint8_t*>(a_out);
    const size_t lds = gemv_lds_bytes(K);
    // A kernel gets 64 KiB of dynamic LDS without asking; longer activation rows (K > 43 008) ask first.
#define A81W41_GEMV_LAUNCH(W)                                                                                          \
    do {                                                                                                               \
        if (lds > 64 * 1024) {                                                                                         \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_a81w41_fp16_kernel<PRO, W>),  \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimitBytes);     \
            if (e != hipSuccess) return e;                                                                             \
        }                                                                                                              \
        hipLaunchKernelGGL((gemv_a81w41_fp16_kernel<PRO, W>), dim3(grid), dim3(64 * W), lds, s, a_or_x, nb_n, nb_k,      \
                           wpg_log2, ao, bt, pro);                                                                         \
    } while (0)
    switch (t.waves) {
        case 16: A81W41_GEMV_LAUNCH(16); break;
        case 8: A81W41_GEMV_LAUNCH(8); break;
        default: A81W41_GEMV_LAUNCH(4);
    }
#undef A81W41_GEMV_LAUNCH
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemv_fp16(const void* A, const void* B, float* C, int N, int K, hipStream_t s) {
    return launch<kProBlob>(A, nullptr, 1, &B, &C, &N, K, GemvPrologue{}, s);
}

hipError_t launch_gemv_a80w40(const void* A, const void* B, float* C, int N, int K, hipStream_t s) {
    return launch<kProBlobA80>(A, nullptr, 1, &B, &C, &N, K, GemvPrologue{}, s);
}

hipError_t launch_gemv_fused(const float* x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs,
                             const int* Ns, int K, hipStream_t s) {
    return launch<kProX>(x, a_out, n_mat, Bs, Cs, Ns, K, GemvPrologue{}, s);
}

hipError_t launch_gemv_silu_mul(const float* gate_up, void* a_out, const void* B, float* C, int N, int K, hipStream_t s) {
    return launch<kProSiluMul>(gate_up, a_out, 1, &B, &C, &N, K, GemvPrologue{}, s);
}

bool gemv_add_norm_fits(int K) { return K % 64 == 0 && K / 4 <= 4 * 64 * 4 && gemv_lds_bytes(K) <= kLdsLimitBytes; }

hipError_t launch_gemv_add_norm(const float* x, const GemvPrologue& pro, void* a_out, const void* B, float* C, int N,
                                int K, hipStream_t s) {
    return launch<kProAddNorm>(x, a_out, 1, &B, &C, &N, K, pro, s);
}

bool gemv_pair_fits(int N, int K) { return gemv_add_norm_fits(K) && N % 64 == 0; }

hipError_t launch_gemv_add_norm_silu_pair(const float* x, const GemvPrologue& pro, const void* B_gate_up, int N, int K,
                                          hipStream_t s) {
    float* no_c = nullptr;
    return launch<kProAddNormPair>(x, nullptr, 1, &B_gate_up, &no_c, &N, K, pro, s);
}

}  // namespace a81w41
