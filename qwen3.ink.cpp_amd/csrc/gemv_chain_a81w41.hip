// M = 1 contraction as a link of a chain of overlapping launches (chain.h): the same arithmetic, in the same
// order, as gemv_a81w41_fp16_kernel -- block dots with v_dot4_i32_i8, the reference's two fma per 32-block
// (quantized_gemx_kernels.cc:181-188), per-lane sums over a wave's steps, rows of 16 lanes, then the waves of a
// column group in wave order -- so a chained launch returns the bits of the plain one (same waves per group).
// What differs is when things happen:
//   1. every wave requests its first two steps of weight blocks (they do not depend on the activation row);
//   2. the workgroup waits for the launch it depends on, which may still be running on the same CUs;
//   3. the activation row is read with agent-scope loads, quantised (or copied) into LDS;
//   4. the steps are consumed with two further steps in flight;
//   5. outputs leave with agent-scope stores and the workgroup signals.
// Workgroups have 8 waves and a launch has at most one workgroup per CU (two waves per SIMD, under 128
// registers, a fraction of the LDS), so that two consecutive links of a chain always fit on the chip together:
// a waiting consumer can never keep its producer's workgroups from being placed.
#include "chain.h"
#include "gemv_common.h"

namespace a81w41 {
namespace {

using namespace gemv;

constexpr int kWaves = 8, kThreads = 64 * kWaves;

// The work of one wave as a sequence of items: item i = (round i / spw, step wig + (i % spw) * wpg); in round r
// the workgroup's slot s works on column group group_of(r, s).
struct Walk {
    int nb_n, nb_k, wpg, spw, slots, grid, block;
    int n_rounds;  // uniform over the workgroup
    bool pair;
    __device__ __forceinline__ int group_of(int round, int slot) const {
        if (!pair) return (block + round * grid) * slots + slot;
        // paired output: unit u = 32 outputs of silu(gate) * up = gate groups 4u..4u+3 and up groups 4u..4u+3,
        // walked in 8 / slots rounds
        const int per_unit = 8 / slots, u = block + (round / per_unit) * grid, w = (round % per_unit) * slots + slot;
        if (8 * u >= nb_n) return nb_n;  // past the last unit
        return w < 4 ? 4 * u + w : (nb_n >> 1) + 4 * u + (w - 4);
    }
};

template <int PRO>
__global__ __launch_bounds__(kThreads) void gemv_chain_kernel(const void* __restrict__ A_or_x, int nb_n, int nb_k,
                                                              int wpg_log2, int n_rounds, uint8_t* __restrict__ a_out,
                                                              const ChainLink link, const GemvBatch bt,
                                                              const GemvPrologue pro) {
    extern __shared__ __align__(16) uint32_t lds[];  // nb_k*24 words of activations, 2*kWaves*32 floats, 64 floats
    constexpr bool kFromBlob = PRO == kProBlob;
    constexpr bool kPair = PRO == kProAddNormPair;
    constexpr bool kAddNorm = PRO == kProAddNorm || PRO == kProAddNormPair;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 3, pp = sub >> 1;
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    const int wpg = 1 << wpg_log2;
    Walk wk;
    wk.nb_n = nb_n, wk.nb_k = nb_k, wk.wpg = wpg, wk.spw = (n_steps + wpg - 1) >> wpg_log2;
    wk.slots = kWaves >> wpg_log2, wk.grid = gridDim.x, wk.block = blockIdx.x, wk.n_rounds = n_rounds, wk.pair = kPair;
    const int slot = wave >> wpg_log2, wig = wave & (wpg - 1);
    const int blk_in_step = lane >> 2;
    const int n_items = n_rounds * wk.spw;

    auto request = [&](BlockLoads& L, int item) {
        const int round = item / wk.spw, sidx = item - round * wk.spw;
        const int g = wk.group_of(round, slot);
        const int blk = (wig + sidx * wpg) * kBlocksPerStep + blk_in_step;
        const bool valid = item < n_items && g < nb_n && blk < nb_k;
        load_block<true>(L, locate(bt, valid ? g : 0, nb_k).B + (size_t)(valid ? blk : 0) * kWBlock16, sub, valid);
    };

    // 1. what does not depend on the producer
    BlockLoads q0, q1, q2;
    request(q0, 0);
    request(q1, 1);
    constexpr int kChunk = 2;  // float4 (or 8-byte blob words) per thread and pass over the row
    float4 nw[kAddNorm ? kChunk : 1];
    if (kAddNorm) {
        const float4* w4 = reinterpret_cast<const float4*>(pro.norm_w);
#pragma unroll
        for (int u = 0; u < kChunk; u++) {
            const int i = u * kThreads + tid;
            nw[kAddNorm ? u : 0] = (i < 16 * nb_k) ? w4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // 2. the producer is complete (or the wait gave up: the kernel then runs on whatever is there)
    chain_wait(link);

    // 3. the activation row
    if (!kFromBlob) {
        const float* x = static_cast<const float*>(A_or_x);
        const int n_vec = 16 * nb_k;
        for (int base = 0; base < n_vec; base += kChunk * kThreads) {
            float4 v[kChunk], rr[kAddNorm ? kChunk : 1];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_vec) ? load16_agent_f4(x + 4 * (size_t)i) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            if (kAddNorm) {
#pragma unroll
                for (int u = 0; u < kChunk; u++) {
                    const int i = base + u * kThreads + tid;
                    rr[kAddNorm ? u : 0] = (i < n_vec && pro.res_in != nullptr) ? load16_agent_f4(pro.res_in + 4 * (size_t)i)
                                                                                : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            if (kAddNorm) {  // the whole row is in this one pass (the launcher checks)
                const bool has_res = pro.res_in != nullptr;
                // sum of squares per float4, then over each aligned group of 64 float4, then over the groups by
                // the same tree: the plain kernel's order, whatever its workgroup width
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
                        if (blockIdx.x == 0) store16_agent_f4(pro.res_out + 4 * (size_t)i, v[u]);
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
                        v[u] = make_float4((v[u].x * inv) * nw[kAddNorm ? u : 0].x, (v[u].y * inv) * nw[kAddNorm ? u : 0].y,
                                           (v[u].z * inv) * nw[kAddNorm ? u : 0].z, (v[u].w * inv) * nw[kAddNorm ? u : 0].w);
                }
            }
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                if (base + u * kThreads >= n_vec) break;  // empty slice (uniform over the workgroup)
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
                        store_agent(reinterpret_cast<uint32_t*>(ob + 8 + 32 * lh + 4 * p), qz.packed);
                        if (p == 0) {
                            store_agent(reinterpret_cast<uint16_t*>(ob) + lh, d16);
                            store_agent(reinterpret_cast<uint16_t*>(ob) + 2 + lh, s16);
                        }
                    }
                }
            }
        }
    } else {
        // nine 8-byte words per 72 B block -> 24-word LDS image
        const unsigned long long* A64 = static_cast<const unsigned long long*>(A_or_x);
        const int n_w = 9 * nb_k;
        for (int base = 0; base < n_w; base += kChunk * kThreads) {
            unsigned long long v[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_w) ? load_agent(A64 + i) : 0ull;
            }
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                if (i < n_w) {
                    const uint32_t lo = (uint32_t)v[u], hi = (uint32_t)(v[u] >> 32);
                    const int sb = i / 9, w = i - sb * 9;
                    uint32_t* dst = lds + sb * kLdsWordsPerSb;
                    if (w == 0) {  // s_low | s_high, scaled_sum_low | scaled_sum_high
                        dst[8] = __float_as_uint(f16_bits_to_f32(lo & 0xffff));
                        dst[12 + 8] = __float_as_uint(f16_bits_to_f32(lo >> 16));
                        dst[9] = __float_as_uint(f16_bits_to_f32(hi & 0xffff));
                        dst[12 + 9] = __float_as_uint(f16_bits_to_f32(hi >> 16));
                    } else {
                        const int qi = 2 * (w - 1);  // q words qi, qi+1: same 32-block, packs p, p+1
                        dst[lds_q_word(qi >> 3, qi & 7)] = lo;
                        dst[lds_q_word(qi >> 3, (qi & 7) + 1)] = hi;
                    }
                }
            }
        }
    }
    lds_barrier();  // the activation image is complete

    // 4. the steps, two further ones in flight
    float* red = reinterpret_cast<float*>(lds + nb_k * kLdsWordsPerSb);
    float* pair_vals = red + 2 * kWaves * 32;  // 64 floats behind the reduction area
    int parity = 0;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto step = [&](const BlockLoads& L, int item) {
        const int round = item / wk.spw, sidx = item - round * wk.spw;
        const int blk = (wig + sidx * wpg) * kBlocksPerStep + blk_in_step;
        const bool valid = blk < nb_k;  // a group past the end was loaded as zeros
        consume_block<false>(L, lds + (valid ? blk : 0) * kLdsWordsPerSb + 12 * pp, pp, acc);
        if (sidx != wk.spw - 1) return;
        // the round's groups are finished (uniform over the workgroup)
        sum_rows_of_16(acc);
        float* r = red + parity * (kWaves * 32);
        if ((lane & 15) < 2) {
            float4* dst = reinterpret_cast<float4*>(r + wave * 32 + (lane >> 4) * 8 + 4 * (lane & 1));
            *dst = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
        lds_barrier();
        if (tid < 8 * wk.slots) {  // thread (s, col) sums slot s's waves and rows in order and stores
            const int s_ = tid >> 3, col = tid & 7;
            const int gs = wk.group_of(round, s_);
            const float* rs = r + (s_ << wpg_log2) * 32 + col;
            float v = 0.f;
            for (int w = 0; w < 4 * wpg; w++) v += rs[w * 8];
            if (kPair) {  // sum w*8 + col of the unit's 64: gate 0..31, up 32..63
                pair_vals[((round % (8 / wk.slots)) * wk.slots + s_) * 8 + col] = v;
            } else if (gs < nb_n) {
                store_agent(locate(bt, gs, nb_k).C + col, v);
            }
        }
        parity ^= 1;  // this buffer is rewritten only after the next round's barrier
#pragma unroll
        for (int c = 0; c < 4; c++) acc[c] = 0.f;
        if (kPair && (round + 1) % (8 / wk.slots) == 0) {  // the unit's 64 sums are complete
            lds_barrier();
            const int u = wk.block + (round / (8 / wk.slots)) * wk.grid;
            if (tid < 32 && 8 * u < nb_n) {  // both halves of the wave's first 32 lanes active: u is uniform
                const float gt = pair_vals[tid], up = pair_vals[32 + tid];
                const float act = (gt * (1.0f / (1.0f + expf(-gt)))) * up;  // Qwen3SiLuMul, QwenOperator.cc:697-713
                store_quantized_value_fp16<true>(pro.pair_out, u * 32 + tid, act);
            }
        }
    };
    for (int i = 0; i < n_items; i += 3) {  // n_items is uniform over the workgroup
        request(q2, i + 2);
        step(q0, i);
        if (i + 1 >= n_items) break;
        request(q0, i + 3);
        step(q1, i + 1);
        if (i + 2 >= n_items) break;
        request(q1, i + 4);
        step(q2, i + 2);
    }

    // 5. outputs acknowledged, then the signal
    chain_signal(link, gridDim.x);
}

int log2_floor(int v) {
    int l = 0;
    while ((2 << l) <= v) l++;
    return l;
}

template <int PRO>
hipError_t launch(const void* a_or_x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs, const int* Ns, int K,
                  const GemvPrologue& pro, const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s) {
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
    constexpr bool kPair = PRO == kProAddNormPair;
    constexpr bool kAddNorm = PRO == kProAddNorm || PRO == kProAddNormPair;
    if (kAddNorm && 16 * nb_k > 2 * kThreads) return hipErrorInvalidValue;  // the norm holds the row in one pass
    if (kPair && (n_mat != 1 || nb_n % 8 || pro.pair_out == nullptr)) return hipErrorInvalidValue;
    // waves per column group: what the plain launch of this shape uses (same order of additions), at most a workgroup
    int wpg_log2 = gemv_waves_per_group_log2(nb_n, nb_k, kPair);
    if (wpg_log2 > log2_floor(kWaves)) wpg_log2 = log2_floor(kWaves);
    const int slots = kWaves >> wpg_log2;
    // rounds of (slots) groups -- or of units of 8 groups -- dealt over at most one workgroup per CU, evenly
    const int per_unit = kPair ? 8 / slots : 1;
    const int units = kPair ? nb_n / 8 : (nb_n + slots - 1) / slots;
    const int passes = (units + cus - 1) / cus;
    const int grid = (units + passes - 1) / passes;
    const int n_rounds = passes * per_unit;
    const size_t lds = (size_t)(nb_k * kLdsWordsPerSb + 2 * kWaves * 32 + 64) * sizeof(uint32_t);
    if (lds > 64 * 1024) return hipErrorInvalidValue;  // K <= 40960: half of a CU's LDS at most, without asking
    hipLaunchKernelGGL((gemv_chain_kernel<PRO>), dim3(grid), dim3(kThreads), lds, s, a_or_x, nb_n, nb_k, wpg_log2, n_rounds,
                       static_cast<uint8_t*>(a_out), link, bt, pro);
    if (grid_out) *grid_out = (unsigned)grid;
    return hipGetLastError();
}

}  // namespace

bool gemv_chain_fits(int K, bool add_norm) {
    return K % 64 == 0 && (!add_norm || K / 4 <= 2 * kThreads) &&
           (size_t)((K / 64) * kLdsWordsPerSb + 2 * kWaves * 32 + 64) * sizeof(uint32_t) <= 64 * 1024;
}

hipError_t launch_gemv_chain_blob(const void* A, const void* B, float* C, int N, int K, const ChainLink& link, int cus,
                                  unsigned* grid_out, hipStream_t s) {
    return launch<kProBlob>(A, nullptr, 1, &B, &C, &N, K, GemvPrologue{}, link, cus, grid_out, s);
}

hipError_t launch_gemv_chain_fused(const float* x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs,
                                   const int* Ns, int K, const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s) {
    return launch<kProX>(x, a_out, n_mat, Bs, Cs, Ns, K, GemvPrologue{}, link, cus, grid_out, s);
}

hipError_t launch_gemv_chain_add_norm(const float* x, const GemvPrologue& pro, void* a_out, const void* B, float* C, int N,
                                      int K, const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s) {
    return launch<kProAddNorm>(x, a_out, 1, &B, &C, &N, K, pro, link, cus, grid_out, s);
}

hipError_t launch_gemv_chain_add_norm_silu_pair(const float* x, const GemvPrologue& pro, const void* B_gate_up, int N, int K,
                                                const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s) {
    float* no_c = nullptr;
    return launch<kProAddNormPair>(x, nullptr, 1, &B_gate_up, &no_c, &N, K, pro, link, cus, grid_out, s);
}

}  // namespace a81w41
