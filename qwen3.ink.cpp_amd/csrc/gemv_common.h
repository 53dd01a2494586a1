// Pieces shared by the M = 1 kernels (gemv_a81w41.hip, gemv_chain_a81w41.hip): the lane's view of a weight
// block, the joint numbering of the column groups of a batch of matrices, the LDS image of the quantised
// activation row, and the per-step arithmetic.
#pragma once
#include "a81w41_kernels.h"
#include "quantize_common.h"

namespace a81w41 {
namespace gemv {

constexpr int kMaxWaves = 16;
constexpr int kBlocksPerStep = 16;  // blocks a wave consumes per step
// LDS image of one activation super-block: for pp = 0,1: 4 q_low words (packs
// pp,pp+2,pp+4,pp+6), 4 q_high words, dA_pp, sA_pp, 2 pad words  -> 2 x 48 B.
constexpr int kLdsWordsPerSb = 24;

__device__ __forceinline__ int dpp_xor2(int v) { return dpp_i<kDppXor2>(v); }

struct BlockLoads {
    uint4 w[4];    // packs pp, pp+2, pp+4, pp+6 (this lane's 4 columns)
    uint2 sc, mn;  // 4 fp16 scales / mins of 32-block lh = pp, columns 4h..4h+3
};

template <bool MINS>
__device__ __forceinline__ void load_block(BlockLoads& L, const uint8_t* blk, int sub, bool valid) {
    if (valid) {
        const int h = sub & 1, pp = sub >> 1;
        const uint8_t* q = blk + 64 + 16 * h + 32 * pp;
#pragma unroll
        for (int j = 0; j < 4; j++) L.w[j] = *reinterpret_cast<const uint4*>(q + 64 * j);
        L.sc = *reinterpret_cast<const uint2*>(blk + 8 * sub);
        L.mn = MINS ? *reinterpret_cast<const uint2*>(blk + 32 + 8 * sub) : make_uint2(0, 0);
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) L.w[j] = make_uint4(0, 0, 0, 0);
        L.sc = make_uint2(0, 0);
        L.mn = make_uint2(0, 0);
    }
}

// Up to kGemvMaxBatch weight matrices that share the activation row (and K) are
// contracted by one launch: their column groups are numbered back to back.
struct GemvBatch {
    const uint8_t* B[kGemvMaxBatch];
    float* C[kGemvMaxBatch];
    int end[kGemvMaxBatch];  // exclusive end of matrix j's column groups in the joint numbering
};

struct GroupRef {
    const uint8_t* B;  // first block of the column group
    float* C;          // its 8 outputs
};

__device__ __forceinline__ GroupRef locate(const GemvBatch& bt, int g, int nb_k) {
    int j = 0, first = 0;
#pragma unroll
    for (int t = 0; t + 1 < kGemvMaxBatch; t++) {
        if (g >= bt.end[t]) {
            j = t + 1;
            first = bt.end[t];
        }
    }
    const int lg = g - first;
    return {bt.B[j] + (size_t)lg * nb_k * kWBlock16, bt.C[j] + (size_t)lg * 8};
}

// Workgroup barrier that orders LDS traffic only: every LDS access this wave has issued is done, global
// loads stay in flight.  __syncthreads() would drain them too (loads and stores share one counter),
// i.e. wait for the weight blocks requested ahead at every barrier.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt = 0; vector-memory and export counters left alone
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// LDS word of q word (32-block lh, pack p) inside a super-block image.
__device__ __forceinline__ int lds_q_word(int lh, int p) { return 12 * (p & 1) + 4 * lh + (p >> 1); }

// What the activation row is made from (template parameter PRO of the kernel).
// kProBlobA80: a 72 B-block blob again, contracted the A80W40 way.
// kProAddNormPair: kProAddNorm in front, paired gate|up output behind.
enum : int { kProBlob = 0, kProX = 1, kProSiluMul = 2, kProAddNorm = 3, kProBlobA80 = 4, kProAddNormPair = 5 };

// Paired output: the groups a workgroup walks, in its own order v = b*slots + slot + i*g_stride
// (grid = N/64 workgroups, 8/slots iterations each): workgroup b's w-th group (w = i*slots + slot) is
// gate group 4b + w for w < 4, up group 4b + w - 4 after that.
__device__ __forceinline__ int pair_group(int v, int g_stride, int slots, int nb_n) {
    const int i = v / g_stride, rem = v - i * g_stride;
    const int b = rem / slots, w = i * slots + (rem - b * slots);
    return w < 4 ? 4 * b + w : (nb_n >> 1) + 4 * b + (w - 4);
}

// Sum of squares of a row for the add + norm prologues, in an order that does not depend on the workgroup's
// width (so the chained kernel, with other workgroups, finds the same bits): per float4, then over each aligned
// group of 64 float4 (a wave's slice: wave_sum_fixed_order), then over the groups by the same tree
// (sum_groups_fixed_order).
__device__ __forceinline__ float wave_sum_fixed_order(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<0x140>(v);  // row_mirror: the other eight lanes of the row of 16
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
// The groups' sums (at most 64, in part[0 .. n_groups)) added by the same tree, by wave 0; the total goes to part[64].
// Between two workgroup barriers.
__device__ __forceinline__ void sum_groups_fixed_order(float* part, int n_groups, int wave, int lane) {
    if (wave == 0) {
        const float total = wave_sum_fixed_order(lane < n_groups ? part[lane] : 0.f);
        if (lane == 0) part[64] = total;
    }
}

// One step of a lane: the four packs of its block (4 columns, both 32-blocks) against the block's image in LDS
// (a = image + 12 * pp), exact int32 partial dots, one DPP add for the per-(column, 32-block) dot, and the
// reference's two fma for 32-block lh = pp (quantized_gemx_kernels.cc:181-188).  kA80: codes count as code - 8,
// no min term (gemv_repack_A80W40, quantized_gemx_kernels.cc:39-109).
template <bool kA80>
__device__ __forceinline__ void consume_block(const BlockLoads& cur, const uint32_t* a, int pp, float (&acc)[4]) {
    const uint4 aql = *reinterpret_cast<const uint4*>(a);
    const uint4 aqh = *reinterpret_cast<const uint4*>(a + 4);
    const float2 par = *reinterpret_cast<const float2*>(a + 8);  // dA_pp, sA_pp
    const uint32_t al[4] = {aql.x, aql.y, aql.z, aql.w};
    const uint32_t ah[4] = {aqh.x, aqh.y, aqh.z, aqh.w};

    int il[4] = {0, 0, 0, 0}, ih[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t w4[4] = {cur.w[j].x, cur.w[j].y, cur.w[j].z, cur.w[j].w};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t lo = w4[c] & 0x0f0f0f0fu;
            const uint32_t hi = (w4[c] >> 4) & 0x0f0f0f0fu;
            il[c] = __builtin_amdgcn_sdot4((int)lo, (int)al[j], il[c], false);
            ih[c] = __builtin_amdgcn_sdot4((int)hi, (int)ah[j], ih[c], false);
        }
    }
    if (kA80) {  // sum((code - 8) q) = sum(code q) - 8 sum(q), over the bytes this lane dotted
        int sl = 0, sh = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            sl = __builtin_amdgcn_sdot4(0x01010101, (int)al[j], sl, false);
            sh = __builtin_amdgcn_sdot4(0x01010101, (int)ah[j], sh, false);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) {
            il[c] -= 8 * sl;
            ih[c] -= 8 * sh;
        }
    }
    const uint32_t sc[2] = {cur.sc.x, cur.sc.y}, mn[2] = {cur.mn.x, cur.mn.y};
#pragma unroll
    for (int c = 0; c < 4; c++) {
        il[c] += dpp_xor2(il[c]);  // exact int32 block dots of columns 4h+c
        ih[c] += dpp_xor2(ih[c]);
        const int idot = pp ? ih[c] : il[c];
        const float dW = f16_bits_to_f32((sc[c >> 1] >> (16 * (c & 1))) & 0xffff);
        const float mW = f16_bits_to_f32((mn[c >> 1] >> (16 * (c & 1))) & 0xffff);
        const float s = __fmul_rn(par.x, dW);
        acc[c] = __fmaf_rn((float)idot, s, acc[c]);
        if (!kA80) acc[c] = __fmaf_rn(mW, par.y, acc[c]);
    }
}

// Sum inside each row of 16 lanes over the lanes that share h: rotate by 8 and 4 (keeps lane % 4), then swap
// the two pp lanes.  Every lane of a row ends up with the row's total for its h.
__device__ __forceinline__ void sum_rows_of_16(float (&acc)[4]) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
        float v = acc[c];
        v += dpp_f<0x128>(v);  // row_ror:8
        v += dpp_f<0x124>(v);  // row_ror:4
        v += dpp_f<kDppXor2>(v);
        acc[c] = v;
    }
}

}  // namespace gemv
}  // namespace a81w41
