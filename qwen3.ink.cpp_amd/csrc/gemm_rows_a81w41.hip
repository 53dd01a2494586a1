// Few-row contraction (M <= 8): C[M][N] = quantised activations (80 B blocks, fp32
// params) x int4 weights (384 B blocks, fp32 params) without the matrix cores.
//
// With so few rows the time is the time to stream the weights once, so this kernel is the
// M = 1 kernel's design with fp32 parameters and MR rows per pass: persistent workgroups keep
// all rows' quantised activations in LDS, a wave consumes 16 consecutive 384 B blocks (6 KiB
// contiguous) per step with 128-bit loads, 4 lanes per block
//   lane = 4*blk + sub,  h = sub & 1 (columns 4h..4h+3),  pp = sub >> 1
// the lane unpacks its four packs pp, pp+2, pp+4, pp+6 once and then, row by row, forms the
// exact int32 partial block dots with v_dot4_i32_i8, merges the two pp lanes with one DPP add
// and applies the reference's epilogue for 32-block lh = pp
//   acc = fma(float(idot), fl(dA*dW), acc);  acc = fma(mW, sA, acc)
// (quantized_gemx_kernels.cc:509-512).  Partial sums are reduced across lanes, then across the
// waves of the column group in a fixed order (deterministic output).
//
// FUSED: the rows come as fp32 and every workgroup quantises them itself on its way into LDS
// (quantize_row_q8_1_repack_fp32, quantized_gemx_kernels.cc:803-911, the same device function as the
// stand-alone quantiser; workgroup 0 also writes the 80 B blocks out, so the caller's scratch holds what
// the reference's buffer would).  One launch instead of two; every workgroup reads M*K*4 bytes of rows, so it
// pays for few rows only (gemm_rows_fused_preferred).
#include "a81w41_kernels.h"
#include "quantize_common.h"

namespace a81w41 {
namespace {

constexpr int kBlocksPerStep = 16;
constexpr int kLdsWordsPerSb = 24;  // per row and super-block: for pp = 0,1: 4 q_low words (packs pp,pp+2,pp+4,pp+6),
                                    // 4 q_high words, dA_pp, sA_pp, 2 pad words
constexpr int kRowsWaves = 8;

__device__ __forceinline__ int lds_q_word(int lh, int p) { return 12 * (p & 1) + 4 * lh + (p >> 1); }

struct RowsLoads {
    uint4 w[4];     // packs pp, pp+2, pp+4, pp+6 (this lane's 4 columns)
    float4 sc, mn;  // scales / mins of 32-block lh = pp, columns 4h..4h+3
};

__device__ __forceinline__ void rows_load(RowsLoads& L, const uint8_t* blk, int sub, bool valid) {
    if (valid) {
        const int h = sub & 1, pp = sub >> 1;
        const uint8_t* q = blk + 128 + 16 * h + 32 * pp;
#pragma unroll
        for (int j = 0; j < 4; j++) L.w[j] = *reinterpret_cast<const uint4*>(q + 64 * j);
        L.sc = *reinterpret_cast<const float4*>(blk + 32 * pp + 16 * h);
        L.mn = *reinterpret_cast<const float4*>(blk + 64 + 32 * pp + 16 * h);
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) L.w[j] = make_uint4(0, 0, 0, 0);
        L.sc = make_float4(0.f, 0.f, 0.f, 0.f);
        L.mn = make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

// Workgroup barrier that orders LDS traffic only: global loads stay in flight (__syncthreads() would
// drain them: loads and stores share one counter).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt = 0; vector-memory and export counters left alone
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

template <int MR, bool FUSED>
__global__ __launch_bounds__(64 * kRowsWaves) void gemm_rows_a81w41_fp32_kernel(const uint8_t* __restrict__ A,
                                                                              const uint8_t* __restrict__ B,
                                                                              float* __restrict__ C, int M, int N,
                                                                              int nb_n, int nb_k, int wpg_log2,
                                                                              uint8_t* __restrict__ a_out) {
    extern __shared__ __align__(16) uint32_t lds[];  // MR*nb_k*24 words of activations, then 2*kRowsWaves*32*MR floats
    constexpr int kThreads = 64 * kRowsWaves;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 3, pp = sub >> 1;
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    const int wpg = 1 << wpg_log2;                    // waves per column group
    const int slots = kRowsWaves >> wpg_log2;         // column groups in flight per workgroup
    const int slot = wave >> wpg_log2, wig = wave & (wpg - 1);
    const int spw = (n_steps + wpg - 1) >> wpg_log2;  // steps per wave per group
    const int blk_in_step = lane >> 2;
    const int g_stride = gridDim.x * slots;

    int gb = blockIdx.x * slots;  // slot 0's group: the loop bound, uniform over the workgroup
    int g = gb + slot, si = 0;
    RowsLoads cur;

    // Activation rows -> LDS images (rows past M are zero: they contribute nothing and are not stored).
    // Loads are requested four per thread at a time, and the first weight blocks right behind the first
    // four: the vector-memory counter retires in order, so whatever is requested first is waited for first.
    auto request_first_weights = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        const int blk = wig * kBlocksPerStep + blk_in_step;
        rows_load(cur, B + ((size_t)g * nb_k + blk) * kWBlock32, sub, g < nb_n && blk < nb_k);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (FUSED) {
        // one float4 per thread and slice, eight lanes per 32-block; row m's blocks follow row m-1's
        const float4* x4 = reinterpret_cast<const float4*>(A);
        const int n_vec = M * nb_k * 16, n_all = MR * nb_k * 16;
        constexpr int kChunk = 4;
        for (int base = 0; base < n_all; base += kChunk * kThreads) {
            float4 v[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_vec) ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            if (base == 0) request_first_weights();
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                if (base + u * kThreads >= n_all) break;  // empty slice (uniform over the workgroup)
                const int i = base + u * kThreads + tid;
                const Quant4 qz = quantize_float4_of_block32(v[u]);  // rows past M: zeros in, zero block out
                if (i < n_all) {
                    const int b32 = i >> 3, p = i & 7, b = b32 >> 1, lh = b32 & 1;  // b = row*nb_k + sb
                    uint32_t* dst = lds + b * kLdsWordsPerSb;
                    dst[lds_q_word(lh, p)] = qz.packed;
                    if (p == 0) {
                        dst[12 * lh + 8] = __float_as_uint(qz.d);
                        dst[12 * lh + 9] = __float_as_uint(qz.ssum);
                    }
                    if (a_out != nullptr && blockIdx.x == 0 && i < n_vec) {
                        uint8_t* ob = a_out + (size_t)b * kABlock32;
                        *reinterpret_cast<uint32_t*>(ob + 16 + 32 * lh + 4 * p) = qz.packed;
                        if (p == 0) {
                            reinterpret_cast<float*>(ob)[lh] = qz.d;
                            reinterpret_cast<float*>(ob)[2 + lh] = qz.ssum;
                        }
                    }
                }
            }
        }
    } else {
        const uint4* A128 = reinterpret_cast<const uint4*>(A);  // five 16-byte pieces per 80 B block
        const int n_pieces = M * nb_k * 5, n_all = MR * nb_k * 5;
        constexpr int kChunk = 4;
        for (int base = 0; base < n_all; base += kChunk * kThreads) {
            uint4 v[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                v[u] = (i < n_pieces) ? A128[i] : make_uint4(0, 0, 0, 0);
            }
            if (base == 0) request_first_weights();
#pragma unroll
            for (int u = 0; u < kChunk; u++) {
                const int i = base + u * kThreads + tid;
                if (i >= n_all) break;
                const int b = i / 5, piece = i - b * 5;  // b = row*nb_k + sb
                uint32_t* dst = lds + b * kLdsWordsPerSb;
                if (piece == 0) {  // dA_low, dA_high, sA_low, sA_high
                    dst[8] = v[u].x;
                    dst[12 + 8] = v[u].y;
                    dst[9] = v[u].z;
                    dst[12 + 9] = v[u].w;
                } else {
                    const int qi = 4 * (piece - 1);  // q words qi..qi+3: 32-block qi >> 3, packs (qi & 7)..+3
                    const int lh = qi >> 3, p0 = qi & 7;
                    dst[lds_q_word(lh, p0)] = v[u].x;
                    dst[lds_q_word(lh, p0 + 1)] = v[u].y;
                    dst[lds_q_word(lh, p0 + 2)] = v[u].z;
                    dst[lds_q_word(lh, p0 + 3)] = v[u].w;
                }
            }
        }
    }
    lds_barrier();  // the images are complete; the first weight blocks may still be on their way

    float* red = reinterpret_cast<float*>(lds + MR * nb_k * kLdsWordsPerSb);
    int parity = 0;
    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[m][c] = 0.f;

    while (gb < nb_n) {  // gb, si advance identically in every wave: uniform over the workgroup
        const int step = wig + si * wpg;
        const int blk = step * kBlocksPerStep + blk_in_step;
        const bool valid = blk < nb_k;
        int ng = g, nsi = si + 1;
        if (nsi == spw) {
            nsi = 0;
            ng = g + g_stride;
        }
        RowsLoads nxt;
        {
            const int nblk = (wig + nsi * wpg) * kBlocksPerStep + blk_in_step;
            rows_load(nxt, B + ((size_t)ng * nb_k + nblk) * kWBlock32, sub, ng < nb_n && nblk < nb_k);
        }

        // unpack once: lo[j][c] / hi[j][c] = the four codes of pack pp+2j, column 4h+c, low / high 32-block
        uint32_t lo[4][4], hi[4][4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t w4[4] = {cur.w[j].x, cur.w[j].y, cur.w[j].z, cur.w[j].w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                lo[j][c] = w4[c] & 0x0f0f0f0fu;
                hi[j][c] = (w4[c] >> 4) & 0x0f0f0f0fu;
            }
        }
        const float dW[4] = {cur.sc.x, cur.sc.y, cur.sc.z, cur.sc.w};
        const float mW[4] = {cur.mn.x, cur.mn.y, cur.mn.z, cur.mn.w};
        const uint32_t* a0 = lds + (valid ? blk : 0) * kLdsWordsPerSb + 12 * pp;
#pragma unroll
        for (int m = 0; m < MR; m++) {
            const uint32_t* a = a0 + m * nb_k * kLdsWordsPerSb;
            const uint4 aql = *reinterpret_cast<const uint4*>(a);
            const uint4 aqh = *reinterpret_cast<const uint4*>(a + 4);
            const float2 par = *reinterpret_cast<const float2*>(a + 8);  // dA_pp, sA_pp
            const uint32_t al[4] = {aql.x, aql.y, aql.z, aql.w};
            const uint32_t ah[4] = {aqh.x, aqh.y, aqh.z, aqh.w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                int il = 0, ih = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    il = __builtin_amdgcn_sdot4((int)lo[j][c], (int)al[j], il, false);
                    ih = __builtin_amdgcn_sdot4((int)hi[j][c], (int)ah[j], ih, false);
                }
                il += dpp_i<kDppXor2>(il);  // exact int32 block dots of column 4h+c
                ih += dpp_i<kDppXor2>(ih);
                const int idot = pp ? ih : il;
                const float s = __fmul_rn(par.x, dW[c]);
                acc[m][c] = __fmaf_rn((float)idot, s, acc[m][c]);
                acc[m][c] = __fmaf_rn(mW[c], par.y, acc[m][c]);
            }
        }
        cur = nxt;

        if (nsi == 0) {  // group finished (uniform over the workgroup)
            // Sum inside each row of 16 lanes over the lanes that share h: rotate by 8 and 4
            // (keeps lane % 4), then swap the two pp lanes; lanes 0 and 1 of each row publish.
            float* r = red + parity * (kRowsWaves * 32 * MR);
#pragma unroll
            for (int m = 0; m < MR; m++) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    float v = acc[m][c];
                    v += dpp_f<0x128>(v);  // row_ror:8
                    v += dpp_f<0x124>(v);  // row_ror:4
                    v += dpp_f<kDppXor2>(v);
                    acc[m][c] = v;
                }
                if ((lane & 15) < 2) {
                    float4* dst = reinterpret_cast<float4*>(r + (wave * MR + m) * 32 + (lane >> 4) * 8 + 4 * (lane & 1));
                    *dst = make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
                }
            }
            lds_barrier();  // not __syncthreads(): the next item's weight blocks stay in flight
            if (tid < 8 * slots * MR) {  // thread (s, m, col) sums slot s's waves and lane rows in order and stores
                const int col = tid & 7, m = (tid >> 3) % MR, s_ = tid / (8 * MR);
                const int gs = gb + s_;
                float v = 0.f;
                for (int w = 0; w < wpg; w++) {
                    const float* rs = r + (((s_ << wpg_log2) + w) * MR + m) * 32 + col;
                    for (int q = 0; q < 4; q++) v += rs[q * 8];
                }
                if (gs < nb_n && m < M) C[(size_t)m * N + gs * 8 + col] = v;
            }
            parity ^= 1;  // this buffer is rewritten only after the next group's barrier
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int c = 0; c < 4; c++) acc[m][c] = 0.f;
            gb += g_stride;
        }
        g = ng;
        si = nsi;
    }
}

template <int MR>
size_t rows_lds_bytes(int K) {
    return ((size_t)MR * (K / 64) * kLdsWordsPerSb + 2 * kRowsWaves * 32 * MR) * sizeof(uint32_t);
}

template <int MR, bool FUSED>
hipError_t launch_rows(const void* A, const void* B, float* C, int M, int N, int K, void* a_out, hipStream_t s) {
    const size_t lds = rows_lds_bytes<MR>(K);
    if (lds > 64 * 1024) {  // a kernel gets 64 KiB of dynamic LDS without asking (asked per call: per device, no shared flag)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_rows_a81w41_fp32_kernel<MR, FUSED>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimitBytes);
        if (e != hipSuccess) return e;
    }
    const int nb_k = K / 64, nb_n = N / 8;
    const int n_steps = (nb_k + kBlocksPerStep - 1) / kBlocksPerStep;
    int wpg_log2 = 0;
    while ((2 << wpg_log2) <= n_steps && (2 << wpg_log2) <= kRowsWaves) wpg_log2++;
    const int slots = kRowsWaves >> wpg_log2;
    const int wgs = (nb_n + slots - 1) / slots;
    const int max_grid = lds * 2 <= (size_t)kLdsLimitBytes ? 512 : 256;  // what the CUs hold at once
    const int grid = wgs < max_grid ? wgs : max_grid;
    hipLaunchKernelGGL((gemm_rows_a81w41_fp32_kernel<MR, FUSED>), dim3(grid), dim3(64 * kRowsWaves), lds, s,
                       static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), C, M, N, nb_n, nb_k, wpg_log2,
                       static_cast<uint8_t*>(a_out));
    return hipGetLastError();
}

template <bool FUSED>
hipError_t launch_rows_any(const void* A, const void* B, float* C, int M, int N, int K, void* a_out, hipStream_t s) {
    switch (M) {
        case 1: return launch_rows<1, FUSED>(A, B, C, M, N, K, a_out, s);
        case 2: return launch_rows<2, FUSED>(A, B, C, M, N, K, a_out, s);
        case 3: return launch_rows<3, FUSED>(A, B, C, M, N, K, a_out, s);
        case 4: return launch_rows<4, FUSED>(A, B, C, M, N, K, a_out, s);
        case 5: return launch_rows<5, FUSED>(A, B, C, M, N, K, a_out, s);
        case 6: return launch_rows<6, FUSED>(A, B, C, M, N, K, a_out, s);
        case 7: return launch_rows<7, FUSED>(A, B, C, M, N, K, a_out, s);
        case 8: return launch_rows<8, FUSED>(A, B, C, M, N, K, a_out, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// One instantiation per row count: the dot products of a row that does not exist would cost as much
// as those of one that does (about 1.2 us per row on the 4096 -> 12288 shape).
bool gemm_rows_fits(int M, int K) {
    if (M < 1 || M > 8) return false;
    const size_t lds = ((size_t)M * (K / 64) * kLdsWordsPerSb + 2 * kRowsWaves * 32 * M) * sizeof(uint32_t);  // rows_lds_bytes<M>
    return lds <= (size_t)kLdsLimitBytes;
}

hipError_t launch_gemm_rows_fp32(const void* A, const void* B, float* C, int M, int N, int K, hipStream_t s) {
    return launch_rows_any<false>(A, B, C, M, N, K, nullptr, s);
}

// Whether the one-launch form (rows quantised by every workgroup) beats quantiser launch + contraction launch.
// Every workgroup reads and quantises all M*K values.  Measured on MI355X (one launch against two, us per call):
// K = 4096, N = 12288: 2 rows 10.9 / 12.2, 3 rows 12.7 / 12.8, 4 rows 14.5 / 13.4, 8 rows 22.5 / 18.4;
// N = 4096: 6.4 / 7.4, 7.6 / 7.8, 8.5 / 8.0; N = 1024: 5.2 / 6.2, 6.5 / 6.7, 7.4 / 7.1; K = 12288: 2 rows 16.9 / 13.0.
bool gemm_rows_fused_preferred(int M, int K) {
    const int mode = tuning_env_int("A81W41_ROWS_FUSED");  // tuning builds: 1 = never, 2 = whenever it fits
    if (mode == 1) return false;
    if (!gemm_rows_fits(M, K)) return false;
    if (mode == 2) return true;
    return (long long)M * K <= 12288;
}

hipError_t launch_gemm_rows_fused(const float* x, void* a_out, const void* B, float* C, int M, int N, int K, hipStream_t s) {
    return launch_rows_any<true>(x, B, C, M, N, K, a_out, s);
}

}  // namespace a81w41
