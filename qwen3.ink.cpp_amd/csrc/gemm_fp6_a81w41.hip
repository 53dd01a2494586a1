// M > 32 contraction of the layer object: the A81W41 arithmetic on gfx950's block-scaled matrix op
// v_mfma_scale_f32_32x32x64_f8f6f4 in its fp6 (E2M3) mode, which runs at twice the int8 rate.
//
// Why fp6 is exact here.  An E2M3 value with exponent field 0 or 1 is its 4 low bits / 8, so the bit
// pattern s|0|c (sign, a zero, a 4-bit magnitude) is the integer +-c scaled by 1/8: every integer in
// [-15, 15] is an fp6 number.  Weight codes are 0..15.  An int8 activation q = 16*qh + ql with
// qh = q >> 4 in [-8, 7] and ql = q & 15 in [0, 15].  One 64-deep instruction therefore forms the exact
// dot product of one 32-block: lanes 0..31 bring the 32 qh (block scale 2^4), lanes 32..63 the 32 ql,
// against the block's 32 codes on both halves; products and partial sums are integers below 2^24, so
// the fp32 result is float(sum(code*q)) itself -- the value the reference gets from its int32 dot and
// cvtepi32_ps (quantized_gemx_kernels.cc:430-457,509).  No integer-to-float conversion is left for the
// vector ALU (it costs more than the matrix op on this chip, where the two pipes of a SIMD take turns).
// The rest is the reference's epilogue per (row, column, 32-block), in fp32:
//   acc = fma(float(idot), fl(dA*dW), acc)       fl(dA*dW): v_mfma_f32_32x32x1_2b_f32 (exact products, one rounding)
//   acc = fma(mW, sA, acc)                       four 32-blocks at a time on v_mfma_f32_32x32x16_bf16: sA is kept as
//                                                three bf16 pieces (hi + mid + lo = sA exactly), mW as two (16
//                                                significant bits: exact for mins that come from bf16 or fp16 weights),
//                                                and s_hi*w_hi + s_hi*w_lo + s_mid*w_hi + s_lo*w_hi of a block fill
//                                                four of the op's 16 K slots.  Dropped: s_mid*w_lo and s_lo*w_lo, below
//                                                2^-17 of a term, and nothing at all when mW is a bf16 number.
//
// Operand formats (private to the layer object; made once from the reference's blobs):
//   W6: per (32-column panel, 32-block) 1 KiB: chunk 0 = [32 columns][16 B] fp6 codes k = 0..20 (+2 bits),
//       chunk 1 = [32 columns][16 B] rest of the codes (8 B), dW (fp32), mW as two bf16 pieces (hi | lo << 16).
//   A6: per (32-row panel, 32-block) 2 KiB: piece 0 (qh) then piece 1 (ql), each laid out like a W6 panel
//       with dA (fp32) and two of the scaled sum's three bf16 pieces in chunk 1: hi | mid in piece 0's copy, lo in
//       piece 1's (the two lane halves of the contraction kernel exchange them).
// A lane reads its operand with two 16-byte loads; lanes of a half-wave read consecutive 16 bytes.
//
// Tiling: 128 x 256 tiles of C per workgroup, 8 waves of 64 x 64 (two row panels against two column panels),
// one workgroup per CU (two waves per SIMD, up to 256 registers each).  Operands go from memory straight
// into registers, one 32-block ahead of their use; the waves of a workgroup share them through the CU's
// vector cache (a row panel is read by four waves, a column panel by two: three quarters of the loads hit).
// No LDS, no barrier in the loop.  Measured on this chip: data returned into registers -- from LDS or from
// the vector cache alike -- costs the receiving SIMD about 25 clocks per 16 bytes x 64 lanes, on top of its
// matrix and vector ops (about 120 clocks per 32 x 32 x 32 here), and LDS reads do not overlap with matrix
// ops while cache loads do; a first version staged through LDS (direct-to-LDS copies, 128 x 128 tiles, one
// barrier per block) ran 12-18 % slower than this one at every size.
// The (tile, 32-block) work units of a launch are cut into equal
// contiguous runs, one per workgroup (stream-K): a run that covers part of a tile parks a partial tile, an
// arrival counter per split tile tells the last contributor to add the parts in contributor order, so the
// result does not depend on timing.
#include "a81w41_kernels.h"
#include "agent_access.h"
#include "quantize_common.h"

#include <mutex>
#include <type_traits>
#include <vector>

namespace a81w41 {
namespace fp6 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

constexpr int kPanelA = 2048, kPanelB = 1024;  // bytes per (32-row / 32-column panel, 32-block)
constexpr int kThreads = 512;
constexpr int kTileM = 128, kTileN = 256;       // rows and columns of a workgroup's tile
constexpr int kTileWords = kTileM * kTileN;     // fp32 words of a partial tile

// fp6 pattern of an integer in [-15, 15]
__host__ __device__ __forceinline__ uint32_t fp6_of_int(int v) { return v < 0 ? (0x20u | (uint32_t)(-v)) : (uint32_t)v; }

// x as two bf16 pieces, hi | lo << 16: hi = bf16(x), lo = bf16(x - hi), both rounded to nearest even.
__host__ __device__ __forceinline__ uint32_t bf16_rne_bits(float x) {
    union { float f; uint32_t u; } v = {x};
    return (v.u + 0x7fffu + ((v.u >> 16) & 1u)) >> 16;
}
__host__ __device__ __forceinline__ uint32_t split_bf16x2(float x) {
    const uint32_t hi = bf16_rne_bits(x);
    union { uint32_t u; float f; } h = {hi << 16};
    return hi | (bf16_rne_bits(x - h.f) << 16);  // the subtraction is exact
}
// x as three bf16 pieces hi + mid + lo = x exactly (24 significant bits): hi | mid << 16 in .x, lo in .y
__host__ __device__ __forceinline__ uint2 split_bf16x3(float x) {
    const uint32_t hi = bf16_rne_bits(x);
    union { uint32_t u; float f; } h = {hi << 16};
    const float r1 = x - h.f;  // exact
    const uint32_t mid = bf16_rne_bits(r1);
    union { uint32_t u; float f; } m = {mid << 16};
    return make_uint2(hi | (mid << 16), bf16_rne_bits(r1 - m.f));  // what is left has at most 8 significant bits
}

// ---- operand preparation ------------------------------------------------------------------------

// Six dwords of 32 six-bit patterns from the eight 24-bit pieces (4 patterns each) the lanes of a
// group of 8 hold: dword d = bits [32 d, 32 d + 32) of the 192-bit string sum(piece_j << 24 j).
__device__ __forceinline__ void gather_fp6_dwords(uint32_t piece, int lane, uint32_t (&dw)[6]) {
    uint32_t p[8];
    const int base = lane & ~7;
#pragma unroll
    for (int j = 0; j < 8; j++) p[j] = (uint32_t)__shfl((int)piece, base + j, 64);
    dw[0] = p[0] | (p[1] << 24);
    dw[1] = (p[1] >> 8) | (p[2] << 16);
    dw[2] = (p[2] >> 16) | (p[3] << 8);
    dw[3] = p[4] | (p[5] << 24);
    dw[4] = (p[5] >> 8) | (p[6] << 16);
    dw[5] = (p[6] >> 16) | (p[7] << 8);
}

__device__ __forceinline__ uint32_t fp6_piece_of_bytes(uint32_t packed_q, bool high) {
    uint32_t piece = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int q = (int)(int8_t)(packed_q >> (8 * i));
        const int v = high ? (q >> 4) : (q & 15);
        piece |= fp6_of_int(v) << (6 * i);
    }
    return piece;
}

// Stores one 32-block of one row into A6.  The 8 lanes of the group each hold 4 of the block's int8 (packed);
// lanes 0..3 write the four 16-byte chunks (piece = lane >> 1, chunk = lane & 1).
__device__ __forceinline__ void store_a6_block(uint8_t* __restrict__ a6, int row, int blk, int nb, uint32_t packed_q, float d,
                                               float ssum, int lane) {
    uint32_t hi[6], lo[6];
    gather_fp6_dwords(fp6_piece_of_bytes(packed_q, true), lane, hi);
    gather_fp6_dwords(fp6_piece_of_bytes(packed_q, false), lane, lo);
    const int j = lane & 7;
    if (j < 4) {
        const int piece = j >> 1, chunk = j & 1;
        const uint32_t* dw = piece ? lo : hi;
        uint4 v;
        if (chunk == 0) {
            v = make_uint4(dw[0], dw[1], dw[2], dw[3]);
        } else {
            // the scaled sum as three bf16 pieces: hi | mid in the high piece's copy (read by lanes 0..31 of the
            // contraction kernel), lo in the low piece's copy (lanes 32..63)
            const uint2 s3 = split_bf16x3(ssum);
            v = make_uint4(dw[4], dw[5], __float_as_uint(d), piece == 0 ? s3.x : s3.y);
        }
        uint8_t* dst = a6 + ((size_t)(row >> 5) * nb + blk) * kPanelA + piece * 1024 + chunk * 512 + (row & 31) * 16;
        *reinterpret_cast<uint4*>(dst) = v;
    }
}

// fp32 rows -> the reference's 80 B blocks (y80, may be null) and A6; rows M .. rows_padded-1 become zero blocks.
// One float4 per thread, 8 lanes per 32-block (the arithmetic of quantize_row_q8_1_repack_fp32).
template <bool ALIGNED>
__global__ __launch_bounds__(256) void quantize_a6_kernel(const float* __restrict__ x, uint8_t* __restrict__ y80,
                                                          uint8_t* __restrict__ a6, int M, int rows_padded, int K) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one float4 each
    const int per_row = K >> 2;
    const int row = (int)(t / per_row);
    const int c4 = (int)(t - (int64_t)row * per_row);
    const int blk = c4 >> 3, j = c4 & 7;
    const bool in_grid = row < rows_padded, real = row < M;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (real) {
        if (ALIGNED) {
            v = reinterpret_cast<const float4*>(x)[t];
        } else {
            const float* p = x + 4 * t;
            v = make_float4(p[0], p[1], p[2], p[3]);
        }
    }
    const Quant4 qz = quantize_float4_of_block32(v);
    if (!in_grid) return;  // uniform over each group of 8 lanes
    if (real && y80 != nullptr) {
        uint8_t* b80 = y80 + ((size_t)row * (K >> 6) + (blk >> 1)) * kABlock32;
        *reinterpret_cast<uint32_t*>(b80 + 16 + 32 * (blk & 1) + 4 * j) = qz.packed;
        if (j == 0) {
            float* p = reinterpret_cast<float*>(b80);
            p[blk & 1] = qz.d;
            p[2 + (blk & 1)] = qz.ssum;
        }
    }
    store_a6_block(a6, row, blk, K >> 5, qz.packed, qz.d, qz.ssum, threadIdx.x & 63);
}

// 80 B blocks (already quantised rows) -> A6.  Same thread mapping: thread (row, blk, j) takes dword j of the block's int8.
__global__ __launch_bounds__(256) void a80_to_a6_kernel(const uint8_t* __restrict__ y80, uint8_t* __restrict__ a6, int M,
                                                        int rows_padded, int K) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int per_row = K >> 2;
    const int row = (int)(t / per_row);
    const int c4 = (int)(t - (int64_t)row * per_row);
    const int blk = c4 >> 3, j = c4 & 7;
    if (row >= rows_padded) return;
    uint32_t packed = 0;
    float d = 0.f, ssum = 0.f;
    if (row < M) {
        const uint8_t* b80 = y80 + ((size_t)row * (K >> 6) + (blk >> 1)) * kABlock32;
        packed = *reinterpret_cast<const uint32_t*>(b80 + 16 + 32 * (blk & 1) + 4 * j);
        d = reinterpret_cast<const float*>(b80)[blk & 1];
        ssum = reinterpret_cast<const float*>(b80)[2 + (blk & 1)];
    }
    store_a6_block(a6, row, blk, K >> 5, packed, d, ssum, threadIdx.x & 63);
}

// 384 B weight blocks -> W6, one thread per (column, 32-block); columns N .. 32*panels-1 become zero columns.
__global__ __launch_bounds__(256) void w384_to_w6_kernel(const uint8_t* __restrict__ w384, uint8_t* __restrict__ w6, int N,
                                                         int n_padded, int nb) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int n = (int)(t / nb), blk = (int)(t - (int64_t)n * nb);
    if (n >= n_padded) return;
    uint32_t dw[6] = {0, 0, 0, 0, 0, 0};
    float dW = 0.f, mW = 0.f;
    if (n < N) {
        const int g = n >> 3, jj = n & 7, sb = blk >> 1, h = blk & 1;
        const uint8_t* src = w384 + ((size_t)g * (nb >> 1) + sb) * kWBlock32;
        const float* par = reinterpret_cast<const float*>(src);
        dW = par[8 * h + jj];
        mW = par[16 + 8 * h + jj];
        unsigned long long acc = 0;  // bit string under construction
        int filled = 0, out = 0;
#pragma unroll
        for (int p = 0; p < 8; p++) {  // q_coupled[32 p + 4 jj + ii] holds k = 4 p + ii (low nibble) and 32 + 4 p + ii (high)
            const uint32_t w = *reinterpret_cast<const uint32_t*>(src + 128 + 32 * p + 4 * jj);
#pragma unroll
            for (int ii = 0; ii < 4; ii++) {
                const uint32_t code = (w >> (8 * ii + 4 * h)) & 15u;
                acc |= (unsigned long long)code << filled;
                filled += 6;
                if (filled >= 32) {
                    dw[out++] = (uint32_t)acc;
                    acc >>= 32;
                    filled -= 32;
                }
            }
        }
    }
    uint8_t* dst = w6 + ((size_t)(n >> 5) * nb + blk) * kPanelB + (n & 31) * 16;
    *reinterpret_cast<uint4*>(dst) = make_uint4(dw[0], dw[1], dw[2], dw[3]);
    *reinterpret_cast<uint4*>(dst + 512) = make_uint4(dw[4], dw[5], __float_as_uint(dW), split_bf16x2(mW));
}

// ---- the contraction ----------------------------------------------------------------------------

struct Plan {  // one launch: T tiles x nb blocks = U work units, cut into `grid` equal runs
    int tiles_m, tiles_n, nb, grid;
    long long units;
};

__host__ __device__ __forceinline__ long long run_start(const Plan& p, int b) { return p.units * b / p.grid; }
// the workgroup whose run holds unit u
__host__ __device__ __forceinline__ int run_owner(const Plan& p, long long u) { return (int)(((u + 1) * p.grid - 1) / p.units); }

// Operand of one 32 x 32 sub-tile side for one 32-block: 6 dwords of fp6 patterns and two fp32 parameters
// (d and scaled sum of an activation row, or scale and min of a weight column), as read from a panel.
// Dwords 0..5 are the matrix op's operand (a 32 x 6-bit operand occupies six registers; the op does not look at
// the other two), dwords 6 and 7 the two parameters.
typedef v8i Frag;

__device__ __forceinline__ Frag read_frag(const uint8_t* p) {
    const v4i lo = *reinterpret_cast<const v4i*>(p), hi = *reinterpret_cast<const v4i*>(p + 512);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_a81w41_fp6_kernel(
    const uint8_t* __restrict__ A6, const uint8_t* __restrict__ W6, int M, int N, int nb, int tiles_m, int tiles_n,
    int panels_m, int panels_n, long long units, float* __restrict__ C, float* __restrict__ partials,
    unsigned* __restrict__ arrivals) {
    __shared__ unsigned s_arrived;
    const Plan plan = {tiles_m, tiles_n, nb, (int)gridDim.x, units};
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 2, wc = wave & 3;  // this wave's 64 rows (panels 2 wr, 2 wr + 1) x 64 columns (panels 2 wc, 2 wc + 1) of the tile
    const int r = lane & 31, h = lane >> 5;
    // E8M0 block scales: patterns are integers / 8 on both sides (2^3 each); the qh piece counts 16-fold
    const int scale_a = 127 + 3 + 4 * (1 - h), scale_b = 127 + 3;
    const uint32_t lane_a = (uint32_t)h * 1024u + (uint32_t)r * 16u, lane_b = (uint32_t)r * 16u;

    // Workgroups are dealt to the 8 XCDs round robin; run = (XCD, index inside it) makes an XCD's runs
    // neighbours in the unit space, so that the row tiles of a column panel (which share its weights) and
    // the contributors of a split tile meet in one L2.
    const int per_xcd = plan.grid >> 3;
    const int run = (plan.grid & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    const long long u_begin = run_start(plan, run), u_end = run_start(plan, run + 1);
    long long u = u_begin;
    while (u < u_end) {
        const int t = (int)(u / nb), k0 = (int)(u - (long long)t * nb);
        const int k1 = (int)min((long long)nb, (long long)k0 + (u_end - u));
        const int n_steps = k1 - k0;
        const int ty = t % tiles_m, tx = t / tiles_m;

        // Operands come straight from memory into registers (the 8 waves of the workgroup share them through the
        // vector cache): per 32-block, two 16-byte loads per 32 x 32 operand.  Panels past the last one alias it;
        // what is computed from them is never stored.
        const uint8_t* pa[2];
        const uint8_t* pb[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int panel_a = min(kTileM / 32 * ty + 2 * wr + i, panels_m - 1);
            const int panel_b = min(kTileN / 32 * tx + 2 * wc + i, panels_n - 1);
            pa[i] = A6 + ((size_t)panel_a * nb + k0) * kPanelA;  // wave-uniform
            pb[i] = W6 + ((size_t)panel_b * nb + k0) * kPanelB;
        }
        auto load_step = [&](int step, Frag (&fa)[2], Frag (&fb)[2]) {
            const int s = min(step, n_steps - 1);  // past the end the last block is read again
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = read_frag(pa[i] + (size_t)s * kPanelA + lane_a);
                fb[i] = read_frag(pb[i] + (size_t)s * kPanelB + lane_b);
            }
        };

        v16f acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = v16f{0};
        const bool rows_live = kTileM * ty + 64 * wr < M;  // else every row of this wave is past M

        // min terms of up to four 32-blocks (zero pieces where the run ends early): lane half 0 brings blocks 0 and 1,
        // half 1 blocks 2 and 3, four K slots per block: (s_hi, s_hi, s_mid, s_lo) against (w_hi, w_lo, w_hi, w_hi).
        // Lanes 0..31 read hi | mid of a scaled sum, lanes 32..63 its lo: ya = this lane's word for the half's own
        // two blocks, za = its word for the other half's two blocks, which the partner lane (same row, other half)
        // needs; one exchange per block gives every lane all three pieces of its own blocks.
        auto min_terms = [&](const uint32_t (&ya)[2][2], const uint32_t (&za)[2][2], const uint32_t (&yb)[2][2]) {
            v4i opa[2], opb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
#pragma unroll
                for (int k = 0; k < 2; k++) {
                    const uint32_t got = (uint32_t)__shfl_xor((int)za[i][k], 32, 64);
                    const uint32_t himid = h ? got : ya[i][k], lo = h ? ya[i][k] : got;
                    opa[i][2 * k] = (int)__builtin_amdgcn_perm(himid, himid, 0x01000100u);  // hi, hi
                    opa[i][2 * k + 1] = (int)((himid >> 16) | (lo << 16));                       // mid, lo
                    opb[i][2 * k] = (int)yb[i][k];                                                  // hi, lo
                    opb[i][2 * k + 1] = (int)__builtin_amdgcn_perm(yb[i][k], yb[i][k], 0x01000100u);  // hi, hi
                }
            }
            typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
            auto bf = [](const v4i& v) { return __builtin_bit_cast(v8bf, v); };
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf(opa[i]), bf(opb[j]), acc[i][j], 0, 0, 0);
        };

        // one 32-block of the wave's 64 x 64: per row panel the scale products of both column panels in one fp32
        // matrix op (both lane halves bring the rows' d, half j column panel j's scale), then two block dots
        // with 16 fma each
        auto compute = [&](const Frag (&fa)[2], const Frag (&fb)[2]) {
            const v16f z16 = {0};
            const v32f z32 = {0};
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const v32f Sc =
                    __builtin_amdgcn_mfma_f32_32x32x1f32(__int_as_float(fa[i][6]), __int_as_float(h ? fb[1][6] : fb[0][6]), z32, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const v16f P = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], z16, 2, 2, 0, scale_a, 0, scale_b);
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[i][j][v] = __fmaf_rn(P[v], Sc[16 * j + v], acc[i][j][v]);
                }
            }
        };

        if (rows_live) {
            Frag fa[2][2], fb[2][2];  // two sets: the one in use and the next step's, in flight
            load_step(0, fa[0], fb[0]);
            for (int step0 = 0; step0 < n_steps; step0 += 4) {
                uint32_t ya[2][2] = {{0, 0}, {0, 0}}, za[2][2] = {{0, 0}, {0, 0}}, yb[2][2] = {{0, 0}, {0, 0}};
#pragma unroll
                for (int u4 = 0; u4 < 4; u4++) {
                    const int step = step0 + u4;
                    if (step >= n_steps) break;  // uniform over the workgroup
                    load_step(step + 1, fa[(u4 + 1) & 1], fb[(u4 + 1) & 1]);
                    const Frag(&ca)[2] = fa[u4 & 1];
                    const Frag(&cb)[2] = fb[u4 & 1];
                    if ((u4 >> 1) == h) {  // this lane half's block: keep its min-term pieces
#pragma unroll
                        for (int i = 0; i < 2; i++) {
                            ya[i][u4 & 1] = (uint32_t)ca[i][7];
                            yb[i][u4 & 1] = (uint32_t)cb[i][7];
                        }
                    } else {  // the other half's block: the partner lane needs this lane's word of its scaled sums
#pragma unroll
                        for (int i = 0; i < 2; i++) za[i][u4 & 1] = (uint32_t)ca[i][7];
                    }
                    compute(ca, cb);
                }
                min_terms(ya, za, yb);
            }
        }

        // Result registers of sub-tile (i, j): register v, lane (r, h): column 32 j + r, row 32 i + 8 (v/4) + 4 h + v%4.
        const int m_base = kTileM * ty + 64 * wr, n_base = kTileN * tx + 64 * wc;
        auto store_tile = [&](const v16f (&x)[2][2]) {
            if (!rows_live) return;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int n = n_base + 32 * j + r;
                    if (n >= N) continue;
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int m = m_base + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
                        if (m < M) C[(size_t)m * N + n] = x[i][j][v];
                    }
                }
        };

        if (n_steps == nb) {
            store_tile(acc);
        } else {
            // Part of a tile: park it and count arrivals; the contributor that arrives last adds the parts in
            // contributor order.  Partial tiles and counters are accessed at agent scope only, ordered by waiting
            // for the stores and by workgroup barriers.
            const long long tile_u0 = (long long)t * nb;
            const int first = run_owner(plan, tile_u0), last = run_owner(plan, tile_u0 + nb - 1);
            const int b = run;
            const int slot = run_start(plan, b) >= tile_u0 ? 2 * b : 2 * b + 1;
            // element (register quad q, thread) of a partial tile at [slot][q][thread][4]: 4 KiB per wave-wide access
            float* mine = partials + (size_t)slot * kTileWords + 4 * tid;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                        store16_agent(mine + (size_t)(8 * i + 4 * j + q) * 4 * kThreads, v);
                    }
            wait_vmcnt<0>();
            __syncthreads();
            if (tid == 0) s_arrived = atomicAdd(&arrivals[first], 1u);
            __syncthreads();
            if (s_arrived == (unsigned)(last - first)) {
                v16f sum[2][2];
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) sum[i][j] = v16f{0};
                for (int c = first; c <= last; c++) {
                    if (c == b) {  // this workgroup's own part is still in registers: the same values it parked
#pragma unroll
                        for (int i = 0; i < 2; i++)
#pragma unroll
                            for (int j = 0; j < 2; j++) sum[i][j] += acc[i][j];
                        continue;
                    }
                    const int cs = run_start(plan, c) >= tile_u0 ? 2 * c : 2 * c + 1;
                    const float* p = partials + (size_t)cs * kTileWords + 4 * tid;
                    v4f l[16];
#pragma unroll
                    for (int q = 0; q < 16; q++) l[q] = load16_agent(p + (size_t)q * 4 * kThreads);
                    wait_vmcnt<0>();
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int q = 0; q < 16; q++)
#pragma unroll
                        for (int e = 0; e < 4; e++) sum[q >> 3][(q >> 2) & 1][4 * (q & 3) + e] += l[q][e];
                }
                store_tile(sum);
                if (tid == 0) __hip_atomic_store(&arrivals[first], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();  // s_arrived is free again
        }
        u += n_steps;
    }
}

// ---- host side ----------------------------------------------------------------------------------

constexpr int kMaxDevices = 64;
struct Dev {
    int slots = 0;  // resident workgroups (two per CU)
};
Dev g_dev[kMaxDevices];
std::mutex g_mutex;

hipError_t resident_workgroups(int& slots) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_dev[dev].slots == 0) {
        int per_cu = 0, cus = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(&gemm_a81w41_fp6_kernel), kThreads,
                                                         0);
        if (e != hipSuccess) return e;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (per_cu < 1 || cus < 1) return hipErrorInvalidValue;
        g_dev[dev].slots = cus;  // one workgroup (two waves per SIMD) per CU
    }
    slots = g_dev[dev].slots;
    return hipSuccess;
}

// Runs of at least kMinRun blocks (a shorter run is mostly start-up and hand-over), at most one run per
// resident workgroup.
constexpr int kMinRun = 16;
Plan make_plan(int M, int N, int K, int slots) {
    Plan p;
    p.tiles_m = (M + kTileM - 1) / kTileM;
    p.tiles_n = (N + kTileN - 1) / kTileN;
    p.nb = K / 32;
    p.units = (long long)p.tiles_m * p.tiles_n * p.nb;
    long long g = p.units / kMinRun;
    if (g < 1) g = 1;
    if (g > slots) g = slots;
    p.grid = (int)g;
    return p;
}

}  // namespace fp6

using namespace fp6;

bool gemm_fp6_preferred(int M, int N, int K) {
    if (M < kGemmFp6MinRows) return false;
    const int mode = tuning_env_int("A81W41_FP6_MODE");  // tuning builds: 1 = never, 2 = whenever M allows
    if (mode == 1) return false;
    if (mode == 2) return true;
    // Measured crossover on the layer shapes of Qwen3-8B: the block-scaled kernel wins once every CU gets a
    // run of about 48 blocks of 128 x 256 tiles that are mostly live rows; below that its partial tiles
    // (128 KiB each) cost more than the faster matrix op saves.
    const long long units = (long long)((M + kTileM - 1) / kTileM) * ((N + kTileN - 1) / kTileN) * (K / 32);
    return M >= 256 && units >= 12288;
}

size_t gemm_fp6_a6_bytes(int64_t rows, int K) { return (size_t)((rows + 31) / 32) * (size_t)(K / 32) * kPanelA; }
size_t gemm_fp6_w6_bytes(int N, int K) { return (size_t)((N + 31) / 32) * (size_t)(K / 32) * kPanelB; }

hipError_t launch_w384_to_w6(const void* w384, void* w6, int N, int K, hipStream_t s) {
    const int nb = K / 32, n_padded = (N + 31) / 32 * 32;
    const long long threads = (long long)n_padded * nb;
    hipLaunchKernelGGL(w384_to_w6_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, static_cast<const uint8_t*>(w384),
                       static_cast<uint8_t*>(w6), N, n_padded, nb);
    return hipGetLastError();
}

hipError_t launch_quantize_a6(const float* x, void* y80, void* a6, int M, int K, hipStream_t s) {
    const int rows_padded = (M + 31) / 32 * 32;
    const long long threads = (long long)rows_padded * (K / 4);
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0)
        hipLaunchKernelGGL(quantize_a6_kernel<true>, dim3(grid), dim3(256), 0, s, x, static_cast<uint8_t*>(y80),
                           static_cast<uint8_t*>(a6), M, rows_padded, K);
    else
        hipLaunchKernelGGL(quantize_a6_kernel<false>, dim3(grid), dim3(256), 0, s, x, static_cast<uint8_t*>(y80),
                           static_cast<uint8_t*>(a6), M, rows_padded, K);
    return hipGetLastError();
}

hipError_t launch_a80_to_a6(const void* y80, void* a6, int M, int K, hipStream_t s) {
    const int rows_padded = (M + 31) / 32 * 32;
    const long long threads = (long long)rows_padded * (K / 4);
    hipLaunchKernelGGL(a80_to_a6_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, static_cast<const uint8_t*>(y80),
                       static_cast<uint8_t*>(a6), M, rows_padded, K);
    return hipGetLastError();
}

hipError_t launch_gemm_fp6(const void* a6, const void* w6, float* C, int M, int N, int K, const GemmScratch& ws, hipStream_t s) {
    int slots = 0;
    hipError_t e = resident_workgroups(slots);
    if (e != hipSuccess) return e;
    // a run parks at most two partial tiles (its first and its last tile), one counter per run; the scratch is
    // max_partials units of 16 KiB and as many counters: a device with more CUs than the scratch has room for
    // gets fewer, longer runs
    const long long room = (long long)ws.max_partials * 4096 / (2 * kTileWords);
    if (room < 1) return hipErrorInvalidValue;
    if (slots > room) slots = (int)room;
    if (slots > ws.max_partials) slots = ws.max_partials;
    const Plan p = make_plan(M, N, K, slots);
    hipLaunchKernelGGL(gemm_a81w41_fp6_kernel, dim3(p.grid), dim3(kThreads), 0, s, static_cast<const uint8_t*>(a6),
                       static_cast<const uint8_t*>(w6), M, N, p.nb, p.tiles_m, p.tiles_n, (M + 31) / 32, (N + 31) / 32, p.units, C,
                       ws.partials, ws.arrivals);
    return hipGetLastError();
}

// Host-side walk of the work units of a launch (no device): every (tile, block) exactly once, runs contiguous,
// contributor ranges and partial slots consistent between the parking and the merging side.
int gemm_fp6_plan_selfcheck(int M, int N, int K, int slots) {
    const Plan p = make_plan(M, N, K, slots);
    if (p.grid < 1 || p.grid > slots || p.units < 1) return -1;
    const int T = p.tiles_m * p.tiles_n;
    std::vector<int> covered((size_t)T, 0), slot_used((size_t)2 * p.grid, 0), parts((size_t)T, 0);
    long long prev_end = 0;
    for (int b = 0; b < p.grid; b++) {
        const long long u0 = run_start(p, b), u1 = run_start(p, b + 1);
        if (u0 != prev_end || u1 < u0) return -2;
        prev_end = u1;
        for (long long u = u0; u < u1;) {
            if (run_owner(p, u) != b) return -3;
            const int t = (int)(u / p.nb), k0 = (int)(u - (long long)t * p.nb);
            const int k1 = (int)std::min<long long>(p.nb, k0 + (u1 - u));
            covered[t] += k1 - k0;
            if (k1 - k0 != p.nb) {
                const long long tile_u0 = (long long)t * p.nb;
                const int first = run_owner(p, tile_u0), last = run_owner(p, tile_u0 + p.nb - 1);
                if (b < first || b > last || first < 0 || last >= p.grid) return -4;
                const int slot = u0 >= tile_u0 ? 2 * b : 2 * b + 1;
                if (slot_used[slot]++) return -5;
                parts[t]++;
            }
            u += k1 - k0;
        }
    }
    if (prev_end != p.units) return -6;
    int split = 0;
    for (int t = 0; t < T; t++) {
        if (covered[t] != p.nb) return -7;
        if (parts[t]) {
            const long long tile_u0 = (long long)t * p.nb;
            if (parts[t] != run_owner(p, tile_u0 + p.nb - 1) - run_owner(p, tile_u0) + 1) return -8;
            split++;
        }
    }
    return split;
}

}  // namespace a81w41
