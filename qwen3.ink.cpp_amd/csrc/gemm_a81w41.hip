// M > 1 contraction: C[M][N] = quantised activations (80 B blocks, fp32 params)
// x int4 weights (384 B blocks, fp32 params) on the gfx950 matrix cores.
//
// Arithmetic per (32 rows x 32 columns x one 64-K super-block), one wave:
//   2 x v_mfma_i32_32x32x32_i8      exact int32 block dots, low and high 32-block
//   1 x v_mfma_f32_32x32x1_2b_f32   the rank-1 scale products fl(dA[m]*dW[n]) of both 32-blocks
//   1 x v_mfma_f32_32x32x2_f32      the min term  mW_low*sA_low + mW_high*sA_high
// and then only cvt + fma per accumulator element on the vector ALU:
//   acc = fma(float(idot), fl(dA*dW), acc)          (quantized_gemx_kernels.cc:509-510)
// The min term accumulates into the same registers through the matrix op's C operand
// (:511-512; the summation order differs from the reference's, covered by the tolerance).
// Matrix-core ops and vector-ALU ops of a SIMD do not overlap in time on this
// chip (measured: their durations add), and cvt + fma per (row, column, 32-block)
// is the floor for per-32 scales on both operands, so the sum of the four matrix
// ops and the 64 vector ops per sub-tile is the budget to approach.
//
// Tiling: 64 x 64 tiles of C, 4 waves of 32 x 32, persistent workgroups, four per CU (124
// registers per lane, 32 KiB of LDS each).  Per super-block a wave reads its operands from LDS, issues
// the four matrix ops and runs their epilogue right behind them, on one set of product registers;
// what it waits for -- LDS, matrix results, the barrier, copies -- the other three waves of its SIMD
// fill.  (Software pipelines over two sets of product registers, which limit a CU to two workgroups,
// were 6-15 % slower; so was operand lookahead at three per CU.)  The K range of the tiles of the
// last, partial round of the grid may be split (see Schedule).  Calls with at most 32 rows go to the
// kernels made for them (gemm_rows_a81w41.hip, gemm_rows32_a81w41.hip); this one serves them only as the
// free-standing fallback of shapes those do not take.
//
// Staging.  Per super-block a workgroup needs
//   A stage: its rows' whole 80 B blocks, row stride 80 B (conflict-free 128-bit reads)
//   B stage: its columns' 384 B weight blocks
// copied global -> LDS by direct-to-LDS loads (global_load_lds_dwordx4: no register
// staging), S stages deep; one s_waitcnt + s_barrier per super-block.  A wave's
// outstanding-load count identifies the stage that has landed, so only real
// copies are ever issued (same count every stage).
//
// Operand layout of the 32x32x32 int8 op: lane l supplies row (or column) l%32 and
// K bytes 16*(l/32)..+15 of the 32-block; both operands use the same split, so
// the pairing of K indices is consistent.  Weight bytes of column 8g+jj, K
// 4p..4p+3 are dword jj of pack p of q_coupled (QwenOperator.cc:835-847); low
// nibbles are the low 32-block, high nibbles the high one; a lane unpacks its
// four dwords into both int8 operands.
// Result lane l, register v: column l%32, row 8*(v/4) + 4*(l/32) + v%4.
#include "a81w41_kernels.h"

#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <vector>

namespace a81w41 {
namespace gemm_detail {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt until at most N vector-memory loads are outstanding and every LDS read this
// wave has issued has returned (gfx9 encoding: vmcnt = bits 3:0 and 15:14, expcnt 6:4 left
// at its maximum, lgkmcnt 11:8 = 0).  The LDS part matters before a barrier after which
// another wave's copy may overwrite the buffer those reads came from.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0070);
}

// One wave-wide direct-to-LDS copy: lane i moves 16 bytes from its own global
// address to lds_base + 16*i (lds_base is wave-uniform).
__device__ __forceinline__ void copy_wave_16B_to_lds(const uint8_t* global_src, uint8_t* lds_base) {
    __builtin_amdgcn_global_load_lds(global_src, (lds_ptr_t)lds_base, 16, 0, 0);
}

constexpr int kTileThreads = 256;
constexpr int kPartialWords = 4096;  // one fp32 partial tile (64 x 64)

// The four waves of a workgroup are 2 x 2 over a 64 x 64 tile.  A stage is 320 activation chunks + 192 weight
// chunks of 16 bytes: two full 64-lane copies per wave.
struct Geom {
    static constexpr int kTileM = 64, kTileN = 64;
    static constexpr int kStageB = kTileM * kABlock32;                    // offset of the B part
    static constexpr int kStage = kStageB + (kTileN / 8) * kWBlock32;     // 8192 bytes
    static constexpr int kCopies = 2;                                     // per wave and stage
    // Stages in LDS; all but one are in flight.  Deeper rings (6 and 8 stages) were measured: no gain.
    static constexpr int kRing = 4;
    static constexpr int kLdsBytes = kRing * kStage;
};

struct TileOps {  // matrix-core operands of one wave for one super-block
    v4i Al, Ah;
    uint32_t w[4];
    float dA, sA, dW, mW;
};
struct TileProd {  // matrix-core results waiting for the vector-ALU epilogue
    v16i Fl, Fh;
    v32f Sc;
};
struct TileDma {
    const uint8_t* base[3];  // wave-uniform: super-block 0 of the tile's rows / column groups
    uint32_t step[3];        // bytes per super-block
    uint32_t voff[3];        // per-lane byte offset from base
    uint32_t lds_off[3];     // wave-uniform offset of the copy inside a stage
};
struct TileRead {     // per-lane LDS byte offsets inside a stage
    uint32_t a;       // the row's 80 B block
    uint32_t dW, mW;  // column's scale / min of 32-block kh
    uint32_t w[4];    // column's four nibble dwords
};

// The B part of a stage holds the eight 384 B blocks of the tile's columns, block gl in 16-byte
// slots 24*gl .. 24*gl+23, with the block's chunks rotated by 2*(gl%4) slots: chunk k sits in
// slot 24*gl + (k + 2*(gl%4)) % 24.  The 32 lanes of a half wave read the same chunk index of
// four consecutive blocks; the rotation spreads those over all 32 LDS banks (unrotated, the
// four blocks would hit the same eight).
__device__ __forceinline__ uint32_t b_slot_byte(int gl, int k, int jj) {
    return Geom::kStageB + (24 * gl + (k + 2 * (gl & 3)) % 24) * 16 + 4 * (jj & 3);
}

// This wave's two direct-to-LDS copies of a stage for super-block sb.
__device__ __forceinline__ void tile_issue(const TileDma& d, uint8_t* lds, int buf, int sb, int lane) {
#pragma unroll
    for (int i = 0; i < Geom::kCopies; i++) {
        // keep the wave-uniform part of the address in scalar registers: saddr + 32-bit lane offset
        const uint64_t ub = reinterpret_cast<uint64_t>(d.base[i]) + (uint64_t)sb * d.step[i];
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)ub);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(ub >> 32));
        const uint8_t* sbase = reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
        copy_wave_16B_to_lds(sbase + d.voff[i], lds + buf * Geom::kStage + d.lds_off[i]);
    }
}

__device__ __forceinline__ void tile_read(TileOps& o, const uint8_t* lds, int buf, const TileRead& rd, int kh) {
    const uint8_t* st = lds + buf * Geom::kStage;
    const uint8_t* row = st + rd.a;
    o.Al = *reinterpret_cast<const v4i*>(row + 16 + 16 * kh);
    o.Ah = *reinterpret_cast<const v4i*>(row + 48 + 16 * kh);
    o.dA = *reinterpret_cast<const float*>(row + 4 * kh);
    o.sA = *reinterpret_cast<const float*>(row + 8 + 4 * kh);
    o.dW = *reinterpret_cast<const float*>(st + rd.dW);
    o.mW = *reinterpret_cast<const float*>(st + rd.mW);
#pragma unroll
    for (int t = 0; t < 4; t++) o.w[t] = *reinterpret_cast<const uint32_t*>(st + rd.w[t]);
}

// The four matrix-core ops of one super-block.
__device__ __forceinline__ void tile_mfma(const TileOps& o, TileProd& F, v16f& acc) {
    const v16i zero16 = {0};
    const v32f zero32 = {0};
    v4i Bl, Bh;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        Bl[t] = (int)(o.w[t] & 0x0f0f0f0fu);
        Bh[t] = (int)((o.w[t] >> 4) & 0x0f0f0f0fu);
    }
    F.Fl = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.Al, Bl, zero16, 0, 0, 0);
    F.Fh = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.Ah, Bh, zero16, 0, 0, 0);
    // registers 0..15: fl(dA*dW) of the low 32-block, 16..31: of the high one
    F.Sc = __builtin_amdgcn_mfma_f32_32x32x1f32(o.dA, o.dW, zero32, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(o.sA, o.mW, acc, 0, 0, 0);  // the min term, straight into the accumulator
}

__device__ __forceinline__ void tile_epilogue(const TileProd& F, v16f& acc) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc[v] = __fmaf_rn((float)F.Fl[v], F.Sc[v], acc[v]);
        acc[v] = __fmaf_rn((float)F.Fh[v], F.Sc[16 + v], acc[v]);
    }
}

// Work list of one launch.  Tiles are numbered so that column panels x = 8*j + c go to the
// workgroups with index = c (mod 8), which share an XCD and its L2, with the row tiles of a
// panel next to each other.  Items [0, whole) are whole tiles; the remaining r tiles (the last,
// partial round of the persistent grid) have their K range cut into c chunks each, item
// whole + ch*r + tr being chunk ch of tile whole + tr.  Workgroup b takes items b, b + grid, ...
// Workgroups are dispatched in index order and the SIMDs favour the older of two resident
// waves, so the low-index workgroups, which get the extra items, are also the faster ones.
struct Schedule {
    int tiles_m, tiles_n;
    int whole, r, c, chunk;
    int items;
    int band;  // row tiles per band (see tile_xy)
};

// Within an XCD (c = tau mod 8) the tiles are walked band by band: `band` row tiles high, all of the
// XCD's column panels wide, row tiles of a panel next to each other.  The workgroups of an XCD that
// run at the same time then share about band rows' activations and 128 / band panels' weights in its
// L2, instead of every row tile's activations against two panels when there are many row tiles.
__host__ __device__ __forceinline__ void tile_xy(int tau, int tiles_m, int tiles_n, int band, int& x, int& y) {
    const int tn8 = tiles_n & ~7, main_tiles = tn8 * tiles_m;
    if (tau < main_tiles) {
        const int c = tau & 7, j = tau >> 3;
        const int npx = tn8 >> 3;                    // column panels per XCD
        const int full = (tiles_m / band) * band;    // rows in full bands
        int y0, h, jj;
        if (j < full * npx) {
            const int b = j / (band * npx);
            y0 = b * band, h = band, jj = j - b * band * npx;
        } else {
            y0 = full, h = tiles_m - full, jj = j - full * npx;
        }
        y = y0 + jj % h;
        x = (jj / h) * 8 + c;
    } else {
        const int e = tau - main_tiles;
        x = tn8 + e / tiles_m;
        y = e % tiles_m;
    }
}

// Wait until stage n (the oldest not yet consumed) has landed for every wave, then refill the
// buffer of stage n-1, which nobody reads any more; kRing-2 stages stay in flight.
#define A81W41_TILE_READY(BUF, SB)                                                  \
    do {                                                                            \
        __builtin_amdgcn_sched_barrier(0); /* nothing above may sink below */      \
        wait_vmcnt<(kRing - 2) * Geom::kCopies>();                                  \
        __builtin_amdgcn_s_barrier();                                               \
        __builtin_amdgcn_sched_barrier(0); /* no LDS read below may rise above */  \
        tile_issue(dma, lds, (BUF), k0 + min((SB), n_sb - 1), lane);                \
    } while (0)

__device__ __forceinline__ void tile_kernel_body(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                 float* __restrict__ C, int M, int N, int nb_k, const Schedule& sc,
                                                 float* __restrict__ partials, unsigned* __restrict__ arrivals, uint8_t* lds,
                                                 unsigned& s_arrived) {
    constexpr int kTileM = Geom::kTileM, kTileN = Geom::kTileN, kRing = Geom::kRing;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, kh = lane >> 5;
    const int nb_n = N >> 3;
    const int row0 = (wave >> 1) * 32, col0 = (wave & 1) * 32;

    TileRead rd;
    {
        rd.a = (row0 + r) * kABlock32;
        const int col = col0 + r, gl = col >> 3, jj = col & 7;
        rd.dW = b_slot_byte(gl, 2 * kh + (jj >> 2), jj);
        rd.mW = b_slot_byte(gl, 4 + 2 * kh + (jj >> 2), jj);
#pragma unroll
        for (int t = 0; t < 4; t++) rd.w[t] = b_slot_byte(gl, 8 + 2 * (4 * kh + t) + (jj >> 2), jj);
    }

    for (int item = blockIdx.x; item < sc.items; item += gridDim.x) {
        int tau, k0, n_sb, part = -1;  // part >= 0: index of this item's partial tile
        if (item < sc.whole) {
            tau = item;
            k0 = 0;
            n_sb = nb_k;
        } else {
            const int k = item - sc.whole;
            const int tr = k % sc.r, ch = k / sc.r;
            tau = sc.whole + tr;
            k0 = ch * sc.chunk;
            n_sb = sc.chunk;
            part = tr * sc.c + ch;
        }
        int tx, ty;
        tile_xy(tau, sc.tiles_m, sc.tiles_n, sc.band, tx, ty);
        const int m_base = ty * kTileM, n_base = tx * kTileN;

        // Copy q = i*4 + wave of a stage moves chunks 64q..64q+63: copies 0..4 are activation rows (5 chunks per
        // row), 5..7 weight blocks.  Rows past M alias the last row and column groups past N the last group;
        // neither is ever stored.
        TileDma dma;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = i * 4 + wave;
            const int c = q * 64 + lane;
            dma.lds_off[i] = q * 1024;
            if (q < 5) {
                const int row = c / 5, piece = c - row * 5;
                const int m_rel = min(m_base + row, M - 1) - m_base;
                dma.base[i] = A + (size_t)m_base * nb_k * kABlock32;
                dma.step[i] = kABlock32;
                dma.voff[i] = (uint32_t)m_rel * nb_k * kABlock32 + 16 * piece;
            } else {
                const int s = c - 320;
                const int gl = s / 24, pos = s - gl * 24;
                const int k = (pos - 2 * (gl & 3) + 24) % 24;  // slot pos of block gl holds chunk k
                const int g_rel = min((n_base >> 3) + gl, nb_n - 1) - (n_base >> 3);
                dma.base[i] = B + (size_t)(n_base >> 3) * nb_k * kWBlock32;
                dma.step[i] = kWBlock32;
                dma.voff[i] = (uint32_t)g_rel * nb_k * kWBlock32 + 16 * k;
            }
        }

        v16f acc = {0};
        const bool wave_live = m_base + row0 < M;  // else: rows all past M

        // Stage n lives in buffer n % kRing; past the chunk's end its last super-block is copied
        // again, which keeps the per-wave load count uniform (never used).  READY number n makes
        // stage n visible and refills the buffer of stage n-1, which every wave has read by then (the
        // wait in front of the barrier covers its LDS reads).  A step is: operands from LDS, the four
        // matrix ops, their epilogue -- one set of product registers and no lookahead, so that four
        // workgroups fit a CU; what a wave waits for (LDS, matrix results, the barrier, copies) the
        // other three waves of its SIMD fill.
#pragma unroll
        for (int st = 0; st < kRing - 1; st++) tile_issue(dma, lds, st, k0 + min(st, n_sb - 1), lane);
        if (wave_live) {
            for (int t = 0; t < n_sb; t += kRing) {
#pragma unroll
                for (int p = 0; p < kRing; p++) {
                    const int u = t + p;
                    A81W41_TILE_READY((p + kRing - 1) % kRing, u + kRing - 1);
                    if (u < n_sb) {
                        TileOps o;
                        TileProd F;
                        tile_read(o, lds, p, rd, kh);
                        tile_mfma(o, F, acc);
                        tile_epilogue(F, acc);
                    }
                }
            }
        } else {  // only keep the copy ring and the barriers going
            for (int t = 0; t < n_sb; t += kRing) {
#pragma unroll
                for (int p = 0; p < kRing; p++) A81W41_TILE_READY((p + kRing - 1) % kRing, t + p + kRing - 1);
            }
        }
        wait_vmcnt<0>();  // the tail copies have landed: the ring can be reused

        const int n = n_base + col0 + r;
        const int m0 = m_base + row0;
        if (part < 0) {
            if (wave_live && n < N) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + 8 * (v >> 2) + 4 * kh + (v & 3);
                    if (m < M) C[(size_t)m * N + n] = acc[v];
                }
            }
            __syncthreads();  // every wave is done with the ring
        } else {
            // K-split tile: park this chunk's partial tile and count arrivals; the last workgroup to
            // arrive adds the chunks in chunk order, so the result does not depend on who is last.
            // Partial tiles and counters are accessed only with agent-scope relaxed atomics, which
            // are coherent across the XCDs' L2s on their own; they are ordered by waiting for the
            // stores and by the workgroup barriers, so no L2-wide write-back or invalidate is needed.
            // 8-byte element v of thread tid sits at [part][v][tid]: 512 contiguous bytes per wave.
            unsigned long long* mine = reinterpret_cast<unsigned long long*>(partials) + (size_t)part * (kPartialWords / 2) + tid;
#pragma unroll
            for (int v = 0; v < 8; v++) {
                const float lo = acc[2 * v], hi = acc[2 * v + 1];
                const unsigned long long bits = ((unsigned long long)__float_as_uint(hi) << 32) | __float_as_uint(lo);
                __hip_atomic_store(mine + v * kTileThreads, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            wait_vmcnt<0>();
            __syncthreads();
            const int tr = part / sc.c;
            if (tid == 0) s_arrived = atomicAdd(&arrivals[tr], 1u);
            __syncthreads();
            if (s_arrived == (unsigned)(sc.c - 1)) {
                float sum[16];
#pragma unroll
                for (int v = 0; v < 16; v++) sum[v] = 0.f;
                for (int ch = 0; ch < sc.c; ch++) {
                    unsigned long long* p = reinterpret_cast<unsigned long long*>(partials) + (size_t)(tr * sc.c + ch) * (kPartialWords / 2) + tid;
                    unsigned long long bits[8];
#pragma unroll
                    for (int v = 0; v < 8; v++)
                        bits[v] = __hip_atomic_load(p + v * kTileThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int v = 0; v < 8; v++) {
                        sum[2 * v] += __uint_as_float((unsigned)bits[v]);
                        sum[2 * v + 1] += __uint_as_float((unsigned)(bits[v] >> 32));
                    }
                }
                if (wave_live && n < N) {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int m = m0 + 8 * (v >> 2) + 4 * kh + (v & 3);
                        if (m < M) C[(size_t)m * N + n] = sum[v];
                    }
                }
                // back to zero for the next launch that uses this scratch
                if (tid == 0) __hip_atomic_store(&arrivals[tr], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();  // s_arrived and the ring are free again
        }
    }
}
#undef A81W41_TILE_READY

// The operands and the schedule come first, as scalars: those 14 dwords are in registers when a wave starts
// (kernel-argument preloading), so the first copies do not wait for a load from the argument buffer; C and the
// split scratch, needed at the end of a tile only, follow.
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_a81w41_tile64_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int nb_k, int tiles_m, int tiles_n, int whole,
    int r, int c, int chunk, int band, float* __restrict__ C, float* __restrict__ partials, unsigned* __restrict__ arrivals) {
    extern __shared__ __align__(16) uint8_t lds[];  // kRing stages
    __shared__ unsigned s_arrived;
    const Schedule sc = {tiles_m, tiles_n, whole, r, c, chunk, whole + r * c, band};
    tile_kernel_body(A, B, C, M, N, nb_k, sc, partials, arrivals, lds, s_arrived);
}

// ---- scratch of the K-split path --------------------------------------------------------------
// A scratch is `max_partials` partial tiles of kPartialWords floats plus as many arrival counters, which
// are zero between launches.  Launches that share a scratch must not overlap in time, so every owner
// has its own: a context (all of its layers' calls), a stream (the free-standing GEMM entry point: calls
// on one stream are ordered by the stream, calls on different streams get different scratches), or the
// file-scope array below for the entry point that may not allocate.
constexpr int kMaxPartials = 4096;  // room for every tile of a launch that does not fill the chip to be cut in four
constexpr int kMaxDevices = 64;
constexpr int kMaxStreamsPerDevice = 16;  // scratches kept per device; a further stream takes over the least recently used one

// Static scratch of the allocation-free entry point: 2048 partial tiles (32 MiB) and their counters per
// device, held from the moment the code object is loaded until the process ends.
constexpr int kStaticPartials = 2048;
struct __align__(256) StaticScratch {
    float partials[(size_t)kStaticPartials * kPartialWords];
    unsigned arrivals[kStaticPartials];
};
static __device__ __align__(256) StaticScratch scratch;

struct DeviceInfo {
    int slots = 0;  // workgroups of the tile kernels the device holds at once (four per CU)
    int cus = 0;
    StaticScratch* static_scratch = nullptr;  // this device's copy of `scratch`
    struct {
        hipStream_t stream;
        GemmScratch ws;
        unsigned long long last_use;
    } by_stream[kMaxStreamsPerDevice];
    int n_streams = 0;
    unsigned long long uses = 0;
};
DeviceInfo g_dev[kMaxDevices];
std::mutex g_dev_mutex;

// Occupancy and CU count of the current device (queried once per device); g_dev_mutex held.
hipError_t device_info_locked(DeviceInfo*& out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    DeviceInfo& d = g_dev[dev];
    if (d.slots == 0) {
        int per_cu = 0, cus = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(&gemm_a81w41_tile64_kernel),
                                                         kTileThreads, Geom::kLdsBytes);
        if (e != hipSuccess) return e;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (per_cu < 1 || cus < 1) return hipErrorInvalidValue;
        d.cus = cus;
        d.slots = per_cu * cus;
    }
    out = &d;
    return hipSuccess;
}

__global__ void clear_counters_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// The schedule of one launch (see Schedule): a pure function of the shape and of the device's size.
// Returns false when the K split the shape calls for needs more than max_partials partial tiles.
bool make_schedule(int M, int N, int K, int slots_fit, int cus, int max_partials, Schedule& sc, int& grid) {
    const int nb_k = K / 64;
    sc.tiles_m = (M + Geom::kTileM - 1) / Geom::kTileM;
    sc.tiles_n = (N + Geom::kTileN - 1) / Geom::kTileN;
    const int T = sc.tiles_m * sc.tiles_n;
    // The kernels fit four workgroups per CU; how many the schedule counts on depends on the number of
    // tiles T per CU (measured at N = 4096, M = 128..1536): up to 2 per CU, four (finer K split over
    // more workgroups); up to 2.67, two (one round of two-per-CU tiles plus a split remainder beats a
    // sparse round of slower ones: 640 rows 144 against 155 us); up to 4, three (832 rows 179 against
    // 201 us); from 4 on, four.
    const int fit = slots_fit / cus;
    int per_cu = fit;
    if (T > 2 * cus && T < 4 * cus) per_cu = 3 * T <= 8 * cus ? 2 : 3;
    if (per_cu > fit) per_cu = fit;
    const int env_per_cu = tuning_env_int("A81W41_GEMM_PER_CU");
    if (env_per_cu >= 1 && env_per_cu <= fit) per_cu = env_per_cu;
    const int slots = per_cu * cus;
    sc.whole = (T / slots) * slots;
    sc.r = T - sc.whole;
    // Split the last, partial round: in two, so that the chunks go to the first (faster) half
    // of the grid; in four when even then less than 3/4 of the grid would have one.
    int c = 1;
    auto valid = [&](int cc) { return cc >= 1 && cc <= 16 && nb_k % (Geom::kRing * cc) == 0 && (long long)sc.r * cc <= kMaxPartials; };
    if (sc.r > 0) {
        if (valid(2)) c = 2;
        if (valid(4) && sc.r * 4 <= slots * 3 / 4) c = 4;
        // a launch that does not fill the chip once, over a long K: quarters still leave 48 steps per chunk
        // (down_proj at 322 rows: 75.6 against 79.8 us)
        if (valid(4) && sc.whole == 0 && nb_k / 4 >= 48) c = 4;
        const int env_c = tuning_env_int("A81W41_GEMM_SPLIT");
        if (env_c > 0 && valid(env_c)) c = env_c;
    }
    if (c == 1) {
        sc.whole = T;
        sc.r = 0;
    }
    // Bands of 4 row tiles: neutral up to 16 row tiles, 5-8 % faster from 24 on (gate at 4096 rows: 860 -> 807 us;
    // 2, 3, 6 and 8 measured the same within noise).
    sc.band = sc.tiles_m < 4 ? sc.tiles_m : 4;
    const int env_band = tuning_env_int("A81W41_GEMM_BAND");
    if (env_band > 0) sc.band = env_band < sc.tiles_m ? env_band : sc.tiles_m;
    sc.c = c;
    sc.chunk = nb_k / c;
    sc.items = sc.whole + sc.r * c;
    grid = sc.items < slots ? sc.items : slots;
    return sc.r * c <= max_partials;
}

hipError_t launch_tiles(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws, hipStream_t s) {
    DeviceInfo* d = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_dev_mutex);
        const hipError_t e = device_info_locked(d);
        if (e != hipSuccess) return e;
    }
    Schedule sc;
    int grid = 0;
    if (!make_schedule(M, N, K, d->slots, d->cus, ws.max_partials, sc, grid)) return hipErrorInvalidValue;
    const int nb_k = K / 64;
    hipLaunchKernelGGL(gemm_a81w41_tile64_kernel, dim3(grid), dim3(kTileThreads), Geom::kLdsBytes, s,
                       static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), M, N, nb_k, sc.tiles_m, sc.tiles_n, sc.whole,
                       sc.r, sc.c, sc.chunk, sc.band, C, ws.partials, ws.arrivals);
    return hipGetLastError();
}

// Which kernel a call goes to: 0 the few-row kernel (no scratch), 2 the 64 x 64 tiles, and for 9 .. 32 rows the
// one-row-panel kernel: 3 with its operands loaded straight into registers, 4 with wave-private LDS stages.
int pick_kernel(int M, int N, int K) {
    // Measurement aids (tuning builds): A81W41_GEMM_TUNE=tile keeps few-row calls off the few-row kernel,
    // A81W41_GEMM_TUNE=Tile64 keeps every call on the 64 x 64 tiles.
    const char* tune_s = tuning_env("A81W41_GEMM_TUNE");
    const char tune = tune_s ? tune_s[0] : '\0';
    const bool tile_only = tune == 't' || tune == 'T';
    // 7 and 8 rows over a long K on a wide layer: the few-row kernel's time grows by 1.4 us per row there (down_proj:
    // 19.3 and 20.7 us forward) and passes the one-row-panel kernel's 18 us
    const bool long_k_rows = M >= 7 && K >= 8192 && N > 2048;
    if (!tile_only && gemm_rows_fits(M, K) && !long_k_rows) return 0;
    if (M > 32 || tune == 'T') return 2;
    // At most 32 rows: such a call is bound by streaming the weights once, and 64 x 64 tiles (or 32 x 128 ones, an
    // arrangement this file used to have) cut K 8- to 16-fold between workgroups, whose last arriver's merge then
    // dominates; the one-row-panel kernel cuts K inside the workgroup.  Forward at 9 .. 32 rows, us, against the
    // 32 x 128 tiles: N = 1024, K = 4096 8.9 against 14.1 (registers; staged 9.3); gate_proj 18.0 .. 18.6 against
    // 20.2 .. 21.5 and down_proj 17.9 .. 18.3 against 22.9 .. 23.2 (staged; with register loads gate_proj at 32 rows
    // took 32: nine load instructions per wave and super-block on the CU's cache path).
    const int rows32_mode = tuning_env_int("A81W41_GEMM_ROWS32");         // tuning builds: 1 always registers, 2 never
    const int staged_mode = tuning_env_int("A81W41_GEMM_ROWS32_STAGED");  // tuning builds: 1 always staged, 2 never
    if (staged_mode == 1) return 4;
    if (rows32_mode == 1) return 3;
    if (N <= 2048 && rows32_mode != 2) return 3;
    if (staged_mode != 2) return 4;
    return 2;
}

}  // namespace gemm_detail

using namespace gemm_detail;

const char* gemm_kernel_name(int M, int N, int K) {
    switch (pick_kernel(M, N, K)) {
        case 0: return "rows (2..8 rows resident in LDS, v_dot4, weights streamed once)";
        case 3: return "rows32 (int8 matrix ops, one row panel, K split inside the workgroup)";
        case 4: return "rows32_staged (int8 matrix ops, one row panel, K split inside the workgroup, wave-private LDS stages)";
        default: return "tile64 (int8 matrix ops, 64 x 64 tiles, LDS-staged)";
    }
}

bool gemm_rows32_staged_preferred(int M, int N, int K) { return M >= 2 && pick_kernel(M, N, K) == 4; }

hipError_t gemm_scratch_create(GemmScratch* out) {
    out->partials = nullptr;
    out->arrivals = nullptr;
    out->max_partials = 0;
    float* p = nullptr;
    unsigned* a = nullptr;
    hipError_t e = hipMalloc(&p, (size_t)kMaxPartials * kPartialWords * sizeof(float));
    if (e != hipSuccess) return e;
    e = hipMalloc(&a, kMaxPartials * sizeof(unsigned));
    if (e == hipSuccess) e = hipMemset(a, 0, kMaxPartials * sizeof(unsigned));
    if (e != hipSuccess) {
        (void)hipFree(p);
        (void)hipFree(a);
        return e;
    }
    out->partials = p;
    out->arrivals = a;
    out->max_partials = kMaxPartials;
    return hipSuccess;
}

size_t gemm_scratch_bytes(const GemmScratch& ws) {
    return (size_t)ws.max_partials * (kPartialWords * sizeof(float) + sizeof(unsigned));
}

void gemm_scratch_destroy(GemmScratch* ws) {
    (void)hipFree(ws->partials);
    (void)hipFree(ws->arrivals);
    ws->partials = nullptr;
    ws->arrivals = nullptr;
    ws->max_partials = 0;
}

hipError_t gemm_scratch_for_stream(hipStream_t s, GemmScratch* out) {
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    DeviceInfo* d = nullptr;
    hipError_t e = device_info_locked(d);
    if (e != hipSuccess) return e;
    for (int i = 0; i < d->n_streams; i++)
        if (d->by_stream[i].stream == s) {
            d->by_stream[i].last_use = ++d->uses;
            *out = d->by_stream[i].ws;
            return hipSuccess;
        }
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    e = hipStreamIsCapturing(s, &cap);
    if (e != hipSuccess) return e;
    if (cap != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;  // cannot allocate or wait under capture
    if (d->n_streams == kMaxStreamsPerDevice) {
        // Every scratch is taken: the stream that used its own longest ago (it may not even exist any more) hands it
        // over.  Work that still uses it may be in flight, so the device is drained first; the counters are zero
        // between launches, so nothing needs clearing.
        e = hipDeviceSynchronize();
        if (e != hipSuccess) return e;
        int lru = 0;
        for (int i = 1; i < d->n_streams; i++)
            if (d->by_stream[i].last_use < d->by_stream[lru].last_use) lru = i;
        d->by_stream[lru].stream = s;
        d->by_stream[lru].last_use = ++d->uses;
        *out = d->by_stream[lru].ws;
        return hipSuccess;
    }
    GemmScratch ws;
    e = gemm_scratch_create(&ws);
    if (e != hipSuccess) return e;
    d->by_stream[d->n_streams].stream = s;
    d->by_stream[d->n_streams].ws = ws;
    d->by_stream[d->n_streams].last_use = ++d->uses;
    d->n_streams++;
    *out = ws;
    return hipSuccess;
}

hipError_t gemm_static_scratch(GemmScratch* out) {
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    DeviceInfo* d = nullptr;
    hipError_t e = device_info_locked(d);
    if (e != hipSuccess) return e;
    if (d->static_scratch == nullptr) {
        // `scratch` names the array for the host compiler only; its address on the current device comes from here
        StaticScratch* ptr = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        d->static_scratch = ptr;
    }
    out->partials = d->static_scratch->partials;
    out->arrivals = d->static_scratch->arrivals;
    out->max_partials = kStaticPartials;
    return hipSuccess;
}

int gemm_static_scratch_tiles() { return kStaticPartials; }

int gemm_partial_tiles(int M, int N, int K) {
    const int kernel = pick_kernel(M, N, K);
    if (kernel == 0) return 0;
    if (kernel == 3 || kernel == 4) {  // a share of a column panel parks 4 KiB, a quarter of a partial-tile unit
        const int split = gemm_rows32_split(N, K, kernel == 4);
        return split > 1 ? ((N + 31) / 32 * split + 3) / 4 : 0;
    }
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    DeviceInfo* d = nullptr;
    if (device_info_locked(d) != hipSuccess) return -1;
    Schedule sc;
    int grid = 0;
    make_schedule(M, N, K, d->slots, d->cus, kMaxPartials, sc, grid);
    return sc.r * sc.c;
}

hipError_t clear_gemm_counters(const GemmScratch& ws, hipStream_t s) {
    const int n = ws.max_partials;
    hipLaunchKernelGGL(clear_counters_kernel, dim3((n + 255) / 256), dim3(256), 0, s, ws.arrivals, n);
    return hipGetLastError();
}

hipError_t launch_gemm_fp32(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws, hipStream_t s) {
    switch (pick_kernel(M, N, K)) {
        case 0: return launch_gemm_rows_fp32(A, B, C, M, N, K, s);
        case 3: return launch_gemm_rows32_fp32(A, B, C, M, N, K, ws, s);
        case 4: return launch_gemm_rows32_fp32(A, B, C, M, N, K, ws, s, true);
        default: return launch_tiles(A, B, C, M, N, K, ws, s);
    }
}

// Host-side check of the work list a launch would walk (no device needed): every whole tile once, every
// chunk of every split tile once, partial-tile indices distinct and below the scratch size.
int gemm_schedule_selfcheck(int M, int N, int K, int slots_fit, int cus) {
    Schedule sc;
    int grid = 0;
    if (!make_schedule(M, N, K, slots_fit, cus, kMaxPartials, sc, grid)) return -1;
    const int T = sc.tiles_m * sc.tiles_n, nb_k = K / 64;
    if (sc.whole + sc.r != T || sc.items != sc.whole + sc.r * sc.c || sc.chunk * sc.c != nb_k) return -2;
    if (grid < 1 || grid > slots_fit) return -3;
    std::vector<int> covered((size_t)T, 0), part_used((size_t)kMaxPartials, 0);
    for (int b = 0; b < grid; b++)
        for (int item = b; item < sc.items; item += grid) {
            if (item < sc.whole) {
                covered[item] += nb_k;
            } else {
                const int k = item - sc.whole, tr = k % sc.r, ch = k / sc.r, part = tr * sc.c + ch;
                if (part < 0 || part >= kMaxPartials || part_used[part]++) return -4;
                if (ch * sc.chunk + sc.chunk > nb_k) return -5;
                covered[sc.whole + tr] += sc.chunk;
            }
        }
    for (int t = 0; t < T; t++)
        if (covered[t] != nb_k) return -6;
    // the tile numbering is one-to-one onto the tiles
    std::vector<int> seen((size_t)T, 0);
    for (int tau = 0; tau < T; tau++) {
        int x = -1, y = -1;
        tile_xy(tau, sc.tiles_m, sc.tiles_n, sc.band, x, y);
        if (x < 0 || x >= sc.tiles_n || y < 0 || y >= sc.tiles_m || seen[(size_t)y * sc.tiles_n + x]++) return -7;
    }
    return sc.r * sc.c;
}

}  // namespace a81w41
