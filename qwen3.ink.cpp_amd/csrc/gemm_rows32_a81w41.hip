// 9 .. 32-row contraction on the reference's blobs (80 B activation blocks, 384 B weight blocks): one 32-row
// panel against every 32-column panel.  Such a call is bound by streaming the weights once, so the work is cut
// for memory parallelism, not for operand reuse: a workgroup of four waves owns (column panel, share of K), its
// waves cut the share in four, and every wave loads its operands straight from memory into registers, kDepth
// super-blocks ahead of their use -- no LDS staging, no barrier in the loop, 12 waves per CU with about 5 KB of
// weights in flight each.  The four results of a workgroup meet in LDS; where K is shared between workgroups the
// shares are parked and counted, and whoever arrives last adds them in share order (deterministic), with the
// same agent-scope hand-over as the tile kernels.
//
// Arithmetic per (32 rows x 32 columns x one 64-K super-block), the reference's per (row, column, 32-block)
// (quantized_gemx_kernels.cc:430-457,509-520): two v_mfma_i32_32x32x32_i8 give the exact int32 block dots (low
// and high 32-block), one v_mfma_f32_32x32x1_2b_f32 the scale products fl(dA dW) of both blocks, one
// v_mfma_f32_32x32x2_f32 adds mW_low sA_low + mW_high sA_high into the accumulator, and the vector ALU does
// acc = fma(float(idot), fl(dA dW), acc) for both blocks.
// Operand placement: lane (r, h) = (lane & 31, lane >> 5).  The matrix op sums over (h, byte j) of its two
// operands, so any assignment of k to (h, j) works that both sides share; here k = 16 h + j inside a 32-block.
// The activation side is then 16 contiguous int8 of row r, the weight side the four dwords
// q_coupled[32 (4 h + m) + 4 jj ..] (m = 0..3) of column 8 g + jj, whose low / high nibbles are the codes of the
// low / high 32-block at those same k.
#include "a81w41_kernels.h"
#include "agent_access.h"

namespace a81w41 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

constexpr int kThreads = 256;
constexpr int kDepth = 3;       // super-blocks of operands in flight per wave
constexpr int kMaxSplit = 6;    // shares of K per column panel (each costs the last arriver one trip to memory)
constexpr int kTargetGroups = 768;

struct Operands {  // of one lane for one super-block
    v4i a_low, a_high;   // 16 int8 of the row's low / high 32-block
    v4i a_par;           // d_low, d_high, scaled_sum_low, scaled_sum_high (fp32 bits)
    uint32_t w[4];       // coupled codes: low nibbles = low block, high nibbles = high block
    float dw_low, dw_high, mw_low, mw_high;
};

__device__ __forceinline__ Operands load_operands(const uint8_t* __restrict__ a_row, const uint8_t* __restrict__ b_col, int sb,
                                                  int h) {
    Operands o;
    const uint8_t* ab = a_row + (size_t)sb * kABlock32;
    o.a_par = *reinterpret_cast<const v4i*>(ab);
    o.a_low = *reinterpret_cast<const v4i*>(ab + 16 + 16 * h);
    o.a_high = *reinterpret_cast<const v4i*>(ab + 48 + 16 * h);
    const uint8_t* bb = b_col + (size_t)sb * kWBlock32;  // already offset by 4 jj
    const float* par = reinterpret_cast<const float*>(bb);
    o.dw_low = par[0];
    o.dw_high = par[8];
    o.mw_low = par[16];
    o.mw_high = par[24];
#pragma unroll
    for (int m = 0; m < 4; m++) o.w[m] = *reinterpret_cast<const uint32_t*>(bb + 128 + 128 * h + 32 * m);
    return o;
}

__global__ __launch_bounds__(kThreads) void gemm_a81w41_rows32_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                     int M, int N, int nbk, int split, float* __restrict__ C,
                                                                     float* __restrict__ partials,
                                                                     unsigned* __restrict__ arrivals) {
    __shared__ __align__(16) float s_part[4][1024];  // [wave][register v][lane]
    __shared__ unsigned s_arrived;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int panel = (int)blockIdx.x / split, share = (int)blockIdx.x - panel * split;
    const int s_lo = (int)((long long)nbk * share / split), s_hi = (int)((long long)nbk * (share + 1) / split);
    const int k_lo = s_lo + (s_hi - s_lo) * wave / 4, k_hi = s_lo + (s_hi - s_lo) * (wave + 1) / 4;
    const int n_steps = k_hi - k_lo;
    // rows past M and columns past N alias the last real one; what is computed from them is never stored
    const int row = min(r, M - 1), col = min(32 * panel + r, N - 1);
    const uint8_t* a_row = A + ((size_t)row * nbk + k_lo) * kABlock32;
    const uint8_t* b_col = B + ((size_t)(col >> 3) * nbk + k_lo) * kWBlock32 + 4 * (col & 7);

    v16f acc = {0};
    if (n_steps > 0) {
        Operands ring[kDepth];
#pragma unroll
        for (int d = 0; d < kDepth - 1; d++) ring[d] = load_operands(a_row, b_col, min(d, n_steps - 1), h);
        for (int step0 = 0; step0 < n_steps; step0 += kDepth) {
#pragma unroll
            for (int u = 0; u < kDepth; u++) {
                const int step = step0 + u;
                if (step >= n_steps) break;  // uniform over the wave
                // past the end of the wave's range the last super-block is read again
                ring[(u + kDepth - 1) % kDepth] = load_operands(a_row, b_col, min(step + kDepth - 1, n_steps - 1), h);
                const Operands& o = ring[u];
                v4i b_low, b_high;
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    b_low[m] = (int)(o.w[m] & 0x0f0f0f0fu);
                    b_high[m] = (int)((o.w[m] >> 4) & 0x0f0f0f0fu);
                }
                const v16i zi = {0};
                const v32f z32 = {0};
                const v16i i_low = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a_low, b_low, zi, 0, 0, 0);
                const v16i i_high = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a_high, b_high, zi, 0, 0, 0);
                // lane half h brings block h's parameters: registers 0..15 = low block, 16..31 = high block
                const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(__int_as_float(h ? o.a_par[1] : o.a_par[0]),
                                                                    h ? o.dw_high : o.dw_low, z32, 0, 0, 0);
                // min terms of both blocks: the op's two K slots are the two lane halves
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(h ? o.a_par[3] : o.a_par[2]), h ? o.mw_high : o.mw_low,
                                                           acc, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    acc[v] = __fmaf_rn((float)i_low[v], sc[v], acc[v]);
                    acc[v] = __fmaf_rn((float)i_high[v], sc[16 + v], acc[v]);
                }
            }
        }
    }
#pragma unroll
    for (int v = 0; v < 16; v++) s_part[wave][64 * v + lane] = acc[v];
    __syncthreads();
    // thread t adds the four waves' elements 4 t .. 4 t + 3 (register v = t / 16, lanes 4 (t % 16) ..), in wave order
    v4f sum = *reinterpret_cast<const v4f*>(&s_part[0][4 * tid]);
#pragma unroll
    for (int w = 1; w < 4; w++) sum += *reinterpret_cast<const v4f*>(&s_part[w][4 * tid]);
    // element (v, lane): row 8 (v / 4) + 4 (lane / 32) + v % 4, column 32 panel + lane % 32
    auto store_out = [&](const v4f& x) {
        const int v = tid >> 4, l0 = 4 * (tid & 15);
        const int m = 8 * (v >> 2) + 4 * (l0 >> 5) + (v & 3);
        const int n = 32 * panel + (l0 & 31);
        if (m >= M) return;
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (n + e < N) C[(size_t)m * N + n + e] = x[e];
    };
    if (split == 1) {
        store_out(sum);
        return;
    }
    store16_agent(partials + (size_t)blockIdx.x * 1024 + 4 * tid, sum);
    wait_vmcnt<0>();
    __syncthreads();
    if (tid == 0) s_arrived = atomicAdd(&arrivals[panel], 1u);
    __syncthreads();
    if (s_arrived == (unsigned)(split - 1)) {
        static_assert(kMaxSplit <= 8, "the shares of a panel are fetched in one trip");
        const float* p = partials + (size_t)panel * split * 1024 + 4 * tid;
        v4f l[kMaxSplit];
#pragma unroll
        for (int c = 0; c < kMaxSplit; c++) l[c] = load16_agent(p + (size_t)min(c, split - 1) * 1024);
        wait_vmcnt<0>();
        __builtin_amdgcn_sched_barrier(0);
        v4f total = l[0];
#pragma unroll
        for (int c = 1; c < kMaxSplit; c++)
            if (c < split) total += l[c];
        store_out(total);
        if (tid == 0) __hip_atomic_store(&arrivals[panel], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace

// Shares of K per column panel: about three workgroups per CU, at least four super-blocks per workgroup.
int gemm_rows32_split(int N, int K) {
    const int panels = (N + 31) / 32, nbk = K / 64;
    int split = (kTargetGroups + panels - 1) / panels;
    if (split > kMaxSplit) split = kMaxSplit;
    if (split > nbk / 4) split = nbk / 4;
    return split < 1 ? 1 : split;
}

hipError_t launch_gemm_rows32_fp32(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws,
                                   hipStream_t s) {
    if (M < 1 || M > 32) return hipErrorInvalidValue;
    const int panels = (N + 31) / 32, split = gemm_rows32_split(N, K);
    // a share parks 4 KiB; the scratch is max_partials units of 16 KiB and as many counters
    if (split > 1 && ((long long)panels * split > (long long)ws.max_partials * 4 || panels > ws.max_partials)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm_a81w41_rows32_kernel, dim3(panels * split), dim3(kThreads), 0, s, static_cast<const uint8_t*>(A),
                       static_cast<const uint8_t*>(B), M, N, K / 64, split, C, ws.partials, ws.arrivals);
    return hipGetLastError();
}

}  // namespace a81w41
