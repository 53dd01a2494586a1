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
//
// STAGED (wide layers): the same work division, but a wave's operands of a super-block -- its 32 rows' 80 B blocks
// and its four 384 B weight blocks, 4 KiB -- are copied global -> LDS by four direct-to-LDS loads of 64 x 16 bytes
// into a ring of the wave's own (no barrier in the loop: a wave waits for its own copies only), and read from there.
// Per-lane register loads cost the CU's cache path one slot per instruction whatever their width: nine per wave and
// super-block there, four here.  The weight blocks' 16-byte chunks are rotated by 2 (g mod 4) slots inside the stage
// so that the four blocks a half wave reads in one instruction fall into different LDS banks.
#include "a81w41_kernels.h"
#include "agent_access.h"

namespace a81w41 {
namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

constexpr int kThreads = 256;
constexpr int kDepth = 3;       // super-blocks of operands in flight per wave
constexpr int kMaxSplit = 6;    // shares of K per column panel (each costs the last arriver one trip to memory)
constexpr int kTargetGroups = 768;
// Staged form: at most four shares.  Measured at 16 rows (forward, us; shares in brackets): q/o 11.1 (4) against 12.0 (6);
// qkv 12.9 (4), 14.0 (3), 13.3 (2); down_proj 16.9 (4), 17.9 (6), 20.4 (2); gate/up 17.0 (2 or 1), 21.6 (3, 4).
constexpr int kMaxSplitStaged = 4;

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

// ---- staged operands -------------------------------------------------------------------------------------------
constexpr int kStageA = 32 * kABlock32, kStage = kStageA + 4 * kWBlock32;  // 2560 + 1536 = 4096 bytes
constexpr int kRing = 3;                                                     // stages per wave; all but one in flight
static_assert(kStage == 4 * 64 * 16, "a stage is exactly four wave-wide 16-byte copies");

// byte offset inside a stage of (weight block gl = 0..3, 16-byte chunk k = 0..23, byte `within` of the chunk)
__device__ __forceinline__ uint32_t stage_b_byte(int gl, int k, int within) {
    return kStageA + (24 * gl + (k + 2 * (gl & 3)) % 24) * 16 + within;
}

struct StageCopy {       // per lane: where its 16 bytes of each of the four copies come from
    const uint8_t* src[4];  // at the wave's first super-block
    uint32_t step[4];       // bytes per super-block (80 for an activation chunk, 384 for a weight chunk)
};
struct StageRead {  // per lane byte offsets inside a stage
    uint32_t row, dw, mw, w[4];
};

__device__ __forceinline__ void stage_issue(const StageCopy& c, uint8_t* stage, int sb) {
#pragma unroll
    for (int i = 0; i < 4; i++)
        __builtin_amdgcn_global_load_lds(c.src[i] + (size_t)sb * c.step[i], (lds_ptr_t)(stage + 1024 * i), 16, 0, 0);
}

__device__ __forceinline__ Operands stage_read(const uint8_t* stage, const StageRead& rd, int h) {
    Operands o;
    const uint8_t* row = stage + rd.row;
    o.a_par = *reinterpret_cast<const v4i*>(row);
    o.a_low = *reinterpret_cast<const v4i*>(row + 16 + 16 * h);
    o.a_high = *reinterpret_cast<const v4i*>(row + 48 + 16 * h);
    // only this lane half's block parameters are read; both fields get them (the caller selects by h)
    o.dw_low = o.dw_high = *reinterpret_cast<const float*>(stage + rd.dw);
    o.mw_low = o.mw_high = *reinterpret_cast<const float*>(stage + rd.mw);
#pragma unroll
    for (int m = 0; m < 4; m++) o.w[m] = *reinterpret_cast<const uint32_t*>(stage + rd.w[m]);
    return o;
}

template <bool STAGED>
__global__ __launch_bounds__(kThreads) void gemm_a81w41_rows32_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                     int M, int N, int nbk, int split, float* __restrict__ C,
                                                                     float* __restrict__ partials,
                                                                     unsigned* __restrict__ arrivals,
                                                                     const uint8_t* __restrict__ At) {
    // STAGED: every wave's ring of kRing stages (12 KiB), whose first 4 KiB take the wave's partial result after
    // the loop; else just the four partial results [wave][register v][lane]
    extern __shared__ __align__(16) uint8_t s_dyn[];
    constexpr int kWaveBytes = STAGED ? kRing * kStage : 4096;
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
    // one super-block: the four matrix ops and their epilogue
    auto contract = [&](const Operands& o) {
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
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(h ? o.a_par[3] : o.a_par[2]), h ? o.mw_high : o.mw_low, acc,
                                                   0, 0, 0);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            acc[v] = __fmaf_rn((float)i_low[v], sc[v], acc[v]);
            acc[v] = __fmaf_rn((float)i_high[v], sc[16 + v], acc[v]);
        }
    };
    if (STAGED) {
        uint8_t* ring = s_dyn + wave * kWaveBytes;
        StageCopy cp;
        const int nb_n = N >> 3;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = 64 * i + lane;  // 16-byte chunk of the stage: 0..159 activation rows, 160..255 weight blocks
            if (c < 160) {
                const int rw = c / 5, piece = c - 5 * rw;
                if (At != nullptr) {  // the rows of a super-block next to each other: 2560 contiguous bytes per stage
                    // (row slots past M hold whatever an earlier call left there: a row's values only ever reach
                    // that row's outputs, which are not stored)
                    cp.src[i] = At + ((size_t)k_lo * 32 + rw) * kABlock32 + 16 * piece;
                    cp.step[i] = 32 * kABlock32;
                } else {
                    cp.src[i] = A + ((size_t)min(rw, M - 1) * nbk + k_lo) * kABlock32 + 16 * piece;
                    cp.step[i] = kABlock32;
                }
            } else {
                const int sl = c - 160, gl = sl / 24, pos = sl - 24 * gl;
                const int k = (pos - 2 * (gl & 3) + 24) % 24;  // slot pos of block gl holds chunk k
                cp.src[i] = B + ((size_t)min(4 * panel + gl, nb_n - 1) * nbk + k_lo) * kWBlock32 + 16 * k;
                cp.step[i] = kWBlock32;
            }
        }
        StageRead rd;
        {
            const int gl = r >> 3, jj = r & 7;
            rd.row = r * kABlock32;
            rd.dw = stage_b_byte(gl, 2 * h + (jj >> 2), 4 * (jj & 3));
            rd.mw = stage_b_byte(gl, 4 + 2 * h + (jj >> 2), 4 * (jj & 3));
#pragma unroll
            for (int m = 0; m < 4; m++) rd.w[m] = stage_b_byte(gl, 8 + 8 * h + 2 * m + (jj >> 2), 4 * (jj & 3));
        }
        if (n_steps > 0) {
            // stage n lives in buffer n % kRing; past the end the last super-block is copied again (never used),
            // which keeps the count of outstanding copies the same at every wait
#pragma unroll
            for (int st = 0; st < kRing - 1; st++) stage_issue(cp, ring + st * kStage, min(st, n_steps - 1));
            for (int step0 = 0; step0 < n_steps; step0 += kRing) {
#pragma unroll
                for (int u = 0; u < kRing; u++) {
                    const int step = step0 + u;
                    if (step >= n_steps) break;  // uniform over the wave
                    __builtin_amdgcn_sched_barrier(0);
                    wait_vmcnt<4 * (kRing - 2)>();  // stage `step` has landed; this wave's LDS reads are over
                    __builtin_amdgcn_sched_barrier(0);
                    stage_issue(cp, ring + ((u + kRing - 1) % kRing) * kStage, min(step + kRing - 1, n_steps - 1));
                    contract(stage_read(ring + u * kStage, rd, h));
                }
            }
            wait_vmcnt<0>();  // the tail copies have landed: the ring can take the partial result
        }
    } else if (n_steps > 0) {
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
                contract(ring[u]);
            }
        }
    }
    auto part_of = [&](int w) { return reinterpret_cast<float*>(s_dyn + w * kWaveBytes); };  // [register v][lane]
#pragma unroll
    for (int v = 0; v < 16; v++) part_of(wave)[64 * v + lane] = acc[v];
    __syncthreads();
    // thread t adds the four waves' elements 4 t .. 4 t + 3 (register v = t / 16, lanes 4 (t % 16) ..), in wave order
    v4f sum = *reinterpret_cast<const v4f*>(part_of(0) + 4 * tid);
#pragma unroll
    for (int w = 1; w < 4; w++) sum += *reinterpret_cast<const v4f*>(part_of(w) + 4 * tid);
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
int gemm_rows32_split(int N, int K, bool staged) {
    const int panels = (N + 31) / 32, nbk = K / 64;
    const int env_groups = tuning_env_int("A81W41_ROWS32_GROUPS");  // tuning builds only
    const int target = env_groups > 0 ? env_groups : kTargetGroups;
    int split = (target + panels - 1) / panels;
    if (split > (staged ? kMaxSplitStaged : kMaxSplit)) split = staged ? kMaxSplitStaged : kMaxSplit;
    if (split > nbk / 4) split = nbk / 4;
    return split < 1 ? 1 : split;
}

size_t gemm_rows32_a_by_superblock_bytes(int K) { return (size_t)(K / 64) * 32 * kABlock32; }

hipError_t launch_gemm_rows32_fp32(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws,
                                   hipStream_t s, bool staged, const void* a_by_superblock) {
    if (M < 1 || M > 32) return hipErrorInvalidValue;
    const int panels = (N + 31) / 32, split = gemm_rows32_split(N, K, staged);
    // a share parks 4 KiB; the scratch is max_partials units of 16 KiB and as many counters
    if (split > 1 && ((long long)panels * split > (long long)ws.max_partials * 4 || panels > ws.max_partials)) return hipErrorInvalidValue;
    if (staged)
        hipLaunchKernelGGL(gemm_a81w41_rows32_kernel<true>, dim3(panels * split), dim3(kThreads), 4 * kRing * kStage, s,
                           static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), M, N, K / 64, split, C, ws.partials,
                           ws.arrivals, static_cast<const uint8_t*>(a_by_superblock));
    else
        hipLaunchKernelGGL(gemm_a81w41_rows32_kernel<false>, dim3(panels * split), dim3(kThreads), 4 * 4096, s,
                           static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), M, N, K / 64, split, C, ws.partials,
                           ws.arrivals, static_cast<const uint8_t*>(nullptr));
    return hipGetLastError();
}

}  // namespace a81w41
