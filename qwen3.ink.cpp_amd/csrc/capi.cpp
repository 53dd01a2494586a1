// C ABI of the A81W41 library (declared in include/a81w41.h): argument checks,
// host-side weight repack, device-memory ownership for the layer objects and
// the M-dispatch of the linear layer.  All arithmetic on activations happens
// in the HIP kernels; nothing here computes on the CPU except the load-time
// byte shuffle of the weights.
#include "../../include/a81w41.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <memory>
#include <new>
#include <algorithm>
#include <string>
#include <thread>
#include <vector>

#include "a81w41_kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(A81W41_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                        \
    do {                                                     \
        hipError_t _e = (expr);                              \
        if (_e != hipSuccess) return hip_fail(_e, #expr);    \
    } while (0)

bool shape_ok(int N, int K) { return N > 0 && K > 0 && N % 8 == 0 && K % 64 == 0; }

// IEEE-754 binary32 -> binary16, round to nearest even (GGML_FP32_TO_FP16 at
// QwenOperator.cc:821-824).  Load-time only.
uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, mag = x & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((mag >> 13) & 0x3ffu));
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) return (uint16_t)sign;
    const int e = (int)(mag >> 23);
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;
    int drop = 13;
    uint32_t base = 0;
    if (e >= 113) {
        base = (uint32_t)(e - 112) << 10;
        m &= 0x7fffffu;
    } else {
        drop = 126 - e;
    }
    uint32_t q = m >> drop;
    const uint32_t rem = m & ((1u << drop) - 1u), half = 1u << (drop - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));
}

// Weight repack shared by both parameter widths.  Block (g, sb) at index
// g*(K/64)+sb; params [s_low[8] s_high[8] min_low[8] min_high[8]] then
// q_coupled[32p + 4jj + ii] = B[8g+jj][32sb + 4p + ii]  (QwenOperator.cc:812-847).
template <bool FP32>
void repack(int K, int N, uint8_t* out, const float* SB, const float* MinB, const uint8_t* B) {
    const int nb_k = K / 64, nb_n = N / 8, ld = K / 32;
    constexpr int BS = FP32 ? a81w41::kWBlock32 : a81w41::kWBlock16;
    constexpr int QOFF = FP32 ? 128 : 64;
    auto run = [=](int g_begin, int g_end) {
    for (int g = g_begin; g < g_end; g++) {
        for (int sb = 0; sb < nb_k; sb++) {
            uint8_t* blk = out + ((size_t)g * nb_k + sb) * BS;
            for (int jj = 0; jj < 8; jj++) {
                const size_t row = (size_t)(8 * g + jj) * ld + 2 * sb;
                const float par[4] = {SB[row], SB[row + 1], MinB ? MinB[row] : 0.f, MinB ? MinB[row + 1] : 0.f};
                for (int a = 0; a < (MinB ? 4 : 2); a++) {  // no MinB (repack_w80_weight): the min fields stay unwritten
                    if (FP32) {
                        memcpy(blk + 4 * (8 * a + jj), &par[a], 4);
                    } else {
                        const uint16_t hbits = f32_to_f16(par[a]);
                        memcpy(blk + 2 * (8 * a + jj), &hbits, 2);
                    }
                }
                const uint8_t* src = B + (size_t)(8 * g + jj) * (K / 2) + 32 * sb;
                for (int p = 0; p < 8; p++) memcpy(blk + QOFF + 32 * p + 4 * jj, src + 4 * p, 4);
            }
        }
    }
    };
    // Column groups are independent: split them over a few host threads for big layers.
    const int n_thr = (int)std::min<size_t>(8, std::max<size_t>(1, (size_t)N * K >> 22));
    if (n_thr == 1) {
        run(0, nb_n);
        return;
    }
    std::vector<std::thread> pool;
    for (int t = 0; t < n_thr; t++)
        pool.emplace_back(run, (int)((int64_t)nb_n * t / n_thr), (int)((int64_t)nb_n * (t + 1) / n_thr));
    for (auto& th : pool) th.join();
}

int check_device() {
    static int cached = -1;
    if (cached == 0) return A81W41_OK;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) return fail(A81W41_ERR_NO_DEVICE, "no HIP device visible (%s)", hipGetErrorString(e));
    hipDeviceProp_t prop;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(A81W41_ERR_NO_DEVICE, "device is %s, this library is built for gfx950 only", prop.gcnArchName);
    cached = 0;
    return A81W41_OK;
}

}  // namespace

struct a81w41_context {
    a81w41::GemmScratch gemm_scratch;  // partial tiles of the GEMM's K split: this context's own
    void* act_scratch = nullptr;  // quantised activations, sized for the fp32 layout
    size_t act_bytes = 0;
    void* a6_scratch = nullptr;   // the same rows in the M > 32 kernel's operand format
    size_t a6_bytes = 0;
    int64_t max_elems = 0;
    float* x_stage = nullptr;  // device staging for forward_host
    float* y_stage = nullptr;
    size_t x_bytes = 0, y_bytes = 0;
    a81w41::ChainState chain;  // overlapping dependent launches (a81w41_context_chain_*), created at first use
    bool chain_ready = false;
};

struct a81w41_linear {
    a81w41_context* ctx = nullptr;
    int N = 0, K = 0;
    void* w16 = nullptr;  // device, 320 B blocks
    void* w32 = nullptr;  // device, 384 B blocks
    void* w6 = nullptr;   // device, the block-scaled kernel's operand format, derived from w32
    int kernel_choice = A81W41_KERNEL_AUTO;
};

namespace a81w41 {
const GemmScratch& context_gemm_scratch(const a81w41_context* ctx) { return ctx->gemm_scratch; }
void* context_a6_scratch(const a81w41_context* ctx) { return ctx->a6_scratch; }
size_t context_resident_bytes(const a81w41_context* ctx) {
    return ctx->act_bytes + ctx->a6_bytes + ctx->x_bytes + ctx->y_bytes + gemm_scratch_bytes(ctx->gemm_scratch);
}
ChainState* context_chain(a81w41_context* ctx) {
    if (!ctx->chain_ready) {
        if (chain_create(&ctx->chain) != hipSuccess) return nullptr;
        ctx->chain_ready = true;
    }
    return &ctx->chain;
}
const void* linear_w6(const a81w41_linear* layer) { return layer->w6; }
bool linear_block_scaled(const a81w41_linear* l, int M) {
    if (!l->w6 || M < kGemmFp6MinRows || l->kernel_choice == A81W41_KERNEL_INT8) return false;
    return l->kernel_choice == A81W41_KERNEL_BLOCK_SCALED || gemm_fp6_preferred(M, l->N, l->K);
}
// Lets the other translation units of the library leave their message where a81w41_last_error() finds it.
int report_failure(int status, const char* message) { return fail(status, "%s", message); }
uint16_t float_to_half_bits(float f) { return f32_to_f16(f); }
}  // namespace a81w41

extern "C" {

const char* a81w41_status_string(int status) {
    switch (status) {
        case A81W41_OK: return "ok";
        case A81W41_ERR_INVALID_ARG: return "invalid argument";
        case A81W41_ERR_HIP: return "HIP runtime error";
        case A81W41_ERR_IO: return "weight file error";
        case A81W41_ERR_NO_DEVICE: return "no gfx950 device";
        default: return "unknown status";
    }
}

const char* a81w41_last_error(void) { return g_err; }

size_t a81w41_weight_blob_bytes(int K, int N, int fp32) {
    if (!shape_ok(N, K)) return 0;
    return (size_t)N / 8 * (size_t)(K / 64) * (fp32 ? a81w41::kWBlock32 : a81w41::kWBlock16);
}

size_t a81w41_act_blob_bytes(int64_t k, int fp32) {
    if (k < 0 || k % 64) return 0;
    return (size_t)(k / 64) * (fp32 ? a81w41::kABlock32 : a81w41::kABlock16);
}

static int repack_checked(bool fp32, int K, int N, int qblk, void* out, const float* SB, const float* MinB,
                          const uint8_t* B) {
    if (qblk != A81W41_QK) return fail(A81W41_ERR_INVALID_ARG, "Q_BLK_SIZE must be 32, got %d", qblk);
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    if (!out || !SB || !MinB || !B) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (fp32)
        repack<true>(K, N, static_cast<uint8_t*>(out), SB, MinB, B);
    else
        repack<false>(K, N, static_cast<uint8_t*>(out), SB, MinB, B);
    return A81W41_OK;
}

int a81w41_repack_w81_weight_fp16(int K, int N, int Q_BLK_SIZE, void* B_repack, const float* SB,
                                  const float* MinB, const uint8_t* B) {
    return repack_checked(false, K, N, Q_BLK_SIZE, B_repack, SB, MinB, B);
}

int a81w41_repack_w81_weight_fp32(int K, int N, int Q_BLK_SIZE, void* B_repack, const float* SB,
                                  const float* MinB, const uint8_t* B) {
    return repack_checked(true, K, N, Q_BLK_SIZE, B_repack, SB, MinB, B);
}

int a81w41_repack_w80_weight(int K, int N, int Q_BLK_SIZE, void* B_repack, const float* SB, const uint8_t* B) {
    if (Q_BLK_SIZE != A81W41_QK) return fail(A81W41_ERR_INVALID_ARG, "Q_BLK_SIZE must be 32, got %d", Q_BLK_SIZE);
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    if (!B_repack || !SB || !B) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    repack<false>(K, N, static_cast<uint8_t*>(B_repack), SB, nullptr, B);
    return A81W41_OK;
}

int a81w41_quantize_weight_q40(const float* w, int N, int K, uint8_t* weight_int4, float* scale) {
    if (!w || !weight_int4 || !scale) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (N < 1 || K < 64 || K % 64) return fail(A81W41_ERR_INVALID_ARG, "need N >= 1 and K a positive multiple of 64, got N=%d K=%d", N, K);
    const size_t n_sb = (size_t)N * K / 64;
    for (size_t sb = 0; sb < n_sb; sb++) {
        uint8_t code[2][32];
        for (int h = 0; h < 2; h++) {
            const float* x = w + sb * 64 + 32 * h;
            float vmax = x[0];  // the element of largest magnitude (the first on ties), with its sign
            for (int i = 1; i < 32; i++) vmax = fabsf(x[i]) > fabsf(vmax) ? x[i] : vmax;
            const float d = vmax / -8.0f;
            const float id = d == 0.0f ? 0.0f : 1.0f / d;
            scale[2 * sb + h] = d;
            for (int i = 0; i < 32; i++) {
                float v = x[i] * id + 8.5f;  // two fp32 roundings (contraction is off), like the numpy expression
                v = v < 0.0f ? 0.0f : (v > 15.0f ? 15.0f : v);
                code[h][i] = (uint8_t)v;  // truncation, like astype(uint8)
            }
        }
        for (int e = 0; e < 32; e++) weight_int4[sb * 32 + e] = (uint8_t)(code[0][e] | (code[1][e] << 4));
    }
    return A81W41_OK;
}

int a81w41_quantize_weight_q41(const float* w, int N, int K, uint8_t* weight_int4, float* scale, float* offset) {
    if (!w || !weight_int4 || !scale || !offset) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (N < 1 || K < 64 || K % 64) return fail(A81W41_ERR_INVALID_ARG, "need N >= 1 and K a positive multiple of 64, got N=%d K=%d", N, K);
    const size_t n_sb = (size_t)N * K / 64;
    for (size_t sb = 0; sb < n_sb; sb++) {
        uint8_t code[2][32];
        for (int h = 0; h < 2; h++) {
            const float* x = w + sb * 64 + 32 * h;
            float mx = x[0], mn = x[0];
            for (int i = 1; i < 32; i++) {
                mx = x[i] > mx ? x[i] : mx;
                mn = x[i] < mn ? x[i] : mn;
            }
            const float d = (mx - mn) / 15.0f;
            const float id = d == 0.0f ? 0.0f : 1.0f / d;
            scale[2 * sb + h] = d;
            offset[2 * sb + h] = mn;
            for (int i = 0; i < 32; i++) {
                float r = nearbyintf((x[i] - mn) * id);  // default rounding mode: half to even, like np.round
                r = r < 0.0f ? 0.0f : (r > 15.0f ? 15.0f : r);
                code[h][i] = (uint8_t)r;
            }
        }
        for (int e = 0; e < 32; e++) weight_int4[sb * 32 + e] = (uint8_t)(code[0][e] | (code[1][e] << 4));
    }
    return A81W41_OK;
}

static int quantize_checked(bool fp32, const float* x, void* vy, int64_t k, void* stream, bool write_sums = true) {
    if (k < 0 || k % 64) return fail(A81W41_ERR_INVALID_ARG, "k must be a non-negative multiple of 64, got %lld", (long long)k);
    if (k == 0) return A81W41_OK;
    if (!x || !vy) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if ((reinterpret_cast<uintptr_t>(x) & 3) || (reinterpret_cast<uintptr_t>(vy) & 7))
        return fail(A81W41_ERR_INVALID_ARG, "x must be 4-byte and vy 8-byte aligned");
    if (int st = check_device()) return st;
    HIP_TRY(a81w41::launch_quantize(x, vy, k / 64, fp32, static_cast<hipStream_t>(stream), write_sums));
    return A81W41_OK;
}

int a81w41_quantize_row_q8_0_repack(const float* x_dev, void* vy_dev, int64_t k, void* stream) {
    return quantize_checked(false, x_dev, vy_dev, k, stream, false);
}

int a81w41_quantize_row_q8_1_repack_fp16(const float* x_dev, void* vy_dev, int64_t k, void* stream) {
    return quantize_checked(false, x_dev, vy_dev, k, stream);
}

int a81w41_quantize_row_q8_1_repack_fp32(const float* x_dev, void* vy_dev, int64_t k, void* stream) {
    return quantize_checked(true, x_dev, vy_dev, k, stream);
}

// The K-split scratch of the free-standing GEMM entry points: one per stream, so that calls on different
// streams never share partial tiles; none is needed (or created) for calls that do not split K.
static int stream_scratch(void* stream, int M, int N, int K, a81w41::GemmScratch* ws) {
    if (a81w41::gemm_partial_tiles(M, N, K) == 0) return A81W41_OK;
    const hipError_t e = a81w41::gemm_scratch_for_stream(static_cast<hipStream_t>(stream), ws);
    if (e == hipErrorStreamCaptureUnsupported)
        return fail(A81W41_ERR_INVALID_ARG,
                    "the first K-split GEMM call on a stream allocates (or takes over) that stream's scratch and cannot be captured: "
                    "call once before the capture, use a layer object, or a81w41_gemm_repack_A81W41_fp32_static");
    if (e == hipErrorOutOfMemory) return fail(A81W41_ERR_HIP, "GEMM scratch: out of device memory (64 MiB per stream, at most 16 streams' worth)");
    if (e != hipSuccess) return hip_fail(e, "gemm_scratch_for_stream");
    return A81W41_OK;
}

static int contract_args_ok(const void* A, const void* B, const void* C, int M, int N, int K) {
    if (M < 1) return fail(A81W41_ERR_INVALID_ARG, "M must be >= 1, got %d", M);
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    if (!A || !B || !C) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if ((reinterpret_cast<uintptr_t>(B) & 15) || (reinterpret_cast<uintptr_t>(C) & 3))
        return fail(A81W41_ERR_INVALID_ARG, "weight blob must be 16-byte aligned (the reference allocates it 64-byte aligned)");
    return check_device();
}

int a81w41_gemv_repack_A81W41_fp16(const void* A_repack_dev, const void* B_repack_dev, float* C_dev, int M,
                                   int N, int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, C_dev, M, N, K)) return st;
    if (reinterpret_cast<uintptr_t>(A_repack_dev) & 7)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 8-byte aligned");
    if (a81w41::gemv_lds_bytes(K) > a81w41::kLdsLimitBytes)
        return fail(A81W41_ERR_INVALID_ARG, "K=%d exceeds the LDS-resident activation row (max K = %d)", K, a81w41::gemv_max_k());
    HIP_TRY(a81w41::launch_gemv_fp16(A_repack_dev, B_repack_dev, C_dev, N, K, static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_gemm_repack_A81W41_fp32(const void* A_repack_dev, const void* B_repack_dev, float* C_dev, int M,
                                   int N, int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, C_dev, M, N, K)) return st;
    if (reinterpret_cast<uintptr_t>(A_repack_dev) & 15)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 16-byte aligned");
    a81w41::GemmScratch ws;
    if (int st = stream_scratch(stream, M, N, K, &ws)) return st;
    HIP_TRY(a81w41::launch_gemm_fp32(A_repack_dev, B_repack_dev, C_dev, M, N, K, ws, static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_gemm_repack_A81W41_fp32_static(const void* A_repack_dev, const void* B_repack_dev, float* C_dev, int M,
                                          int N, int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, C_dev, M, N, K)) return st;
    if (reinterpret_cast<uintptr_t>(A_repack_dev) & 15)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 16-byte aligned");
    const int need = a81w41::gemm_partial_tiles(M, N, K);
    if (need < 0) return fail(A81W41_ERR_HIP, "cannot query the device");
    if (need > a81w41::gemm_static_scratch_tiles())
        return fail(A81W41_ERR_INVALID_ARG,
                    "M=%d N=%d K=%d parks %d partial tiles, the static scratch holds %d: use a81w41_gemm_repack_A81W41_fp32",
                    M, N, K, need, a81w41::gemm_static_scratch_tiles());
    a81w41::GemmScratch ws;
    HIP_TRY(a81w41::gemm_static_scratch(&ws));
    // the array keeps what the last call left: the counters must start at zero
    if (need > 0) HIP_TRY(a81w41::clear_gemm_counters(ws, static_cast<hipStream_t>(stream)));
    HIP_TRY(a81w41::launch_gemm_fp32(A_repack_dev, B_repack_dev, C_dev, M, N, K, ws, static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_gemm_schedule_selfcheck(int M, int N, int K, int resident_workgroups, int cus) {
    if (M < 1 || !shape_ok(N, K) || cus < 1 || resident_workgroups < cus || resident_workgroups % cus)
        return fail(A81W41_ERR_INVALID_ARG, "bad arguments") * -100;
    return a81w41::gemm_schedule_selfcheck(M, N, K, resident_workgroups, cus);
}

int a81w41_gemm_fp6_plan_selfcheck(int M, int N, int K, int resident_workgroups) {
    if (M < 1 || !shape_ok(N, K) || resident_workgroups < 1) return fail(A81W41_ERR_INVALID_ARG, "bad arguments") * -100;
    return a81w41::gemm_fp6_plan_selfcheck(M, N, K, resident_workgroups);
}

int a81w41_gemv_repack_A80W40(const void* A_repack_dev, const void* B_repack_dev, float* C_dev, int M, int N,
                              int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, C_dev, M, N, K)) return st;
    if (reinterpret_cast<uintptr_t>(A_repack_dev) & 7)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 8-byte aligned");
    if (a81w41::gemv_lds_bytes(K) > a81w41::kLdsLimitBytes)
        return fail(A81W41_ERR_INVALID_ARG, "K=%d exceeds the LDS-resident activation row (max K = %d)", K, a81w41::gemv_max_k());
    HIP_TRY(a81w41::launch_gemv_a80w40(A_repack_dev, B_repack_dev, C_dev, N, K, static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

size_t a81w41_gemm_repack_A80W40_workspace_bytes(int M, int N, int K) {
    if (M < 1 || !shape_ok(N, K)) return 0;
    return a81w41::gemm_a80w40_workspace_bytes(M, N, K);
}

int a81w41_gemm_repack_A80W40(const void* A_repack_dev, const void* B_repack_dev, float* C_dev, int M, int N,
                              int K, void* workspace_dev, size_t workspace_bytes, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, C_dev, M, N, K)) return st;
    if (reinterpret_cast<uintptr_t>(A_repack_dev) & 7)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 8-byte aligned");
    if (!workspace_dev || (reinterpret_cast<uintptr_t>(workspace_dev) & 15))
        return fail(A81W41_ERR_INVALID_ARG, "workspace must be a 16-byte aligned device buffer");
    const size_t need = a81w41::gemm_a80w40_workspace_bytes(M, N, K);
    if (workspace_bytes < need)
        return fail(A81W41_ERR_INVALID_ARG, "workspace of %zu bytes is too small, M=%d N=%d K=%d needs %zu", workspace_bytes,
                    M, N, K, need);
    a81w41::GemmScratch ws;
    if (int st = stream_scratch(stream, M, N, K, &ws)) return st;
    HIP_TRY(a81w41::launch_gemm_a80w40(A_repack_dev, B_repack_dev, C_dev, M, N, K, workspace_dev, ws,
                                       static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_block_idot_A80W40(const void* A_repack_dev, const void* B_repack_dev, int32_t* out_dev, int M, int N,
                             int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, out_dev, M, N, K)) return st;
    HIP_TRY(a81w41::launch_block_idot(A_repack_dev, false, B_repack_dev, false, out_dev, M, N, K,
                                      static_cast<hipStream_t>(stream), true));
    return A81W41_OK;
}

int a81w41_block_idot(const void* A_repack_dev, int a_fp32, const void* B_repack_dev, int b_fp32,
                      int32_t* out_dev, int M, int N, int K, void* stream) {
    if (int st = contract_args_ok(A_repack_dev, B_repack_dev, out_dev, M, N, K)) return st;
    HIP_TRY(a81w41::launch_block_idot(A_repack_dev, a_fp32 != 0, B_repack_dev, b_fp32 != 0, out_dev, M, N, K,
                                      static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_context_create(int max_rows, int max_cols, a81w41_context** out) {
    if (!out) return fail(A81W41_ERR_INVALID_ARG, "null out pointer");
    *out = nullptr;
    if (max_rows < 1 || max_cols < 64 || max_cols % 64)
        return fail(A81W41_ERR_INVALID_ARG, "need max_rows >= 1 and max_cols a positive multiple of 64");
    if (int st = check_device()) return st;
    std::unique_ptr<a81w41_context> ctx(new (std::nothrow) a81w41_context);
    if (!ctx) return fail(A81W41_ERR_HIP, "out of host memory");
    ctx->max_elems = (int64_t)max_rows * max_cols;
    ctx->act_bytes = (size_t)(ctx->max_elems / 64) * a81w41::kABlock32;
    HIP_TRY(a81w41::gemm_scratch_create(&ctx->gemm_scratch));
    // A6 holds 2 B per value, rows padded to a multiple of 32 (calls that use it have more than 32 rows)
    ctx->a6_bytes = 4 * (size_t)ctx->max_elems;
    hipError_t e = hipMalloc(&ctx->act_scratch, ctx->act_bytes);
    if (e == hipSuccess) e = hipMalloc(&ctx->a6_scratch, ctx->a6_bytes);
    if (e != hipSuccess) {
        a81w41::gemm_scratch_destroy(&ctx->gemm_scratch);
        (void)hipFree(ctx->act_scratch);
        return hip_fail(e, "hipMalloc(activation scratch)");
    }
    // the chain's stream, events and counters exist from the start, so that a chain can be opened under stream capture
    if (!a81w41::context_chain(ctx.get())) {
        a81w41_context_destroy(ctx.release());
        return fail(A81W41_ERR_HIP, "cannot create the chain's stream, events and counters");
    }
    *out = ctx.release();
    return A81W41_OK;
}

void a81w41_context_destroy(a81w41_context* ctx) {
    if (!ctx) return;
    a81w41::gemm_scratch_destroy(&ctx->gemm_scratch);
    if (ctx->chain_ready) a81w41::chain_destroy(&ctx->chain);
    (void)hipFree(ctx->act_scratch);
    (void)hipFree(ctx->a6_scratch);
    (void)hipFree(ctx->x_stage);
    (void)hipFree(ctx->y_stage);
    delete ctx;
}

void* a81w41_context_activation_scratch_dev(const a81w41_context* ctx) { return ctx ? ctx->act_scratch : nullptr; }

// The most rows a call of a K-wide layer may have on this context.
static int max_rows_of(const a81w41_context* ctx, int K) {
    const int64_t rows = ctx->max_elems / K;
    return rows > 0x7fffffff ? 0x7fffffff : (int)rows;
}

// Derives the block-scaled kernel's weight operand from the 384 B blob (on the device, synchronous).
static hipError_t build_w6(a81w41_linear* l) {
    if (l->w6 || !l->w32) return hipSuccess;
    hipError_t e = hipMalloc(&l->w6, a81w41::gemm_fp6_w6_bytes(l->N, l->K));
    if (e == hipSuccess) e = a81w41::launch_w384_to_w6(l->w32, l->w6, l->N, l->K, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) {
        (void)hipFree(l->w6);
        l->w6 = nullptr;
    }
    return e;
}

int a81w41_linear_create_from_blobs(a81w41_context* ctx, int N, int K, const void* blob_fp16,
                                    const void* blob_fp32, a81w41_linear** out) {
    if (!out) return fail(A81W41_ERR_INVALID_ARG, "null out pointer");
    *out = nullptr;
    if (!ctx) return fail(A81W41_ERR_INVALID_ARG, "null context");
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    if (!blob_fp16 && !blob_fp32) return fail(A81W41_ERR_INVALID_ARG, "at least one blob is required");
    std::unique_ptr<a81w41_linear> l(new (std::nothrow) a81w41_linear);
    if (!l) return fail(A81W41_ERR_HIP, "out of host memory");
    l->ctx = ctx;
    l->N = N;
    l->K = K;
    hipError_t e = hipSuccess;
    if (blob_fp16) {
        const size_t b = a81w41_weight_blob_bytes(K, N, 0);
        e = hipMalloc(&l->w16, b);
        if (e == hipSuccess) e = hipMemcpy(l->w16, blob_fp16, b, hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && blob_fp32) {
        const size_t b = a81w41_weight_blob_bytes(K, N, 1);
        e = hipMalloc(&l->w32, b);
        if (e == hipSuccess) e = hipMemcpy(l->w32, blob_fp32, b, hipMemcpyHostToDevice);
        // the operand format of the block-scaled kernel (a third copy, 1 B per weight): only where a call this
        // context admits can be routed there
        if (e == hipSuccess && a81w41::gemm_fp6_preferred(max_rows_of(ctx, K), N, K)) e = build_w6(l.get());
    }
    if (e != hipSuccess) {
        (void)hipFree(l->w16);
        (void)hipFree(l->w32);
        (void)hipFree(l->w6);
        return hip_fail(e, "uploading weight blobs");
    }
    *out = l.release();
    return A81W41_OK;
}

int a81w41_linear_create(a81w41_context* ctx, int N, int K, const uint8_t* weight_int4, const float* scale,
                         const float* offset, a81w41_linear** out) {
    if (out) *out = nullptr;
    if (!weight_int4 || !scale || !offset) return fail(A81W41_ERR_INVALID_ARG, "null weight arrays");
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    std::vector<uint8_t> b16(a81w41_weight_blob_bytes(K, N, 0)), b32(a81w41_weight_blob_bytes(K, N, 1));
    repack<false>(K, N, b16.data(), scale, offset, weight_int4);
    repack<true>(K, N, b32.data(), scale, offset, weight_int4);
    return a81w41_linear_create_from_blobs(ctx, N, K, b16.data(), b32.data(), out);
}

static int read_file(const std::string& name, void* dst, size_t bytes) {
    FILE* f = fopen(name.c_str(), "rb");
    if (!f) return fail(A81W41_ERR_IO, "cannot open %s", name.c_str());
    const size_t got = fread(dst, 1, bytes, f);
    fclose(f);
    if (got != bytes) return fail(A81W41_ERR_IO, "%s: expected %zu bytes, read %zu", name.c_str(), bytes, got);
    return A81W41_OK;
}

int a81w41_linear_load(a81w41_context* ctx, const char* path, int dim_x, int dim_y, int dim_z,
                       a81w41_linear** out) {
    if (out) *out = nullptr;
    if (!path) return fail(A81W41_ERR_INVALID_ARG, "null path");
    if (dim_x != 1) return fail(A81W41_ERR_INVALID_ARG, "weight_dim_x must be 1, got %d", dim_x);
    const int N = dim_y, K = dim_z;
    if (!shape_ok(N, K)) return fail(A81W41_ERR_INVALID_ARG, "need K %% 64 == 0 and N %% 8 == 0, got K=%d N=%d", K, N);
    const std::string p(path);
    std::vector<uint8_t> w4((size_t)N * K / 2);
    std::vector<float> sc((size_t)N * K / 32), of((size_t)N * K / 32);
    if (int st = read_file(p + "weight_int4.bin", w4.data(), w4.size())) return st;
    if (int st = read_file(p + "scaling_factor_int4.bin", sc.data(), sc.size() * 4)) return st;
    if (int st = read_file(p + "offset_int4.bin", of.data(), of.size() * 4)) return st;
    return a81w41_linear_create(ctx, N, K, w4.data(), sc.data(), of.data(), out);
}

void a81w41_linear_destroy(a81w41_linear* l) {
    if (!l) return;
    (void)hipFree(l->w16);
    (void)hipFree(l->w32);
    (void)hipFree(l->w6);
    delete l;
}

size_t a81w41_linear_resident_bytes(const a81w41_linear* l, size_t* fp16_blob, size_t* fp32_blob, size_t* block_scaled) {
    if (!l) return 0;
    const size_t b16 = l->w16 ? a81w41_weight_blob_bytes(l->K, l->N, 0) : 0;
    const size_t b32 = l->w32 ? a81w41_weight_blob_bytes(l->K, l->N, 1) : 0;
    const size_t b6 = l->w6 ? a81w41::gemm_fp6_w6_bytes(l->N, l->K) : 0;
    if (fp16_blob) *fp16_blob = b16;
    if (fp32_blob) *fp32_blob = b32;
    if (block_scaled) *block_scaled = b6;
    return b16 + b32 + b6;
}

const char* a81w41_linear_kernel_name(const a81w41_linear* l, int M) {
    if (!l || M < 1) return "";
    if (M == 1) return "gemv (v_dot4, fused quantiser prologue, weights streamed once)";
    if (a81w41::gemm_rows_fused_preferred(M, l->K)) return "rows_fused (2..8 rows quantised in the prologue, resident in LDS, v_dot4, one launch)";
    if (a81w41::linear_block_scaled(l, M)) return "block_scaled (fp6 block-scaled matrix ops, 128 x 256 tiles, stream-K)";
    return a81w41::gemm_kernel_name(M, l->N, l->K);
}

int a81w41_linear_in_features(const a81w41_linear* l) { return l ? l->K : 0; }
int a81w41_linear_out_features(const a81w41_linear* l) { return l ? l->N : 0; }
const void* a81w41_linear_weight_fp16_dev(const a81w41_linear* l) { return l ? l->w16 : nullptr; }
const void* a81w41_linear_weight_fp32_dev(const a81w41_linear* l) { return l ? l->w32 : nullptr; }

// One-row call on a context whose chain is open: the fused quantise + contract launch as the chain's next link.
static int chained_forward(a81w41_context* ctx, int n, const void* const* Bs, float* const* Cs, const int* Ns, int K,
                           const float* x_dev, int M, void* stream) {
    a81w41::ChainState& ch = ctx->chain;
    if (M != 1) return fail(A81W41_ERR_INVALID_ARG, "a chain is open on this context: only one-row calls (M = 1), got M = %d", M);
    if (static_cast<hipStream_t>(stream) != ch.main)
        return fail(A81W41_ERR_INVALID_ARG, "a chain is open on this context: calls must name the stream it was opened on");
    for (int j = 0; j < n; j++) {
        if (!Bs[j]) return fail(A81W41_ERR_INVALID_ARG, "layer has no fp16-parameter blob (needed for M == 1)");
        if (reinterpret_cast<uintptr_t>(Cs[j]) & 3) return fail(A81W41_ERR_INVALID_ARG, "y must be 4-byte aligned");
    }
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15) || !a81w41::gemv_chain_fits(K, false))
        return fail(A81W41_ERR_INVALID_ARG, "a chained call needs x 16-byte aligned and K <= 40960, got K = %d", K);
    if (int st = check_device()) return st;
    hipStream_t s = nullptr;
    const a81w41::ChainLink link = a81w41::chain_next(&ch, &s);
    unsigned grid = 0;
    HIP_TRY(a81w41::launch_gemv_chain_fused(x_dev, ctx->act_scratch, n, Bs, Cs, Ns, K, link, ch.cus, &grid, s));
    a81w41::chain_launched(&ch, grid);
    return A81W41_OK;
}

int a81w41_context_chain_begin(a81w41_context* ctx, void* stream) {
    if (!ctx) return fail(A81W41_ERR_INVALID_ARG, "null context");
    if (int st = check_device()) return st;
    a81w41::ChainState* ch = a81w41::context_chain(ctx);
    if (!ch) return fail(A81W41_ERR_HIP, "cannot create the chain's stream, events and counters");
    if (ch->open) return fail(A81W41_ERR_INVALID_ARG, "a chain is already open on this context");
    HIP_TRY(a81w41::chain_begin(ch, static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_context_chain_end(a81w41_context* ctx) {
    if (!ctx || !ctx->chain_ready || !ctx->chain.open) return fail(A81W41_ERR_INVALID_ARG, "no chain is open on this context");
    HIP_TRY(a81w41::chain_end(&ctx->chain));
    return A81W41_OK;
}

int a81w41_context_chain_status(a81w41_context* ctx, int* gave_up) {
    if (!ctx || !gave_up) return fail(A81W41_ERR_INVALID_ARG, "null argument");
    *gave_up = 0;
    if (!ctx->chain_ready) return A81W41_OK;
    if (ctx->chain.open) return fail(A81W41_ERR_INVALID_ARG, "close the chain first");
    bool bad = false;
    HIP_TRY(a81w41::chain_status(&ctx->chain, &bad));
    *gave_up = bad ? 1 : 0;
    return A81W41_OK;
}

int a81w41_context_chain_selfcheck_stuck_wait(a81w41_linear* l, const float* x_dev, float* y_dev, unsigned polls, void* stream) {
    if (!l || !x_dev || !y_dev) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    a81w41_context* ctx = l->ctx;
    a81w41::ChainState* ch = a81w41::context_chain(ctx);
    if (!ch) return fail(A81W41_ERR_HIP, "cannot create the chain's stream, events and counters");
    if (ch->open) return fail(A81W41_ERR_INVALID_ARG, "close the chain first");
    if (!l->w16 || (reinterpret_cast<uintptr_t>(x_dev) & 15) || (reinterpret_cast<uintptr_t>(y_dev) & 3) ||
        !a81w41::gemv_chain_fits(l->K, false))
        return fail(A81W41_ERR_INVALID_ARG, "needs the fp16-parameter blob, x 16-byte aligned, K <= 40960");
    if (int st = check_device()) return st;
    a81w41::ChainLink link;
    link.wait = ch->counters;  // zero at rest, and nothing will count on it
    link.wait_for = 1;
    link.status = ch->counters + a81w41::kChainRing;
    link.spin_limit = polls;
    const void* Bs[1] = {l->w16};
    float* Cs[1] = {y_dev};
    HIP_TRY(a81w41::launch_gemv_chain_fused(x_dev, ctx->act_scratch, 1, Bs, Cs, &l->N, l->K, link, ch->cus, nullptr,
                                            static_cast<hipStream_t>(stream)));
    return A81W41_OK;
}

int a81w41_context_chain_set_spin_limit(a81w41_context* ctx, unsigned polls) {
    if (!ctx) return fail(A81W41_ERR_INVALID_ARG, "null context");
    a81w41::ChainState* ch = a81w41::context_chain(ctx);
    if (!ch) return fail(A81W41_ERR_HIP, "cannot create the chain's stream, events and counters");
    if (ch->open) return fail(A81W41_ERR_INVALID_ARG, "close the chain first");
    ch->spin_limit = polls;
    return A81W41_OK;
}

int a81w41_linear_forward(a81w41_linear* l, const float* x_dev, int M, float* y_dev, void* stream) {
    if (!l || !x_dev || !y_dev) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (M < 1) return fail(A81W41_ERR_INVALID_ARG, "M must be >= 1, got %d", M);
    a81w41_context* ctx = l->ctx;
    if ((int64_t)M * l->K > ctx->max_elems)
        return fail(A81W41_ERR_INVALID_ARG, "M*K = %lld exceeds the context's activation scratch (%lld)",
                    (long long)M * l->K, (long long)ctx->max_elems);
    if (ctx->chain_ready && ctx->chain.open) {  // a link of the context's open chain
        const void* Bs[1] = {l->w16};
        float* Cs[1] = {y_dev};
        return chained_forward(ctx, 1, Bs, Cs, &l->N, l->K, x_dev, M, stream);
    }
    // QwenOperator.cc:96-120: the precision of the activation parameters follows M.
    if (M > 1) {
        if (!l->w32) return fail(A81W41_ERR_INVALID_ARG, "layer has no fp32-parameter blob (needed for M > 1)");
        if (a81w41::linear_block_scaled(l, M)) {
            // same quantised rows (the scratch still receives the reference's 80 B blocks), contracted by the
            // block-scaled matrix ops from the private operand formats
            if ((reinterpret_cast<uintptr_t>(x_dev) & 3) || (reinterpret_cast<uintptr_t>(y_dev) & 3))
                return fail(A81W41_ERR_INVALID_ARG, "x and y must be 4-byte aligned");
            if (int st = check_device()) return st;
            HIP_TRY(a81w41::launch_quantize_a6(x_dev, ctx->act_scratch, ctx->a6_scratch, M, l->K, static_cast<hipStream_t>(stream)));
            HIP_TRY(a81w41::launch_gemm_fp6(ctx->a6_scratch, l->w6, y_dev, M, l->N, l->K, ctx->gemm_scratch,
                                            static_cast<hipStream_t>(stream)));
            return A81W41_OK;
        }
        if ((reinterpret_cast<uintptr_t>(x_dev) & 15) == 0 && a81w41::gemm_rows_fused_preferred(M, l->K)) {
            // few rows: one launch, every workgroup quantises the rows itself, workgroup 0 also fills the scratch
            if (int st = contract_args_ok(x_dev, l->w32, y_dev, M, l->N, l->K)) return st;
            HIP_TRY(a81w41::launch_gemm_rows_fused(x_dev, ctx->act_scratch, l->w32, y_dev, M, l->N, l->K,
                                                   static_cast<hipStream_t>(stream)));
            return A81W41_OK;
        }
        if (a81w41::gemm_rows32_staged_preferred(M, l->N, l->K) &&
            a81w41::gemm_rows32_a_by_superblock_bytes(l->K) <= ctx->a6_bytes) {
            // up to 32 rows on a wide layer: the quantiser also writes the blocks with a super-block's rows next to each
            // other (into the scratch of the block-scaled kernel's operands, which such a call does not use), and the
            // contraction stages its activations from there; same arithmetic, same bits as from the 80 B blocks alone
            if (int st = contract_args_ok(ctx->act_scratch, l->w32, y_dev, M, l->N, l->K)) return st;
            if (reinterpret_cast<uintptr_t>(x_dev) & 3) return fail(A81W41_ERR_INVALID_ARG, "x must be 4-byte aligned");
            HIP_TRY(a81w41::launch_quantize(x_dev, ctx->act_scratch, (int64_t)M * l->K / 64, true, static_cast<hipStream_t>(stream),
                                            true, ctx->a6_scratch, l->K / 64));
            HIP_TRY(a81w41::launch_gemm_rows32_fp32(ctx->act_scratch, l->w32, y_dev, M, l->N, l->K, ctx->gemm_scratch,
                                                    static_cast<hipStream_t>(stream), true, ctx->a6_scratch));
            return A81W41_OK;
        }
        if (int st = a81w41_quantize_row_q8_1_repack_fp32(x_dev, ctx->act_scratch, (int64_t)M * l->K, stream)) return st;
        if (int st = contract_args_ok(ctx->act_scratch, l->w32, y_dev, M, l->N, l->K)) return st;
        HIP_TRY(a81w41::launch_gemm_fp32(ctx->act_scratch, l->w32, y_dev, M, l->N, l->K, ctx->gemm_scratch,
                                         static_cast<hipStream_t>(stream)));
        return A81W41_OK;
    }
    if (!l->w16) return fail(A81W41_ERR_INVALID_ARG, "layer has no fp16-parameter blob (needed for M == 1)");
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15) == 0 && a81w41::gemv_lds_bytes(l->K) <= a81w41::kLdsLimitBytes) {
        // one launch: every workgroup quantises x itself, workgroup 0 also fills the scratch
        if ((reinterpret_cast<uintptr_t>(y_dev) & 3)) return fail(A81W41_ERR_INVALID_ARG, "y must be 4-byte aligned");
        if (int st = check_device()) return st;
        const void* Bs[1] = {l->w16};
        float* Cs[1] = {y_dev};
        HIP_TRY(a81w41::launch_gemv_fused(x_dev, ctx->act_scratch, 1, Bs, Cs, &l->N, l->K,
                                          static_cast<hipStream_t>(stream)));
        return A81W41_OK;
    }
    if (int st = a81w41_quantize_row_q8_1_repack_fp16(x_dev, ctx->act_scratch, (int64_t)M * l->K, stream)) return st;
    return a81w41_gemv_repack_A81W41_fp16(ctx->act_scratch, l->w16, y_dev, M, l->N, l->K, stream);
}

int a81w41_linear_forward_quantized(a81w41_linear* l, const void* a_blob_dev, int M, float* y_dev, void* stream) {
    if (!l || !a_blob_dev || !y_dev) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (M < 2) return fail(A81W41_ERR_INVALID_ARG, "M must be >= 2 (80 B blocks are the M > 1 format), got %d", M);
    if (!l->w32) return fail(A81W41_ERR_INVALID_ARG, "layer has no fp32-parameter blob (needed for M > 1)");
    a81w41_context* ctx = l->ctx;
    if ((int64_t)M * l->K > ctx->max_elems)
        return fail(A81W41_ERR_INVALID_ARG, "M*K = %lld exceeds the context's scratch (%lld)", (long long)M * l->K,
                    (long long)ctx->max_elems);
    if (int st = contract_args_ok(a_blob_dev, l->w32, y_dev, M, l->N, l->K)) return st;
    if (reinterpret_cast<uintptr_t>(a_blob_dev) & 15)
        return fail(A81W41_ERR_INVALID_ARG, "activation blob must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (a81w41::linear_block_scaled(l, M)) {
        HIP_TRY(a81w41::launch_a80_to_a6(a_blob_dev, ctx->a6_scratch, M, l->K, s));
        HIP_TRY(a81w41::launch_gemm_fp6(ctx->a6_scratch, l->w6, y_dev, M, l->N, l->K, ctx->gemm_scratch, s));
        return A81W41_OK;
    }
    HIP_TRY(a81w41::launch_gemm_fp32(a_blob_dev, l->w32, y_dev, M, l->N, l->K, ctx->gemm_scratch, s));
    return A81W41_OK;
}

int a81w41_linear_set_kernel(a81w41_linear* l, int choice) {
    if (!l) return fail(A81W41_ERR_INVALID_ARG, "null layer");
    if (choice != A81W41_KERNEL_AUTO && choice != A81W41_KERNEL_INT8 && choice != A81W41_KERNEL_BLOCK_SCALED)
        return fail(A81W41_ERR_INVALID_ARG, "unknown kernel choice %d", choice);
    if (choice == A81W41_KERNEL_INT8) {  // the third weight copy is of no use any more
        HIP_TRY(hipDeviceSynchronize());
        (void)hipFree(l->w6);
        l->w6 = nullptr;
    } else if (l->w32 && (choice == A81W41_KERNEL_BLOCK_SCALED || a81w41::gemm_fp6_preferred(max_rows_of(l->ctx, l->K), l->N, l->K))) {
        HIP_TRY(build_w6(l));  // allocates and synchronises: not for a stream that is being captured
    }
    l->kernel_choice = choice;
    return A81W41_OK;
}

int a81w41_linear_forward_multi(int n, a81w41_linear* const* layers, const float* x_dev, int M,
                                float* const* ys_dev, void* stream) {
    if (n < 1 || !layers || !ys_dev || !x_dev) return fail(A81W41_ERR_INVALID_ARG, "null pointer or n < 1");
    for (int i = 0; i < n; i++) {
        if (!layers[i] || !ys_dev[i]) return fail(A81W41_ERR_INVALID_ARG, "null layer or output %d", i);
        if (layers[i]->K != layers[0]->K || layers[i]->ctx != layers[0]->ctx)
            return fail(A81W41_ERR_INVALID_ARG, "layers of one call must share K and the context");
    }
    a81w41_linear* l0 = layers[0];
    if (l0->ctx->chain_ready && l0->ctx->chain.open) {
        if (n > a81w41::kGemvMaxBatch)
            return fail(A81W41_ERR_INVALID_ARG, "at most %d layers per call while a chain is open", a81w41::kGemvMaxBatch);
        const void* Bs[a81w41::kGemvMaxBatch];
        float* Cs[a81w41::kGemvMaxBatch];
        int Ns[a81w41::kGemvMaxBatch];
        for (int j = 0; j < n; j++) {
            Bs[j] = layers[j]->w16;
            Cs[j] = ys_dev[j];
            Ns[j] = layers[j]->N;
        }
        return chained_forward(l0->ctx, n, Bs, Cs, Ns, l0->K, x_dev, M, stream);
    }
    const bool one_launch = M == 1 && (reinterpret_cast<uintptr_t>(x_dev) & 15) == 0 &&
                            a81w41::gemv_lds_bytes(l0->K) <= a81w41::kLdsLimitBytes;
    if (!one_launch) {  // same results, one call per layer (each re-quantises x into the scratch)
        for (int i = 0; i < n; i++)
            if (int st = a81w41_linear_forward(layers[i], x_dev, M, ys_dev[i], stream)) return st;
        return A81W41_OK;
    }
    if (int st = check_device()) return st;
    for (int i0 = 0; i0 < n; i0 += a81w41::kGemvMaxBatch) {
        const int cnt = n - i0 < a81w41::kGemvMaxBatch ? n - i0 : a81w41::kGemvMaxBatch;
        const void* Bs[a81w41::kGemvMaxBatch];
        float* Cs[a81w41::kGemvMaxBatch];
        int Ns[a81w41::kGemvMaxBatch];
        for (int j = 0; j < cnt; j++) {
            if (!layers[i0 + j]->w16) return fail(A81W41_ERR_INVALID_ARG, "layer %d has no fp16-parameter blob", i0 + j);
            Bs[j] = layers[i0 + j]->w16;
            Cs[j] = ys_dev[i0 + j];
            Ns[j] = layers[i0 + j]->N;
        }
        HIP_TRY(a81w41::launch_gemv_fused(x_dev, l0->ctx->act_scratch, cnt, Bs, Cs, Ns, l0->K,
                                          static_cast<hipStream_t>(stream)));
    }
    return A81W41_OK;
}

int a81w41_linear_forward_host(a81w41_linear* l, const float* x_host, int M, float* y_host) {
    if (!l || !x_host || !y_host) return fail(A81W41_ERR_INVALID_ARG, "null pointer");
    if (M < 1) return fail(A81W41_ERR_INVALID_ARG, "M must be >= 1, got %d", M);
    a81w41_context* ctx = l->ctx;
    const size_t xb = (size_t)M * l->K * 4, yb = (size_t)M * l->N * 4;
    if (xb > ctx->x_bytes) {
        (void)hipFree(ctx->x_stage);
        ctx->x_stage = nullptr;
        ctx->x_bytes = 0;
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&ctx->x_stage), xb));
        ctx->x_bytes = xb;
    }
    if (yb > ctx->y_bytes) {
        (void)hipFree(ctx->y_stage);
        ctx->y_stage = nullptr;
        ctx->y_bytes = 0;
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&ctx->y_stage), yb));
        ctx->y_bytes = yb;
    }
    HIP_TRY(hipMemcpy(ctx->x_stage, x_host, xb, hipMemcpyHostToDevice));
    if (int st = a81w41_linear_forward(l, ctx->x_stage, M, ctx->y_stage, nullptr)) return st;
    HIP_TRY(hipMemcpy(y_host, ctx->y_stage, yb, hipMemcpyDeviceToHost));  // synchronises the default stream
    return A81W41_OK;
}

}  // extern "C"
