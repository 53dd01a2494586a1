// Internal launcher interface between the C ABI (capi.cpp, qwen3_model.cpp) and the HIP kernels.
// Every launcher validates nothing: the callers check shapes and alignment first.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "chain.h"

namespace a81w41 {

// Environment overrides of the kernel selection exist in tuning builds only (make TUNING=1); the
// default build never reads the environment.
inline const char* tuning_env(const char* name) {
#ifdef A81W41_TUNING
    return getenv(name);
#else
    (void)name;
    return nullptr;
#endif
}
inline int tuning_env_int(const char* name) {
    const char* v = tuning_env(name);
    return v ? atoi(v) : 0;
}

constexpr int kWBlock16 = 320;  // q4_repack_2x8_fp16
constexpr int kWBlock32 = 384;  // q4_repack_2x8_fp32
constexpr int kABlock16 = 72;   // q8_repack_1x2_fp16
constexpr int kABlock32 = 80;   // q8_repack_1x2_fp32

// write_sums = false: the scaled-sum fields of the blocks are left as they are
// (quantize_row_q8_0_repack, quantized_gemx_kernels.cc:584-682).
// y_by_superblock (fp32 parameters, at most 32 rows of nb_k super-blocks; may be null): a second copy of the blocks,
// block (row, sb) at (32 sb + row) * 80, for launch_gemm_rows32_fp32's staged form.
hipError_t launch_quantize(const float* x, void* y, int64_t nb64, bool fp32, hipStream_t s, bool write_sums = true,
                           void* y_by_superblock = nullptr, int nb_k = 0);
// Persistent GEMV grid: at most this many workgroups (8 per CU on 256 CUs).
constexpr int kGemvMaxGrid = 2048;
constexpr int kLdsLimitBytes = 160 * 1024;
int gemv_lds_bytes(int K);
int gemv_max_k();  // the longest row whose quantised form fits the LDS next to the reduction areas
hipError_t launch_gemv_fp16(const void* A, const void* B, float* C, int N, int K, hipStream_t s);
// Same contraction with the fp16-parameter quantiser fused in front: x is K fp32
// values (16-byte aligned); a_out (may be null) receives the K/64 72 B blocks.
// n_mat <= kGemvMaxBatch weight matrices that share x and K go in one launch.
constexpr int kGemvMaxBatch = 4;
hipError_t launch_gemv_fused(const float* x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs,
                             const int* Ns, int K, hipStream_t s);
// Variants of the fused M = 1 launch whose activation row is computed in the prologue:
//   silu_mul : x[j] = silu(gate_up[j]) * gate_up[K + j]  (gate_up: 2K fp32, 16-byte aligned)
//   add_norm : r = x + res_in (res_in may be null); x' = r / sqrt(mean(r^2) + eps) * norm_w;
//              workgroup 0 writes r to res_out, which must not be the buffer of x or res_in
//              (other workgroups are still reading those).  Needs gemv_add_norm_fits(K).
struct GemvPrologue {
    const float* res_in = nullptr;
    float* res_out = nullptr;
    const float* norm_w = nullptr;
    float eps = 0.f;
    uint8_t* pair_out = nullptr;  // launch_gemv_add_norm_silu_pair: the 72 B blocks of silu(gate) * up
};
hipError_t launch_gemv_silu_mul(const float* gate_up, void* a_out, const void* B, float* C, int N, int K, hipStream_t s);
bool gemv_add_norm_fits(int K);
hipError_t launch_gemv_add_norm(const float* x, const GemvPrologue& pro, void* a_out, const void* B, float* C, int N,
                                int K, hipStream_t s);
// add_norm in front, and behind it, instead of the N = 2 I outputs of a gate|up matrix (gate rows, then
// up rows), the quantised 72 B blocks of silu(gate) * up in pro.pair_out: the next linear's input, to
// be contracted with launch_gemv_fp16.  I % 32 == 0; needs gemv_add_norm_fits(K).
bool gemv_pair_fits(int N, int K);
hipError_t launch_gemv_add_norm_silu_pair(const float* x, const GemvPrologue& pro, const void* B_gate_up, int N, int K,
                                          hipStream_t s);
int gemv_waves_per_group_log2(int nb_n, int nb_k, bool paired_output);

// ---- chains of overlapping launches, host side (chain.hip; the device side is in chain.h) ----------------------
// Between chain_begin and chain_end every launch is a link: it goes to the stream chain_next names (the caller's
// stream and the chain's own side stream in turn), waits inside the kernel for the link before it, and its
// workgroup count is reported with chain_launched.  Works under stream capture (the side stream joins the capture
// through the fork event and leaves it through the join event).
constexpr int kChainRing = 4;  // completion counters in rotation; the status word follows them
struct ChainState {
    unsigned* counters = nullptr;  // device
    hipStream_t side = nullptr, main = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool open = false;
    int n = 0;               // launches of the open chain so far
    unsigned prev_grid = 0;  // workgroups of the last one
    unsigned spin_limit = 1u << 16;  // polls (about a microsecond each) before a wait gives up
    int cus = 0;
};
hipError_t chain_create(ChainState* st);
void chain_destroy(ChainState* st);
hipError_t chain_begin(ChainState* st, hipStream_t main);
ChainLink chain_next(const ChainState* st, hipStream_t* stream);
void chain_launched(ChainState* st, unsigned grid);
hipError_t chain_end(ChainState* st);  // the caller's stream waits for the side stream; clears the last counter
// Synchronises both streams; *gave_up = some wait of a chain since the last call gave up (counters are then reset).
hipError_t chain_status(ChainState* st, bool* gave_up);
// The same launches as links of a chain of overlapping launches (chain.h, gemv_chain_a81w41.hip): same bits as
// the plain launches while K < 16384; at most `cus` workgroups of 8 waves; *grid_out = workgroups launched (what
// the next link waits for).  gemv_chain_fits: K a multiple of 64, the quantised row within 64 KiB of LDS, and
// for the add + norm prologue K <= 4096.
bool gemv_chain_fits(int K, bool add_norm);
hipError_t launch_gemv_chain_blob(const void* A, const void* B, float* C, int N, int K, const ChainLink& link, int cus,
                                  unsigned* grid_out, hipStream_t s);
hipError_t launch_gemv_chain_fused(const float* x, void* a_out, int n_mat, const void* const* Bs, float* const* Cs,
                                   const int* Ns, int K, const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s);
hipError_t launch_gemv_chain_add_norm(const float* x, const GemvPrologue& pro, void* a_out, const void* B, float* C, int N,
                                      int K, const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s);
hipError_t launch_gemv_chain_add_norm_silu_pair(const float* x, const GemvPrologue& pro, const void* B_gate_up, int N, int K,
                                                const ChainLink& link, int cus, unsigned* grid_out, hipStream_t s);
// Scratch of the GEMM's K-split path: partial tiles and their arrival counters (zero between launches).
// Launches that share a scratch must not overlap in time.
struct GemmScratch {
    float* partials = nullptr;
    unsigned* arrivals = nullptr;
    int max_partials = 0;
};
hipError_t gemm_scratch_create(GemmScratch* out);  // 64 MiB + counters on the current device
void gemm_scratch_destroy(GemmScratch* ws);
size_t gemm_scratch_bytes(const GemmScratch& ws);
// The scratch that belongs to stream s on the current device, created at the first call for that stream
// (which therefore must not come while s is being captured: hipErrorStreamCaptureUnsupported).
hipError_t gemm_scratch_for_stream(hipStream_t s, GemmScratch* out);
// The current device's copy of the library's file-scope scratch array (nothing is allocated).
hipError_t gemm_static_scratch(GemmScratch* out);
int gemm_static_scratch_tiles();
// Partial tiles the schedule of an M x N x K call parks (0: no K split); -1 if the device cannot be queried.
int gemm_partial_tiles(int M, int N, int K);
hipError_t clear_gemm_counters(const GemmScratch& ws, hipStream_t s);
// hipErrorInvalidValue if the call's schedule needs more partial tiles than ws holds.
hipError_t launch_gemm_fp32(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws, hipStream_t s);
// Which of the M > 1 kernels launch_gemm_fp32 sends a call of this shape to (a name for reports).
const char* gemm_kernel_name(int M, int N, int K);
// Walks the work list of a launch of the 64 x 64-tile kernel on the host for a device with
// slots_fit resident workgroups on cus CUs: >= 0 (the partial tiles used) if every tile and chunk is
// covered exactly once and no partial tile is shared, else a negative code.
int gemm_schedule_selfcheck(int M, int N, int K, int slots_fit, int cus);
// ---- the layer object's M > 32 path: block-scaled fp6 matrix ops on private operand formats (gemm_fp6_a81w41.hip)
// A6: quantised activations as two 4-bit pieces per value in fp6 patterns, W6: weight codes as fp6 patterns,
// both with fp32 parameters, in 32-row / 32-column panels.  Rows and columns are padded to multiples of 32.
constexpr int kGemmFp6MinRows = 33;  // calls with fewer rows stay on the int8 kernels
// Whether a call of this shape goes to the block-scaled kernel (false: the int8 kernels are as fast or faster).
bool gemm_fp6_preferred(int M, int N, int K);
size_t gemm_fp6_a6_bytes(int64_t rows, int K);
size_t gemm_fp6_w6_bytes(int N, int K);
hipError_t launch_w384_to_w6(const void* w384, void* w6, int N, int K, hipStream_t s);  // once per layer
// fp32 rows -> 80 B blocks (y80, may be null: exactly what launch_quantize(fp32) writes) and A6
hipError_t launch_quantize_a6(const float* x, void* y80, void* a6, int M, int K, hipStream_t s);
hipError_t launch_a80_to_a6(const void* y80, void* a6, int M, int K, hipStream_t s);  // rows already in 80 B blocks
// C[M][N]; hipErrorInvalidValue if ws is smaller than a context's scratch
hipError_t launch_gemm_fp6(const void* a6, const void* w6, float* C, int M, int N, int K, const GemmScratch& ws, hipStream_t s);
// Host-side walk of a launch's work units for a device holding `slots` workgroups: >= 0 (tiles whose K range is
// shared between workgroups) if every (tile, block) is covered once and the partial-tile slots are consistent.
int gemm_fp6_plan_selfcheck(int M, int N, int K, int slots);

// Few-row variant (M <= 8, activation rows resident in LDS, no matrix cores), used by
// launch_gemm_fp32 when gemm_rows_fits(): same arguments and results within the same tolerance.
bool gemm_rows_fits(int M, int K);
hipError_t launch_gemm_rows_fp32(const void* A, const void* B, float* C, int M, int N, int K, hipStream_t s);
// The same with the fp32-parameter quantiser fused in front (x: M x K fp32, 16-byte aligned; a_out, may be null,
// receives the M*K/64 blocks of 80 B): one launch for quantiser + contraction, where that is the faster form.
bool gemm_rows_fused_preferred(int M, int K);
hipError_t launch_gemm_rows_fused(const float* x, void* a_out, const void* B, float* C, int M, int N, int K, hipStream_t s);
// 9 <= M <= 32: one row panel, operands loaded straight into registers, K cut inside and between workgroups.
int gemm_rows32_split(int N, int K, bool staged = false);
// staged: operands through wave-private LDS stages (wide layers); a_by_superblock (staged only, may be null): the copy of
// A that launch_quantize writes with a super-block's rows next to each other (32 row slots per super-block).
hipError_t launch_gemm_rows32_fp32(const void* A, const void* B, float* C, int M, int N, int K, const GemmScratch& ws,
                                   hipStream_t s, bool staged = false, const void* a_by_superblock = nullptr);
bool gemm_rows32_staged_preferred(int M, int N, int K);  // whether launch_gemm_fp32 would take the staged form
size_t gemm_rows32_a_by_superblock_bytes(int K);
// w80: codes count as code - 8 (the A80W40 variant).
hipError_t launch_block_idot(const void* A, bool a_fp32, const void* B, bool b_fp32, int32_t* out,
                             int M, int N, int K, hipStream_t s, bool w80 = false);

// ---- the A80W40 variant: 72 B / 320 B blocks, codes read as code - 8, no min term ----------
hipError_t launch_gemv_a80w40(const void* A, const void* B, float* C, int N, int K, hipStream_t s);
// M x N from fp16-parameter blocks on both sides (gemm_repack_A80W40): both operands are
// rewritten into the workspace as 80 B / 384 B blocks with min = -8 d_w and
// scaled sum = d_a * sum(q) (both exact), then contracted by launch_gemm_fp32.
size_t gemm_a80w40_workspace_bytes(int M, int N, int K);
hipError_t launch_gemm_a80w40(const void* A, const void* B, float* C, int M, int N, int K, void* workspace,
                              const GemmScratch& ws, hipStream_t s);


}  // namespace a81w41
struct a81w41_context;
namespace a81w41 {
// The K-split scratch a context owns, and its A6 scratch (capi.cpp).
const GemmScratch& context_gemm_scratch(const a81w41_context* ctx);
size_t context_resident_bytes(const a81w41_context* ctx);  // its scratches
ChainState* context_chain(a81w41_context* ctx);
void* context_a6_scratch(const a81w41_context* ctx);
}  // namespace a81w41
struct a81w41_linear;
namespace a81w41 {
const void* linear_w6(const a81w41_linear* layer);  // null if the layer has no fp32-parameter blob
bool linear_block_scaled(const a81w41_linear* layer, int M);  // an M-row call of this layer contracts on the block-scaled kernel

// Records `message` as the calling thread's last error and returns `status` (capi.cpp).
int report_failure(int status, const char* message);
// IEEE binary32 -> binary16, round to nearest even (host, capi.cpp).
uint16_t float_to_half_bits(float f);

// ---- operators around the linears in the Qwen3 forward pass (qwen3_ops.hip) ----------------
// head_dim is 128; positions are read from device memory (pos_dev[0] = tokens already cached).
hipError_t launch_embed_rows(const int* ids, const void* table_fp16, float* out, int M, int hidden, int vocab, hipStream_t s);
hipError_t launch_add_rmsnorm(const float* x, const float* res_in, const float* w, float* res_out, float* norm_out, int M,
                              int hidden, float eps, hipStream_t s);
// Same, with the normalised rows written as 80 B activation blocks (what the fp32-parameter
// quantiser would make of norm_out) to q_out.  hidden % 64 == 0.
hipError_t launch_add_rmsnorm_quant(const float* x, const float* res_in, const float* w, float* res_out, void* q_out, int M,
                                    int hidden, float eps, hipStream_t s);
hipError_t launch_qk_norm_rope_cache(float* qkv, int row_stride, int M, int n_q, int n_kv, const float* q_w, const float* k_w,
                                     const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache, void* v_cache,
                                     int max_seq, float eps, hipStream_t s);
size_t attention_lds_bytes(int max_seq, int threads);
// variant 0: matrix cores when attention_prefill_fits(), else the vector kernel; 1: always the vector kernel.
hipError_t launch_attention(const float* q, int q_row_stride, const void* k_cache, const void* v_cache, const int* pos_dev,
                            float* out, int out_row_stride, int M, int n_q, int n_kv, int max_seq, float scale, hipStream_t s,
                            int variant = 0);
// Matrix-core variant for many new tokens (M > 8, n_q / n_kv in {1, 2, 4, 8}); launch_attention uses it
// when attention_prefill_fits().  Same arguments and, to rounding noise, the same results.
bool attention_prefill_fits(int M, int n_q, int n_kv);
// With q_out the result goes there as the 80 B activation blocks of the [M][n_q*128] rows (what the
// fp32-parameter quantiser would make of them) and out is not written.  heads_per_workgroup: 0 = chosen
// from the number of query tiles, else 1, 2, 4 or 8 (a divisor of n_q / n_kv).
hipError_t launch_attention_prefill(const float* q, int q_row_stride, const void* k_cache, const void* v_cache,
                                    const int* pos_dev, float* out, int out_row_stride, int M, int n_q, int n_kv, int max_seq,
                                    float scale, hipStream_t s, void* q_out = nullptr, int heads_per_workgroup = 0);
// qk_norm_rope_cache + attention for one new token in one launch (qkv: that token's fused row).
// The result goes to out as fp32, or, if q_out is not null, to q_out as the 72 B activation blocks
// the fp16-parameter quantiser would make of it (out is then not written).
hipError_t launch_attention_one_token(const float* qkv, int n_q, int n_kv, const float* q_w, const float* k_w,
                                      const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache, void* v_cache,
                                      float* out, void* q_out, int max_seq, float eps, float scale, hipStream_t s,
                                      const ChainLink* link = nullptr);  // link: the launch is a link of a chain (chain.h)
// The same with the context of every head cut into `splits` (<= kAttentionMaxSplits) shares, one workgroup
// each, for long contexts.  partials: n_q * splits * 132 floats; arrivals: n_q counters, zero before the
// first launch (every launch leaves them zero).  Launches that share them must not overlap in time.
constexpr int kAttentionMaxSplits = 16;
hipError_t launch_attention_one_token_split(const float* qkv, int n_q, int n_kv, const float* q_w, const float* k_w,
                                            const float* cos_t, const float* sin_t, const int* pos_dev, void* k_cache,
                                            void* v_cache, float* out, void* q_out, float* partials, unsigned* arrivals,
                                            int splits, int max_seq, float eps, float scale, hipStream_t s,
                                            const ChainLink* link = nullptr);
hipError_t launch_silu_mul(const float* gate_up, float* out, int M, int inter, hipStream_t s);
// silu(gate) * up as 80 B activation blocks of the [M][inter] result.  inter % 64 == 0, gate_up 16-byte aligned.
hipError_t launch_silu_mul_quant(const float* gate_up, void* q_out, int M, int inter, hipStream_t s);
hipError_t launch_argmax_token(const float* logits, int n, int* next_id, int* history, int history_len, int* step_dev,
                               hipStream_t s);
hipError_t launch_advance(int* pos_dev, int by, hipStream_t s);

}  // namespace a81w41
