/*
 * a81w41.h -- C ABI of the MI355X (gfx950) A81W41 quantized linear layer.
 *
 * Drop-in boundary for the reference's linear-layer hot path: Q8_1-style
 * activation quantisation, Q4_1-style int4 weights in the 8-column x 64-K
 * interleaved block packing, and the GEMV / GEMM that contracts them with the
 *     d_w * d_a * sum(q_w * q_a) + m_w * s_a
 * epilogue into fp32.  Blob layouts are byte-for-byte the reference's
 * (qwen3/include/qwen/QwenOperator.h:48-80):
 *
 *   weights, fp16 params : 320 B per (8 columns x 64 K)   fp16 s_low[8] s_high[8] min_low[8] min_high[8]; u8 q_coupled[256]
 *   weights, fp32 params : 384 B                          same with fp32 params
 *   activations, fp16    :  72 B per 64 K                 fp16 s_low s_high scaled_sum_low scaled_sum_high; i8 q_low[32] q_high[32]
 *   activations, fp32    :  80 B                          same with fp32 params
 *   block (g = n/8, sb = k/64) of a weight blob sits at index g*(K/64)+sb.
 *
 * Every function returns an a81w41_status (0 = ok) instead of the reference's
 * asserts; a81w41_last_error() gives the message of the calling thread's last
 * failure.  "dev" pointers are device (HBM) addresses, `stream` is a
 * hipStream_t passed as void* (NULL = the default stream); device entry points
 * only enqueue work and do not synchronise.  There is no CPU fallback.
 */
#ifndef A81W41_H
#define A81W41_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define A81W41_QK 32               /* quantisation group, QwenConfig.h:8 */
#define A81W41_W_BLOCK_FP16 320
#define A81W41_W_BLOCK_FP32 384
#define A81W41_A_BLOCK_FP16 72
#define A81W41_A_BLOCK_FP32 80

typedef enum {
    A81W41_OK = 0,
    A81W41_ERR_INVALID_ARG = 1, /* shape / alignment / null pointer: what the reference asserts on */
    A81W41_ERR_HIP = 2,         /* a HIP runtime call failed */
    A81W41_ERR_IO = 3,          /* weight file missing or short (reference: std::runtime_error) */
    A81W41_ERR_NO_DEVICE = 4    /* no gfx950 device visible */
} a81w41_status;

const char *a81w41_status_string(int status);
const char *a81w41_last_error(void);

/* Bytes of a repacked weight blob for a K x N layer, and of the quantised form
 * of k activations (k = M*K).  fp32 != 0 selects the fp32-parameter layouts. */
size_t a81w41_weight_blob_bytes(int K, int N, int fp32);
size_t a81w41_act_blob_bytes(int64_t k, int fp32);

/* ---- load time, host memory ------------------------------------------------
 * Replace repack_w81_weight_fp16 / repack_w81_weight_fp32
 * (QwenOperator.h:83-84, QwenOperator.cc:801-892): same argument order.
 * B is weight_int4.bin [N][K/2], SB / MinB are scaling_factor_int4.bin /
 * offset_int4.bin [N][K/32], B_repack receives N*K/512 blocks.
 * Requires K % 64 == 0, N % 8 == 0, Q_BLK_SIZE == 32. */
int a81w41_repack_w81_weight_fp16(int K, int N, int Q_BLK_SIZE, void *B_repack, const float *SB,
                                  const float *MinB, const uint8_t *B);
int a81w41_repack_w81_weight_fp32(int K, int N, int Q_BLK_SIZE, void *B_repack, const float *SB,
                                  const float *MinB, const uint8_t *B);

/* Offline weight quantiser that produces those three files: quantize_row_q41_tinyml,
 * notebooks/quantize_methods.py:68-125.  w is fp32 [N][K] (PyTorch's out x in); per
 * 32-block d = (max-min)/15, id = 1/d (0 if d == 0), code = clip(rne((x-min)*id), 0, 15),
 * byte e of a 64-K super-block = code[e] | code[32+e] << 4.  scale = d, offset = min.
 * Host memory, load time.  Requires K % 64 == 0. */
int a81w41_quantize_weight_q41(const float *w, int N, int K, uint8_t *weight_int4, float *scale,
                               float *offset);

/* ---- device kernels --------------------------------------------------------
 * Replace quantize_row_q8_1_repack_fp16 / _fp32 (QwenOperator.h:277-278,
 * quantized_gemx_kernels.cc:693-911).  x_dev: k floats, vy_dev: k/64 blocks.
 * k % 64 == 0.  Bit-exact with the reference for finite inputs. */
int a81w41_quantize_row_q8_1_repack_fp16(const float *x_dev, void *vy_dev, int64_t k, void *stream);
int a81w41_quantize_row_q8_1_repack_fp32(const float *x_dev, void *vy_dev, int64_t k, void *stream);

/* Replace gemv_repack_A81W41_fp16 (QwenOperator.h:299-304,
 * quantized_gemx_kernels.cc:111-193): C[0..N) = row 0 of A (72 B blocks)
 * against the 320 B weight blob; M is ignored like in the reference; C is
 * fully overwritten. */
int a81w41_gemv_repack_A81W41_fp16(const void *A_repack_dev, const void *B_repack_dev, float *C_dev,
                                   int M, int N, int K, void *stream);

/* Replace gemm_repack_A81W41_fp32 (QwenOperator.h:293-298,
 * quantized_gemx_kernels.cc:349-582): C[M][N] row-major from 80 B activation
 * blocks and the 384 B weight blob.  Any M >= 1 (rows past M are never read).
 * Calls with M > 8 may split the K range of some tiles and park partial tiles in a
 * scratch (64 MiB) that belongs to `stream`: it is allocated by the first such call on
 * that stream (which therefore cannot be captured into a graph; later calls can) and kept
 * until the process ends.  A device keeps at most 16 of them: the first call on a 17th
 * stream waits for the device to be idle and takes over the scratch of the stream that
 * used its own longest ago (streams come and go; their scratches are reused).  Calls on one
 * stream are ordered by the stream, calls on different streams use different scratches, so
 * no two launches share partial tiles -- with one caveat: a captured graph keeps the
 * scratch of the stream it was captured on wherever it is replayed, so its replays must
 * not overlap with K-split calls on that stream.  Results do not depend on timing. */
int a81w41_gemm_repack_A81W41_fp32(const void *A_repack_dev, const void *B_repack_dev, float *C_dev,
                                   int M, int N, int K, void *stream);

/* The same contraction for callers that cannot allocate device memory (code under HIP graph
 * capture from the first call on, tight serving loops, harnesses that forbid it).  No
 * counterpart in the reference.  Same arguments and the same results bit for bit as
 * a81w41_gemm_repack_A81W41_fp32; never calls hipMalloc / hipFree.  The partial tiles of the K
 * split go to a file-scope device array of the library: 2048 tiles = 32 MiB plus 8 KiB of
 * counters, held by every GPU the library runs on from load to process end.  A shape whose
 * schedule parks more partial tiles than that (on a 256-CU device only launches of 683 .. 767
 * tiles of 64 x 64 over K >= 12288, e.g. M = 700 on 12288 -> 4096) is rejected with A81W41_ERR_INVALID_ARG.  All calls
 * on one GPU share the array, whatever their streams: calls that overlap in time race. */
int a81w41_gemm_repack_A81W41_fp32_static(const void *A_repack_dev, const void *B_repack_dev,
                                          float *C_dev, int M, int N, int K, void *stream);

/* Test hook, host only (no device is touched): walks the work list the 64 x 64-tile kernel would be
 * launched with for an M x N x K call on a device that holds `resident_workgroups` of its workgroups on
 * `cus` compute units.  Returns the number of
 * partial tiles the K split parks (>= 0) if every tile and every K chunk is covered exactly
 * once, the tile numbering is one-to-one and no two chunks share a partial tile; a negative
 * code names the violated property. */
int a81w41_gemm_schedule_selfcheck(int M, int N, int K, int resident_workgroups, int cus);

/* Test hook, host only: the same for the layer object's M > 32 kernel (128 x 128 tiles, the (tile,
 * 32-block) units of a launch cut into equal contiguous runs): every unit exactly once, contributor
 * ranges and partial-tile slots consistent.  Returns the number of tiles shared between workgroups. */
int a81w41_gemm_fp6_plan_selfcheck(int M, int N, int K, int resident_workgroups);

/* The int32 block dots both kernels form before scaling (iacc_low / iacc_high,
 * quantized_gemx_kernels.cc:161-168 and :430-457), exposed for parity checks:
 * out_dev[(m*N + n)*(K/32) + 2*sb + h], h = 0 low / 1 high 32-block.
 * a_fp32 / b_fp32 select the 80 B / 384 B layouts. */
int a81w41_block_idot(const void *A_repack_dev, int a_fp32, const void *B_repack_dev, int b_fp32,
                      int32_t *out_dev, int M, int N, int K, void *stream);

/* ---- the A80W40 variant -------------------------------------------------------------------
 * The symmetric twin of the path: the same 320 B weight and 72 B activation blocks, int4
 * codes that mean code - 8, no mins and no scaled sums,
 *     C[m][n] = sum over 32-blocks of d_w * d_a * sum((code - 8) * q).
 * The reference keeps these free functions but never calls them.  The min_* fields of the
 * weight blocks and the scaled_sum_* fields of the activation blocks are neither written
 * nor read by any function of this group, exactly like in the reference. */
/* Replaces repack_w80_weight (QwenOperator.h:82, QwenOperator.cc:757-799).  Host memory. */
int a81w41_repack_w80_weight(int K, int N, int Q_BLK_SIZE, void *B_repack, const float *SB,
                             const uint8_t *B);
/* Offline weight quantiser of the variant: quantize_row_q40_tinyml,
 * notebooks/quantize_methods.py:12-66.  Per 32-block d = (element of largest magnitude) / -8,
 * id = 1/d (0 if d == 0), code = uint8(clip(x*id + 8.5, 0, 15)); bytes paired as for q41.
 * The notebook's offsets are all 0 and its zero points all 8: not produced.  Host memory. */
int a81w41_quantize_weight_q40(const float *w, int N, int K, uint8_t *weight_int4, float *scale);
/* Replaces quantize_row_q8_0_repack (QwenOperator.h:276, quantized_gemx_kernels.cc:584-682):
 * 72 B blocks with fp16 scales and the int8 payload. */
int a81w41_quantize_row_q8_0_repack(const float *x_dev, void *vy_dev, int64_t k, void *stream);
/* Replaces gemv_repack_A80W40 (QwenOperator.h:286-291, quantized_gemx_kernels.cc:39-109):
 * row 0 of A only, M ignored, C fully overwritten. */
int a81w41_gemv_repack_A80W40(const void *A_repack_dev, const void *B_repack_dev, float *C_dev,
                              int M, int N, int K, void *stream);
/* Replaces gemm_repack_A80W40 (QwenOperator.h:280-285, quantized_gemx_kernels.cc:195-347):
 * C[M][N] from 72 B activation blocks and the 320 B weight blob, any M >= 1 and any N % 8 == 0
 * (the reference's 2 x 2 blocking reads past the blob when N/8 is odd; this does not).
 * Both operands are first rewritten into `workspace_dev` in the 80 B / 384 B form of the
 * A81W41 contraction (min = -8 d_w, scaled sum = d_a * sum(q), both exact), which then runs
 * on the matrix cores; the same per-stream scratch as a81w41_gemm_repack_A81W41_fp32's is used.
 * The workspace is the caller's: 16-byte aligned, at least ..._workspace_bytes(M, N, K). */
size_t a81w41_gemm_repack_A80W40_workspace_bytes(int M, int N, int K);
int a81w41_gemm_repack_A80W40(const void *A_repack_dev, const void *B_repack_dev, float *C_dev,
                              int M, int N, int K, void *workspace_dev, size_t workspace_bytes,
                              void *stream);
/* The variant's int32 block dots sum((code - 8) * q), laid out like a81w41_block_idot's
 * (iacc_low / iacc_high, quantized_gemx_kernels.cc:85-91).  fp16-parameter blocks. */
int a81w41_block_idot_A80W40(const void *A_repack_dev, const void *B_repack_dev, int32_t *out_dev,
                             int M, int N, int K, void *stream);

/* ---- layer objects ---------------------------------------------------------
 * a81w41_context replaces ModelContext (QwenOperator.h:34-43): it owns the
 * device scratch every layer quantises its activations into, sized for
 * max_rows x max_cols activations (the reference sizes it for 4096 x 12288,
 * QwenForCausalLM.cc:101-113), and the 64 MiB of partial tiles its layers' M > 8 calls
 * may park.  Like the reference's, it is shared by all its layers, so forward calls on
 * one context must not overlap; calls on different contexts may. */
typedef struct a81w41_context a81w41_context;
typedef struct a81w41_linear a81w41_linear;

int a81w41_context_create(int max_rows, int max_cols, a81w41_context **out);
void a81w41_context_destroy(a81w41_context *ctx);
/* The scratch itself (context_->activation_buffer.get(), QwenOperator.cc:94): after a
 * forward call it holds that call's quantised activations, M*K/64 blocks of 72 B
 * (M == 1) or 80 B (M > 1), exactly as the reference's buffer does. */
void *a81w41_context_activation_scratch_dev(const a81w41_context *ctx);

/* Replaces the body of the Qwen_Linear_with_bias_Int4 constructor
 * (QwenOperator.h:112-157) after the four files are in memory: repacks the
 * host arrays twice (320 B and 384 B layouts) and uploads both blobs. */
int a81w41_linear_create(a81w41_context *ctx, int N, int K, const uint8_t *weight_int4,
                         const float *scale, const float *offset, a81w41_linear **out);
/* Same from already repacked host blobs (either may be NULL if that path is never used). */
int a81w41_linear_create_from_blobs(a81w41_context *ctx, int N, int K, const void *blob_fp16,
                                    const void *blob_fp32, a81w41_linear **out);
/* The constructor itself: reads <path>weight_int4.bin, scaling_factor_int4.bin,
 * offset_int4.bin (zero_point_int4.bin is loaded by the reference but never
 * used).  (dim_x, dim_y, dim_z) = (1, N, K) as in QwenOperator.h:112. */
int a81w41_linear_load(a81w41_context *ctx, const char *path, int dim_x, int dim_y, int dim_z,
                       a81w41_linear **out);
void a81w41_linear_destroy(a81w41_linear *layer);

/* Device memory the layer's weights occupy, in total and per copy: the reference's two blobs
 * (0.625 and 0.75 B per weight, QwenOperator.h:142-154) and, where the layer has it, the
 * block-scaled kernel's operand format (1 B per weight).  The third copy exists only for layers
 * that a call the context admits (max_rows x max_cols) can send to that kernel, or after
 * a81w41_linear_set_kernel(layer, A81W41_KERNEL_BLOCK_SCALED); A81W41_KERNEL_INT8 frees it.
 * Out-pointers may be NULL. */
size_t a81w41_linear_resident_bytes(const a81w41_linear *layer, size_t *fp16_blob, size_t *fp32_blob,
                                    size_t *block_scaled);
/* Which kernel a forward call of M rows of this layer runs on (a static string for reports:
 * "gemv ...", "rows ...", "rows_fused ...", "rows32 ...", "rows32_staged ...", "tile64 ...", "block_scaled ..."). */
const char *a81w41_linear_kernel_name(const a81w41_linear *layer, int M);
int a81w41_linear_in_features(const a81w41_linear *layer);  /* K */
int a81w41_linear_out_features(const a81w41_linear *layer); /* N */
const void *a81w41_linear_weight_fp16_dev(const a81w41_linear *layer);
const void *a81w41_linear_weight_fp32_dev(const a81w41_linear *layer);

/* Replaces Qwen_Linear_with_bias_Int4::forward (QwenOperator.h:224,
 * QwenOperator.cc:80-124): y[M][N] = linear(x[M][K]) with the reference's
 * dispatch -- M == 1: fp16-parameter quantiser + GEMV on the 320 B blob,
 * M > 1: fp32-parameter quantiser + GEMM on the 384 B blob.  Device pointers. */
int a81w41_linear_forward(a81w41_linear *layer, const float *x_dev, int M, float *y_dev, void *stream);
/* The contraction half of forward for M > 1 (QwenOperator.cc:104-108: the gemm_repack_A81W41_fp32
 * call on the context's buffer): rows that are already quantised, M*K/64 blocks of 80 B, 16-byte
 * aligned, contracted by whichever kernel the layer's forward would pick for M rows.  For callers
 * whose producer writes quantised blocks itself (as the model's norm, SiLU and attention epilogues
 * do), and for tests that need hand-made int8 rows. */
int a81w41_linear_forward_quantized(a81w41_linear *layer, const void *a_blob_dev, int M, float *y_dev,
                                    void *stream);
/* Which kernel M > 32 calls of this layer contract on.  The layer keeps, beside
 * the reference's two blobs, its fp32-parameter weights in the operand format of
 * gfx950's block-scaled matrix op (exact for these integers, twice the int8
 * rate); by default a call goes there when its shape is one where that kernel is
 * the faster one (A81W41_KERNEL_AUTO).  Its block dots are the reference's
 * integers bit for bit; its min terms fma(mW, sA, acc) are formed from bf16
 * pieces (sA exactly, as three; mW as two, i.e. to 16 significant bits, exact
 * for mins taken from bf16 or fp16 weights), so a call on that kernel agrees
 * with the int8 kernels to about 2e-5 of the row norm where they agree with
 * the reference to 1e-6 (the bar of the path is 1e-4).  The other two values
 * exist for tests, measurements and callers short of memory: A81W41_KERNEL_INT8
 * keeps every call on the int8 kernels and frees the layer's third weight copy,
 * A81W41_KERNEL_BLOCK_SCALED sends every call of more than 32 rows to the
 * block-scaled one, building that copy if the layer has none (this allocates and
 * synchronises: not on a stream that is being captured).  No counterpart in the
 * reference, which has one kernel per precision (quantized_gemx_kernels.cc:349). */
enum { A81W41_KERNEL_AUTO = 0, A81W41_KERNEL_INT8 = 1, A81W41_KERNEL_BLOCK_SCALED = 2 };
int a81w41_linear_set_kernel(a81w41_linear *layer, int choice);
/* Several layers applied to the same input in one call: ys_dev[i] = layers[i](x).
 * The reference does this by storing q, k and v as one 4096 -> 6144 layer
 * (QwenAttention.cc:29,78-83) and exports gate_up_proj the same way; here the
 * layers stay separate objects and, for M == 1, their column groups are
 * contracted by a single kernel launch (up to 4 layers per launch).  Results are
 * identical to n separate a81w41_linear_forward calls.  All layers must share K
 * and the context. */
int a81w41_linear_forward_multi(int n, a81w41_linear *const *layers, const float *x_dev, int M,
                                float *const *ys_dev, void *stream);
/* Same with host pointers (copies in, runs, copies out, synchronises): what a
 * caller holding Matrix3D<float> buffers uses. */
int a81w41_linear_forward_host(a81w41_linear *layer, const float *x_host, int M, float *y_host);

/* ---- chains of one-row calls that overlap ----------------------------------
 * A decode step is a chain of one-row linears, each waiting for the one before
 * (QwenDecoderLayer.cc:39-105).  Between chain_begin and chain_end the one-row
 * a81w41_linear_forward / _forward_multi calls of a context's layers are such a
 * chain: every call still depends on the call before it (its x may be that
 * call's y), exactly as on a stream, and returns the same bits as outside a
 * chain, but the launches take turns on two streams, so that a call starts
 * while its predecessor runs, requests its first weight blocks (which do not
 * depend on x), and waits for the predecessor inside the kernel.  Measured on
 * MI355X this hand-over is slower than the kernel boundary it replaces (the
 * counters and flags of a 256-workgroup launch are served one at a time on the
 * memory side of the eight L2s), so a chain is an option for experiments, not
 * the default path of anything.  Rules: calls
 * name the stream given to chain_begin; M == 1 only; x 16-byte aligned;
 * buffers the calls read or write are not touched by other work on the GPU
 * between begin and end; chain_end makes the caller's stream wait for the whole
 * chain.  Begin ... end may be captured into a HIP graph (stream capture) and
 * replayed.  Every in-kernel wait is bounded (spin limit in polls of roughly a
 * microsecond, default 65536): a wait that gives up sets a status word and the
 * kernels still run to their end; a81w41_context_chain_status synchronises,
 * reports it (results of that chain are then invalid) and clears it.
 * No counterpart in the reference, whose calls run one after the other on the
 * CPU. */
int a81w41_context_chain_begin(a81w41_context *ctx, void *stream);
int a81w41_context_chain_end(a81w41_context *ctx);
int a81w41_context_chain_status(a81w41_context *ctx, int *gave_up);
int a81w41_context_chain_set_spin_limit(a81w41_context *ctx, unsigned polls);
/* Test hook for the give-up path: one chained one-row call of `layer` whose wait nothing will
 * ever satisfy, with a spin limit of `polls`.  The kernel gives up, sets the status word, runs
 * to its end (y = layer(x) all the same, since x is there) and a81w41_context_chain_status then
 * reports gave_up = 1.  No chain may be open on the layer's context. */
int a81w41_context_chain_selfcheck_stuck_wait(a81w41_linear *layer, const float *x_dev, float *y_dev,
                                              unsigned polls, void *stream);


/* ---- the Qwen3 forward pass around the layer ---------------------------------------------
 * Replaces Qwen3ForCausalLM / Qwen3Model / Qwen3DecoderLayer / Qwen3Attention
 * (QwenForCausalLM.cc:11-60, QwenDecoder.cc:53-141, QwenDecoderLayer.cc:39-118,
 * QwenAttention.cc:52-208) for one token stream on one GPU: embedding, RMSNorm, the fused
 * q+k+v projection (QwenAttention.cc:29,78), per-head q/k RMSNorm, rotate-half RoPE, GQA
 * attention over a KV cache, o projection, gate+up projection, SiLU*mul, down projection,
 * residual adds, final norm, lm_head on the last token, greedy argmax.  Every linear is an
 * a81w41_linear with the reference's M-dispatch.  Differences from the reference, by design:
 * the KV cache is fp16 (the reference's is fp32), gate and up are one 2*intermediate-wide
 * linear, head_dim is fixed at 128. */
typedef struct {
    int n_layers, hidden, n_q_heads, n_kv_heads, intermediate, vocab;
    int max_seq;       /* KV-cache rows per head; also the longest prompt */
    float rope_theta;  /* 1e6 for Qwen3-8B */
    float rms_eps;     /* 1e-6, QwenOperator.h:242 */
} a81w41_qwen3_config;
typedef struct a81w41_qwen3 a81w41_qwen3;

/* Allocates buffers, KV cache and RoPE tables; weights are set afterwards. */
int a81w41_qwen3_create(const a81w41_qwen3_config *cfg, a81w41_qwen3 **out);
void a81w41_qwen3_destroy(a81w41_qwen3 *model);
/* The constructor chain Qwen3ForCausalLM -> Qwen3Model -> Qwen3DecoderLayer -> Qwen3Attention
 * (QwenForCausalLM.cc:71-121, QwenDecoder.cc:23-51, QwenDecoderLayer.cc:8-30,
 * QwenAttention.cc:13-47): creates the model and reads the reference's directory tree
 *   <root>/lm_head/{weight_int4,scaling_factor_int4,offset_int4}.bin
 *   <root>/model/embed_tokens/weight.bin (fp32), <root>/model/norm/weight.bin
 *   <root>/model/rotary_emb/{cos,sin}_cached.bin (optional; computed from rope_theta if absent)
 *   <root>/model/layers/layer<i>/{input_layernorm,post_attention_layernorm}/weight.bin
 *   <root>/model/layers/layer<i>/self_attn/{qkv_proj/,o_proj/,q_norm/weight.bin,k_norm/weight.bin,scaling.bin}
 *   <root>/model/layers/layer<i>/mlp/{gate_proj/,up_proj/,down_proj/}
 * gate_proj and up_proj are joined into the one gate_up linear. */
int a81w41_qwen3_load(const char *root, const a81w41_qwen3_config *cfg, a81w41_qwen3 **out);
/* which: 0 qkv_proj (N = (n_q+2 n_kv)*128, K = hidden), 1 o_proj, 2 gate_up_proj
 * (N = 2*intermediate: gate rows then up rows), 3 down_proj; layer -1: lm_head (which ignored).
 * Host arrays in the reference's file formats (see a81w41_linear_create). */
int a81w41_qwen3_set_linear(a81w41_qwen3 *model, int layer, int which, const uint8_t *weight_int4,
                            const float *scale, const float *offset);
/* Same from repacked host blobs (either may be NULL; lm_head needs only the fp16 one). */
int a81w41_qwen3_set_linear_blobs(a81w41_qwen3 *model, int layer, int which, const void *blob_fp16,
                                  const void *blob_fp32);
/* which: 0 input_layernorm [hidden], 1 post_attention_layernorm [hidden], 2 q_norm [128],
 * 3 k_norm [128]; layer -1: the final norm [hidden].  Host fp32. */
int a81w41_qwen3_set_norm(a81w41_qwen3 *model, int layer, int which, const float *weight);
/* Embedding table [vocab][hidden] as IEEE binary16 bit patterns, host. */
int a81w41_qwen3_set_embedding(a81w41_qwen3 *model, const uint16_t *table_fp16);
/* Test switches: each keeps one fusion of the one-token / prefill pass off, so that the fused
 * pass can be compared with the separate kernels, or fixes the attention's key split.  The
 * results of a pass do not change by a bit with UNFUSED, ATTN_FP32, NO_PAIR and CHAIN.
 * With CHAIN on, the one-token pass runs its linears and attention as a chain of overlapping
 * launches (see a81w41_context_chain_begin); a81w41_qwen3_chain_status reports whether a wait
 * of such a chain has given up since the last call. */
enum {
    A81W41_QWEN3_OPT_UNFUSED = 0,          /* separate elementwise kernels and quantiser launches */
    A81W41_QWEN3_OPT_ATTN_FP32 = 1,        /* one-token attention writes fp32, o_proj quantises it */
    A81W41_QWEN3_OPT_NO_PAIR = 2,          /* gate_up writes fp32, down_proj's prologue does SiLU*mul */
    A81W41_QWEN3_OPT_VECTOR_ATTENTION = 3, /* prefill attention on the vector kernel */
    A81W41_QWEN3_OPT_ATTENTION_SPLIT = 4,  /* value 1..16: shares per head of the one-token attention; 0: automatic */
    A81W41_QWEN3_OPT_CHAIN = 5,            /* one-token pass as a chain of overlapping launches (off by default: slower) */
    A81W41_QWEN3_OPT_CHAIN_SPIN_LIMIT = 6  /* value: polls before an in-kernel wait of the chained pass gives up; 0: default */
};
int a81w41_qwen3_set_option(a81w41_qwen3 *model, int option, int value);
int a81w41_qwen3_chain_status(a81w41_qwen3 *model, int *gave_up); /* synchronises */
/* Device memory the model holds, in total and by kind (out-pointers may be NULL): the linears'
 * weight copies (a81w41_linear_resident_bytes), the other weights (fp16 embedding table, norms,
 * rotation tables), the fp16 KV cache, and activation buffers + scratches.  The reference reports
 * 14.0 GiB resident for the same model with fp32 embedding and KV cache (README.md:41). */
size_t a81w41_qwen3_resident_bytes(const a81w41_qwen3 *model, size_t *linear_weights,
                                   size_t *other_weights, size_t *kv_cache, size_t *buffers);
/* Parity hook: copies the first `count` floats of one of the model's activation buffers to the host
 * after the work enqueued so far has finished.  After a pass the buffers hold what the LAST layer left
 * (the fused passes skip some of them: switch A81W41_QWEN3_OPT_UNFUSED on to have every stage written):
 * RESIDUAL [rows][hidden] the residual stream after the final add, NORMED its final RMSNorm,
 * QKV [rows][(n_q + 2 n_kv)*128] with q normalised and rotated in place and k, v as projected (their
 * normalised / rotated / binary16 form is what the cache holds), ATTENTION [rows][n_q*128],
 * BLOCK_OUT [rows][hidden] the down projection, GATE_UP [rows][2*intermediate], ACT [rows][intermediate]
 * = silu(gate)*up, LOGITS [vocab] of the last token. */
enum {
    A81W41_QWEN3_BUF_RESIDUAL = 0, A81W41_QWEN3_BUF_NORMED = 1, A81W41_QWEN3_BUF_QKV = 2,
    A81W41_QWEN3_BUF_ATTENTION = 3, A81W41_QWEN3_BUF_BLOCK_OUT = 4, A81W41_QWEN3_BUF_GATE_UP = 5,
    A81W41_QWEN3_BUF_ACT = 6, A81W41_QWEN3_BUF_LOGITS = 7
};
int a81w41_qwen3_read_buffer(a81w41_qwen3 *model, int which, float *host_out, size_t count);
/* Forget the cached context (position 0). */
int a81w41_qwen3_reset(a81w41_qwen3 *model);
/* Qwen3ForCausalLM::forward: n_tokens new token ids (host) on top of the cached context;
 * logits of the last token ([vocab] fp32) are copied to logits_host if it is not NULL.
 * Synchronises. */
int a81w41_qwen3_forward(a81w41_qwen3 *model, const int *token_ids, int n_tokens, float *logits_host);
/* Prefill the prompt, then n_new greedy tokens (the first from the prompt's logits, the others
 * from n_new - 1 decode steps replayed from one captured HIP graph).  out_tokens: n_new ids,
 * host.  prefill_ms / decode_ms (may be NULL): device time of the prompt pass and of all
 * decode steps. */
int a81w41_qwen3_generate_greedy(a81w41_qwen3 *model, const int *prompt, int n_prompt, int n_new,
                                 int *out_tokens, double *prefill_ms, double *decode_ms);

/* Parity hook: the attention step of the forward pass on its own.  q_dev: [M][q_row_stride] fp32,
 * head h of token m at q_dev[m*q_row_stride + 128 h] (already normalised and rotated);
 * k_cache_dev / v_cache_dev: fp16 [n_kv][max_seq][128] holding positions 0 .. pos+M-1, where pos
 * is read from pos_dev[0]; token m attends keys 0 .. pos+m.  out_dev: [M][out_row_stride] fp32.
 * variant 0: what the forward pass would pick for this M; 1: the vector kernel; 2: the
 * matrix-core kernel (needs M > 8 and n_q / n_kv in {1, 2, 4, 8}); 3, 4, 5, 6: the same with
 * 1, 2, 4, 8 query heads of a KV group per workgroup (a divisor of n_q / n_kv) instead of the
 * number the kernel picks from the count of query tiles. */
int a81w41_qwen3_attention(const float *q_dev, int q_row_stride, const void *k_cache_dev,
                           const void *v_cache_dev, const int *pos_dev, float *out_dev,
                           int out_row_stride, int M, int n_q, int n_kv, int max_seq, float scale,
                           int variant, void *stream);

/* Parity hook: the one-token step of the forward pass on its own -- per-head RMSNorm of the token's
 * query and key (QwenAttention.cc:78-122), rotate-half RoPE at position pos (ops/RotaryPosEmb.cc:6-78),
 * append of the fp16-rounded key and value at row pos of the caches, attention over rows 0 .. pos
 * (QwenAttention.cc:150-195).  qkv_dev: the token's fused row [(n_q + 2 n_kv) * 128] fp32; q_w / k_w: the
 * two norm weights [128]; cos_dev / sin_dev: [max_seq][128] fp32; pos is read from pos_dev[0];
 * out_dev: [n_q * 128] fp32.  splits = 1: one workgroup per head; 2 .. 16: every head's context cut
 * into that many shares, merged by the share that finishes last (the entry point allocates and frees
 * the shares' scratch itself, so it is not for hot loops). */
int a81w41_qwen3_attention_one_token(const float *qkv_dev, int n_q, int n_kv, const float *q_w_dev,
                                     const float *k_w_dev, const float *cos_dev, const float *sin_dev,
                                     const int *pos_dev, void *k_cache_dev, void *v_cache_dev,
                                     float *out_dev, int max_seq, float eps, float scale, int splits,
                                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* A81W41_H */
