// M x N contraction of the A80W40 variant (gemm_repack_A80W40,
// quantized_gemx_kernels.cc:195-347): fp16-parameter blocks on both sides, codes read
// as code - 8, no min term:
//   C[m][n] = sum over 32-blocks of  float(sum((code - 8) q)) * (d_a d_w).
// Since sum((code - 8) q) = sum(code q) - 8 sum(q), this is the A81W41 contraction with
//   min = -8 d_w        (exact: a power-of-two multiple)
//   scaled sum = d_a * sum(q)   (exact in fp32: an 11-bit significand times |sum| <= 4064)
// and d_a d_w itself is exact in fp32 (two 11-bit significands), so every term that enters
// the fp32 accumulation is the same real number the reference adds; only the grouping of
// the additions differs.  Two element-wise kernels rewrite the operands into the caller's
// workspace as 80 B / 384 B blocks and the matrix-core kernel of the A81W41 path does the
// rest.  The rewrite reads 0.625 B and writes 0.75 B per weight on every call, about a
// fifth of the contraction's own time at M = 322; a caller that keeps weights in this
// variant for many calls should keep the 384 B form instead.
#include "a81w41_kernels.h"
#include "quantize_common.h"

namespace a81w41 {
namespace {

// One thread per 4-byte word of the 80 B output block: words 0,1 = d_low, d_high;
// 2,3 = d * sum(q) of the low / high 32-block; 4..19 = the 64 int8.
__global__ __launch_bounds__(256) void a80_act_to_fp32_kernel(const uint32_t* __restrict__ in,
                                                              uint32_t* __restrict__ out, int64_t n_words) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_words) return;
    const int64_t b = t / 20;
    const int w = (int)(t - b * 20);
    const uint32_t* src = in + b * 18;  // 72 B block: scales | (unset sums) | 16 words of q
    if (w >= 4) {
        out[t] = src[2 + (w - 4)];
        return;
    }
    const int h = w & 1;
    const float d = f16_bits_to_f32((src[0] >> (16 * h)) & 0xffff);
    if (w < 2) {
        out[t] = __float_as_uint(d);
        return;
    }
    int sum = 0;
#pragma unroll
    for (int p = 0; p < 8; p++) sum = __builtin_amdgcn_sdot4(0x01010101, (int)src[2 + 8 * h + p], sum, false);
    out[t] = __float_as_uint(__fmul_rn(d, (float)sum));
}

// One thread per 16 bytes of the 384 B output block: chunks 0..3 = s_low[8], s_high[8] widened to
// fp32; 4..7 = -8 * the same; 8..23 = q_coupled.
__global__ __launch_bounds__(256) void w80_to_w81_fp32_kernel(const uint8_t* __restrict__ in,
                                                              uint4* __restrict__ out, int64_t n_chunks) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_chunks) return;
    const int64_t b = t / 24;
    const int c = (int)(t - b * 24);
    const uint8_t* src = in + b * kWBlock16;  // 16 fp16 scales | (unset mins) | 256 B of codes
    if (c >= 8) {
        out[t] = *reinterpret_cast<const uint4*>(src + 64 + 16 * (c - 8));
        return;
    }
    const uint2 h4 = *reinterpret_cast<const uint2*>(src + 8 * (c & 3));  // four consecutive fp16 scales
    const float f = c < 4 ? 1.0f : -8.0f;                                 // exact either way
    uint4 o;
    o.x = __float_as_uint(__fmul_rn(f, f16_bits_to_f32(h4.x & 0xffff)));
    o.y = __float_as_uint(__fmul_rn(f, f16_bits_to_f32(h4.x >> 16)));
    o.z = __float_as_uint(__fmul_rn(f, f16_bits_to_f32(h4.y & 0xffff)));
    o.w = __float_as_uint(__fmul_rn(f, f16_bits_to_f32(h4.y >> 16)));
    out[t] = o;
}

size_t round_up_256(size_t b) { return (b + 255) & ~(size_t)255; }

}  // namespace

size_t gemm_a80w40_workspace_bytes(int M, int N, int K) {
    const size_t nb_k = (size_t)K / 64;
    return round_up_256((size_t)M * nb_k * kABlock32) + round_up_256((size_t)N / 8 * nb_k * kWBlock32);
}

hipError_t launch_gemm_a80w40(const void* A, const void* B, float* C, int M, int N, int K, void* workspace,
                              const GemmScratch& ws, hipStream_t s) {
    const size_t nb_k = (size_t)K / 64;
    uint8_t* a32 = static_cast<uint8_t*>(workspace);
    uint8_t* b32 = a32 + round_up_256((size_t)M * nb_k * kABlock32);
    const int64_t a_words = (int64_t)M * nb_k * (kABlock32 / 4);
    const int64_t b_chunks = (int64_t)(N / 8) * nb_k * (kWBlock32 / 16);
    hipLaunchKernelGGL(a80_act_to_fp32_kernel, dim3((unsigned)((a_words + 255) / 256)), dim3(256), 0, s,
                       static_cast<const uint32_t*>(A), reinterpret_cast<uint32_t*>(a32), a_words);
    hipLaunchKernelGGL(w80_to_w81_fp32_kernel, dim3((unsigned)((b_chunks + 255) / 256)), dim3(256), 0, s,
                       static_cast<const uint8_t*>(B), reinterpret_cast<uint4*>(b32), b_chunks);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    return launch_gemm_fp32(a32, b32, C, M, N, K, ws, s);
}

}  // namespace a81w41
