// Device-side arithmetic of the Q8_1-style activation quantiser, shared by the
// stand-alone kernel and the fused prologue of the M = 1 contraction.
// Follows quantized_gemx_kernels.cc:711-780 operation by operation.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace a81w41 {

template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(dpp_i<CTRL>(__float_as_int(v)));
}
// quad_perm [1,0,3,2] = 0xB1, quad_perm [2,3,0,1] = 0x4E, row_half_mirror = 0x141
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141;

// After these three steps every lane of an aligned group of 8 holds the group's reduction:
// xor1 and xor2 make each quad uniform, half-mirror then brings in the other quad.
__device__ __forceinline__ float group8_max(float v) {
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    return v;
}
__device__ __forceinline__ int group8_sum(int v) {
    unsigned u = (unsigned)v;  // wrapping adds, like _mm256_add_epi32
    u += (unsigned)dpp_i<kDppXor1>((int)u);
    u += (unsigned)dpp_i<kDppXor2>((int)u);
    u += (unsigned)dpp_i<kDppHalfMirror>((int)u);
    return (int)u;
}

// round-to-nearest-even conversion with the x86 semantics the reference runs
// on: values outside int32 (and NaN) give 0x80000000.  That only happens when a
// block's amax is so small that 127/amax overflows to +inf.
__device__ __forceinline__ int rne_i32(float v) {
    return (fabsf(v) < 2147483648.0f) ? (int)rintf(v) : (int)0x80000000;
}
__device__ __forceinline__ int sat8(int r) { return min(127, max(-128, r)); }

struct Quant4 {
    uint32_t packed;  // four int8 in memory order
    float d;          // amax / 127 (fp32, unrounded)
    float ssum;       // d * float(sum of the block's 32 q), one fp32 multiply
};

// Eight consecutive lanes hold the eight float4 of one 32-block.
__device__ __forceinline__ Quant4 quantize_float4_of_block32(float4 v) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = group8_max(amax);
    const float d = amax / 127.f;                            // IEEE divide, :735
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;   // :737
    const int r0 = rne_i32(v.x * id), r1 = rne_i32(v.y * id), r2 = rne_i32(v.z * id),
              r3 = rne_i32(v.w * id);
    // the reference sums the int32 values before the saturating packs, wrapping
    const int sum = group8_sum((int)((unsigned)r0 + (unsigned)r1 + (unsigned)r2 + (unsigned)r3));
    const int q0 = sat8(r0), q1 = sat8(r1), q2 = sat8(r2), q3 = sat8(r3);
    Quant4 out;
    out.packed = (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) |
                 ((uint32_t)(q3 & 0xff) << 24);
    out.d = d;
    float ssum = __fmul_rn(d, (float)sum);  // :777
    // Keep the fp32 product a value of its own: otherwise the compiler folds
    // multiply + fp16 conversion into v_fma_mixlo_f16, which rounds once instead
    // of twice and differs from the reference on fp16 ties.
    asm volatile("" : "+v"(ssum));
    out.ssum = ssum;
    return out;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

// One value per lane, 32 consecutive lanes (an aligned half wave, all active) holding one 32-block of
// a row: the fp16-parameter quantiser (quantize_row_q8_1_repack_fp16, quantized_gemx_kernels.cc:693-801)
// written into the row's 72 B blocks.  col = the value's index in the row.  AGENT: the stores are agent-scope
// stores (a consumer on another XCD reads the blocks while this kernel is still running).
template <bool AGENT = false>
__device__ __forceinline__ void store_quantized_value_fp16(uint8_t* __restrict__ blob, int col, float v) {
    float amax = fabsf(v);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float d = amax / 127.f;
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
    const int r = rne_i32(v * id);
    unsigned sum = (unsigned)r;  // wrapping, like the reference's int32 lanes
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) sum += (unsigned)__shfl_xor((int)sum, off, 64);
    uint8_t* blk = blob + (col >> 6) * 72;
    const int h = (col >> 5) & 1, i = col & 31;
    if (AGENT)
        __hip_atomic_store(blk + 8 + 32 * h + i, (uint8_t)sat8(r), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        blk[8 + 32 * h + i] = (uint8_t)sat8(r);
    if (i == 0) {
        float ssum = __fmul_rn(d, (float)(int)sum);
        asm volatile("" : "+v"(ssum));  // keep the fp32 product: two roundings, as in the reference
        uint16_t* par = reinterpret_cast<uint16_t*>(blk);
        if (AGENT) {
            __hip_atomic_store(par + h, f32_to_f16_bits(d), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(par + 2 + h, f32_to_f16_bits(ssum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            par[h] = f32_to_f16_bits(d);
            par[2 + h] = f32_to_f16_bits(ssum);
        }
    }
}

}  // namespace a81w41
