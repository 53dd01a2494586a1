// Activation quantiser: fp32 -> Q8_1-style blocks (int8 x 32, scale, scaled sum),
// two 32-blocks per 64-wide super-block, fp16 or fp32 parameters
// (quantize_row_q8_1_repack_fp16 / _fp32, quantized_gemx_kernels.cc:693-911).
//
// Mapping: 8 lanes own one 32-block (a float4 each, so a wave reads 1 KiB
// contiguous); the max and the integer sum are reduced over those 8 lanes with
// DPP row operations.  HBM traffic is 4 B in + ~1.2 B out per element.
// quantize_row_q8_0_repack (:584-682) is the same arithmetic without the sums.
#include "a81w41_kernels.h"
#include "quantize_common.h"

namespace a81w41 {
namespace {

// yt (fp32 parameters only, may be null): a second copy of the blocks with the rows of a super-block next to each
// other, block (row, sb) at (32 sb + row) * 80 -- what the 9..32-row contraction kernel stages per super-block in
// one contiguous piece.  nb_k = super-blocks per row; at most 32 rows.
template <bool FP32, bool ALIGNED>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const float* __restrict__ x,
                                                            uint8_t* __restrict__ y, int64_t nb64,
                                                            bool write_sums, uint8_t* __restrict__ yt, int nb_k) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one float4 each
    const int64_t sb = t >> 4;
    const int h = (int)(t >> 3) & 1;  // low / high 32-block
    const int j = (int)t & 7;         // which float4 of the block
    const bool valid = sb < nb64;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (valid) {
        if (ALIGNED) {
            v = reinterpret_cast<const float4*>(x)[t];
        } else {
            const float* p = x + 4 * t;
            v = make_float4(p[0], p[1], p[2], p[3]);
        }
    }
    const Quant4 qz = quantize_float4_of_block32(v);
    if (!valid) return;
    constexpr int BS = FP32 ? kABlock32 : kABlock16;
    constexpr int QOFF = FP32 ? 16 : 8;
    uint8_t* blk = y + sb * BS;
    *reinterpret_cast<uint32_t*>(blk + QOFF + 32 * h + 4 * j) = qz.packed;
    if (FP32 && yt != nullptr) {
        const int64_t row = sb / nb_k, sbr = sb - row * nb_k;
        uint8_t* tb = yt + (sbr * 32 + row) * BS;
        *reinterpret_cast<uint32_t*>(tb + QOFF + 32 * h + 4 * j) = qz.packed;
        if (j == 0) {
            float* p = reinterpret_cast<float*>(tb);
            p[h] = qz.d;
            p[2 + h] = qz.ssum;
        }
    }
    if (j == 0) {
        if (FP32) {
            float* p = reinterpret_cast<float*>(blk);
            p[h] = qz.d;
            if (write_sums) p[2 + h] = qz.ssum;
        } else {
            uint16_t* p = reinterpret_cast<uint16_t*>(blk);
            p[h] = f32_to_f16_bits(qz.d);
            if (write_sums) p[2 + h] = f32_to_f16_bits(qz.ssum);
        }
    }
}

}  // namespace

hipError_t launch_quantize(const float* x, void* y, int64_t nb64, bool fp32, hipStream_t s, bool write_sums, void* y_by_superblock,
                           int nb_k) {
    if (nb64 == 0) return hipSuccess;
    if (y_by_superblock != nullptr && (!fp32 || !write_sums || nb_k < 1 || nb64 % nb_k || nb64 / nb_k > 32)) return hipErrorInvalidValue;
    uint8_t* yt = static_cast<uint8_t*>(y_by_superblock);
    const int64_t threads = nb64 * 16;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    uint8_t* yb = static_cast<uint8_t*>(y);
#define LAUNCH(F, A) hipLaunchKernelGGL((quantize_q8_1_kernel<F, A>), dim3(grid), dim3(256), 0, s, x, yb, nb64, write_sums, yt, nb_k)
    if (fp32) {
        if (aligned) LAUNCH(true, true); else LAUNCH(true, false);
    } else {
        if (aligned) LAUNCH(false, true); else LAUNCH(false, false);
    }
#undef LAUNCH
    return hipGetLastError();
}

}  // namespace a81w41
