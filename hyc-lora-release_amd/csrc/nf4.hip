// NF4 (4-bit NormalFloat) block-wise weight dequantisation for gfx950, bitsandbytes 0.43 layout.
//
// The reference keeps its frozen weights as bitsandbytes NF4 with double quantisation and turns
// them into dense bf16 with BF.dequantize_nf4 on every use (models/utils/compute_utils.py:19, :29).
// Format (bitsandbytes/functional.py dequantize_4bit, csrc/kernels.cu kDequantizeBlockwise):
//   * two codes per byte, the element with the EVEN index in the high nibble;
//   * value = table[code] * absmax[element / blocksize], an fp32 product rounded to the output type;
//   * nested ("double quant") statistics: absmax[b] = code2[absmax_code[b]] * absmax2[b / blocksize2]
//     + offset, all fp32 (dequantize_blockwise followed by `absmax += offset`; offset is a device scalar).
// One lane turns 4 packed bytes into one 16-byte chunk of 8 bf16 values; the 16-entry table sits
// in LDS.  HBM-bound: 0.5 + 2 bytes per element.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kNf4Threads = 256;

template <bool NESTED>
__global__ __launch_bounds__(kNf4Threads) void nf4_dequant_kernel(const uint8_t* __restrict__ packed,
                                                                  const void* __restrict__ absmax, const float* __restrict__ code2,
                                                                  const float* __restrict__ absmax2, const float* __restrict__ offset_p, int blocksize2,
                                                                  const float* __restrict__ table, uint16_t* __restrict__ out,
                                                                  int64_t n, int blocksize) {
    __shared__ float tbl[16];
    if (threadIdx.x < 16) tbl[threadIdx.x] = table[threadIdx.x];
    __syncthreads();
    const int64_t chunk = (int64_t)blockIdx.x * kNf4Threads + threadIdx.x;
    const int64_t e0 = chunk * 8;
    if (e0 >= n) return;
    const int64_t blk = e0 / blocksize;                    // blocksize % 8 == 0: a chunk never straddles blocks
    float am;
    if constexpr (NESTED) am = code2[((const uint8_t*)absmax)[blk]] * absmax2[blk / blocksize2] + (offset_p ? *offset_p : 0.0f);
    else am = ((const float*)absmax)[blk];
    const uint32_t w = *reinterpret_cast<const uint32_t*>(packed + chunk * 4);
    float f[8];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (w >> (8 * b)) & 0xffu;
        f[2 * b] = tbl[byte >> 4] * am;
        f[2 * b + 1] = tbl[byte & 15u] * am;
    }
    if (e0 + 8 <= n) {
        st16_nt(out + e0, pack8(f));
    } else {
        for (int j = 0; e0 + j < n; ++j) out[e0 + j] = f_to_bf(f[j]);
    }
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_nf4_dequant(const void* packed, const void* absmax, int nested, const float* code2,
                               const float* absmax2, const float* offset, int64_t blocksize2, const float* table, void* out,
                               int64_t n, int64_t blocksize, void* stream) {
    if (n < 0 || blocksize <= 0 || blocksize % 8 != 0 || n % 2 != 0) return HYC_ERR_SHAPE;
    if (nested && blocksize2 <= 0) return HYC_ERR_SHAPE;
    if (n == 0) return HYC_OK;
    if (!packed || !absmax || !table || !out || (nested && (!code2 || !absmax2))) return HYC_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(packed) & 3u) || !aligned16(out)) return HYC_ERR_ALIGN;
    const int64_t blocks = cdiv(cdiv(n, (int64_t)8), (int64_t)kNf4Threads);
    if (blocks > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (nested)
        hipLaunchKernelGGL(nf4_dequant_kernel<true>, dim3((unsigned)blocks), dim3(kNf4Threads), 0, st, (const uint8_t*)packed,
                           absmax, code2, absmax2, offset, (int)blocksize2, table, (uint16_t*)out, n, (int)blocksize);
    else
        hipLaunchKernelGGL(nf4_dequant_kernel<false>, dim3((unsigned)blocks), dim3(kNf4Threads), 0, st, (const uint8_t*)packed,
                           absmax, code2, absmax2, offset, 1, table, (uint16_t*)out, n, (int)blocksize);
    return check_launch();
}
