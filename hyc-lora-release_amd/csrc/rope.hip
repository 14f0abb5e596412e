// Rotary position embedding, in place, for gfx950.
//
// x[b, s, h, :] is rotated by the angle table row s:  with the head split in two halves (x1, x2),
//     x1' = x1*cos - x2*sin,   x2' = x2*cos + x1*sin        (backward: sin -> -sin),
// reading only the first half of each cos/sin row (operators/rope_kernels.py:54-78).  Arithmetic is
// done in the table's type, as the reference converts x to it: a bf16 table rounds after every
// multiply and add, an fp32 table computes in fp32 and rounds once on the store.
//
// One lane owns one 16-byte chunk (8 dims) of the first half and the matching chunk of the second
// half of one head; chunks of a head, then heads, then positions are consecutive lanes, so a
// [B,S,H,D] tensor is read and written in whole cache lines.  Strides let the same kernel rotate a
// [B,H,S,D] tensor (or a slice of a fused qkv buffer) without a transposed copy.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kRopeThreads = 256;

template <bool TABLE_F32>
__global__ __launch_bounds__(kRopeThreads) void rope_kernel(uint16_t* __restrict__ x, const void* __restrict__ cos_t,
                                                            const void* __restrict__ sin_t, int64_t items, int S, int H,
                                                            int chunks, int64_t stride_b, int64_t stride_s,
                                                            int64_t stride_h, int64_t stride_cos, int64_t stride_sin,
                                                            float sin_sign) {
    const int64_t it = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x;
    if (it >= items) return;
    const int c = (int)(it % chunks);
    int64_t r = it / chunks;
    const int h = (int)(r % H);
    r /= H;
    const int s = (int)(r % S);
    const int64_t b = r / S;
    uint16_t* p1 = x + b * stride_b + s * stride_s + h * stride_h + c * 8;
    uint16_t* p2 = p1 + chunks * 8;
    const u32x4 v1 = ld16_nt(p1), v2 = ld16_nt(p2);
    float x1[8], x2[8], cf[8], sf[8], o1[8], o2[8];
    unpack8(v1, x1);
    unpack8(v2, x2);
    if (TABLE_F32) {
        const float* cp = (const float*)cos_t + s * stride_cos + c * 8;
        const float* sp = (const float*)sin_t + s * stride_sin + c * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            cf[j] = cp[j];
            sf[j] = sp[j] * sin_sign;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            o1[j] = x1[j] * cf[j] - x2[j] * sf[j];
            o2[j] = x2[j] * cf[j] + x1[j] * sf[j];
        }
    } else {
        unpack8(ld16((const uint16_t*)cos_t + s * stride_cos + c * 8), cf);
        unpack8(ld16((const uint16_t*)sin_t + s * stride_sin + c * 8), sf);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float sj = sf[j] * sin_sign;
            o1[j] = rbf(x1[j] * cf[j]) - rbf(x2[j] * sj);
            o2[j] = rbf(x2[j] * cf[j]) + rbf(x1[j] * sj);
        }
    }
    st16_nt(p1, pack8(o1));
    st16_nt(p2, pack8(o2));
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_rope(void* x, const void* cos_t, const void* sin_t, int table_is_fp32, int64_t B, int64_t S,
                        int64_t H, int64_t head_dim, int64_t stride_b, int64_t stride_s, int64_t stride_h,
                        int64_t stride_cos, int64_t stride_sin, int backward, void* stream) {
    if (B < 0 || S < 0 || H < 0 || head_dim <= 0 || head_dim % 16 != 0) return HYC_ERR_SHAPE;
    if (B == 0 || S == 0 || H == 0) return HYC_OK;
    if (!x || !cos_t || !sin_t) return HYC_ERR_NULL;
    if (S > INT32_MAX || H > INT32_MAX || head_dim > 65536) return HYC_ERR_SHAPE;
    const int talign = table_is_fp32 ? 4 : 8;      // table rows must keep 16-byte chunks aligned
    if (!aligned16(x) || !aligned16(cos_t) || !aligned16(sin_t) || stride_b % 8 || stride_s % 8 || stride_h % 8 ||
        stride_cos % talign || stride_sin % talign)
        return HYC_ERR_ALIGN;
    if (stride_cos < head_dim / 2 || stride_sin < head_dim / 2) return HYC_ERR_SHAPE;
    const int chunks = (int)(head_dim / 16);
    const int64_t items = B * S * H * chunks;
    const int64_t blocks = cdiv(items, kRopeThreads);
    if (blocks > INT32_MAX) return HYC_ERR_SHAPE;
    const float sgn = backward ? -1.0f : 1.0f;
    hipStream_t st = (hipStream_t)stream;
    if (table_is_fp32)
        hipLaunchKernelGGL(rope_kernel<true>, dim3((unsigned)blocks), dim3(kRopeThreads), 0, st, (uint16_t*)x, cos_t, sin_t,
                           items, (int)S, (int)H, chunks, stride_b, stride_s, stride_h, stride_cos, stride_sin, sgn);
    else
        hipLaunchKernelGGL(rope_kernel<false>, dim3((unsigned)blocks), dim3(kRopeThreads), 0, st, (uint16_t*)x, cos_t, sin_t,
                           items, (int)S, (int)H, chunks, stride_b, stride_s, stride_h, stride_cos, stride_sin, sgn);
    return check_launch();
}
