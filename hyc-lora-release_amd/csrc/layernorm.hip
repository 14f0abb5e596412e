// LayerNorm forward / backward (input gradient) for gfx950.
//
//   forward :  mean = sum(x)/N;  var = sum((x - mean)^2)/N  (second pass over the registers, like the
//              reference's second loop);  rstd = 1/sqrt(var + eps);  y = (x - mean)*rstd*w + b
//              (operators/layernorm_kernels.py:27-56, all in fp32, one rounding on the store)
//   backward:  x^ = (x - mean)*rstd;  wdy = w*dy;  c1 = mean(x^ * wdy);  c2 = mean(wdy);
//              dx = (wdy - (x^*c1 + c2)) * rstd                                    (:92-104)
// The reference's backward also accumulates dw / db partials behind a spin lock and then throws
// them away (layernorm_backward returns (dx, None, None), :150-198); they are not computed here.
// One wave owns one row, the row held in registers (N <= 8192): one read, one write.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kLnThreads = 256;
constexpr int kLnWaves = kLnThreads / kWave;

template <bool W32>
__device__ __forceinline__ void ln_load8(const void* p, int col, float (&f)[8]) {
    if constexpr (W32) {
        const f32x4 a = *reinterpret_cast<const f32x4*>((const float*)p + col);
        const f32x4 b = *reinterpret_cast<const f32x4*>((const float*)p + col + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
        f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    } else {
        unpack8(ld16((const uint16_t*)p + col), f);
    }
}

template <int CH, bool W32>
__global__ __launch_bounds__(kLnThreads) void layernorm_fwd_kernel(const uint16_t* __restrict__ x, const void* __restrict__ w,
                                                                   const void* __restrict__ b, uint16_t* __restrict__ y,
                                                                   float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                                   int64_t rows, int N, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kLnWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint16_t* xr = x + row * N;
    u32x4 xv[CH];
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        xv[c] = u32x4{0, 0, 0, 0};
        if (col < N) xv[c] = ld16_nt(xr + col);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float f[8];
        unpack8(xv[c], f);
#pragma unroll
        for (int j = 0; j < 8; ++j) s += f[j];
    }
    const float mean = wave_sum(s) / (float)N;
    float v = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < N) {
            float f[8];
            unpack8(xv[c], f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float d = f[j] - mean;
                v = fmaf(d, d, v);
            }
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(v) / (float)N + eps);
    if (lane == 0) {
        mean_out[row] = mean;
        rstd_out[row] = rstd;
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < N) {
            float f[8], wf[8], bf[8], o[8];
            unpack8(xv[c], f);
            ln_load8<W32>(w, col, wf);
            ln_load8<W32>(b, col, bf);
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = ((f[j] - mean) * rstd) * wf[j] + bf[j];
            st16_nt(y + row * N + col, pack8(o));
        }
    }
}

template <int CH, bool W32>
__global__ __launch_bounds__(kLnThreads) void layernorm_bwd_kernel(const uint16_t* __restrict__ dy, const uint16_t* __restrict__ x,
                                                                   const void* __restrict__ w, const float* __restrict__ mean_in,
                                                                   const float* __restrict__ rstd_in, uint16_t* __restrict__ dx,
                                                                   int64_t rows, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kLnWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float mean = mean_in[row], rstd = rstd_in[row];
    const float inv_n = 1.0f / (float)N;
    u32x4 xv[CH], gv[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        xv[c] = u32x4{0, 0, 0, 0};
        gv[c] = u32x4{0, 0, 0, 0};
        if (col < N) {
            xv[c] = ld16_nt(x + row * N + col);
            gv[c] = ld16_nt(dy + row * N + col);
        }
    }
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < N) {
            float xf[8], gf[8], wf[8];
            unpack8(xv[c], xf);
            unpack8(gv[c], gf);
            ln_load8<W32>(w, col, wf);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = (xf[j] - mean) * rstd, wdy = wf[j] * gf[j];
                s1 = fmaf(xh, wdy, s1);
                s2 += wdy;
            }
        }
    }
    const float c1 = wave_sum(s1) * inv_n, c2 = wave_sum(s2) * inv_n;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < N) {
            float xf[8], gf[8], wf[8], o[8];
            unpack8(xv[c], xf);
            unpack8(gv[c], gf);
            ln_load8<W32>(w, col, wf);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = (xf[j] - mean) * rstd, wdy = wf[j] * gf[j];
                o[j] = (wdy - (xh * c1 + c2)) * rstd;
            }
            st16_nt(dx + row * N + col, pack8(o));
        }
    }
}

template <bool W32>
static int ln_launch_fwd(const uint16_t* x, const void* w, const void* b, uint16_t* y, float* mean, float* rstd,
                         int64_t rows, int N, float eps, hipStream_t st) {
    const dim3 grid((unsigned)cdiv(rows, (int64_t)kLnWaves)), block(kLnThreads);
#define HYC_LNF(CH) hipLaunchKernelGGL((layernorm_fwd_kernel<CH, W32>), grid, block, 0, st, x, w, b, y, mean, rstd, rows, N, eps)
    if (N <= 512) HYC_LNF(1);
    else if (N <= 1024) HYC_LNF(2);
    else if (N <= 2048) HYC_LNF(4);
    else if (N <= 4096) HYC_LNF(8);
    else HYC_LNF(16);
#undef HYC_LNF
    return check_launch();
}

template <bool W32>
static int ln_launch_bwd(const uint16_t* dy, const uint16_t* x, const void* w, const float* mean, const float* rstd,
                         uint16_t* dx, int64_t rows, int N, hipStream_t st) {
    const dim3 grid((unsigned)cdiv(rows, (int64_t)kLnWaves)), block(kLnThreads);
#define HYC_LNB(CH) hipLaunchKernelGGL((layernorm_bwd_kernel<CH, W32>), grid, block, 0, st, dy, x, w, mean, rstd, dx, rows, N)
    if (N <= 512) HYC_LNB(1);
    else if (N <= 1024) HYC_LNB(2);
    else if (N <= 2048) HYC_LNB(4);
    else if (N <= 4096) HYC_LNB(8);
    else HYC_LNB(16);
#undef HYC_LNB
    return check_launch();
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_layernorm_fwd(const void* x, const void* weight, const void* bias, int params_are_fp32, void* y,
                                 float* mean, float* rstd, int64_t rows, int64_t N, float eps, void* stream) {
    if (rows < 0 || N < 0 || N % 8 != 0 || N > 8192) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!x || !weight || !bias || !y || !mean || !rstd) return HYC_ERR_NULL;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(bias) || !aligned16(y)) return HYC_ERR_ALIGN;
    if (cdiv(rows, (int64_t)kLnWaves) > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    return params_are_fp32
               ? ln_launch_fwd<true>((const uint16_t*)x, weight, bias, (uint16_t*)y, mean, rstd, rows, (int)N, eps, st)
               : ln_launch_fwd<false>((const uint16_t*)x, weight, bias, (uint16_t*)y, mean, rstd, rows, (int)N, eps, st);
}

extern "C" int hyc_layernorm_bwd(const void* dy, const void* x, const void* weight, int params_are_fp32,
                                 const float* mean, const float* rstd, void* dx, int64_t rows, int64_t N, void* stream) {
    if (rows < 0 || N < 0 || N % 8 != 0 || N > 8192) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!dy || !x || !weight || !mean || !rstd || !dx) return HYC_ERR_NULL;
    if (!aligned16(dy) || !aligned16(x) || !aligned16(weight) || !aligned16(dx)) return HYC_ERR_ALIGN;
    if (cdiv(rows, (int64_t)kLnWaves) > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    return params_are_fp32
               ? ln_launch_bwd<true>((const uint16_t*)dy, (const uint16_t*)x, weight, mean, rstd, (uint16_t*)dx, rows, (int)N, st)
               : ln_launch_bwd<false>((const uint16_t*)dy, (const uint16_t*)x, weight, mean, rstd, (uint16_t*)dx, rows, (int)N, st);
}
