// RMSNorm forward fused with the two compressions that follow it in a decoder layer, for gfx950.
//
// The layer normalises x, keeps a channel-base compressed copy of x for the norm's backward and a
// quantised copy of the normalised output for the backward of the projections that consume it
// (models/llama/fused_llama_layer_intra_inter_full_fuse.py:97-126: rmsnorm_forward,
// compression_pack_channel_base(x), compression_pack_quant_base(x_norm)).  Done separately that is
// three reads of x / x_norm; here the row is read once and everything is produced from registers:
//     y      = bf16(x * rstd * w), rstd = 1/sqrt(mean(x^2) + eps)        (rmsnorm_kernels.py:34-54)
//     q_y    = Q(y; scale_y)                                              packed codes
//     x_out  = x[:, outlier channels];  q_x = Q(x with those channels zeroed; scale_x)
// One wave owns one row, each lane CH 16-byte chunks of it, as in the plain forward kernel; the
// per-column steps are re-read per row (L2 hits, like the norm weight).  The row is parked in LDS
// after the sum of squares (each lane reads back only what it wrote, so no barrier is involved)
// and the second phase walks the chunks in a rolled loop: one copy of the quantiser code and a
// few dozen live registers instead of CH unrolled copies, which is what keeps enough waves
// resident to hide the latency of the per-chunk constant loads.
// Only frozen (calibrated) steps can be used here: during calibration the steps of y depend on y.
#include "hyc_pack.hpp"

namespace hyc {

constexpr int kNcThreads = 256;
constexpr int kNcWaves = kNcThreads / kWave;

struct NormCompressArgs {
    const uint16_t* x; const void* w; uint16_t* y; float* rstd;
    const uint16_t* scale_y; uint8_t* q_y;              // q_y == nullptr: no quantised copy of y
    const uint16_t* scale_x; uint8_t* q_x;              // q_x == nullptr: no compressed copy of x
    const uint16_t* otable; uint16_t* xo;               // otable[c] = 1 + position of channel c in the outlier list, 0 = none
    int64_t rows;
    int N, k;
    float eps;
};

template <int QBIT>
__device__ __forceinline__ void quantise_chunk(const float (&f)[8], const uint16_t* scale, int col, int chunk, bool active,
                                               uint8_t* qrow) {
    QuantCols<QBIT> qc;
    qc.load(scale, col, active);
    const float zero8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t lo, hi;
    if (__ballot(!qc.fast) != 0ull) codes_to_words<QBIT, false, false>(f, qc, zero8, lo, hi);
    else codes_to_words<QBIT, false, true>(f, qc, zero8, lo, hi);
    store_packed<QBIT, true>(qrow, chunk, active, lo, hi);
}

template <int CH, int QBIT, bool W32>
__global__ __launch_bounds__(kNcThreads) __attribute__((amdgpu_waves_per_eu(4)))
void rmsnorm_fwd_compress_kernel(const NormCompressArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kNcWaves + (threadIdx.x >> 6);
    if (row >= a.rows) return;                          // whole waves leave together
    const int N = a.N;
    const uint16_t* xr = a.x + row * N;
    const int row_bytes = N * QBIT / 8;
    extern __shared__ u32x4 nc_rows[];                  // [waves][CH * 64] chunks
    u32x4* park = nc_rows + (threadIdx.x >> 6) * (CH * kWave);
    float ss = 0.0f;
    {
        u32x4 xv[CH];
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
            for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
            park[c * kWave + lane] = xv[c];
        }
    }
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)N + a.eps);
    if (lane == 0) a.rstd[row] = rstd;
#pragma unroll 1
    for (int c = 0; c * kWave * 8 < N; ++c) {           // uniform bound: chunks some lane of the wave has
        const int chunk = c * kWave + lane;
        const int col = chunk * 8;
        const bool active = col < N;
        const u32x4 xc = park[chunk];
        float f[8];
        unpack8(xc, f);
        {
            float wf[8] = {0, 0, 0, 0, 0, 0, 0, 0}, o[8];
            if (active) {
                if constexpr (W32) {
                    const f32x4 w0 = *reinterpret_cast<const f32x4*>((const float*)a.w + col);
                    const f32x4 w1 = *reinterpret_cast<const f32x4*>((const float*)a.w + col + 4);
                    wf[0] = w0.x; wf[1] = w0.y; wf[2] = w0.z; wf[3] = w0.w;
                    wf[4] = w1.x; wf[5] = w1.y; wf[6] = w1.z; wf[7] = w1.w;
                } else {
                    unpack8(ld16((const uint16_t*)a.w + col), wf);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (f[j] * rstd) * wf[j];
            const u32x4 yv = pack8(o);
            if (active) st16_nt(a.y + row * N + col, yv);
            if (a.q_y) {
                float fy[8];
                unpack8(yv, fy);
                quantise_chunk<QBIT>(fy, a.scale_y, col, chunk, active, a.q_y + row * row_bytes);
            }
        }
        if (a.q_x) {
            if (a.k > 0) {
                u32x4 tv = {0, 0, 0, 0};
                if (active) tv = ld16(a.otable + col);
                if ((tv.x | tv.y | tv.z | tv.w) != 0u) {
                    const uint32_t td[4] = {tv.x, tv.y, tv.z, tv.w};
                    const uint32_t xd[4] = {xc.x, xc.y, xc.z, xc.w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t p = (td[j >> 1] >> (16 * (j & 1))) & 0xffffu;
                        if (p) {
                            a.xo[row * a.k + (p - 1)] = (uint16_t)(xd[j >> 1] >> (16 * (j & 1)));
                            f[j] = 0.0f;
                        }
                    }
                }
            }
            quantise_chunk<QBIT>(f, a.scale_x, col, chunk, active, a.q_x + row * row_bytes);
        }
    }
}

// otable[c] = 1 + i for c = oidx[i], everything else 0 (table cleared by the first kernel)
__global__ void otable_fill_kernel(uint16_t* __restrict__ table, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) table[i] = 0;
}
__global__ void otable_mark_kernel(const int64_t* __restrict__ oidx, int k, int n, uint16_t* __restrict__ table) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < k) {
        const int64_t c = oidx[i];
        if (c >= 0 && c < n) table[c] = (uint16_t)(i + 1);
    }
}

template <int QBIT, bool W32>
static int launch_nc(const NormCompressArgs& a, hipStream_t st) {
    const dim3 grid((unsigned)cdiv(a.rows, (int64_t)kNcWaves)), block(kNcThreads);
#define HYC_NC(CH) \
    hipLaunchKernelGGL((rmsnorm_fwd_compress_kernel<CH, QBIT, W32>), grid, block, kNcWaves * CH * kWave * 16, st, a)
    if (a.N <= 512) HYC_NC(1);
    else if (a.N <= 1024) HYC_NC(2);
    else if (a.N <= 2048) HYC_NC(4);
    else if (a.N <= 4096) HYC_NC(8);
    else HYC_NC(16);
#undef HYC_NC
    return check_launch();
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_outlier_table(const int64_t* outlier_idx, int64_t k, int64_t N, uint16_t* table, void* stream) {
    if (k < 0 || N < 0 || k > 65535 || N > (1 << 28)) return HYC_ERR_SHAPE;
    if (N == 0) return HYC_OK;
    if (!table || (k > 0 && !outlier_idx)) return HYC_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(otable_fill_kernel, dim3((unsigned)cdiv(N, (int64_t)256)), dim3(256), 0, st, table, (int)N);
    if (k > 0)
        hipLaunchKernelGGL(otable_mark_kernel, dim3((unsigned)cdiv(k, (int64_t)256)), dim3(256), 0, st, outlier_idx, (int)k,
                           (int)N, table);
    return check_launch();
}

extern "C" int hyc_rmsnorm_fwd_compress(const void* x, const void* weight, int weight_is_fp32, void* y, float* rstd,
                                        int64_t rows, int64_t N, float eps, int q_bit, const void* scale_y, void* q_y,
                                        const void* scale_x, void* q_x, const uint16_t* outlier_table, int64_t k,
                                        void* x_outlier, void* stream) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (rows < 0 || N < 0 || N % 32 != 0 || N > 8192 || k < 0 || k > 65535) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!x || !weight || !y || !rstd) return HYC_ERR_NULL;
    if ((q_y && !scale_y) || (q_x && !scale_x) || (q_x && k > 0 && (!outlier_table || !x_outlier))) return HYC_ERR_NULL;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || (scale_y && !aligned16(scale_y)) ||
        (scale_x && !aligned16(scale_x)) || (outlier_table && !aligned16(outlier_table)))
        return HYC_ERR_ALIGN;
    if ((q_y && (reinterpret_cast<uintptr_t>(q_y) & 7u)) || (q_x && (reinterpret_cast<uintptr_t>(q_x) & 7u)))
        return HYC_ERR_ALIGN;
    if (cdiv(rows, (int64_t)kNcWaves) > INT32_MAX) return HYC_ERR_SHAPE;
    NormCompressArgs a;
    a.x = (const uint16_t*)x; a.w = weight; a.y = (uint16_t*)y; a.rstd = rstd;
    a.scale_y = (const uint16_t*)scale_y; a.q_y = (uint8_t*)q_y;
    a.scale_x = (const uint16_t*)scale_x; a.q_x = (uint8_t*)q_x;
    a.otable = outlier_table; a.xo = (uint16_t*)x_outlier;
    a.rows = rows; a.N = (int)N; a.k = q_x ? (int)k : 0; a.eps = eps;
    hipStream_t st = (hipStream_t)stream;
#define HYC_NC_Q(QB) (weight_is_fp32 ? launch_nc<QB, true>(a, st) : launch_nc<QB, false>(a, st))
    if (q_bit == 8) return HYC_NC_Q(8);
    if (q_bit == 4) return HYC_NC_Q(4);
    return HYC_NC_Q(2);
#undef HYC_NC_Q
}
