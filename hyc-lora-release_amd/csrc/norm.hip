// RMSNorm forward / backward for gfx950.
//
// One wave owns one row: each lane keeps CH 16-byte chunks of the row in registers, so the
// row is read once, reduced with a wave-level sum and written once.  Rows longer than
// 64*8*16 = 8192 channels fall back to a two-pass loop over the row (second pass hits L2).
//
// Backward also produces the weight gradient dw = sum_rows dy * x^ without the reference's
// spin-lock accumulation (operators/rmsnorm_kernels.py:103-113): each wave accumulates its
// rows in fp32 registers, the workgroup combines its waves in LDS and writes one partial
// row; a second kernel adds the partial rows in a fixed order.  Deterministic, no atomics.
#include <mutex>

#include "hyc_common.hpp"

namespace hyc {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / kWave;
constexpr int kNormMaxBlocks = 512;
constexpr int kNormMaxRegisterRow = 8192;      // longest row the backward kernel holds in registers

// Scratch of hyc_rmsnorm_bwd_static: the fp32 partial rows of the weight gradient, for the largest
// launch the backward kernel makes (kNormMaxBlocks workgroups x rows of kNormMaxRegisterRow
// channels = 16 MiB).  Lives in every GPU's memory from the moment the library's code object is
// loaded there until the process ends.  In host code the array's NAME is only a handle: the
// device address is obtained once per device with hipGetSymbolAddress (static_scratch() below)
// and only that pointer is ever handed to a kernel.
constexpr int64_t kStaticScratchBytes = (int64_t)kNormMaxBlocks * kNormMaxRegisterRow * (int64_t)sizeof(float);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

template <bool W32>
__device__ __forceinline__ void load_w8(const void* w, int col, float (&wf)[8]) {
    if constexpr (W32) {
        const f32x4 a = *reinterpret_cast<const f32x4*>((const float*)w + col);
        const f32x4 b = *reinterpret_cast<const f32x4*>((const float*)w + col + 4);
        wf[0] = a.x; wf[1] = a.y; wf[2] = a.z; wf[3] = a.w;
        wf[4] = b.x; wf[5] = b.y; wf[6] = b.z; wf[7] = b.w;
    } else {
        unpack8(ld16((const uint16_t*)w + col), wf);
    }
}

// y = bf16(x * rstd * w), rstd = 1/sqrt(mean(x^2) + eps)   (operators/rmsnorm_kernels.py:34-54)
template <int CH, bool W32>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_kernel(const uint16_t* __restrict__ x, const void* __restrict__ w,
                                                                   uint16_t* __restrict__ y, float* __restrict__ rstd_out,
                                                                   int64_t rows, int N, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kNormWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint16_t* xr = x + row * N;
    u32x4 xv[CH];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        xv[c] = u32x4{0, 0, 0, 0};
        if (col < N) xv[c] = ld16_nt(xr + col);
    }
    // Summation order (shared with the fused norm + compress kernels, whose results must be the
    // same bits): the 8 squares of a chunk as one fused-multiply-add chain from zero, a lane's
    // chunks added in column order, then the butterfly over the lanes.
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float f[8];
        unpack8(xv[c], f);
        ss += chunk_sumsq(f);
    }
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)N + eps);
    if (lane == 0) rstd_out[row] = rstd;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < N) {
            float f[8], wf[8], o[8];
            unpack8(xv[c], f);
            load_w8<W32>(w, col, wf);
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (f[j] * rstd) * wf[j];
            st16_nt(y + row * N + col, pack8(o));
        }
    }
}

// Long rows: the row does not fit in registers; read it twice.
template <bool W32>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_long_kernel(const uint16_t* __restrict__ x, const void* __restrict__ w,
                                                                        uint16_t* __restrict__ y, float* __restrict__ rstd_out,
                                                                        int64_t rows, int N, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kNormWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint16_t* xr = x + row * N;
    float ss = 0.0f;
    for (int col = lane * 8; col < N; col += kWave * 8) {
        float f[8];
        unpack8(ld16(xr + col), f);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
    }
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)N + eps);
    if (lane == 0) rstd_out[row] = rstd;
    for (int col = lane * 8; col < N; col += kWave * 8) {
        float f[8], wf[8], o[8];
        unpack8(ld16(xr + col), f);
        load_w8<W32>(w, col, wf);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (f[j] * rstd) * wf[j];
        st16(y + row * N + col, pack8(o));
    }
}

// dx = (w*dy - (x^*c1 + c2)) * rstd,  c1 = mean(x^ * w*dy),  c2 = mean(w*dy),  x^ = x*rstd.
// The c2 term belongs to LayerNorm; the reference keeps it for RMSNorm
// (operators/rmsnorm_kernels.py:92-100) and so does this kernel.
// RES: dx = bf16(bf16(that) + residual) - the gradient arriving over the residual connection,
// which the layers add right after this call (`grad_norm + grad_output`,
// models/llama/fused_llama_layer_intra_inter_full_fuse.py:393, :493): the same two roundings as the
// separate add, without its pass over three tensors.
template <int CH, bool W32, bool DW, bool RES>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_bwd_kernel(const uint16_t* __restrict__ dy, const uint16_t* __restrict__ x,
                                                                   const void* __restrict__ w, const float* __restrict__ rstd_in,
                                                                   const uint16_t* __restrict__ res,
                                                                   uint16_t* __restrict__ dx, float* __restrict__ dw_partial,
                                                                   int64_t rows, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    // The weight is re-read per row (8 KiB at N=4096, cache-resident) rather than held in
    // registers: together with the dw accumulators it would cost an occupancy step.
    float dwacc[DW ? CH : 1][8];
    if constexpr (DW) {
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) dwacc[c][j] = 0.0f;
    }
    const float inv_n = 1.0f / (float)N;
    for (int64_t row = (int64_t)blockIdx.x * kNormWaves + wave; row < rows; row += (int64_t)gridDim.x * kNormWaves) {
        const float rstd = rstd_in[row];
        u32x4 xv[CH], gv[CH], rv[RES ? CH : 1];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            xv[c] = u32x4{0, 0, 0, 0};
            gv[c] = u32x4{0, 0, 0, 0};
            if constexpr (RES) rv[c] = u32x4{0, 0, 0, 0};
            if (col < N) {
                xv[c] = ld16_nt(x + row * N + col);
                gv[c] = ld16_nt(dy + row * N + col);
                if constexpr (RES) rv[c] = ld16_nt(res + row * N + col);
            }
        }
        // Summation order (shared with the form that reads x from its codes, whose results must
        // be the same bits): each chunk's two sums as chains from zero, a lane's chunks added in
        // column order, then the butterfly over the lanes.
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            float xf[8], gf[8], wf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            unpack8(xv[c], xf);
            unpack8(gv[c], gf);
            if (col < N) load_w8<W32>(w, col, wf);
            float p1 = 0.0f, p2 = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = xf[j] * rstd, wdy = wf[j] * gf[j];
                p1 = fmaf(xh, wdy, p1);
                p2 += wdy;
                if constexpr (DW) dwacc[c][j] = fmaf(gf[j], xh, dwacc[c][j]);
            }
            s1 += p1;
            s2 += p2;
        }
        const float c1 = wave_sum(s1) * inv_n, c2 = wave_sum(s2) * inv_n;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            if (col < N) {
                float xf[8], gf[8], wf[8], o[8];
                unpack8(xv[c], xf);
                unpack8(gv[c], gf);
                load_w8<W32>(w, col, wf);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float xh = xf[j] * rstd, wdy = wf[j] * gf[j];
                    o[j] = (wdy - (xh * c1 + c2)) * rstd;
                }
                if constexpr (RES) {
                    float rf[8];
                    unpack8(rv[c], rf);
#pragma unroll
                    for (int j = 0; j < 8; ++j) o[j] = rbf(o[j]) + rf[j];
                }
                st16_nt(dx + row * N + col, pack8(o));
            }
        }
    }
    if constexpr (DW) {
        // combine the workgroup's waves through LDS, one chunk index at a time, wave order fixed
        __shared__ float red[kNormWaves][kWave * 8];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 8; ++j) red[wave][lane * 8 + j] = dwacc[c][j];
            __syncthreads();
            for (int i = threadIdx.x; i < kWave * 8; i += kNormThreads) {
                const int col = c * kWave * 8 + i;
                if (col < N) {
                    float s = red[0][i];
#pragma unroll
                    for (int v = 1; v < kNormWaves; ++v) s += red[v][i];
                    dw_partial[(int64_t)blockIdx.x * N + col] = s;
                }
            }
        }
    }
}

// dw[c] = sum over partial rows, fixed order; output in the weight's dtype.  A workgroup owns 64
// columns; thread (g = tid / 16, c4 = tid % 16) adds rows g, g + 16, g + 32, ... of four columns, four
// loads in flight, and the 16 row groups are then added in order through LDS.  (One thread per column
// walking all partial rows by itself was a chain of several hundred dependent loads on 16 workgroups:
// 70 us for 4 MB.)
template <bool W32>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int nparts, int N,
                                                                void* __restrict__ dw) {
    __shared__ f32x4 red[16][16];
    const int c4 = threadIdx.x & 15, g = threadIdx.x >> 4;
    const int col = (blockIdx.x * 16 + c4) * 4;
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    if (col < N) {
        const float* p0 = partial + col;
        int p = g;
        for (; p + 48 < nparts; p += 64) {
            f32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4*>(p0 + (int64_t)(p + 16 * u) * N);
#pragma unroll
            for (int u = 0; u < 4; ++u) s += v[u];
        }
        for (; p < nparts; p += 16) s += *reinterpret_cast<const f32x4*>(p0 + (int64_t)p * N);
    }
    red[g][c4] = s;
    __syncthreads();
    if (g != 0 || col >= N) return;
    f32x4 t = red[0][c4];
#pragma unroll
    for (int k = 1; k < 16; ++k) t += red[k][c4];
    if constexpr (W32) {
        *reinterpret_cast<f32x4*>((float*)dw + col) = t;
    } else {
        *reinterpret_cast<u32x2*>((uint16_t*)dw + col) = u32x2{pk_bf16(t.x, t.y), pk_bf16(t.z, t.w)};
    }
}

// Workgroups of the backward launch that also leaves dw partials (one partial row each).  Rows of up to
// 4096 channels leave room for two such waves per SIMD, longer ones for one: [4096 x 4096] takes 32 us
// with two rows per wave against 37 with four, [4096 x 8192] 73 us with four against 84 with two.
static int bwd_blocks(int64_t rows, int64_t N) {
    int64_t b = cdiv(rows, kNormWaves * (N <= 4096 ? 2 : 4));
    if (b > kNormMaxBlocks) b = kNormMaxBlocks;
    if (b < 1) b = 1;
    return (int)b;
}

template <bool W32>
static int launch_fwd(const uint16_t* x, const void* w, uint16_t* y, float* rstd, int64_t rows, int N, float eps,
                      hipStream_t st) {
    const dim3 grid((unsigned)cdiv(rows, kNormWaves)), block(kNormThreads);
#define HYC_FWD(CH) hipLaunchKernelGGL((rmsnorm_fwd_kernel<CH, W32>), grid, block, 0, st, x, w, y, rstd, rows, N, eps)
    // a row is held in registers, CH chunks of 8 per lane; the steps between the powers of two keep
    // rows of 3072, 5120, 6144 and 7168 from paying for registers they do not fill
    if (N <= 512) HYC_FWD(1);
    else if (N <= 1024) HYC_FWD(2);
    else if (N <= 2048) HYC_FWD(4);
    else if (N <= 3072) HYC_FWD(6);
    else if (N <= 4096) HYC_FWD(8);
    else if (N <= 5120) HYC_FWD(10);
    else if (N <= 6144) HYC_FWD(12);
    else if (N <= 7168) HYC_FWD(14);
    else if (N <= 8192) HYC_FWD(16);
    else hipLaunchKernelGGL((rmsnorm_fwd_long_kernel<W32>), grid, block, 0, st, x, w, y, rstd, rows, N, eps);
#undef HYC_FWD
    return check_launch();
}

template <bool W32, bool DW, bool RES>
static int launch_bwd_r(const uint16_t* dy, const uint16_t* x, const void* w, const float* rstd, const uint16_t* res,
                        uint16_t* dx, float* partial, int64_t rows, int N, int blocks, hipStream_t st) {
    const dim3 grid((unsigned)blocks), block(kNormThreads);
#define HYC_BWD(CH) hipLaunchKernelGGL((rmsnorm_bwd_kernel<CH, W32, DW, RES>), grid, block, 0, st, dy, x, w, rstd, res, dx, partial, rows, N)
    if (N <= 512) HYC_BWD(1);
    else if (N <= 1024) HYC_BWD(2);
    else if (N <= 2048) HYC_BWD(4);
    else if (N <= 3072) HYC_BWD(6);
    else if (N <= 4096) HYC_BWD(8);
    else if (N <= 5120) HYC_BWD(10);
    else if (N <= 6144) HYC_BWD(12);
    else if (N <= 7168) HYC_BWD(14);
    else HYC_BWD(16);
#undef HYC_BWD
    return check_launch();
}
template <bool W32, bool DW>
static int launch_bwd(const uint16_t* dy, const uint16_t* x, const void* w, const float* rstd, const uint16_t* res,
                      uint16_t* dx, float* partial, int64_t rows, int N, int blocks, hipStream_t st) {
    return res ? launch_bwd_r<W32, DW, true>(dy, x, w, rstd, res, dx, partial, rows, N, blocks, st)
               : launch_bwd_r<W32, DW, false>(dy, x, w, rstd, res, dx, partial, rows, N, blocks, st);
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_rmsnorm_fwd(const void* x, const void* weight, int weight_is_fp32, void* y, float* rstd,
                               int64_t rows, int64_t N, float eps, void* stream) {
    if (rows < 0 || N < 0 || N % 8 != 0 || N > 65536) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!x || !weight || !y || !rstd) return HYC_ERR_NULL;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y)) return HYC_ERR_ALIGN;
    if (cdiv(rows, kNormWaves) > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    return weight_is_fp32 ? launch_fwd<true>((const uint16_t*)x, weight, (uint16_t*)y, rstd, rows, (int)N, eps, st)
                          : launch_fwd<false>((const uint16_t*)x, weight, (uint16_t*)y, rstd, rows, (int)N, eps, st);
}

extern "C" int64_t hyc_rmsnorm_bwd_workspace(int64_t rows, int64_t N) {
    if (rows <= 0 || N <= 0) return 0;
    return (int64_t)bwd_blocks(rows, N) * N * (int64_t)sizeof(float);
}

namespace hyc {
int rmsnorm_bwd_dense_slab(const void* dy, const void* x, const void* weight, int weight_is_fp32, const float* rstd,
                           const void* residual, void* dx, int64_t rows, int64_t N, void* stream);   // norm_compress.hip
}

static int rmsnorm_bwd_any(const void* dy, const void* x, const void* weight, int weight_is_fp32, const float* rstd,
                           const void* residual, void* dx, void* dw, void* workspace, int64_t workspace_bytes,
                           int64_t rows, int64_t N, void* stream) {
    if (rows < 0 || N < 0 || N % 8 != 0 || N > 8192) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!dy || !x || !weight || !rstd || !dx) return HYC_ERR_NULL;
    if (!aligned16(dy) || !aligned16(x) || !aligned16(weight) || !aligned16(dx) || !aligned16(residual)) return HYC_ERR_ALIGN;
    const uint16_t* res = (const uint16_t*)residual;
    hipStream_t st = (hipStream_t)stream;
    const int blocks = bwd_blocks(rows, N);
    int rc;
    if (dw) {
        if (!workspace) return HYC_ERR_NULL;
        if (!aligned16(workspace) || !aligned16(dw)) return HYC_ERR_ALIGN;
        if (workspace_bytes < hyc_rmsnorm_bwd_workspace(rows, N)) return HYC_ERR_WORKSPACE;
        rc = weight_is_fp32
                 ? launch_bwd<true, true>((const uint16_t*)dy, (const uint16_t*)x, weight, rstd, res, (uint16_t*)dx, (float*)workspace, rows, (int)N, blocks, st)
                 : launch_bwd<false, true>((const uint16_t*)dy, (const uint16_t*)x, weight, rstd, res, (uint16_t*)dx, (float*)workspace, rows, (int)N, blocks, st);
        if (rc != HYC_OK) return rc;
        const dim3 grid((unsigned)cdiv(N, 64)), block(256);
        if (weight_is_fp32) hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel<true>, grid, block, 0, st, (const float*)workspace, blocks, (int)N, dw);
        else hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel<false>, grid, block, 0, st, (const float*)workspace, blocks, (int)N, dw);
        return check_launch();
    }
    // Rows longer than 4096 channels leave a row-per-wave kernel one or two waves per SIMD (3.4 - 3.9 TB/s);
    // the column-slab kernel of the fused norm files takes them where the shape fits (same bits).
    if (N > 4096) {
        rc = hyc::rmsnorm_bwd_dense_slab(dy, x, weight, weight_is_fp32, rstd, residual, dx, rows, N, stream);
        if (rc <= 0) return rc;
    }
    // without dw the grid need not be capped, but the same persistent loop is used
    return weight_is_fp32
               ? launch_bwd<true, false>((const uint16_t*)dy, (const uint16_t*)x, weight, rstd, res, (uint16_t*)dx, nullptr, rows, (int)N, (int)(cdiv(rows, kNormWaves) > 65535 * 16 ? 65535 * 16 : cdiv(rows, kNormWaves)), st)
               : launch_bwd<false, false>((const uint16_t*)dy, (const uint16_t*)x, weight, rstd, res, (uint16_t*)dx, nullptr, rows, (int)N, (int)(cdiv(rows, kNormWaves) > 65535 * 16 ? 65535 * 16 : cdiv(rows, kNormWaves)), st);
}

extern "C" int hyc_rmsnorm_bwd(const void* dy, const void* x, const void* weight, int weight_is_fp32,
                               const float* rstd, void* dx, void* dw, void* workspace, int64_t workspace_bytes,
                               int64_t rows, int64_t N, void* stream) {
    return rmsnorm_bwd_any(dy, x, weight, weight_is_fp32, rstd, nullptr, dx, dw, workspace, workspace_bytes, rows, N, stream);
}

// Device address of `scratch` on the current device; looked up once per device.
static int static_scratch(void** out) {
    constexpr int kMaxDevices = 64;
    static void* ptrs[kMaxDevices] = {};
    static std::mutex lock;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return HYC_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(lock);
    if (!ptrs[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return HYC_ERR_LAUNCH;
        }
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return HYC_OK;
}

extern "C" int64_t hyc_rmsnorm_bwd_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int hyc_rmsnorm_bwd_static(const void* dy, const void* x, const void* weight, int weight_is_fp32,
                                      const float* rstd, void* dx, void* dw, int64_t rows, int64_t N, void* stream) {
    // sizes first, so that a caller learns about an oversized request without any device work
    if (rows < 0 || N < 0 || N % 8 != 0) return HYC_ERR_SHAPE;
    if (N > kNormMaxRegisterRow || hyc_rmsnorm_bwd_workspace(rows, N) > kStaticScratchBytes) return HYC_ERR_WORKSPACE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!dw) return HYC_ERR_NULL;
    void* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != HYC_OK) return rc;
    return rmsnorm_bwd_any(dy, x, weight, weight_is_fp32, rstd, nullptr, dx, dw, ws, kStaticScratchBytes, rows, N, stream);
}

extern "C" int hyc_rmsnorm_bwd_add(const void* dy, const void* x, const void* weight, int weight_is_fp32,
                                   const float* rstd, const void* residual, void* dx, void* dw, void* workspace,
                                   int64_t workspace_bytes, int64_t rows, int64_t N, void* stream) {
    if (!residual && rows > 0 && N > 0) return HYC_ERR_NULL;
    return rmsnorm_bwd_any(dy, x, weight, weight_is_fp32, rstd, residual, dx, dw, workspace, workspace_bytes, rows, N, stream);
}
