// Calibration statistics for gfx950: per-channel min / max / sum of squares of batch
// element 0, the outlier-channel choice (top-k of the bf16 channel norms with a defined
// tie rule) and the per-channel step / zero point derived from them.
//
// These run only while a layer calibrates (the first few training iterations), so the
// design goal is one deterministic pass over the data and no atomics, not peak bandwidth.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kStatThreads = 1024;          // 8 column lanes x 128 row lanes
constexpr int kStatColLanes = 8;            // x 8 channels = 64 channels (128 B) per workgroup
constexpr int kStatRowLanes = kStatThreads / kStatColLanes;
constexpr int kSelThreads = 1024;
constexpr int kSelMaxN = 32768;             // channel keys live in LDS (128 KiB)

// One workgroup reduces 64 channels over all M rows.  Thread (rowlane, collane) walks rows
// rowlane, rowlane+128, ... of its 16-byte chunk; a wave therefore reads 8 rows x 128 B per
// load.  The reduction order is fixed (lane tree, then waves in order), so results do not
// change from run to run.
__global__ __launch_bounds__(kStatThreads) void channel_stats_kernel(const uint16_t* __restrict__ x, int M, int N,
                                                                     int64_t stride_m, int head_dim,
                                                                     int64_t stride_h, float* __restrict__ out) {
    const int collane = threadIdx.x & (kStatColLanes - 1);
    const int rowlane = threadIdx.x >> 3;
    const int col0 = (blockIdx.x * kStatColLanes + collane) * 8;
    const bool active = col0 < N;
    float mn[8], mx[8], sq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { mn[j] = INFINITY; mx[j] = -INFINITY; sq[j] = 0.0f; }
    if (active) {
        const int h = col0 / head_dim;
        const uint16_t* p = x + (int64_t)h * stride_h + (col0 - h * head_dim);
        for (int m = rowlane; m < M; m += kStatRowLanes) {
            float f[8];
            unpack8(ld16(p + (int64_t)m * stride_m), f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                // torch.max/min propagate NaN; fminf/fmaxf would drop it
                mn[j] = (f[j] < mn[j] || f[j] != f[j]) ? f[j] : mn[j];
                mx[j] = (f[j] > mx[j] || f[j] != f[j]) ? f[j] : mx[j];
                sq[j] = fmaf(f[j], f[j], sq[j]);
            }
        }
    }
    // lanes that differ in bits 3..5 hold other rows of the same columns
#pragma unroll
    for (int o = 8; o < kWave; o <<= 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float a = __shfl_xor(mn[j], o, kWave), b = __shfl_xor(mx[j], o, kWave);
            mn[j] = (a < mn[j] || a != a) ? a : mn[j];
            mx[j] = (b > mx[j] || b != b) ? b : mx[j];
            sq[j] += __shfl_xor(sq[j], o, kWave);
        }
    }
    __shared__ float red[kStatThreads / kWave][3][kStatColLanes * 8];
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & (kWave - 1)) < kStatColLanes) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            red[wave][0][collane * 8 + j] = mn[j];
            red[wave][1][collane * 8 + j] = mx[j];
            red[wave][2][collane * 8 + j] = sq[j];
        }
    }
    __syncthreads();
    if (threadIdx.x < kStatColLanes * 8) {
        const int c = blockIdx.x * kStatColLanes * 8 + threadIdx.x;
        if (c < N) {
            float a = red[0][0][threadIdx.x], b = red[0][1][threadIdx.x], s = red[0][2][threadIdx.x];
            for (int w = 1; w < kStatThreads / kWave; ++w) {
                const float a2 = red[w][0][threadIdx.x], b2 = red[w][1][threadIdx.x];
                a = (a2 < a || a2 != a2) ? a2 : a;
                b = (b2 > b || b2 != b2) ? b2 : b;
                s += red[w][2][threadIdx.x];
            }
            out[c] = a;
            out[N + c] = b;
            out[2 * (int64_t)N + c] = s;
        }
    }
}

// Single workgroup: choose the k channels with the largest bf16 norm (ties: lower channel
// first), then write the step (and optionally the zero point) of every channel.
//   key = bf16_bits(norm) << 16 | (0xffff - channel)   -> plain unsigned max = the rule above.
__global__ __launch_bounds__(kSelThreads) void channel_select_kernel(const float* __restrict__ stats, int N, int k,
                                                                     int q_bit, int add_eps,
                                                                     int64_t* __restrict__ idx_out,
                                                                     uint16_t* __restrict__ scale_out,
                                                                     int8_t* __restrict__ zp_out) {
    extern __shared__ uint32_t keys[];   // [N] keys; 0 marks a chosen channel
    __shared__ uint32_t wave_best[kSelThreads / kWave];
    __shared__ uint32_t winner;
    const int tid = threadIdx.x;
    const float* mn = stats;
    const float* mx = stats + N;
    const float* sq = stats + 2 * (int64_t)N;

    if (k > 0) {
        uint32_t best = 0;
        for (int c = tid; c < N; c += kSelThreads) {
            // torch: bf16 norm = bf16(sqrt(fp32 sum of squares)); a NaN norm sorts first, as in torch.sort
            const float nrm = sqrtf(sq[c]);
            uint32_t nb = f_to_bf(nrm);
            if (nrm != nrm) nb = 0xffffu;
            const uint32_t key = (nb << 16) | (0xffffu - (uint32_t)c);
            keys[c] = key;
            best = key > best ? key : best;
        }
        __syncthreads();
        for (int it = 0; it < k; ++it) {
            const uint32_t wb = wave_max_u32(best);
            if ((tid & (kWave - 1)) == 0) wave_best[tid >> 6] = wb;
            __syncthreads();
            if (tid < kWave) {
                uint32_t v = tid < kSelThreads / kWave ? wave_best[tid] : 0u;
                v = wave_max_u32(v);
                if (tid == 0) winner = v;
            }
            __syncthreads();
            const uint32_t win = winner;
            const int wc = (int)(0xffffu - (win & 0xffffu));
            if (tid == 0) idx_out[it] = wc;
            if (wc % kSelThreads == tid) {       // the owner retires the channel and rescans its own keys
                keys[wc] = 0u;
                best = 0;
                for (int c = tid; c < N; c += kSelThreads) best = keys[c] > best ? keys[c] : best;
            }
            // `winner` is rewritten only after the next barrier pair, so no extra barrier is needed here
        }
        __syncthreads();
    }

    const float levels = (float)((1 << q_bit) - 1);
    const float half = (float)(1 << (q_bit - 1));
    for (int c = tid; c < N; c += kSelThreads) {
        const bool chosen = (k > 0) && keys[c] == 0u;
        const float lo = chosen ? 0.0f : mn[c];
        const float hi = chosen ? 0.0f : mx[c];
        const float d = rbf(hi - lo);                 // bf16 subtraction
        float s = rbf(d / levels);                    // bf16 / int
        if (add_eps && s == 0.0f) s = rbf(s + 1e-3f); // scale += (scale == 0) * 1e-3
        scale_out[c] = f_to_bf(s);
        if (zp_out) {
            // z = -round_half_even(min / s) - 2^(q-1), each step in bf16, then a C cast to int8
            const float t = rbf(lo / s);
            const float z = rbf(rbf(-rintf(t)) - half);
            int zi = (z != z) ? 0 : (int)fminf(fmaxf(z, -2147483648.0f), 2147483520.0f);
            zp_out[c] = (int8_t)zi;
        }
    }
}

}  // namespace hyc

using namespace hyc;

/* see hyclora.h */
extern "C" int hyc_channel_stats(const void* x, int64_t M, int64_t N, int64_t stride_m, int64_t head_dim,
                                 int64_t stride_h, float* stats, void* stream) {
    if (M < 0 || N < 0 || N % 8 != 0 || M > INT32_MAX || N > (1 << 28)) return HYC_ERR_SHAPE;
    if (N == 0) return HYC_OK;
    if (!stats || (M > 0 && !x)) return HYC_ERR_NULL;
    if (head_dim <= 0 || head_dim % 8 != 0 || N % head_dim != 0) return HYC_ERR_SHAPE;
    if (!aligned16(x) || stride_m % 8 != 0 || stride_h % 8 != 0) return HYC_ERR_ALIGN;
    const dim3 grid((unsigned)cdiv(N, kStatColLanes * 8)), block(kStatThreads);
    hipLaunchKernelGGL(channel_stats_kernel, grid, block, 0, (hipStream_t)stream, (const uint16_t*)x, (int)M, (int)N,
                       stride_m, (int)head_dim, stride_h, stats);
    return check_launch();
}

extern "C" int hyc_channel_select(const float* stats, int64_t N, int64_t k, int q_bit, int add_eps,
                                  int64_t* outlier_idx, void* scale, int8_t* zero_point, void* stream) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (N < 0 || k < 0 || k > N || k > 65535) return HYC_ERR_SHAPE;
    if (k > 0 && N > kSelMaxN) return HYC_ERR_SHAPE;
    if (N > (1 << 28)) return HYC_ERR_SHAPE;
    if (N == 0) return HYC_OK;
    if (!stats || !scale || (k > 0 && !outlier_idx)) return HYC_ERR_NULL;
    const size_t lds = k > 0 ? (size_t)N * sizeof(uint32_t) : 0;
    if (lds > 64 * 1024) {
        if (hipFuncSetAttribute((const void*)channel_select_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return HYC_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(channel_select_kernel, dim3(1), dim3(kSelThreads), lds, (hipStream_t)stream, stats, (int)N,
                       (int)k, q_bit, add_eps, outlier_idx, (uint16_t*)scale, zero_point);
    return check_launch();
}
