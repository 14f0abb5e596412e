// Calibration statistics for gfx950: per-channel min / max / sum of squares of batch
// element 0, the outlier-channel choice (top-k of the bf16 channel norms with a defined
// tie rule) and the per-channel step / zero point derived from them.
//
// Three kernels, no atomics on global memory, the same bits on every run:
//   channel_stats_kernel   the bandwidth-bound pass over [M, N]: rows split over workgroups as in the
//                          quantiser (lane = 16-byte chunk, a wave reads 1 KiB of one row per instruction);
//                          each workgroup leaves one partial row of (min, max, sum of squares) per strip of rows
//   channel_steps_kernel   one thread per channel: folds the strips in order, writes the step (and zero
//                          point) the channel has when it is not an outlier channel, and its sort key
//   channel_pick_kernel    one workgroup: the k largest keys by a radix select, the list in order, and the
//                          step of the chosen channels
#include <string.h>

#include "hyc_common.hpp"

namespace hyc {

constexpr int kStatThreads = 512;           // 8 waves; wave w of a workgroup reads rows w, w+8, ... of the strip
constexpr int kStatWaves = kStatThreads / kWave;
constexpr int kStatTileCols = kWave * 8;    // 512 channels = 1 KiB of a row per wave instruction
constexpr int kStatUnroll = 8;              // rows (KiB) a wave has in flight
constexpr int kStatFold = 32;                // strips one thread of the fold fetches at once
constexpr int kStatMaxStrips = 4 * kStatFold;
constexpr int kSelThreads = 1024;
constexpr int kSelMaxN = 32768;             // 32 keys per thread of the picking workgroup
constexpr int kSelRankMax = 1024;           // up to this many outlier channels are ordered by counting
constexpr int kSelReplicas = 32;            // copies of each histogram bin, one per LDS bank

// Waves the statistics launch aims for (hyc_set_tuning "stats_waves"): enough to keep every CU's memory
// pipeline full, few enough that the per-strip partial rows stay a small fraction of the input.
static Knob g_stat_waves{4096};

static int stat_strips(int64_t M, int64_t N) {
    const int64_t col_tiles = cdiv(N, kStatTileCols);
    int64_t strips = g_stat_waves.get() / (kStatWaves * col_tiles);
    const int64_t most = cdiv(M, (int64_t)kStatWaves * 4);          // at least four rows per wave
    if (strips > most) strips = most;
    if (strips > kStatMaxStrips) strips = kStatMaxStrips;
    return (int)(strips < 1 ? 1 : strips);
}

// torch.max / torch.min propagate NaN; fminf / fmaxf would drop it
__device__ __forceinline__ float nan_min(float a, float b) { return (b < a || b != b) ? b : a; }
__device__ __forceinline__ float nan_max(float a, float b) { return (b > a || b != b) ? b : a; }

// Workgroup (column tile, strip): 512 channels x rows [strip * rows_per_strip, ...).  Order of the sum of
// squares: a lane adds its rows in ascending order, then the eight waves are added in order, then (in
// channel_steps_kernel) the strips.
__global__ __launch_bounds__(kStatThreads) void channel_stats_kernel(const uint16_t* __restrict__ x, int M, int N,
                                                                     int64_t stride_m, int head_dim,
                                                                     int64_t stride_h, int rows_per_strip,
                                                                     float* __restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tiles = (N + kStatTileCols - 1) / kStatTileCols;
    const int col_tile = blockIdx.x % col_tiles, strip = blockIdx.x / col_tiles;
    const int col0 = col_tile * kStatTileCols + lane * 8;
    const bool active = col0 < N;
    const int row_begin = strip * rows_per_strip;
    const int row_end = min(M, row_begin + rows_per_strip);
    float mn[8], mx[8], sq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { mn[j] = INFINITY; mx[j] = -INFINITY; sq[j] = 0.0f; }
    if (active) {
        const int h = col0 / head_dim;
        const uint16_t* p = x + (int64_t)h * stride_h + (col0 - h * head_dim);
        auto take = [&](const u32x4 v) {
            float f[8];
            unpack8(v, f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                mn[j] = nan_min(mn[j], f[j]);
                mx[j] = nan_max(mx[j], f[j]);
                sq[j] = fmaf(f[j], f[j], sq[j]);
            }
        };
        // eight rows are requested before the first is used; past the strip's end the request repeats row m
        // and is dropped, so the last batch costs one memory round trip like the others
        for (int m = row_begin + wave; m < row_end; m += kStatUnroll * kStatWaves) {
            u32x4 v[kStatUnroll];
#pragma unroll
            for (int u = 0; u < kStatUnroll; ++u) {
                const int r = m + u * kStatWaves;
                v[u] = ld16_nt(p + (int64_t)(r < row_end ? r : m) * stride_m);      // streaming: +2 points of bandwidth
            }
#pragma unroll
            for (int u = 0; u < kStatUnroll; ++u)
                if (m + u * kStatWaves < row_end) take(v[u]);
        }
    }
    __shared__ float red[kStatWaves][3][kStatTileCols];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        red[wave][0][lane * 8 + j] = mn[j];
        red[wave][1][lane * 8 + j] = mx[j];
        red[wave][2][lane * 8 + j] = sq[j];
    }
    __syncthreads();
    // thread t folds channel t of the tile over the eight waves
    float* dst = out + (int64_t)strip * 3 * N;
    for (int c = threadIdx.x; c < kStatTileCols; c += kStatThreads) {
        const int col = col_tile * kStatTileCols + c;
        if (col >= N) break;
        float a = red[0][0][c], b = red[0][1][c], q = red[0][2][c];
#pragma unroll
        for (int w = 1; w < kStatWaves; ++w) {
            a = nan_min(a, red[w][0][c]);
            b = nan_max(b, red[w][1][c]);
            q += red[w][2][c];
        }
        dst[col] = a;
        dst[N + col] = b;
        dst[2 * (int64_t)N + col] = q;
    }
}

// step = bf16( bf16(max - min) / (2^q - 1) ) (+ 1e-3 where it is zero, on request), and the zero point
// z = -round_half_even(min / step) - 2^(q-1), each operation rounded to bf16, then a C cast to int8
// (operators/compress_function.py:50-54, :67-77, :93-104).
__device__ __forceinline__ void step_of(float lo, float hi, int q_bit, int add_eps, uint16_t* scale_at, int8_t* zp_at) {
    const float levels = (float)((1 << q_bit) - 1);
    const float half = (float)(1 << (q_bit - 1));
    const float d = rbf(hi - lo);                 // bf16 subtraction
    float s = rbf(d / levels);                    // bf16 / int
    if (add_eps && s == 0.0f) s = rbf(s + 1e-3f); // scale += (scale == 0) * 1e-3
    *scale_at = f_to_bf(s);
    if (zp_at) {
        const float t = rbf(lo / s);
        const float z = rbf(rbf(-rintf(t)) - half);
        const int zi = (z != z) ? 0 : (int)fminf(fmaxf(z, -2147483648.0f), 2147483520.0f);
        *zp_at = (int8_t)zi;
    }
}

// 64 channels per workgroup, four threads per channel: thread (channel, g) folds strips 32g .. 32g+31 in
// order (all fetched at once: one memory round trip, not one per strip), the four results are folded in
// order through LDS and left in the rows of strip 0.  Then, per channel: the step and zero point it has as a
// non-outlier and, with want_keys, its sort key
//   key = bf16_bits(norm) << 16 | (0xffff - channel)     norm = bf16(sqrt(fp32 sum of squares)), as torch's
// whose plain unsigned order is "norm descending, then channel ascending"; a NaN norm sorts first, as in
// torch.sort.  No two channels share a key and no key is zero (channel < 32768).
__global__ __launch_bounds__(256) void channel_steps_kernel(float* __restrict__ part, int strips, int N, int q_bit,
                                                             int add_eps, int want_keys, uint32_t* __restrict__ keys,
                                                             uint16_t* __restrict__ scale_out, int8_t* __restrict__ zp_out) {
    __shared__ float red[4][3][64];
    const int cl = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + cl;
    const bool live = c < N;
    const int64_t step = 3 * (int64_t)N;
    const int first = g * kStatFold;
    float a = INFINITY, b = -INFINITY, q = 0.0f;
    if (live && first < strips) {
        float va[kStatFold], vb[kStatFold], vq[kStatFold];
#pragma unroll
        for (int u = 0; u < kStatFold; ++u) {
            const float* p = part + (int64_t)(first + u < strips ? first + u : first) * step + c;
            va[u] = p[0];
            vb[u] = p[N];
            vq[u] = p[2 * (int64_t)N];
        }
        a = va[0]; b = vb[0]; q = vq[0];
#pragma unroll
        for (int u = 1; u < kStatFold; ++u) {
            if (first + u < strips) {
                a = nan_min(a, va[u]);
                b = nan_max(b, vb[u]);
                q += vq[u];
            }
        }
    }
    red[g][0][cl] = a;
    red[g][1][cl] = b;
    red[g][2][cl] = q;
    __syncthreads();
    if (g != 0 || !live) return;
    for (int w = 1; w < 4 && w * kStatFold < strips; ++w) {
        a = nan_min(a, red[w][0][cl]);
        b = nan_max(b, red[w][1][cl]);
        q += red[w][2][cl];
    }
    if (strips > 1) {
        part[c] = a;
        part[N + c] = b;
        part[2 * (int64_t)N + c] = q;
    }
    if (want_keys) {
        const float nrm = sqrtf(q);
        uint32_t nb = f_to_bf(nrm);
        if (nrm != nrm) nb = 0xffffu;
        keys[c] = (nb << 16) | (0xffffu - (uint32_t)c);
    }
    step_of(a, b, q_bit, add_eps, scale_out + c, zp_out ? zp_out + c : nullptr);
}

// Single workgroup: the k channels with the largest keys, in descending key order, and their step (that of
// an all-zero column, since their values are split off before the rest is quantised).
// The k-th largest key K is found by a radix select over the key's four bytes.  Each thread holds its keys in
// registers; a pass histograms one byte of the keys that still match the bytes found so far, in LDS with one
// copy of the 256 bins per bank (the top byte is the same for nearly every channel: a single copy would
// serialise the whole workgroup on one address), the copies are summed, and one wave scans the bins from the
// top.  The chosen channels are the keys >= K; a chosen key's place in the list is the number of chosen keys
// above it.
template <int KPT>
__global__ __launch_bounds__(kSelThreads) void channel_pick_kernel(const uint32_t* __restrict__ keys, int N, int k,
                                                                   int q_bit, int add_eps, int64_t* __restrict__ idx_out,
                                                                   uint16_t* __restrict__ scale_out,
                                                                   int8_t* __restrict__ zp_out) {
    __shared__ uint32_t hist[256 * kSelReplicas];
    __shared__ uint32_t total[256];
    __shared__ uint32_t chosen_keys[kSelRankMax];
    __shared__ uint32_t n_chosen;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    uint32_t key[KPT];
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
        const int c = tid + u * kSelThreads;
        key[u] = c < N ? keys[c] : 0u;            // 0: no channel; below every real key
    }
    if (tid == 0) n_chosen = 0;
#pragma unroll
    for (int i = 0; i < 256 * kSelReplicas / kSelThreads; ++i) hist[i * kSelThreads + tid] = 0;
    __syncthreads();
    uint32_t prefix = 0, mask = 0, remaining = (uint32_t)k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        // two barriers per pass: the copies are cleared by the thread that has just summed them, and every
        // wave scans the 256 totals for itself instead of waiting for one wave's answer
#pragma unroll
        for (int u = 0; u < KPT; ++u)
            if (key[u] != 0u && (key[u] & mask) == prefix)
                atomicAdd(&hist[((key[u] >> shift) & 0xffu) * kSelReplicas + (lane & (kSelReplicas - 1))], 1u);
        __syncthreads();
        {   // thread t: bin t / 4, a quarter of its copies; the four quarters meet with quad permutes
            const int bin = tid >> 2, part = tid & 3;
            uint32_t* mine = &hist[bin * kSelReplicas + part * (kSelReplicas / 4)];
            uint32_t v = 0;
#pragma unroll
            for (int i = 0; i < kSelReplicas / 4; ++i) { v += mine[i]; mine[i] = 0; }
            v += quad_xor1(v);
            v += quad_xor2(v);
            if (part == 0) total[bin] = v;
        }
        __syncthreads();
        {
            // lane l owns bins 255 - 4l .. 252 - 4l: ascending lanes walk the bins from the top
            const int top = 255 - 4 * lane;
            const uint32_t h0 = total[top], h1 = total[top - 1], h2 = total[top - 2], h3 = total[top - 3];
            const uint32_t own = h0 + h1 + h2 + h3;
            const uint32_t incl = wave_inclusive_scan(own), excl = incl - own;
            const bool here = excl < remaining && remaining <= incl;       // exactly one lane: it holds the bin of the k-th key
            const uint32_t r = remaining - excl;
            uint32_t bin, left;
            if (r <= h0) { bin = top; left = r; }
            else if (r <= h0 + h1) { bin = top - 1; left = r - h0; }
            else if (r <= h0 + h1 + h2) { bin = top - 2; left = r - h0 - h1; }
            else { bin = top - 3; left = r - h0 - h1 - h2; }
            const int src = __builtin_ctzll(__ballot(here));
            prefix |= (uint32_t)__builtin_amdgcn_readlane((int)bin, src) << shift;
            remaining = (uint32_t)__builtin_amdgcn_readlane((int)left, src);
        }
        mask |= 0xffu << shift;
    }
    const uint32_t kth_key = prefix;
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
        if (key[u] >= kth_key && key[u] != 0u) {
            chosen_keys[atomicAdd(&n_chosen, 1u)] = key[u];
            const int c = tid + u * kSelThreads;
            step_of(0.0f, 0.0f, q_bit, add_eps, scale_out + c, zp_out ? zp_out + c : nullptr);
        }
    }
    __syncthreads();
    if (tid < k) {
        const uint32_t mine = chosen_keys[tid];
        int rank = 0;
        for (int j0 = 0; j0 < k; j0 += 8) {          // eight entries per LDS round trip
            uint32_t other[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) other[u] = chosen_keys[(j0 + u) & (kSelRankMax - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) rank += (j0 + u < k) && other[u] > mine;
        }
        idx_out[rank] = (int64_t)(0xffffu - (mine & 0xffffu));
    }
}

// The same choice for lists longer than kSelRankMax: k rounds of a block-wide maximum over keys held in LDS.
__global__ __launch_bounds__(kSelThreads) void channel_pick_rounds_kernel(const uint32_t* __restrict__ keys_in, int N, int k,
                                                                          int q_bit, int add_eps,
                                                                          int64_t* __restrict__ idx_out,
                                                                          uint16_t* __restrict__ scale_out,
                                                                          int8_t* __restrict__ zp_out) {
    extern __shared__ uint32_t keys[];   // [N] keys; 0 marks a chosen channel
    __shared__ uint32_t wave_best[kSelThreads / kWave];
    __shared__ uint32_t winner;
    const int tid = threadIdx.x;
    uint32_t best = 0;
    for (int c = tid; c < N; c += kSelThreads) {
        const uint32_t key = keys_in[c];
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
            step_of(0.0f, 0.0f, q_bit, add_eps, scale_out + wc, zp_out ? zp_out + wc : nullptr);
        }
        // `winner` is rewritten only after the next barrier pair, so no extra barrier is needed here
    }
}

int tune_stats(const char* key, int value) {
    if (strcmp(key, "stats_waves") != 0) return 1;
    if (value < 4 || value > (1 << 20)) return HYC_ERR_ARG;
    g_stat_waves.set(value);
    return HYC_OK;
}

}  // namespace hyc

using namespace hyc;

/* see hyclora.h */
extern "C" int64_t hyc_channel_stats_strips(int64_t M, int64_t N) {
    if (M <= 0 || N <= 0 || N > (1 << 28) || M > INT32_MAX) return 1;
    return stat_strips(M, N);
}

extern "C" int hyc_channel_stats(const void* x, int64_t M, int64_t N, int64_t stride_m, int64_t head_dim,
                                 int64_t stride_h, float* stats, int64_t stats_bytes, void* stream) {
    if (M < 0 || N < 0 || N % 8 != 0 || M > INT32_MAX || N > (1 << 28)) return HYC_ERR_SHAPE;
    if (N == 0) return HYC_OK;
    if (!stats || (M > 0 && !x)) return HYC_ERR_NULL;
    if (head_dim <= 0 || head_dim % 8 != 0 || N % head_dim != 0) return HYC_ERR_SHAPE;
    if (!aligned16(x) || stride_m % 8 != 0 || stride_h % 8 != 0) return HYC_ERR_ALIGN;
    const int strips = M > 0 ? stat_strips(M, N) : 1;
    if (stats_bytes < ((int64_t)strips * 3 + 1) * N * (int64_t)sizeof(float)) return HYC_ERR_WORKSPACE;
    const int rows_per_strip = (int)cdiv(M > 0 ? M : 1, strips);
    const int64_t col_tiles = cdiv(N, kStatTileCols);
    hipLaunchKernelGGL(channel_stats_kernel, dim3((unsigned)(col_tiles * strips)), dim3(kStatThreads), 0,
                       (hipStream_t)stream, (const uint16_t*)x, (int)M, (int)N, stride_m, (int)head_dim, stride_h,
                       rows_per_strip, stats);
    return check_launch();
}

extern "C" int hyc_channel_select(float* stats, int64_t strips, int64_t N, int64_t k, int q_bit, int add_eps,
                                  int64_t* outlier_idx, void* scale, int8_t* zero_point, void* stream) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (N < 0 || k < 0 || k > N || k > 65535 || strips < 1 || strips > kStatMaxStrips) return HYC_ERR_SHAPE;
    if (k > 0 && N > kSelMaxN) return HYC_ERR_SHAPE;
    if (N > (1 << 28)) return HYC_ERR_SHAPE;
    if (N == 0) return HYC_OK;
    if (!stats || !scale || (k > 0 && !outlier_idx)) return HYC_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    uint32_t* keys = reinterpret_cast<uint32_t*>(stats + strips * 3 * N);      // the row after the strips
    hipLaunchKernelGGL(channel_steps_kernel, dim3((unsigned)cdiv(N, 64)), dim3(256), 0, st, stats, (int)strips, (int)N,
                       q_bit, add_eps, k > 0 ? 1 : 0, keys, (uint16_t*)scale, zero_point);
    if (k > 0 && k <= kSelRankMax) {
        const dim3 one(1), block(kSelThreads);
#define HYC_PICK(KPT) hipLaunchKernelGGL((channel_pick_kernel<KPT>), one, block, 0, st, (const uint32_t*)keys, (int)N, (int)k, \
                                         q_bit, add_eps, outlier_idx, (uint16_t*)scale, zero_point)
        if (N <= 4 * kSelThreads) HYC_PICK(4);
        else if (N <= 8 * kSelThreads) HYC_PICK(8);
        else if (N <= 16 * kSelThreads) HYC_PICK(16);
        else HYC_PICK(32);
#undef HYC_PICK
    } else if (k > 0) {
        const size_t lds = (size_t)N * sizeof(uint32_t);
        if (lds > 48 * 1024 &&
            hipFuncSetAttribute((const void*)channel_pick_rounds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return HYC_ERR_LAUNCH;
        hipLaunchKernelGGL(channel_pick_rounds_kernel, dim3(1), dim3(kSelThreads), lds, st, (const uint32_t*)keys, (int)N,
                           (int)k, q_bit, add_eps, outlier_idx, (uint16_t*)scale, zero_point);
    }
    return check_launch();
}
