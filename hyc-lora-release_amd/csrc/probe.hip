// Memory-only probe: a kernel that does nothing but load and store bf16 [T, N] tensors with the access
// shapes of the kernels of this library, so that a benchmark can put the rate the memory system gives a
// read / write mix beside the rate of the kernel that has that mix.  No arithmetic of the path is in it.
//   shape 0  "tile": a wave owns 128 columns (16 lanes x 16 bytes) and four rows per instruction and walks
//            a strip of rows in 16-row tiles - the fused LoRA-SiLU and LoRA-add kernels
//   shape 1  "row" : a wave owns 512 columns (1 KiB) of one row per instruction, four rows in flight - the
//            quantiser and the statistics kernel
#include "hyc_common.hpp"

namespace hyc {

struct ProbeArgs {
    const u32x4* r[3];
    u32x4* w[3];
    int64_t T;
    int C;                 // 16-byte chunks per row
    int col_tiles;
    int rows_per_wave;
};

template <int NR, int NW, bool TILE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void stream_probe_kernel(const ProbeArgs p) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int ct = blockIdx.x % p.col_tiles;
    const int64_t rt = blockIdx.x / p.col_tiles;
    const int chunk = TILE ? ct * 16 + (lane & 15) : ct * kWave + lane;
    const int g = TILE ? lane >> 4 : 0;
    if (chunk >= p.C) return;
    const int64_t r0 = (rt * 4 + wave) * (int64_t)p.rows_per_wave;
    int64_t r1 = r0 + p.rows_per_wave;
    if (r1 > p.T) r1 = p.T;
    constexpr int STEP = TILE ? 16 : 4;
    for (int64_t r = r0; r < r1; r += STEP) {
        u32x4 v[4][NR];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t row = TILE ? r + 4 * g + u : r + u;
#pragma unroll
            for (int k = 0; k < NR; ++k) v[u][k] = row < r1 ? ld16_nt(p.r[k] + row * p.C + chunk) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t row = TILE ? r + 4 * g + u : r + u;
            u32x4 o = v[u][0];
#pragma unroll
            for (int k = 1; k < NR; ++k) o ^= v[u][k];
#pragma unroll
            for (int k = 0; k < NW; ++k) {
                o.x += (uint32_t)k;
                if (row < r1) st16_nt(p.w[k] + row * p.C + chunk, o);
            }
        }
    }
}

template <int NR, int NW>
static void probe_launch(const ProbeArgs& p, int shape, unsigned grid, hipStream_t st) {
    if (shape == 0) hipLaunchKernelGGL((stream_probe_kernel<NR, NW, true>), dim3(grid), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((stream_probe_kernel<NR, NW, false>), dim3(grid), dim3(256), 0, st, p);
}

}  // namespace hyc

using namespace hyc;

/* see hyclora.h */
extern "C" int hyc_stream_probe(const void* const* reads, int n_reads, void* const* writes, int n_writes, int64_t T,
                                int64_t N, int shape, int rows_per_wave, void* stream) {
    if (!reads || !writes) return HYC_ERR_NULL;
    if (n_reads < 1 || n_reads > 3 || n_writes < 1 || n_writes > 3 || (shape != 0 && shape != 1)) return HYC_ERR_ARG;
    if (T < 0 || N < 0 || N % 8 != 0 || N > (1 << 28) || T > INT32_MAX) return HYC_ERR_SHAPE;
    if (rows_per_wave < 4 || rows_per_wave > 4096 || rows_per_wave % (shape == 0 ? 16 : 4) != 0) return HYC_ERR_ARG;
    if (T == 0 || N == 0) return HYC_OK;
    ProbeArgs p{};
    for (int k = 0; k < n_reads; ++k) {
        if (!reads[k]) return HYC_ERR_NULL;
        if (!aligned16(reads[k])) return HYC_ERR_ALIGN;
        p.r[k] = (const u32x4*)reads[k];
    }
    for (int k = 0; k < n_writes; ++k) {
        if (!writes[k]) return HYC_ERR_NULL;
        if (!aligned16(writes[k])) return HYC_ERR_ALIGN;
        p.w[k] = (u32x4*)writes[k];
    }
    p.T = T;
    p.C = (int)(N / 8);
    p.col_tiles = (int)cdiv(p.C, shape == 0 ? 16 : kWave);
    p.rows_per_wave = rows_per_wave;
    const int64_t grid = p.col_tiles * cdiv(T, 4 * (int64_t)rows_per_wave);
    if (grid > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define HYC_PROBE(NR, NW) if (n_reads == NR && n_writes == NW) probe_launch<NR, NW>(p, shape, (unsigned)grid, st);
    HYC_PROBE(1, 1) HYC_PROBE(1, 2) HYC_PROBE(1, 3)
    HYC_PROBE(2, 1) HYC_PROBE(2, 2) HYC_PROBE(2, 3)
    HYC_PROBE(3, 1) HYC_PROBE(3, 2) HYC_PROBE(3, 3)
#undef HYC_PROBE
    return check_launch();
}
