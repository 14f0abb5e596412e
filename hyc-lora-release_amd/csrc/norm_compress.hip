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
// Two kernels: the general one below, and a column-slab form further down for rows that are a
// whole number of 512-column slabs.
// General form: one wave owns one row, each lane CH 16-byte chunks of it, as in the plain forward kernel; the
// per-column steps are re-read per row (L2 hits, like the norm weight).  The row is parked in LDS
// after the sum of squares (each lane reads back only what it wrote, so no barrier is involved)
// and the second phase walks the chunks in a rolled loop: one copy of the quantiser code and a
// few dozen live registers instead of CH unrolled copies, which is what keeps enough waves
// resident to hide the latency of the per-chunk constant loads.
// Only frozen (calibrated) steps can be used here: during calibration the steps of y depend on y.
#include <cstring>
#include <type_traits>

#include "hyc_pack.hpp"

namespace hyc {

// Entry j of a lane's eight outlier-table entries: 1 + position in the channel list, 0 for an ordinary channel.
// A position past the list (a table built for another, longer list) is read as "ordinary channel": the
// kernels index x_outlier[row * k + position] with it.
__device__ __forceinline__ uint32_t table_pos(const uint32_t (&td)[4], int j, int k) {
    const uint32_t p = (td[j >> 1] >> (16 * (j & 1))) & 0xffffu;
    return p <= (uint32_t)k ? p : 0u;
}


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

// LoRA-A down contraction out of the same pass (column-slab kernel only): xa = y @ A for up to four
// blocks of 16 adapter rows, y being the bf16 output the kernel has just formed.  The layers compute
// `x_norm @ lora_A^T` for q, k and v (gate and up) right after the norm
// (models/utils/compute_utils.py:22 via fused_llama_layer_intra_inter_full_fuse.py:111-117, :218-226),
// each a library GEMM that reads the [T, N] output again.
constexpr int kXaBlocks = 4;
// Rows per matrix-core tile: 16 (every row of the 16x16x16 form used) where the tiles of all waves fit
// in LDS, i.e. up to 8 waves = 4096 columns - one workgroup per compute unit then - and 8 (rows 8..15 of
// the form stay empty) for wider rows.  Halving the tile doubles the adapter bytes pulled from L2 per
// row, which is what this phase is bound by (measured: ~10 TB/s of L2 hits).
template <int MAXW> constexpr int kXaRowsFor = MAXW <= 8 ? 16 : 8;
constexpr int kXaPitch = kWave * 8 + 8;      // bf16 elements per row of a wave's y tile in LDS (16 bytes of padding)
struct XaArgs {
    const uint16_t* w[kXaBlocks];    // block b: 16 consecutive rows of an adapter weight [R, N] (lora_A.weight), row-major
    uint16_t* out[kXaBlocks];        // its 16 result columns: out[b][row * stride[b] + j]
    int64_t stride[kXaBlocks];
    int valid[kXaBlocks];            // how many of the 16 rows exist (a rank that is not a multiple of 16)
    int nb;                          // blocks in use, 0 = no contraction
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
            ss += chunk_sumsq(f);                       // the plain forward kernel's order
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
                        const uint32_t p = table_pos(td, j, a.k);
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

// ------------------------------------------------------------------------------------
// Column-slab form for rows that are a whole number of 512-column slabs (hidden sizes 4096, 5120,
// 8192 ...) and even row counts.
//
// In the row-per-wave kernel above every wave re-reads the per-column constants of all its chunks
// (norm weight, two steps with their reciprocals, the outlier table) for a single row, and all
// waves of the launch move through "load, reduce, store" together.  Here a workgroup has one wave
// per slab and walks a strip of rows: a lane keeps ONE chunk of columns, so its constants live in
// registers for the whole strip, and the strip is streamed two rows at a time with the next two
// requested as soon as the current ones are unpacked (the rolling prefetch of the fused LoRA
// kernels).  The price is a workgroup-wide sum per row: each wave leaves its lanes' chunk sums in
// LDS, one barrier per two rows, and every wave then adds the slabs of each lane in column order
// and runs the butterfly over the lanes - the plain forward kernel's summation order, so rstd, y
// and all codes are the same bits as from the kernel above.  The partial sums are double-buffered:
// a wave can be at most one step ahead of the slowest one.
constexpr int kSlabRows = 2;                        // rows per step; row counts must be a multiple of it
static Knob g_slab_rows_per_group{0};               // strip height per workgroup; 0 = from the row count
static Knob g_slab_enabled{1};

// Compute units of the current device (asked once; 256 if the query fails).
static int compute_units() {
    static int n = 0;
    if (n == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            n = v;
        else
            n = 256;
    }
    return n;
}

// MAXW: the most waves a workgroup may have (8: rows up to 4096 columns, 16: up to 8192).  Four
// waves per SIMD either way: two workgroups of 8 waves or one of 16 on a compute unit.
// XA: also the LoRA-A contraction described at XaArgs.  A wave keeps the bf16 output of its slab for
// a tile of kXaRows rows in LDS, turns it into the A operand of v_mfma_f32_16x16x16_bf16 (K runs over
// the slab's 512 columns, 32 per step: lane (i, g) supplies columns 32m + 8g .. +7 of row i as two
// operands, and the adapter rows are loaded in the same column order, 16 bytes a lane, so that two
// consecutive steps consume whole 128-byte lines), and leaves a [rows x 16] fp32 partial per block;
// the slabs' partials are added in column order through LDS and rounded once.
template <int QBIT, bool W32, int MAXW, bool XA>
__global__ __launch_bounds__(MAXW * kWave) __attribute__((amdgpu_waves_per_eu(XA && MAXW <= 8 ? 2 : 4)))
void rmsnorm_fwd_compress_slab_kernel(const NormCompressArgs a, const XaArgs xa, int rows_per_group) {
    constexpr int G = kSlabRows;
    constexpr int kXaRows = kXaRowsFor<MAXW>;
    extern __shared__ float slab_part[];                // [2][G][waves][64], then (XA) [waves][kXaRows][kXaPitch] bf16
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;
    uint16_t* const ytile = reinterpret_cast<uint16_t*>(slab_part + 2 * G * nw * kWave) + wave * (kXaRows * kXaPitch);
    const int chunk = wave * kWave + lane;
    const int col = chunk * 8;
    const int N = a.N;
    const int row_bytes = N * QBIT / 8;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_group;
    int64_t r1 = r0 + rows_per_group;
    if (r1 > a.rows) r1 = a.rows;
    if (r0 >= r1) return;                               // whole workgroups leave together

    // per-column constants, once per strip
    float wf[8];
    if constexpr (W32) {
        const f32x4 w0 = *reinterpret_cast<const f32x4*>((const float*)a.w + col);
        const f32x4 w1 = *reinterpret_cast<const f32x4*>((const float*)a.w + col + 4);
        wf[0] = w0.x; wf[1] = w0.y; wf[2] = w0.z; wf[3] = w0.w;
        wf[4] = w1.x; wf[5] = w1.y; wf[6] = w1.z; wf[7] = w1.w;
    } else {
        unpack8(ld16((const uint16_t*)a.w + col), wf);
    }
    QuantCols<QBIT> qy, qx;
    qy.load(a.q_y ? a.scale_y : a.scale_x, col, a.q_y != nullptr);      // an unused set reads as steps of 1
    qx.load(a.q_x ? a.scale_x : a.scale_y, col, a.q_x != nullptr);
    u32x4 tv = {0, 0, 0, 0};
    if (a.q_x && a.k > 0) tv = ld16(a.otable + col);
    const uint32_t td[4] = {tv.x, tv.y, tv.z, tv.w};
    const bool has_outlier = (tv.x | tv.y | tv.z | tv.w) != 0u;
    const bool fast = __ballot(!(qy.fast && qx.fast)) == 0ull;          // uniform across the wave
    const float zero8[8] = {0, 0, 0, 0, 0, 0, 0, 0};

    u32x4 xv[G];
    auto request = [&](int64_t r) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g) xv[g] = ld16_nt(a.x + (r + g) * N + col);
    };
    auto step = [&](int64_t r, int buf, int tile_row, auto ahead_tag, auto fast_tag) __attribute__((always_inline)) {
        constexpr bool AHEAD = decltype(ahead_tag)::value;
        constexpr bool FAST = decltype(fast_tag)::value;
        float f[G][8];
        float* mine = slab_part + ((buf * G) * nw + wave) * kWave + lane;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            unpack8(xv[g], f[g]);
            mine[g * nw * kWave] = chunk_sumsq(f[g]);
        }
        if constexpr (AHEAD) request(r + G);
        // A barrier that orders LDS only: __syncthreads() would also wait for every global access in
        // flight - the rows just requested and the previous step's stores.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        float rstd[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float* all = slab_part + ((buf * G + g) * nw) * kWave + lane;
            float t = 0.0f;
#pragma unroll 4
            for (int w = 0; w < nw; ++w) t += all[w * kWave];            // slabs in column order
            t = wave_sum(t);
            rstd[g] = 1.0f / sqrtf(t / (float)N + a.eps);
        }
        if (wave == 0 && lane == 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) a.rstd[r + g] = rstd[g];
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int64_t row = r + g;
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (f[g][j] * rstd[g]) * wf[j];
            const u32x4 yv = pack8(o);
            st16_nt(a.y + row * N + col, yv);
            if constexpr (XA) *reinterpret_cast<u32x4*>(ytile + (tile_row + g) * kXaPitch + 8 * lane) = yv;
            uint32_t lo, hi;
            if (a.q_y) {
                float fy[8];
                unpack8(yv, fy);
                codes_to_words<QBIT, false, FAST>(fy, qy, zero8, lo, hi);
                store_packed<QBIT, true>(a.q_y + row * row_bytes, chunk, true, lo, hi);
            }
            if (a.q_x) {
                if (has_outlier) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t p = table_pos(td, j, a.k);
                        if (p) {
                            a.xo[row * a.k + (p - 1)] = (uint16_t)(__float_as_uint(f[g][j]) >> 16);
                            f[g][j] = 0.0f;
                        }
                    }
                }
                codes_to_words<QBIT, false, FAST>(f[g], qx, zero8, lo, hi);
                store_packed<QBIT, true>(a.q_x + row * row_bytes, chunk, true, lo, hi);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // The LoRA-A contraction of the tile rows [t0, t0 + nrows) that the steps above left in LDS.
    auto contract = [&](int64_t t0, int nrows) __attribute__((always_inline)) {
        const int i = lane & 15, g = lane >> 4;
        f32x4 acc[kXaBlocks];
        const uint16_t* wp[kXaBlocks];
#pragma unroll
        for (int b = 0; b < kXaBlocks; ++b) {
            acc[b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const bool have = b < xa.nb && i < xa.valid[b];
            wp[b] = have ? xa.w[b] + (int64_t)i * N + wave * (kWave * 8) + 8 * g : nullptr;
        }
        const uint16_t* yrow = ytile + i * kXaPitch + 8 * g;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");          // the tile rows written by this wave's other lanes
        __builtin_amdgcn_wave_barrier();
        u32x4 bw[2][kXaBlocks];
        auto fetch = [&](int m, u32x4 (&dst)[kXaBlocks]) __attribute__((always_inline)) {
#pragma unroll
            for (int b = 0; b < kXaBlocks; ++b) {
                dst[b] = u32x4{0, 0, 0, 0};
                if (b < xa.nb && wp[b]) dst[b] = ld16(wp[b] + 32 * m);
            }
        };
        fetch(0, bw[0]);
#pragma unroll 2
        for (int m = 0; m < kWave * 8 / 32; m += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (m + h + 1 < kWave * 8 / 32) fetch(m + h + 1, bw[(h + 1) & 1]);
                u32x4 av = {0, 0, 0, 0};
                if (i < kXaRows) av = *reinterpret_cast<const u32x4*>(yrow + 32 * (m + h));
                const s16x4 a0 = __builtin_bit_cast(s16x4, u32x2{av.x, av.y});
                const s16x4 a1 = __builtin_bit_cast(s16x4, u32x2{av.z, av.w});
#pragma unroll
                for (int b = 0; b < kXaBlocks; ++b) {
                    if (b < xa.nb) {
                        const u32x4 w4 = bw[h & 1][b];
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a0, __builtin_bit_cast(s16x4, u32x2{w4.x, w4.y}), acc[b], 0, 0, 0);
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a1, __builtin_bit_cast(s16x4, u32x2{w4.z, w4.w}), acc[b], 0, 0, 0);
                    }
                }
            }
        }
        // the slab's partial, rows x (16 per block), into this wave's own tile region (its reads of it
        // are done: a wave's LDS operations complete in order)
        float* part = reinterpret_cast<float*>(ytile);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (g < kXaRows / 4) {
#pragma unroll
            for (int b = 0; b < kXaBlocks; ++b) {
                if (b < xa.nb) {
                    const float e[4] = {acc[b].x, acc[b].y, acc[b].z, acc[b].w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) part[(4 * g + v) * (16 * kXaBlocks) + 16 * b + i] = e[v];
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        const float* all = reinterpret_cast<const float*>(reinterpret_cast<const uint16_t*>(slab_part + 2 * G * nw * kWave));
        constexpr int kWaveFloats = kXaRows * kXaPitch / 2;             // a wave's tile region in floats
        for (int o = threadIdx.x; o < kXaRows * 16 * kXaBlocks; o += blockDim.x) {
            const int row = o / (16 * kXaBlocks), c = o % (16 * kXaBlocks), b = c >> 4, j = c & 15;
            if (row < nrows && b < xa.nb && j < xa.valid[b]) {
                float sum = 0.0f;
                for (int w = 0; w < nw; ++w) sum += all[w * kWaveFloats + o];          // slabs in column order
                xa.out[b][(t0 + row) * xa.stride[b] + j] = f_to_bf(sum);
            }
        }
    };
    auto run = [&](auto fast_tag) __attribute__((always_inline)) {
        request(r0);
        int64_t r = r0;
        int buf = 0;
        if (r + G < r1) {
            step(r, buf, (int)(r - r0), std::true_type{}, fast_tag);
            for (r += G, buf ^= 1; r + G < r1; r += G, buf ^= 1) step(r, buf, (int)(r - r0), std::true_type{}, fast_tag);
        }
        step(r, buf, (int)(r - r0), std::false_type{}, fast_tag);
    };
    // every wave of the workgroup makes the same number of steps whichever branch it takes
    if (fast) run(std::true_type{});
    else run(std::false_type{});
    // With the contraction a workgroup's strip is one tile (the launch sees to that), so this comes
    // when nothing of the row loop is live any more: its registers are the contraction's.
    if constexpr (XA) contract(r0, (int)(r1 - r0));
}

// ------------------------------------------------------------------------------------
// RMSNorm backward that reads its input from the channel-base compressed copy the forward kernels
// above leave behind (codes, steps, outlier values), in the same column-slab decomposition: the
// layers otherwise restore x to a dense tensor first
// (outlier_addition_fuse_decompression_dequantization, then rmsnorm_backward:
// models/llama/fused_llama_layer_intra_inter_full_fuse.py:386-393, :486-493).  A lane's per-column
// constants (norm weight, step, outlier positions) stay in registers for a strip of rows; a row's
// two sums (x^ . w dy and w dy) go through LDS like the forward kernel's sum of squares, in the
// dense backward kernel's summation order, so dx is the same bits as from dequantise + backward.
// Optionally adds the residual connection's gradient, like hyc_rmsnorm_bwd_add.
struct NormBwdCodesArgs {
    const uint16_t* x;                                  // the norm's input itself (QBIT = 0) instead of its compressed copy
    const uint16_t* dy; const uint8_t* q_x; const uint16_t* scale_x;
    const uint16_t* otable; const uint16_t* xo;
    const void* w; const float* rstd; const uint16_t* res; uint16_t* dx;
    int64_t rows;
    int N, k;
};

template <int QBIT, bool W32, int MAXW, bool RES>
__global__ __launch_bounds__(MAXW * kWave) __attribute__((amdgpu_waves_per_eu(4)))
void rmsnorm_bwd_codes_slab_kernel(const NormBwdCodesArgs a, int rows_per_group) {
    constexpr int G = RES ? 1 : kSlabRows;              // with a residual: one row per step, or registers spill
    extern __shared__ float slab_part[];                // [2][G][2][waves][64]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;
    const int chunk = wave * kWave + lane;
    const int col = chunk * 8;
    const int N = a.N;
    // QBIT = 0: x is read as it is (the stand-alone backward for rows longer than a wave holds well);
    // everything after the load is the same code, so the results are the same bits
    constexpr bool DENSE = QBIT == 0;
    constexpr int QB = DENSE ? 8 : QBIT;
    const int row_bytes = N * QB / 8;
    constexpr float kHalf = (float)(1 << (QB - 1));
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_group;
    int64_t r1 = r0 + rows_per_group;
    if (r1 > a.rows) r1 = a.rows;
    if (r0 >= r1) return;                               // whole workgroups leave together

    // Per-column constants, kept packed where they are bf16 (registers are what limits this kernel
    // to four waves per SIMD): norm weight, steps, and the lane's outlier columns.
    float wf[W32 ? 8 : 1];
    u32x4 wp = {0, 0, 0, 0};
    if constexpr (W32) {
        const f32x4 w0 = *reinterpret_cast<const f32x4*>((const float*)a.w + col);
        const f32x4 w1 = *reinterpret_cast<const f32x4*>((const float*)a.w + col + 4);
        wf[0] = w0.x; wf[1] = w0.y; wf[2] = w0.z; wf[3] = w0.w;
        wf[4] = w1.x; wf[5] = w1.y; wf[6] = w1.z; wf[7] = w1.w;
    } else {
        wp = ld16((const uint16_t*)a.w + col);
    }
    auto weight8 = [&](float (&out)[8]) __attribute__((always_inline)) {
        if constexpr (W32) {
#pragma unroll
            for (int j = 0; j < 8; ++j) out[j] = wf[j];
        } else {
            unpack8(wp, out);
        }
    };
    u32x4 sp = {0, 0, 0, 0};
    if constexpr (!DENSE) sp = ld16(a.scale_x + col);
    // Outlier columns of this lane: the first two are fetched ahead with the row (slots 1 and 2 of
    // `oslot`, two bits a column), any further one when it is used (slot 3).  Few lanes have any.
    u32x4 tv = {0, 0, 0, 0};
    if (!DENSE && a.k > 0) tv = ld16(a.otable + col);
    const uint32_t td[4] = {tv.x, tv.y, tv.z, tv.w};
    uint32_t oslot = 0, opos0 = 0, opos1 = 0;
    {
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t p = table_pos(td, j, a.k);
            if (p) {
                oslot |= (uint32_t)(cnt < 2 ? cnt + 1 : 3) << (2 * j);
                if (cnt == 0) opos0 = p - 1;
                if (cnt == 1) opos1 = p - 1;
                ++cnt;
            }
        }
    }
    const PackedSlot<QB> slot(chunk);
    const float inv_n = 1.0f / (float)N;

    u32x2 cw[G];
    u32x4 xd[DENSE ? G : 1];
    u32x4 gv[G];
    float rs[G];
    uint32_t ov[G][2];
    auto request = [&](int64_t r) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int64_t row = r + g;
            if constexpr (DENSE) xd[g] = ld16_nt(a.x + row * N + col);
            else cw[g] = ld8(a.q_x + row * row_bytes + slot.offset);
            gv[g] = ld16_nt(a.dy + row * N + col);
            rs[g] = a.rstd[row];
            if (!DENSE && oslot) {
                ov[g][0] = a.xo[row * a.k + opos0];
                if (oslot & 0xaaaau) ov[g][1] = a.xo[row * a.k + opos1];        // a second outlier column
            }
        }
    };
    auto step = [&](int64_t r, int buf, auto ahead_tag) __attribute__((always_inline)) {
        constexpr bool AHEAD = decltype(ahead_tag)::value;
        // What a row needs after the barrier is kept packed (x is a bf16 value by construction) and
        // unpacked again there: 12 registers a row instead of 24.
        u32x4 xp[G], gp[G];
        float rstd[G];
        float* mine = slab_part + ((buf * G) * 2 * nw + wave) * kWave + lane;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float c[8], gf[8], x[8], sf[8], w8[8];
            unpack8(gv[g], gf);
            weight8(w8);
            gp[g] = gv[g];
            rstd[g] = rs[g];
            if constexpr (DENSE) {
                xp[g] = xd[g];
            } else {
            slot.decode(cw[g], c);
            unpack8(sp, sf);
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = (c[j] - kHalf) * sf[j];  // the dequantiser's arithmetic ...
            if (oslot) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t code = (oslot >> (2 * j)) & 3u;
                    if (code == 1) x[j] = __uint_as_float(ov[g][0] << 16);
                    else if (code == 2) x[j] = __uint_as_float(ov[g][1] << 16);
                    else if (code == 3) {
                        const uint32_t p = table_pos(td, j, a.k);
                        x[j] = __uint_as_float((uint32_t)a.xo[(r + g) * a.k + (p - 1)] << 16);
                    }
                }
            }
            xp[g] = pack8(x);                                           // ... and its rounding to bf16
            }
            unpack8(xp[g], x);
            float p1 = 0.0f, p2 = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = x[j] * rstd[g], wdy = w8[j] * gf[j];
                p1 = fmaf(xh, wdy, p1);
                p2 += wdy;
            }
            mine[(g * 2 + 0) * nw * kWave] = p1;
            mine[(g * 2 + 1) * nw * kWave] = p2;
            __builtin_amdgcn_sched_barrier(0);          // one row at a time: fewer live temporaries
        }
        // The residual is asked for only now, for the rows of THIS step (the barrier and the sums
        // below cover most of its latency): fetched a step ahead like the rest it would need
        // registers this kernel does not have at four waves per SIMD.
        u32x4 rv[RES ? G : 1];
        if constexpr (RES) {
#pragma unroll
            for (int g = 0; g < G; ++g) rv[g] = ld16_nt(a.res + (r + g) * N + col);
        }
        if constexpr (AHEAD) request(r + G);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");   // LDS-only barrier, see above
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float* all = slab_part + ((buf * G + g) * 2 * nw) * kWave + lane;
            float t1 = 0.0f, t2 = 0.0f;
#pragma unroll 4
            for (int w = 0; w < nw; ++w) {
                t1 += all[w * kWave];
                t2 += all[(nw + w) * kWave];
            }
            const float c1 = wave_sum(t1) * inv_n, c2 = wave_sum(t2) * inv_n;
            float x[8], gf[8], rf[8], w8[8], o[8];
            unpack8(xp[g], x);
            unpack8(gp[g], gf);
            weight8(w8);
            if constexpr (RES) unpack8(rv[g], rf);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = x[j] * rstd[g], wdy = w8[j] * gf[j];
                o[j] = (wdy - (xh * c1 + c2)) * rstd[g];
                if constexpr (RES) o[j] = rbf(o[j]) + rf[j];
            }
            st16_nt(a.dx + (r + g) * N + col, pack8(o));
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    request(r0);
    int64_t r = r0;
    int buf = 0;
    if (r + G < r1) {
        step(r, buf, std::true_type{});
        for (r += G, buf ^= 1; r + G < r1; r += G, buf ^= 1) step(r, buf, std::true_type{});
    }
    step(r, buf, std::false_type{});
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

static bool slab_shape(int64_t rows, int64_t N) {
    return N % (kWave * 8) == 0 && N / (kWave * 8) <= 16 && rows % kSlabRows == 0;
}

// Launch with more dynamic LDS than the 64 KiB a kernel may use without asking.
template <typename K>
static void launch_slab(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t st, const NormCompressArgs& a,
                        const XaArgs& xa, int rows_per_group) {
    if (lds > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kernel, grid, block, lds, st, a, xa, rows_per_group);
}

template <int QBIT, bool W32>
static int launch_nc(const NormCompressArgs& a, const XaArgs& xa, hipStream_t st) {
    if ((g_slab_enabled.get() || xa.nb > 0) && slab_shape(a.rows, a.N)) {
        const int waves = a.N / (kWave * 8);
        // Strip height: all workgroups resident at once (16 waves per compute unit), each walking as
        // long a strip as that allows - the per-column constants are set up once per strip.
        int rows_per_group = g_slab_rows_per_group.get();
        if (rows_per_group == 0) {
            const int64_t resident = (int64_t)compute_units() * (16 / (waves <= 8 ? waves : 16));
            rows_per_group = (int)(cdiv(cdiv(a.rows, resident), (int64_t)kSlabRows) * kSlabRows);
        }
        if (xa.nb > 0) rows_per_group = waves <= 8 ? kXaRowsFor<8> : kXaRowsFor<16>;      // one matrix-core tile per workgroup
        const int64_t groups = cdiv(a.rows, (int64_t)rows_per_group);
        if (groups > INT32_MAX) return HYC_ERR_SHAPE;
        size_t lds = 2 * kSlabRows * waves * kWave * sizeof(float);
        const dim3 grid((unsigned)groups), block(waves * kWave);
        if (xa.nb > 0) {
            if constexpr (W32) {
                return HYC_ERR_ARG;                             // the contraction is built for bf16 norm weights only
            } else {
                lds += (size_t)waves * rows_per_group * kXaPitch * sizeof(uint16_t);
                if (waves <= 8) launch_slab(rmsnorm_fwd_compress_slab_kernel<QBIT, false, 8, true>, grid, block, lds, st, a, xa, rows_per_group);
                else launch_slab(rmsnorm_fwd_compress_slab_kernel<QBIT, false, 16, true>, grid, block, lds, st, a, xa, rows_per_group);
            }
        } else if (waves <= 8) {
            launch_slab(rmsnorm_fwd_compress_slab_kernel<QBIT, W32, 8, false>, grid, block, lds, st, a, xa, rows_per_group);
        } else {
            launch_slab(rmsnorm_fwd_compress_slab_kernel<QBIT, W32, 16, false>, grid, block, lds, st, a, xa, rows_per_group);
        }
        return check_launch();
    }
    if (xa.nb > 0) return HYC_ERR_SHAPE;                        // only the column-slab kernel contracts
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

int tune_norm_compress(const char* key, int value) {
    if (strcmp(key, "norm_compress_slab") == 0) {
        if (value != 0 && value != 1) return HYC_ERR_ARG;
        g_slab_enabled.set(value);
        return HYC_OK;
    }
    if (strcmp(key, "norm_compress_rows_per_group") == 0) {
        if (value < 0 || value > 65536 || value % kSlabRows != 0) return HYC_ERR_ARG;   // 0: choose from the row count
        g_slab_rows_per_group.set(value);
        return HYC_OK;
    }
    return 1;
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

static int norm_compress_any(const void* x, const void* weight, int weight_is_fp32, void* y, float* rstd,
                             int64_t rows, int64_t N, float eps, int q_bit, const void* scale_y, void* q_y,
                             const void* scale_x, void* q_x, const uint16_t* outlier_table, int64_t k,
                             void* x_outlier, const XaArgs& xa, void* stream) {
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
#define HYC_NC_Q(QB) (weight_is_fp32 ? launch_nc<QB, true>(a, xa, st) : launch_nc<QB, false>(a, xa, st))
    if (q_bit == 8) return HYC_NC_Q(8);
    if (q_bit == 4) return HYC_NC_Q(4);
    return HYC_NC_Q(2);
#undef HYC_NC_Q
}

extern "C" int hyc_rmsnorm_fwd_compress(const void* x, const void* weight, int weight_is_fp32, void* y, float* rstd,
                                        int64_t rows, int64_t N, float eps, int q_bit, const void* scale_y, void* q_y,
                                        const void* scale_x, void* q_x, const uint16_t* outlier_table, int64_t k,
                                        void* x_outlier, void* stream) {
    XaArgs none{};
    return norm_compress_any(x, weight, weight_is_fp32, y, rstd, rows, N, eps, q_bit, scale_y, q_y, scale_x, q_x,
                             outlier_table, k, x_outlier, none, stream);
}

extern "C" int hyc_rmsnorm_fwd_compress_lora(const void* x, const void* weight, void* y, float* rstd, int64_t rows, int64_t N,
                                             float eps, int q_bit, const void* scale_y, void* q_y, const void* scale_x,
                                             void* q_x, const uint16_t* outlier_table, int64_t k, void* x_outlier,
                                             int n_adapters, const void* const* adapter_weight, const int64_t* adapter_rank,
                                             void* const* adapter_out, void* stream) {
    if (n_adapters < 1 || n_adapters > kXaBlocks) return HYC_ERR_ARG;
    if (!adapter_weight || !adapter_rank || !adapter_out) return HYC_ERR_NULL;
    if (rows < 0 || N < 0) return HYC_ERR_SHAPE;
    if (rows > 0 && N > 0 && !slab_shape(rows, N)) return HYC_ERR_SHAPE;
    XaArgs xa{};
    for (int g = 0; g < n_adapters; ++g) {
        const int64_t R = adapter_rank[g];
        if (R < 1 || R > 16 * kXaBlocks) return HYC_ERR_RANK;
        if (!adapter_weight[g] || !adapter_out[g]) return HYC_ERR_NULL;
        if (!aligned16(adapter_weight[g])) return HYC_ERR_ALIGN;
        for (int64_t r0 = 0; r0 < R; r0 += 16) {               // an adapter of rank R occupies ceil(R / 16) blocks
            if (xa.nb == kXaBlocks) return HYC_ERR_RANK;
            xa.w[xa.nb] = (const uint16_t*)adapter_weight[g] + r0 * N;
            xa.out[xa.nb] = (uint16_t*)adapter_out[g] + r0;
            xa.stride[xa.nb] = R;
            xa.valid[xa.nb] = (int)(R - r0 < 16 ? R - r0 : 16);
            ++xa.nb;
        }
    }
    return norm_compress_any(x, weight, 0, y, rstd, rows, N, eps, q_bit, scale_y, q_y, scale_x, q_x, outlier_table, k,
                             x_outlier, xa, stream);
}

// Shared launch of the slab backward: q_bit 2 / 4 / 8 = x from its codes, 0 = x itself.
static int launch_bwd_slab(const NormBwdCodesArgs& a, int q_bit, int weight_is_fp32, hipStream_t st) {
    const int64_t rows = a.rows;
    const int waves = a.N / (kWave * 8);
    int rows_per_group = g_slab_rows_per_group.get();
    if (rows_per_group == 0) {
        const int64_t resident = (int64_t)compute_units() * (16 / (waves <= 8 ? waves : 16));
        rows_per_group = (int)(cdiv(cdiv(rows, resident), (int64_t)kSlabRows) * kSlabRows);
    }
    const int64_t groups = cdiv(rows, (int64_t)rows_per_group);
    if (groups > INT32_MAX) return HYC_ERR_SHAPE;
    const size_t lds = 2 * kSlabRows * 2 * waves * kWave * sizeof(float);
    const dim3 grid((unsigned)groups), block(waves * kWave);
#define HYC_NBC(QB, W32, MAXW)                                                                                          \
    do {                                                                                                                \
        if (a.res) hipLaunchKernelGGL((rmsnorm_bwd_codes_slab_kernel<QB, W32, MAXW, true>), grid, block, lds, st, a, rows_per_group); \
        else hipLaunchKernelGGL((rmsnorm_bwd_codes_slab_kernel<QB, W32, MAXW, false>), grid, block, lds, st, a, rows_per_group);      \
    } while (0)
#define HYC_NBC_W(QB)                                                      \
    do {                                                                   \
        if (weight_is_fp32) { if (waves <= 8) HYC_NBC(QB, true, 8); else HYC_NBC(QB, true, 16); }   \
        else { if (waves <= 8) HYC_NBC(QB, false, 8); else HYC_NBC(QB, false, 16); }                \
    } while (0)
    if (q_bit == 8) HYC_NBC_W(8);
    else if (q_bit == 4) HYC_NBC_W(4);
    else if (q_bit == 2) HYC_NBC_W(2);
    else HYC_NBC_W(0);
#undef HYC_NBC_W
#undef HYC_NBC
    return check_launch();
}

namespace hyc {
// RMSNorm backward (dx only) of a dense input in the column-slab form; norm.hip sends rows longer than
// 4096 channels here.  Returns 1 when the shape does not fit the slabs (the caller keeps its own kernel).
int rmsnorm_bwd_dense_slab(const void* dy, const void* x, const void* weight, int weight_is_fp32, const float* rstd,
                           const void* residual, void* dx, int64_t rows, int64_t N, void* stream) {
    if (!g_slab_enabled.get() || !slab_shape(rows, N)) return 1;       // "norm_compress_slab" 0: the row-per-wave kernel
    NormBwdCodesArgs a{};
    a.x = (const uint16_t*)x; a.dy = (const uint16_t*)dy; a.w = weight; a.rstd = rstd;
    a.res = (const uint16_t*)residual; a.dx = (uint16_t*)dx; a.rows = rows; a.N = (int)N; a.k = 0;
    return launch_bwd_slab(a, 0, weight_is_fp32, (hipStream_t)stream);
}
}  // namespace hyc

extern "C" int hyc_rmsnorm_bwd_codes(const void* dy, const void* q_x, const void* scale_x, const uint16_t* outlier_table,
                                     int64_t k, const void* x_outlier, int q_bit, const void* weight, int weight_is_fp32,
                                     const float* rstd, const void* residual, void* dx, int64_t rows, int64_t N,
                                     void* stream) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (rows < 0 || N < 0 || k < 0 || k > 65535) return HYC_ERR_SHAPE;
    if (N % (kWave * 8) != 0 || N / (kWave * 8) > 16 || rows % kSlabRows != 0) return HYC_ERR_SHAPE;
    if (rows == 0 || N == 0) return HYC_OK;
    if (!dy || !q_x || !scale_x || !weight || !rstd || !dx || (k > 0 && (!outlier_table || !x_outlier))) return HYC_ERR_NULL;
    if (!aligned16(dy) || !aligned16(scale_x) || !aligned16(weight) || !aligned16(dx) || !aligned16(residual) ||
        (outlier_table && !aligned16(outlier_table)) || (reinterpret_cast<uintptr_t>(q_x) & 7u))
        return HYC_ERR_ALIGN;
    NormBwdCodesArgs a{};
    a.dy = (const uint16_t*)dy; a.q_x = (const uint8_t*)q_x; a.scale_x = (const uint16_t*)scale_x;
    a.otable = outlier_table; a.xo = (const uint16_t*)x_outlier; a.w = weight; a.rstd = rstd;
    a.res = (const uint16_t*)residual; a.dx = (uint16_t*)dx; a.rows = rows; a.N = (int)N; a.k = (int)k;
    return launch_bwd_slab(a, q_bit, weight_is_fp32, (hipStream_t)stream);
}
