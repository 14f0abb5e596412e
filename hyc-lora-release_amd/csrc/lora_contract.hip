// The skinny LoRA products that stream a whole [T, N] tensor X for a rank-R result, for gfx950:
//
//   P1 = U^T . X   [R, N]   (contraction over the T rows;    U is [T, R])
//   P2 = X . V^T   [T, R]   (contraction over the N columns; V is [R, N])
//
// from ONE read of X, which is either dense bf16 or - for P1 - the packed codes of a compressed
// activation, dequantised in registers.  These are the four rank-R GEMMs of lora_forward /
// lora_backward (models/utils/compute_utils.py:22, :30-33):
//   x @ A                      P2 with V = A^T (the [R, in] layout nn.Linear keeps lora_A.weight in)
//   grad_y @ B^T, xa^T @ grad_y   P2 and P1 of the same X = grad_y in one pass
//   x^T @ grad_medium          P1, with x taken straight from its codes where the layer saved it
//                              compressed (the reference dequantises first,
//                              fused_llama_layer_intra_inter_full_fuse.py:375-383, :469-481).
// A library GEMM runs each of them at a fraction of the memory rate (output tiles 16 wide) and
// reads X once per product.
//
// Layout.  A workgroup of 4 waves owns a strip of 256 rows and a group of column tiles (128
// columns each); wave w walks rows 64w .. 64w+63 of the strip, 16 at a time.  X is held twice:
//   "chunk" form  lane (j = l%16, g = l/16): rows 4g .. 4g+3, columns 8j .. 8j+7  (16-byte loads)
//   "row"   form  lane (i = l%16, g = l/16): row i, columns 16s + 4g .. +3, s = 0..7
// P1 uses the chunk form as the B operand of v_mfma_f32_16x16x16_bf16 with permuted column slots
// (MFMA u takes column 8j + u of every lane), so a lane ends up with 8 consecutive columns of 4
// LoRA rows; P2 uses the row form as the A operand, K running over the columns.  Only the chunk
// form is loaded from memory (256 contiguous bytes per row and instruction); the row form is the
// same tile turned through LDS, wave by wave.
// Sums across waves (P1: the four waves of a workgroup through LDS, then across strips; P2: across
// column groups) go through fp32 partial buffers in a fixed order - no atomics, so results do not
// depend on scheduling - and a small second kernel adds the partials and rounds to bf16.
#include "hyc_pack.hpp"

namespace hyc {

constexpr int kCtThreads = 256;
constexpr int kCtWaves = kCtThreads / kWave;
#ifndef HYC_CT_STEPS
#define HYC_CT_STEPS 4
#endif
constexpr int kCtSteps = HYC_CT_STEPS;                    // 16-row steps per wave
constexpr int kCtStrip = kCtWaves * kCtSteps * 16;        // 256 rows per workgroup
constexpr int kCtTile = 128;                              // columns per tile
constexpr int kCtPitch = kCtTile + 8;                     // LDS row pitch of a transposed tile (bf16 elements)
static Knob g_ct_max_groups{32};                          // column groups (bounds the P2 partials); see hyc_set_tuning

struct ContractArgs {
    const uint16_t* x;                   // dense X [T, N]
    const uint8_t* q;                    // or packed codes [T, N*q_bit/8] with
    const uint16_t* s; const uint16_t* zp;   //   steps / zero points bf16 [N]
    const uint16_t* u;                   // [T, R]
    const uint16_t* v;                   // [R, N], or [N, R] with v_transposed
    float* part1;                        // [strips][16*NB][N]
    float* part2;                        // [groups][T][16*NB]
    int64_t T;
    int N, C, R;
    int tiles_per_group, groups, v_transposed;
    int passes;                          // the rank is covered 16*NB at a time; see the kernel
    int64_t n_blocks;                    // strips * groups
};

__device__ __forceinline__ s16x4 pick_column(const u32x4 (&xv)[4], int u8) {
    // element u8 (0..7) of the four rows a lane holds in chunk form, as one MFMA operand
    const uint32_t sel = (u8 & 1) ? 0x07060302u : 0x05040100u;
    const int d = u8 >> 1;
    auto dw = [&](const u32x4& r) { return d == 0 ? r.x : (d == 1 ? r.y : (d == 2 ? r.z : r.w)); };
    const u32x2 pk = {__builtin_amdgcn_perm(dw(xv[1]), dw(xv[0]), sel), __builtin_amdgcn_perm(dw(xv[3]), dw(xv[2]), sel)};
    return __builtin_bit_cast(s16x4, pk);
}

template <int QBIT, bool ZP, bool P1, bool P2, int NB, bool MULTI = false>
__global__ __launch_bounds__(kCtThreads) void lora_contract_kernel(const ContractArgs a) {
    static_assert(QBIT == 0 || !P2, "the column contraction reads dense X only");
    __shared__ float red[P1 ? kCtWaves * 16 * kCtTile : 1];
    __shared__ __attribute__((aligned(16))) uint16_t tr[P2 ? kCtWaves : 1][P2 ? 16 * kCtPitch : 8];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    // Workgroups go round-robin over the 8 XCDs, each with its own L2.  A 128-column tile of packed
    // codes is 16*q bytes per row, so 8/q neighbouring tiles share every 128-byte line: the block
    // index is permuted so that those tiles run on one XCD and the line is fetched from HBM once
    // (measured before: 2.1x the algorithmic bytes at q = 4).
    constexpr int kShare = QBIT ? 8 / QBIT : 1;
    int64_t logical = blockIdx.x;
    if constexpr (kShare > 1) {
        const int64_t super = logical / (8 * kShare);
        const int local = (int)(logical % (8 * kShare));
        logical = super * (8 * kShare) + (local % 8) * kShare + local / 8;
    }
    if (logical >= a.n_blocks) return;                          // padding of the permuted grid (uniform)
    const int group = (int)(logical % a.groups);
    const int64_t strip = logical / a.groups;
    const int64_t row_base = strip * kCtStrip + (int64_t)wave * (kCtSteps * 16);
    constexpr int QB = QBIT ? QBIT : 8;
    constexpr float kHalf = (float)(1 << (QB - 1));
    const int row_bytes = a.N * QB / 8;

    // Ranks beyond 16*NB are covered in passes over the workgroup's tiles, 16*NB LoRA rows at a time:
    // every accumulator and operand of the contraction scales with the number of rank blocks held at
    // once (about 100 registers per block), and with more than one block the kernel is down to one wave
    // per SIMD with nothing to hide its loads behind.  A later pass finds the tiles in the cache the
    // first one pulled them through.
    // (MULTI is a template parameter: with the loop bound read from the arguments the one-pass kernel
    // of the usual ranks ran 42 instead of 31 us.)
    const int passes = MULTI ? a.passes : 1;
    const int rows_all = 16 * NB * passes;                    // LoRA rows of a partial plane
    for (int pass = 0; pass < passes; ++pass) {
    const int rb = pass * 16 * NB;
    f32x4 acc2[P2 ? kCtSteps : 1][NB];
    if constexpr (P2) {
#pragma unroll
        for (int st = 0; st < kCtSteps; ++st)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) acc2[st][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    for (int ct = 0; ct < a.tiles_per_group; ++ct) {
        const int col_tile = group * a.tiles_per_group + ct;
        const int c0 = col_tile * kCtTile;
        if (c0 >= a.N) break;                                   // uniform over the workgroup
        const int chunk = col_tile * (kCtTile / 8) + j;
        const bool active = chunk < a.C;

        // V operand of the column contraction: lane (r = 16nb + j, g), columns c0 + 16s + 4g .. +3
        s16x4 vop[P2 ? NB : 1][8];
        if constexpr (P2) {
            if (a.v_transposed) {
                // [N, R] layout: the four columns of an operand are R elements apart; all loads
                // first, packing afterwards, so that they overlap
                // (whole dwords, the wanted half picked afterwards: 16-bit loads into register halves
                // would each wait for the one before)
                uint32_t e[NB][8][4];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const int r = rb + 16 * nb + j;
#pragma unroll
                    for (int s8 = 0; s8 < 8; ++s8) {
                        const int col = c0 + 16 * s8 + 4 * g;
                        const bool ok = r < a.R && col < a.N;
                        const uint16_t* p = a.v + (ok ? (int64_t)col * a.R + (r & ~1) : 0);
#pragma unroll
                        for (int kk = 0; kk < 4; ++kk)
                            e[nb][s8][kk] = ok ? *reinterpret_cast<const uint32_t*>(p + kk * a.R) : 0u;
                    }
                }
                const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;     // high or low halves of two dwords
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int s8 = 0; s8 < 8; ++s8) {
                        const u32x2 w = {__builtin_amdgcn_perm(e[nb][s8][1], e[nb][s8][0], sel),
                                         __builtin_amdgcn_perm(e[nb][s8][3], e[nb][s8][2], sel)};
                        vop[nb][s8] = __builtin_bit_cast(s16x4, w);
                    }
            } else {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const int r = rb + 16 * nb + j;
#pragma unroll
                    for (int s8 = 0; s8 < 8; ++s8) {
                        const int col = c0 + 16 * s8 + 4 * g;
                        u32x2 w = {0, 0};
                        if (r < a.R && col < a.N) w = ld8(a.v + (int64_t)r * a.N + col);
                        vop[nb][s8] = __builtin_bit_cast(s16x4, w);
                    }
                }
            }
        }
        // per-column constants of the dequantiser
        float sc[8], zz[8];
        PackedSlot<QB> slot(chunk);
        if constexpr (QBIT != 0) {
            u32x4 sv = {0, 0, 0, 0}, zv = {0, 0, 0, 0};
            if (active) sv = ld16(a.s + chunk * 8);
            unpack8(sv, sc);
            if constexpr (ZP) {
                if (active) zv = ld16(a.zp + chunk * 8);
            }
            unpack8(zv, zz);
        }

        f32x4 acc1[P1 ? NB : 1][8];
        if constexpr (P1) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int u8 = 0; u8 < 8; ++u8) acc1[nb][u8] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }

        // every load of the tile is issued before the first MFMA: a wave sees the memory latency once
        u32x4 xv[kCtSteps][4];
        uint32_t uw[P1 ? kCtSteps : 1][NB][4];
        {
#pragma unroll
            for (int st = 0; st < kCtSteps; ++st) {
                const int64_t t0 = row_base + 16 * st;
                // chunk form of the tile
#pragma unroll
                for (int vv = 0; vv < 4; ++vv) {
                    const int64_t t = t0 + 4 * g + vv;
                    xv[st][vv] = u32x4{0, 0, 0, 0};
                    if (active && t < a.T) {
                        if constexpr (QBIT == 0) {
                            xv[st][vv] = ld16(a.x + t * a.N + chunk * 8);
                        } else {
                            const u32x2 w = ld8(a.q + t * row_bytes + slot.offset);
                            xv[st][vv].x = w.x;
                            xv[st][vv].y = w.y;
                        }
                    }
                }
                // U operand: lane (r = 16nb + j, g), rows t0 + 4g .. +3 (whole dwords, see above)
#pragma unroll
                for (int nb = 0; nb < (P1 ? NB : 0); ++nb) {
                    const int r = rb + 16 * nb + j;
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        const int64_t t = t0 + 4 * g + kk;
                        const bool ok = r < a.R && t < a.T;
                        uw[st][nb][kk] = ok ? *reinterpret_cast<const uint32_t*>(a.u + t * a.R + (r & ~1)) : 0u;
                    }
                }
            }
        }
#pragma unroll
        for (int st = 0; st < kCtSteps; ++st) {
            if constexpr (P1) {
                if constexpr (QBIT != 0) {
#pragma unroll
                    for (int vv = 0; vv < 4; ++vv) {
                        const bool live = active && row_base + 16 * st + 4 * g + vv < a.T;
                        float c[8], f[8];
                        slot.decode(u32x2{xv[st][vv].x, xv[st][vv].y}, c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            if constexpr (ZP) f[e] = rbf((c[e] - kHalf) - zz[e]) * sc[e];
                            else f[e] = (c[e] - kHalf) * sc[e];
                        }
                        xv[st][vv] = live ? pack8(f) : u32x4{0, 0, 0, 0};
                    }
                }
                s16x4 uop[NB];
                const uint32_t usel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const u32x2 pk = {__builtin_amdgcn_perm(uw[st][nb][1], uw[st][nb][0], usel),
                                      __builtin_amdgcn_perm(uw[st][nb][3], uw[st][nb][2], usel)};
                    uop[nb] = __builtin_bit_cast(s16x4, pk);
                }
#pragma unroll
                for (int u8 = 0; u8 < 8; ++u8) {
                    const s16x4 xop = pick_column(xv[st], u8);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        acc1[nb][u8] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(uop[nb], xop, acc1[nb][u8], 0, 0, 0);
                }
            }
            if constexpr (P2) {
                // row form of the tile (lane (i = j, g): row i, columns 16s + 4g .. +3) through this
                // wave's corner of LDS: read straight from memory it would be 16 rows x 32 bytes per
                // load instruction
                uint16_t* tw = tr[wave];
#pragma unroll
                for (int vv = 0; vv < 4; ++vv) *reinterpret_cast<u32x4*>(tw + (4 * g + vv) * kCtPitch + 8 * j) = xv[st][vv];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int s8 = 0; s8 < 8; ++s8) {
                    const u32x2 w = *reinterpret_cast<const u32x2*>(tw + j * kCtPitch + 16 * s8 + 4 * g);
                    const s16x4 xop = __builtin_bit_cast(s16x4, w);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        acc2[st][nb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(xop, vop[nb][s8], acc2[st][nb], 0, 0, 0);
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }

        if constexpr (P1) {
            // add the four waves' tiles in wave order and hand the strip's partial to memory
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                __syncthreads();
#pragma unroll
                for (int u8 = 0; u8 < 8; ++u8) {
                    const f32x4 v4 = acc1[nb][u8];
                    const float e[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
                    for (int vv = 0; vv < 4; ++vv) red[(wave * 16 + 4 * g + vv) * kCtTile + 8 * j + u8] = e[vv];
                }
                __syncthreads();
                // thread tid owns 8 consecutive columns of one LoRA row
                const int tid = threadIdx.x;
                const int r = tid >> 4, cc = (tid & 15) * 8;
                if (c0 + cc < a.N) {
                    float sum[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) sum[e] = red[r * kCtTile + cc + e];
#pragma unroll
                    for (int w = 1; w < kCtWaves; ++w)
#pragma unroll
                        for (int e = 0; e < 8; ++e) sum[e] += red[(w * 16 + r) * kCtTile + cc + e];
                    float* dst = a.part1 + ((strip * rows_all + rb + 16 * nb + r) * (int64_t)a.N + c0 + cc);
                    *reinterpret_cast<f32x4*>(dst) = f32x4{sum[0], sum[1], sum[2], sum[3]};
                    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{sum[4], sum[5], sum[6], sum[7]};
                }
            }
        }
    }

    if constexpr (P2) {
#pragma unroll
        for (int st = 0; st < kCtSteps; ++st)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const f32x4 v4 = acc2[st][nb];
                const float e[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
                for (int vv = 0; vv < 4; ++vv) {
                    const int64_t t = row_base + 16 * st + 4 * g + vv;
                    if (t < a.T) a.part2[((int64_t)group * a.T + t) * rows_all + rb + 16 * nb + j] = e[vv];
                }
            }
    }
    }   // pass
}

// out[i][c] = bf16( sum_k part[k][i][c] ), i < rows_out, c < cols_out, partial planes of
// [rows_part][cols_part] floats; two such reductions per launch (either may be empty).
struct ReduceJob {
    const float* part; uint16_t* out;
    int64_t rows_out, rows_part;
    int cols_out, cols_part, planes;
    int64_t blocks;
    int transposed;          // out is [cols_out][rows_out]: rows_out <= 64 and even, cols_out % 4 == 0
};
constexpr int kReduceTCols = 64;     // columns a block of the transposed form owns (all rows of them)

// out[c][i] = bf16( sum_k part[k][i][c] ): the sums of kReduceTCols columns x all rows meet in LDS and leave as
// one contiguous run of the transposed output.  Planes are added in index order, as in the plain form, so
// the values are the plain form's.
__device__ __forceinline__ void reduce_transposed(const ReduceJob& jb, int64_t blk) {
    __shared__ uint16_t tile[kReduceTCols * 64];
    const int c4 = threadIdx.x & 15, r0 = threadIdx.x >> 4;
    const int64_t c0 = blk * kReduceTCols;
    const int64_t c = c0 + 4 * c4;
    const int rows = (int)jb.rows_out;
    const int64_t plane = jb.rows_part * (int64_t)jb.cols_part;
    if (c < jb.cols_out) {
        for (int r = r0; r < rows; r += 16) {
            const float* p = jb.part + (int64_t)r * jb.cols_part + c;
            f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
            int k = 0;
            for (; k + 4 <= jb.planes; k += 4) {
                f32x4 v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4*>(p + (k + u) * plane);
#pragma unroll
                for (int u = 0; u < 4; ++u) sum += v[u];
            }
            for (; k < jb.planes; ++k) sum += *reinterpret_cast<const f32x4*>(p + k * plane);
            const uint32_t lo = pk_bf16(sum.x, sum.y), hi = pk_bf16(sum.z, sum.w);
            tile[(4 * c4 + 0) * rows + r] = (uint16_t)lo;
            tile[(4 * c4 + 1) * rows + r] = (uint16_t)(lo >> 16);
            tile[(4 * c4 + 2) * rows + r] = (uint16_t)hi;
            tile[(4 * c4 + 3) * rows + r] = (uint16_t)(hi >> 16);
        }
    }
    __syncthreads();
    const int64_t cols_here = jb.cols_out - c0 < kReduceTCols ? jb.cols_out - c0 : kReduceTCols;
    const int n_pairs = (int)(cols_here * rows / 2);
    uint32_t* out = reinterpret_cast<uint32_t*>(jb.out + c0 * rows);
    const uint32_t* src = reinterpret_cast<const uint32_t*>(tile);
    for (int i = threadIdx.x; i < n_pairs; i += 256) out[i] = src[i];
}

// A thread owns W neighbouring outputs of one row (cols_out % W == 0) and reads one W-wide vector
// per plane; planes are added in index order.
template <int W>
__global__ __launch_bounds__(256) void contract_reduce_kernel(const ReduceJob j0, const ReduceJob j1) {
    typedef float fvec __attribute__((ext_vector_type(W)));
    const bool second = (int64_t)blockIdx.x >= j0.blocks;
    const ReduceJob& jb = second ? j1 : j0;
    const int64_t blk = second ? blockIdx.x - j0.blocks : blockIdx.x;
    if (jb.transposed) {                  // the same for every thread of the block
        reduce_transposed(jb, blk);
        return;
    }
    const int64_t n_out = jb.rows_out * jb.cols_out;
    const int64_t idx = (blk * 256 + threadIdx.x) * W;
    if (idx >= n_out) return;
    const int64_t plane = jb.rows_part * (int64_t)jb.cols_part;
    const int64_t i = idx / jb.cols_out;
    const float* p = jb.part + i * jb.cols_part + (idx - i * jb.cols_out);
    float sum[W];
#pragma unroll
    for (int e = 0; e < W; ++e) sum[e] = 0.0f;
    int k = 0;
    for (; k + 4 <= jb.planes; k += 4) {                    // four planes in flight
        fvec v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const fvec*>(p + (k + u) * plane);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < W; ++e) sum[e] += v[u][e];
    }
    for (; k < jb.planes; ++k) {
        const fvec v = *reinterpret_cast<const fvec*>(p + k * plane);
#pragma unroll
        for (int e = 0; e < W; ++e) sum[e] += v[e];
    }
    uint32_t* out = reinterpret_cast<uint32_t*>(jb.out + idx);
#pragma unroll
    for (int e = 0; e < W; e += 2) out[e / 2] = pk_bf16(sum[e], sum[e + 1]);
}

// ------------------------------------------------------------------------------------
template <int QBIT, bool ZP, bool P1, bool P2>
static void contract_launch_nb(ContractArgs a, dim3 grid, int nb, hipStream_t st) {
    // nb = rank blocks of 16.  One or two are held at once; three run as three passes of one, four as
    // two passes of two (measured on [4096, 11008], both products: 101 and 109 us against 120 and 279 us
    // for kernels that held three or four blocks at once and spilled).
    const dim3 block(kCtThreads);
    a.passes = nb <= 2 ? 1 : (nb == 3 ? 3 : 2);
    if (nb == 1) hipLaunchKernelGGL((lora_contract_kernel<QBIT, ZP, P1, P2, 1>), grid, block, 0, st, a);
    else if (nb == 2) hipLaunchKernelGGL((lora_contract_kernel<QBIT, ZP, P1, P2, 2>), grid, block, 0, st, a);
    else if (nb == 3) hipLaunchKernelGGL((lora_contract_kernel<QBIT, ZP, P1, P2, 1, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((lora_contract_kernel<QBIT, ZP, P1, P2, 2, true>), grid, block, 0, st, a);
}

static int64_t contract_geometry(int64_t T, int64_t N, int64_t R, int* tiles_per_group, int* groups, int64_t* strips,
                                 int* nb) {
    const int64_t tiles = cdiv(N, kCtTile);
    *tiles_per_group = (int)cdiv(tiles, g_ct_max_groups.get());
    *groups = (int)cdiv(tiles, *tiles_per_group);
    *strips = cdiv(T, kCtStrip);
    *nb = (int)cdiv(R, 16);
    return 0;
}

int tune_contract(const char* key, int value) {
    if (strcmp(key, "contract_max_groups") == 0) {
        if (value < 1 || value > 65536) return HYC_ERR_ARG;
        g_ct_max_groups.set(value);
        return HYC_OK;
    }
    return 1;
}

}  // namespace hyc

using namespace hyc;

extern "C" int64_t hyc_lora_contract_workspace(int64_t T, int64_t N, int64_t R, int want_p1, int want_p2) {
    if (T <= 0 || N <= 0 || R < 2 || R > 64) return 0;
    int tpg, groups, nb;
    int64_t strips;
    contract_geometry(T, N, R, &tpg, &groups, &strips, &nb);
    int64_t bytes = 0;
    if (want_p1) bytes += strips * 16 * nb * N * 4;
    if (want_p2) bytes += (int64_t)groups * T * 16 * nb * 4;
    return bytes;
}

extern "C" int hyc_lora_contract(const void* x, const void* q, const void* scale, const void* zero_point, int q_bit,
                                 const void* u, const void* v, int v_transposed, void* p1, int p1_transposed, void* p2,
                                 void* workspace, int64_t workspace_bytes, int64_t T, int64_t N, int64_t R,
                                 void* stream) {
    const bool codes = q != nullptr;
    const bool want1 = p1 != nullptr, want2 = p2 != nullptr;
    if (codes && q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (T < 0 || N < 0 || N % 32 != 0 || N > (1 << 28) || T > ((int64_t)1 << 40)) return HYC_ERR_SHAPE;
    if (R < 2 || R > 64 || R % 2 != 0) return HYC_ERR_RANK;
    if (!want1 && !want2) return HYC_ERR_NULL;
    if (codes ? (x != nullptr || !scale || want2) : (x == nullptr)) return HYC_ERR_ARG;
    if ((want1 && !u) || (want2 && !v) || !workspace) return HYC_ERR_NULL;
    if (T * N == 0) return HYC_OK;
    if ((x && !aligned16(x)) || (scale && !aligned16(scale)) || (zero_point && !aligned16(zero_point)) ||
        (q && (reinterpret_cast<uintptr_t>(q) & 7u)) || (v && (reinterpret_cast<uintptr_t>(v) & 7u)) ||
        (reinterpret_cast<uintptr_t>(u) & 3u) || !aligned16(workspace) ||
        (p1 && (reinterpret_cast<uintptr_t>(p1) & 3u)) || (p2 && (reinterpret_cast<uintptr_t>(p2) & 3u)))
        return HYC_ERR_ALIGN;
    if (v && !v_transposed && ((N * 2) % 8 != 0)) return HYC_ERR_ALIGN;
    ContractArgs a{};
    a.x = (const uint16_t*)x; a.q = (const uint8_t*)q; a.s = (const uint16_t*)scale; a.zp = (const uint16_t*)zero_point;
    a.u = (const uint16_t*)u; a.v = (const uint16_t*)v; a.v_transposed = v_transposed;
    a.T = T; a.N = (int)N; a.C = (int)(N / 8); a.R = (int)R;
    int nb;
    int64_t strips;
    contract_geometry(T, N, R, &a.tiles_per_group, &a.groups, &strips, &nb);
    const int64_t bytes1 = want1 ? strips * 16 * nb * N * 4 : 0;
    const int64_t bytes2 = want2 ? (int64_t)a.groups * T * 16 * nb * 4 : 0;
    if (workspace_bytes < bytes1 + bytes2) return HYC_ERR_ARG;
    a.part1 = (float*)workspace;
    a.part2 = (float*)((char*)workspace + bytes1);
    a.n_blocks = strips * a.groups;
    const int64_t pad = codes ? 8 * (8 / q_bit) : 1;            // see the block-index permutation in the kernel
    if (cdiv(a.n_blocks, pad) * pad > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)(cdiv(a.n_blocks, pad) * pad));
    hipStream_t st = (hipStream_t)stream;
    if (codes) {
        const bool zp = zero_point != nullptr;
#define HYC_CT_CODES(QB)                                                                   \
        do {                                                                               \
            if (zp) contract_launch_nb<QB, true, true, false>(a, grid, nb, st);            \
            else contract_launch_nb<QB, false, true, false>(a, grid, nb, st);              \
        } while (0)
        if (q_bit == 8) HYC_CT_CODES(8);
        else if (q_bit == 4) HYC_CT_CODES(4);
        else HYC_CT_CODES(2);
#undef HYC_CT_CODES
    } else if (want1 && want2) {
        contract_launch_nb<0, false, true, true>(a, grid, nb, st);
    } else if (want1) {
        contract_launch_nb<0, false, true, false>(a, grid, nb, st);
    } else {
        contract_launch_nb<0, false, false, true>(a, grid, nb, st);
    }
    if (hipGetLastError() != hipSuccess) return HYC_ERR_LAUNCH;
    ReduceJob j1{}, j2{};
    const int w = (want2 && R % 4 != 0) ? 2 : 4;             // N % 32 == 0; R is even
    if (want1) {
        j1.part = a.part1; j1.out = (uint16_t*)p1; j1.rows_out = R; j1.rows_part = 16 * nb;
        j1.cols_out = (int)N; j1.cols_part = (int)N; j1.planes = (int)strips;
        j1.blocks = cdiv(R * N, 256 * w);
        if (p1_transposed) {
            j1.transposed = 1;
            j1.blocks = cdiv(N, kReduceTCols);
        }
    }
    if (want2) {
        j2.part = a.part2; j2.out = (uint16_t*)p2; j2.rows_out = T; j2.rows_part = T;
        j2.cols_out = (int)R; j2.cols_part = 16 * nb; j2.planes = a.groups;
        j2.blocks = cdiv(T * R, 256 * w);
    }
    if (j1.blocks + j2.blocks > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 rgrid((unsigned)(j1.blocks + j2.blocks));
    if (w == 4) hipLaunchKernelGGL(contract_reduce_kernel<4>, rgrid, dim3(256), 0, st, j1, j2);
    else hipLaunchKernelGGL(contract_reduce_kernel<2>, rgrid, dim3(256), 0, st, j1, j2);
    return check_launch();
}
