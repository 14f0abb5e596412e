// LoRA add around the compressed copy of a projection's frozen part, for gfx950.
//
//   plain    :  y = bf16(x + bf16(xa . b))  [ then y = bf16(residual + y) ]   (x may be y: in place)
//   quantise :  q = pack(code(x; s [, z])),  y as above    - x is read once for both
//   restore  :  x = DQ(q; s [, z]),          y as above    - the dense x never reaches memory
//
// The reference does each of these in three to four passes over [T, N]: the LoRA product
// written out, the quantiser (or dequantiser), and the add
// (models/utils/compute_utils.py:21-24 with fused_llama_layer_intra_inter_full_fuse.py:128-140
// in forward, :416-417, :439-441, :447-449 in backward; compute_utils.py:34-35 for the same add
// on the input gradient).  Here the rank-R product is an MFMA tile held in registers
// (hyc_lora_tile.hpp) and each kernel moves its algorithmic bytes once: 4, 4 + q/8 and
// 2 + q/8 bytes per element.
//
// For q and k the sum is rotated next (rope_forward, operators/rope_kernels.py:36-109; in the
// layers fused_llama_layer_intra_inter_full_fuse.py:151-152 and again after the rebuild in
// backward, :444, :452).  With head_dim 128 a column tile is exactly one head: the two halves of
// a head sit 8 lanes apart in the 16-lane row group, one DPP row rotate away, so the quantise and
// restore forms can apply the rotation before the store (same arithmetic as rope.hip).
#include <type_traits>

#include "hyc_lora_tile.hpp"

namespace hyc {

constexpr int kAddThreads = 256;
constexpr int kAddWaves = kAddThreads / kWave;
constexpr int kAddPlainColTiles = 4;        // column tiles side by side in a workgroup of the plain add
static Knob g_add_rows_per_wave[3]{0, 48, 48};   // plain (0 = chosen per shape), quantise, restore; see hyc_set_tuning

enum { kAddPlain = 0, kAddQuant = 1, kAddRestore = 2 };

struct LoraAddArgs {
    const uint16_t* xa; const uint16_t* b;
    const uint16_t* s; const uint16_t* zp;      // steps / zero points bf16 [N] (quantise, restore)
    const uint16_t* x;                          // dense input (plain, quantise)
    const uint16_t* res;                        // optional residual added to the sum (plain)
    const void* cos_t; const void* sin_t;       // optional rotation of the sum (quantise, restore); row s = t % S
    int64_t stride_cos, stride_sin;
    int S, rope_f32;
    uint8_t* q;                                 // packed codes: output of quantise, input of restore
    uint16_t* y;
    int64_t T;
    int N, C, R;
    int rows_per_wave, col_tiles;
    int b_transposed;                           // b is [N, R] instead of [R, N]
};

// lane <- the lane 8 further round its row of 16 (the other half of the head)
__device__ __forceinline__ uint32_t other_half(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128 /* row_ror:8 */, 0xF, 0xF, false);
}

// Rotates the 8 dims a lane holds of row t: y <- y*cos + partner*(+-sin), first half of the head
// (lanes 0-7 of the row group) with -sin, second half with +sin.  yv is the bf16-rounded sum.
// (cv, sv: the lane's 8 cos / sin values of the row, bf16 tables only - loaded with the tile)
template <bool F32>
__device__ __forceinline__ u32x4 rope_chunk(const LoraAddArgs& a, u32x4 yv, int64_t t, int j, u32x4 cv, u32x4 sv) {
    const u32x4 pv = {other_half(yv.x), other_half(yv.y), other_half(yv.z), other_half(yv.w)};
    const float sgn = j < 8 ? -1.0f : 1.0f;
    float y[8], p[8], cf[8], sf[8], o[8];
    unpack8(yv, y);
    unpack8(pv, p);
    if constexpr (F32) {
        const int s = (int)(t % a.S);
        const int c = (j & 7) * 8;
        const float* cp = (const float*)a.cos_t + s * a.stride_cos + c;
        const float* sp = (const float*)a.sin_t + s * a.stride_sin + c;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = y[e] * cp[e] + p[e] * (sp[e] * sgn);
    } else {
        unpack8(cv, cf);
        unpack8(sv, sf);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = rbf(y[e] * cf[e]) + rbf(p[e] * (sf[e] * sgn));
    }
    return pack8(o);
}

template <int QBIT, int KSTEPS, int MODE, bool ZP, bool FAST, bool RES = false, int ROPE = 0>
__device__ __forceinline__ void lora_add_rows(const LoraAddArgs& a, int64_t row_begin, int64_t row_end, int lane,
                                              int chunk, bool active, const QuantCols<QBIT>& qc, const float (&z)[8],
                                              const BOperand<KSTEPS>& B) {
    const int g = lane >> 4;
    const int col0 = chunk * 8;
    const int row_bytes = a.N * QBIT / 8;
    constexpr float kHalf = (float)(1 << (QBIT - 1));
    const PackedSlot<QBIT> slot(chunk);
    for (int64_t row0 = row_begin; row0 < row_end; row0 += kTileRows) {
        u32x4 xv[4], rv[RES ? 4 : 1], cv[ROPE == 1 ? 4 : 1], sv[ROPE == 1 ? 4 : 1];
        u32x2 w[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            xv[v] = u32x4{0, 0, 0, 0};
            w[v] = u32x2{0, 0};
            if constexpr (RES) rv[v] = u32x4{0, 0, 0, 0};
            if (active && t < row_end) {
                if constexpr (MODE == kAddRestore) w[v] = ld8(a.q + t * row_bytes + slot.offset);
                else xv[v] = ld16_nt(a.x + t * a.N + col0);
                if constexpr (RES) rv[v] = ld16_nt(a.res + t * a.N + col0);
            }
            if constexpr (ROPE == 1) {
                // table row of this position with the tile's other loads (rows past the end: the last row's)
                const int sp = (int)((t < row_end ? t : row_end - 1) % a.S);
                const int c = (lane & 7) * 8;
                cv[v] = ld16((const uint16_t*)a.cos_t + sp * a.stride_cos + c);
                sv[v] = ld16((const uint16_t*)a.sin_t + sp * a.stride_sin + c);
            }
        }
        uint32_t L[4][4];
        lora_tile_bf16<KSTEPS>(a.xa, a.R, row0, row_end, lane, B, L);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            const bool live = active && t < row_end;
            float f[8], y[8];
            if constexpr (MODE == kAddRestore) {
                float c[8];
                slot.decode(w[v], c);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if constexpr (ZP) f[j] = rbf(rbf((c[j] - kHalf) - z[j]) * qc.s[j]);
                    else f[j] = rbf((c[j] - kHalf) * qc.s[j]);
                }
            } else {
                unpack8(xv[v], f);
            }
            if constexpr (MODE == kAddQuant) {
                uint32_t lo, hi;
                // rows past the end still take part in the quad exchange; their stores are masked
                const int64_t tq = t < row_end ? t : row_end - 1;
                codes_to_words<QBIT, ZP, FAST>(f, qc, z, lo, hi);
                store_packed<QBIT, false>(a.q + tq * row_bytes, chunk, live, lo, hi);
            }
            if constexpr (RES) {
                float r[8];
                unpack8(rv[v], r);
#pragma unroll
                for (int j = 0; j < 8; ++j) y[j] = r[j] + rbf(f[j] + lora_elem(L[v], j));
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) y[j] = f[j] + lora_elem(L[v], j);
            }
            u32x4 yv = pack8(y);
            if constexpr (ROPE != 0) {
                // every lane of the row group takes part in the exchange; rows past the end hold zeros
                yv = rope_chunk<ROPE == 2>(a, yv, t < row_end ? t : row_end - 1, lane & 15, cv[ROPE == 1 ? v : 0],
                                           sv[ROPE == 1 ? v : 0]);
            }
            if (live) st16_nt(a.y + t * a.N + col0, yv);
        }
    }
}

template <int QBIT, int KSTEPS, int MODE, bool ZP>
__device__ __forceinline__ void lora_add_block(const LoraAddArgs& a, int block) {
    // the plain form shares no code lines, but four column tiles side by side (a workgroup touches 1 KiB of a row at
    // a time) are worth 4 % at N = 4096 and 10 % at N = 14336 (47.5 -> 42.8 us), nothing at N = 11008
    constexpr int CT = MODE == kAddPlain ? kAddPlainColTiles : kColTilesPerGroup<QBIT>, RS = kAddWaves / CT;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = (block % a.col_tiles) * CT + wave % CT;     // a.col_tiles counts groups of CT tiles
    const int64_t row_tile = block / a.col_tiles;
    const int chunk = col_tile * (kTileCols / 8) + (lane & 15);
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;

    QuantCols<QBIT> qc;
    float z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (MODE == kAddQuant) {
        qc.load(a.s, col0, active);
    } else if constexpr (MODE == kAddRestore) {
        u32x4 sv = {0, 0, 0, 0};
        if (active) sv = ld16(a.s + col0);
        unpack8(sv, qc.s);
        qc.fast = false;
    }
    if constexpr (ZP) {
        if (active) unpack8(ld16(a.zp + col0), z);
    }
    BOperand<KSTEPS> B;
    B.load(a.b, a.N, a.R, col0, active, lane >> 4, a.b_transposed != 0);

    const int64_t row_begin = (row_tile * RS + wave / CT) * (int64_t)a.rows_per_wave;
    int64_t row_end = row_begin + a.rows_per_wave;
    if (row_end > a.T) row_end = a.T;
    if (row_begin >= row_end) return;
    bool fast = false;
    if constexpr (MODE == kAddQuant && !ZP) fast = __ballot(!qc.fast) == 0ull;
    if constexpr (MODE != kAddPlain) {
        if (a.cos_t) {                                          // uniform over the grid
            auto run = [&](auto fast_tag) {
                constexpr bool F = decltype(fast_tag)::value;
                if (a.rope_f32) lora_add_rows<QBIT, KSTEPS, MODE, ZP, F, false, 2>(a, row_begin, row_end, lane, chunk, active, qc, z, B);
                else lora_add_rows<QBIT, KSTEPS, MODE, ZP, F, false, 1>(a, row_begin, row_end, lane, chunk, active, qc, z, B);
            };
            if constexpr (MODE == kAddQuant && !ZP) {
                if (fast) { run(std::true_type{}); return; }
            }
            run(std::false_type{});
            return;
        }
    }
    if constexpr (MODE == kAddQuant && !ZP) {
        if (fast) {
            lora_add_rows<QBIT, KSTEPS, MODE, ZP, true>(a, row_begin, row_end, lane, chunk, active, qc, z, B);
            return;
        }
    }
    if constexpr (MODE == kAddPlain) {
        if (a.res) {
            lora_add_rows<QBIT, KSTEPS, MODE, ZP, false, true>(a, row_begin, row_end, lane, chunk, active, qc, z, B);
            return;
        }
    }
    lora_add_rows<QBIT, KSTEPS, MODE, ZP, false>(a, row_begin, row_end, lane, chunk, active, qc, z, B);
}

template <int QBIT, int KSTEPS, int MODE, bool ZP>
__global__ __launch_bounds__(kAddThreads) void lora_add_kernel(const LoraAddArgs a) {
    lora_add_block<QBIT, KSTEPS, MODE, ZP>(a, (int)blockIdx.x);
}

// Several operand sets in one launch (the q, k and v projections of a layer: same rows, rank and code
// width, each its own width, steps, adapter, rotation tables or none): the grid is the members' grids one
// after the other.  A [4096, 4096] or [4096, 1024] operand alone is one short generation of waves - its
// launch is mostly ramp and drain; together the members run like one wide operand.
constexpr int kAddGroupMax = 4;
struct LoraAddGroup {
    LoraAddArgs m[kAddGroupMax];
    int first_block[kAddGroupMax + 1];
    int count;
};

template <int QBIT, int KSTEPS, int MODE, bool ZP>
__global__ __launch_bounds__(kAddThreads) void lora_add_group_kernel(const LoraAddGroup g) {
    int mi = 0;
#pragma unroll
    for (int i = 1; i < kAddGroupMax; ++i)
        if (i < g.count && (int)blockIdx.x >= g.first_block[i]) mi = i;
    lora_add_block<QBIT, KSTEPS, MODE, ZP>(g.m[mi], (int)blockIdx.x - g.first_block[mi]);
}

// ------------------------------------------------------------------------------------
template <int QB, int MODE, bool ZP>
static void add_group_launch_k(const LoraAddGroup& g, dim3 grid, int ksteps, hipStream_t st) {
    const dim3 block(kAddThreads);
    if (ksteps == 1) hipLaunchKernelGGL((lora_add_group_kernel<QB, 1, MODE, ZP>), grid, block, 0, st, g);
    else if (ksteps == 2) hipLaunchKernelGGL((lora_add_group_kernel<QB, 2, MODE, ZP>), grid, block, 0, st, g);
    else if (ksteps == 3) hipLaunchKernelGGL((lora_add_group_kernel<QB, 3, MODE, ZP>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((lora_add_group_kernel<QB, 4, MODE, ZP>), grid, block, 0, st, g);
}

template <int QB, int MODE, bool ZP>
static void add_launch_k(const LoraAddArgs& a, dim3 grid, int ksteps, hipStream_t st) {
    const dim3 block(kAddThreads);
    if (ksteps == 1) hipLaunchKernelGGL((lora_add_kernel<QB, 1, MODE, ZP>), grid, block, 0, st, a);
    else if (ksteps == 2) hipLaunchKernelGGL((lora_add_kernel<QB, 2, MODE, ZP>), grid, block, 0, st, a);
    else if (ksteps == 3) hipLaunchKernelGGL((lora_add_kernel<QB, 3, MODE, ZP>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((lora_add_kernel<QB, 4, MODE, ZP>), grid, block, 0, st, a);
}

// Checks one operand set and fills in its launch shape: 1 = launch `blocks` workgroups, HYC_OK = nothing to do,
// negative = error.
// Strip height of the plain add.  The kernel keeps three waves per SIMD resident (3072 on the 256 compute units):
// a launch of 4096 waves runs as one full generation and a third of one.  Of 32, 48 and 64 rows a wave the height
// whose wave count fills its generations best is taken, 32 unless another is better by a twentieth (measured on
// [4096, N]: N = 4096 14.5 us at 48 rows against 16.1 at 32; N = 5120, 11008, 14336 fastest at 32).
static int plain_rows_per_wave(int64_t T, int col_tiles) {
    constexpr double kResident = 3.0 * 4 * 256;
    int best = 32;
    double best_fill = 0.0;
    for (int rows = 32; rows <= 64; rows += 16) {
        const double waves = (double)kAddWaves * col_tiles * (double)cdiv(T, (int64_t)rows);
        if (rows == 32 && waves <= kResident) return 32;            // everything is resident at once anyway
        const double generations = (double)cdiv((int64_t)waves, (int64_t)kResident);
        const double fill = waves / (generations * kResident);
        if (fill > best_fill * (rows == 32 ? 1.0 : 1.05)) {
            best_fill = fill;
            best = rows;
        }
    }
    return best;
}

template <int MODE>
static int add_prepare(LoraAddArgs& a, int64_t T, int64_t N, int64_t R, int q_bit, int64_t& blocks) {
    blocks = 0;
    if (MODE != kAddPlain && q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (T < 0 || N < 0 || N % 32 != 0 || N > (1 << 28) || T > ((int64_t)1 << 40)) return HYC_ERR_SHAPE;
    if (R < 4 || R > 64 || R % 4 != 0) return HYC_ERR_RANK;
    if (T * N == 0) return HYC_OK;
    if (!a.xa || !a.b || !a.y) return HYC_ERR_NULL;
    if (MODE != kAddRestore && !a.x) return HYC_ERR_NULL;
    if (MODE != kAddPlain && (!a.q || !a.s)) return HYC_ERR_NULL;
    if (a.res && !aligned16(a.res)) return HYC_ERR_ALIGN;
    if (a.cos_t) {
        // the rotation pairs dims 64 apart inside one 128-column tile: heads of 128 dims, whole tiles only
        if (MODE == kAddPlain || !a.sin_t || N % kTileCols != 0 || a.S <= 0) return HYC_ERR_ARG;
        const int talign = a.rope_f32 ? 4 : 8;
        if (!aligned16(a.cos_t) || !aligned16(a.sin_t) || a.stride_cos % talign || a.stride_sin % talign ||
            a.stride_cos < kTileCols / 2 || a.stride_sin < kTileCols / 2)
            return HYC_ERR_ALIGN;
    }
    if (!(a.b_transposed ? (reinterpret_cast<uintptr_t>(a.b) & 7u) == 0 : aligned16(a.b)) || !aligned16(a.y) || (a.x && !aligned16(a.x)) || (a.s && !aligned16(a.s)) ||
        (a.zp && !aligned16(a.zp)))
        return HYC_ERR_ALIGN;
    if ((reinterpret_cast<uintptr_t>(a.xa) & 7u) || (a.q && (reinterpret_cast<uintptr_t>(a.q) & 7u))) return HYC_ERR_ALIGN;
    a.T = T;
    a.N = (int)N;
    a.C = (int)(N / 8);
    a.R = (int)R;
    const int ct = MODE == kAddPlain ? kAddPlainColTiles : 8 / q_bit;
    a.col_tiles = (int)cdiv(cdiv(N, kTileCols), ct);
    a.rows_per_wave = g_add_rows_per_wave[MODE].get();
    if (a.rows_per_wave == 0) a.rows_per_wave = plain_rows_per_wave(T, a.col_tiles);
    const int64_t row_tiles = cdiv(T, (int64_t)(kAddWaves / ct) * a.rows_per_wave);
    if (row_tiles * a.col_tiles > INT32_MAX) return HYC_ERR_SHAPE;
    blocks = row_tiles * a.col_tiles;
    return 1;
}

template <int MODE>
static int add_launch(LoraAddArgs& a, int64_t T, int64_t N, int64_t R, int q_bit, void* stream) {
    int64_t blocks;
    const int rc = add_prepare<MODE>(a, T, N, R, q_bit, blocks);
    if (rc <= 0) return rc;
    const dim3 grid((unsigned)blocks);
    const int ksteps = (int)cdiv(R, 16);
    hipStream_t st = (hipStream_t)stream;
    if constexpr (MODE == kAddPlain) {
        add_launch_k<8, MODE, false>(a, grid, ksteps, st);
    } else {
        const bool zp = a.zp != nullptr;
        if (q_bit == 8) { if (zp) add_launch_k<8, MODE, true>(a, grid, ksteps, st); else add_launch_k<8, MODE, false>(a, grid, ksteps, st); }
        else if (q_bit == 4) { if (zp) add_launch_k<4, MODE, true>(a, grid, ksteps, st); else add_launch_k<4, MODE, false>(a, grid, ksteps, st); }
        else { if (zp) add_launch_k<2, MODE, true>(a, grid, ksteps, st); else add_launch_k<2, MODE, false>(a, grid, ksteps, st); }
    }
    return check_launch();
}

static void member_args(const hyc_lora_add_member& m, LoraAddArgs& a, bool quant) {
    a = LoraAddArgs{};
    a.b_transposed = m.b_transposed;
    a.xa = (const uint16_t*)m.xa; a.b = (const uint16_t*)m.b; a.y = (uint16_t*)m.y;
    if (quant) a.x = (const uint16_t*)m.x;
    a.s = (const uint16_t*)m.scale; a.zp = (const uint16_t*)m.zero_point; a.q = (uint8_t*)m.q;
    a.cos_t = m.cos_t; a.sin_t = m.sin_t; a.rope_f32 = m.table_is_fp32; a.S = (int)m.seq_len;
    a.stride_cos = m.stride_cos; a.stride_sin = m.stride_sin;
}

template <int MODE>
static int add_group_launch(const hyc_lora_add_member* members, int count, int64_t T, int64_t R, int q_bit, void* stream) {
    if (!members) return HYC_ERR_NULL;
    if (count < 1 || count > kAddGroupMax) return HYC_ERR_ARG;
    LoraAddGroup g{};
    int64_t total = 0;
    int n = 0;
    const bool zp = members[0].zero_point != nullptr;
    for (int i = 0; i < count; ++i) {
        const hyc_lora_add_member& m = members[i];
        if ((m.zero_point != nullptr) != zp) return HYC_ERR_ARG;            // one kernel: all with a zero point or none
        if ((m.cos_t != nullptr) != (m.sin_t != nullptr)) return HYC_ERR_NULL;
        if (m.cos_t && (m.seq_len <= 0 || m.seq_len > INT32_MAX)) return HYC_ERR_SHAPE;
        LoraAddArgs a;
        member_args(m, a, MODE == kAddQuant);
        int64_t blocks;
        const int rc = add_prepare<MODE>(a, T, m.N, R, q_bit, blocks);
        if (rc < 0) return rc;
        if (rc == 0) continue;                                              // an empty member
        g.m[n] = a;
        g.first_block[n] = (int)total;
        total += blocks;
        if (total > INT32_MAX) return HYC_ERR_SHAPE;
        ++n;
    }
    if (n == 0) return HYC_OK;
    g.count = n;
    g.first_block[n] = (int)total;
    const dim3 grid((unsigned)total);
    const int ksteps = (int)cdiv(R, 16);
    hipStream_t st = (hipStream_t)stream;
    if (q_bit == 8) { if (zp) add_group_launch_k<8, MODE, true>(g, grid, ksteps, st); else add_group_launch_k<8, MODE, false>(g, grid, ksteps, st); }
    else if (q_bit == 4) { if (zp) add_group_launch_k<4, MODE, true>(g, grid, ksteps, st); else add_group_launch_k<4, MODE, false>(g, grid, ksteps, st); }
    else { if (zp) add_group_launch_k<2, MODE, true>(g, grid, ksteps, st); else add_group_launch_k<2, MODE, false>(g, grid, ksteps, st); }
    return check_launch();
}

// ------------------------------------------------------------------------------------
// Sum of two or three LoRA adds in one pass: y = t_0 (+) t_1 (+) t_2 with t_i = bf16(x_i + bf16(xa_i . b_i)) and
// every (+) a bf16 addition - the bits of the chain hyc_lora_add(x_0), hyc_lora_add(x_1, residual = y),
// hyc_lora_add(x_2, residual = y), which is how the input gradients of projections that share an input (q, k, v;
// gate, up) are accumulated (`grad_x += grad_x_temp`), without writing and re-reading the running sum.  Rank <= 16.
constexpr int kAddSumMax = 3;
struct LoraSumArgs {
    const uint16_t* xa[kAddSumMax]; const uint16_t* b[kAddSumMax]; const uint16_t* x[kAddSumMax];
    int b_transposed[kAddSumMax];
    uint16_t* y;
    int64_t T;
    int N, C, R;
    int rows_per_wave, col_tiles;
};

template <int NSRC>
__global__ __launch_bounds__(kAddThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void lora_add_sum_kernel(const LoraSumArgs a) {
    constexpr int CT = kAddPlainColTiles, RS = kAddWaves / CT;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = ((int)blockIdx.x % a.col_tiles) * CT + wave % CT;
    const int64_t row_tile = (int)blockIdx.x / a.col_tiles;
    const int chunk = col_tile * (kTileCols / 8) + (lane & 15);
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;
    const int g = lane >> 4;
    BOperand<1> B[NSRC];
#pragma unroll
    for (int i = 0; i < NSRC; ++i) B[i].load(a.b[i], a.N, a.R, col0, active, g, a.b_transposed[i] != 0);
    const int64_t row_begin = (row_tile * RS + wave / CT) * (int64_t)a.rows_per_wave;
    int64_t row_end = row_begin + a.rows_per_wave;
    if (row_end > a.T) row_end = a.T;
    for (int64_t row0 = row_begin; row0 < row_end; row0 += kTileRows) {
        u32x4 xv[NSRC][4];
#pragma unroll
        for (int i = 0; i < NSRC; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t t = row0 + 4 * g + v;
                xv[i][v] = u32x4{0, 0, 0, 0};
                if (active && t < row_end) xv[i][v] = ld16_nt(a.x[i] + t * a.N + col0);
            }
        // the running sum is a bf16 value after every step, so it is carried packed (4 registers a row); the
        // terms are kept apart in the instruction schedule, or their temporaries add up to a wave per SIMD less
        u32x4 acc[4];
#pragma unroll
        for (int i = 0; i < NSRC; ++i) {
            uint32_t L[4][4];
            lora_tile_bf16<1>(a.xa[i], a.R, row0, row_end, lane, B[i], L);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float f[8], s[8], y[8];
                unpack8(xv[i][v], f);
                if (i != 0) unpack8(acc[v], s);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float t = f[j] + lora_elem(L[v], j);
                    y[j] = i == 0 ? t : s[j] + rbf(t);
                }
                acc[v] = pack8(y);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            if (active && t < row_end) st16_nt(a.y + t * a.N + col0, acc[v]);
        }
    }
}

int tune_add(const char* key, int value) {
    static const char* keys[3] = {"add_rows_per_wave", "add_quant_rows_per_wave", "add_restore_rows_per_wave"};
    for (int m = 0; m < 3; ++m) {
        if (strcmp(key, keys[m]) == 0) {
            if (value == 0 && m == kAddPlain) {              // back to the per-shape choice
                g_add_rows_per_wave[m].set(0);
                return HYC_OK;
            }
            if (value < kTileRows || value > 65536 || value % kTileRows != 0) return HYC_ERR_ARG;
            g_add_rows_per_wave[m].set(value);
            return HYC_OK;
        }
    }
    return 1;
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_lora_add(const void* xa, const void* b, int b_transposed, const void* x, const void* residual,
                            void* y, int64_t T, int64_t N, int64_t R, void* stream) {
    LoraAddArgs a{};
    a.b_transposed = b_transposed;
    a.xa = (const uint16_t*)xa; a.b = (const uint16_t*)b; a.x = (const uint16_t*)x; a.y = (uint16_t*)y;
    a.res = (const uint16_t*)residual;
    return add_launch<kAddPlain>(a, T, N, R, 8, stream);
}

extern "C" int hyc_lora_add_quant(const void* xa, const void* b, int b_transposed, const void* x, const void* scale,
                                  const void* zero_point, void* q, void* y, int64_t T, int64_t N, int64_t R,
                                  int q_bit, void* stream) {
    LoraAddArgs a{};
    a.b_transposed = b_transposed;
    a.xa = (const uint16_t*)xa; a.b = (const uint16_t*)b; a.x = (const uint16_t*)x; a.y = (uint16_t*)y;
    a.s = (const uint16_t*)scale; a.zp = (const uint16_t*)zero_point; a.q = (uint8_t*)q;
    return add_launch<kAddQuant>(a, T, N, R, q_bit, stream);
}

extern "C" int hyc_lora_add_restore(const void* xa, const void* b, int b_transposed, const void* q,
                                    const void* scale, const void* zero_point, void* y, int64_t T, int64_t N,
                                    int64_t R, int q_bit, void* stream) {
    LoraAddArgs a{};
    a.b_transposed = b_transposed;
    a.xa = (const uint16_t*)xa; a.b = (const uint16_t*)b; a.y = (uint16_t*)y;
    a.s = (const uint16_t*)scale; a.zp = (const uint16_t*)zero_point; a.q = (uint8_t*)const_cast<void*>(q);
    return add_launch<kAddRestore>(a, T, N, R, q_bit, stream);
}

extern "C" int hyc_lora_add_quant_rope(const void* xa, const void* b, int b_transposed, const void* x, const void* scale,
                                       const void* zero_point, void* q, void* y, const void* cos_t, const void* sin_t,
                                       int table_is_fp32, int64_t seq_len, int64_t stride_cos, int64_t stride_sin,
                                       int64_t T, int64_t N, int64_t R, int q_bit, void* stream) {
    if (!cos_t || !sin_t) return HYC_ERR_NULL;
    if (seq_len <= 0 || seq_len > INT32_MAX) return HYC_ERR_SHAPE;
    LoraAddArgs a{};
    a.b_transposed = b_transposed;
    a.xa = (const uint16_t*)xa; a.b = (const uint16_t*)b; a.x = (const uint16_t*)x; a.y = (uint16_t*)y;
    a.s = (const uint16_t*)scale; a.zp = (const uint16_t*)zero_point; a.q = (uint8_t*)q;
    a.cos_t = cos_t; a.sin_t = sin_t; a.rope_f32 = table_is_fp32; a.S = (int)seq_len;
    a.stride_cos = stride_cos; a.stride_sin = stride_sin;
    return add_launch<kAddQuant>(a, T, N, R, q_bit, stream);
}

extern "C" int hyc_lora_add_restore_rope(const void* xa, const void* b, int b_transposed, const void* q,
                                         const void* scale, const void* zero_point, void* y, const void* cos_t,
                                         const void* sin_t, int table_is_fp32, int64_t seq_len, int64_t stride_cos,
                                         int64_t stride_sin, int64_t T, int64_t N, int64_t R, int q_bit,
                                         void* stream) {
    if (!cos_t || !sin_t) return HYC_ERR_NULL;
    if (seq_len <= 0 || seq_len > INT32_MAX) return HYC_ERR_SHAPE;
    LoraAddArgs a{};
    a.b_transposed = b_transposed;
    a.xa = (const uint16_t*)xa; a.b = (const uint16_t*)b; a.y = (uint16_t*)y;
    a.s = (const uint16_t*)scale; a.zp = (const uint16_t*)zero_point; a.q = (uint8_t*)const_cast<void*>(q);
    a.cos_t = cos_t; a.sin_t = sin_t; a.rope_f32 = table_is_fp32; a.S = (int)seq_len;
    a.stride_cos = stride_cos; a.stride_sin = stride_sin;
    return add_launch<kAddRestore>(a, T, N, R, q_bit, stream);
}

extern "C" int hyc_lora_add_quant_group(const hyc_lora_add_member* members, int count, int64_t T, int64_t R, int q_bit,
                                        void* stream) {
    return add_group_launch<kAddQuant>(members, count, T, R, q_bit, stream);
}

extern "C" int hyc_lora_add_restore_group(const hyc_lora_add_member* members, int count, int64_t T, int64_t R,
                                          int q_bit, void* stream) {
    return add_group_launch<kAddRestore>(members, count, T, R, q_bit, stream);
}

extern "C" int hyc_lora_add_sum(const hyc_lora_sum_member* members, int count, void* y, int64_t T, int64_t N, int64_t R,
                                void* stream) {
    if (!members) return HYC_ERR_NULL;
    if (count < 2 || count > kAddSumMax) return HYC_ERR_ARG;
    if (T < 0 || N < 0 || N % 32 != 0 || N > (1 << 28) || T > ((int64_t)1 << 40)) return HYC_ERR_SHAPE;
    if (R < 4 || R > 16 || R % 4 != 0) return HYC_ERR_RANK;
    if (T * N == 0) return HYC_OK;
    if (!y) return HYC_ERR_NULL;
    if (!aligned16(y)) return HYC_ERR_ALIGN;
    LoraSumArgs a{};
    for (int i = 0; i < count; ++i) {
        const hyc_lora_sum_member& m = members[i];
        if (!m.xa || !m.b || !m.x) return HYC_ERR_NULL;
        if (!aligned16(m.x) || (reinterpret_cast<uintptr_t>(m.xa) & 7u) ||
            !(m.b_transposed ? (reinterpret_cast<uintptr_t>(m.b) & 7u) == 0 : aligned16(m.b)))
            return HYC_ERR_ALIGN;
        a.xa[i] = (const uint16_t*)m.xa; a.b[i] = (const uint16_t*)m.b; a.x[i] = (const uint16_t*)m.x;
        a.b_transposed[i] = m.b_transposed;
    }
    a.y = (uint16_t*)y;
    a.T = T;
    a.N = (int)N;
    a.C = (int)(N / 8);
    a.R = (int)R;
    a.rows_per_wave = g_add_rows_per_wave[kAddPlain].get();
    if (a.rows_per_wave == 0) a.rows_per_wave = 32;
    a.col_tiles = (int)cdiv(cdiv(N, kTileCols), kAddPlainColTiles);
    const int64_t row_tiles = cdiv(T, (int64_t)(kAddWaves / kAddPlainColTiles) * a.rows_per_wave);
    if (row_tiles * a.col_tiles > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)(row_tiles * a.col_tiles)), block(kAddThreads);
    if (count == 2) hipLaunchKernelGGL((lora_add_sum_kernel<2>), grid, block, 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL((lora_add_sum_kernel<3>), grid, block, 0, (hipStream_t)stream, a);
    return check_launch();
}
