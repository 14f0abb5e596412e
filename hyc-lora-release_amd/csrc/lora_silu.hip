// Fused LoRA-SiLU-Hadamard forward and backward for gfx950.
//
//   forward :  q1 = Q(x1; s1), q2 = Q(x2; s2)                      (packed codes, saved for backward)
//              y1 = x1 + bf16(xa1 . b1),  y2 = x2 + bf16(xa2 . b2)   (LoRA up-projection, K = rank)
//              o  = (y1 * bf16(sigmoid(y1))) * y2
//   backward:  x1 = DQ(q1; s1), x2 = DQ(q2; s2), y1, y2, sigma as above,
//              o, grad_gate = (g*y2) * (sigma * (1 + y1*(1 - sigma))), grad_up = g * silu(y1)
//   (operators/triton_fuse_lora_silu_hadamard_forward_kernels.py:104-146,
//    operators/triton_fuse_lora_silu_hadamard_backward_kernels.py:106-149; bf16 after every
//    arithmetic operation, as there.)
//
// Both kernels move 7-9 bytes per element pair and do 64 MFMA flops for it: they are HBM-bound
// and are laid out for the memory system first.  A wave owns a tile of 128 columns and walks
// down a strip of rows 16 at a time; the rank-R contraction runs on the matrix cores in the
// "one lane = one 16-byte chunk" ownership (hyc_lora_tile.hpp).
// The LoRA-B operand registers are built once per wave and reused for the whole strip.
#include <type_traits>

#include "hyc_lora_tile.hpp"

namespace hyc {

constexpr int kFuseThreads = 256;                  // 4 waves
// Both kernels need ~210-250 VGPRs (LoRA-B operands, per-column constants and a 16-row tile of two
// tensors), i.e. two waves per SIMD.  Telling the compiler so makes it schedule for latency hiding
// inside the wave instead of chasing a third wave it cannot get without spilling
// (measured on [4096 x 11008], q=4: 126 -> 93 us forward, 122 -> 99 us backward).
#define HYC_FUSE_KERNEL(DEEP) __global__ __launch_bounds__(kFuseThreads) __attribute__((amdgpu_waves_per_eu(KSTEPS >= DEEP ? 1 : 2, KSTEPS >= DEEP ? 1 : 2)))
constexpr int kFuseWaves = kFuseThreads / kWave;
#ifndef HYC_FWD_DEEP
#define HYC_FWD_DEEP 2
#endif
#ifndef HYC_BWD_DEEP
#define HYC_BWD_DEEP 3
#endif
#ifndef HYC_ROLL_DEEP
#define HYC_ROLL_DEEP 1
#endif
// Cache policy of the packed codes.  At 2 and 4 bits a tile's codes are a quarter / half of a 128-byte line
// and the rest of the line belongs to a neighbouring wave: ordinary stores and loads, so that the pieces
// meet in L2.  At 8 bits a wave writes and reads whole lines that nobody else touches: streaming accesses
// (forward 95.0 -> 91.2 us, backward 117.7 -> 116.4 us on [4096, 14336]).
template <int QBIT> constexpr bool kStreamCodes = QBIT == 8;
// At 2 bits a tile's codes are 32 bytes a row, a quarter of a line, and the four pieces of a line come from the
// four waves of a workgroup at four moments: 29 MB of 2-bit codes cost the forward kernel more time than 59 MB
// of 4-bit codes.  There the waves hand their pieces over through LDS and each line goes to memory whole, from
// one wave (forward 75.9 -> 71.9 us on [4096, 14336]).  At 4 bits (half lines) the same exchange gains 2 us on
// [4096, 14336] and loses 1.4 us on [4096, 11008] - a barrier per tile couples waves that otherwise run
// independently - and is left out.
template <int QBIT> constexpr bool kMergeCodeLines = QBIT == 2;
// Column tiles side by side in a workgroup (its four waves are CT tiles x 4/CT row strips).  The tiles that share
// a line of codes must be together (kColTilesPerGroup: 4 / 2 / 1 at 2 / 4 / 8 bits).  At 8 bits four tiles side
// by side - a workgroup then touches 1 KiB of a row at a time instead of four rows' 256 bytes - are worth
// 8 us forward and 3.6 us backward on [4096, 14336] (91.1 -> 83.0, 110.5 -> 106.9 us) and 2 / 1 us on
// [4096, 11008]; at 4 bits four instead of two change nothing forward and lose 1.8 us backward on [4096, 11008].
template <int QBIT> constexpr int kFuseColTiles = QBIT == 4 ? 2 : 4;
static_assert(kFuseColTiles<2> % kColTilesPerGroup<2> == 0 && kFuseColTiles<4> % kColTilesPerGroup<4> == 0 &&
              kFuseColTiles<8> % kColTilesPerGroup<8> == 0, "tiles that share a code line stay in one workgroup");

// Strip heights (backward, forward; see hyc_set_tuning).  0 = by code width and size: a wave sets up its
// LoRA-B operands and per-column constants once per strip, which in the [N, R] layout of LoRA-B is 16
// scattered 8-byte loads per lane; 96-row strips spread that over six tiles once the tensor is
// large enough to fill the machine with such strips (forward 70 -> 66 us on [4096, 11008]).  At 8 bits
// short strips do better, 32 rows in both directions (forward 68.3 / 70.8 % of the peak on [4096, 11008] /
// [4096, 14336] against 66.6 / 66.9 % at 96 rows, backward 67.1 / 68.7 % against 66.1 / 68.3 % at 16 and 64.0 /
// 64.8 % at 96), and 16 rows on tensors too small to fill the machine ([512, 4096]: 5.7 against 7.3 us).
static Knob g_fuse_rows_per_wave[2]{0, 0};

static int fuse_rows_per_wave(bool fwd, int q_bit, int64_t T, int64_t N) {
    const int set = g_fuse_rows_per_wave[fwd ? 1 : 0].get();
    if (set) return set;
    const bool large = T * N >= ((int64_t)1 << 24);
    if (q_bit == 8) return large ? 32 : 16;
    if (!fwd) return 32;
    return large ? 96 : 32;
}

struct FuseArgs {
    const uint16_t* xa1; const uint16_t* b1; const uint16_t* s1;
    const uint16_t* xa2; const uint16_t* b2; const uint16_t* s2;
    const uint16_t* x1; const uint16_t* x2;     // forward inputs
    uint8_t* q1; uint8_t* q2;                   // packed codes (forward output / backward input)
    const uint16_t* g;                          // backward: upstream gradient
    uint16_t* o; uint16_t* gg; uint16_t* gu;    // outputs: hadamard, grad_gate, grad_up
    int64_t T;                                  // rows
    int N, C, R;                                // columns, chunks per row, LoRA rank
    int rows_per_wave, col_tiles;
    int b_transposed;                           // b1, b2 are [N, R] instead of [R, N]
};

// ------------------------------------------------------------------------------------
template <int QBIT, int KSTEPS, bool FAST>
__device__ __forceinline__ void fuse_fwd_rows(const FuseArgs& a, int64_t row_begin, int64_t row_end, int lane, int chunk,
                                              bool active, const QuantCols<QBIT>& c1, const QuantCols<QBIT>& c2,
                                              const BOperand<KSTEPS>& B1, const BOperand<KSTEPS>& B2) {
    const int g = lane >> 4;
    const int row_bytes = a.N * QBIT / 8;
    const float zero8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    auto load_x = [&](int64_t row0, u32x4 (&xv1)[4], u32x4 (&xv2)[4]) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            xv1[v] = u32x4{0, 0, 0, 0};
            xv2[v] = u32x4{0, 0, 0, 0};
            if (active && t < row_end) {
                xv1[v] = ld16_nt(a.x1 + t * a.N + chunk * 8);
                xv2[v] = ld16_nt(a.x2 + t * a.N + chunk * 8);
            }
        }
    };
    for (int64_t row0 = row_begin; row0 < row_end; row0 += kTileRows) {
        u32x4 xv1[4], xv2[4];
        load_x(row0, xv1, xv2);
        uint32_t L1[4][4], L2[4][4];
        lora_tile_bf16<KSTEPS>(a.xa1, a.R, row0, row_end, lane, B1, L1);
        lora_tile_bf16<KSTEPS>(a.xa2, a.R, row0, row_end, lane, B2, L2);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            const bool live = active && t < row_end;
            float f1[8], f2[8], of[8];
            unpack8(xv1[v], f1);
            unpack8(xv2[v], f2);
            uint32_t lo, hi;
            // rows past the end still take part in the quad exchange; their stores are masked
            const int64_t tq = t < row_end ? t : row_end - 1;
            codes_to_words<QBIT, false, FAST>(f1, c1, zero8, lo, hi);
            store_packed<QBIT, false>(a.q1 + tq * row_bytes, chunk, live, lo, hi);
            codes_to_words<QBIT, false, FAST>(f2, c2, zero8, lo, hi);
            store_packed<QBIT, false>(a.q2 + tq * row_bytes, chunk, live, lo, hi);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float y1 = rbf(f1[j] + lora_elem(L1[v], j));
                y1 = rbf(y1 * rbf(sigmoidf_(y1)));
                const float y2 = rbf(f2[j] + lora_elem(L2[v], j));
                of[j] = y1 * y2;
            }
            if (live) st16_nt(a.o + t * a.N + chunk * 8, pack8(of));
            // keep the rows apart in the instruction schedule: interleaving all four multiplies the
            // live temporaries and costs a whole occupancy step
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Interior strips (every lane inside the tensor, whole 16-row tiles): no predicate guards a memory
// operation, so the compiler can count the outstanding ones exactly, and the strip is walked as a
// rolling prefetch that needs no second set of registers: as soon as a row of the current tile
// has been unpacked, the same registers are requested again for that row of the NEXT tile (the
// LoRA-A operands likewise, right after the matrix instructions that read them).  Every wait is
// then for data requested a whole tile earlier, and the stores of the rows in between stay in
// flight (loads and stores retire through one in-order counter).  The first tile is peeled so
// that the loop is entered in the state its back edge carries; the last one requests nothing.
template <int QBIT, int KSTEPS, bool MERGE = false>
__device__ __forceinline__ void fuse_fwd_rows_full(const FuseArgs& a, int64_t row_begin, int64_t row_end, int lane,
                                                   int chunk, const QuantCols<QBIT>& c1, const QuantCols<QBIT>& c2,
                                                   const BOperand<KSTEPS>& B1, const BOperand<KSTEPS>& B2,
                                                   int wave = 0, uint8_t* stage = nullptr) {
    const int g = lane >> 4, i = lane & 15;
    const int row_bytes = a.N * QBIT / 8;
    // MERGE: the waves of a workgroup that share the 128-byte lines of a row's codes (CT neighbouring column
    // tiles) hand their pieces over through LDS, and every line is written to memory whole, by one wave
    constexpr int CT = kFuseColTiles<QBIT>, RS = kFuseWaves / CT;
    constexpr int kUnit = kTileRows * 128;                    // a unit's 16 rows x one line, per tensor
    constexpr int kBuf = 2 * RS * kUnit;                      // both tensors of all units
    constexpr int BPL = 32 / CT;                              // bytes a lane writes out: 16 rows x 128 B over CT waves
    const int unit = wave / CT, wiu = wave % CT;
    const int loc = packed_store_offset<QBIT>(chunk) & 127;
    const int out_row = (kTileRows / CT) * wiu + (lane * BPL) / 128, out_col = (lane * BPL) % 128;
    const int64_t line0 = (int64_t)((chunk >> 4) / CT) * 128;  // the unit's line inside a packed row
    int buf = 0;
    const float zero8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    u32x4 xv1[4], xv2[4];
    u32x2 A1[KSTEPS], A2[KSTEPS];
    auto request_a = [&](int64_t row0) {
        request_lora_a<KSTEPS>(a.xa1, a.R, row0 + i, g, A1);
        request_lora_a<KSTEPS>(a.xa2, a.R, row0 + i, g, A2);
    };
    auto request_row = [&](int64_t row0, int v) {
        const int64_t off = (row0 + 4 * g + v) * a.N + chunk * 8;
        xv1[v] = ld16_nt(a.x1 + off);
        xv2[v] = ld16_nt(a.x2 + off);
    };
    auto work = [&](int64_t row0, auto ahead_tag) {
        constexpr bool AHEAD = decltype(ahead_tag)::value;
        uint32_t L1[4][4], L2[4][4];
        u32x2 M1[KSTEPS], M2[KSTEPS];
        mask_lora_a<KSTEPS>(a.R, g, A1, M1);
        mask_lora_a<KSTEPS>(a.R, g, A2, M2);
        lora_tile_bf16_regs<KSTEPS>(M1, B1, L1);
        lora_tile_bf16_regs<KSTEPS>(M2, B2, L2);
        if constexpr (AHEAD) request_a(row0 + kTileRows);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t r = row0 + 4 * g + v;
            float f1[8], f2[8], of[8];
            unpack8(xv1[v], f1);
            unpack8(xv2[v], f2);
            if constexpr (AHEAD) request_row(row0 + kTileRows, v);
            uint32_t lo, hi;
            if constexpr (MERGE) {
                uint8_t* s1 = stage + buf * kBuf + unit * kUnit + (4 * g + v) * 128 + loc;
                codes_to_words<QBIT, false, true>(f1, c1, zero8, lo, hi);
                merge_packed<QBIT>(chunk, lo, hi);
                if (packed_store_lane<QBIT>(chunk)) *reinterpret_cast<uint32_t*>(s1) = lo;
                codes_to_words<QBIT, false, true>(f2, c2, zero8, lo, hi);
                merge_packed<QBIT>(chunk, lo, hi);
                if (packed_store_lane<QBIT>(chunk)) *reinterpret_cast<uint32_t*>(s1 + RS * kUnit) = lo;
            } else {
                codes_to_words<QBIT, false, true>(f1, c1, zero8, lo, hi);
                store_packed<QBIT, kStreamCodes<QBIT>>(a.q1 + r * row_bytes, chunk, true, lo, hi);
                codes_to_words<QBIT, false, true>(f2, c2, zero8, lo, hi);
                store_packed<QBIT, kStreamCodes<QBIT>>(a.q2 + r * row_bytes, chunk, true, lo, hi);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float y1 = rbf(f1[j] + lora_elem(L1[v], j));
                y1 = rbf(y1 * rbf(sigmoidf_(y1)));
                const float y2 = rbf(f2[j] + lora_elem(L2[v], j));
                of[j] = y1 * y2;
            }
            st16_nt(a.o + r * a.N + chunk * 8, pack8(of));
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (MERGE) {
            // LDS-only barrier: the rows just requested and the stores above stay in flight
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            const uint8_t* s1 = stage + buf * kBuf + unit * kUnit + out_row * 128 + out_col;
            const int64_t at = (row0 + out_row) * row_bytes + line0 + out_col;
            if constexpr (BPL == 8) {
                const u32x2 w1 = *reinterpret_cast<const u32x2*>(s1), w2 = *reinterpret_cast<const u32x2*>(s1 + RS * kUnit);
                st8(a.q1 + at, w1);
                st8(a.q2 + at, w2);
            } else {
                const u32x4 w1 = *reinterpret_cast<const u32x4*>(s1), w2 = *reinterpret_cast<const u32x4*>(s1 + RS * kUnit);
                st16(a.q1 + at, w1);
                st16(a.q2 + at, w2);
            }
            buf ^= 1;
        }
    };
    request_a(row_begin);
#pragma unroll
    for (int v = 0; v < 4; ++v) request_row(row_begin, v);
    int64_t row0 = row_begin;
    if (row0 + kTileRows < row_end) {
        work(row0, std::true_type{});
        for (row0 += kTileRows; row0 + kTileRows < row_end; row0 += kTileRows) work(row0, std::true_type{});
    }
    work(row0, std::false_type{});
}

template <int QBIT, int KSTEPS>
HYC_FUSE_KERNEL(HYC_FWD_DEEP) void lora_silu_fwd_kernel(const FuseArgs a) {
    constexpr int CT = kFuseColTiles<QBIT>, RS = kFuseWaves / CT;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = (blockIdx.x % a.col_tiles) * CT + wave % CT;     // a.col_tiles counts groups of CT tiles
    const int64_t row_tile = blockIdx.x / a.col_tiles;
    const int chunk = col_tile * (kTileCols / 8) + (lane & 15);
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;

    // the set-up steps are kept apart in the schedule (each has many short-lived temporaries)
    QuantCols<QBIT> c1, c2;
    c1.load(a.s1, col0, active);
    __builtin_amdgcn_sched_barrier(0);
    c2.load(a.s2, col0, active);
    __builtin_amdgcn_sched_barrier(0);
    BOperand<KSTEPS> B1, B2;
    B1.load(a.b1, a.N, a.R, col0, active, lane >> 4, a.b_transposed != 0);
    __builtin_amdgcn_sched_barrier(0);
    B2.load(a.b2, a.N, a.R, col0, active, lane >> 4, a.b_transposed != 0);
    __builtin_amdgcn_sched_barrier(0);

    const int64_t row_begin = (row_tile * RS + wave / CT) * (int64_t)a.rows_per_wave;
    int64_t row_end = row_begin + a.rows_per_wave;
    if (row_end > a.T) row_end = a.T;
    constexpr bool kRoll = KSTEPS == 1 || (HYC_ROLL_DEEP && KSTEPS >= HYC_FWD_DEEP);
    constexpr bool kCanMerge = kRoll && kMergeCodeLines<QBIT>;
    __shared__ __align__(16) uint8_t stage[kCanMerge ? 2 * 2 * RS * kTileRows * 128 : 16];
    const bool slow = __ballot(!(c1.fast && c2.fast)) != 0ull;
    bool merged = false;
    if constexpr (kCanMerge) {
        // every wave of the workgroup votes before any of them leaves: the merged walk has a barrier per tile,
        // so all of them must take it, with strips of the same whole number of tiles
        const bool mine = !slow && (col_tile + 1) * (kTileCols / 8) <= a.C && row_end - row_begin == a.rows_per_wave &&
                          a.rows_per_wave % kTileRows == 0;
        merged = __syncthreads_and(mine) != 0;
    }
    if (row_begin >= row_end) return;
    const bool full = (col_tile + 1) * (kTileCols / 8) <= a.C && (row_end - row_begin) % kTileRows == 0;   // uniform
    if constexpr (kCanMerge) {
        if (merged) {
            fuse_fwd_rows_full<QBIT, KSTEPS, true>(a, row_begin, row_end, lane, chunk, c1, c2, B1, B2, wave, stage);
            return;
        }
    }
    if (slow)
        fuse_fwd_rows<QBIT, KSTEPS, false>(a, row_begin, row_end, lane, chunk, active, c1, c2, B1, B2);
    else if ((KSTEPS == 1 || (HYC_ROLL_DEEP && KSTEPS >= HYC_FWD_DEEP)) && full)                  // deeper ranks have no registers to spare for it
        fuse_fwd_rows_full<QBIT, KSTEPS>(a, row_begin, row_end, lane, chunk, c1, c2, B1, B2);
    else
        fuse_fwd_rows<QBIT, KSTEPS, true>(a, row_begin, row_end, lane, chunk, active, c1, c2, B1, B2);
}

// ------------------------------------------------------------------------------------
template <int QBIT, int KSTEPS>
HYC_FUSE_KERNEL(HYC_BWD_DEEP) void lora_silu_bwd_kernel(const FuseArgs a) {
    constexpr int CT = kFuseColTiles<QBIT>, RS = kFuseWaves / CT;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = (blockIdx.x % a.col_tiles) * CT + wave % CT;
    const int64_t row_tile = blockIdx.x / a.col_tiles;
    const int chunk = col_tile * (kTileCols / 8) + (lane & 15);
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;
    const int g = lane >> 4;
    constexpr float kHalf = (float)(1 << (QBIT - 1));

    // dequantisation is (code - 2^(q-1)) * step rounded to bf16; as code * step + (-2^(q-1) * step) in one
    // fused multiply-add it is the same number (both products and their sum are exact in fp32: at most 8 x 8
    // significant bits) and the code's byte converts with a single instruction
    float s1[8], s2[8], n1[8], n2[8];
    {
        u32x4 v1 = {0, 0, 0, 0}, v2 = {0, 0, 0, 0};
        if (active) { v1 = ld16(a.s1 + col0); v2 = ld16(a.s2 + col0); }
        unpack8(v1, s1);
        unpack8(v2, s2);
#pragma unroll
        for (int j = 0; j < 8; ++j) { n1[j] = -kHalf * s1[j]; n2[j] = -kHalf * s2[j]; }
    }
    BOperand<KSTEPS> B1, B2;
    B1.load(a.b1, a.N, a.R, col0, active, g, a.b_transposed != 0);
    B2.load(a.b2, a.N, a.R, col0, active, g, a.b_transposed != 0);
    const PackedSlot<QBIT> slot(chunk);
    const int row_bytes = a.N * QBIT / 8;

    const int64_t row_begin = (row_tile * RS + wave / CT) * (int64_t)a.rows_per_wave;
    int64_t row_end = row_begin + a.rows_per_wave;
    if (row_end > a.T) row_end = a.T;

    // one row of 8 element pairs: codes + upstream gradient -> hadamard, grad_gate, grad_up
    auto row_math = [&](const float (&cd1)[8], const float (&cd2)[8], const float (&gf)[8], const uint32_t (&La)[4],
                        const uint32_t (&Lb)[4], uint16_t* o_at, uint16_t* gg_at, uint16_t* gu_at) {
        float of[8], gg[8], gu[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // at 2 bits the four values -2s, -s, 0, s are bf16 numbers already
            const float d1 = fmaf(cd1[j], s1[j], n1[j]), d2 = fmaf(cd2[j], s2[j], n2[j]);
            const float x1 = QBIT == 2 ? d1 : rbf(d1);
            const float x2 = QBIT == 2 ? d2 : rbf(d2);
            const float y1 = rbf(x1 + lora_elem(La, j));
            const float y2 = rbf(x2 + lora_elem(Lb, j));
            const float sig = rbf(sigmoidf_(y1));
            const float sil = rbf(y1 * sig);
            of[j] = sil * y2;
            const float gh1 = rbf(gf[j] * y2);
            gu[j] = gf[j] * sil;
            const float dsilu = rbf(sig * rbf(1.0f + rbf(y1 * rbf(1.0f - sig))));
            gg[j] = gh1 * dsilu;
        }
        st16_nt(o_at, pack8(of));
        st16_nt(gg_at, pack8(gg));
        st16_nt(gu_at, pack8(gu));
    };

    // Interior strips at rank 16: the rolling prefetch of fuse_fwd_rows_full - a row's registers
    // are requested again for the next tile as soon as the row has been taken out of them.
    const bool full = (KSTEPS == 1 || (HYC_ROLL_DEEP && KSTEPS >= HYC_BWD_DEEP)) && (col_tile + 1) * (kTileCols / 8) <= a.C && row_begin < row_end &&
                      (row_end - row_begin) % kTileRows == 0 && a.N <= (1 << 24);      // uniform across the wave
    if (full) {
        const int i = lane & 15;
        u32x2 w1[4], w2[4], A1[KSTEPS], A2[KSTEPS];
        u32x4 gv[4];
        // addresses as (wave-uniform row base) + (lane offset that never changes): the row bases are advanced
        // with scalar instructions, one vector add per access is left
        const uint32_t lane_q = (uint32_t)(4 * g * row_bytes + slot.offset);
        const uint32_t lane_x = (uint32_t)(4 * g * a.N + col0) * 2u;
        auto in_row = [](const void* base, int64_t uniform_bytes, uint32_t lane_bytes) {
            return reinterpret_cast<const char*>(base) + uniform_bytes + lane_bytes;
        };
        auto out_row = [](void* base, int64_t uniform_bytes, uint32_t lane_bytes) {
            return reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(base) + uniform_bytes + lane_bytes);
        };
        auto request_a = [&](int64_t row0) {
            request_lora_a<KSTEPS>(a.xa1, a.R, row0 + i, g, A1);
            request_lora_a<KSTEPS>(a.xa2, a.R, row0 + i, g, A2);
        };
        auto request_row = [&](int64_t row0, int v) {
            if constexpr (kStreamCodes<QBIT>) {
                w1[v] = ld8_nt(in_row(a.q1, (row0 + v) * row_bytes, lane_q));
                w2[v] = ld8_nt(in_row(a.q2, (row0 + v) * row_bytes, lane_q));
            } else {
                w1[v] = ld8(in_row(a.q1, (row0 + v) * row_bytes, lane_q));
                w2[v] = ld8(in_row(a.q2, (row0 + v) * row_bytes, lane_q));
            }
            gv[v] = ld16_nt(in_row(a.g, (row0 + v) * a.N * 2, lane_x));
        };
        auto work = [&](int64_t row0, auto ahead_tag) {
            constexpr bool AHEAD = decltype(ahead_tag)::value;
            uint32_t L1[4][4], L2[4][4];
            u32x2 M1[KSTEPS], M2[KSTEPS];
            mask_lora_a<KSTEPS>(a.R, g, A1, M1);
            mask_lora_a<KSTEPS>(a.R, g, A2, M2);
            lora_tile_bf16_regs<KSTEPS>(M1, B1, L1);
            lora_tile_bf16_regs<KSTEPS>(M2, B2, L2);
            if constexpr (AHEAD) request_a(row0 + kTileRows);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float cd1[8], cd2[8], gf[8];
                slot.decode(w1[v], cd1);
                slot.decode(w2[v], cd2);
                unpack8(gv[v], gf);
                if constexpr (AHEAD) request_row(row0 + kTileRows, v);
                const int64_t ub = (row0 + v) * a.N * 2;
                row_math(cd1, cd2, gf, L1[v], L2[v], out_row(a.o, ub, lane_x), out_row(a.gg, ub, lane_x), out_row(a.gu, ub, lane_x));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        request_a(row_begin);
#pragma unroll
        for (int v = 0; v < 4; ++v) request_row(row_begin, v);
        int64_t row0 = row_begin;
        if (row0 + kTileRows < row_end) {
            work(row0, std::true_type{});
            for (row0 += kTileRows; row0 + kTileRows < row_end; row0 += kTileRows) work(row0, std::true_type{});
        }
        work(row0, std::false_type{});
        return;
    }

    for (int64_t row0 = row_begin; row0 < row_end; row0 += kTileRows) {
        u32x2 w1[4], w2[4];
        u32x4 gv[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            w1[v] = u32x2{0, 0};
            w2[v] = u32x2{0, 0};
            gv[v] = u32x4{0, 0, 0, 0};
            if (active && t < row_end) {
                w1[v] = ld8(a.q1 + t * row_bytes + slot.offset);
                w2[v] = ld8(a.q2 + t * row_bytes + slot.offset);
                gv[v] = ld16_nt(a.g + t * a.N + col0);
            }
        }
        uint32_t L1[4][4], L2[4][4];
        lora_tile_bf16<KSTEPS>(a.xa1, a.R, row0, row_end, lane, B1, L1);
        lora_tile_bf16<KSTEPS>(a.xa2, a.R, row0, row_end, lane, B2, L2);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t t = row0 + 4 * g + v;
            if (!(active && t < row_end)) continue;
            float cd1[8], cd2[8], gf[8];
            slot.decode(w1[v], cd1);
            slot.decode(w2[v], cd2);
            unpack8(gv[v], gf);
            row_math(cd1, cd2, gf, L1[v], L2[v], a.o + t * a.N + col0, a.gg + t * a.N + col0, a.gu + t * a.N + col0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// ------------------------------------------------------------------------------------
static int fuse_check(const FuseArgs& a, int64_t T, int64_t N, int64_t R, int q_bit, bool fwd) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (T < 0 || N < 0 || N % 32 != 0 || N > (1 << 28) || T > ((int64_t)1 << 40)) return HYC_ERR_SHAPE;
    if (R < 4 || R > 64 || R % 4 != 0) return HYC_ERR_RANK;
    if (T * N == 0) return HYC_OK;
    const void* need[] = {a.xa1, a.b1, a.s1, a.xa2, a.b2, a.s2, a.q1, a.q2, a.o,
                          fwd ? (const void*)a.x1 : (const void*)a.g, fwd ? (const void*)a.x2 : (const void*)a.gg,
                          fwd ? (const void*)a.o : (const void*)a.gu};
    for (const void* p : need) if (!p) return HYC_ERR_NULL;
    if (a.b_transposed ? ((reinterpret_cast<uintptr_t>(a.b1) | reinterpret_cast<uintptr_t>(a.b2)) & 7u) != 0
                       : !(aligned16(a.b1) && aligned16(a.b2)))
        return HYC_ERR_ALIGN;
    const void* al16[] = {a.s1, a.s2, a.o, fwd ? (const void*)a.x1 : (const void*)a.g,
                          fwd ? (const void*)a.x2 : (const void*)a.gg, fwd ? (const void*)a.o : (const void*)a.gu};
    for (const void* p : al16) if (!aligned16(p)) return HYC_ERR_ALIGN;
    const void* al8[] = {a.xa1, a.xa2, a.q1, a.q2};
    for (const void* p : al8) if (reinterpret_cast<uintptr_t>(p) & 7u) return HYC_ERR_ALIGN;
    return 1;
}

#define HYC_FUSE_LAUNCH_K(KERNEL, QB)                                                                     \
    do {                                                                                                  \
        if (ksteps == 1) hipLaunchKernelGGL((KERNEL<QB, 1>), grid, block, 0, st, a);                      \
        else if (ksteps == 2) hipLaunchKernelGGL((KERNEL<QB, 2>), grid, block, 0, st, a);                 \
        else if (ksteps == 3) hipLaunchKernelGGL((KERNEL<QB, 3>), grid, block, 0, st, a);                 \
        else hipLaunchKernelGGL((KERNEL<QB, 4>), grid, block, 0, st, a);                                  \
    } while (0)
#define HYC_FUSE_LAUNCH(KERNEL)                                  \
    do {                                                         \
        if (q_bit == 8) HYC_FUSE_LAUNCH_K(KERNEL, 8);            \
        else if (q_bit == 4) HYC_FUSE_LAUNCH_K(KERNEL, 4);       \
        else HYC_FUSE_LAUNCH_K(KERNEL, 2);                       \
    } while (0)

static int fuse_launch(FuseArgs& a, int64_t T, int64_t N, int64_t R, int q_bit, bool fwd, void* stream) {
    const int rc = fuse_check(a, T, N, R, q_bit, fwd);
    if (rc <= 0) return rc;
    a.T = T;
    a.N = (int)N;
    a.C = (int)(N / 8);
    a.R = (int)R;
    a.rows_per_wave = fuse_rows_per_wave(fwd, q_bit, T, N);
    const int ct = q_bit == 4 ? kFuseColTiles<4> : kFuseColTiles<8>;      // = kFuseColTiles<2>
    a.col_tiles = (int)cdiv(cdiv(N, kTileCols), ct);           // workgroups along the columns
    const int64_t row_tiles = cdiv(T, (int64_t)(kFuseWaves / ct) * a.rows_per_wave);
    if (row_tiles * a.col_tiles > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)(row_tiles * a.col_tiles)), block(kFuseThreads);
    const int ksteps = (int)cdiv(R, 16);
    hipStream_t st = (hipStream_t)stream;
    if (fwd) HYC_FUSE_LAUNCH(lora_silu_fwd_kernel);
    else HYC_FUSE_LAUNCH(lora_silu_bwd_kernel);
    return check_launch();
}

int tune_fuse(const char* key, int value) {
    const bool both = strcmp(key, "fuse_rows_per_wave") == 0;
    const bool fwd = both || strcmp(key, "fuse_fwd_rows_per_wave") == 0;
    const bool bwd = both || strcmp(key, "fuse_bwd_rows_per_wave") == 0;
    if (fwd || bwd) {
        if (value < 0 || value > 65536 || value % kTileRows != 0) return HYC_ERR_ARG;     // 0: by size
        if (bwd) g_fuse_rows_per_wave[0].set(value);
        if (fwd) g_fuse_rows_per_wave[1].set(value);
        return HYC_OK;
    }
    return 1;
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_lora_silu_mul_fwd(const void* xa1, const void* b1, const void* x1, const void* s1,
                                     const void* xa2, const void* b2, const void* x2, const void* s2,
                                     void* q1, void* q2, void* o, int64_t T, int64_t N, int64_t R, int q_bit,
                                     int b_transposed, void* stream) {
    FuseArgs a{};
    a.b_transposed = b_transposed;
    a.xa1 = (const uint16_t*)xa1; a.b1 = (const uint16_t*)b1; a.s1 = (const uint16_t*)s1;
    a.xa2 = (const uint16_t*)xa2; a.b2 = (const uint16_t*)b2; a.s2 = (const uint16_t*)s2;
    a.x1 = (const uint16_t*)x1; a.x2 = (const uint16_t*)x2;
    a.q1 = (uint8_t*)q1; a.q2 = (uint8_t*)q2; a.o = (uint16_t*)o;
    return fuse_launch(a, T, N, R, q_bit, true, stream);
}

extern "C" int hyc_lora_silu_mul_bwd(const void* xa1, const void* b1, const void* q1, const void* s1,
                                     const void* xa2, const void* b2, const void* q2, const void* s2,
                                     const void* grad_o, void* o, void* grad_gate, void* grad_up, int64_t T,
                                     int64_t N, int64_t R, int q_bit, int b_transposed, void* stream) {
    FuseArgs a{};
    a.b_transposed = b_transposed;
    a.xa1 = (const uint16_t*)xa1; a.b1 = (const uint16_t*)b1; a.s1 = (const uint16_t*)s1;
    a.xa2 = (const uint16_t*)xa2; a.b2 = (const uint16_t*)b2; a.s2 = (const uint16_t*)s2;
    a.q1 = (uint8_t*)q1; a.q2 = (uint8_t*)q2;
    a.g = (const uint16_t*)grad_o; a.o = (uint16_t*)o; a.gg = (uint16_t*)grad_gate; a.gu = (uint16_t*)grad_up;
    return fuse_launch(a, T, N, R, q_bit, false, stream);
}
