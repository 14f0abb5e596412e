// The rank-R LoRA up-projection of one 16-row x 128-column tile on the matrix cores, in the
// lane ownership the packed-code format wants.  Shared by the fused LoRA-SiLU kernels and the
// LoRA-add kernels.
//
// The contraction runs as v_mfma_f32_16x16x16_bf16 with the *column slots permuted*: MFMA number
// t (t = 0..7) is fed columns c0 + 8j + t (j = 0..15) of the LoRA-B tile, so that lane l, which
// receives column slot j = l % 16 of every MFMA result, ends up with the 8 consecutive columns
// c0 + 8j .. c0 + 8j + 7 of rows 4*(l/16) .. 4*(l/16)+3: "one lane = one 16-byte chunk", no LDS,
// no transposes, every global access a full 256-byte run per row.
#pragma once

#include "hyc_pack.hpp"

namespace hyc {

constexpr int kTileCols = 128;                     // 16 lanes x 8 columns
constexpr int kTileRows = 16;
// A 128-column tile of packed codes is 16*q bytes per row, i.e. 1/2 (q=4) or 1/4 (q=2) of a
// 128-byte cache line.  Workgroups are spread round-robin over the 8 XCDs, each with its own L2,
// so column tiles that share a line are given to the waves of ONE workgroup: 8/q neighbouring
// column tiles x (q/2) row strips per workgroup.  (With one column tile per workgroup the
// fused backward kernel fetched every code line twice: +45 MB of HBM reads on [4096 x 11008].)
template <int QBIT> constexpr int kColTilesPerGroup = 8 / QBIT;

// LoRA-B operands of one 128-column tile: for each 16-deep K step and each of the 8 MFMAs, the
// 4 bf16 values b[16*ks + 4g + kk][c0 + 8j + t], kk = 0..3, for lane (g = l/16, j = l%16).
// b is either [R, N] row-major or, with `transposed`, [N, R] row-major - the layout nn.Linear
// keeps lora_B.weight in, where the four k of one column are one 8-byte load.
template <int KSTEPS>
struct BOperand {
    s16x4 v[KSTEPS][8];
    __device__ __forceinline__ void load(const uint16_t* b, int N, int R, int col0, bool active, int g,
                                         bool transposed = false) {
        if (transposed) {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const int k = 16 * ks + 4 * g;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    u32x2 r = {0, 0};
                    if (active && k < R) r = ld8(b + (int64_t)(col0 + t) * R + k);
                    v[ks][t] = __builtin_bit_cast(s16x4, r);
                }
            }
            return;
        }
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            uint32_t rows[4][4];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int k = 16 * ks + 4 * g + kk;
                u32x4 r = {0, 0, 0, 0};
                if (active && k < R) r = ld16(b + (int64_t)k * N + col0);
                rows[kk][0] = r.x; rows[kk][1] = r.y; rows[kk][2] = r.z; rows[kk][3] = r.w;
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                uint32_t e[4];
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) e[kk] = (t & 1) ? (rows[kk][t >> 1] >> 16) : (rows[kk][t >> 1] & 0xffffu);
                const u32x2 pk = {e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
                v[ks][t] = __builtin_bit_cast(s16x4, pk);
            }
        }
    }
};

// acc[t][v]: column col0 + t, row row0 + 4g + v
template <int KSTEPS>
__device__ __forceinline__ void lora_tile(const uint16_t* xa, int R, int64_t row0, int64_t T, int lane,
                                          const BOperand<KSTEPS>& B, f32x4 (&acc)[8]) {
    const int i = lane & 15, g = lane >> 4;
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const int k = 16 * ks + 4 * g;
        u32x2 av = {0, 0};
        if (row0 + i < T && k < R) av = ld8(xa + (row0 + i) * R + k);
        const s16x4 A = __builtin_bit_cast(s16x4, av);
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, B.v[ks][t], acc[t], 0, 0, 0);
    }
}

__device__ __forceinline__ float acc_elem(const f32x4& a, int v) {
    return v == 0 ? a.x : (v == 1 ? a.y : (v == 2 ? a.z : a.w));
}

// LoRA term of one 16-row tile, already rounded to bf16 (the reference rounds the dot product
// before adding it): L[v][p] holds columns 2p, 2p+1 of row row0 + 4g + v as packed bf16.
// Rounding here, two values per v_cvt_pk_bf16_f32, also halves the accumulator footprint.
template <int KSTEPS>
__device__ __forceinline__ void lora_tile_bf16(const uint16_t* xa, int R, int64_t row0, int64_t T, int lane,
                                               const BOperand<KSTEPS>& B, uint32_t (&L)[4][4]) {
    f32x4 acc[8];
    lora_tile<KSTEPS>(xa, R, row0, T, lane, B, acc);
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int p = 0; p < 4; ++p) L[v][p] = pk_bf16(acc_elem(acc[2 * p], v), acc_elem(acc[2 * p + 1], v));
}
// The same with the LoRA-A operand already in registers (A[ks] = the four bf16
// xa[row0 + l%16][16*ks + 4*(l/16) .. +3] of lane l), for callers that load a tile ahead of its use.
template <int KSTEPS>
__device__ __forceinline__ void lora_tile_bf16_regs(const u32x2 (&A)[KSTEPS], const BOperand<KSTEPS>& B,
                                                    uint32_t (&L)[4][4]) {
    f32x4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const s16x4 Av = __builtin_bit_cast(s16x4, A[ks]);
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Av, B.v[ks][t], acc[t], 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int p = 0; p < 4; ++p) L[v][p] = pk_bf16(acc_elem(acc[2 * p], v), acc_elem(acc[2 * p + 1], v));
}
// Requests the LoRA-A operand of one tile row (row = row0 + l%16) without touching it.
template <int KSTEPS>
__device__ __forceinline__ void request_lora_a(const uint16_t* xa, int R, int64_t row, int g, u32x2 (&A)[KSTEPS]) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const int k = 16 * ks + 4 * g;
        A[ks] = ld8(xa + row * R + (k < R ? k : 0));         // past the rank: any valid address, see below
    }
}
// Zeroes the operands past the rank (a rank that is not a multiple of 16).  Done when the operand
// is used, not when it is requested: touching the value would wait for the load.
template <int KSTEPS>
__device__ __forceinline__ void mask_lora_a(int R, int g, const u32x2 (&A)[KSTEPS], u32x2 (&M)[KSTEPS]) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const bool ok = 16 * ks + 4 * g < R;
        M[ks] = u32x2{ok ? A[ks].x : 0u, ok ? A[ks].y : 0u};
    }
}

__device__ __forceinline__ float lora_elem(const uint32_t (&Lv)[4], int j) {
    return (j & 1) ? bf_hi(Lv[j >> 1]) : bf_lo(Lv[j >> 1]);
}

}  // namespace hyc
