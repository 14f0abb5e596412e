// Lane-level building blocks of the packed-code format, shared by the standalone
// quantise / dequantise kernels and the fused LoRA-SiLU kernels.
//
// A lane owns chunk `chunk` of a row: the 8 consecutive channels 8*chunk .. 8*chunk+7.
// Four neighbouring lanes (a DPP quad) own the four chunks of one 32-column block, which is
// the unit the packed layout is defined on (operators/compress_function_kernel.py:77-112):
//   q=8  chunk a  -> bytes 8a..8a+7 of the block, no sharing;
//   q=4  chunks a and a^2 share bytes 8(a&1)..8(a&1)+7, chunk a in nibble a>>1;
//   q=2  all four chunks share bytes 0..7, chunk a in bit pair a.
#pragma once

#include "hyc_common.hpp"

namespace hyc {

// Per-lane column constants of the quantiser: step, enlarged reciprocal (hyc_recip_nudged),
// and whether every one of the lane's 8 steps may use the reciprocal path.
template <int QBIT>
struct QuantCols {
    float s[8], rn[8];
    bool fast;
    __device__ __forceinline__ void load(const uint16_t* scale, int col0, bool active) {
        u32x4 sv = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};   // 1.0 for idle lanes
        if (active) sv = ld16(scale + col0);
        unpack8(sv, s);
        fast = true;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            rn[j] = __builtin_amdgcn_rcpf(s[j]) * HYC_RECIP_NUDGE;   // within HYC_RECIP_SLACK of hyc_recip_nudged
            fast = fast && hyc_scale_is_fast(s[j]);
        }
    }
};

// Device form of hyc_code_word_fast: the same fused multiply-add, with the clamp done by one
// v_med3_f32.  With a NaN among its operands the instruction returns
// min(min(src0, src1), src2), each min dropping a NaN operand; with the lower bound in src2 a
// NaN therefore comes out as the lower bound (code 0), like the host form.  The operand order
// matters for exactly that case, hence inline assembly instead of the commutative builtin.
template <int QBIT>
__device__ __forceinline__ uint32_t code_word_fast_dev(float x, float rn) {
    const float m = fmaf(x, rn, HYC_MAGIC + (float)(1 << (QBIT - 1)));
    float mc;
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(mc) : "v"(m), "v"(HYC_MAGIC + (float)((1 << QBIT) - 1)), "v"(HYC_MAGIC));
    return __float_as_uint(mc);
}

// low bytes of four dwords -> one dword (byte j from w_j)
__device__ __forceinline__ uint32_t low_bytes(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
    const uint32_t w01 = __builtin_amdgcn_perm(w1, w0, 0x0c0c0400u);   // selector 0-3: bytes of 2nd operand, 4-7: of 1st
    const uint32_t w23 = __builtin_amdgcn_perm(w3, w2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(w23, w01, 0x05040100u);
}

// 8 values -> 8 codes, one per byte of (lo, hi).
template <int QBIT, bool ZP, bool FAST>
__device__ __forceinline__ void codes_to_words(const float (&f)[8], const QuantCols<QBIT>& q, const float (&z)[8],
                                               uint32_t& lo, uint32_t& hi) {
    if constexpr (FAST && !ZP) {
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = code_word_fast_dev<QBIT>(f[j], q.rn[j]);
        lo = low_bytes(w[0], w[1], w[2], w[3]);
        hi = low_bytes(w[4], w[5], w[6], w[7]);
    } else {
        int c[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if constexpr (ZP) {
                // zero-point form: IEEE quotient, then + z, then exact roundf
                c[j] = hyc_code_from_t_exact(f[j] / q.s[j] + z[j], QBIT);
            } else {
                c[j] = hyc_code_from_t(f[j] / q.s[j], QBIT);
            }
        }
        lo = (uint32_t)c[0] | ((uint32_t)c[1] << 8) | ((uint32_t)c[2] << 16) | ((uint32_t)c[3] << 24);
        hi = (uint32_t)c[4] | ((uint32_t)c[5] << 8) | ((uint32_t)c[6] << 16) | ((uint32_t)c[7] << 24);
    }
}

// Merge the quad's code words into packed bytes; on return (lo, hi) hold what this lane stores:
// q=8 both dwords, q=4 and q=2 one dword (returned in lo).  Every lane of the quad must call this
// (the exchange is a DPP quad permute).
template <int QBIT>
__device__ __forceinline__ void merge_packed(int chunk, uint32_t& lo, uint32_t& hi) {
    const int quad = chunk & 3;
    if constexpr (QBIT == 4) {
        const int sub = quad >> 1;
        lo <<= 4 * sub;
        hi <<= 4 * sub;
        lo |= quad_xor2(lo);
        hi |= quad_xor2(hi);
        lo = sub ? hi : lo;
    } else if constexpr (QBIT == 2) {
        lo <<= 2 * quad;
        hi <<= 2 * quad;
        lo |= quad_xor1(lo);
        hi |= quad_xor1(hi);
        lo |= quad_xor2(lo);
        hi |= quad_xor2(hi);
        lo = (quad & 1) ? hi : lo;
    }
}

// Byte offset inside a packed row of what merge_packed left in this lane, and whether this
// lane stores at all (at q=2 only two lanes of the quad do).
template <int QBIT>
__device__ __forceinline__ int packed_store_offset(int chunk) {
    const int quad = chunk & 3, blk = chunk >> 2;
    if constexpr (QBIT == 8) return chunk * 8;
    else if constexpr (QBIT == 4) return blk * 16 + 8 * (quad & 1) + 4 * (quad >> 1);
    else return blk * 8 + 4 * (quad & 1);
}
template <int QBIT>
__device__ __forceinline__ bool packed_store_lane(int chunk) { return QBIT != 2 || (chunk & 3) < 2; }

template <int QBIT, bool NT = false>
__device__ __forceinline__ void store_merged(uint8_t* qrow, int chunk, bool active, uint32_t lo, uint32_t hi) {
    if (!(active && packed_store_lane<QBIT>(chunk))) return;
    uint8_t* p = qrow + packed_store_offset<QBIT>(chunk);
    if constexpr (QBIT == 8) {
        if constexpr (NT) st8_nt(p, u32x2{lo, hi});
        else st8(p, u32x2{lo, hi});
    } else {
        if constexpr (NT) st4_nt(p, lo);
        else *reinterpret_cast<uint32_t*>(p) = lo;
    }
}

// merge + store in one step
template <int QBIT, bool NT = false>
__device__ __forceinline__ void store_packed(uint8_t* qrow, int chunk, bool active, uint32_t lo, uint32_t hi) {
    merge_packed<QBIT>(chunk, lo, hi);
    store_merged<QBIT, NT>(qrow, chunk, active, lo, hi);
}

// Where a chunk's codes sit inside a packed row: the 8 bytes at `offset`, each shifted
// right by `shift` and masked with `mask` (replicated per byte).
template <int QBIT>
struct PackedSlot {
    int offset;
    int shift;
    static constexpr uint32_t mask = QBIT == 8 ? 0xffffffffu : (QBIT == 4 ? 0x0f0f0f0fu : 0x03030303u);
    __device__ __forceinline__ explicit PackedSlot(int chunk) {
        const int quad = chunk & 3, blk = chunk >> 2;
        if constexpr (QBIT == 8) { offset = chunk * 8; shift = 0; }
        else if constexpr (QBIT == 4) { offset = blk * 16 + 8 * (quad & 1); shift = 4 * (quad >> 1); }
        else { offset = blk * 8; shift = 2 * quad; }
    }
    // the 8 codes of the chunk as floats
    __device__ __forceinline__ void decode(u32x2 w, float (&c)[8]) const {
        uint32_t lo = (w.x >> shift) & mask, hi = (w.y >> shift) & mask;
        if constexpr (QBIT != 8) {
            // the masked words are made opaque: a code is then one byte-to-float conversion of them; left to
            // itself the compiler extracts every code from the packed word with a bit-field instruction first
            asm("" : "+v"(lo));
            asm("" : "+v"(hi));
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) c[j] = (float)(((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xffu);
    }
};

}  // namespace hyc
