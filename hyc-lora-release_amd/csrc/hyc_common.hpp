// Device-side helpers shared by the gfx950 kernels: bf16 packing, 128-bit accesses,
// wave64 cross-lane primitives and the error/launch plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/hyclora.h"
#include "hyc_quant_math.h"

namespace hyc {

constexpr int kWave = 64;

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---- bf16 <-> fp32 -----------------------------------------------------------------
__device__ __forceinline__ float bf_lo(uint32_t pk) { return __builtin_bit_cast(float, pk << 16); }
__device__ __forceinline__ float bf_hi(uint32_t pk) { return __builtin_bit_cast(float, pk & 0xffff0000u); }
__device__ __forceinline__ float bf_to_f(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }

// two fp32 -> packed bf16x2 (round to nearest even; v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pk_bf16(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// round an fp32 value to bf16 precision, result kept as fp32: converting the pair (0, x) leaves
// bf16(x) in the high half over a zero low half, which already is the fp32 bit pattern (one
// instruction, no shift back)
__device__ __forceinline__ float rbf(float x) { return __builtin_bit_cast(float, pk_bf16(0.0f, x)); }
__device__ __forceinline__ uint16_t f_to_bf(float x) { return (uint16_t)(pk_bf16(x, 0.0f) & 0xffffu); }

// 8 bf16 held as 4 dwords -> 8 floats
__device__ __forceinline__ void unpack8(const u32x4 v, float (&f)[8]) {
    f[0] = bf_lo(v.x); f[1] = bf_hi(v.x);
    f[2] = bf_lo(v.y); f[3] = bf_hi(v.y);
    f[4] = bf_lo(v.z); f[5] = bf_hi(v.z);
    f[6] = bf_lo(v.w); f[7] = bf_hi(v.w);
}
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 v;
    v.x = pk_bf16(f[0], f[1]); v.y = pk_bf16(f[2], f[3]);
    v.z = pk_bf16(f[4], f[5]); v.w = pk_bf16(f[6], f[7]);
    return v;
}

// ---- 128-bit / 64-bit global accesses ----------------------------------------------
__device__ __forceinline__ u32x4 ld16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void st16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
__device__ __forceinline__ u32x2 ld8(const void* p) { return *reinterpret_cast<const u32x2*>(p); }
__device__ __forceinline__ void st8(void* p, u32x2 v) { *reinterpret_cast<u32x2*>(p) = v; }
// streaming (non-temporal) forms for data that is touched once
__device__ __forceinline__ u32x4 ld16_nt(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st16_nt(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x2 ld8_nt(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
}
__device__ __forceinline__ void st8_nt(void* p, u32x2 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
}
__device__ __forceinline__ void st4_nt(void* p, uint32_t v) {
    __builtin_nontemporal_store(v, reinterpret_cast<uint32_t*>(p));
}

// ---- wave64 cross-lane -------------------------------------------------------------
// DPP quad permutes: lane <- lane ^ 1 and lane <- lane ^ 2 inside each group of 4 lanes.
__device__ __forceinline__ uint32_t quad_xor1(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t quad_xor2(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
// sum of the squares of one 8-element chunk: a fused-multiply-add chain from zero
__device__ __forceinline__ float chunk_sumsq(const float (&f)[8]) {
    float p = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) p = fmaf(f[j], f[j], p);
    return p;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t w = (uint32_t)__shfl_xor((int)v, o, kWave);
        v = v > w ? v : w;
    }
    return v;
}

// Inclusive prefix sum over the 64 lanes with DPP moves only (no LDS traffic): a shift-and-add scan
// inside each row of 16 lanes (lanes without a source add 0), then the last lane of row 0 / 2 is
// added to row 1 / 3, then lane 31 (sum of rows 0-1) to rows 2-3.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);    // row_shr:1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);    // row_shr:2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);    // row_shr:4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);    // row_shr:8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);   // row_bcast:15 -> rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);   // row_bcast:31 -> rows 2, 3
    return v;
}

// logistic function; the callers round the result to bf16, so the 1-ulp hardware
// reciprocal and exponential are ample
__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// ---- host side ----------------------------------------------------------------------
inline int check_launch() {
    return hipGetLastError() == hipSuccess ? HYC_OK : HYC_ERR_LAUNCH;
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__host__ __device__ inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }


// A launch-shape knob behind hyc_set_tuning (a benchmarking aid): an entry point reads it once per launch,
// hyc_set_tuning writes it, both relaxed - a caller on another thread gets the old or the new value for its
// launch, never a torn one.
struct Knob {
    std::atomic<int> v;
    constexpr Knob(int x) : v(x) {}
    int get() const { return v.load(std::memory_order_relaxed); }
    void set(int x) { v.store(x, std::memory_order_relaxed); }
};

// Per-file tuning hooks behind hyc_set_tuning: HYC_OK / HYC_ERR_* if the key belongs to the
// file, 1 if it does not.
int tune_quant(const char* key, int value);
int tune_fuse(const char* key, int value);
int tune_add(const char* key, int value);
int tune_contract(const char* key, int value);
int tune_norm_compress(const char* key, int value);
int tune_stats(const char* key, int value);

}  // namespace hyc
