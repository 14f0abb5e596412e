// Per-channel quantise + sub-byte pack and its inverse for gfx950.
//
// Work decomposition (both directions): a lane owns one 16-byte chunk of a row, i.e. 8
// consecutive channels, and walks down a strip of rows, so the per-channel constants
// (step, its reciprocal, zero point) live in registers for the whole strip.  A wave64
// therefore reads 1 KiB of contiguous bf16 per row with one 128-bit load per lane; a
// workgroup is 4 waves that take neighbouring row strips of the same 512 channels.
//
// Packed layout (fixed by the reference's 32-column tiles,
// operators/compress_function_kernel.py:77-112): in every block of 32 columns, with
// epp = 8/q codes per byte and w = 32/epp, byte j collects columns j + i*w, code i at bit
// q*i.  In chunk terms (4 chunks a = 0..3 per block):
//   q=8  chunk a  -> bytes 8a..8a+7, no sharing;
//   q=4  chunks a and a^2 share bytes 8(a&1)..8(a&1)+7, chunk a in nibble a>>1;
//   q=2  all four chunks share bytes 0..7, chunk a in bit pair a.
// Each lane spreads its 8 codes over a 64-bit word (one code per byte, pre-shifted into
// its sub-byte slot); the sharing lanes then OR their words together with DPP quad
// permutes — no LDS, no bpermute — and each stores a different dword of the result, so
// the wave writes one contiguous run per row.
//
// Cache policy (measured on MI355X, [4096, 11008] bf16): the activation is touched once, so
// its loads (quantise) and stores (dequantise) are non-temporal — that alone is worth ~25 %
// on the dequantiser, whose stores otherwise evict useful lines.  The packed codes are stored
// and loaded with ordinary cache policy: the kernel that reads the codes next waits behind
// non-temporal stores on their way to memory, and neighbouring lanes of the dequantiser read
// the same 8 bytes and rely on the cache to merge those requests.
#include <type_traits>

#include "hyc_pack.hpp"

namespace hyc {

#ifndef HYC_Q_WAVES
#define HYC_Q_WAVES 4
#endif
#ifndef HYC_Q_UNROLL
#define HYC_Q_UNROLL 4
#endif
constexpr int kQuantWaves = HYC_Q_WAVES;      // waves per workgroup
constexpr int kQuantThreads = kQuantWaves * kWave;
#ifndef HYC_QO_WAVES
#define HYC_QO_WAVES 4
#endif
#ifndef HYC_D_UNROLL
#define HYC_D_UNROLL 2
#endif
constexpr int kRowUnroll = HYC_Q_UNROLL;       // quantiser: independent 128-bit loads in flight per lane
constexpr int kDeqUnroll = HYC_D_UNROLL;       // dequantiser: rows per group

static Knob g_quant_rows_per_wave{8};     // strip heights; see hyc_set_tuning
static Knob g_dequant_rows_per_wave{2};
static Knob g_quant_outlier_rows_per_wave{8};     // the same two with an outlier list
static Knob g_dequant_outlier_rows_per_wave{8};

struct QuantArgs {
    uint16_t* x;            // bf16 activations (input of quantise / output of dequantise)
    const uint16_t* scale;  // bf16 [N]
    const uint16_t* zp;     // bf16 [N] or null
    uint8_t* q;             // packed codes, contiguous [T, N*q/8]
    const int64_t* oidx;    // outlier channels or null
    uint16_t* xo;           // bf16 [T, k]
    int64_t T;              // B*M rows
    int64_t stride_b, stride_m, stride_h;
    int M, N, C;            // C = N/8 chunks per row
    int head_dim;
    int k;
    int zero_input;
    int rows_per_wave;
    int col_tiles;
};

// Which of this lane's 8 columns are outlier channels, and at which position of the list.
// The wave scans the list 64 entries at a time; only entries that fall into the wave's
// 512-column window are broadcast and examined.
struct OutlierLane {
    uint32_t mask = 0;        // bit j: column col0 + j is an outlier
    uint32_t pos[4] = {0, 0, 0, 0};  // 16-bit list positions, two per dword
    // dword p of the lane's chunk with its outlier columns cleared: d & keep(p)
    __device__ __forceinline__ uint32_t keep(int p) const {
        const uint32_t two = mask >> (2 * p);
        return ~(((two & 1u) ? 0x0000ffffu : 0u) | ((two & 2u) ? 0xffff0000u : 0u));
    }
};

__device__ __forceinline__ OutlierLane find_outliers(const int64_t* oidx, int k, int wave_col0, int col0, int lane) {
    OutlierLane o;
    for (int base = 0; base < k; base += kWave) {
        const int e = base + lane;
        const int ch = (e < k) ? (int)oidx[e] : -1;
        const bool hit = (unsigned)(ch - wave_col0) < (unsigned)(kWave * 8);
        unsigned long long hits = __ballot(hit);
        while (hits) {
            const int src = __ffsll((long long)hits) - 1;
            hits &= hits - 1;
            const int c = __builtin_amdgcn_readlane(ch, src);
            const int d = c - col0;
            if ((unsigned)d < 8u) {
                o.mask |= 1u << d;
                const uint32_t p = (uint32_t)(base + src) << (16 * (d & 1));
                const uint32_t keep = 0xffff0000u >> (16 * (d & 1));
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    if ((d >> 1) == w) o.pos[w] = (o.pos[w] & keep) | p;
            }
        }
    }
    return o;
}

__device__ __forceinline__ uint32_t outlier_pos(const OutlierLane& o, int j) {
    return (o.pos[j >> 1] >> (16 * (j & 1))) & 0xffffu;
}

// One of four dwords by a run-time index (three selects; the operands stay in registers).
__device__ __forceinline__ uint32_t pick4(uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, int p) {
    const uint32_t lo = (p & 1) ? d1 : d0, hi = (p & 1) ? d3 : d2;
    return (p & 2) ? hi : lo;
}
__device__ __forceinline__ uint32_t outlier_pos_dyn(const OutlierLane& o, int j) {
    return (pick4(o.pos[0], o.pos[1], o.pos[2], o.pos[3], j >> 1) >> (16 * (j & 1))) & 0xffffu;
}

// The quantiser's outlier step.  A lane owns at most one outlier column as a rule, so the first one
// is handled without a branch: its value is picked out of the row's chunk in compute (first_value)
// and stored next to the row's codes, as one more predicated store whose place in the order of
// memory operations is fixed.  Whatever a lane holds beyond that - and all of them when the input
// is to be zeroed in place - goes through extract_rest: a loop over the set bits with stores
// inside, which makes the compiler wait for every outstanding load and store before it, and which
// is deliberately not unrolled (eight predicated copies of the body per row once made this kernel
// sixty thousand instructions long).
struct OutlierFirst {
    int j = 0;            // the lane's lowest outlier column (0 if it has none)
    uint32_t pos = 0;     // its position in the list
    uint32_t rest = 0;    // mask bits beyond it
    OutlierFirst() = default;
    __device__ __forceinline__ explicit OutlierFirst(const OutlierLane& o) {
        if (o.mask) {
            j = __ffs((int)o.mask) - 1;
            pos = outlier_pos_dyn(o, j);
            rest = o.mask & (o.mask - 1);
        }
    }
    __device__ __forceinline__ uint32_t first_value(const u32x4& v) const {
        return (pick4(v.x, v.y, v.z, v.w, j >> 1) >> (16 * (j & 1))) & 0xffffu;
    }
};

__device__ __forceinline__ void extract_rest(const OutlierLane& o, uint32_t bits, const u32x4& v, uint16_t* xo_row,
                                             uint16_t* x_chunk, bool zero_input) {
#pragma clang loop unroll(disable)
    while (bits) {
        const int j = __ffs((int)bits) - 1;
        bits &= bits - 1;
        xo_row[outlier_pos_dyn(o, j)] = (uint16_t)(pick4(v.x, v.y, v.z, v.w, j >> 1) >> (16 * (j & 1)));
        if (zero_input) x_chunk[j] = 0;
    }
}

// Walks the rows t = b*M + m of a [B, M, .] tensor with independent batch and row strides
// without a division per row.
struct RowCursor {
    int64_t off;   // b*stride_b + m*stride_m
    int m;
    __device__ __forceinline__ RowCursor(int64_t t, int M, int64_t stride_b, int64_t stride_m) {
        const int64_t b = t / M;
        m = (int)(t - b * M);
        off = b * stride_b + m * stride_m;
    }
    __device__ __forceinline__ void next(int M, int64_t stride_b, int64_t stride_m) {
        ++m;
        off += stride_m;
        if (m == M) {
            m = 0;
            off += stride_b - (int64_t)M * stride_m;
        }
    }
};

// Element offset of the chunk that starts at column col0 (see hyclora.h: head layout).
__device__ __forceinline__ int64_t chunk_offset(int col0, int head_dim, int64_t stride_h) {
    const int h = col0 / head_dim;
    return (int64_t)h * stride_h + (col0 - h * head_dim);
}

// ------------------------------------------------------------------------------------
// quantise + pack
// ------------------------------------------------------------------------------------
// Loads the lane's chunk of kRowUnroll consecutive rows starting at the cursor (rows at or past
// row1 are skipped) and advances the cursor.
template <bool FULL>
__device__ __forceinline__ void load_rows(const QuantArgs& a, RowCursor& cur, int64_t t0, int64_t row1, bool active,
                                          int64_t coff, u32x4 (&v)[kRowUnroll], int64_t (&roff)[kRowUnroll]) {
#pragma unroll
    for (int u = 0; u < kRowUnroll; ++u) {
        roff[u] = cur.off;                 // element offset of the row (only the outlier step reads it)
        if constexpr (FULL) {
            v[u] = ld16_nt(a.x + cur.off + coff);
        } else {
            v[u] = u32x4{0, 0, 0, 0};
            if (active && t0 + u < row1) v[u] = ld16_nt(a.x + cur.off + coff);
        }
        cur.next(a.M, a.stride_b, a.stride_m);
    }
}

// Order of memory operations inside the strip loop: the loads of the NEXT row group are issued
// before the stores of the current one.  The hardware counts loads and stores with one in-order
// counter (vmcnt), so waiting for loads that were issued after stores also waits for those stores;
// issuing the loads first lets the wave wait for its data while its stores are still in flight.
// The loaded registers are free by then (the codes of the current group are already packed), so
// this costs no extra registers.
//
// FULL = the wave's tile lies completely inside the tensor (all 64 lanes active, the strip is a
// whole number of row groups).  That variant has no predicates or branches around its memory
// operations, which is what lets the compiler count outstanding operations exactly and emit
// s_waitcnt vmcnt(<stores in flight>) instead of vmcnt(0) at the top of the loop.
template <int QBIT, bool ZP, bool OUTL, bool FAST, bool FULL>
__device__ __forceinline__ void quant_rows(const QuantArgs& a, int64_t row0, int64_t row1, bool active, int chunk,
                                           int64_t coff, const QuantCols<QBIT>& qc, const float (&z)[8]) {
    const int row_bytes = a.N * QBIT / 8;
    if (row0 >= row1) return;
    RowCursor cur(row0, a.M, a.stride_b, a.stride_m);
    u32x4 v[kRowUnroll];
    int64_t roff[kRowUnroll];
    load_rows<FULL>(a, cur, row0, row1, active, coff, v, roff);
    // the first rows are already on their way while the wave looks up its outlier columns
    OutlierLane ol;
    if constexpr (OUTL) ol = find_outliers(a.oidx, a.k, (chunk & ~(kWave - 1)) * 8, chunk * 8, chunk & (kWave - 1));
    const OutlierFirst of(ol);
    const bool in_place = OUTL && a.zero_input != 0;
    const uint32_t loop_bits = in_place ? ol.mask : of.rest;     // what extract_rest handles, per lane
    const bool store_first = OUTL && ol.mask != 0 && !in_place;
    uint32_t first[OUTL ? kRowUnroll : 1];
    auto compute = [&](u32x4 (&v)[kRowUnroll], int64_t t0, uint32_t (&lo)[kRowUnroll], uint32_t (&hi)[kRowUnroll]) {
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u) {
            const int64_t t = t0 + u;
            if constexpr (OUTL) {
                first[u] = of.first_value(v[u]);
                asm volatile("" : "+v"(first[u]));     // picked here, not at the store: the row's registers take the next loads
                if (loop_bits && (FULL || (active && t < row1)))
                    extract_rest(ol, loop_bits, v[u], a.xo + t * a.k, a.x + roff[u] + coff, in_place);
                v[u] = u32x4{v[u].x & ol.keep(0), v[u].y & ol.keep(1), v[u].z & ol.keep(2), v[u].w & ol.keep(3)};
            }
            float f[8];
            unpack8(v[u], f);
            codes_to_words<QBIT, ZP, FAST>(f, qc, z, lo[u], hi[u]);
            merge_packed<QBIT>(chunk, lo[u], hi[u]);       // rows past row1 hold zeros; never stored
        }
    };
    auto store = [&](int64_t t0, const uint32_t (&lo)[kRowUnroll], const uint32_t (&hi)[kRowUnroll]) {
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u) {
            const int64_t t = t0 + u;
            store_merged<QBIT, false>(a.q + t * row_bytes, chunk, FULL || (active && t < row1), lo[u], hi[u]);
            if constexpr (OUTL) {
                if (store_first && (FULL || (active && t < row1))) a.xo[t * a.k + of.pos] = (uint16_t)first[u];
            }
        }
    };
    // The first group is peeled so that the loop is always entered with "4 loads, then 4 stores"
    // outstanding, the same state its back edge carries; otherwise the wait at the loop top has
    // to cover the entry case (loads only) and ends up waiting for the stores as well.
    uint32_t lo[kRowUnroll], hi[kRowUnroll];
    int64_t t0 = row0;
    compute(v, t0, lo, hi);
    if (t0 + kRowUnroll < row1) {
        load_rows<FULL>(a, cur, t0 + kRowUnroll, row1, active, coff, v, roff);
        store(t0, lo, hi);
        for (t0 += kRowUnroll; t0 + kRowUnroll < row1; t0 += kRowUnroll) {
            compute(v, t0, lo, hi);
            load_rows<FULL>(a, cur, t0 + kRowUnroll, row1, active, coff, v, roff);
            store(t0, lo, hi);
        }
        compute(v, t0, lo, hi);                                // last group: nothing left to load
    }
    store(t0, lo, hi);
}

template <int QBIT, bool ZP, bool OUTL>
__global__ __launch_bounds__(kQuantThreads) __attribute__((amdgpu_waves_per_eu(OUTL ? HYC_QO_WAVES : 4)))
void quant_pack_kernel(const QuantArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = blockIdx.x % a.col_tiles;
    const int64_t row_tile = blockIdx.x / a.col_tiles;
    const int chunk = col_tile * kWave + lane;
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;

    QuantCols<QBIT> qc;
    qc.load(a.scale, col0, active);
    float z[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = 0.0f;
    if constexpr (ZP) {
        if (active) unpack8(ld16(a.zp + col0), z);
    }
    const int64_t coff = active ? chunk_offset(col0, a.head_dim, a.stride_h) : 0;
    const int64_t row0 = (row_tile * kQuantWaves + wave) * (int64_t)a.rows_per_wave;
    int64_t row1 = row0 + a.rows_per_wave;
    if (row1 > a.T) row1 = a.T;

    const bool full = (col_tile + 1) * kWave <= a.C && row1 - row0 == a.rows_per_wave &&
                      a.rows_per_wave % kRowUnroll == 0;      // uniform across the wave
    // one slow column anywhere in the wave sends the whole wave down the IEEE-division path
    if (ZP || __ballot(!qc.fast) != 0ull)
        quant_rows<QBIT, ZP, OUTL, false, false>(a, row0, row1, active, chunk, coff, qc, z);
    else if (full)
        quant_rows<QBIT, ZP, OUTL, true, true>(a, row0, row1, active, chunk, coff, qc, z);
    else
        quant_rows<QBIT, ZP, OUTL, true, false>(a, row0, row1, active, chunk, coff, qc, z);
}

// ------------------------------------------------------------------------------------
// unpack + dequantise
// ------------------------------------------------------------------------------------
template <int QBIT, bool ZP, bool OUTL>
__global__ __launch_bounds__(kQuantThreads) void unpack_dequant_kernel(const QuantArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col_tile = blockIdx.x % a.col_tiles;
    const int64_t row_tile = blockIdx.x / a.col_tiles;
    const int chunk = col_tile * kWave + lane;
    const bool active = chunk < a.C;
    const int col0 = chunk * 8;
    constexpr float kHalf = (float)(1 << (QBIT - 1));

    float s[8], z[8];
    {
        u32x4 sv = {0, 0, 0, 0};
        if (active) sv = ld16(a.scale + col0);
        unpack8(sv, s);
#pragma unroll
        for (int j = 0; j < 8; ++j) z[j] = 0.0f;
        if constexpr (ZP) {
            if (active) unpack8(ld16(a.zp + col0), z);
        }
    }
    OutlierLane ol;
    OutlierFirst of;

    const int64_t coff = active ? chunk_offset(col0, a.head_dim, a.stride_h) : 0;
    const int64_t row0 = (row_tile * kQuantWaves + wave) * (int64_t)a.rows_per_wave;
    int64_t row1 = row0 + a.rows_per_wave;
    if (row1 > a.T) row1 = a.T;
    const int row_bytes = a.N * QBIT / 8;

    const PackedSlot<QBIT> slot(chunk);

    if (row0 >= row1) return;
    const bool full = (col_tile + 1) * kWave <= a.C && row1 - row0 == a.rows_per_wave &&
                      a.rows_per_wave % kDeqUnroll == 0;      // uniform: no predicate needed anywhere
    auto run = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        RowCursor cur(row0, a.M, a.stride_b, a.stride_m);
        u32x2 w[kDeqUnroll];
        auto load_codes = [&](int64_t t0) {
#pragma unroll
            for (int u = 0; u < kDeqUnroll; ++u) {
                if constexpr (FULL) {
                    w[u] = ld8(a.q + (t0 + u) * row_bytes + slot.offset);
                } else {
                    w[u] = u32x2{0, 0};
                    if (active && t0 + u < row1) w[u] = ld8(a.q + (t0 + u) * row_bytes + slot.offset);
                }
            }
        };
        // The value of a lane's first outlier column travels with the codes of its row, so that the
        // row's store waits for one round of memory latency and not for two.  Further outlier columns
        // of the same lane (rare) are fetched where they are inserted.
        uint32_t ovf[OUTL ? kDeqUnroll : 1];
        auto load_outliers = [&](int64_t t0) {
            if constexpr (OUTL) {
                if (ol.mask) {
#pragma unroll
                    for (int u = 0; u < kDeqUnroll; ++u) {
                        const int64_t t = t0 + u;
                        if (FULL || (active && t < row1)) ovf[u] = a.xo[t * a.k + of.pos];
                    }
                }
            }
        };
        u32x4 o[kDeqUnroll];
        uint16_t* xrow[kDeqUnroll];
        auto compute = [&](int64_t t0) {
#pragma unroll
            for (int u = 0; u < kDeqUnroll; ++u) {
                const int64_t t = t0 + u;
                float c[8], f[8];
                slot.decode(w[u], c);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if constexpr (ZP) {
                        // bf16 arithmetic step by step: (c - 2^(q-1)) is exact, minus z rounds to bf16
                        f[j] = rbf((c[j] - kHalf) - z[j]) * s[j];
                    } else {
                        // not fma(c, s, -2^(q-1) s): that loses the sign of zero and turns an
                        // infinite step into NaN where the reference's product does not
                        f[j] = (c[j] - kHalf) * s[j];
                    }
                }
                o[u] = pack8(f);
                xrow[u] = a.x + cur.off + coff;
                cur.next(a.M, a.stride_b, a.stride_m);
                if constexpr (OUTL) {
                    if (ol.mask && (FULL || (active && t < row1))) {
                        uint32_t d[4] = {o[u].x & ol.keep(0), o[u].y & ol.keep(1), o[u].z & ol.keep(2), o[u].w & ol.keep(3)};
                        auto insert = [&](int j, uint32_t value) {
#pragma unroll
                            for (int p = 0; p < 4; ++p) d[p] |= (j >> 1) == p ? value << (16 * (j & 1)) : 0u;
                        };
                        insert(of.j, ovf[u]);
                        uint32_t bits = of.rest;
#pragma clang loop unroll(disable)
                        while (bits) {
                            const int j = __ffs((int)bits) - 1;
                            bits &= bits - 1;
                            insert(j, a.xo[t * a.k + outlier_pos_dyn(ol, j)]);
                        }
                        o[u] = u32x4{d[0], d[1], d[2], d[3]};
                    }
                }
            }
        };
        auto store = [&](int64_t t0) {
#pragma unroll
            for (int u = 0; u < kDeqUnroll; ++u)
                if (FULL || (active && t0 + u < row1)) st16_nt(xrow[u], o[u]);
        };
        // next group's loads go out before this group's stores (see quant_rows)
        load_codes(row0);
        // the first codes are already on their way while the wave looks up its outlier columns
        if constexpr (OUTL) {
            ol = find_outliers(a.oidx, a.k, col_tile * kWave * 8, col0, lane);
            of = OutlierFirst(ol);
        }
        load_outliers(row0);
        int64_t t0 = row0;
        compute(t0);                              // first group peeled, as in quant_rows
        if (t0 + kDeqUnroll < row1) {
            load_codes(t0 + kDeqUnroll);
            load_outliers(t0 + kDeqUnroll);
            store(t0);
            for (t0 += kDeqUnroll; t0 + kDeqUnroll < row1; t0 += kDeqUnroll) {
                compute(t0);
                load_codes(t0 + kDeqUnroll);
                load_outliers(t0 + kDeqUnroll);
                store(t0);
            }
            compute(t0);
        }
        store(t0);
    };
    if (full) run(std::true_type{});
    else run(std::false_type{});
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
static int check_common(const void* x, const void* scale, const void* q, const int64_t* oidx, int64_t k,
                        const void* xo, int64_t B, int64_t M, int64_t N, int64_t stride_b, int64_t stride_m,
                        int64_t head_dim, int64_t stride_h, int q_bit) {
    if (q_bit != 2 && q_bit != 4 && q_bit != 8) return HYC_ERR_QBIT;
    if (B < 0 || M < 0 || N < 0 || k < 0 || k > 65535) return HYC_ERR_SHAPE;
    if (N % 32 != 0 || N > (1 << 28) || M > INT32_MAX || B * M > (int64_t)1 << 40) return HYC_ERR_SHAPE;
    if (B * M * N == 0) return HYC_OK;
    if (!x || !scale || !q) return HYC_ERR_NULL;
    if (k > 0 && (!oidx || !xo)) return HYC_ERR_NULL;
    if (head_dim <= 0 || head_dim % 8 != 0 || N % head_dim != 0) return HYC_ERR_SHAPE;
    if (!aligned16(x) || !aligned16(scale) || !aligned16(q)) return HYC_ERR_ALIGN;
    if (stride_b % 8 != 0 || stride_m % 8 != 0 || stride_h % 8 != 0) return HYC_ERR_ALIGN;
    return 1;  // proceed
}

static QuantArgs make_args(const void* x, const void* scale, const void* zp, const void* q, const int64_t* oidx,
                           int64_t k, const void* xo, int zero_input, int64_t B, int64_t M, int64_t N,
                           int64_t stride_b, int64_t stride_m, int64_t head_dim, int64_t stride_h,
                           int rows_per_wave) {
    QuantArgs a;
    a.x = (uint16_t*)x;
    a.scale = (const uint16_t*)scale;
    a.zp = (const uint16_t*)zp;
    a.q = (uint8_t*)q;
    a.oidx = oidx;
    a.xo = (uint16_t*)xo;
    a.T = B * M;
    a.stride_b = stride_b;
    a.stride_m = stride_m;
    a.stride_h = stride_h;
    a.M = (int)M;
    a.N = (int)N;
    a.C = (int)(N / 8);
    a.head_dim = (int)head_dim;
    a.k = (int)k;
    a.zero_input = zero_input;
    a.rows_per_wave = rows_per_wave;
    a.col_tiles = (int)cdiv(a.C, kWave);
    return a;
}

#define HYC_LAUNCH_QBIT(KERNEL, QB)                                                                 \
    do {                                                                                            \
        if (zp && k)       hipLaunchKernelGGL((KERNEL<QB, true, true>), grid, block, 0, st, a);    \
        else if (zp)       hipLaunchKernelGGL((KERNEL<QB, true, false>), grid, block, 0, st, a);   \
        else if (k)        hipLaunchKernelGGL((KERNEL<QB, false, true>), grid, block, 0, st, a);   \
        else               hipLaunchKernelGGL((KERNEL<QB, false, false>), grid, block, 0, st, a);  \
    } while (0)

#define HYC_LAUNCH(KERNEL)                                       \
    do {                                                         \
        if (q_bit == 8) HYC_LAUNCH_QBIT(KERNEL, 8);              \
        else if (q_bit == 4) HYC_LAUNCH_QBIT(KERNEL, 4);         \
        else HYC_LAUNCH_QBIT(KERNEL, 2);                         \
    } while (0)

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_quant_pack(const void* x, const void* scale, const void* zero_point, void* q,
                              const int64_t* outlier_idx, int64_t k, void* x_outlier, int zero_input, int64_t B,
                              int64_t M, int64_t N, int64_t stride_b, int64_t stride_m, int64_t head_dim,
                              int64_t stride_h, int q_bit, void* stream) {
    const int rc = check_common(x, scale, q, outlier_idx, k, x_outlier, B, M, N, stride_b, stride_m, head_dim,
                                stride_h, q_bit);
    if (rc <= 0) return rc;
    if (zero_point && !aligned16(zero_point)) return HYC_ERR_ALIGN;
    const void* zp = zero_point;
    QuantArgs a = make_args(x, scale, zp, q, outlier_idx, k, x_outlier, zero_input, B, M, N, stride_b, stride_m,
                            head_dim, stride_h, (outlier_idx && k) ? g_quant_outlier_rows_per_wave.get() : g_quant_rows_per_wave.get());
    const int64_t row_tiles = cdiv(a.T, (int64_t)kQuantWaves * a.rows_per_wave);
    if (row_tiles * a.col_tiles > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)(row_tiles * a.col_tiles)), block(kQuantThreads);
    hipStream_t st = (hipStream_t)stream;
    HYC_LAUNCH(quant_pack_kernel);
    return check_launch();
}

extern "C" int hyc_unpack_dequant(const void* q, const void* scale, const void* zero_point, void* x,
                                  const int64_t* outlier_idx, int64_t k, const void* x_outlier, int64_t B,
                                  int64_t M, int64_t N, int64_t stride_b, int64_t stride_m, int64_t head_dim,
                                  int64_t stride_h, int q_bit, void* stream) {
    const int rc = check_common(x, scale, q, outlier_idx, k, x_outlier, B, M, N, stride_b, stride_m, head_dim,
                                stride_h, q_bit);
    if (rc <= 0) return rc;
    if (zero_point && !aligned16(zero_point)) return HYC_ERR_ALIGN;
    if (!((reinterpret_cast<uintptr_t>(q) & 7u) == 0)) return HYC_ERR_ALIGN;
    const void* zp = zero_point;
    QuantArgs a = make_args(x, scale, zp, q, outlier_idx, k, x_outlier, 0, B, M, N, stride_b, stride_m, head_dim,
                            stride_h, (outlier_idx && k) ? g_dequant_outlier_rows_per_wave.get() : g_dequant_rows_per_wave.get());
    const int64_t row_tiles = cdiv(a.T, (int64_t)kQuantWaves * a.rows_per_wave);
    if (row_tiles * a.col_tiles > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)(row_tiles * a.col_tiles)), block(kQuantThreads);
    hipStream_t st = (hipStream_t)stream;
    HYC_LAUNCH(unpack_dequant_kernel);
    return check_launch();
}

int hyc::tune_quant(const char* key, int value) {
    Knob* const knobs[4] = {&g_quant_rows_per_wave, &g_dequant_rows_per_wave, &g_quant_outlier_rows_per_wave,
                           &g_dequant_outlier_rows_per_wave};
    const char* const names[4] = {"quant_rows_per_wave", "dequant_rows_per_wave", "quant_outlier_rows_per_wave",
                                  "dequant_outlier_rows_per_wave"};
    for (int i = 0; i < 4; ++i) {
        if (strcmp(key, names[i]) != 0) continue;
        if (value < 1 || value > 4096) return HYC_ERR_ARG;
        knobs[i]->set(value);
        return HYC_OK;
    }
    return 1;  // not one of this file's keys
}
