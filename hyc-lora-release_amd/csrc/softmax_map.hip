// Attention-map compression for gfx950: exact k-th value of a bf16 tensor (the keep
// threshold), ordered compaction of the kept entries to (int64 index, bf16 value) pairs,
// the dense restore, and the softmax backward that consumes the map.
//
// The threshold is an exact order statistic.  A bf16 tensor has at most 65536 distinct
// values, so one pass that histograms the bit patterns followed by a scan of the
// histogram gives the k-th value without sorting or copying the tensor to fp32.
//
// Compaction keeps the ascending index order torch's to_sparse() produces.  The flattened
// tensor is cut into segments of kSeg elements, one per wave: pass 1 counts the kept
// entries of each segment, a single workgroup turns the counts into offsets, pass 2
// writes each segment's entries at its offset (lane-ordered with a wave prefix sum).
// The same offsets let the restore kernel rebuild every segment independently: stage the
// segment in LDS (zeros, then its entries), then stream it out with 128-bit stores.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kHistThreads = 1024;
constexpr int kHistLdsBins = 16384;   // keys 0x8000..0xBFFF: bf16 values in [+0, 2), 64 KiB of counters
constexpr int kSeg = 4096;            // elements per compaction segment (one wave)
constexpr int kSegThreads = 256;      // 4 segments per workgroup
constexpr int kSegSteps = kSeg / (kWave * 8);
#ifndef HYC_SW_WAVES
#define HYC_SW_WAVES 4
#endif
constexpr int kStageEntries = 1024;   // kept entries of a segment that sparse_write gathers in LDS

// Monotonic 16-bit key of a bf16 bit pattern: ascending key = ascending value, NaN last
// (torch.kthvalue orders NaN above everything).
__device__ __forceinline__ uint32_t bf16_key(uint32_t bits) {
    if ((bits & 0x7fffu) > 0x7f80u) return 0xffffu;
    return (bits & 0x8000u) ? (0x7fffu - (bits & 0x7fffu)) : (0x8000u | bits);
}
__device__ __forceinline__ uint32_t key_to_bf16(uint32_t key) {
    if (key == 0xffffu) return 0x7fc0u;
    return (key & 0x8000u) ? (key & 0x7fffu) : (0x8000u | (0x7fffu - key));
}

__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

// ---- histogram of bit patterns ------------------------------------------------------
__device__ __forceinline__ void hist_add(uint32_t bits, uint32_t* lds, uint32_t* hist, uint32_t& zeros) {
    if (bits == 0) { ++zeros; return; }           // +0 is by far the most common value of a masked softmax
    const uint32_t key = bf16_key(bits);
    const uint32_t rel = key - 0x8000u;
    if (rel < (uint32_t)kHistLdsBins) atomicAdd(&lds[rel], 1u);
    else atomicAdd(&hist[key], 1u);
}

__global__ __launch_bounds__(kHistThreads) void hist16_kernel(const uint16_t* __restrict__ a, int64_t n,
                                                              uint32_t* __restrict__ hist) {
    __shared__ uint32_t lds[kHistLdsBins];
    for (int i = threadIdx.x; i < kHistLdsBins; i += kHistThreads) lds[i] = 0;
    __syncthreads();
    uint32_t zeros = 0;
    const int64_t chunks = n / 8;
    for (int64_t c = blockIdx.x * (int64_t)kHistThreads + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * kHistThreads) {
        const u32x4 v = ld16(a + c * 8);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            hist_add(d[j] & 0xffffu, lds, hist, zeros);
            hist_add(d[j] >> 16, lds, hist, zeros);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 7)) hist_add(a[chunks * 8 + threadIdx.x], lds, hist, zeros);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) zeros += (uint32_t)__shfl_xor((int)zeros, o, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && zeros) atomicAdd(&lds[0], zeros);
    __syncthreads();
    for (int i = threadIdx.x; i < kHistLdsBins; i += kHistThreads) {
        const uint32_t v = lds[i];
        if (v) atomicAdd(&hist[0x8000 + i], v);
    }
}

// Single workgroup: the k-th smallest value (1-based) from the histogram.  Wave w takes bins
// 4096w .. 4096w+4095 in sixteen coalesced 1 KiB loads (load i: lane l holds bins 4096w + 256i + 4l .. +3),
// so the bins stay in registers in ascending order by (wave, load, lane, component).  Their running count is
// a lane scan per load, a carry from load to load, and the waves' totals through LDS.
__global__ __launch_bounds__(1024) void hist_select_kernel(const uint32_t* __restrict__ hist, int64_t kth,
                                                           float* __restrict__ thr) {
    __shared__ unsigned long long wave_total[1024 / kWave];
    const int t = threadIdx.x, lane = t & (kWave - 1), wave = t >> 6;
    u32x4 h[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) h[i] = ld16(hist + wave * 4096 + i * 256 + lane * 4);
    // (the bins hold 32-bit counts of a tensor of fewer than 2^32 elements, so a wave's running count fits 32 bits)
    uint32_t incl[16];                    // count of the wave's bins up to and including this lane's four of load i
    uint32_t carry = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t v = wave_inclusive_scan(h[i].x + h[i].y + h[i].z + h[i].w);
        incl[i] = carry + v;
        carry += (uint32_t)__builtin_amdgcn_readlane((int)v, kWave - 1);
    }
    if (lane == 0) wave_total[wave] = carry;
    __syncthreads();
    unsigned long long before = 0;
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    const unsigned long long k = (unsigned long long)kth;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t c[4] = {h[i].x, h[i].y, h[i].z, h[i].w};
        const unsigned long long hi = before + incl[i];
        unsigned long long cum = hi - ((unsigned long long)c[0] + c[1] + c[2] + c[3]);
        if (cum < k && k <= hi) {          // true for exactly one (thread, load)
            int bin = 3;
#pragma unroll
            for (int j = 3; j >= 0; --j) {
                unsigned long long upto = cum;
                for (int jj = 0; jj <= j; ++jj) upto += c[jj];
                if (upto >= k) bin = j;
            }
            *thr = __builtin_bit_cast(float, key_to_bf16((uint32_t)(wave * 4096 + i * 256 + lane * 4 + bin)) << 16);
        }
    }
}

// ---- ordered compaction ---------------------------------------------------------------
// kept: a > thr and a != 0 (to_sparse drops exact zeros).  A NaN element is kept too: the reference
// multiplies by the mask before to_sparse, and NaN * 0 is NaN, which is not zero.  The caller
// passes thr already rounded to bf16: torch compares a bf16 tensor with a 0-d fp32
// threshold in bf16.
__device__ __forceinline__ bool keep(uint32_t bits, float thr) {
    const float v = bf_to_f((uint16_t)bits);
    return (v > thr || v != v) && v != 0.0f;
}

// Loads the 8 elements of chunk `c` of the flattened tensor, zero-filling past n.
__device__ __forceinline__ void load_chunk(const uint16_t* a, int64_t c, int64_t n, uint32_t (&e)[8]) {
    const int64_t i0 = c * 8;
    if (i0 + 8 <= n) {
        const u32x4 v = ld16(a + i0);
        e[0] = v.x & 0xffffu; e[1] = v.x >> 16; e[2] = v.y & 0xffffu; e[3] = v.y >> 16;
        e[4] = v.z & 0xffffu; e[5] = v.z >> 16; e[6] = v.w & 0xffffu; e[7] = v.w >> 16;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = (i0 + j < n) ? a[i0 + j] : 0u;
    }
}

// The same chunk as four dwords (element 2p in the low half of dword p).
__device__ __forceinline__ u32x4 load_chunk_packed(const uint16_t* a, int64_t c, int64_t n) {
    const int64_t i0 = c * 8;
    if (i0 + 8 <= n) return ld16(a + i0);
    uint32_t d[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j)
        if (i0 + j < n) d[j >> 1] |= (uint32_t)a[i0 + j] << (16 * (j & 1));
    return u32x4{d[0], d[1], d[2], d[3]};
}
__device__ __forceinline__ uint32_t chunk_elem(const u32x4& v, int j) {
    const uint32_t d = (j >> 1) == 0 ? v.x : ((j >> 1) == 1 ? v.y : ((j >> 1) == 2 ? v.z : v.w));
    return (j & 1) ? d >> 16 : d & 0xffffu;
}

// cmp_mask 0xffff compares the element, 0x7fff its magnitude (|a| > thr).
__global__ __launch_bounds__(kSegThreads) void sparse_count_kernel(const uint16_t* __restrict__ a, int64_t n,
                                                                   const float* __restrict__ thr_p, int64_t nseg,
                                                                   uint32_t* __restrict__ counts, uint32_t cmp_mask) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t seg = blockIdx.x * (int64_t)(kSegThreads / kWave) + (threadIdx.x >> 6);
    if (seg >= nseg) return;
    const float thr = rbf(*thr_p);
    uint32_t cnt = 0;
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {
        const int64_t c = seg * (kSeg / 8) + s * kWave + lane;
        if (c * 8 < n) {
            uint32_t e[8];
            load_chunk(a, c, n, e);
#pragma unroll
            for (int j = 0; j < 8; ++j) cnt += keep(e[j] & cmp_mask, thr) ? 1u : 0u;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt += (uint32_t)__shfl_xor((int)cnt, o, kWave);
    if (lane == 0) counts[seg] = cnt;
}

// offsets[s] = sum of counts[0..s), offsets[nseg] = total.  Workgroup b scans the 1024 counts of
// its own tile (one per thread: wave shuffles plus one LDS step across the 16 waves) and finds
// the sum of everything in front of the tile by itself, adding up counts[0 .. 1024 b) with all its
// threads: redundant reads of a few hundred KB from L2 instead of a second launch or a chain of
// workgroups waiting for each other.  Launch with max(1, ceil(nseg / 1024)) workgroups.
__global__ __launch_bounds__(1024) void seg_scan_kernel(const uint32_t* __restrict__ counts, int64_t nseg,
                                                        int64_t* __restrict__ offsets) {
    __shared__ long long part[16];
    __shared__ uint32_t wave_tot[16];
    const int t = threadIdx.x, lane = t & (kWave - 1), wave = t >> 6;
    const int64_t base = (int64_t)blockIdx.x * 1024;
    long long front = 0;
    int64_t f = t;
    for (; f + 7 * 1024 < base; f += 8 * 1024) {           // eight independent loads in flight
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = counts[f + u * 1024];
#pragma unroll
        for (int u = 0; u < 8; ++u) front += v[u];
    }
    for (; f < base; f += 1024) front += counts[f];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) front += __shfl_xor(front, o, kWave);
    const int64_t i = base + t;
    const uint32_t c = i < nseg ? counts[i] : 0u;
    uint32_t inc = c;                                       // inclusive scan inside the wave
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)inc, o, kWave);
        if (lane >= o) inc += up;
    }
    if (lane == 0) part[wave] = front;
    if (lane == kWave - 1) wave_tot[wave] = inc;
    __syncthreads();
    long long at = 0;
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        at += part[w];
        before += w < wave ? wave_tot[w] : 0u;
        total += wave_tot[w];
    }
    if (i < nseg) offsets[i] = at + before + (inc - c);
    if (t == 0 && base + 1024 >= nseg) offsets[nseg] = at + total;
}

__global__ __launch_bounds__(kSegThreads) __attribute__((amdgpu_waves_per_eu(HYC_SW_WAVES)))
void sparse_write_kernel(const uint16_t* __restrict__ a, int64_t n,
                                                                   const float* __restrict__ thr_p, int64_t nseg,
                                                                   const int64_t* __restrict__ offsets,
                                                                   int64_t* __restrict__ idx_out,
                                                                   uint16_t* __restrict__ val_out, uint32_t cmp_mask,
                                                                   int64_t capacity) {
    // capacity: entries idx_out / val_out have room for.  Entries whose output position lies at or
    // past it are not written (the caller sees from seg_offsets' last element that the list did not
    // fit and writes it again into buffers of the right size).
    __shared__ uint32_t stage[kSegThreads / kWave][kStageEntries];
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t seg = blockIdx.x * (int64_t)(kSegThreads / kWave) + (threadIdx.x >> 6);
    if (seg >= nseg) return;
    const float thr = rbf(*thr_p);
    const int64_t base = offsets[seg];
    if (offsets[seg + 1] == base || base >= capacity) return;     // nothing kept in this segment, or no room left
    // all of the segment's loads are issued before anything depends on them; the chunks stay packed
    // (4 registers each) so that enough waves fit on a SIMD
    u32x4 e[kSegSteps];
    uint32_t mask[kSegSteps], inc[kSegSteps];
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {
        const int64_t c = seg * (kSeg / 8) + s * kWave + lane;
        e[s] = u32x4{0, 0, 0, 0};
        if (c * 8 < n) e[s] = load_chunk_packed(a, c, n);
    }
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {
        mask[s] = 0;                                  // elements past n were loaded as zeros and are never kept
#pragma unroll
        for (int j = 0; j < 8; ++j) mask[s] |= keep(chunk_elem(e[s], j) & cmp_mask, thr) ? (1u << j) : 0u;
    }
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {            // independent inclusive prefixes over the lanes
        inc[s] = wave_inclusive_scan(__popc(mask[s]));
    }
    uint32_t before[kSegSteps], total = 0;            // kept entries in the steps in front
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {
        before[s] = total;
        total += (uint32_t)__shfl((int)inc[s], kWave - 1, kWave);
    }
    if (total <= kStageEntries) {
        // usual case (a few percent kept): gather the wave's entries in LDS in output order, then
        // write them with contiguous stores - one 512-byte run of indices per instruction instead
        // of a handful of scattered 8-byte stores
        uint32_t* st = stage[threadIdx.x >> 6];
#pragma unroll
        for (int s = 0; s < kSegSteps; ++s) {
            uint32_t w = before[s] + (inc[s] - __popc(mask[s]));
            const uint32_t rel = (uint32_t)(s * kWave + lane) * 8;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (mask[s] & (1u << j)) st[w++] = ((rel + j) << 16) | chunk_elem(e[s], j);
            }
        }
        __builtin_amdgcn_wave_barrier();               // LDS writes of this wave are visible to its lanes
        const int64_t first = seg * (int64_t)kSeg;
        const uint32_t room = capacity - base < (int64_t)total ? (uint32_t)(capacity - base) : total;
        for (uint32_t k = lane; k < room; k += kWave) {
            const uint32_t v = st[k];
            idx_out[base + k] = first + (v >> 16);
            val_out[base + k] = (uint16_t)v;
        }
        return;
    }
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) {             // dense segment: store straight from registers
        const int64_t c = seg * (kSeg / 8) + s * kWave + lane;
        int64_t w = base + before[s] + (inc[s] - __popc(mask[s]));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (mask[s] & (1u << j)) {
                if (w < capacity) {
                    idx_out[w] = c * 8 + j;
                    val_out[w] = (uint16_t)chunk_elem(e[s], j);
                }
                ++w;
            }
        }
    }
}

// Segment offsets of an existing ascending index list: offsets[s] = first entry whose
// index is >= s*kSeg.  Entry e fills the offsets of all segments that begin between its
// predecessor's segment and its own.
__global__ void seg_offsets_kernel(const int64_t* __restrict__ idx, int64_t nnz, int64_t nseg,
                                   int64_t* __restrict__ offsets) {
    const int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (e > nnz) return;
    const int64_t prev = e == 0 ? -1 : idx[e - 1] / kSeg;
    int64_t cur = e == nnz ? nseg : idx[e] / kSeg;
    if (cur > nseg) cur = nseg;
    for (int64_t s = prev + 1; s <= cur; ++s) offsets[s] = e;
}

// ---- dense restore ----------------------------------------------------------------------
__global__ __launch_bounds__(kSegThreads) void sparse_restore_kernel(const int64_t* __restrict__ idx,
                                                                     const uint16_t* __restrict__ val,
                                                                     const int64_t* __restrict__ offsets,
                                                                     int64_t nseg, int64_t n,
                                                                     uint16_t* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) uint16_t stage[kSegThreads / kWave][kSeg];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t seg = blockIdx.x * (int64_t)(kSegThreads / kWave) + wave;
    const bool live = seg < nseg;
    u32x4* st = reinterpret_cast<u32x4*>(stage[wave]);
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) st[s * kWave + lane] = u32x4{0, 0, 0, 0};
    __syncthreads();
    if (live) {
        const int64_t e0 = offsets[seg], e1 = offsets[seg + 1];
        const int64_t first = seg * kSeg;
        for (int64_t e = e0 + lane; e < e1; e += kWave) {
            const int64_t rel = idx[e] - first;
            if (rel >= 0 && rel < kSeg) stage[wave][rel] = val[e];
        }
    }
    __syncthreads();
    if (live) {
#pragma unroll
        for (int s = 0; s < kSegSteps; ++s) {
            const int64_t i0 = seg * kSeg + (int64_t)(s * kWave + lane) * 8;
            if (i0 + 8 <= n) {
                st16_nt(out + i0, st[s * kWave + lane]);
            } else {
                for (int j = 0; j < 8 && i0 + j < n; ++j) out[i0 + j] = stage[wave][(s * kWave + lane) * 8 + j];
            }
        }
    }
}

// ---- scaled, masked softmax forward (+ kept-entry count) ------------------------------------
// a = bf16(softmax_fp32(t)),  t = bf16(bf16(s * scale) + mask)   (the mask term only if given):
// the three torch passes "matmul / sqrt(d)", "+ attention_mask", "softmax(dtype=bf16)"
// (models/llama/fused_llama_layer_intra_inter_full_fuse.py:159-167) in one read and one write.
// One wave per row, the row held in registers (CH chunks of 8 per lane).  Row r uses mask row
// (r / rows_per_batch) * mask_stride_b + (r % mask_rows) * mask_stride_row.
// COUNT = 1: a wave walks the 4096/n rows of one compaction segment and also leaves the number of
// entries the compaction will keep (a > threshold, a != 0) in counts[segment], which saves
// hyc_sparse_count's pass over the map.
// COUNT = 2: the same for row lengths that do not divide a segment (n <= 4096, a multiple of 8): a
// wave's rows (at most 4096 elements) lie in at most two segments, a chunk of 8 never straddles
// one, and the wave adds its two counts to counts[] with integer atomics (zeroed by the caller;
// the sums do not depend on the order of the additions).
template <int CH, int COUNT>
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const uint16_t* __restrict__ s, const uint16_t* __restrict__ mask,
                                                          uint16_t* __restrict__ out, int64_t rows, int n, float scale,
                                                          int mask_rows, int64_t rows_per_batch, int64_t mask_stride_b,
                                                          int64_t mask_stride_row, const float* __restrict__ thr_p,
                                                          uint32_t* __restrict__ counts, int rows_per_wave) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t w = blockIdx.x * 4ll + (threadIdx.x >> 6);
    const int64_t row_begin = w * rows_per_wave;
    __shared__ uint32_t wg_counts[COUNT == 2 ? 6 : 1];
    if constexpr (COUNT == 2) {                     // every wave of the workgroup reaches both barriers
        if (threadIdx.x < 6) wg_counts[threadIdx.x] = 0;
        __syncthreads();
    }
    if (COUNT != 2 && row_begin >= rows) return;
    float thr = 0.0f;
    if constexpr (COUNT != 0) thr = rbf(*thr_p);
    uint32_t cnt = 0, cnt_next = 0;
    const int64_t seg_first = (row_begin * n) / kSeg;
    for (int r = 0; r < rows_per_wave; ++r) {
        const int64_t row = row_begin + r;
        if (row >= rows) break;
        const int64_t base = row * n;
        const uint16_t* mrow = nullptr;
        if (mask) mrow = mask + (row / rows_per_batch) * mask_stride_b + (row % mask_rows) * mask_stride_row;
        u32x4 sv[CH], mv[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            sv[c] = u32x4{0, 0, 0, 0};
            mv[c] = u32x4{0, 0, 0, 0};
            if (col < n) {
                sv[c] = ld16_nt(s + base + col);
                if (mrow) mv[c] = ld16(mrow + col);
            }
        }
        float t[CH][8];
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            float mf[8];
            unpack8(sv[c], t[c]);
            unpack8(mv[c], mf);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float v = rbf(t[c][j] * scale);
                if (mrow) v = rbf(v + mf[j]);
                t[c][j] = col < n ? v : -INFINITY;
                mx = fmaxf(mx, t[c][j]);
            }
        }
        mx = wave_max(mx);
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                t[c][j] = __expf(t[c][j] - mx);
                sum += t[c][j];
            }
        sum = wave_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int col = (c * kWave + lane) * 8;
            if (col < n) {
#pragma unroll
                for (int j = 0; j < 8; ++j) t[c][j] *= inv;
                const u32x4 ov = pack8(t[c]);
                st16_nt(out + base + col, ov);
                if constexpr (COUNT != 0) {
                    const uint32_t d[4] = {ov.x, ov.y, ov.z, ov.w};
                    uint32_t c8 = 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j) c8 += keep((d[j >> 1] >> (16 * (j & 1))) & 0xffffu, thr) ? 1u : 0u;
                    if (COUNT == 1 || (base + col) / kSeg == seg_first) cnt += c8;
                    else cnt_next += c8;
                }
            }
        }
    }
    if constexpr (COUNT != 0) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cnt += (uint32_t)__shfl_xor((int)cnt, o, kWave);
        if constexpr (COUNT == 1) {
            if (lane == 0) counts[w] = cnt;
        } else {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) cnt_next += (uint32_t)__shfl_xor((int)cnt_next, o, kWave);
            // the workgroup's waves hold neighbouring rows, mostly of the same segments: their counts
            // meet in LDS first (the workgroup's rows span at most 4 * 4096 elements, 5 segments) and
            // one thread per segment adds to memory
            const int64_t seg_wg = (blockIdx.x * 4ll * rows_per_wave * n) / kSeg;
            if (lane == 0) {
                if (cnt) atomicAdd(&wg_counts[seg_first - seg_wg], cnt);
                if (cnt_next) atomicAdd(&wg_counts[seg_first + 1 - seg_wg], cnt_next);
            }
        }
    }
    if constexpr (COUNT == 2) {
        __syncthreads();
        if (threadIdx.x < 6 && wg_counts[threadIdx.x])
            atomicAdd(&counts[(blockIdx.x * 4ll * rows_per_wave * n) / kSeg + threadIdx.x], wg_counts[threadIdx.x]);
    }
}

// ---- restore + softmax backward in one pass ----------------------------------------------
// From the compressed map (idx, val, seg_offsets) and the upstream gradient g, writes
//   a  = the restored dense map (optional, the caller needs it for grad_v = a^T @ grad_o) and
//   o  = bf16((g - sum_row bf16(a*g)) * a) * out_scale     (the layer's grad_s / sqrt(head_dim) folded in)
// without reading a dense map back from HBM.  One wave rebuilds one 4096-element segment in LDS
// exactly like sparse_restore_kernel; the segment holds 4096/n whole rows (n = 512 .. 4096), and
// each row is SPR = n/512 wave-wide steps, so its sum is a plain wave reduction.
template <int SPR>
__global__ __launch_bounds__(kSegThreads) void softmax_bwd_restore_kernel(const int64_t* __restrict__ idx,
                                                                          const uint16_t* __restrict__ val,
                                                                          const int64_t* __restrict__ offsets,
                                                                          const uint16_t* __restrict__ g, int64_t nseg,
                                                                          uint16_t* __restrict__ a_out,
                                                                          uint16_t* __restrict__ o_out, float out_scale) {
    __shared__ __attribute__((aligned(16))) uint16_t stage[kSegThreads / kWave][kSeg];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t seg = blockIdx.x * (int64_t)(kSegThreads / kWave) + wave;
    const bool live = seg < nseg;
    u32x4* st = reinterpret_cast<u32x4*>(stage[wave]);
    // The segment's share of the gradient is requested before anything else: its latency then covers
    // the two dependent round trips of the rebuild (offsets, then indices and values) instead of
    // following them.  For rows of 2048 and 4096 the 32 registers that hold it would cost waves per SIMD if the
    // row's map values were kept in registers between the row sum and the output as well, so there the
    // values are read from LDS a second time instead (kReread).
    constexpr bool kAhead = true;
    constexpr bool kReread = SPR >= 4;
    u32x4 gall[kAhead ? kSegSteps : 1];
    if constexpr (kAhead) {
#pragma unroll
        for (int c = 0; c < kSegSteps; ++c) {
            gall[c] = u32x4{0, 0, 0, 0};
            if (live) gall[c] = ld16_nt(g + seg * kSeg + (int64_t)(c * kWave + lane) * 8);
        }
    }
#pragma unroll
    for (int s = 0; s < kSegSteps; ++s) st[s * kWave + lane] = u32x4{0, 0, 0, 0};
    __syncthreads();
    if (live) {
        const int64_t e0 = offsets[seg], e1 = offsets[seg + 1];
        const int64_t first = seg * kSeg;
        for (int64_t e = e0 + lane; e < e1; e += kWave) {
            const int64_t rel = idx[e] - first;
            if (rel >= 0 && rel < kSeg) stage[wave][rel] = val[e];
        }
    }
    __syncthreads();
    if (!live) return;
#pragma unroll
    for (int r = 0; r < kSegSteps / SPR; ++r) {             // rows of this segment
        u32x4 yv[SPR], gv[SPR];
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < SPR; ++s) {
            const int c = (r * SPR + s) * kWave + lane;      // chunk inside the segment
            yv[s] = st[c];
            if constexpr (kAhead) gv[s] = gall[r * SPR + s];
            else gv[s] = ld16_nt(g + seg * kSeg + (int64_t)c * 8);
        }
#pragma unroll
        for (int s = 0; s < SPR; ++s) {
            float yf[8], gf[8];
            unpack8(yv[s], yf);
            unpack8(gv[s], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc += rbf(yf[j] * gf[j]);
        }
        acc = wave_sum(acc);
#pragma unroll
        for (int s = 0; s < SPR; ++s) {
            const int c = (r * SPR + s) * kWave + lane;
            float yf[8], gf[8], of[8];
            u32x4 y = yv[s];
            if constexpr (kReread) {
                // made opaque so that the compiler reads LDS again here instead of keeping the first read alive
                asm volatile("" ::: "memory");
                y = st[c];
            }
            unpack8(y, yf);
            unpack8(gv[s], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) of[j] = rbf((gf[j] - acc) * yf[j]) * out_scale;   // bf16 result, then the bf16 scaling
            st16_nt(o_out + seg * kSeg + (int64_t)c * 8, pack8(of));       // ordinary stores: 166 against 149 us
            if (a_out) st16_nt(a_out + seg * kSeg + (int64_t)c * 8, y);
        }
    }
}

// The same for any row length n <= 4096 that is a multiple of 8 (sequence lengths that are not a
// power of two): a wave takes the whole rows that fit into one stage of 4096 elements, which lie in
// at most two segments of the compressed map; it walks the entries of those segments and keeps the
// ones that fall into its rows.  A row is STEPS = ceil(n / 512) wave-wide steps, lanes past the end
// of the row idle; chunk c of a row belongs to lane c % 64 as in softmax_bwd_kernel, so the row sums
// are added in the same order and the results are the same bits as restore followed by that kernel.
template <int STEPS, int NRMAX>
__global__ __launch_bounds__(kSegThreads) void softmax_bwd_restore_rows_kernel(const int64_t* __restrict__ idx,
                                                                               const uint16_t* __restrict__ val,
                                                                               const int64_t* __restrict__ offsets,
                                                                               const uint16_t* __restrict__ g, int64_t rows,
                                                                               int n, int rows_per_wave,
                                                                               uint16_t* __restrict__ a_out,
                                                                               uint16_t* __restrict__ o_out, float out_scale) {
    // NRMAX bounds rows_per_wave (the host chooses both from n), so that the gradient of all the wave's
    // rows can be requested before the rebuild, as in the kernel above.
    __shared__ __attribute__((aligned(16))) uint16_t stage[kSegThreads / kWave][kSeg];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t r0 = (blockIdx.x * (int64_t)(kSegThreads / kWave) + wave) * rows_per_wave;
    if (r0 >= rows) return;                                  // waves share nothing: no workgroup barrier below
    const int nr = rows - r0 < rows_per_wave ? (int)(rows - r0) : rows_per_wave;
    const int cpr = n / 8;                                   // chunks per row
    const int64_t flat0 = r0 * n;
    const int span = nr * n;
    u32x4 gall[NRMAX][STEPS];
#pragma unroll
    for (int r = 0; r < NRMAX; ++r)
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int c = s * kWave + lane;
            gall[r][s] = u32x4{0, 0, 0, 0};
            if (r < nr && c < cpr) gall[r][s] = ld16_nt(g + flat0 + (int64_t)r * n + c * 8);
        }
    u32x4* st = reinterpret_cast<u32x4*>(stage[wave]);
    for (int c = lane; c < nr * cpr; c += kWave) st[c] = u32x4{0, 0, 0, 0};
    const int64_t seg_a = flat0 / kSeg, seg_b = (flat0 + span - 1) / kSeg;
    const int64_t e0 = offsets[seg_a], e1 = offsets[seg_b + 1];
    // a wave's LDS operations are carried out in the order it issues them: the zeros above land first
    for (int64_t e = e0 + lane; e < e1; e += kWave) {
        const int64_t rel = idx[e] - flat0;
        if (rel >= 0 && rel < span) stage[wave][rel] = val[e];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int r = 0; r < NRMAX; ++r) {
        if (r >= nr) break;                                  // uniform over the wave
        const int64_t row_at = flat0 + (int64_t)r * n;
        u32x4 yv[STEPS];
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int c = s * kWave + lane;
            yv[s] = u32x4{0, 0, 0, 0};
            if (c < cpr) yv[s] = st[r * cpr + c];
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            float yf[8], gf[8];
            unpack8(yv[s], yf);
            unpack8(gall[r][s], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc += rbf(yf[j] * gf[j]);
        }
        acc = wave_sum(acc);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int c = s * kWave + lane;
            if (c >= cpr) continue;
            float yf[8], gf[8], of[8];
            unpack8(yv[s], yf);
            unpack8(gall[r][s], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) of[j] = rbf((gf[j] - acc) * yf[j]) * out_scale;
            st16_nt(o_out + row_at + c * 8, pack8(of));
            if (a_out) st16_nt(a_out + row_at + c * 8, yv[s]);
        }
    }
}

// ---- softmax backward ---------------------------------------------------------------------
// o = bf16( (g - sum_row bf16(y*g)) * y ), the row sum accumulated in fp32
// (operators/softmax_kernels.py:31-35).  One wave per row; rows of up to 64*8*CH
// elements are held in registers so y and g are read once.
template <int CH>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const uint16_t* __restrict__ y, const uint16_t* __restrict__ g,
                                                          uint16_t* __restrict__ o, int64_t rows, int n) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = blockIdx.x * 4ll + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t base = row * n;
    u32x4 yv[CH], gv[CH];
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        yv[c] = u32x4{0, 0, 0, 0};
        gv[c] = u32x4{0, 0, 0, 0};
        if (col < n) {
            yv[c] = ld16_nt(y + base + col);
            gv[c] = ld16_nt(g + base + col);
        }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float yf[8], gf[8];
        unpack8(yv[c], yf);
        unpack8(gv[c], gf);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += rbf(yf[j] * gf[j]);
    }
    acc = wave_sum(acc);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int col = (c * kWave + lane) * 8;
        if (col < n) {
            float yf[8], gf[8], of[8];
            unpack8(yv[c], yf);
            unpack8(gv[c], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) of[j] = (gf[j] - acc) * yf[j];
            st16(o + base + col, pack8(of));          // ordinary store: 9 % faster here than a non-temporal one
        }
    }
}

// any row length / alignment: element-wise accesses, two passes over the row
__global__ __launch_bounds__(256) void softmax_bwd_generic_kernel(const uint16_t* __restrict__ y,
                                                                  const uint16_t* __restrict__ g,
                                                                  uint16_t* __restrict__ o, int64_t rows, int64_t n) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = blockIdx.x * 4ll + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t base = row * n;
    float acc = 0.0f;
    for (int64_t i = lane; i < n; i += kWave) acc += rbf(bf_to_f(y[base + i]) * bf_to_f(g[base + i]));
    acc = wave_sum(acc);
    for (int64_t i = lane; i < n; i += kWave)
        o[base + i] = f_to_bf((bf_to_f(g[base + i]) - acc) * bf_to_f(y[base + i]));
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_hist16(const void* a, int64_t n, uint32_t* hist, void* stream) {
    if (n < 0 || n >= ((int64_t)1 << 32)) return HYC_ERR_SHAPE;
    if (!hist || (n > 0 && !a)) return HYC_ERR_NULL;
    if (n > 0 && !aligned16(a)) return HYC_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(64), dim3(1024), 0, st, hist, (int64_t)65536, 0u);
    if (n > 0) {
        int64_t blocks = cdiv(cdiv(n, 8), kHistThreads * 4);
        if (blocks > 512) blocks = 512;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(hist16_kernel, dim3((unsigned)blocks), dim3(kHistThreads), 0, st, (const uint16_t*)a, n, hist);
    }
    return check_launch();
}

extern "C" int hyc_hist_select(const uint32_t* hist, int64_t kth, float* threshold, void* stream) {
    if (!hist || !threshold) return HYC_ERR_NULL;
    if (kth < 1) return HYC_ERR_ARG;
    hipLaunchKernelGGL(hist_select_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, hist, kth, threshold);
    return check_launch();
}

extern "C" int64_t hyc_sparse_num_segments(int64_t n) { return n <= 0 ? 0 : cdiv(n, kSeg); }

extern "C" int hyc_sparse_count(const void* a, int64_t n, const float* threshold, int compare_abs, uint32_t* seg_counts,
                                int64_t* seg_offsets, void* stream) {
    if (n < 0) return HYC_ERR_SHAPE;
    if (!seg_offsets || !threshold) return HYC_ERR_NULL;
    const int64_t nseg = hyc_sparse_num_segments(n);
    if (nseg > 0 && (!a || !seg_counts)) return HYC_ERR_NULL;
    if (nseg > 0 && !aligned16(a)) return HYC_ERR_ALIGN;
    if (cdiv(nseg, 4) > INT32_MAX) return HYC_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (nseg > 0)
        hipLaunchKernelGGL(sparse_count_kernel, dim3((unsigned)cdiv(nseg, 4)), dim3(kSegThreads), 0, st,
                           (const uint16_t*)a, n, threshold, nseg, seg_counts, compare_abs ? 0x7fffu : 0xffffu);
    hipLaunchKernelGGL(seg_scan_kernel, dim3((unsigned)(nseg > 1024 ? cdiv(nseg, 1024) : 1)), dim3(1024), 0, st, seg_counts, nseg, seg_offsets);
    return check_launch();
}

static int sparse_write_any(const void* a, int64_t n, const float* threshold, int compare_abs,
                            const int64_t* seg_offsets, int64_t capacity, int64_t* indices, void* values, void* stream) {
    if (n < 0 || capacity < 0) return HYC_ERR_SHAPE;
    const int64_t nseg = hyc_sparse_num_segments(n);
    if (nseg == 0) return HYC_OK;
    if (!a || !threshold || !seg_offsets || !indices || !values) return HYC_ERR_NULL;
    if (!aligned16(a)) return HYC_ERR_ALIGN;
    hipLaunchKernelGGL(sparse_write_kernel, dim3((unsigned)cdiv(nseg, 4)), dim3(kSegThreads), 0, (hipStream_t)stream,
                       (const uint16_t*)a, n, threshold, nseg, seg_offsets, indices, (uint16_t*)values,
                       compare_abs ? 0x7fffu : 0xffffu, capacity);
    return check_launch();
}

extern "C" int hyc_sparse_write(const void* a, int64_t n, const float* threshold, int compare_abs,
                                const int64_t* seg_offsets, int64_t* indices, void* values, void* stream) {
    return sparse_write_any(a, n, threshold, compare_abs, seg_offsets, INT64_MAX, indices, values, stream);
}

extern "C" int hyc_sparse_write_bounded(const void* a, int64_t n, const float* threshold, int compare_abs,
                                        const int64_t* seg_offsets, int64_t capacity, int64_t* indices, void* values,
                                        void* stream) {
    if (capacity == 0) return n < 0 ? HYC_ERR_SHAPE : HYC_OK;      // no room: nothing to write
    return sparse_write_any(a, n, threshold, compare_abs, seg_offsets, capacity, indices, values, stream);
}

extern "C" int hyc_sparse_segment_offsets(const int64_t* indices, int64_t nnz, int64_t n, int64_t* seg_offsets,
                                          void* stream) {
    if (n < 0 || nnz < 0) return HYC_ERR_SHAPE;
    if (!seg_offsets || (nnz > 0 && !indices)) return HYC_ERR_NULL;
    const int64_t nseg = hyc_sparse_num_segments(n);
    hipLaunchKernelGGL(seg_offsets_kernel, dim3((unsigned)cdiv(nnz + 1, 256)), dim3(256), 0, (hipStream_t)stream,
                       indices, nnz, nseg, seg_offsets);
    return check_launch();
}

extern "C" int hyc_sparse_restore(const int64_t* indices, const void* values, const int64_t* seg_offsets, int64_t n,
                                  void* out, void* stream) {
    if (n < 0) return HYC_ERR_SHAPE;
    const int64_t nseg = hyc_sparse_num_segments(n);
    if (nseg == 0) return HYC_OK;
    if (!seg_offsets || !out) return HYC_ERR_NULL;
    if (!aligned16(out)) return HYC_ERR_ALIGN;
    hipLaunchKernelGGL(sparse_restore_kernel, dim3((unsigned)cdiv(nseg, 4)), dim3(kSegThreads), 0, (hipStream_t)stream,
                       indices, (const uint16_t*)values, seg_offsets, nseg, n, (uint16_t*)out);
    return check_launch();
}

extern "C" int hyc_softmax_bwd(const void* y, const void* grad_y, void* out, int64_t rows, int64_t n, void* stream) {
    if (rows < 0 || n < 0) return HYC_ERR_SHAPE;
    if (rows == 0 || n == 0) return HYC_OK;
    if (!y || !grad_y || !out) return HYC_ERR_NULL;
    if (cdiv(rows, 4) > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)cdiv(rows, 4)), block(256);
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (n % 8 == 0) && n <= 4096 && aligned16(y) && aligned16(grad_y) && aligned16(out);
    const uint16_t* yp = (const uint16_t*)y;
    const uint16_t* gp = (const uint16_t*)grad_y;
    uint16_t* op = (uint16_t*)out;
    if (!vec) hipLaunchKernelGGL(softmax_bwd_generic_kernel, grid, block, 0, st, yp, gp, op, rows, n);
    else if (n <= 512) hipLaunchKernelGGL(softmax_bwd_kernel<1>, grid, block, 0, st, yp, gp, op, rows, (int)n);
    else if (n <= 1024) hipLaunchKernelGGL(softmax_bwd_kernel<2>, grid, block, 0, st, yp, gp, op, rows, (int)n);
    else if (n <= 2048) hipLaunchKernelGGL(softmax_bwd_kernel<4>, grid, block, 0, st, yp, gp, op, rows, (int)n);
    else hipLaunchKernelGGL(softmax_bwd_kernel<8>, grid, block, 0, st, yp, gp, op, rows, (int)n);
    return check_launch();
}

extern "C" int hyc_softmax_bwd_restore(const int64_t* indices, const void* values, const int64_t* seg_offsets,
                                       const void* grad_y, void* a_out, void* out, int64_t rows, int64_t n,
                                       float out_scale, void* stream) {
    if (rows < 0 || n < 8 || n > 4096 || n % 8 != 0) return HYC_ERR_SHAPE;
    if (rows == 0) return HYC_OK;
    if (!seg_offsets || !grad_y || !out) return HYC_ERR_NULL;
    if (!aligned16(grad_y) || !aligned16(out) || (a_out && !aligned16(a_out))) return HYC_ERR_ALIGN;
    if ((n != 512 && n != 1024 && n != 2048 && n != 4096) || (rows * n) % kSeg != 0) {
        // rows that do not tile the segments of the map
        // rows per wave: what fits one 4096-element stage, at most 8 (short rows leave lanes idle instead)
        const int steps = (int)cdiv(n, (int64_t)kWave * 8);
        const int rpw = kSeg / n > 8 ? 8 : (int)(kSeg / n);
        const int64_t waves = cdiv(rows, (int64_t)rpw);
        if (cdiv(waves, 4) > INT32_MAX) return HYC_ERR_SHAPE;
        const dim3 grid((unsigned)cdiv(waves, 4)), block(kSegThreads);
        hipStream_t st = (hipStream_t)stream;
#define HYC_SBR(STEPS, NRMAX)                                                                                   \
        hipLaunchKernelGGL((softmax_bwd_restore_rows_kernel<STEPS, NRMAX>), grid, block, 0, st, indices,        \
                           (const uint16_t*)values, seg_offsets, (const uint16_t*)grad_y, rows, (int)n, rpw,    \
                           (uint16_t*)a_out, (uint16_t*)out, out_scale)
        switch (steps) {                                    // NRMAX = the largest rpw of that range of n
            case 1: HYC_SBR(1, 8); break;                   // n <= 512
            case 2: HYC_SBR(2, 7); break;                   // 520 .. 1024: 7 .. 4 rows
            case 3: HYC_SBR(3, 3); break;                   // 1032 .. 1536: 3 or 2
            case 4: HYC_SBR(4, 2); break;                   // 1544 .. 2048
            case 5: HYC_SBR(5, 1); break;
            case 6: HYC_SBR(6, 1); break;
            case 7: HYC_SBR(7, 1); break;
            default: HYC_SBR(8, 1); break;
        }
#undef HYC_SBR
        return check_launch();
    }
    const int64_t nseg = rows * n / kSeg;
    if (cdiv(nseg, 4) > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)cdiv(nseg, 4)), block(kSegThreads);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* vp = (const uint16_t*)values;
    const uint16_t* gp = (const uint16_t*)grad_y;
    uint16_t* ap = (uint16_t*)a_out;
    uint16_t* op = (uint16_t*)out;
    if (n == 512) hipLaunchKernelGGL(softmax_bwd_restore_kernel<1>, grid, block, 0, st, indices, vp, seg_offsets, gp, nseg, ap, op, out_scale);
    else if (n == 1024) hipLaunchKernelGGL(softmax_bwd_restore_kernel<2>, grid, block, 0, st, indices, vp, seg_offsets, gp, nseg, ap, op, out_scale);
    else if (n == 2048) hipLaunchKernelGGL(softmax_bwd_restore_kernel<4>, grid, block, 0, st, indices, vp, seg_offsets, gp, nseg, ap, op, out_scale);
    else hipLaunchKernelGGL(softmax_bwd_restore_kernel<8>, grid, block, 0, st, indices, vp, seg_offsets, gp, nseg, ap, op, out_scale);
    return check_launch();
}

extern "C" int hyc_softmax_fwd(const void* s, const void* mask, void* out, int64_t rows, int64_t n, float scale,
                               int64_t mask_rows, int64_t rows_per_batch, int64_t mask_stride_b, int64_t mask_stride_row,
                               const float* threshold, uint32_t* seg_counts, int64_t* seg_offsets, void* stream) {
    if (rows < 0 || n < 0) return HYC_ERR_SHAPE;
    if (n % 8 != 0 || n > 8192) return HYC_ERR_SHAPE;
    const bool count = threshold || seg_counts || seg_offsets;
    if (count && !(threshold && seg_counts && seg_offsets)) return HYC_ERR_NULL;
    if (count && n > kSeg) return HYC_ERR_SHAPE;
    // rows that tile the segments: one count per wave; otherwise atomic sums into zeroed counts
#ifdef HYC_FORCE_GENERAL
    const bool tiled = false;
#else
    const bool tiled = count && n >= 512 && kSeg % n == 0 && (rows * n) % kSeg == 0;
#endif
    if (rows == 0 || n == 0) {
        if (count) hipLaunchKernelGGL(seg_scan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, seg_counts, (int64_t)0, seg_offsets);
        return count ? check_launch() : HYC_OK;
    }
    if (!s || !out) return HYC_ERR_NULL;
    if (!aligned16(s) || !aligned16(out)) return HYC_ERR_ALIGN;
    if (mask) {
        if (!aligned16(mask) || mask_stride_b % 8 || mask_stride_row % 8) return HYC_ERR_ALIGN;
        if (mask_rows <= 0 || rows_per_batch <= 0 || (mask_stride_row != 0 && mask_stride_row < n)) return HYC_ERR_SHAPE;
    } else {
        mask_rows = rows_per_batch = 1;
    }
    const int rpw = tiled ? (int)(kSeg / n) : 1;
    const int64_t nseg = count ? cdiv(rows * n, (int64_t)kSeg) : 0;
    if (count && !tiled) {
        const int64_t fb = cdiv(nseg, 256);
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)(fb > 1024 ? 1024 : fb)), dim3(256), 0, (hipStream_t)stream,
                           seg_counts, nseg, 0u);
    }
    const int64_t waves = cdiv(rows, (int64_t)rpw);
    if (cdiv(waves, 4) > INT32_MAX) return HYC_ERR_SHAPE;
    const dim3 grid((unsigned)cdiv(waves, 4)), block(256);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* sp = (const uint16_t*)s;
    const uint16_t* mp = (const uint16_t*)mask;
    uint16_t* op = (uint16_t*)out;
#define HYC_SMF(CH)                                                                                                     \
    do {                                                                                                                \
        if (tiled)                                                                                                      \
            hipLaunchKernelGGL((softmax_fwd_kernel<CH, 1>), grid, block, 0, st, sp, mp, op, rows, (int)n, scale,         \
                               (int)mask_rows, rows_per_batch, mask_stride_b, mask_stride_row, threshold, seg_counts, rpw); \
        else if (count)                                                                                                 \
            hipLaunchKernelGGL((softmax_fwd_kernel<CH, 2>), grid, block, 0, st, sp, mp, op, rows, (int)n, scale,         \
                               (int)mask_rows, rows_per_batch, mask_stride_b, mask_stride_row, threshold, seg_counts, rpw); \
        else                                                                                                            \
            hipLaunchKernelGGL((softmax_fwd_kernel<CH, 0>), grid, block, 0, st, sp, mp, op, rows, (int)n, scale,         \
                               (int)mask_rows, rows_per_batch, mask_stride_b, mask_stride_row, threshold, seg_counts, rpw); \
    } while (0)
    if (n <= 512) HYC_SMF(1);
    else if (n <= 1024) HYC_SMF(2);
    else if (n <= 2048) HYC_SMF(4);
    else if (n <= 4096) HYC_SMF(8);
    else HYC_SMF(16);
#undef HYC_SMF
    if (count) {
        hipLaunchKernelGGL(seg_scan_kernel, dim3((unsigned)(nseg > 1024 ? cdiv(nseg, 1024) : 1)), dim3(1024), 0, st, seg_counts, nseg, seg_offsets);
    }
    return check_launch();
}
