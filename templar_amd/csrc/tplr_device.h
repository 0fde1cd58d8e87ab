// Device-side building blocks shared by the codec kernels (gfx950, wave64).
//
// Layout used everywhere: one wavefront owns one 64x64 chunk.  The chunk lives either
// in registers (64 floats per lane: lane = row or column, register index = the other
// coordinate) or in an LDS tile with a row stride of 68 floats, which makes both the
// row-per-lane 16-byte accesses and the column-per-lane 4-byte accesses bank-conflict
// free.  The 4 padding floats of every tile row double as 128 eight-byte slots for the
// top-k candidate list.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dct64_gen.h"

namespace tplr {

constexpr int kChunk = 64;
constexpr int kLd = 68;                    // tile row stride in floats
constexpr int kTileFloats = kChunk * kLd;  // 4352 floats = 17408 bytes
constexpr int kCandCap = 128;              // candidate slots hidden in the tile padding

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD one contiguous range of
// work items so that neighbouring chunks (which share output cache lines) meet in one L2.
// The grid must be launched with 8 * ceil(n / 8) blocks; ids >= n are idle.
__device__ __forceinline__ int64_t xcd_contiguous(int64_t bid, int64_t grid) {
    const int64_t per = grid >> 3;
    return (bid & 7) * per + (bid >> 3);
}

__device__ __forceinline__ uint64_t* cand_slot(float* tile, int s) {
    return reinterpret_cast<uint64_t*>(tile + (s >> 1) * kLd + kChunk + ((s & 1) << 1));
}

// All NaNs share the top key so that they tie and fall back to index order.
__device__ __forceinline__ uint32_t mag_key(uint32_t bits) {
    const uint32_t a = bits & 0x7fffffffu;
    return a > 0x7f800000u ? 0x7fffffffu : a;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
    return x;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = __shfl_xor(x, off);
        x = o > x ? o : x;
    }
    return x;
}

__device__ __forceinline__ float wave_sum_f32(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
    return x;
}

// registers (lane = row) -> tile rows
__device__ __forceinline__ void regs_to_tile_rows(const float (&v)[64], float* tile, int lane) {
    float4* row = reinterpret_cast<float4*>(tile + lane * kLd);
#pragma unroll
    for (int c = 0; c < 16; ++c) row[c] = make_float4(v[4 * c], v[4 * c + 1], v[4 * c + 2], v[4 * c + 3]);
}

__device__ __forceinline__ void tile_rows_to_regs(float (&v)[64], const float* tile, int lane) {
    const float4* row = reinterpret_cast<const float4*>(tile + lane * kLd);
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const float4 t = row[c];
        v[4 * c] = t.x;
        v[4 * c + 1] = t.y;
        v[4 * c + 2] = t.z;
        v[4 * c + 3] = t.w;
    }
}

// registers (lane = column, register = row) <-> tile
__device__ __forceinline__ void regs_to_tile_cols(const float (&v)[64], float* tile, int lane) {
#pragma unroll
    for (int r = 0; r < 64; ++r) tile[r * kLd + lane] = v[r];
}

__device__ __forceinline__ void tile_cols_to_regs(float (&v)[64], const float* tile, int lane) {
#pragma unroll
    for (int r = 0; r < 64; ++r) v[r] = tile[r * kLd + lane];
}

// 16 KB of contiguous memory (a chunk in the (Y, X, 64, 64) layout) <-> tile, coalesced.
__device__ __forceinline__ void flat_to_tile(const float* __restrict__ src, float* tile, int lane) {
    const float4* s = reinterpret_cast<const float4*>(src);
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int q = c * 64 + lane;  // float4 index: row = q / 16, col = (q % 16) * 4
        *reinterpret_cast<float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2)) = s[q];
    }
}

__device__ __forceinline__ void tile_to_flat(const float* tile, float* __restrict__ dst, int lane) {
    float4* d = reinterpret_cast<float4*>(dst);
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int q = c * 64 + lane;
        d[q] = *reinterpret_cast<const float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2));
    }
}

// ---------------------------------------------------------------------------------------
// Top-k of the 4096 values of one chunk by magnitude.
//
// On entry lane L holds v[d] = value with flat index L*64 + d, and the same values are in
// the tile (rows).  On exit lanes hold the k selected elements in canonical order
// (descending magnitude, lowest index first on ties): element i < 64 in lane i (idx0/val0),
// element 64 + i in lane i (idx1/val1, only when k > 64).
//
// Method: a cheap lower bound T0 for the k-th largest magnitude comes from per-lane
// maxima (k <= 32) or per-lane top-2 (k <= 128): the k-th largest of those is met by at
// least k elements.  Everything >= T0 (typically 1.1-1.4 k elements) is compacted into the
// candidate slots and bitonic-sorted on the 64-bit key (magnitude bits, ~index).  If more
// than 128 elements pass, an exact bitwise search for the k-th largest magnitude runs
// instead (rare: constant or all-zero chunks, pathological ties).
// ---------------------------------------------------------------------------------------
struct Selected {
    uint32_t idx0, idx1;
    float val0, val1;
};

template <bool kTwo>
__device__ __forceinline__ void lane_stats(const float (&v)[64], uint32_t& b1, uint32_t& b2) {
    float m1 = __builtin_fabsf(v[0]);
    float m2 = 0.0f;
#pragma unroll
    for (int d = 1; d < 64; ++d) {
        const float a = __builtin_fabsf(v[d]);
        if (kTwo) m2 = __builtin_amdgcn_fmed3f(m1, m2, a);
        m1 = __builtin_fmaxf(m1, a);
    }
    b1 = __float_as_uint(m1);
    b2 = __float_as_uint(m2);
}

// k-th largest of the lane statistics, as magnitude bits (wave-uniform).
template <bool kTwo>
__device__ __forceinline__ uint32_t stat_threshold(uint32_t b1, uint32_t b2, int k) {
    uint32_t t = 0;
    for (int bit = 30; bit >= 0; --bit) {
        const uint32_t c = t | (1u << bit);
        int cnt = __popcll(__ballot(b1 >= c));
        if (kTwo) cnt += __popcll(__ballot(b2 >= c));
        if (cnt >= k) t = c;
    }
    return t;
}

// 64-bit per-lane mask (hi: d = 0..31 at bits 31..0, lo: d = 32..63) of the values that are
// not below the float threshold.  A superset is fine here, so NaN and any denormal-flush
// behaviour of the compare only add candidates.
__device__ __forceinline__ void filter_masks(const float (&v)[64], float thr, uint32_t& mhi, uint32_t& mlo) {
    uint32_t hi = 0, lo = 0;
#pragma unroll
    for (int d = 0; d < 32; ++d)
        asm volatile("v_cmp_nlt_f32_e64 vcc, |%1|, %2\n\tv_addc_co_u32_e32 %0, vcc, %0, %0, vcc"
                     : "+v"(hi)
                     : "v"(v[d]), "s"(thr)
                     : "vcc");
#pragma unroll
    for (int d = 32; d < 64; ++d)
        asm volatile("v_cmp_nlt_f32_e64 vcc, |%1|, %2\n\tv_addc_co_u32_e32 %0, vcc, %0, %0, vcc"
                     : "+v"(lo)
                     : "v"(v[d]), "s"(thr)
                     : "vcc");
    mhi = hi;
    mlo = lo;
}

// Exact masks: strictly-greater and equal to key t (integer compares on canonical keys).
__device__ __forceinline__ void exact_masks(const float (&v)[64], uint32_t t, uint32_t& ghi, uint32_t& glo,
                                            uint32_t& ehi, uint32_t& elo) {
    uint32_t gh = 0, gl = 0, eh = 0, el = 0;
#pragma unroll
    for (int d = 0; d < 64; ++d) {
        const uint32_t key = mag_key(__float_as_uint(v[d]));
        const uint32_t g = key > t ? 1u : 0u;
        const uint32_t e = key == t ? 1u : 0u;
        if (d < 32) {
            gh = (gh << 1) | g;
            eh = (eh << 1) | e;
        } else {
            gl = (gl << 1) | g;
            el = (el << 1) | e;
        }
    }
    ghi = gh;
    glo = gl;
    ehi = eh;
    elo = el;
}

// (inlined on purpose: a call would force the register-resident chunk through scratch memory)
__device__ __forceinline__ uint32_t count_ge(const float (&v)[64], uint32_t c) {
    uint32_t n = 0;
#pragma unroll
    for (int d = 0; d < 64; ++d) n += mag_key(__float_as_uint(v[d])) >= c ? 1u : 0u;
    return wave_sum_u32(n);
}

// keep only the first `keep` set bits (in d order = from bit 31 of hi down) of a mask pair
__device__ __forceinline__ void keep_first(uint32_t& hi, uint32_t& lo, int keep) {
    uint32_t h = 0, l = 0;
    while (keep > 0 && hi) {
        const uint32_t b = 0x80000000u >> __builtin_clz(hi);
        h |= b;
        hi &= ~b;
        --keep;
    }
    while (keep > 0 && lo) {
        const uint32_t b = 0x80000000u >> __builtin_clz(lo);
        l |= b;
        lo &= ~b;
        --keep;
    }
    hi = h;
    lo = l;
}

__device__ __forceinline__ uint64_t u64_max(uint64_t a, uint64_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint64_t u64_min(uint64_t a, uint64_t b) { return a > b ? b : a; }

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t x, int j) {
    const uint32_t lo = __shfl_xor(static_cast<uint32_t>(x), j);
    const uint32_t hi = __shfl_xor(static_cast<uint32_t>(x >> 32), j);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// bitonic sort, descending, of 64 (one per lane) or 128 (two per lane) keys
__device__ __forceinline__ void sort64_desc(uint64_t& e, int lane) {
#pragma unroll
    for (int k2 = 2; k2 <= 64; k2 <<= 1) {
#pragma unroll
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            const uint64_t o = shfl_xor_u64(e, j);
            const bool keepmax = ((lane & k2) == 0) == ((lane & j) == 0);
            e = keepmax ? u64_max(e, o) : u64_min(e, o);
        }
    }
}

__device__ __forceinline__ void sort128_desc(uint64_t& e0, uint64_t& e1, int lane) {
#pragma unroll
    for (int k2 = 2; k2 <= 128; k2 <<= 1) {
#pragma unroll
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            if (j == 64) {
                // only reached with k2 = 128: one descending block, lower half keeps the max
                const uint64_t a = u64_max(e0, e1), b = u64_min(e0, e1);
                e0 = a;
                e1 = b;
            } else {
                const uint64_t o0 = shfl_xor_u64(e0, j);
                const uint64_t o1 = shfl_xor_u64(e1, j);
                const bool low = (lane & j) == 0;
                const bool up0 = (lane & k2) == 0;         // element index = lane
                const bool up1 = ((lane + 64) & k2) == 0;  // element index = lane + 64
                e0 = (up0 == low) ? u64_max(e0, o0) : u64_min(e0, o0);
                e1 = (up1 == low) ? u64_max(e1, o1) : u64_min(e1, o1);
            }
        }
    }
}

template <bool kTwo>
__device__ __forceinline__ Selected select_topk(const float (&v)[64], float* tile, int lane, int k) {
    uint32_t b1, b2;
    lane_stats<kTwo>(v, b1, b2);
    const uint32_t t0 = stat_threshold<kTwo>(b1, b2, k);
    uint32_t mhi, mlo;
    filter_masks(v, __uint_as_float(t0), mhi, mlo);
    uint32_t cnt = __popc(mhi) + __popc(mlo);
    uint32_t total = wave_sum_u32(cnt);

    if (total > static_cast<uint32_t>(kCandCap) || total < static_cast<uint32_t>(k)) {
        // Exact search for the k-th largest key, from the bits t0 and the maximum share.
        const uint32_t vmax = wave_max_u32(mag_key(b1));
        uint32_t t = mag_key(t0);
        uint32_t n_ge = count_ge(v, t);
        if (n_ge > static_cast<uint32_t>(kCandCap)) {
            const uint32_t diff = t ^ vmax;
            const int top = diff ? 31 - __builtin_clz(diff) : -1;
            t = top >= 0 ? (t & ~((2u << top) - 1u)) : t;
#pragma nounroll
            for (int bit = top; bit >= 0; --bit) {
                const uint32_t c = t | (1u << bit);
                const uint32_t n = count_ge(v, c);
                if (n >= static_cast<uint32_t>(k)) {
                    t = c;
                    n_ge = n;
                    if (n <= static_cast<uint32_t>(kCandCap)) break;
                }
            }
        }
        uint32_t ghi, glo, ehi, elo;
        exact_masks(v, t, ghi, glo, ehi, elo);
        if (n_ge > static_cast<uint32_t>(kCandCap)) {
            // more ties at the threshold than slots: take the lowest-index ties only
            const uint32_t g = wave_sum_u32(__popc(ghi) + __popc(glo));
            const uint32_t ties = __popc(ehi) + __popc(elo);
            uint32_t incl = ties;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const uint32_t o = __shfl_up(incl, off);
                if (lane >= off) incl += o;
            }
            const int need = k - static_cast<int>(g);
            const int before = static_cast<int>(incl - ties);
            int keep = need - before;
            keep = keep < 0 ? 0 : keep;
            keep_first(ehi, elo, keep);
        }
        mhi = ghi | ehi;
        mlo = glo | elo;
        cnt = __popc(mhi) + __popc(mlo);
        total = wave_sum_u32(cnt);
    }

    // exclusive prefix of the per-lane counts
    uint32_t incl = cnt;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    uint32_t slot = incl - cnt;

    // compaction: (magnitude key, ~index) into the candidate slots
    const float* row = tile + lane * kLd;
    while (mhi) {
        const int d = __builtin_clz(mhi);
        mhi &= ~(0x80000000u >> d);
        const uint32_t key = mag_key(__float_as_uint(row[d]));
        *cand_slot(tile, slot++) = (static_cast<uint64_t>(key) << 32) | (0xffffffffu - (lane * 64 + d));
    }
    while (mlo) {
        const int d = 32 + __builtin_clz(mlo);
        mlo &= ~(0x80000000u >> (d - 32));
        const uint32_t key = mag_key(__float_as_uint(row[d]));
        *cand_slot(tile, slot++) = (static_cast<uint64_t>(key) << 32) | (0xffffffffu - (lane * 64 + d));
    }
    __syncthreads();

    Selected out;
    out.idx1 = 0;
    out.val1 = 0.0f;
    if (total <= 64) {
        uint64_t e = lane < static_cast<int>(total) ? *cand_slot(tile, lane) : 0ull;
        sort64_desc(e, lane);
        out.idx0 = 0xffffffffu - static_cast<uint32_t>(e);
    } else {
        uint64_t e0 = *cand_slot(tile, lane);
        uint64_t e1 = lane + 64 < static_cast<int>(total) ? *cand_slot(tile, lane + 64) : 0ull;
        sort128_desc(e0, e1, lane);
        out.idx0 = 0xffffffffu - static_cast<uint32_t>(e0);
        out.idx1 = 0xffffffffu - static_cast<uint32_t>(e1);
    }
    // lanes beyond k may hold padding (index 0xffffffff - 0 wraps to a huge value): clamp
    out.idx0 &= 4095u;
    out.idx1 &= 4095u;
    out.val0 = tile[(out.idx0 >> 6) * kLd + (out.idx0 & 63)];
    if (k > 64) out.val1 = tile[(out.idx1 >> 6) * kLd + (out.idx1 & 63)];
    return out;
}

// Write the selection of one row: values (row, k) and 12-bit packed indices.
__device__ __forceinline__ void emit_selected(const Selected& s, int lane, int k, int64_t row,
                                              uint8_t* __restrict__ idx12, float* __restrict__ val) {
    float* vrow = val + row * k;
    uint8_t* irow = idx12 + row * (k + (k >> 1));
    if (lane < k) vrow[lane] = s.val0;
    const uint32_t p0 = __shfl_xor(s.idx0, 1);
    if (!(lane & 1) && lane < k) {
        const uint32_t w = s.idx0 | (p0 << 12);
        uint8_t* o = irow + 3 * (lane >> 1);
        o[0] = static_cast<uint8_t>(w);
        o[1] = static_cast<uint8_t>(w >> 8);
        o[2] = static_cast<uint8_t>(w >> 16);
    }
    if (k > 64) {
        if (lane + 64 < k) vrow[lane + 64] = s.val1;
        const uint32_t p1 = __shfl_xor(s.idx1, 1);
        if (!(lane & 1) && lane + 64 < k) {
            const uint32_t w = s.idx1 | (p1 << 12);
            uint8_t* o = irow + 3 * ((lane + 64) >> 1);
            o[0] = static_cast<uint8_t>(w);
            o[1] = static_cast<uint8_t>(w >> 8);
            o[2] = static_cast<uint8_t>(w >> 16);
        }
    }
}

}  // namespace tplr
