// Device-side building blocks shared by the codec kernels (gfx950, wave64).
//
// Layout used everywhere: one wavefront owns one 64x64 chunk.  The chunk lives either
// in registers (64 floats per lane: lane = row or column, register index = the other
// coordinate) or in an LDS tile with a row stride of 68 floats, which makes both the
// row-per-lane 16-byte accesses and the column-per-lane 4-byte accesses bank-conflict
// free.  The decode kernel uses the 4 padding floats of a tile row as per-lane scratch slots.
//
// Hand-scheduled sequences.  The compiler inserts the wait states this hardware needs between dependent
// instructions, but it does not look into inline assembly, and the assembler adds none.  Every assembly block
// in this file and in tplr_hip.hip therefore pads for its own hazards, inside the block and at its edges (the
// instruction after a block is the compiler's and may be of any kind).  The hazards, the rule applied, and where:
//
//   hazard                                                   rule here                        sequences
//   -------------------------------------------------------  -------------------------------  ---------------------------
//   a vector instruction writes a scalar register pair       two other instructions (or       filter16 (compares run three
//   (compare result, carry-out) and a later VECTOR           s_nop 1 / s_nop 0 + one          ahead of the add-with-carry
//   instruction reads that pair as a lane mask or carry-in   instruction) between the         chain, through three pairs);
//   (v_cndmask, v_addc_co).  A scalar instruction reading    vector write and the vector      cmp_exchange, cx32_* (compare
//   the pair in between (s_xnor) is interlocked by the       read                             or borrow -> s_xnor -> s_nop 0
//   hardware and counts as one of the two.                                                    -> select)
//   a vector instruction writes a vector register and a      s_nop 1 (two wait states)        end of cmp_exchange, cx32_*,
//   data-parallel (DPP) instruction reads it as its moved    after the write, also when the   cx32_xor4 (after its v_mov_dpp),
//   source                                                   write is the compiler's and the  sort64_desc_u32 / sort128_*_u32
//                                                            DPP read is in a block (a        entry and the J == 64 step
//                                                            leading "s_nop 1" on the value)
//   vcc written inside a block and read by the next          the blocks name vcc / scc as     all blocks that touch them
//   instruction of the same block                            clobbers and keep their own use
//                                                            two instructions from the write
//   a value that must not be hoisted out of a loop or        empty asm volatile("" : "+v")    select_topk (lane-derived
//   merged with its copies (the optimiser then keeps         on the value: an opaque copy     addresses), k_decode_aggregate
//   dozens of loop-invariant registers alive and spills)     the optimiser cannot see         (unit counts, peer count),
//                                                            through, no instruction          dct64_inv_hooked call-outs
//   a 16-byte buffer store reads its data registers after    no such store is issued from     (16-byte row stores were tried
//   issue: rewriting one in the next instruction changes     hand-written code; the           and dropped; k_row_sumsq_vec
//   what is stored                                           compiler's own are padded by it  and the calibration fills are
//                                                                                             compiler-scheduled)
//
// A new block, or a reordering of an old one, has to be checked against these rows; the select tests with ties,
// NaNs and short keys (tests/test_gpu_kernels.py) are the ones that fail when a mask or a partner is read early.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef TPLR_DCT_MATRIX_CORES
#define TPLR_DCT_MATRIX_CORES 0  // 1: a measurement build, see dct64_fwd_matrix below
#endif
#include "dct64_gen.h"

namespace tplr {

constexpr int kChunk = 64;
constexpr int kLd = 68;                    // tile row stride in floats
constexpr int kTileFloats = kChunk * kLd;  // 4352 floats = 17408 bytes: a whole chunk
constexpr int kHalfRows = 32;
constexpr int kHalfFloats = kHalfRows * kLd;  // 8704 bytes: the encode side stages half a chunk at a time
constexpr int kCandCap = 128;                 // top-k candidate slots (8 bytes each)

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD one contiguous range of
// work items so that neighbouring chunks (which share output cache lines) meet in one L2.
// The grid must be launched with 8 * ceil(n / 8) blocks; ids >= n are idle.
__device__ __forceinline__ int64_t xcd_contiguous(int64_t bid, int64_t grid) {
    const int64_t per = grid >> 3;
    return (bid & 7) * per + (bid >> 3);
}

// -----------------------------------------------------------------------------------------
// Measurement variant (TPLR_DCT_MATRIX_CORES=1, off in the product): the forward 64-point transform with its
// odd half on the matrix cores.
//
// After the 32 input butterflies the odd-indexed outputs are a 32-point DCT-IV of the differences
// d[n] = x[n] - x[63-n]: 250 of the 535 vector instructions of the factorised transform.  Here that half is the
// dense product Y = C4 D (32x32 times 32x64: one column per lane) with 32 v_mfma_f32_32x32x2_f32, which run
// beside the vector ALU work of the other resident waves (and beside this wave's even half).
//
// Operand layout of the instruction (wave64): A: lane l holds A[l%32][l/32]; B: lane l holds B[l/32][l%32];
// D: lane l, register r holds D[8(r/4) + 4(l/32) + r%4][l%32].  Lanes 0..31 and 32..63 form two column groups
// with one accumulator each.  v_permlane32_swap(a, b) exchanges the upper half of a with the lower half of b,
// which turns the register pair (d[2s], d[2s+1]) of every lane into the B operands of both groups for K-step s,
// and turns the two accumulators back into one result pair per lane.
//
// It exists to put a number on the choice of vector code for the transform: the encode launch of the 1B set takes
// 1.68 ms this way against 0.94 ms.  Each 32x32x2 fp32 instruction holds the matrix pipeline of its SIMD for 64
// cycles, 4 096 cycles per chunk, and the SIMD issues next to no vector instruction meanwhile: the matrix work comes
// on top of the vector work, not beside it, and the factorised odd half costs the vector ALU 1 000 cycles.  Its
// coefficients differ from dct64_fwd's in the last bits, so a build with it selects other elements on near-ties than
// the stand-alone transform kernels, which keep the vector code.
// -----------------------------------------------------------------------------------------
#if TPLR_DCT_MATRIX_CORES
typedef float v16f __attribute__((ext_vector_type(16)));

// y = C4_32 d for the 64 lanes' vectors; ca = this lane's row of kDct4Lane
__device__ __forceinline__ void dct4_32_matrix(const float (&d)[32], float (&y)[32], const float (&ca)[16]) {
    v16f acc_lo = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    v16f acc_hi = acc_lo;
    // (the exchange as an assembly statement with both registers read and written: through the compiler's
    // builtin the second accumulator chain was seen to be dropped; the wait states keep a matrix instruction
    // from reading a register the exchange has just written)
    auto swap_halves = [](float& a, float& b) { asm volatile("v_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b)); };
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        float b0 = d[2 * s], b1 = d[2 * s + 1];
        swap_halves(b0, b1);
        acc_lo = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[s], b0, acc_lo, 0, 0, 0);
        acc_hi = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[s], b1, acc_hi, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        float q0 = acc_lo[r], q1 = acc_hi[r];
        swap_halves(q0, q1);
        const int i = 8 * (r >> 2) + (r & 3);
        y[i] = q0;
        y[i + 4] = q1;
    }
}

__device__ __forceinline__ void load_dct4_operand(float (&ca)[16], int lane) {
    const float4* row = reinterpret_cast<const float4*>(&kDct4Lane[lane][0]);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 t = row[q];
        ca[4 * q] = t.x, ca[4 * q + 1] = t.y, ca[4 * q + 2] = t.z, ca[4 * q + 3] = t.w;
    }
}

// v <- sqrt(32) * DCT-II(v) (orthonormal), one 64-vector per lane; all 64 lanes must be active.
// `ca` is the lane's row of kDct4Lane (load_dct4_operand), kept by the caller across its loop.
__device__ __forceinline__ void dct64_fwd_matrix(float (&v)[64], const float (&ca)[16]) {
    float t[64];
    dct64_fwd_head(v, t);
    float d[32], y[32];
#pragma unroll
    for (int n = 0; n < 32; ++n) d[n] = t[63 - n];
    dct4_32_matrix(d, y, ca);
    dct64_fwd_even(t, v);
#pragma unroll
    for (int m = 0; m < 32; ++m) v[2 * m + 1] = y[m];
}
#endif

// One wavefront per workgroup: LDS instructions of a wave execute in order, so lanes only need
// the compiler to keep program order.  (A workgroup barrier would also drain the vector-memory
// counter and stall the prefetch of the next chunk.)
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
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

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS round
// trips): four shifted adds inside each row of 16 lanes, then the row totals are broadcast
// into the following rows.
__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t x) {
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x111, 0xf, 0xf, false));  // row_shr:1
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x112, 0xf, 0xf, false));  // row_shr:2
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x114, 0xf, 0xf, false));  // row_shr:4
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x118, 0xf, 0xf, false));  // row_shr:8
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x142, 0xa, 0xf, false));  // row_bcast:15
    x += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x143, 0xc, 0xf, false));  // row_bcast:31
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
// On entry lane L holds w[d] = value with flat index L*64 + d.  On exit lanes hold the k
// selected elements in canonical order (descending magnitude, lowest index first on ties):
// element i < 64 in lane i (idx0/val0), element 64 + i in lane i (idx1/val1, only for k > 64).
//
// Method: a cheap lower bound T0 for the k-th largest magnitude comes from per-lane maxima
// (k <= 32) or the maxima of each lane's two half rows (k <= 128): the k-th largest of those is met by at least k
// elements, and so are its leading bits with the rest cleared, which is as far as the search
// goes.  Everything >= T0 (typically 1.1-1.5 k elements) is compacted into 8-byte candidate
// slots - (magnitude bits, 4095 - index, sign) - in index order and bitonic-sorted, on 32-bit
// keys (magnitude above T0, slot) while the magnitudes span few enough binades, on the slots
// themselves otherwise.  If more than 128 elements pass, an exact bitwise search for the k-th
// largest magnitude runs instead (rare: constant or all-zero chunks, pathological ties).  The
// only LDS needed besides the 128 slots is a 32-row staging buffer (its rows' padding words
// included) from which the candidates are read with run-time column indices.
// NaN payload bits are not kept: a selected NaN comes out as the quiet NaN of its sign.
// ---------------------------------------------------------------------------------------
struct Selected {
    uint32_t idx0, idx1;
    float val0, val1;
};

// max(|a|, |b|, |c|) in one instruction (a quiet NaN loses against a number)
__device__ __forceinline__ float max3_abs(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, |%1|, |%2|, |%3|" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// largest magnitude among v[kFrom .. kFrom + kCount - 1]: kCount / 2 instructions
template <int kFrom, int kCount>
__device__ __forceinline__ float max_abs_of(const float (&v)[64]) {
    static_assert(kCount >= 4 && kCount % 2 == 0, "a first triple, then pairs, then the last one");
    float m = max3_abs(v[kFrom], v[kFrom + 1], v[kFrom + 2]);
#pragma unroll
    for (int d = 3; d + 1 < kCount; d += 2) m = max3_abs(m, v[kFrom + d], v[kFrom + d + 1]);
    return max3_abs(m, v[kFrom + kCount - 1], v[kFrom + kCount - 1]);
}

// The statistics the threshold is taken from: magnitudes of distinct elements of the lane's row, one (the largest)
// or two (the largest of each half of the row).  The k-th largest of the wave's statistics is met by at least k
// elements of the chunk, whichever elements they are, and the halves' maxima cost a quarter of the instructions of
// the row's two largest while passing as few candidates.
template <bool kTwo>
__device__ __forceinline__ void lane_stats(const float (&v)[64], uint32_t& b1, uint32_t& b2) {
    if (kTwo) {
        b1 = __float_as_uint(max_abs_of<0, 32>(v));
        b2 = __float_as_uint(max_abs_of<32, 32>(v));
    } else {
        b1 = __float_as_uint(max_abs_of<0, 64>(v));
        b2 = 0;
    }
}

// The search for the k-th largest lane statistic is a chain of dependent steps (vector compare, scalar count,
// scalar select), one per bit, and a wave does little else meanwhile.  The threshold only has to be a lower bound
// of the k-th largest magnitude: the search stops early and leaves the lower bits zero, which lets through the
// few more candidates whose magnitudes lie within 2^-8 (two statistics per lane) or 2^-11 (one) of the exact
// one.  With one statistic per lane a looser bound would also often leave more than 32 lanes holding candidates,
// and the select then parks its rows in two turns.
#ifndef TPLR_THRESHOLD_LOW_BIT_TWO
#define TPLR_THRESHOLD_LOW_BIT_TWO 15
#endif
#ifndef TPLR_THRESHOLD_LOW_BIT_ONE
#define TPLR_THRESHOLD_LOW_BIT_ONE 12
#endif
template <bool kTwo>
constexpr int kThresholdLowBit = kTwo ? TPLR_THRESHOLD_LOW_BIT_TWO : TPLR_THRESHOLD_LOW_BIT_ONE;

// A lower bound of the k-th largest of the lane statistics, as magnitude bits (wave-uniform): its leading bits.
template <bool kTwo>
__device__ __forceinline__ uint32_t stat_threshold(uint32_t b1, uint32_t b2, int k) {
    uint32_t t = 0;
    for (int bit = 30; bit >= kThresholdLowBit<kTwo>; --bit) {
        const uint32_t c = t | (1u << bit);
        int cnt = __popcll(__ballot(b1 >= c));
        if (kTwo) cnt += __popcll(__ballot(b2 >= c));
        if (cnt >= k) t = c;
    }
    return t;
}

// The larger of the two thresholds that two sets of lane statistics give (rows and columns of an
// untransformed chunk), in one search: a candidate passes when either set has k entries at or
// above it.
template <bool kTwo>
__device__ __forceinline__ uint32_t stat_threshold_either(uint32_t b1, uint32_t b2, uint32_t c1, uint32_t c2, int k) {
    uint32_t t = 0;
    for (int bit = 30; bit >= kThresholdLowBit<kTwo>; --bit) {
        const uint32_t c = t | (1u << bit);
        int nb = __popcll(__ballot(b1 >= c)), nc = __popcll(__ballot(c1 >= c));
        if (kTwo) nb += __popcll(__ballot(b2 >= c)), nc += __popcll(__ballot(c2 >= c));
        if (nb >= k || nc >= k) t = c;
    }
    return t;
}

// 64-bit per-lane mask (hi: d = 0..31 at bits 31..0, lo: d = 32..63) of the values that are
// not below the float threshold.  A superset is fine here, so NaN and any denormal-flush
// behaviour of the compare only add candidates.
__device__ __forceinline__ void filter16(uint32_t& m, float thr, float x0, float x1, float x2, float x3, float x4,
                                         float x5, float x6, float x7, float x8, float x9, float x10, float x11,
                                         float x12, float x13, float x14, float x15) {
    // m = (m << 16) | predicate bits, first value in the highest bit: a compare writes a lane mask,
    // add-with-carry of m to itself shifts it in.  A vector instruction that reads a scalar register
    // pair which a vector instruction has just written needs two other instructions in between on
    // this hardware, and the compiler does not look into inline assembly: the compares run three
    // ahead of the adds, through three mask registers in turn.
    uint64_t t0, t1, t2;
    asm("v_cmp_nlt_f32_e64 %[t0], |%[a0]|, %[t]\n\t"
        "v_cmp_nlt_f32_e64 %[t1], |%[a1]|, %[t]\n\t"
        "v_cmp_nlt_f32_e64 %[t2], |%[a2]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]\n\t"
        "v_cmp_nlt_f32_e64 %[t0], |%[a3]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t1]\n\t"
        "v_cmp_nlt_f32_e64 %[t1], |%[a4]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t2]\n\t"
        "v_cmp_nlt_f32_e64 %[t2], |%[a5]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]\n\t"
        "v_cmp_nlt_f32_e64 %[t0], |%[a6]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t1]\n\t"
        "v_cmp_nlt_f32_e64 %[t1], |%[a7]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t2]\n\t"
        "v_cmp_nlt_f32_e64 %[t2], |%[a8]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]\n\t"
        "v_cmp_nlt_f32_e64 %[t0], |%[a9]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t1]\n\t"
        "v_cmp_nlt_f32_e64 %[t1], |%[a10]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t2]\n\t"
        "v_cmp_nlt_f32_e64 %[t2], |%[a11]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]\n\t"
        "v_cmp_nlt_f32_e64 %[t0], |%[a12]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t1]\n\t"
        "v_cmp_nlt_f32_e64 %[t1], |%[a13]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t2]\n\t"
        "v_cmp_nlt_f32_e64 %[t2], |%[a14]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]\n\t"
        "v_cmp_nlt_f32_e64 %[t0], |%[a15]|, %[t]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t1]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t2]\n\t"
        "v_addc_co_u32_e64 %[m], vcc, %[m], %[m], %[t0]"
        : [m] "+v"(m), [t0] "=&s"(t0), [t1] "=&s"(t1), [t2] "=&s"(t2)
        : [t] "s"(thr), [a0] "v"(x0), [a1] "v"(x1), [a2] "v"(x2), [a3] "v"(x3), [a4] "v"(x4), [a5] "v"(x5),
          [a6] "v"(x6), [a7] "v"(x7), [a8] "v"(x8), [a9] "v"(x9), [a10] "v"(x10), [a11] "v"(x11), [a12] "v"(x12),
          [a13] "v"(x13), [a14] "v"(x14), [a15] "v"(x15)
        : "vcc");
}

// 64-bit per-lane mask (hi: d = 0..31 at bits 31..0, lo: d = 32..63) of the values that are
// not below the float threshold.  A superset is fine here, so NaN and any denormal-flush
// behaviour of the compare only add candidates.
__device__ __forceinline__ void filter_masks(const float (&v)[64], float thr, uint32_t& mhi, uint32_t& mlo) {
    uint32_t hi = 0, lo = 0;
    filter16(hi, thr, v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9], v[10], v[11], v[12], v[13], v[14], v[15]);
    filter16(hi, thr, v[16], v[17], v[18], v[19], v[20], v[21], v[22], v[23], v[24], v[25], v[26], v[27], v[28], v[29],
             v[30], v[31]);
    filter16(lo, thr, v[32], v[33], v[34], v[35], v[36], v[37], v[38], v[39], v[40], v[41], v[42], v[43], v[44], v[45],
             v[46], v[47]);
    filter16(lo, thr, v[48], v[49], v[50], v[51], v[52], v[53], v[54], v[55], v[56], v[57], v[58], v[59], v[60], v[61],
             v[62], v[63]);
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

// x of lane ^ J.  Distances below 16 stay inside a row of 16 lanes and are data-parallel moves
// (no trip through the LDS crossbar, whose queue the sort would otherwise fill); 16 and 32 cross rows.
template <int J>
__device__ __forceinline__ uint32_t lane_xor_u32(uint32_t x) {
    const int v = static_cast<int>(x);
    if constexpr (J == 1) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false));  // quad_perm:[1,0,3,2]
    } else if constexpr (J == 2) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false));  // quad_perm:[2,3,0,1]
    } else if constexpr (J == 4) {
        // lanes 0-3 and 8-11 of a row take lane + 4, lanes 4-7 and 12-15 take lane - 4
        const int t = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xf, 0x5, false);                 // row_shl:4
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(t, v, 0x114, 0xf, 0xa, false));  // row_shr:4
    } else if constexpr (J == 8) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(v, v, 0x128, 0xf, 0xf, false));  // row_ror:8
    } else {
        return static_cast<uint32_t>(__shfl_xor(v, J));
    }
}

template <int J>
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t x) {
    const uint32_t lo = lane_xor_u32<J>(static_cast<uint32_t>(x));
    const uint32_t hi = lane_xor_u32<J>(static_cast<uint32_t>(x >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// lanes (bit i = lane i) that keep the larger key in the compare-exchange with partner lane ^ j
// of a bitonic stage of block size k2 (descending result); `base` is the element index of lane 0
constexpr uint64_t keepmax_mask(int k2, int j, int base) {
    uint64_t m = 0;
    for (int lane = 0; lane < 64; ++lane) {
        const int i = base + lane;
        if (((i & k2) == 0) == ((i & j) == 0)) m |= 1ull << lane;
    }
    return m;
}

// e <- max(e, o) on the lanes of `keepmax`, min(e, o) elsewhere: one 64-bit compare, one scalar
// xnor with the lane mask, two selects.
__device__ __forceinline__ uint64_t cmp_exchange(uint64_t e, uint64_t o, uint64_t keepmax) {
    uint64_t take;
    // (the s_nop keeps the selects, which read the mask as a vector operand, two instructions away from
    // the vector compare that first wrote the register pair)
    asm("v_cmp_gt_u64_e64 %0, %1, %2\n\ts_xnor_b64 %0, %0, %3\n\ts_nop 0"
        : "=&s"(take)
        : "v"(o), "v"(e), "s"(keepmax)
        : "scc");
    uint32_t lo, hi;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(lo) : "v"(static_cast<uint32_t>(e)), "v"(static_cast<uint32_t>(o)), "s"(take));
    // (the next stage may read the result with a data-parallel move, which must stay two instructions
    // behind the vector write of its source; the compiler does not see the write inside the assembly)
    asm("v_cndmask_b32_e64 %0, %1, %2, %3\n\ts_nop 1"
        : "=v"(hi)
        : "v"(static_cast<uint32_t>(e >> 32)), "v"(static_cast<uint32_t>(o >> 32)), "s"(take));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// bitonic sort, descending, of 64 (one per lane) or 128 (two per lane) keys
template <int K2, int J>
__device__ __forceinline__ void sort64_step(uint64_t& e) {
    e = cmp_exchange(e, shfl_xor_u64<J>(e), keepmax_mask(K2, J, 0));
    if constexpr (J > 1)
        sort64_step<K2, J / 2>(e);
    else if constexpr (K2 < 64)
        sort64_step<K2 * 2, K2>(e);
}

__device__ __forceinline__ void sort64_desc(uint64_t& e, int) { sort64_step<2, 1>(e); }

template <int K2, int J>
__device__ __forceinline__ void sort128_step(uint64_t& e0, uint64_t& e1) {
    if constexpr (J == 64) {
        // only reached with K2 = 128: one descending block, the lower half keeps the max
        const uint64_t a = e0 > e1 ? e0 : e1, b = e0 > e1 ? e1 : e0;
        e0 = a;
        e1 = b;
    } else {
        e0 = cmp_exchange(e0, shfl_xor_u64<J>(e0), keepmax_mask(K2, J, 0));
        e1 = cmp_exchange(e1, shfl_xor_u64<J>(e1), keepmax_mask(K2, J, 64));
    }
    if constexpr (J > 1)
        sort128_step<K2, J / 2>(e0, e1);
    else if constexpr (K2 < 128)
        sort128_step<K2 * 2, K2>(e0, e1);
}

__device__ __forceinline__ void sort128_desc(uint64_t& e0, uint64_t& e1, int) { sort128_step<2, 1>(e0, e1); }

// ---- the same network on 32-bit keys, one per lane.  A subtract whose first source comes from the partner lane by a
// data-parallel move leaves "partner < mine" as its borrow, a select with the same source takes the partner: two
// vector instructions per compare-exchange where the partner is reachable by one such move (lane distances 1, 2
// and 8), three at distance 4 (a reversal inside quads, then one inside groups of eight), and a trip through the
// LDS crossbar for 16 and 32.  The wait states are those of the 64-bit form: a vector instruction reads a
// condition two instructions after the vector instruction that first wrote it, a data-parallel move reads a
// register two instructions after it was written.
#define TPLR_CX32_DPP(NAME, CTRL)                                                          \
    __device__ __forceinline__ uint32_t NAME(uint32_t e, uint64_t keepmax) {               \
        uint32_t out, diff;                                                                \
        asm("v_sub_co_u32_dpp %1, vcc, %2, %2 " CTRL " row_mask:0xf bank_mask:0xf\n\t"      \
            "s_xnor_b64 vcc, vcc, %3\n\t"                                                  \
            "s_nop 0\n\t"                                                                  \
            "v_cndmask_b32_dpp %0, %2, %2, vcc " CTRL " row_mask:0xf bank_mask:0xf\n\t"     \
            "s_nop 1"                                                                      \
            : "=&v"(out), "=&v"(diff)                                                      \
            : "v"(e), "s"(keepmax)                                                         \
            : "vcc", "scc");                                                               \
        return out;                                                                        \
    }
TPLR_CX32_DPP(cx32_xor1, "quad_perm:[1,0,3,2]")
TPLR_CX32_DPP(cx32_xor2, "quad_perm:[2,3,0,1]")
TPLR_CX32_DPP(cx32_xor8, "row_ror:8")
#undef TPLR_CX32_DPP

__device__ __forceinline__ uint32_t cx32_xor4(uint32_t e, uint64_t keepmax) {
    uint32_t out, diff, rev;
    asm("v_mov_b32_dpp %2, %3 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_sub_co_u32_dpp %1, vcc, %2, %3 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_xnor_b64 vcc, vcc, %4\n\t"
        "s_nop 0\n\t"
        "v_cndmask_b32_dpp %0, %2, %3, vcc row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "=&v"(out), "=&v"(diff), "=&v"(rev)
        : "v"(e), "s"(keepmax)
        : "vcc", "scc");
    return out;
}

__device__ __forceinline__ uint32_t cx32_far(uint32_t e, uint32_t o, uint64_t keepmax) {
    uint32_t out;
    asm("v_cmp_lt_u32_e32 vcc, %1, %2\n\t"
        "s_xnor_b64 vcc, vcc, %3\n\t"
        "s_nop 0\n\t"
        "v_cndmask_b32_e32 %0, %1, %2, vcc\n\t"
        "s_nop 1"
        : "=&v"(out)
        : "v"(o), "v"(e), "s"(keepmax)
        : "vcc", "scc");
    return out;
}

template <int J>
__device__ __forceinline__ uint32_t cx32(uint32_t e, uint64_t keep) {
    if constexpr (J == 1)
        return cx32_xor1(e, keep);
    else if constexpr (J == 2)
        return cx32_xor2(e, keep);
    else if constexpr (J == 4)
        return cx32_xor4(e, keep);
    else if constexpr (J == 8)
        return cx32_xor8(e, keep);
    else
        return cx32_far(e, static_cast<uint32_t>(__shfl_xor(static_cast<int>(e), J)), keep);
}

template <int K2, int J>
__device__ __forceinline__ void sort64_u32_step(uint32_t& e) {
    constexpr uint64_t keep = keepmax_mask(K2, J, 0);
    e = cx32<J>(e, keep);
    if constexpr (J > 1)
        sort64_u32_step<K2, J / 2>(e);
    else if constexpr (K2 < 64)
        sort64_u32_step<K2 * 2, K2>(e);
}

// descending; keys must differ wherever their order matters
__device__ __forceinline__ void sort64_desc_u32(uint32_t& e) {
    asm("s_nop 1" : "+v"(e));  // (the first step reads e by a data-parallel move)
    sort64_u32_step<2, 1>(e);
}

// two keys per lane: element i < 64 in lane i of e0, element 64 + i in lane i of e1
template <int K2, int J>
__device__ __forceinline__ void sort128_u32_step(uint32_t& e0, uint32_t& e1) {
    if constexpr (J == 64) {
        // only reached with K2 = 128: one descending block, the lower half keeps the max
        const uint32_t a = e0 > e1 ? e0 : e1, b = e0 > e1 ? e1 : e0;
        e0 = a;
        e1 = b;
        asm("s_nop 1" : "+v"(e0), "+v"(e1));  // (written by ordinary code, read next by data-parallel moves)
    } else {
        e0 = cx32<J>(e0, keepmax_mask(K2, J, 0));
        e1 = cx32<J>(e1, keepmax_mask(K2, J, 64));
    }
    if constexpr (J > 1)
        sort128_u32_step<K2, J / 2>(e0, e1);
    else if constexpr (K2 < 128)
        sort128_u32_step<K2 * 2, K2>(e0, e1);
}

__device__ __forceinline__ void sort128_desc_u32(uint32_t& e0, uint32_t& e1) {
    asm("s_nop 1" : "+v"(e0), "+v"(e1));
    sort128_u32_step<2, 1>(e0, e1);
}

// `out_scale` multiplies the gathered values (an exact power of two left over by the caller's
// transform; the ordering is taken on the unscaled values).
// `buf` is a kHalfFloats staging buffer, `cand` kCandCap slots; both are free on return.
// kOther: `o1`, `o2` are a second set of lane statistics of the same chunk, e.g. taken over the
// columns: data whose rows differ in scale put most candidates into a few lanes and one direction
// alone passes far too many of them; the threshold is then the larger of the two directions'.
template <bool kTwo, bool kOther = false>
__device__ __forceinline__ Selected select_topk(const float (&w)[64], float* buf, uint64_t* cand, int lane, int k,
                                                float out_scale, uint32_t o1 = 0, uint32_t o2 = 0) {
    uint32_t mhi = 0, mlo = 0, cnt = 0, incl = 0, total = 0;
    uint32_t floor_key;  // no candidate's key is below it (NaN and flushed denormals aside)
    {
        uint32_t b1, b2;
        lane_stats<kTwo>(w, b1, b2);
        const uint32_t t0 = kOther ? stat_threshold_either<kTwo>(b1, b2, o1, o2, k) : stat_threshold<kTwo>(b1, b2, k);
        floor_key = t0;
        filter_masks(w, __uint_as_float(t0), mhi, mlo);
        cnt = __popc(mhi) + __popc(mlo);
        incl = wave_incl_scan_u32(cnt);
        total = __builtin_amdgcn_readlane(incl, 63);

        // (the rare paths below are marked as such: code the compiler lays out of line costs the common path
        // neither taken branches nor instruction fetches)
        if (__builtin_expect(total > static_cast<uint32_t>(kCandCap) || total < static_cast<uint32_t>(k), 0)) {
            // Exact search for the k-th largest key, from the bits t0 and the maximum share.
            const uint32_t vmax = wave_max_u32(kTwo ? (mag_key(b1) > mag_key(b2) ? mag_key(b1) : mag_key(b2)) : mag_key(b1));
            uint32_t t = mag_key(t0);
            uint32_t n_ge = count_ge(w, t);
            if (n_ge > static_cast<uint32_t>(kCandCap)) {
                const uint32_t diff = t ^ vmax;
                const int top = diff ? 31 - __builtin_clz(diff) : -1;
                t = top >= 0 ? (t & ~((2u << top) - 1u)) : t;
#pragma nounroll
                for (int bit = top; bit >= 0; --bit) {
                    const uint32_t c = t | (1u << bit);
                    const uint32_t n = count_ge(w, c);
                    if (n >= static_cast<uint32_t>(k)) {
                        t = c;
                        n_ge = n;
                        if (n <= static_cast<uint32_t>(kCandCap)) break;
                    }
                }
            }
            uint32_t ghi, glo, ehi, elo;
            exact_masks(w, t, ghi, glo, ehi, elo);
            if (n_ge > static_cast<uint32_t>(kCandCap)) {
                // more ties at the threshold than slots: take the lowest-index ties only
                uint32_t g = wave_sum_u32(__popc(ghi) + __popc(glo));
                if (g >= static_cast<uint32_t>(k)) {
                    // k or more keys above the largest statistic: NaNs, which the statistics leave out (a maximum
                    // drops a quiet NaN) and which share the top key - they are the selection, lowest index first
                    t = 0x7fffffffu;
                    exact_masks(w, t, ghi, glo, ehi, elo);
                    g = 0;
                }
                const uint32_t ties = __popc(ehi) + __popc(elo);
                const uint32_t tincl = wave_incl_scan_u32(ties);
                const int need = k - static_cast<int>(g);
                const int before = static_cast<int>(tincl - ties);
                int keep = need - before;
                keep = keep < 0 ? 0 : keep;
                keep_first(ehi, elo, keep);
            }
            mhi = ghi | ehi;
            mlo = glo | elo;
            cnt = __popc(mhi) + __popc(mlo);
            incl = wave_incl_scan_u32(cnt);
            total = __builtin_amdgcn_readlane(incl, 63);
            floor_key = t;
        }
    }
    uint32_t slot = incl - cnt;  // exclusive prefix of the per-lane counts

    // compaction: lanes park their rows in the staging buffer together with a header in the row's four padding
    // words - the two masks, the first slot and the lane the row came from - and the whole wave then reads the
    // candidates out with run-time column indices: lane j takes the columns 0-31 of row j & 31 when j < 32 and its
    // columns 32-63 otherwise, one candidate per trip of a lane-divergent loop.  Two lanes per row halve the
    // length of that loop where a few rows hold most of the candidates, and nobody waits for the other half of
    // the wave.
    auto park = [&](int r) {
        regs_to_tile_rows(w, buf, r);
        *reinterpret_cast<uint4*>(buf + r * kLd + 64) = make_uint4(mhi, mlo, slot, static_cast<uint32_t>(lane));
    };
    auto compact = [&](int n_rows) {
        int who = lane;
        asm volatile("" : "+v"(who));  // (the row address is formed here, not kept across a caller's loop)
        const int r = who & 31;
        if (r < n_rows) {
            const float* row = buf + r * kLd;
            const uint4 h = *reinterpret_cast<const uint4*>(row + 64);
            const bool upper = who >= 32;
            uint32_t m = upper ? h.y : h.x;
            uint32_t at = upper ? h.z + __popc(h.x) : h.z;
            const uint32_t ix0 = h.w * 64 + (upper ? 32u : 0u);
            row += upper ? 32 : 0;
            while (m) {
                const int z = __builtin_clz(m);
                m &= ~(0x80000000u >> z);
                const uint32_t bits = __float_as_uint(row[z]);
                const uint32_t ix = ix0 + z;
                cand[at++] = (static_cast<uint64_t>(mag_key(bits)) << 32) | ((4095u - ix) << 1) | (bits >> 31);
            }
        }
    };
    // The threshold is about the k-th largest lane maximum, so with k <= 32 and no ties there are k lanes that
    // hold candidates: their rows fit the buffer's 32 together, each at its rank among those lanes, and one pass
    // serves all of them.  Otherwise each half of the wave parks its rows in turn.
    const uint64_t holders = __ballot(cnt != 0);
    const int n_holders = __popcll(holders);
    if (!kTwo && n_holders <= 32) {  // wave-uniform
        if (cnt != 0)
            park(static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(holders >> 32),
                                  __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(holders), 0u))));
        wave_lds_fence();
        compact(n_holders);
        wave_lds_fence();
    } else {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            if ((lane >> 5) == half) park(lane & 31);
            wave_lds_fence();
            compact(32);
            wave_lds_fence();
        }
    }

    Selected out;
    out.idx1 = 0;
    out.val1 = 0.0f;
    uint64_t e0, e1 = 0ull;
    // (the slot address is formed here, from a copy of the lane id the optimiser cannot see through: hoisted
    // out of a caller's chunk loop it would only be one more value to keep, or to spill, across the loop)
    int slot_of_lane = lane;
    asm volatile("" : "+v"(slot_of_lane));
    if (total <= 64) {
        const bool mine = slot_of_lane < static_cast<int>(total);
        e0 = mine ? cand[slot_of_lane] : 0ull;
        // Slots were filled in index order, so (magnitude, 63 - slot) orders the candidates as the 64-bit keys
        // do; with the magnitudes taken from the floor it fits 32 bits while they span less than 2^26 (eight
        // binades), and the sort costs a third.  The winner's slot comes back out of the key.
        const uint32_t above = static_cast<uint32_t>(e0 >> 32) - floor_key;
        if (__builtin_expect(__ballot(mine && above >= (1u << 26)) == 0, 1)) {  // wave-uniform
            uint32_t key = mine ? (above << 6) | (63u - static_cast<uint32_t>(slot_of_lane)) : 0u;
            sort64_desc_u32(key);
            e0 = cand[63u - (key & 63u)];
        } else {
            sort64_desc(e0, lane);
        }
    } else {
        const bool mine = slot_of_lane + 64 < static_cast<int>(total);
        e0 = cand[slot_of_lane];
        e1 = mine ? cand[slot_of_lane + 64] : 0ull;
        // the same with seven bits of slot and magnitudes that span less than 2^25 (four binades)
        const uint32_t above0 = static_cast<uint32_t>(e0 >> 32) - floor_key;
        const uint32_t above1 = static_cast<uint32_t>(e1 >> 32) - floor_key;
        if (__builtin_expect(__ballot(above0 >= (1u << 25) || (mine && above1 >= (1u << 25))) == 0, 1)) {  // wave-uniform
            uint32_t key0 = (above0 << 7) | (127u - static_cast<uint32_t>(slot_of_lane));
            uint32_t key1 = mine ? (above1 << 7) | (63u - static_cast<uint32_t>(slot_of_lane)) : 0u;
            sort128_desc_u32(key0, key1);
            e0 = cand[127u - (key0 & 127u)];
            if (kTwo && k > 64) e1 = cand[127u - (key1 & 127u)];
        } else {
            sort128_desc(e0, e1, lane);
        }
    }
    // a slot unpacks to index, and to the value itself: sign bit on top of the magnitude bits
    auto unpack = [&](uint64_t e, uint32_t& ix, float& val) {
        const uint32_t lo = static_cast<uint32_t>(e), key = static_cast<uint32_t>(e >> 32);
        ix = 4095u - ((lo >> 1) & 4095u);
        const uint32_t mag = key == 0x7fffffffu ? 0x7fc00000u : key;
        val = __uint_as_float(mag | (lo << 31)) * out_scale;
    };
    unpack(e0, out.idx0, out.val0);
    if (kTwo && k > 64) unpack(e1, out.idx1, out.val1);  // (kTwo: the instantiation that serves k > 32)
    wave_lds_fence();
    return out;
}

// Write the selection of one row: values (row, k) and 12-bit packed indices.
template <bool kTwo = true>
__device__ __forceinline__ void emit_selected(const Selected& s, int lane, int k, int64_t row,
                                              uint8_t* __restrict__ idx12, float* __restrict__ val) {
    float* vrow = val + row * k;
    uint8_t* irow = idx12 + row * (k + (k >> 1));
    // (lane-derived offsets are formed from a copy of the lane id the optimiser cannot see through, so that
    // they are recomputed here instead of being kept, or spilled, across a caller's chunk loop)
    asm volatile("" : "+v"(lane));
    if (lane < k) vrow[lane] = s.val0;
    const uint32_t p0 = lane_xor_u32<1>(s.idx0);  // (the neighbour's index by a data-parallel move, no LDS trip)
    if (!(lane & 1) && lane < k) {
        const uint32_t w = s.idx0 | (p0 << 12);
        uint8_t* o = irow + 3 * (lane >> 1);
        o[0] = static_cast<uint8_t>(w);
        o[1] = static_cast<uint8_t>(w >> 8);
        o[2] = static_cast<uint8_t>(w >> 16);
    }
    if (kTwo && k > 64) {
        if (lane + 64 < k) vrow[lane + 64] = s.val1;
        const uint32_t p1 = lane_xor_u32<1>(s.idx1);
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
