// libtplr_hip.so - gfx950 kernels and C ABI for templar's gradient codec.
// Reference semantics: src/tplr/compress.py (tplr 2.1.28); the entry points and what each
// replaces are documented in include/tplr_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <mutex>

#include "../../include/tplr_hip.h"
#include "tplr_device.h"

namespace tplr {

// =========================================================================================
// 12-bit pack / unpack (src/tplr/compress.py:51-142)
// =========================================================================================
__global__ __launch_bounds__(256) void k_pack12(const int64_t* __restrict__ idx, int64_t n_pairs,
                                                uint8_t* __restrict__ out, int32_t* __restrict__ err) {
    // one thread packs 4 pairs -> 12 bytes
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t p0 = t * 4;
    if (p0 >= n_pairs) return;
    int64_t worst = 0;
    uint32_t w[4];
    const int np = n_pairs - p0 < 4 ? static_cast<int>(n_pairs - p0) : 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        w[i] = 0;
        if (i < np) {
            const int64_t a = idx[2 * (p0 + i)], b = idx[2 * (p0 + i) + 1];
            worst = a > worst ? a : worst;
            worst = b > worst ? b : worst;
            // the reference narrows to int32 and masks (compress.py:77,95-97)
            const uint32_t ua = static_cast<uint32_t>(a), ub = static_cast<uint32_t>(b);
            w[i] = (ua & 0xfffu) | ((ub & 0xfffu) << 12);
        }
    }
    uint8_t* o = out + p0 * 3;
    if (np == 4 && ((reinterpret_cast<uintptr_t>(o) & 3) == 0)) {
        uint32_t* o32 = reinterpret_cast<uint32_t*>(o);
        o32[0] = w[0] | (w[1] << 24);
        o32[1] = (w[1] >> 8) | (w[2] << 16);
        o32[2] = (w[2] >> 16) | (w[3] << 8);
    } else {
        for (int i = 0; i < np; ++i) {
            o[3 * i] = static_cast<uint8_t>(w[i]);
            o[3 * i + 1] = static_cast<uint8_t>(w[i] >> 8);
            o[3 * i + 2] = static_cast<uint8_t>(w[i] >> 16);
        }
    }
    if (worst > 4095 && err) atomicMax(err, worst > 0x7fffffff ? 0x7fffffff : static_cast<int32_t>(worst));
}

__global__ __launch_bounds__(256) void k_unpack12(const uint8_t* __restrict__ in, int64_t n_pairs,
                                                  int64_t* __restrict__ idx) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t p0 = t * 4;
    if (p0 >= n_pairs) return;
    const int np = n_pairs - p0 < 4 ? static_cast<int>(n_pairs - p0) : 4;
    const uint8_t* s = in + p0 * 3;
    uint32_t w[4];
    if (np == 4 && ((reinterpret_cast<uintptr_t>(s) & 3) == 0)) {
        const uint32_t* s32 = reinterpret_cast<const uint32_t*>(s);
        const uint32_t a = s32[0], b = s32[1], c = s32[2];
        w[0] = a & 0xffffffu;
        w[1] = (a >> 24) | ((b & 0xffffu) << 8);
        w[2] = (b >> 16) | ((c & 0xffu) << 16);
        w[3] = c >> 8;
    } else {
        for (int i = 0; i < np; ++i)
            w[i] = s[3 * i] | (static_cast<uint32_t>(s[3 * i + 1]) << 8) | (static_cast<uint32_t>(s[3 * i + 2]) << 16);
    }
    for (int i = 0; i < np; ++i) {
        idx[2 * (p0 + i)] = static_cast<int64_t>(w[i] & 0xfffu);
        idx[2 * (p0 + i) + 1] = static_cast<int64_t>((w[i] >> 12) & 0xfffu);
    }
}

// =========================================================================================
// chunk loaders / storers for the (R, C) row-major side: lane = column
// =========================================================================================
// Chunk rows through buffer instructions: one resource descriptor per chunk (scalar base,
// byte range for bounds checking), the row offset r*ld in a scalar register and lane*4 as the
// only vector operand, so addressing costs no vector ALU work.  ld*4*63 must fit in 31 bits.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t chunk_rsrc(const void* chunk0, int64_t ld) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(chunk0), 0, static_cast<int>((63 * ld + 64) * 4),
                                             0x00020000);
}

template <int kRow0 = 0, int kRow1 = 64>
__device__ __forceinline__ void load_chunk_rows(float (&v)[64], const void* chunk0, int64_t ld, int lane) {
    const __amdgpu_buffer_rsrc_t rs = chunk_rsrc(chunk0, ld);
    const int ld4 = static_cast<int>(ld) * 4;
#pragma unroll
    for (int r = kRow0; r < kRow1; ++r)
        v[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, r * ld4, 2));
}

// drop (wave-uniform): the stores are issued against a range of zero bytes, whose bounds check
// discards them - the instruction stream stays the same for a chunk that must not be written
__device__ __forceinline__ void store_chunk_rows(const float (&v)[64], void* chunk0, int64_t ld, int lane,
                                                 bool drop = false) {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        chunk0, 0, drop ? 0 : static_cast<int>((63 * ld + 64) * 4), 0x00020000);
    const int ld4 = static_cast<int>(ld) * 4;
#pragma unroll
    for (int r = 0; r < 64; ++r)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v[r]), rs, lane * 4, r * ld4, 2);
}

__device__ __forceinline__ void load_chunk_cols(float (&v)[64], const float* __restrict__ x, int64_t ld,
                                                int64_t y, int64_t xc, int lane) {
    load_chunk_rows(v, x + (y * 64) * ld + xc * 64, ld, lane);
}

__device__ __forceinline__ void store_chunk_cols(const float (&v)[64], float* __restrict__ x, int64_t ld,
                                                 int64_t y, int64_t xc, int lane) {
    store_chunk_rows(v, x + (y * 64) * ld + xc * 64, ld, lane);
}

// forward 2-D transform of the chunk held column-per-lane; result row-per-lane:
// v[d] = coef[lane][d], and the tile is left free
// registers column-per-lane (v[r] = M[r][lane]) -> registers row-per-lane (w[c] = M[lane][c])
// through a 32-row staging buffer: rows 0..31 go first and lanes 0..31 pick theirs up, then rows
// 32..63 for lanes 32..63.  Half the LDS of a whole-chunk tile, which is what lets twice as many
// waves stay resident.
__device__ __forceinline__ void transpose_via_half(const float (&v)[64], float (&w)[64], float* buf, int lane) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int r = 0; r < kHalfRows; ++r) buf[r * kLd + lane] = v[half * kHalfRows + r];
        wave_lds_fence();
        if ((lane >> 5) == half) tile_rows_to_regs(w, buf, lane & 31);
        wave_lds_fence();
    }
}

// Forward 2-D transform of a chunk held column-per-lane (v[r] = X[r][lane]); the result is
// row-per-lane: w[d] = 32 * coef[lane][d] with the transform, X[lane][d] without.
template <bool kUseDct>
__device__ __forceinline__ void chunk_forward(float (&v)[64], float (&w)[64], float* buf, int lane) {
    if (kUseDct) dct64_fwd(v);  // along rows k: v[b] = sum_k X[k][lane] F[k][b]
    transpose_via_half(v, w, buf, lane);
    if (kUseDct) dct64_fwd(w);  // along columns l: w[d] = sum_l T[lane][l] F[l][d]
}

// inverse: tile holds coef rows; result column-per-lane v[k] = x[k][lane]
// (the tile must hold the coefficients times 2^-5: the two passes multiply by 32; kScaleInput
// applies that factor here for callers whose tile holds plain coefficients)
template <bool kUseDct, bool kScaleInput = false>
__device__ __forceinline__ void chunk_inverse(float (&v)[64], float* tile, int lane) {
    if (kUseDct) {
        tile_rows_to_regs(v, tile, lane);
        if (kScaleInput) {
#pragma unroll
            for (int d = 0; d < 64; ++d) v[d] *= kDctPow2Scale;
        }
        dct64_inv(v);  // along d: v[l] = sum_d Y[lane][d] F[l][d]
        wave_lds_fence();
        regs_to_tile_rows(v, tile, lane);
        wave_lds_fence();
    }
    tile_cols_to_regs(v, tile, lane);
    if (kUseDct) dct64_inv(v);  // along b: v[k] = sum_b Z[b][lane] F[k][b]
}

// -----------------------------------------------------------------------------------------
// Persistent kernels walk a contiguous range of the batch's chunk list.  A cursor keeps the
// current tensor's descriptor and the chunk's (y, x) position in wave-uniform registers.
// -----------------------------------------------------------------------------------------
// Pointers that come out of descriptor tables are not kernel arguments, so the compiler
// cannot tell that they are global memory; say so, or it emits FLAT accesses (which also
// count as LDS traffic and serialise against the tile).
typedef float v4f __attribute__((ext_vector_type(4)));
using gfloat = __attribute__((address_space(1))) float;
using gbyte = __attribute__((address_space(1))) uint8_t;

struct Cursor {
    const tplr_tensor_desc* table;
    int n_tensors;
    int t;
    gfloat* base;
    int64_t ld;
    int64_t begin, end;  // chunk ids covered by tensor t
    int X;
    int64_t y;
    int xc;
};

// descriptor fields are the same for every lane: move them to scalar registers so that chunk
// rows are addressed as scalar base + 32-bit lane offset
__device__ __forceinline__ int64_t uniform64(int64_t x) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(x));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(static_cast<uint64_t>(x) >> 32));
    return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

__device__ __forceinline__ void cursor_take(Cursor& c, const tplr_tensor_desc& d) {
    c.base = (gfloat*)uniform64(reinterpret_cast<int64_t>(d.dense));
    c.ld = uniform64(d.ld);
    c.begin = uniform64(d.chunk_begin);
    c.X = __builtin_amdgcn_readfirstlane(d.x_chunks);
    c.end = c.begin + static_cast<int64_t>(c.X) * __builtin_amdgcn_readfirstlane(d.y_chunks);
}

__device__ __forceinline__ void cursor_seek(Cursor& c, const tplr_tensor_desc* table, const tplr_tensor_desc& single,
                                            int n_tensors, int64_t g) {
    c.table = table;
    c.n_tensors = n_tensors;
    c.t = 0;
    if (table) {
        int lo = 0, hi = n_tensors;  // last tensor whose chunk_begin <= g and that is not empty
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table[mid].chunk_begin <= g)
                lo = mid;
            else
                hi = mid;
        }
        c.t = lo;
        cursor_take(c, table[lo]);
    } else {
        cursor_take(c, single);
    }
    const int64_t local = g - c.begin;
    c.y = local / c.X;
    c.xc = static_cast<int>(local - c.y * c.X);
}

// advance to chunk g (= previous chunk + 1)
__device__ __forceinline__ void cursor_next(Cursor& c, int64_t g) {
    if (++c.xc == c.X) {
        c.xc = 0;
        ++c.y;
    }
    while (g >= c.end && c.t + 1 < c.n_tensors) {  // batch mode only: single tensors never get here
        ++c.t;
        cursor_take(c, c.table[c.t]);
        c.y = 0;
        c.xc = 0;
    }
}

// the contiguous slice of [0, total) that workgroup `bid` of a grid of G (multiple of 8) owns;
// workgroups b, b+8, b+16, ... run on the same XCD and take neighbouring slices
// `align` > 1 (a power of two): where slices are long (64 items and more), the boundaries between the
// slices of one XCD fall on multiples of `align` counted from -`first`, i.e. on absolute multiples when
// [0, total) stands for the items first .. first + total - 1 of a longer list
__device__ __forceinline__ void my_range(int64_t total, int64_t& g0, int64_t& g1, int align = 1, int64_t first = 0) {
    const int64_t bid = blockIdx.x, S = gridDim.x >> 3;
    const int64_t xcd = bid & 7, slot = bid >> 3;
    const int64_t per = (total + 7) >> 3;
    const int64_t xb = xcd * per;
    int64_t xe = xb + per;
    xe = xe > total ? total : xe;
    const int64_t len = xe > xb ? xe - xb : 0;
    g0 = xb + len * slot / S;
    g1 = xb + len * (slot + 1) / S;
    if (align > 1 && len >= 64 * S) {
        if (slot > 0) g0 = ((g0 + first) & ~static_cast<int64_t>(align - 1)) - first;
        if (slot + 1 < S) g1 = ((g1 + first) & ~static_cast<int64_t>(align - 1)) - first;
        g0 = g0 < xb ? xb : g0;
        g1 = g1 < xb ? xb : g1;
    }
}

template <int kRow0 = 0, int kRow1 = 64>
__device__ __forceinline__ void load_chunk_cols(float (&v)[64], const Cursor& c, int lane) {
    load_chunk_rows<kRow0, kRow1>(v, (const void*)(c.base + (c.y * 64) * c.ld + static_cast<int64_t>(c.xc) * 64),
                                  c.ld, lane);
}

// =========================================================================================
// standalone transforms
// =========================================================================================
__global__ __launch_bounds__(64) void k_dct2d_fwd(const float* __restrict__ x, int64_t ld, int64_t X,
                                                  int64_t n_chunks, float* __restrict__ coef) {
    __shared__ __align__(16) float tile[kTileFloats];
    const int lane = threadIdx.x;
    const int64_t chunk = xcd_contiguous(blockIdx.x, gridDim.x);
    if (chunk >= n_chunks) return;
    const int64_t y = chunk / X, xc = chunk - y * X;
    float v[64], w[64];
    load_chunk_cols(v, x, ld, y, xc, lane);
    chunk_forward<true>(v, w, tile, lane);
#pragma unroll
    for (int d = 0; d < 64; ++d) w[d] *= kDctPow2Scale;  // exact: 32x the orthonormal transform so far
    regs_to_tile_rows(w, tile, lane);
    __syncthreads();
    tile_to_flat(tile, coef + chunk * 4096, lane);
}

__global__ __launch_bounds__(64) void k_dct2d_inv(const float* __restrict__ coef, int64_t X, int64_t n_chunks,
                                                  float* __restrict__ x, int64_t ld) {
    __shared__ __align__(16) float tile[kTileFloats];
    const int lane = threadIdx.x;
    const int64_t chunk = xcd_contiguous(blockIdx.x, gridDim.x);
    if (chunk >= n_chunks) return;
    const int64_t y = chunk / X, xc = chunk - y * X;
    flat_to_tile(coef + chunk * 4096, tile, lane);
    __syncthreads();
    float v[64];
    chunk_inverse<true, true>(v, tile, lane);
    store_chunk_cols(v, x, ld, y, xc, lane);
}

__global__ __launch_bounds__(64) void k_dct1d(const float* __restrict__ in, int64_t n_vec, int inverse,
                                              float* __restrict__ out) {
    __shared__ __align__(16) float tile[kTileFloats];
    const int lane = threadIdx.x;
    const int64_t base = static_cast<int64_t>(blockIdx.x) * 64;  // 64 vectors per wave
    const int64_t left = n_vec - base;
    // stage 64 vectors (rows) through the tile so that global accesses stay coalesced
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int q = c * 64 + lane;
        const int r = q >> 4;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < left) t = reinterpret_cast<const float4*>(in + base * 64)[q];
        *reinterpret_cast<float4*>(tile + r * kLd + ((q & 15) << 2)) = t;
    }
    __syncthreads();
    float v[64];
    tile_rows_to_regs(v, tile, lane);
    if (inverse)
        dct64_inv(v);
    else
        dct64_fwd(v);
    // one pass is sqrt(32) times the orthonormal transform
#pragma unroll
    for (int d = 0; d < 64; ++d) v[d] *= 0.17677669529663687f;
    __syncthreads();
    regs_to_tile_rows(v, tile, lane);
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int q = c * 64 + lane;
        const int r = q >> 4;
        if (r < left)
            reinterpret_cast<float4*>(out + base * 64)[q] =
                *reinterpret_cast<const float4*>(tile + r * kLd + ((q & 15) << 2));
    }
}

// dense contraction for chunk sizes other than 64 (h, w <= 64)
__global__ __launch_bounds__(256) void k_dct2d_dense(const float* __restrict__ in, int64_t C, int h, int w,
                                                     const float* __restrict__ bh, const float* __restrict__ bw,
                                                     int in_chunked, int out_chunked,
                                                     float* __restrict__ out) {
    __shared__ float sx[64 * 64];
    __shared__ float st[64 * 64];
    __shared__ float sbh[64 * 64];
    __shared__ float sbw[64 * 64];
    const int tid = threadIdx.x;
    const int64_t X = C / w;
    const int64_t chunk = blockIdx.x;
    const int64_t y = chunk / X, xc = chunk - y * X;
    const int hw = h * w;
    for (int i = tid; i < h * h; i += 256) sbh[i] = bh[i];
    for (int i = tid; i < w * w; i += 256) sbw[i] = bw[i];
    for (int i = tid; i < hw; i += 256) {
        const int r = i / w, c = i - r * w;
        sx[i] = in_chunked ? in[chunk * hw + i] : in[(y * h + r) * C + xc * w + c];
    }
    __syncthreads();
    for (int i = tid; i < hw; i += 256) {
        const int b = i / w, l = i - b * w;
        float acc = 0.f;
        for (int k = 0; k < h; ++k) acc = __builtin_fmaf(sbh[k * h + b], sx[k * w + l], acc);
        st[i] = acc;
    }
    __syncthreads();
    for (int i = tid; i < hw; i += 256) {
        const int b = i / w, d = i - b * w;
        float acc = 0.f;
        for (int l = 0; l < w; ++l) acc = __builtin_fmaf(st[b * w + l], sbw[l * w + d], acc);
        if (out_chunked)
            out[chunk * hw + i] = acc;
        else
            out[(y * h + b) * C + xc * w + d] = acc;
    }
}

// =========================================================================================
// top-k select + pack
// =========================================================================================
template <bool kTwo>
__global__ __launch_bounds__(64) void k_topk_rows(const float* __restrict__ coef, int64_t n_rows, int row_len,
                                                  int k, uint8_t* __restrict__ idx12, float* __restrict__ val) {
    __shared__ __align__(16) float tile[kTileFloats];
    __shared__ uint64_t cand[kCandCap];
    const int lane = threadIdx.x;
    const int64_t row = xcd_contiguous(blockIdx.x, gridDim.x);
    if (row >= n_rows) return;
    const float* src = coef + row * row_len;
    if (row_len == 4096) {
        flat_to_tile(src, tile, lane);
    } else {
#pragma unroll 4
        for (int i = 0; i < 64; ++i) {
            const int e = i * 64 + lane;
            tile[i * kLd + lane] = e < row_len ? src[e] : 0.0f;
        }
    }
    __syncthreads();
    float w[64];
    tile_rows_to_regs(w, tile, lane);
    __syncthreads();
    const Selected s = select_topk<kTwo>(w, tile, cand, lane, k, 1.0f);
    emit_selected<kTwo>(s, lane, k, row, idx12, val);
}

// Any k up to the row length: the whole row sorted.  One workgroup of 256 threads per row, the row as
// 4096 keys (magnitude, 4095 - index, sign: the canonical order of select_topk, elements past the row
// as zeros at their own indices, which no real element ranks below) in LDS, a bitonic network of 78
// steps in descending order, then the k leading keys unpacked as select_topk unpacks its candidates.
// Not a fast path: it serves selections larger than the register-resident select holds (k > 128).
__global__ __launch_bounds__(256) void k_topk_rows_sorted(const float* __restrict__ coef, int64_t n_rows, int row_len,
                                                          int k, uint8_t* __restrict__ idx12, float* __restrict__ val) {
    __shared__ uint64_t keys[4096];
    const int tid = threadIdx.x;
    const int64_t row = xcd_contiguous(blockIdx.x, gridDim.x);
    if (row >= n_rows) return;  // (the whole workgroup)
    const float* src = coef + row * row_len;
    for (int e = tid; e < 4096; e += 256) {
        const uint32_t bits = e < row_len ? __float_as_uint(src[e]) : 0u;
        keys[e] = (static_cast<uint64_t>(mag_key(bits)) << 32) | ((4095u - static_cast<uint32_t>(e)) << 1) | (bits >> 31);
    }
    __syncthreads();
    for (int size = 2; size <= 4096; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = tid; i < 2048; i += 256) {
                const int pos = 2 * i - (i & (stride - 1));
                const uint64_t a = keys[pos], b = keys[pos + stride];
                const bool down = (pos & size) == 0;  // this run is sorted in descending order
                if ((a < b) == down) {
                    keys[pos] = b;
                    keys[pos + stride] = a;
                }
            }
            __syncthreads();
        }
    }
    float* vrow = val + row * k;
    uint8_t* irow = idx12 + row * (k + (k >> 1));
    for (int j = tid; j < (k >> 1); j += 256) {
        uint32_t ix[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint64_t e = keys[2 * j + h];
            const uint32_t lo = static_cast<uint32_t>(e), key = static_cast<uint32_t>(e >> 32);
            ix[h] = 4095u - ((lo >> 1) & 4095u);
            const uint32_t mag = key == 0x7fffffffu ? 0x7fc00000u : key;
            vrow[2 * j + h] = __uint_as_float(mag | (lo << 31));
        }
        const uint32_t w = ix[0] | (ix[1] << 12);
        irow[3 * j] = static_cast<uint8_t>(w);
        irow[3 * j + 1] = static_cast<uint8_t>(w >> 8);
        irow[3 * j + 2] = static_cast<uint8_t>(w >> 16);
    }
}

// The 1-D parameters of a set (norm vectors), every tensor a run of rows of 64 elements: transform,
// top-k and pack of all of them in one launch, each tensor read where it lies.  One wave takes up to 64
// rows of one tensor: staged through the tile, a row per lane in registers, the 64-point transform and
// its scale exactly as k_dct1d applies them, then every lane sorts its own 64 coefficients in registers -
// a bitonic network over 64-bit keys (magnitude, 63 - index), the canonical order of select_topk - and
// writes its row's payload: the k leading indices, and their values fetched back from the tile.
template <bool kUseDct>
__global__ __launch_bounds__(64) void k_encode_rows(const tplr_tensor_desc* __restrict__ table, int n_tensors, int k,
                                                    uint8_t* __restrict__ idx12, float* __restrict__ val) {
    __shared__ __align__(16) float tile[kTileFloats];
    const int lane = threadIdx.x;
    // this wave's tensor and group of rows: tensor t has ceil(rows / 64) groups
    int t = 0, grp = blockIdx.x;
    for (; t < n_tensors; ++t) {
        const int groups = (table[t].x_chunks + 63) >> 6;
        if (grp < groups) break;
        grp -= groups;
    }
    if (t >= n_tensors) return;
    const tplr_tensor_desc d = table[t];
    const int left = d.x_chunks - grp * 64;  // rows from this group's first to the tensor's end
    const gfloat* src = (const gfloat*)d.dense + static_cast<int64_t>(grp) * 4096;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int q = c * 64 + lane;
        const int r = q >> 4;
        v4f x = {0.f, 0.f, 0.f, 0.f};
        if (r < left) x = *reinterpret_cast<const __attribute__((address_space(1))) v4f*>(src + q * 4);
        *reinterpret_cast<v4f*>(tile + r * kLd + ((q & 15) << 2)) = x;
    }
    wave_lds_fence();
    float w[64];
    tile_rows_to_regs(w, tile, lane);
    if (kUseDct) {
        dct64_fwd(w);
#pragma unroll
        for (int e = 0; e < 64; ++e) w[e] *= 0.17677669529663687f;  // one pass is sqrt(32) times the orthonormal transform
    }
    wave_lds_fence();
    regs_to_tile_rows(w, tile, lane);
    // Keys (magnitude bits, 63 - index) ordered as unsigned 64-bit integers - held as doubles: for positive,
    // normal, finite doubles the two orders are the same, and a compare-exchange is then one v_max_f64 and one
    // v_min_f64.  One is added to the exponent field so that a zero magnitude is a normal double, and NaNs share
    // a magnitude key just below where that addition would reach the doubles' own infinities and NaNs.
    double key[64];
#pragma unroll
    for (int e = 0; e < 64; ++e) {
        const uint32_t a = __builtin_bit_cast(uint32_t, w[e]) & 0x7fffffffu;
        const uint32_t mag = (a > 0x7f800000u ? 0x7fdfffffu : a) + 0x00100000u;
        key[e] = __builtin_bit_cast(double, (static_cast<uint64_t>(mag) << 32) | static_cast<uint32_t>(63 - e));
    }
    // bitonic sort, descending
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1) {
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
#pragma unroll
            for (int i = 0; i < 64; ++i) {
                const int l = i ^ stride;
                if (l > i) {
                    const bool up = (i & size) != 0 && size < 64;  // this run ascends
                    const double a = key[i], b = key[l];
                    const double hi = __builtin_fmax(a, b), lo = __builtin_fmin(a, b);
                    key[i] = up ? lo : hi;
                    key[l] = up ? hi : lo;
                }
            }
        }
    }
    wave_lds_fence();
    if (lane >= left) return;
    const int64_t row = d.chunk_begin + static_cast<int64_t>(grp) * 64 + lane;
    float* vrow = val + row * k;
    uint8_t* irow = idx12 + row * (k + (k >> 1));
    const float* mine = tile + lane * kLd;
#pragma unroll
    for (int j = 0; j < 64; j += 2) {
        if (j < k) {  // k is even
            const uint32_t i0 = 63u - static_cast<uint32_t>(__builtin_bit_cast(uint64_t, key[j]));
            const uint32_t i1 = 63u - static_cast<uint32_t>(__builtin_bit_cast(uint64_t, key[j + 1]));
            vrow[j] = mine[i0];
            vrow[j + 1] = mine[i1];
            const uint32_t pair = i0 | (i1 << 12);
            uint8_t* o = irow + 3 * (j >> 1);
            o[0] = static_cast<uint8_t>(pair);
            o[1] = static_cast<uint8_t>(pair >> 8);
            o[2] = static_cast<uint8_t>(pair >> 16);
        }
    }
}

// the wave's issue priority (0 .. 3; the instruction takes an immediate, hence the ladder); `level` is wave-uniform
__device__ __forceinline__ void set_wave_priority(int level) {
    if (level == 0) __builtin_amdgcn_s_setprio(0);
    else if (level == 1) __builtin_amdgcn_s_setprio(1);
    else if (level == 2) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(3);
}

// Persistent fused encode: every wave walks its slice of the chunk list.  The kernel is bound by
// vector-ALU issue and by the latencies between its phases, so it is shaped for residency -
// 8.5 KB + 1 KB of LDS and a register budget that admits three to four waves per SIMD - and
// leaves the overlap of one wave's row loads with the other waves' arithmetic to the hardware.
// The three waves of a SIMD pass its issue slots round: the arbiter alone serves the oldest wave first, so
// that the workgroups dispatched last run behind all the way and the launch waits for them.  Each wave
// therefore steps through the priority levels 0, 1, 2 chunk by chunk, the three dispatch layers of a full
// grid one step apart, and changes level once its rows are requested (4 % off the launch; the level
// values, the direction and a change at another phase or every other chunk matter less than 1 %).
// kEf: the miner's momentum update rides on the load (src/tplr/neurons.py:151-152): the chunk of
// the error-feedback tensor becomes ef * decay + grad (two roundings, as mul_ then add_), is
// written back in place and is what gets encoded.
// Without the transform the kernel waits more than it computes, and workgroups of two waves that take alternate
// chunks and meet at a barrier before they request their rows (512 contiguous bytes per row at the same moment) are
// 6 % faster; with the transform, where the vector ALU is the bound, any team is slower (8 % with four waves).
// kEf also writes every chunk back, and rows written together are served sooner: teams of four without the
// transform (8 % off the two-launch miner step against single waves), of two with it (4 %).
template <bool kUseDct, bool kEf = false>
constexpr int encode_team() { return kUseDct ? (kEf ? 2 : 1) : (kEf ? 4 : 2); }

template <bool kTwo, bool kUseDct, bool kEf = false>
__global__ __launch_bounds__((64 * encode_team<kUseDct, kEf>()), 3) void k_encode_topk_pack(const tplr_tensor_desc* __restrict__ table,
                                                            const tplr_tensor_desc single, int n_tensors,
                                                            int64_t total, int k, uint8_t* __restrict__ idx12,
                                                            float* __restrict__ val,
                                                            const tplr_tensor_desc* __restrict__ grad_table,
                                                            float decay) {
    constexpr int T = encode_team<kUseDct, kEf>();
    __shared__ __align__(16) float buf_all[T][kHalfFloats];
    __shared__ uint64_t cand_all[T][kCandCap];
    const int wv = T > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)) : 0;  // wave of the team
    float* const buf = buf_all[wv];
    uint64_t* const cand = cand_all[wv];
    const int lane = threadIdx.x & 63;
    int64_t g0, g1;
    my_range(total, g0, g1, T);
    if (g0 >= g1) return;
    // T > 1: [g0, g1) becomes this wave's share of the team's range, every T-th chunk; every wave of the team arrives
    // at `team_steps` barriers
    const int64_t team_steps = (g1 - g0 + T - 1) / T;
    g0 += wv;
    const int64_t my_steps = g0 < g1 ? (g1 - 1 - g0) / T + 1 : 0;
    if constexpr (T > 1) {
        if (my_steps == 0) {  // wave-uniform: a team with fewer chunks than waves
            for (int64_t i = 0; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
            return;
        }
    }
    Cursor c, cg;
    cursor_seek(c, table, single, n_tensors, g0);
    if (kEf) cursor_seek(cg, grad_table, single, n_tensors, g0);
#if TPLR_DCT_MATRIX_CORES
    float ca[16] = {};
    if (kUseDct) load_dct4_operand(ca, lane);
#endif
    int turn = static_cast<int>(blockIdx.x * 3u / gridDim.x);  // the dispatch layer of a full grid; wave-uniform
    for (int64_t g = g0; g < g1; g += T) {
        float v[64], w[64];
        if constexpr (T > 1) __builtin_amdgcn_s_barrier();  // the team asks for its rows together
        load_chunk_cols(v, c, lane);
        if (kEf) {
            load_chunk_cols(w, cg, lane);
#pragma unroll
            for (int r = 0; r < 64; ++r) {
                const float m = v[r] * decay;
                v[r] = m + w[r];
            }
            store_chunk_cols(v, (float*)c.base, c.ld, c.y, c.xc, lane);
            if (g + T < g1) {
#pragma unroll
                for (int s = 1; s <= T; ++s) cursor_next(cg, g + s);
            }
        }
        if (g + T < g1) {
#pragma unroll
            for (int s = 1; s <= T; ++s) cursor_next(c, g + s);
        }
        // Untransformed gradients often differ in scale from row to row or column to column;
        // the select's threshold statistic is then taken in both directions.  (Coefficients of
        // the transform are mixed across both and one direction is as good as two.)
        set_wave_priority(turn);
        turn = turn == 2 ? 0 : turn + 1;
        uint32_t c1 = 0, c2 = 0;
        if (!kUseDct) lane_stats<kTwo>(v, c1, c2);
#if TPLR_DCT_MATRIX_CORES
        if (kUseDct) dct64_fwd_matrix(v, ca);
        transpose_via_half(v, w, buf, lane);
        if (kUseDct) dct64_fwd_matrix(w, ca);
#else
        chunk_forward<kUseDct>(v, w, buf, lane);
#endif
        const Selected s =
            select_topk<kTwo, !kUseDct>(w, buf, cand, lane, k, kUseDct ? kDctPow2Scale : 1.0f, c1, c2);
        emit_selected<kTwo>(s, lane, k, g, idx12, val);
    }
    if constexpr (T > 1) {
        for (int64_t i = my_steps; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
    }
}

// Measurement aid: the memory side of the encode alone - the same grid, chunk ranges and row loads, nothing else
// (the 64 values of a lane are added up so that the loads are not dropped, and the sum never leaves the wave).
__global__ __launch_bounds__(64, 3) void k_calib_encode(const tplr_tensor_desc* __restrict__ table,
                                                        const tplr_tensor_desc single, int n_tensors, int64_t total,
                                                        float* __restrict__ sink) {
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    Cursor c;
    cursor_seek(c, table, single, n_tensors, g0);
    float s = 0.0f;
    for (int64_t g = g0; g < g1; ++g) {
        float v[64];
        load_chunk_cols(v, c, lane);
        if (g + 1 < g1) cursor_next(c, g + 1);
#pragma unroll
        for (int r = 0; r < 64; ++r) s += v[r];
    }
    if (__float_as_uint(s) == 0x7fedcba9u && sink) sink[0] = s;  // (a NaN pattern no sum produces)
}

// body(Index<0>{}) ... body(Index<N - 1>{}): a loop whose counter is a constant in the body, so that
// arrays indexed by it stay in registers whatever the optimiser thinks of unrolling
template <int I>
struct Index {
    static constexpr int value = I;
};
template <int N, typename Body>
__device__ __forceinline__ void static_for(Body&& body) {
    if constexpr (N > 0) {
        static_for<N - 1>(body);
        body(Index<N - 1>{});
    }
}

// =========================================================================================
// decode side
// =========================================================================================
struct PeerPtrs {
    const uint8_t* idx[TPLR_MAX_PEERS];
    const float* val[TPLR_MAX_PEERS];
};

__device__ __forceinline__ int tile_pos(uint32_t idx) { return (idx >> 6) * kLd + (idx & 63); }

// 12-bit index j of a packed row (byte pointer to the row start)
template <typename BytePtr>
__device__ __forceinline__ uint32_t load_idx12(BytePtr row, int j) {
    BytePtr b = row + 3 * (j >> 1) + (j & 1);
    const uint32_t w = b[0] | (static_cast<uint32_t>(b[1]) << 8);
    return (j & 1) ? (w >> 4) : (w & 0xfffu);
}

typedef uint16_t __attribute__((aligned(1))) unaligned_u16;
using gu16 = __attribute__((address_space(1))) unaligned_u16;
typedef uint32_t __attribute__((aligned(1))) unaligned_u32;
using gu32 = __attribute__((address_space(1))) unaligned_u32;

// The fast scatter adds one peer's entries with a plain read-add-write per wave instruction, which is
// only right when the instruction's destinations are distinct.  A top-k selection has no repeats,
// but payloads come from other machines: so the read is an exchange that leaves a marker in the
// slot until the sum is written back.  A lane that reads the marker has met another lane of its own
// instruction - a repeated index in that peer's row - and the chunk is done again on the exact
// path (exact_scatter in the kernel).  The marker is the largest bit pattern there is (a NaN), so a
// lane remembers having met it with one unsigned maximum per step; a slot otherwise holds zero or
// the result of an addition, which has these bits only if a peer sent that very NaN - and then
// the chunk merely takes the exact path for nothing.
constexpr uint32_t kClaimMark = 0xffffffffu;
constexpr int kMarkWords = 64;                       // one bit per chunk of a wave's range:
constexpr int kMaxChunksPerWave = kMarkWords * 32;   // the longest range a wave can keep marks for
__device__ __forceinline__ float tile_claim(float* slot) {
    return __builtin_bit_cast(float, __hip_atomic_exchange(reinterpret_cast<uint32_t*>(slot), kClaimMark,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT));
}
__device__ __forceinline__ uint32_t seen_mark(uint32_t seen, float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    return seen > b ? seen : b;
}

// Contribution counters, one per coefficient, packed into 32-bit words that LDS atomics update,
// every tile row in words of its own: 4 bits each when at most 15 peers can hit a coefficient
// (8 words per row, 2 KB), 5 bits up to 31 peers (6 per word, 11 words per row, 2.75 KB) - both
// leave room for 8 waves in the 160 KB of a CU - and 8 bits beyond (4 KB, 7 waves).
template <int kBits>
struct Counters {
    static constexpr int kPerWord = 32 / kBits;
    static constexpr int kRowWords = (kChunk + kPerWord - 1) / kPerWord;
    static constexpr int kWords = kChunk * kRowWords;
    static constexpr int kAlloc = (kWords + 255) / 256 * 256;  // cleared 16 bytes per lane at a time
    static constexpr uint32_t kMask = (1u << kBits) - 1u;
    // bits 1 .. kBits-1 of every field: set somewhere <=> that counter is at least 2
    static constexpr uint32_t kMulti = kBits == 4 ? 0xEEEEEEEEu : kBits == 5 ? 0x3DEF7BDEu : 0xFEFEFEFEu;
    __device__ static __forceinline__ uint32_t word(uint32_t e) {
        const uint32_t col = e & 63u;
        return (e >> 6) * kRowWords + (kBits == 5 ? (col * 43u) >> 8 : col / kPerWord);
    }
    __device__ static __forceinline__ uint32_t shift(uint32_t e) {
        const uint32_t col = e & 63u;
        return (kBits == 5 ? col - ((col * 43u) >> 8) * 6u : col % kPerWord) * kBits;
    }
};

// Persistent fused decode.  Per chunk, the peers' entries are accumulated in peer order into an
// LDS tile (sums) and a per-coefficient contribution count; coefficients with several
// contributions are divided by their count; the tile goes through the inverse 2-D DCT.
//
// Fast path (kUnits > 0: k <= 64 and at most kUnits peers): lane j handles entry j of every
// peer, so each address is a scalar base (peer pointer from the kernel arguments + chunk
// offset) plus one lane-constant offset and each clip factor is a scalar; the whole payload of
// a chunk sits in 2 * kUnits registers and is requested a whole transform pass before it is used.
// Generic path (kUnits == 0): any k and peer count, entries loaded where they are used.
// kSubtract (fast path with the transform only): the destination receives destination - result
// instead of the result (the error-feedback update of src/tplr/neurons.py:171); its rows are
// requested before the second pass and arrive during it (without the transform, codes through wide loads:
// requested when the chunk leaves the tile, before it is read out).  With `guard` (one int per tensor, zeroed by the
// caller) a chunk whose result holds a NaN or an infinity is not subtracted - its destination keeps its
// bits - and guard[tensor] becomes 1: the validator's check of the decoded gradient before
// p.data.sub_ (neurons/validator.py:3646-3660).
// kStrided (fast path): the peers' payloads are equally spaced in memory - peer p's index bytes at
// pp.idx[0] + p * stride_idx, its values at pp.val[0] + p * stride_val floats, as a staged window lays
// them out - so every payload address is scalar arithmetic on two base pointers instead of a pair of
// lane broadcasts per peer and chunk.
// kCodes (fast path without the transform): the peers' values arrive as the quantiser's codes, one byte
// each, for a quantiser of at most four bins (templar runs four): pp.val[p] points at bytes, `deq` holds the
// de-quantised value of every code, deq[(t * P + p) * 4 + c] = lookup + shift of tensor t as peer p sent them
// (src/tplr/compress.py:637-643), and a lane picks its entry's value among the four its peer's lane holds.
// A quarter of the value bytes, and the fp32 copy of the payload is never made.
// kWideK (kCodes with equally spaced payloads, k = kWideK = 32 or 64): a load instruction costs this kernel
// about as much as the bytes it brings (every load queues behind the stores of the compute unit's eight
// waves), so one instruction serves several peers: every lane takes four bytes of codes - lane l the codes
// 4 (l mod k/4) .. + 3 of the peer number l / (k/4) among the 256/k peers of that instruction - or the four
// twelve bytes at 12 m of an index row (m = l mod k/8: entries 8 m .. 8 m + 7, peer l / (k/8) of 512/k), and a
// lane fetches its own entry from the lane that holds it with lane permutes when the entry is scattered.
// 8 load instructions per chunk instead of 40 for 20 peers at k = 64, and two register sets of 15
// registers: the payload is requested two chunks ahead, as in the pipeline with the transform.
// kTeam (the pipeline with the transform): workgroups of kTeam waves.  A team owns a contiguous range of chunks and
// deals them out one by one - wave w takes chunks w, w + kTeam, w + 2 kTeam, ... of it - and meets at a barrier
// before every chunk's row stores, so that the team writes kTeam neighbouring chunks, rows of kTeam * 256
// contiguous bytes, at the same moment.  (Persistent waves on ranges of their own write each 2 KB of a tensor row in
// eight visits microseconds apart, and the memory system serves such stores at 5 TB/s where it takes 6-7 TB/s of
// stores that arrive together.)  Each wave keeps its own tile, counters and marks.
template <bool kUseDct, int kUnits, int kWideK = 0, bool kPlain = false>
constexpr int aggregate_team() {
    // the pipeline with the transform up to 16 units (with 24 there are no registers to spare), the one from codes,
    // and (kPlain: fp32 values, no subtraction) the fast path without the transform
    return ((kUseDct && kUnits > 0 && kUnits <= 16) || kWideK > 0 || (kPlain && !kUseDct && kUnits > 0)) ? 4 : 1;
}

template <bool kUseDct, int kUnits, int kCntBits, bool kSubtract = false, bool kStrided = false, bool kCodes = false,
          int kWideK = 0>
__global__ __launch_bounds__((64 * aggregate_team<kUseDct, kUnits, kWideK, !kCodes && !kSubtract>()), 2) void k_decode_aggregate(const PeerPtrs pp, const float* __restrict__ scale, int P,
                                                            int k, const tplr_tensor_desc* __restrict__ table,
                                                            const tplr_tensor_desc single, int n_tensors,
                                                            int64_t first, int64_t total, int reduce_mode,
                                                            int options, float* __restrict__ sumsq,
                                                            int64_t stride_idx, int64_t stride_val,
                                                            const float* __restrict__ deq,
                                                            int32_t* __restrict__ guard) {
    static_assert(!kCodes || (kUnits > 0 && !kUseDct), "codes are served by the fast path without the transform");
    static_assert(!(kCodes && kSubtract) || kWideK > 0, "the subtraction from codes: the wide-load pipeline only");
    static_assert(kWideK == 0 || (kCodes && kStrided && (kWideK == 32 || kWideK == 64)), "wide loads: codes, equally spaced payloads");
    // this launch covers the chunks first .. first + total - 1 of the batch
    // options: bit 0 = per-peer, per-chunk normalisation (generic instantiation); bit 1 = `sumsq` takes two
    // floats per chunk, the sum of squares of the result and the sum of its elements
    const bool normalise = (options & 1) != 0;
    const bool with_sum = (options & 2) != 0;
    // per-chunk statistics of the result in registers (v: a column per lane); a chunk that is to be done
    // again on the exact path writes them there
    auto chunk_stats = [&](const float (&v)[64], int64_t g, bool skip) {
        if (!sumsq) return;  // wave-uniform
        const int lane_ = threadIdx.x & 63;
        float ss = 0.f;
#pragma unroll
        for (int r = 0; r < 64; ++r) ss = __builtin_fmaf(v[r], v[r], ss);
        ss = wave_sum_f32(ss);
        if (with_sum) {
            float sm = 0.f;
#pragma unroll
            for (int r = 0; r < 64; ++r) sm += v[r];
            sm = wave_sum_f32(sm);
            if (lane_ == 0 && !skip) {
                sumsq[2 * g] = ss;
                sumsq[2 * g + 1] = sm;
            }
        } else if (lane_ == 0 && !skip) {
            sumsq[g] = ss;
        }
    };
    // kSubtract with a guard: true (wave-uniform) when the result in registers holds a NaN or an infinity, and
    // then the chunk's tensor is flagged; x * 0 is zero for every finite x and NaN otherwise
    auto guard_trips = [&](const float (&v)[64], int t) -> bool {
        if (!kSubtract || !guard) return false;  // wave-uniform
        float z = 0.f;
#pragma unroll
        for (int r = 0; r < 64; ++r) z = __builtin_fmaf(v[r], 0.0f, z);
        const bool bad = __ballot(z != z) != 0;
        if (bad && (threadIdx.x & 63) == 0) guard[t] = 1;
        return bad;
    };
    using Cnt = Counters<kCntBits>;
    // kPark: lanes and units without an entry scatter "coefficient 4096 + lane", which the address
    // arithmetic of real coefficients maps to 64 tile slots and 8 counter words past the chunk's own
    // (one select per step instead of three); 4-bit counters only: a row of them is 8 whole words
    constexpr bool kPark = kUnits > 0 && kUseDct && kCntBits == 4;
    constexpr int kTeam = aggregate_team<kUseDct, kUnits, kWideK, !kCodes && !kSubtract>();
    const int wv = kTeam > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)) : 0;  // wave of the team
    __shared__ __align__(16) float tile_all[kTeam][kTileFloats + (kPark ? 64 : 0)];
    __shared__ __align__(16) uint32_t cnt_all[kTeam][Cnt::kAlloc + (kPark ? 8 : 0)];
    float* const tile = tile_all[wv];
    uint32_t* const cnt = cnt_all[wv];
    // the marks live in the counters' rounding slack where there is enough of it (5-bit counters:
    // the kernel then still fits eight times into a compute unit's LDS), else in words of their own
    constexpr bool kMarksInSlack = Cnt::kAlloc - Cnt::kWords >= kMarkWords;
    __shared__ uint32_t own_marks[kTeam][kMarksInSlack ? 1 : kMarkWords];
    uint32_t* const marks = kMarksInSlack ? cnt + Cnt::kWords : own_marks[wv];
    constexpr bool kFast = kUnits > 0;
    constexpr int kRegs = kFast ? kUnits : 1;
    const int lane = threadIdx.x & 63;
    int64_t g0, g1;
    // (a team's range begins on a multiple of kTeam chunks of the batch: its waves' rows line up)
    my_range(total, g0, g1, kTeam, first);
    if (g0 >= g1) return;
    g0 += first;
    g1 += first;
    // kTeam > 1: [g0, g1) becomes this wave's share, every kTeam-th chunk from g0; `team_steps` is the longest
    // share of the team (every wave of it has to arrive at that many barriers)
    constexpr int T = kTeam;
    const int64_t team_steps = (g1 - g0 + T - 1) / T;
    g0 += wv;
    const int64_t my_steps = g0 < g1 ? (g1 - 1 - g0) / T + 1 : 0;
    if constexpr (kTeam > 1) {
        if (my_steps == 0) {  // wave-uniform: a team with fewer chunks than waves
            for (int64_t i = 0; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
            return;
        }
    }
    const int64_t g_last = g0 + (my_steps - 1) * T;  // this wave's last chunk

    const int64_t idx_stride = k + (k >> 1);
    // the inverse transform below is 32x the orthonormal one: its input carries the exact 2^-5
    const float out_scale = kUseDct ? kDctPow2Scale : 1.0f;
    const bool lane_on = lane < k;       // fast path: this lane owns an entry
    const int le = lane_on ? lane : 0;   // the other lanes reload entry 0 and stay out of the scatter
    const uint32_t lane_ioff = 3u * (static_cast<uint32_t>(le) >> 1) + (le & 1);  // byte offset of entry `le` in a packed row

    // Fast path: lane p keeps peer p's two payload pointers and its clip factor for the current
    // tensor in registers; unit i gets them as scalars through v_readlane, so that the steady
    // state of the loop contains no scalar memory load (whose wait would also drain the LDS queue).
    const int pl = lane < P ? lane : P - 1;
    const uint64_t my_idx = kFast ? reinterpret_cast<uint64_t>(pp.idx[pl]) : 0;
    const uint64_t my_val = kFast ? reinterpret_cast<uint64_t>(pp.val[pl]) : 0;
    float my_scale = out_scale;
    int t_scale = -1;  // tensor whose clip factors my_scale holds
    auto lane_bcast64 = [&](uint64_t mine, int i) -> uint64_t {
        const uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(mine)), i);
        const uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(mine >> 32)), i);
        return (static_cast<uint64_t>(hi) << 32) | lo;
    };

    uint32_t ix[kRegs];
    float a[kRegs];

    // clip factors of tensor t into my_scale (wave-uniform branch, taken once per tensor)
    float my_tab[kCodes ? 4 : 1] = {};  // (kCodes) lane p: peer p's four de-quantised values for that tensor, times my_scale
    auto load_scale = [&](int t) {
        if constexpr (kCodes) {
            if (t != t_scale) {
                my_scale = (scale ? scale[static_cast<int64_t>(t) * P + pl] : 1.0f) * out_scale;
                const float4 d4 = *reinterpret_cast<const float4*>(deq + (static_cast<int64_t>(t) * P + pl) * 4);
                my_tab[0] = d4.x * my_scale, my_tab[1] = d4.y * my_scale, my_tab[2] = d4.z * my_scale, my_tab[3] = d4.w * my_scale;
                t_scale = t;
            }
        } else if (scale && t != t_scale) {
            my_scale = scale[static_cast<int64_t>(t) * P + pl] * out_scale;
            t_scale = t;
        }
    };
    // (kCodes) the value of code c as unit i's peer sent it, times its clip factor
    auto code_value = [&](uint32_t c, int i) -> float {
        const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_tab[0]), i));
        const float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_tab[kCodes ? 1 : 0]), i));
        const float s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_tab[kCodes ? 2 : 0]), i));
        const float s3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_tab[kCodes ? 3 : 0]), i));
        const float r0 = (c & 1u) ? s1 : s0, r1 = (c & 1u) ? s3 : s2;
        return (c & 2u) ? r1 : r0;
    };
    // unit i's entries of chunk g into its two registers
    auto load_payload = [&](int64_t g, int t) {  // fast path only
        load_scale(t);
        // kStrided: peer after peer by scalar additions from chunk g's place in peer 0's payload
        const gbyte* irow = (const gbyte*)pp.idx[0] + uniform64(g * idx_stride);
        const gfloat* vrow = (const gfloat*)pp.val[0] + uniform64(g * k);
        const gbyte* crow = (const gbyte*)pp.val[0] + uniform64(g * k);  // (kCodes)
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            if constexpr (!kStrided) {
                const int u = i < P ? i : P - 1;  // unused units reload the last peer and stay out of the scatter
                irow = reinterpret_cast<const gbyte*>(lane_bcast64(my_idx, u)) + g * idx_stride;
                vrow = reinterpret_cast<const gfloat*>(lane_bcast64(my_val, u)) + g * k;
                crow = reinterpret_cast<const gbyte*>(lane_bcast64(my_val, u)) + g * k;
            }
            ix[i] = *(const gu16*)(irow + lane_ioff);
            if constexpr (kCodes)
                a[i] = __builtin_bit_cast(float, static_cast<uint32_t>(crow[le]));
            else
                a[i] = vrow[le];
            if (kStrided && i + 1 < P) {  // (unused units reload the last peer)
                irow += stride_idx;
                vrow += stride_val;
                crow += stride_val;  // (kCodes: the stride counts bytes)
            }
        }
    };
    // entry j of peer p of chunk g (generic path and normalise)
    auto load_entry = [&](int p, int j, int64_t g, uint32_t& ixo, float& ao) {
        const gbyte* irow = (const gbyte*)pp.idx[p] + g * idx_stride;
        const uint32_t w = *(const gu16*)(irow + (3 * (j >> 1) + (j & 1)));
        ixo = (j & 1) ? (w >> 4) : (w & 0xfffu);
        if constexpr (kCodes)  // (the caller turns the code into its value)
            ao = __builtin_bit_cast(float, static_cast<uint32_t>(((const gbyte*)pp.val[p] + g * k)[j]));
        else
            ao = ((const gfloat*)pp.val[p] + g * k)[j];
    };

    const bool fast = kFast;  // (normalise is served by the generic instantiation only)

    auto zero_tile = [&]() {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        float4* row = reinterpret_cast<float4*>(tile + lane * kLd);
#pragma unroll
        for (int q = 0; q < 16; ++q) row[q] = z;
        const uint4 zi = make_uint4(0, 0, 0, 0);
        static_assert(Cnt::kWords % 4 == 0, "counters are cleared 16 bytes at a time");
#pragma unroll
        for (int q = 0; q < Cnt::kAlloc / 256; ++q)
            if (q * 64 + lane < Cnt::kWords / 4) reinterpret_cast<uint4*>(cnt)[q * 64 + lane] = zi;
        wave_lds_fence();
    };

    // ---- scatter: sums in peer order and contribution counts.  One instruction carries one
    // peer's entries, whose destinations are distinct (a top-k selection has no duplicates), and
    // LDS instructions of a wave execute in order, so every destination receives its
    // contributions in peer order.  The fast path therefore needs no atomic for the sums; the
    // generic path keeps them.
    // `repeat` collects, per lane, whether the chunk being scattered has to be done again on the
    // exact path: a repeated index inside one wave instruction, or a counter about to wrap.
    uint32_t repeat = 0;  // kClaimMark <=> the chunk has to be done again
    // Chunks found that way are not stored; they are marked - bit i of `marks` for the i-th chunk of
    // the wave's range - and done again after the main loop.
    marks[lane] = 0;
    // The slots that lanes and units without an entry scatter to (a row's padding, the words past the tile) are never
    // cleared with the tile, and LDS keeps what the last kernel on this compute unit left there: a bit pattern that
    // reads as a claim mark would send every chunk to the exact path.
    *reinterpret_cast<float4*>(tile + lane * kLd + kChunk) = make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (kPark) tile[kTileFloats + lane] = 0.f;
    auto mark_redo = [&](int64_t g) {  // wave-uniform call, rare
        const int i = static_cast<int>((g - g0) / T);
        if (lane == 0) marks[i >> 5] |= 1u << (i & 31);
    };
    auto add_entry = [&](uint32_t ixe, float val) {
        // Generic path: atomics add every entry, but entries of one instruction that name the same
        // coefficient are added in the hardware's order, not in entry order, and the 8-bit counter
        // wraps at 256.  Another lane of this instruction has been here <=> the counter field this
        // lane's atomic returns differs from what a read before the instruction saw.
        uint32_t* cw = &cnt[Cnt::word(ixe)];
        const uint32_t sh = Cnt::shift(ixe);
        const uint32_t seen = *cw;
        atomicAdd(&tile[tile_pos(ixe)], val);
        const uint32_t was = atomicAdd(cw, 1u << sh);
        if ((((seen ^ was) >> sh) & Cnt::kMask) != 0u || ((was >> sh) & Cnt::kMask) == Cnt::kMask) repeat = kClaimMark;
    };
    // (unit_lo, unit_hi: the fast path's units to run, for a caller that threads them between other work)
    auto scatter = [&](int64_t g, int t_now, int unit_lo = 0, int unit_hi = 1 << 20) {
        if (fast) {
            if (lane_on) {
#pragma unroll
                for (int i = 0; i < kRegs; ++i) {
                    if (i >= unit_lo && i < unit_hi && i < P) {  // wave-uniform
                        const uint32_t e = (lane & 1) ? (ix[i] >> 4) : (ix[i] & 0xfffu);
                        const float x = kCodes ? code_value(__builtin_bit_cast(uint32_t, a[i]), i)
                                               : a[i] * __builtin_bit_cast(float, __builtin_amdgcn_readlane(
                                                            __builtin_bit_cast(int, my_scale), i));
                        // claim, add, write back: the floating-point LDS atomic costs about 3 cycles
                        // per lane, six times this sequence
                        float* t = &tile[tile_pos(e)];
                        const float cur = tile_claim(t);
                        repeat = seen_mark(repeat, cur);
                        *t = cur + x;
                        atomicAdd(&cnt[Cnt::word(e)], 1u << Cnt::shift(e));
                    }
                }
            }
        } else if (normalise) {
            // per-peer, per-chunk L2 normalisation (compress.py:541-545); simple, unbatched
            for (int p = 0; p < P; ++p) {
                const gfloat* vrow = (const gfloat*)pp.val[p] + g * k;
                float ss = 0.f;
                for (int j = lane; j < k; j += 64) ss += vrow[j] * vrow[j];
                const float nrm = __builtin_sqrtf(wave_sum_f32(ss)) + 1e-8f;
                for (int j = lane; j < k; j += 64) {
                    uint32_t ixe;
                    float ae;
                    load_entry(p, j, g, ixe, ae);
                    add_entry(ixe, (ae / nrm) * out_scale);
                }
            }
        } else {
            for (int p = 0; p < P; ++p) {
                const float s = scale ? scale[static_cast<int64_t>(t_now) * P + p] : 1.0f;
                for (int j = lane; j < k; j += 64) {
                    uint32_t ixe;
                    float ae;
                    load_entry(p, j, g, ixe, ae);
                    add_entry(ixe, (ae * s) * out_scale);
                }
            }
        }
    };

    // ---- mean: lane r scans the counters of row r and divides the coefficients that received
    // more than one contribution (a few per row), one per trip of a lane-divergent loop
    auto mean_pass = [&]() {
        wave_lds_fence();
        if (reduce_mode != TPLR_REDUCE_MEAN) return;
        constexpr int kRowWords = Cnt::kRowWords;
        constexpr uint32_t kMulti = Cnt::kMulti;
        const uint32_t* crow = cnt + lane * kRowWords;
        uint32_t todo = 0;  // bit q: word q of the row holds such a counter
#pragma unroll
        for (int q = 0; q < kRowWords; ++q) todo |= ((crow[q] & kMulti) ? 1u : 0u) << q;
        uint32_t word = 0, m = 0;
        int q = 0;
        while (todo | m) {
            if (m == 0) {
                q = __builtin_ctz(todo);
                todo &= todo - 1;
                word = crow[q];
                m = word & kMulti;
            }
            const int slot = __builtin_ctz(m) / kCntBits;
            const uint32_t n = (word >> (slot * kCntBits)) & Cnt::kMask;
            m &= ~(Cnt::kMask << (slot * kCntBits));
            float* t = &tile[lane * kLd + q * Cnt::kPerWord + slot];
            *t = *t / static_cast<float>(n);
        }
        wave_lds_fence();
    };

    // The same pass in pieces, for the pipeline with the transform: a chunk's 64 row stores are issued at the pace
    // the memory system takes them, and the wave would stand at them with nothing else to do - so the LDS round
    // trips of this pass (on the next chunk's tile) run between groups of those stores.  mean_begin scans the row's
    // counters, mean_trip divides one coefficient in every lane that still has one, mean_finish does the rest.
    struct MeanState {
        uint32_t todo, word, m;
        int q;
    };
    auto mean_begin = [&](MeanState& ms) {
        wave_lds_fence();
        ms.todo = 0, ms.word = 0, ms.m = 0, ms.q = 0;
        if (reduce_mode != TPLR_REDUCE_MEAN) return;
        const uint32_t* crow = cnt + lane * Cnt::kRowWords;
#pragma unroll
        for (int q = 0; q < Cnt::kRowWords; ++q) ms.todo |= ((crow[q] & Cnt::kMulti) ? 1u : 0u) << q;
    };
    auto mean_trip = [&](MeanState& ms) {
        if (ms.todo | ms.m) {
            if (ms.m == 0) {
                ms.q = __builtin_ctz(ms.todo);
                ms.todo &= ms.todo - 1;
                ms.word = cnt[lane * Cnt::kRowWords + ms.q];
                ms.m = ms.word & Cnt::kMulti;
            }
            const int slot = __builtin_ctz(ms.m) / kCntBits;
            const uint32_t n = (ms.word >> (slot * kCntBits)) & Cnt::kMask;
            ms.m &= ~(Cnt::kMask << (slot * kCntBits));
            float* t = &tile[lane * kLd + ms.q * Cnt::kPerWord + slot];
            *t = *t / static_cast<float>(n);
        }
    };
    auto mean_finish = [&](MeanState& ms) {
        while (ms.todo | ms.m) mean_trip(ms);
        wave_lds_fence();
    };

    // ---- exact path for a chunk with repeated indices inside one peer's row (no top-k produces
    // them; the reference sums every entry and divides by the number of entries,
    // src/tplr/compress.py:472-474).  Entries are added in source order - peer by peer, and inside
    // a peer in entry order, repeats one after the other - first the values, then, into the
    // cleared tile, 1.0 per entry, which counts any number of contributions exactly.  Leaves the
    // tile as the fast scatter and mean_pass would; needs 64 free registers.
    auto exact_scatter = [&](int64_t g, int t_now) {
        float sums[64];
#pragma unroll 1
        for (int phase = 0; phase < 2; ++phase) {
            {
                const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
                float4* row = reinterpret_cast<float4*>(tile + lane * kLd);
#pragma unroll
                for (int q = 0; q < 16; ++q) row[q] = z;
                wave_lds_fence();
            }
#pragma unroll 1
            for (int p = 0; p < P; ++p) {
                const gfloat* vrow = (const gfloat*)pp.val[p] + g * k;
                float nrm = 1.0f;
                if (normalise) {
                    float ss = 0.f;
                    for (int j = lane; j < k; j += 64) ss += vrow[j] * vrow[j];
                    nrm = __builtin_sqrtf(wave_sum_f32(ss)) + 1e-8f;
                }
                const float sc = scale ? scale[static_cast<int64_t>(t_now) * P + p] : 1.0f;
#pragma unroll 1
                for (int j0 = 0; j0 < k; j0 += 64) {
                    const int j = j0 + lane;
                    int me = -1;
                    float x = 0.f;
                    if (j < k) {
                        uint32_t ixe;
                        float ae;
                        load_entry(p, j, g, ixe, ae);
                        me = static_cast<int>(ixe);
                        if constexpr (kCodes)
                            ae = deq[(static_cast<int64_t>(t_now) * P + p) * 4 + (__builtin_bit_cast(uint32_t, ae) & 3u)];
                        // the value as the path this kernel was built for forms it
                        x = normalise ? (ae / nrm) * out_scale : fast ? ae * (sc * out_scale) : (ae * sc) * out_scale;
                        if (phase) x = 1.0f;
                    }
                    // rank among the earlier lanes that name the same coefficient; one rank per turn
                    int rank = 0;
                    for (int i = 0; i < 63; ++i) {
                        const int other = __shfl(me, i);
                        rank += (i < lane && other == me && me >= 0) ? 1 : 0;
                    }
                    const int turns = static_cast<int>(wave_max_u32(static_cast<uint32_t>(rank)));
                    for (int r = 0; r <= turns; ++r) {
                        if (me >= 0 && rank == r) {
                            float* t = &tile[tile_pos(static_cast<uint32_t>(me))];
                            *t = *t + x;
                        }
                        wave_lds_fence();
                    }
                }
            }
            if (phase == 0) tile_rows_to_regs(sums, tile, lane);
            wave_lds_fence();
        }
        // row `lane`: sums in registers, counts in the tile
        float* row = tile + lane * kLd;
#pragma unroll
        for (int d = 0; d < 64; ++d) {
            const float n = row[d];
            row[d] = (reduce_mode == TPLR_REDUCE_MEAN && n > 1.0f) ? sums[d] / n : sums[d];
        }
        wave_lds_fence();
    };

    // where a chunk's result goes
    // Without the transform the result is either the dense coefficient tensor (R/64, C/64, 64, 64)
    // (row stride 0 in the descriptor) or, with a row stride, the (R, C) tensor itself: decode
    // without a transform is a pure re-layout (src/tplr/compress.py:281).
    struct Out {
        gfloat* chunk0;
        int64_t ld;
        int t;  // the chunk's tensor: its clip factors
    };
    auto out_of = [&](const Cursor& cu, int64_t g) -> Out {
        return Out{(kUseDct || cu.ld > 0) ? cu.base + (cu.y * 64) * cu.ld + static_cast<int64_t>(cu.xc) * 64
                                          : cu.base + (g - cu.begin) * 4096,
                   cu.ld, cu.t};
    };

    // the cursor from chunk g - T, the wave's last one, to chunk g
    auto cursor_to = [&](Cursor& cu, int64_t g) {
#pragma unroll
        for (int s = T - 1; s >= 0; --s) cursor_next(cu, g - s);
    };

    // ---- the chunks marked for the exact path, one at a time, after the wave's main loop
    auto redo_chunk = [&](int64_t g) {
        Cursor cs;
        cursor_seek(cs, table, single, n_tensors, g);
        const Out o = out_of(cs, g);
        exact_scatter(g, cs.t);
        float v[64];
        gfloat* const dst = (gfloat*)uniform64(reinterpret_cast<int64_t>(o.chunk0));
        const int64_t ld = uniform64(o.ld);
        const bool rows = kUseDct || ld > 0;  // wave-uniform
        if (kUseDct) {
            chunk_inverse<true>(v, tile, lane);
        } else if (rows) {
            tile_cols_to_regs(v, tile, lane);
        } else {
#pragma unroll
            for (int q0 = 0; q0 < 16; ++q0) {
                const int q = q0 * 64 + lane;
                const float4 t = *reinterpret_cast<const float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2));
                v[4 * q0] = t.x, v[4 * q0 + 1] = t.y, v[4 * q0 + 2] = t.z, v[4 * q0 + 3] = t.w;
            }
        }
        wave_lds_fence();
        bool tripped = false;
        if constexpr (kSubtract) {
            chunk_stats(v, g, false);
            tripped = guard_trips(v, cs.t);
            const __amdgpu_buffer_rsrc_t rs = chunk_rsrc((const void*)dst, ld);
            const int ld4 = static_cast<int>(ld) * 4;
#pragma unroll
            for (int r = 0; r < 64; ++r)
                v[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, r * ld4, 0)) - v[r];
        } else {
            chunk_stats(v, g, false);
        }
        if (rows) {
            store_chunk_rows(v, (void*)dst, ld, lane, tripped);
        } else {
#pragma unroll
            for (int q0 = 0; q0 < 16; ++q0)
                reinterpret_cast<float4*>((float*)dst)[q0 * 64 + lane] =
                    make_float4(v[4 * q0], v[4 * q0 + 1], v[4 * q0 + 2], v[4 * q0 + 3]);
        }
    };
    auto redo_marked = [&]() {
        wave_lds_fence();
        const uint32_t mine = marks[lane];
        if (__ballot(mine != 0u) == 0) return;  // wave-uniform: nothing marked, the usual case
#pragma unroll 1
        for (int l = 0; l < kMarkWords; ++l) {
            uint32_t m = __builtin_amdgcn_readlane(static_cast<int>(mine), l);
#pragma unroll 1
            while (m) {
                redo_chunk(g0 + static_cast<int64_t>(l * 32 + __builtin_ctz(m)) * T);
                m &= m - 1;
            }
        }
    };

    // =====================================================================================
    // Fast path with the transform: four chunks in flight per wave.
    //   chunk g      second transform pass in registers, then 64 row stores
    //   chunk g + 1  scattered into the tile, threaded through that pass
    //   chunk g + 2  payload in the other register set, on its way or arrived
    //   chunk g + 3  payload requested into the registers the scatter has just released
    // The scatter is a chain of LDS round trips (read, add, write, one peer after the other: a
    // later peer may hit the same coefficient), far too slow to sit in the open.  Step s of it,
    // at one of the pass's call-outs, completes unit s - 1 (write back, reload its registers) and
    // starts unit s (read).  Everything in there is branch-free: lanes and units without an entry
    // work on a per-lane slot in the tile's padding, and past the end of the wave's range the
    // same (valid) data is scattered into a tile that nobody reads.
    // Payload loads queue behind every store of the compute unit's eight waves, which takes
    // about as long as one chunk; two chunks of distance keep the wave from waiting for them.
    // =====================================================================================
    if constexpr (kFast && kUseDct) {
        struct Set {  // one chunk's values
            float a[kRegs];
            float sc;  // lane p: clip factor of peer p for tensor t, times 2^-5
            int t;
        };
        Set s0, s1;
#pragma unroll
        for (int i = 0; i < kRegs; ++i) s0.a[i] = s1.a[i] = 0.f;
        s0.sc = s1.sc = out_scale;
        s0.t = s1.t = -1;
        auto set_scale = [&](Set& st, int t) {  // wave-uniform branch, taken once per tensor
            if (scale && t != st.t) {
                st.sc = scale[static_cast<int64_t>(t) * P + pl] * out_scale;
                st.t = t;
            }
        };
        // kStrided: `next_v` walks from peer to peer by scalar additions; set_walk puts it on a chunk's place
        // in peer 0's payload
        const gfloat* next_v = (const gfloat*)pp.val[0];
        // (the peer count as the walk sees it: a copy the optimiser cannot see through, renewed per chunk, or it
        // would keep "stride or 0" for every unit in scalar registers of its own across the loop, and spill them)
        int walk_peers = P;
        auto set_walk = [&](int64_t off_v) {
            next_v = (const gfloat*)pp.val[0] + off_v;
            asm volatile("" : "+s"(walk_peers));
        };
        auto set_load_unit = [&](Set& st, int i, int64_t g) {
            const gfloat* vrow = next_v;
            if constexpr (kStrided) {
                if (i + 1 < walk_peers) next_v += stride_val;  // (unused units reload the last peer and stay out of the scatter)
            } else {
                const int u = i < P ? i : P - 1;  // unused units reload the last peer and stay out of the scatter
                vrow = reinterpret_cast<const gfloat*>(lane_bcast64(my_val, u)) + g * k;
            }
            st.a[i] = __builtin_nontemporal_load(vrow + le);  // streaming: 7 % faster than cached here
        };
        // The packed indices come in once per group of G of the wave's chunks instead of once per chunk.  A chunk's
        // index row is 1.5 k bytes, so neighbouring rows share 128-byte lines, and a streaming load per chunk
        // fetches those lines from memory again and again (3.3 x the index bytes at k = 32).  Here the lanes
        // c k/2 .. (c + 1) k/2 - 1 take the row of the group's chunk c, four bytes at 3 (l mod k/2) each - two
        // entries and a byte of the next pair - with one load per peer and group, and entry j of the group's chunk c
        // is fetched from lane (c k + j) / 2 with a lane permute when it is scattered.  The wave's chunks are T
        // apart, so the group's rows are T rows apart; the rows between them are those of the team's other waves,
        // which ask for them at the same moment.  `cur` is the group being scattered, `nxt` the one on its way:
        // requested two chunks before its first use and moved to `cur` at that use.  A lane whose four bytes would
        // end past the rows this launch may read starts one byte earlier and shifts that byte out on arrival.
        const int G = k <= 32 ? 4 : 2;
        const int64_t piece_end = first + total;
        const int64_t idx_end = piece_end * idx_stride;  // bytes of a peer's index rows that this launch may read
        uint32_t cur[kRegs], nxt[kRegs];
        uint32_t nxt_fix = 0;  // bits to shift out of `nxt` when it becomes `cur`
        const bool tiny = idx_end < 4;  // one row of two entries is all there is: three bytes
        // where this lane's four bytes begin, counted from the group's first row (lanes past the group's last pair
        // repeat it)
        int lane_goff;
        {
            const int half_k = k >> 1;
            int c = lane / half_k, q = lane - c * half_k;
            if (c >= G) c = G - 1, q = half_k - 1;
            lane_goff = c * T * static_cast<int>(idx_stride) + 3 * q;
        }
        auto group_load = [&](uint32_t (&dst)[kRegs], int64_t gs, auto first_call) -> uint32_t {
            if (gs >= piece_end) gs = piece_end - 1;  // (a group nobody will scatter)
            // the last pair of the last row starts at idx_end - 3: that lane reads the last four bytes instead, and
            // so does every lane whose row lies past the end (a group's later chunks when the range ends inside it)
            const int64_t want = gs * idx_stride + lane_goff;
            const int64_t from = want < idx_end - 4 ? want : idx_end - 4;
            const uint32_t fix = want == idx_end - 3 ? 8u : 0u;
            const gbyte* grow = (const gbyte*)pp.idx[0];
            if constexpr (kStrided) asm volatile("" : "+s"(walk_peers));
            if constexpr (decltype(first_call)::value) {
                // (k = 2 makes groups of four rows and a launch of one row has one chunk: no other call is reached)
                if (tiny) {
#pragma unroll
                    for (int i = 0; i < kRegs; ++i) {
                        const gbyte* row = (const gbyte*)pp.idx[i < P ? i : P - 1];
                        dst[i] = row[0] | (static_cast<uint32_t>(row[1]) << 8) | (static_cast<uint32_t>(row[2]) << 16);
                    }
                    return 0;
                }
            }
#pragma unroll
            for (int i = 0; i < kRegs; ++i) {
                if constexpr (!kStrided) {
                    const int u = i < P ? i : P - 1;
                    grow = reinterpret_cast<const gbyte*>(lane_bcast64(my_idx, u));
                }
                // (a team's other waves read the rest of these lines at the same moment: cached, not streaming)
                if constexpr (kTeam > 1)
                    dst[i] = *(const gu32*)(grow + from);
                else
                    dst[i] = __builtin_nontemporal_load((const gu32*)(grow + from));
                if constexpr (kStrided) {
                    if (i + 1 < walk_peers) grow += stride_idx;
                }
            }
            return fix;
        };
        // entry `le` of the group's chunk c sits in lane (c k + le) / 2, in its bits 0-11 or 12-23
        const uint32_t pair_shift = (le & 1) * 12;
        const uint32_t pair_lane4 = (static_cast<uint32_t>(le) >> 1) << 2;
        auto group_entry = [&](uint32_t held, uint32_t from4) -> uint32_t {
            return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>(from4), static_cast<int>(held)));
        };
        auto set_load = [&](Set& st, int64_t g, int t) {
            set_scale(st, t);
            if constexpr (kStrided) set_walk(uniform64(g * k));
#pragma unroll
            for (int i = 0; i < kRegs; ++i) set_load_unit(st, i, g);
        };
        auto unit_scale = [&](float sc, int u) {
            return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sc), u));
        };

        Cursor c;
        cursor_seek(c, table, single, n_tensors, g0);
        Out o0 = out_of(c, g0), o1 = o0, o2 = o0;  // destinations of chunks g, g + 1, g + 2
        // the first chunk: plain serial scatter
        set_load(s0, g0, c.t);
        {
            const uint32_t fix = group_load(cur, g0, std::true_type{});
#pragma unroll
            for (int i = 0; i < kRegs; ++i) cur[i] >>= fix;
            if (G == 2) nxt_fix = group_load(nxt, g0 + 2 * T, std::false_type{});
        }
        zero_tile();
        {
#pragma unroll
            for (int i = 0; i < kRegs; ++i) {
                if (i < P) {  // wave-uniform
                    // (every lane takes part in the permute, also those without an entry)
                    const uint32_t e = __builtin_amdgcn_ubfe(group_entry(cur[i], pair_lane4), pair_shift, 12);
                    if (!lane_on) continue;
                    float* t = &tile[tile_pos(e)];
                    const float was = tile_claim(t);
                    repeat = seen_mark(repeat, was);
                    *t = was + s0.a[i] * unit_scale(s0.sc, i);
                    atomicAdd(&cnt[Cnt::word(e)], 1u << Cnt::shift(e));
                }
            }
        }
        bool skip0 = __ballot(repeat == kClaimMark) != 0;  // chunk g: found to hold a repeated index, not stored
        if (skip0) mark_redo(g0);
        repeat = 0;
        mean_pass();
        if (g0 + T < g1) {
            cursor_to(c, g0 + T);
            o1 = out_of(c, g0 + T);
            set_load(s1, g0 + T, c.t);
        }
        if (g0 + 2 * T < g1) {
            cursor_to(c, g0 + 2 * T);
            o2 = out_of(c, g0 + 2 * T);
            set_load(s0, g0 + 2 * T, c.t);
        }
        {
            // The memory counter completes in order, and the compiler sizes every wait for the
            // worse of the ways into the loop.  From the back edge, payload loads are followed by
            // the 64 row stores of a chunk, so a wait for a load needs few of the stores behind it;
            // coming from here there would be no stores, every wait would shrink to "all but the
            // loads behind me", and on the back edge that means "all stores drained".  Give this
            // entry the same shape with 64 stores that write nothing: their descriptor has a
            // range of zero bytes, so the bounds check of the buffer instruction drops them.
            // (Real stores to the first chunk's rows would not do: two stores of one wave to one
            // address were seen to land in either order.)
            const __amdgpu_buffer_rsrc_t nowhere =
                __builtin_amdgcn_make_buffer_rsrc((void*)o0.chunk0, 0, 0, 0x00020000);
#pragma unroll
            for (int r = 0; r < 64; ++r) __builtin_amdgcn_raw_buffer_store_b32(0, nowhere, lane * 4, r * 256, 2);
        }

        // (kStrided) where the chunk loaded last sits in a payload; the loop's loads advance chunk by chunk
        const int64_t loaded_last = g0 + 2 * T < g1 ? g0 + 2 * T : g_last;
        int64_t last_v = uniform64(loaded_last * k);
        const int dummy_pos = kPark ? kTileFloats + lane : lane * kLd + kChunk;
        const uint32_t park = 4096u + lane;  // (kPark) maps to tile[kTileFloats + lane] and cnt[512 + lane / 8]
        // one chunk: `st` holds chunk g + 1 and is refilled with chunk g + 3
        // The two waves that share a SIMD are served oldest first, and on that rule alone the wave of the later
        // workgroup layer falls behind and finishes last.  The waves take turns instead: on every other chunk a
        // wave runs two priority levels up, on opposite chunks in the two layers.  A wave changes level where its
        // own chunk begins, so the turns overlap; one more level while it stores settles those overlaps for the
        // wave that is about to finish a chunk.  (Measured on fifteen peers: 3 % off the launch; raising other
        // phases, other hand-over points or a permanent edge for the late layer gain less or nothing.)
        // (a full grid is two layers of one workgroup per SIMD; on a smaller grid the halves need not share SIMDs,
        // and two waves that happen to hold the same turn are simply served oldest first again)
        const bool late_layer = blockIdx.x * 2 >= gridDim.x;  // wave-uniform
        auto step = [&](int64_t g, Set& st, auto odd) {
            const int turn = decltype(odd)::value != late_layer ? 2 : 0;
            uint32_t from4 = 0;  // four times the lane that holds this lane's entry of chunk g + 1
            {
                const int j = static_cast<int>((g - g0) / T);  // the chunk scattered below is number j + 1 of the wave's
                if constexpr (decltype(odd)::value) {
                    // groups begin at odd steps: G = 4 alternates "request" and "take over", G = 2 does both
                    if (G == 2 || (j & 2)) {
#pragma unroll
                        for (int i = 0; i < kRegs; ++i) cur[i] = nxt[i] >> nxt_fix;
                    }
                    if (G == 2 || !(j & 2))
                        nxt_fix = group_load(nxt, g0 + static_cast<int64_t>((j + 3) & ~(G - 1)) * T, std::false_type{});
                }
                from4 = pair_lane4 + static_cast<uint32_t>(((j + 1) & (G - 1)) * 2 * k);
            }
            float v[64];
            set_wave_priority(turn);  // (the payload requests above still go out at the last chunk's level)
            tile_rows_to_regs(v, tile, lane);
            dct64_inv(v);  // along d: v[l] = sum_d Y[lane][d] F[l][d]
            wave_lds_fence();
            regs_to_tile_rows(v, tile, lane);
            wave_lds_fence();
            tile_cols_to_regs(v, tile, lane);
            wave_lds_fence();

            zero_tile();
            const float sc_now = st.sc;
            const bool more3 = g + 3 * T < g1;
            Out o3 = o2;
            if (more3) {
                cursor_to(c, g + 3 * T);
                o3 = out_of(c, g + 3 * T);
                set_scale(st, c.t);
            }
            const int64_t g_load = more3 ? g + 3 * T : g_last;
            if constexpr (kStrided) {
                if (more3) last_v += T * k;
                set_walk(last_v);
            }
            constexpr int kSteps = kUnits + 1;
            constexpr int kAlways = kUnits > 8 ? kUnits - 8 : 1;  // units every served peer count uses
            int pos = kPark ? dummy_pos * 4 : dummy_pos;  // (kPark: a byte offset)
            float cur_sum = 0.f, add = 0.f;
            // units this lane scatters: a per-lane count compared per unit (a mask per unit, kept across the
            // loop, would take sixteen scalar registers that are not there)
            int my_units = lane_on ? P : 0;
            asm volatile("" : "+v"(my_units));
            // the register with the next unit's entry, on its way from another lane
            uint32_t held = group_entry(cur[0], from4);
            // kSubtract: the destination's rows are requested here and arrive during the pass where the
            // registers for that exist (up to 8 peers' payload in flight); with more peers they are fetched
            // after the pass, sixteen rows at a time, two such groups in flight (kLateRows)
            constexpr bool kLateRows = kSubtract && kUnits > 8;
            float before[kSubtract && !kLateRows ? 64 : 1];
            if constexpr (kSubtract && !kLateRows)
                load_chunk_rows(before, (const void*)uniform64(reinterpret_cast<int64_t>(o0.chunk0)), uniform64(o0.ld), lane);
            // along b: v[k] = sum_b Z[b][lane] F[k][b]
            dct64_inv_hooked(v, [&](auto tag) {
                constexpr int h = decltype(tag)::value;
                // step s runs at call-out (s * kDctHooks) / kSteps
                constexpr int s = (h * kSteps + kDctHooks - 1) / kDctHooks;
                if constexpr (s < kSteps && (s * kDctHooks) / kSteps == h) {
                    if constexpr (s > 0) {
                        repeat = seen_mark(repeat, cur_sum);
                        if constexpr (kPark)
                            *reinterpret_cast<float*>(reinterpret_cast<char*>(tile) + pos) = cur_sum + add;
                        else
                            tile[pos] = cur_sum + add;
                        set_load_unit(st, s - 1, g_load);
                    }
                    if constexpr (s < kUnits) {
                        constexpr int u = s;
                        const bool on = u < kAlways ? lane_on : u < my_units;
                        add = st.a[u] * unit_scale(sc_now, u);
                        const uint32_t packed = __builtin_amdgcn_ubfe(held, pair_shift, 12);
                        if constexpr (kPark) {
                            // byte addresses by hand: slot 4 e + 16 (e >> 6), counter word 4 (e >> 3), its
                            // field 4 (e & 7) bits up - seven instructions from the packed index
                            const uint32_t e = on ? packed : park;
                            const uint32_t e4 = e << 2;
                            pos = static_cast<int>(e4 + ((e >> 2) & 0x7f0u));
                            cur_sum = tile_claim(reinterpret_cast<float*>(reinterpret_cast<char*>(tile) + pos));
                            atomicAdd(reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(cnt) + ((e >> 1) & 0xffcu)),
                                      1u << (e4 & 28u));
                        } else {
                            const uint32_t e = packed;
                            pos = on ? static_cast<int>(e + ((e >> 6) << 2)) : dummy_pos;
                            cur_sum = tile_claim(&tile[pos]);
                            atomicAdd(&cnt[on ? Cnt::word(e) : lane], on ? 1u << Cnt::shift(e) : 0u);
                        }
                        if constexpr (s + 1 < kUnits) held = group_entry(cur[s + 1], from4);
                    }
                }
            });
            bool tripped = false;
            // (kSubtract: the statistics are those of the decoded values, not of the difference)
            if constexpr (kSubtract) chunk_stats(v, g, skip0);
            if constexpr (kSubtract) {
                // (a chunk that is to be done again on the exact path holds claim marks: it is tested there)
                if (!skip0) tripped = guard_trips(v, o0.t);
                if constexpr (!kLateRows) {
#pragma unroll
                    for (int r = 0; r < 64; ++r) v[r] = before[r] - v[r];
                }
            }
            if constexpr (!kSubtract) chunk_stats(v, g, skip0);
            // (the loop-carried destination may have been parked in vector registers: make it
            // scalar again, or every store becomes a loop over distinct descriptors)
            const bool skip1 = g + T < g1 && __ballot(repeat == kClaimMark) != 0;  // wave-uniform, false for top-k payloads
            if (skip1) mark_redo(g + T);
            repeat = 0;
            // the team stores together (a bare barrier: nothing is handed over, no memory operation is waited for)
            if constexpr (kTeam > 1) __builtin_amdgcn_s_barrier();
            // the mean of the next chunk's tile, its trips between the groups of this chunk's stores
            set_wave_priority(turn + 1);
            MeanState ms;
            mean_begin(ms);
            // a chunk that is to be done again is not stored: its descriptor gets a range of zero bytes
            if constexpr (kLateRows) {
                void* chunk0 = (void*)uniform64(reinterpret_cast<int64_t>(o0.chunk0));
                const int64_t ld0 = uniform64(o0.ld);
                const __amdgpu_buffer_rsrc_t rd = chunk_rsrc(chunk0, ld0);
                const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
                    chunk0, 0, (skip0 || tripped) ? 0 : static_cast<int>((63 * ld0 + 64) * 4), 0x00020000);
                const int ld4 = static_cast<int>(ld0) * 4;
                float b[2][16];
                auto fetch = [&](auto qt) {
                    constexpr int q = decltype(qt)::value;
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        b[q & 1][i] = __builtin_bit_cast(
                            float, __builtin_amdgcn_raw_buffer_load_b32(rd, lane * 4, (q * 16 + i) * ld4, 0));
                };
                fetch(Index<0>{});
                fetch(Index<1>{});
                static_for<4>([&](auto qt) {
                    constexpr int q = decltype(qt)::value;
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, b[q & 1][i] - v[q * 16 + i]), wr,
                                                              lane * 4, (q * 16 + i) * ld4, 2);
                    if constexpr (q + 2 < 4) fetch(Index<q + 2>{});
                    mean_trip(ms);
                });
            } else {
                const int64_t ld0 = uniform64(o0.ld);
                const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)uniform64(reinterpret_cast<int64_t>(o0.chunk0)), 0,
                    (skip0 || tripped) ? 0 : static_cast<int>((63 * ld0 + 64) * 4), 0x00020000);
                const int ld4 = static_cast<int>(ld0) * 4;
                // (sixteen groups of four: 1.2 % faster than eight of eight in teams; thirty-two of two 13 % slower)
                static_for<16>([&](auto qt) {
                    constexpr int q = decltype(qt)::value;
#pragma unroll
                    for (int r = q * 4; r < (q + 1) * 4; ++r)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v[r]), wr, lane * 4, r * ld4, 2);
                    mean_trip(ms);
                });
            }
            mean_finish(ms);
            skip0 = skip1;
            o0 = o1;
            o1 = o2;
            o2 = o3;
        };
        for (int64_t g = g0; g < g1; g += 2 * T) {
            step(g, s1, std::false_type{});
            if (g + T < g1) step(g + T, s0, std::true_type{});
        }
        if constexpr (kTeam > 1) {
            for (int64_t i = my_steps; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
        }
        redo_marked();
        return;
    }

    // =====================================================================================
    // Codes through wide loads (kWideK): four chunks in flight.  Chunk g leaves the tile for registers
    // and is stored; chunk g + 1 is scattered into the tile; chunk g + 2's payload sits in the other
    // register set; chunk g + 3's is requested into the registers the scatter has just released.
    // =====================================================================================
    if constexpr (kWideK > 0) {
        constexpr int kPc = 256 / kWideK;                     // peers per register of codes
        constexpr int kPi = 512 / kWideK;                     // peers per load of packed indices (twelve bytes a lane)
        constexpr int kCodeRegs = (kUnits + kPc - 1) / kPc;
        constexpr int kIdxRegs = (kUnits + kPi - 1) / kPi;
        constexpr int kLc = kWideK / 4, kLi = kWideK / 8;     // lanes per peer in either kind of load
        struct WSet {  // one chunk's payload
            uint32_t cw[kCodeRegs];
            uint32_t iw[kIdxRegs][3];
            float tab[4];  // lane p: peer p's four de-quantised values for tensor t, times its clip factor
            int t;
        };
        WSet s0, s1;
        s0.t = s1.t = -1;
        s0.tab[0] = s0.tab[1] = s0.tab[2] = s0.tab[3] = 0.f;
        s1.tab[0] = s1.tab[1] = s1.tab[2] = s1.tab[3] = 0.f;
        // what this lane fetches: codes 4 mc .. 4 mc + 3 of peer (load * kPc + lane / kLc), the twelve bytes at
        // 12 mi of peer (load * kPi + lane / kLi)'s index row: its entries 8 mi .. 8 mi + 7
        const int pc_l = lane / kLc, mc = lane - pc_l * kLc;
        const int pi_l = lane / kLi, mi = lane - pi_l * kLi;
        const int ioff = 12 * mi;
        // what this lane scatters: entry `lane` of every unit, found at lane (unit mod kPc) * kLc + lane / 4 of the
        // unit's code register, byte lane mod 4, and in the three index registers of lane (unit mod kPi) * kLi +
        // lane / 8, twelve bits from bit 12 (lane mod 8) of their 96
        const gbyte* const idx0 = (const gbyte*)pp.idx[0];
        const gbyte* const val0 = (const gbyte*)pp.val[0];
        // where each register's four bytes lie from the chunk's place in peer 0's payload (the host has
        // checked that the payloads of all peers span less than 4 GB)
        uint32_t coff[kCodeRegs], ioff_r[kIdxRegs];
#pragma unroll
        for (int r = 0; r < kCodeRegs; ++r) {
            int p = r * kPc + pc_l;
            p = p < P ? p : P - 1;  // (lanes past the last peer reload it)
            coff[r] = static_cast<uint32_t>(p) * static_cast<uint32_t>(stride_val) + 4u * mc;
        }
#pragma unroll
        for (int r = 0; r < kIdxRegs; ++r) {
            int p = r * kPi + pi_l;
            p = p < P ? p : P - 1;
            ioff_r[r] = static_cast<uint32_t>(p) * static_cast<uint32_t>(stride_idx) + static_cast<uint32_t>(ioff);
        }
        constexpr bool kAllOn = kWideK == 64;  // every lane owns an entry
        const int dummy_pos = lane * kLd + kChunk;  // lanes without an entry work on a slot of their own in the tile's padding
        if constexpr (!kAllOn) {
            tile[dummy_pos] = 0.f;
            wave_lds_fence();
        }
        typedef uint32_t v3u __attribute__((ext_vector_type(3), aligned(4)));
        auto wset_load = [&](WSet& st, int64_t g, int t) {
            if (t != st.t) {  // wave-uniform, once per tensor
                const float sc = (scale ? scale[static_cast<int64_t>(t) * P + pl] : 1.0f) * out_scale;
                const float4 d4 = *reinterpret_cast<const float4*>(deq + (static_cast<int64_t>(t) * P + pl) * 4);
                st.tab[0] = d4.x * sc, st.tab[1] = d4.y * sc, st.tab[2] = d4.z * sc, st.tab[3] = d4.w * sc;
                st.t = t;
            }
            const gbyte* crow = val0 + uniform64(g * kWideK);
            const gbyte* irow = idx0 + uniform64(g * (kWideK + kWideK / 2));
            // (the peer count as this call sees it: a copy the optimiser cannot see through, or it keeps one
            // comparison per register and unit in scalar registers of their own across the chunk loop, and spills them)
            int Pq = P;
            asm volatile("" : "+s"(Pq));
#pragma unroll
            for (int r = 0; r < kCodeRegs; ++r)
                if (r * kPc < Pq)  // wave-uniform
                    st.cw[r] = *(const __attribute__((address_space(1))) uint32_t*)(crow + static_cast<uint64_t>(coff[r]));
#pragma unroll
            for (int r = 0; r < kIdxRegs; ++r)
                if (r * kPi < Pq)  // wave-uniform
                {
                    const v3u w = *(const __attribute__((address_space(1))) v3u*)(irow + static_cast<uint64_t>(ioff_r[r]));
                    st.iw[r][0] = w.x, st.iw[r][1] = w.y, st.iw[r][2] = w.z;
                }
        };
        auto lane_of = [&](float mine, int i) {
            return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), i));
        };
        auto from_lane = [&](uint32_t held, uint32_t from4) {
            return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>(from4), static_cast<int>(held)));
        };
        auto wset_scatter = [&](const WSet& st) {
            // (formed here from a copy of the lane id the optimiser cannot see through: hoisted out of the chunk loop,
            // these and the per-unit permute addresses derived from them would take fifty registers)
            int l2 = le;
            asm volatile("" : "+v"(l2));
            int Pq = P;
            asm volatile("" : "+s"(Pq));
            const uint32_t code_from4 = static_cast<uint32_t>(l2 >> 2) << 2, code_shift = (l2 & 3) * 8;
            const uint32_t idx_from4 = static_cast<uint32_t>(l2 >> 3) << 2;
            // the entry's twelve bits inside two of the three registers: (0, 1) for entries 0-2 of the eight,
            // (1, 2) for 3-5, (2, 2) for 6-7, shifted by less than 32
            const int e8 = l2 & 7;
            const bool first3 = e8 < 3, last2 = e8 >= 6;
            const uint32_t idx_shift = static_cast<uint32_t>(12 * e8 - (first3 ? 0 : last2 ? 64 : 32));
#pragma unroll
            for (int i = 0; i < kUnits; ++i) {
                if (i < Pq) {  // wave-uniform
                    // (every lane takes part in the permutes, also those without an entry)
                    const uint32_t cbits = from_lane(st.cw[i / kPc], code_from4 + (i % kPc) * kLc * 4);
                    const uint32_t w0 = from_lane(st.iw[i / kPi][0], idx_from4 + (i % kPi) * kLi * 4);
                    const uint32_t w1 = from_lane(st.iw[i / kPi][1], idx_from4 + (i % kPi) * kLi * 4);
                    const uint32_t w2 = from_lane(st.iw[i / kPi][2], idx_from4 + (i % kPi) * kLi * 4);
                    const uint32_t ilo = first3 ? w0 : last2 ? w2 : w1, ihi = first3 ? w1 : w2;
                    const float q0 = lane_of(st.tab[0], i), q1 = lane_of(st.tab[1], i);
                    const float q2 = lane_of(st.tab[2], i), q3 = lane_of(st.tab[3], i);
                    const uint32_t cde = cbits >> code_shift;
                    const uint32_t e = __builtin_amdgcn_alignbit(ihi, ilo, idx_shift) & 0xfffu;
                    const float r0 = (cde & 1u) ? q1 : q0, r1 = (cde & 1u) ? q3 : q2;
                    const float xv = (cde & 2u) ? r1 : r0;
                    // branch-free: a lane without an entry adds zero to its own slot and nothing to a counter
                    const bool on = kAllOn || lane_on;
                    const float x = on ? xv : 0.f;
                    float* t = &tile[on ? tile_pos(e) : dummy_pos];
                    const float cur = tile_claim(t);
                    repeat = seen_mark(repeat, cur);
                    *t = cur + x;
                    atomicAdd(&cnt[on ? Cnt::word(e) : static_cast<uint32_t>(lane)], on ? 1u << Cnt::shift(e) : 0u);
                }
            }
        };
        Cursor c;
        cursor_seek(c, table, single, n_tensors, g0);
        Out out_cur = out_of(c, g0), out_next = out_cur, out_after = out_cur;
        wset_load(s0, g0, c.t);
        zero_tile();
        wset_scatter(s0);
        bool skip_cur = __ballot(repeat == kClaimMark) != 0;  // chunk g: found to hold a repeated index, not stored
        if (skip_cur) mark_redo(g0);
        repeat = 0;
        mean_pass();
        if (g0 + T < g1) {
            cursor_to(c, g0 + T);
            out_next = out_of(c, g0 + T);
            wset_load(s1, g0 + T, c.t);
        }
        if (g0 + 2 * T < g1) {
            cursor_to(c, g0 + 2 * T);
            out_after = out_of(c, g0 + 2 * T);
            wset_load(s0, g0 + 2 * T, c.t);
        }
        // (the chunks of a wave are T apart: g + 1 below stands for the wave's next chunk)
        // one chunk: `st` holds chunk g + 1 and is refilled with chunk g + 3.  Chunk g is stored as soon as it has
        // left the tile, so that its 64 registers are free while the next chunk is scattered
        const bool late_layer = blockIdx.x * 2 >= gridDim.x;  // wave-uniform
        auto step = [&](int64_t g, WSet& st, bool odd) {
            const int turn = odd != late_layer ? 2 : 0;
            set_wave_priority(turn);  // the two waves of a SIMD take turns, as above
            {
                // (tile and destination addresses are formed per chunk from an opaque copy of the lane id: hoisted
                // out of the loop they take a hundred registers)
                int lane = threadIdx.x & 63;
                asm volatile("" : "+v"(lane));
                float v[64];
                gfloat* const dst = (gfloat*)uniform64(reinterpret_cast<int64_t>(out_cur.chunk0));
                // kSubtract: the destination is a (R, C) tensor; its rows are requested first and arrive while
                // the tile is read out
                float before[kSubtract ? 64 : 1];
                if constexpr (kSubtract) load_chunk_rows(before, (const void*)dst, uniform64(out_cur.ld), lane);
                if (kSubtract || out_cur.ld > 0) {  // wave-uniform
                    tile_cols_to_regs(v, tile, lane);
                } else {
#pragma unroll
                    for (int q0 = 0; q0 < 16; ++q0) {
                        const int q = q0 * 64 + lane;
                        const float4 t = *reinterpret_cast<const float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2));
                        v[4 * q0] = t.x, v[4 * q0 + 1] = t.y, v[4 * q0 + 2] = t.z, v[4 * q0 + 3] = t.w;
                    }
                }
                wave_lds_fence();
                chunk_stats(v, g, skip_cur);
                bool tripped = false;
                if constexpr (kSubtract) {
                    if (!skip_cur) tripped = guard_trips(v, out_cur.t);
#pragma unroll
                    for (int r = 0; r < 64; ++r) v[r] = before[r] - v[r];
                }
                // the team stores together, one priority level up (as in the pipeline with the transform)
                if constexpr (kTeam > 1) {
                    __builtin_amdgcn_s_barrier();
                    set_wave_priority(turn + 1);
                }
                if (kSubtract || out_cur.ld > 0) {
                    store_chunk_rows(v, (void*)dst, uniform64(out_cur.ld), lane, skip_cur || tripped);
                } else if (!skip_cur) {
#pragma unroll
                    for (int q0 = 0; q0 < 16; ++q0)
                        reinterpret_cast<float4*>((float*)dst)[q0 * 64 + lane] =
                            make_float4(v[4 * q0], v[4 * q0 + 1], v[4 * q0 + 2], v[4 * q0 + 3]);
                }
                if constexpr (kTeam > 1) set_wave_priority(turn);
            }
            const bool more = g + T < g1;
            Out out3 = out_after;
            bool skip_next = false;
            if (more) {
                zero_tile();
                wset_scatter(st);
                if (g + 3 * T < g1) {
                    cursor_to(c, g + 3 * T);
                    out3 = out_of(c, g + 3 * T);
                    wset_load(st, g + 3 * T, c.t);
                }
                skip_next = __ballot(repeat == kClaimMark) != 0;  // wave-uniform, false for top-k payloads
                if (skip_next) mark_redo(g + T);
                repeat = 0;
                mean_pass();
            }
            skip_cur = skip_next;
            out_cur = out_next;
            out_next = out_after;
            out_after = out3;
        };
        for (int64_t g = g0; g < g1; g += 2 * T) {
            step(g, s1, false);
            if (g + T < g1) step(g + T, s0, true);
        }
        if constexpr (kTeam > 1) {
            for (int64_t i = my_steps; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
        }
        redo_marked();
        return;
    }

    // The other variants (coefficient output, generic peer count or k, per-chunk normalisation):
    // a plain three-chunk pipeline.  Chunk g leaves the tile for registers, chunk g + 1 is
    // scattered into the tile, the payload of chunk g + 2 is requested (fast path only).
    Cursor c;
    cursor_seek(c, table, single, n_tensors, g0);
    Out out_cur = out_of(c, g0), out_next = out_cur;
    int t_next = c.t;
    if (fast) load_payload(g0, c.t);
    zero_tile();
    scatter(g0, c.t);
    bool skip_cur = __ballot(repeat == kClaimMark) != 0;  // chunk g: found to hold a repeated index, not stored
    if (skip_cur) mark_redo(g0);
    repeat = 0;
    mean_pass();
    // (the chunks of a wave are T apart: "g + 1" in the comments below stands for the wave's next chunk)
    if (g0 + T < g1) {
        cursor_to(c, g0 + T);
        out_next = out_of(c, g0 + T);
        t_next = c.t;
        if (fast) load_payload(g0 + T, c.t);
    }
    const bool late_layer = blockIdx.x * 2 >= gridDim.x;  // wave-uniform
    for (int64_t g = g0; g < g1; g += T) {
        float v[64];
        const int turn = ((((g - g0) / T) & 1) != 0) != late_layer ? 2 : 0;
        set_wave_priority(turn);  // the two waves of a SIMD take turns, as above
        // ---- first half: everything that needs chunk g's coefficients in the tile
        if (kUseDct) {
            tile_rows_to_regs(v, tile, lane);
            dct64_inv(v);  // along d: v[l] = sum_d Y[lane][d] F[l][d]
            wave_lds_fence();
            regs_to_tile_rows(v, tile, lane);
            wave_lds_fence();
            tile_cols_to_regs(v, tile, lane);
        } else if (out_cur.ld > 0) {  // wave-uniform
            tile_cols_to_regs(v, tile, lane);
        } else {
#pragma unroll
            for (int q0 = 0; q0 < 16; ++q0) {
                const int q = q0 * 64 + lane;
                const float4 t = *reinterpret_cast<const float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2));
                v[4 * q0] = t.x, v[4 * q0 + 1] = t.y, v[4 * q0 + 2] = t.z, v[4 * q0 + 3] = t.w;
            }
        }
        wave_lds_fence();

        // ---- the tile is free: chunk g + 1 moves in, chunk g + 2 is requested
        const bool more = g + T < g1;
        Out out_after = out_next;
        int t_after = t_next;
        // Without the transform chunk g is complete here: its 64 row stores go out first - the wave stands at
        // them at the pace the memory system takes them - and, where the registers allow it (up to 16 peers), the
        // next chunk's scatter, a chain of LDS round trips, runs between groups of them.
        bool stored = false;
        if (!kUseDct && fast && more && out_cur.ld > 0) {  // wave-uniform
            chunk_stats(v, g, skip_cur);
            const int64_t ld_s = uniform64(out_cur.ld);
            const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
                (void*)uniform64(reinterpret_cast<int64_t>(out_cur.chunk0)), 0,
                skip_cur ? 0 : static_cast<int>((63 * ld_s + 64) * 4), 0x00020000);
            const int ld4 = static_cast<int>(ld_s) * 4;
            zero_tile();
            if constexpr (kTeam > 1) {  // the team stores together, one priority level up
                __builtin_amdgcn_s_barrier();
                set_wave_priority(turn + 1);
            }
            if constexpr (kUnits <= 16) {
                constexpr int kGroups = 4, kPerGroup = (kRegs + kGroups - 1) / kGroups;
                static_for<kGroups>([&](auto qt) {
                    constexpr int q = decltype(qt)::value;
#pragma unroll
                    for (int r = q * 16; r < (q + 1) * 16; ++r)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v[r]), wr, lane * 4, r * ld4, 2);
                    scatter(g + T, t_next, q * kPerGroup, (q + 1) * kPerGroup);
                });
            } else {
#pragma unroll
                for (int r = 0; r < 64; ++r)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v[r]), wr, lane * 4, r * ld4, 2);
                scatter(g + T, t_next);
            }
            if constexpr (kTeam > 1) set_wave_priority(turn);
            if (g + 2 * T < g1) {
                cursor_to(c, g + 2 * T);
                out_after = out_of(c, g + 2 * T);
                t_after = c.t;
                load_payload(g + 2 * T, c.t);
            }
            stored = true;
        } else if (more) {
            zero_tile();
            scatter(g + T, t_next);
            if (g + 2 * T < g1) {
                cursor_to(c, g + 2 * T);
                out_after = out_of(c, g + 2 * T);
                t_after = c.t;
                if (fast) load_payload(g + 2 * T, c.t);
            }
        }
        // ---- second half of chunk g, in registers
        if (kUseDct) dct64_inv(v);  // along b: v[k] = sum_b Z[b][lane] F[k][b]
        if (!stored) chunk_stats(v, g, skip_cur);
        const bool skip_next = more && __ballot(repeat == kClaimMark) != 0;  // wave-uniform, false for top-k payloads
        if (skip_next) mark_redo(g + T);
        repeat = 0;
        if (more) mean_pass();

        // (the loop-carried destination may have been parked in vector registers: make it scalar
        // again, or every store becomes a loop over distinct descriptors)
        gfloat* const dst = (gfloat*)uniform64(reinterpret_cast<int64_t>(out_cur.chunk0));
        if constexpr (kTeam > 1) {
            if (!stored) __builtin_amdgcn_s_barrier();  // (every wave of the team: one barrier per chunk, here or above)
        }
        if (stored) {
            // (written above)
        } else if (kUseDct || out_cur.ld > 0) {
            store_chunk_rows(v, (void*)dst, uniform64(out_cur.ld), lane, skip_cur);
        } else if (!skip_cur) {
#pragma unroll
            for (int q0 = 0; q0 < 16; ++q0)
                reinterpret_cast<float4*>((float*)dst)[q0 * 64 + lane] =
                    make_float4(v[4 * q0], v[4 * q0 + 1], v[4 * q0 + 2], v[4 * q0 + 3]);
        }
        skip_cur = skip_next;
        out_cur = out_next;
        out_next = out_after;
        t_next = t_after;
    }
    if constexpr (kTeam > 1) {
        for (int64_t i = my_steps; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
    }
    redo_marked();
}

// The miner's whole error-feedback step for one chunk in one pass, where no quantiser sits between its two
// halves (src/tplr/neurons.py:147-171): ef * decay + grad, the transform, top-k, the payload, and at once the
// subtraction of that payload's reconstruction - what tplr_ef_encode_topk_pack_batch followed by
// tplr_ef_subtract_batch leave, bit for bit, with the tensor read once and written once (48 KB of traffic per
// chunk instead of 81 KB).  The updated chunk stays in 64 registers while it is transformed and selected from;
// the k selected values go back into a cleared tile exactly as the one-peer decode adds them (0 + value * 2^-5),
// through the inverse transform, and the difference is stored.  Two waves per SIMD (a whole tile, 64 more
// registers): the launch moves 14 GB and is bound by that.
// Workgroups are teams of four (two) waves, as in the aggregate: wave w takes every fourth chunk of the team's range,
// the team reads rows of 1 KB at the same moment and meets at a barrier before it stores them (6 % off the launch).
// (at k = 64 the select's instantiation is at the register limit: teams of four are 2 % slower than single
// waves there, teams of two 4.5 % faster)
template <bool kTwo>
constexpr int ef_team() { return kTwo ? 2 : 4; }
template <bool kTwo>
__global__ __launch_bounds__(64 * ef_team<kTwo>(), 2) void k_ef_step(const tplr_tensor_desc* __restrict__ table,
                                                   const tplr_tensor_desc* __restrict__ grad_table, int n_tensors,
                                                   int64_t total, int k, float decay, uint8_t* __restrict__ idx12,
                                                   float* __restrict__ val) {
    constexpr int T = ef_team<kTwo>();
    __shared__ __align__(16) float tile_all[T][kTileFloats];
    __shared__ uint64_t cand_all[T][kCandCap];
    const int wv = T > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)) : 0;
    float* const tile = tile_all[wv];
    uint64_t* const cand = cand_all[wv];
    int64_t g0, g1;
    my_range(total, g0, g1, T);
    if (g0 >= g1) return;
    const int64_t team_steps = (g1 - g0 + T - 1) / T;
    g0 += wv;
    const int64_t my_steps = g0 < g1 ? (g1 - 1 - g0) / T + 1 : 0;
    if (my_steps == 0) {  // wave-uniform: a team with fewer chunks than waves
        if constexpr (T > 1) {
            for (int64_t i = 0; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
        }
        return;
    }
    Cursor c, cg;
    tplr_tensor_desc none = {};
    cursor_seek(c, table, none, n_tensors, g0);
    cursor_seek(cg, grad_table, none, n_tensors, g0);
    for (int64_t g = g0; g < g1; g += T) {
        // (lane-derived addresses are formed per chunk from a copy of the lane id the optimiser cannot see
        // through: hoisted out of the loop they would be spilled)
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        float e[64], v[64], w[64];
        load_chunk_cols(e, c, lane);
        load_chunk_cols(w, cg, lane);
#pragma unroll
        for (int r = 0; r < 64; ++r) {
            const float m = e[r] * decay;
            e[r] = m + w[r];
            v[r] = e[r];
        }
        gfloat* const dst = c.base + (c.y * 64) * c.ld + static_cast<int64_t>(c.xc) * 64;
        const int64_t ld = c.ld;
        if (g + T < g1) {
#pragma unroll
            for (int s = 1; s <= T; ++s) {
                cursor_next(cg, g + s);
                cursor_next(c, g + s);
            }
        }
        // the two waves of a SIMD take turns chunk by chunk, as in the aggregate: two priority levels up on every
        // other chunk, opposite chunks in the two dispatch layers, one more level from the stores to the next
        // chunk's requests (3 % off the launch)
        const int turn = ((((g - g0) / T) & 1) != 0) != (blockIdx.x * 2 >= gridDim.x) ? 2 : 0;  // wave-uniform
        set_wave_priority(turn);
        chunk_forward<true>(v, w, tile, lane);
        const Selected s = select_topk<kTwo, false>(w, tile, cand, lane, k, kDctPow2Scale, 0, 0);
        emit_selected<kTwo>(s, lane, k, g, idx12, val);
        // the payload's reconstruction
        {
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            float4* row = reinterpret_cast<float4*>(tile + lane * kLd);
#pragma unroll
            for (int q = 0; q < 16; ++q) row[q] = z;
        }
        wave_lds_fence();
        if (lane < k) tile[tile_pos(s.idx0)] = 0.0f + s.val0 * kDctPow2Scale;
        wave_lds_fence();
        chunk_inverse<true>(v, tile, lane);
        wave_lds_fence();
#pragma unroll
        for (int r = 0; r < 64; ++r) v[r] = e[r] - v[r];
        if constexpr (T > 1) __builtin_amdgcn_s_barrier();  // the team stores together
        set_wave_priority(turn + 1);
        store_chunk_rows(v, (void*)uniform64(reinterpret_cast<int64_t>(dst)), uniform64(ld), lane);
    }
    if constexpr (T > 1) {
        for (int64_t i = my_steps; i < team_steps; ++i) __builtin_amdgcn_s_barrier();
    }
}

// ef <- ef - (the payload's entries) for chunks that are not transformed (use_dct = 0): the
// reconstruction is the payload itself, so only k elements per chunk change
// (src/tplr/neurons.py:162-171 with decode a pure re-layout).  k <= 64: one entry per lane.  What
// is subtracted at a position is what decompress leaves there (src/tplr/compress.py:472-474):
// the entry, or, when a row names a position more than once (no top-k does), the mean of those
// entries, added in entry order.
__global__ __launch_bounds__(64) void k_ef_subtract_sparse(const uint8_t* __restrict__ idx12,
                                                           const float* __restrict__ val, int k,
                                                           const tplr_tensor_desc* __restrict__ table,
                                                           const tplr_tensor_desc single, int n_tensors,
                                                           int64_t total, const float* __restrict__ factor,
                                                           int32_t* __restrict__ guard) {
    // factor (nullable): every value of tensor t times factor[t] before it is subtracted
    // guard (nullable, one int per tensor, zeroed by the caller): a chunk with an entry that is NaN or infinite
    // after the factor is left as it is and guard[tensor] becomes 1
    __shared__ uint16_t owner[4096];  // the last lane that named a position (never cleared: written before read)
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    Cursor c;
    cursor_seek(c, table, single, n_tensors, g0);
    const int64_t idx_stride = k + (k >> 1);
    for (int64_t g = g0; g < g1; ++g) {
        gfloat* chunk0 = c.base + (c.y * 64) * c.ld + static_cast<int64_t>(c.xc) * 64;
        int me = -1;
        float x = 0.f;
        if (lane < k) {
            me = static_cast<int>(load_idx12(idx12 + g * idx_stride, lane));
            x = val[g * k + lane];
            if (factor) {
                x *= factor[c.t];
                asm volatile("" : "+v"(x));  // a product of its own rounding, never contracted into the subtraction
            }
            owner[me] = static_cast<uint16_t>(lane);
        }
        wave_lds_fence();
        const bool shared_pos = me >= 0 && owner[me] != lane;
        bool first = true;
        if (__ballot(shared_pos) != 0) {  // wave-uniform: some position is named twice
            float sum = 0.f;
            int n = 0;
            for (int i = 0; i < 64; ++i) {
                const int other = __shfl(me, i);
                const float xo = __shfl(x, i);
                if (other == me && me >= 0) {
                    sum += xo;  // entry order, from zero, as the scatter adds them
                    n += 1;
                    first = first && i >= lane;
                }
            }
            x = n > 1 ? sum / static_cast<float>(n) : sum;
        }
        bool tripped = false;
        if (guard) {  // wave-uniform
            tripped = __ballot(me >= 0 && (__builtin_bit_cast(uint32_t, x) & 0x7f800000u) == 0x7f800000u) != 0;
            if (tripped && lane == 0) guard[c.t] = 1;
        }
        if (me >= 0 && first && !tripped) {
            gfloat* t = chunk0 + static_cast<int64_t>(me >> 6) * c.ld + (me & 63);
            *t = *t - x;
        }
        wave_lds_fence();
        if (g + 1 < g1) cursor_next(c, g + 1);
    }
}

// The same for the miner's own step, where the payload was selected from this very tensor a launch ago
// (tplr_ef_encode_topk_pack_batch without the transform): what stands at a selected position is the
// payload's own value, bit for bit, so ef - sent there is own - sent and nothing has to be read from the
// tensor - k scattered four-byte stores per chunk instead of k read-modify-writes.  `own` are the payload's
// values as selected, `sent` what the reference would decompress (the same, or their de-quantised form).  A
// top-k selection names every position once; the next chunk's entries are requested before this chunk's are
// stored.
__global__ __launch_bounds__(64) void k_ef_overwrite_sparse(const uint8_t* __restrict__ idx12,
                                                            const float* __restrict__ sent,
                                                            const float* __restrict__ own, int k,
                                                            const tplr_tensor_desc* __restrict__ table,
                                                            const tplr_tensor_desc single, int n_tensors,
                                                            int64_t total) {
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    Cursor c;
    cursor_seek(c, table, single, n_tensors, g0);
    const int64_t idx_stride = k + (k >> 1);
    const int le = lane < k ? lane : 0;
    auto fetch = [&](int64_t g, uint32_t& me, float& x) {
        me = load_idx12(idx12 + g * idx_stride, le);
        x = own[g * k + le] - sent[g * k + le];
    };
    uint32_t me, me_next = 0;
    float x, x_next = 0.f;
    fetch(g0, me, x);
    for (int64_t g = g0; g < g1; ++g) {
        if (g + 1 < g1) fetch(g + 1, me_next, x_next);
        gfloat* chunk0 = c.base + (c.y * 64) * c.ld + static_cast<int64_t>(c.xc) * 64;
        if (lane < k) chunk0[static_cast<int64_t>(me >> 6) * c.ld + (me & 63)] = x;
        me = me_next;
        x = x_next;
        if (g + 1 < g1) cursor_next(c, g + 1);
    }
}

// -----------------------------------------------------------------------------------------
// Statistics of the packed index streams of up to 32 peers, per tensor:
//   pair[t][p][q] (p < q) = number of entries of peer p that also occur in the same row of peer q,
//                           summed over the tensor's rows: the `(a == b).any(-1).sum(-1)` of
//                           check_uid_index_overlap (src/tplr/neurons.py:1373-1378) before its
//                           division by k and mean over rows;
//   dup[t][p]             = entries of peer p that repeat an earlier entry of their own row
//                           (a top-k selection has none);
//   mx[t][p]              = largest index of peer p (the bounds check of
//                           Comms.check_compressed_indices, src/tplr/comms.py:2573-2581).
// One wave per row at a time: the row's 4096 possible indices each get a 32-bit mask of the peers
// that sent them (LDS, integer atomics), then every entry looks its mask up and counts the
// higher-numbered peers in it.  Totals collect in LDS and go out with one 64-bit atomic per
// non-zero counter when the wave leaves a tensor.
// -----------------------------------------------------------------------------------------
constexpr int kStatPeers = 32;
struct IdxPtrs {
    const uint8_t* idx[kStatPeers];
};


// kPerPass: peers handled by one wave instruction: 2 when k <= 32 (one peer per half of the wave), 1 when
// k <= 64; 0 = rows of any length, entry by entry.  kPasses: wave instructions per row that the
// register arrays are sized for (kPerPass * kPasses peers at most).  kPlanes > 0: shared entries are
// counted in registers - every lane keeps, per pass, one counter per later peer as kPlanes bit planes
// (bit j of plane b = bit b of the count for peer p + 1 + j), incremented with a ripple of ANDs and
// XORs and summed over the lanes every 2^kPlanes - 1 rows; 0 = counted with LDS atomics.
template <int kPerPass, int kPasses = 1, int kPlanes = 0>
__global__ __launch_bounds__(64) void k_index_stats(const IdxPtrs ip, int P, int k,
                                                    const tplr_tensor_desc* __restrict__ table,
                                                    const tplr_tensor_desc single, int n_tensors, int64_t total,
                                                    unsigned long long* __restrict__ pair,
                                                    unsigned long long* __restrict__ dup, int* __restrict__ mx) {
    __shared__ __align__(16) uint32_t mask[4096];
    __shared__ uint32_t pair_l[kStatPeers * kStatPeers];
    __shared__ uint32_t dup_l[kStatPeers];
    __shared__ int mx_l[kStatPeers];
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    const int64_t idx_stride = k + (k >> 1);
    Cursor c;
    cursor_seek(c, table, single, n_tensors, g0);
    auto clear_totals = [&]() {
        for (int i = lane; i < kStatPeers * kStatPeers; i += 64) pair_l[i] = 0;
        if (lane < kStatPeers) dup_l[lane] = 0, mx_l[lane] = -1;
        wave_lds_fence();
    };
    auto flush_totals = [&](int t) {
        wave_lds_fence();
        for (int i = lane; i < kStatPeers * kStatPeers; i += 64) {
            const int p = i / kStatPeers, q = i - p * kStatPeers;
            if (pair_l[i] && p < P && q < P)
                atomicAdd(&pair[(static_cast<int64_t>(t) * P + p) * P + q], static_cast<unsigned long long>(pair_l[i]));
        }
        if (lane < P) {
            if (dup_l[lane]) atomicAdd(&dup[static_cast<int64_t>(t) * P + lane], static_cast<unsigned long long>(dup_l[lane]));
            if (mx_l[lane] >= 0) atomicMax(&mx[static_cast<int64_t>(t) * P + lane], mx_l[lane]);
        }
        wave_lds_fence();
    };
    clear_totals();
    int t_cur = c.t;
    if constexpr (kPerPass > 0) {
        // One entry per lane and peer, all peers of a row in registers; the next row's entries are
        // requested before this row is worked on.  Repeats and maxima are kept per lane and
        // reach the per-tensor totals when those are flushed.
        const int sub = kPerPass == 2 ? lane >> 5 : 0;
        const int j = kPerPass == 2 ? (lane & 31) : lane;
        const bool jon = j < k;
        const int joff = 3 * (j >> 1) + (j & 1);
        const uint32_t jshift = (j & 1) * 4;
        uint32_t cur[kPasses], nxt[kPasses];
        int top[kPasses];
        uint32_t planes[kPlanes ? kPasses : 1][kPlanes ? kPlanes : 1];
#pragma unroll
        for (int i = 0; i < kPasses; ++i) cur[i] = nxt[i] = 0, top[i] = -1;
#pragma unroll
        for (int i = 0; i < (kPlanes ? kPasses : 1); ++i)
#pragma unroll
            for (int b = 0; b < (kPlanes ? kPlanes : 1); ++b) planes[i][b] = 0;
        int pending = 0;  // rows counted in the planes since they were last summed
        auto request = [&](uint32_t (&e)[kPasses], int64_t g) {
#pragma unroll
            for (int i = 0; i < kPasses; ++i) {
                if (i * kPerPass < P) {  // wave-uniform
                    const uint8_t* base = ip.idx[i * kPerPass];
                    if constexpr (kPerPass == 2) base = (sub && i * 2 + 1 < P) ? ip.idx[i * 2 + 1] : base;
                    const gbyte* row = (const gbyte*)base + g * idx_stride;
                    if (jon) e[i] = *(const gu16*)(row + joff);
                }
            }
        };
        // bit planes -> pair counters: for every pass and later peer, the lanes' counts are summed plane
        // by plane with ballots (the two halves of the wave are two peers when kPerPass == 2)
        auto sum_planes = [&]() __attribute__((always_inline)) {
            if constexpr (kPlanes > 0) {
                static_for<kPasses>([&](auto pass) __attribute__((always_inline)) {
                    constexpr int i = decltype(pass)::value;
                    const int p0 = i * kPerPass;
                    if (p0 + 1 < P) {  // wave-uniform
                        const int later = P - 1 - p0;
                        for (int jb = 0; jb < later; ++jb) {
                            uint32_t lo = 0, hi = 0;
#pragma unroll
                            for (int b = 0; b < kPlanes; ++b) {
                                const uint64_t hit = __ballot(((planes[i][b] >> jb) & 1u) != 0u);
                                if constexpr (kPerPass == 2) {
                                    lo += static_cast<uint32_t>(__popc(static_cast<uint32_t>(hit))) << b;
                                    hi += static_cast<uint32_t>(__popc(static_cast<uint32_t>(hit >> 32))) << b;
                                } else {
                                    lo += static_cast<uint32_t>(__popcll(hit)) << b;
                                }
                            }
                            if (lane == 0) {
                                pair_l[p0 * kStatPeers + p0 + 1 + jb] += lo;
                                if (kPerPass == 2 && p0 + 2 + jb < P) pair_l[(p0 + 1) * kStatPeers + p0 + 2 + jb] += hi;
                            }
                        }
#pragma unroll
                        for (int b = 0; b < kPlanes; ++b) planes[i][b] = 0;
                    }
                });
            }
            pending = 0;
        };
        auto fold = [&]() __attribute__((always_inline)) {  // per-lane counts and maxima into the per-tensor totals
            sum_planes();
#pragma unroll
            for (int i = 0; i < kPasses; ++i) {
                const int p = i * kPerPass + sub;
                if (i * kPerPass < P) {
                    if (jon && p < P && top[i] >= 0) atomicMax(&mx_l[p], top[i]);
                    top[i] = -1;
                }
            }
        };
        request(nxt, g0);
        for (int64_t g = g0; g < g1; ++g) {
            if (c.t != t_cur) {  // wave-uniform
                fold();
                flush_totals(t_cur);
                clear_totals();
                t_cur = c.t;
            }
#pragma unroll
            for (int i = 0; i < kPasses; ++i) cur[i] = (nxt[i] >> jshift) & 0xfffu;
            request(nxt, g + 1 < g1 ? g + 1 : g);
            const uint4 z = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 16; ++q) reinterpret_cast<uint4*>(mask)[q * 64 + lane] = z;
            wave_lds_fence();
#pragma unroll
            for (int i = 0; i < kPasses; ++i) {
                const int p = i * kPerPass + sub;
                if (i * kPerPass < P && jon && p < P) {
                    const uint32_t old = atomicOr(&mask[cur[i]], 1u << p);
                    if ((old >> p) & 1u) atomicAdd(&dup_l[p], 1u);  // a repeat inside the row: rare
                    top[i] = top[i] > static_cast<int>(cur[i]) ? top[i] : static_cast<int>(cur[i]);
                }
            }
            wave_lds_fence();
            static_for<kPasses>([&](auto pass) __attribute__((always_inline)) {
                constexpr int i = decltype(pass)::value;
                const int p = i * kPerPass + sub;
                if (i * kPerPass + 1 < P) {  // wave-uniform: a later peer exists
                    // the peers after p that sent this lane's entry too, bit 0 = peer p + 1
                    const uint32_t m = (jon && p + 1 < P) ? mask[cur[i]] >> ((p + 1) & 31) : 0u;
                    if constexpr (kPlanes > 0) {
                        uint32_t carry = m;
#pragma unroll
                        for (int b = 0; b < kPlanes; ++b) {
                            const uint32_t t = planes[i][b] & carry;
                            planes[i][b] ^= carry;
                            carry = t;
                        }
                    } else {
                        uint32_t w = m;
                        while (w) {
                            const int q = p + 1 + __builtin_ctz(w);
                            atomicAdd(&pair_l[p * kStatPeers + q], 1u);
                            w &= w - 1;
                        }
                    }
                }
            });
            wave_lds_fence();
            if (kPlanes > 0 && ++pending == (1 << kPlanes) - 1) sum_planes();
            if (g + 1 < g1) cursor_next(c, g + 1);
        }
        fold();
        flush_totals(t_cur);
        return;
    }
    for (int64_t g = g0; g < g1; ++g) {
        if (c.t != t_cur) {  // wave-uniform
            flush_totals(t_cur);
            clear_totals();
            t_cur = c.t;
        }
        const uint4 z = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int q = 0; q < 16; ++q) reinterpret_cast<uint4*>(mask)[q * 64 + lane] = z;
        wave_lds_fence();
        for (int p = 0; p < P; ++p) {
            const gbyte* row = (const gbyte*)ip.idx[p] + g * idx_stride;
            int top = -1;
            for (int j = lane; j < k; j += 64) {
                const uint32_t e = load_idx12(row, j);
                const uint32_t old = atomicOr(&mask[e], 1u << p);
                if ((old >> p) & 1u) atomicAdd(&dup_l[p], 1u);
                top = top > static_cast<int>(e) ? top : static_cast<int>(e);
            }
            top = static_cast<int>(wave_max_u32(static_cast<uint32_t>(top + 1))) - 1;
            if (lane == 0 && top > mx_l[p]) mx_l[p] = top;
        }
        wave_lds_fence();
        for (int p = 0; p + 1 < P; ++p) {
            const gbyte* row = (const gbyte*)ip.idx[p] + g * idx_stride;
            for (int j = lane; j < k; j += 64) {
                const uint32_t e = load_idx12(row, j);
                uint32_t m = mask[e] >> (p + 1);  // the peers after p that sent e too
                while (m) {
                    const int q = p + 1 + __builtin_ctz(m);
                    atomicAdd(&pair_l[p * kStatPeers + q], 1u);
                    m &= m - 1;
                }
            }
        }
        wave_lds_fence();
        if (g + 1 < g1) cursor_next(c, g + 1);
    }
    flush_totals(t_cur);
}

// De-quantise one peer's flat payload of 8-bit codes: value = lookup[t][code] + shift[t], the
// tensor t found from the row id (TopKCompressor._dequantize_values, src/tplr/compress.py:637-643,
// for every parameter of the set at once).  Four codes per thread.
// The statistical quantiser over each tensor's sent values (src/tplr/compress.py:582-621): the
// reference's three passes - mean, norm of the centred values, codes with per-bin means - as three
// launches over slices of every tensor plus one that finishes the tables.  Partial sums are carried
// in double, kept per (tensor, slice) in a caller-provided workspace and added in slice order by
// whoever needs the total, so every workgroup of a tensor derives the same shift and scale.
// Workspace layout (doubles): sum[T][S], sumsq[T][S], then bins[T][S][2 * n_bins] (sums, counts).
struct QuantSlice {
    const float4* v;
    uchar4* q;
    int64_t n4;  // float4 groups in this slice
    int64_t n;   // values in the whole tensor
    int t, s;
};

__device__ __forceinline__ QuantSlice quant_slice(const float* val, uint8_t* codes, const tplr_tensor_desc* table,
                                                   int k, int S) {
    QuantSlice qs;
    qs.t = blockIdx.x / S;
    qs.s = blockIdx.x - qs.t * S;
    const tplr_tensor_desc d = table[qs.t];
    const int64_t rows = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const int64_t r0 = rows * qs.s / S, r1 = rows * (qs.s + 1) / S;
    qs.v = reinterpret_cast<const float4*>(val + (d.chunk_begin + r0) * k);
    qs.q = codes ? reinterpret_cast<uchar4*>(codes + (d.chunk_begin + r0) * k) : nullptr;
    qs.n4 = (r1 - r0) * k >> 2;  // k is a multiple of 4
    qs.n = rows * k;
    return qs;
}

__device__ __forceinline__ double block256_sum_f64(double x, double* part, int tid) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off);
    __syncthreads();  // `part` may still be read from the previous call
    if ((tid & 63) == 0) part[tid >> 6] = x;
    __syncthreads();
    return (part[0] + part[1]) + (part[2] + part[3]);
}

__device__ __forceinline__ double slices_total(const double* w, int S) {
    double s = 0.0;
    for (int i = 0; i < S; ++i) s += w[i];
    return s;
}

__device__ __forceinline__ float quant_shift(const double* work, int t, int S, int64_t n) {
    return static_cast<float>(slices_total(work + static_cast<int64_t>(t) * S, S) / static_cast<double>(n));  // :594
}

__device__ __forceinline__ float quant_scale(const double* work, int T, int t, int S, int64_t n, int n_bins,
                                             float range_in_sigmas) {
    const double ss = slices_total(work + (static_cast<int64_t>(T) + t) * S, S);
    const float sd = static_cast<float>(sqrt(ss) / sqrt(static_cast<double>(n - 1)));  // :597
    const float scale = range_in_sigmas * sd / static_cast<float>(n_bins);              // :598
    return (scale == 0.f || scale != scale || __builtin_isinf(scale)) ? 1.0f : scale;   // :599-600
}

__global__ __launch_bounds__(256) void k_quant_sum(const float* __restrict__ val, int k,
                                                   const tplr_tensor_desc* __restrict__ table, int S,
                                                   double* __restrict__ work) {
    __shared__ double part[4];
    const int tid = threadIdx.x;
    const QuantSlice qs = quant_slice(val, nullptr, table, k, S);
    double acc = 0.0;
    for (int64_t i = tid; i < qs.n4; i += 256) {
        const float4 x = qs.v[i];
        acc += (static_cast<double>(x.x) + x.y) + (static_cast<double>(x.z) + x.w);
    }
    acc = block256_sum_f64(acc, part, tid);
    if (tid == 0) work[blockIdx.x] = acc;
}

__global__ __launch_bounds__(256) void k_quant_sumsq(const float* __restrict__ val, int k,
                                                     const tplr_tensor_desc* __restrict__ table, int T, int S,
                                                     double* __restrict__ work) {
    __shared__ double part[4];
    const int tid = threadIdx.x;
    const QuantSlice qs = quant_slice(val, nullptr, table, k, S);
    const float shift = quant_shift(work, qs.t, S, qs.n);
    double acc = 0.0;
    for (int64_t i = tid; i < qs.n4; i += 256) {
        const float4 x = qs.v[i];
        const float a = x.x - shift, b = x.y - shift, c = x.z - shift, e = x.w - shift;  // :595
        acc += (static_cast<double>(a) * a + static_cast<double>(b) * b) +
               (static_cast<double>(c) * c + static_cast<double>(e) * e);
    }
    acc = block256_sum_f64(acc, part, tid);
    if (tid == 0) work[static_cast<int64_t>(T) * S + blockIdx.x] = acc;
}

__global__ __launch_bounds__(256) void k_quant_codes(const float* __restrict__ val, int k,
                                                     const tplr_tensor_desc* __restrict__ table, int T, int S, int n_bins,
                                                     float range_in_sigmas, uint8_t* __restrict__ codes,
                                                     double* __restrict__ work) {
    __shared__ double part[4];
    __shared__ double bin_sum[256];
    __shared__ unsigned int bin_cnt[256];
    const int tid = threadIdx.x;
    const QuantSlice qs = quant_slice(val, codes, table, k, S);
    const float shift = quant_shift(work, qs.t, S, qs.n);
    const float scale = quant_scale(work, T, qs.t, S, qs.n, n_bins, range_in_sigmas);
    double* out = work + 2 * static_cast<int64_t>(T) * S + static_cast<int64_t>(blockIdx.x) * 2 * n_bins;
    const float offset = static_cast<float>(n_bins / 2), top = static_cast<float>(n_bins - 1);
    auto code = [&](float x, float& c) {
        c = x - shift;
        float r = __builtin_rintf(c / scale + offset);  // :604-605, ties to even as torch.round
        r = r < 0.f ? 0.f : r;
        r = r > top ? top : r;                          // :606
        return static_cast<uint32_t>(r);
    };
    if (n_bins <= 8) {
        // a handful of bins (templar runs four): per-thread sums, no contended atomics
        double s8[8], c8[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) s8[b] = c8[b] = 0.0;
        auto tally = [&](uint32_t qq, float c) {
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                s8[b] += qq == static_cast<uint32_t>(b) ? static_cast<double>(c) : 0.0;  // :614-617
                c8[b] += qq == static_cast<uint32_t>(b) ? 1.0 : 0.0;
            }
        };
        for (int64_t i = tid; i < qs.n4; i += 256) {
            const float4 x = qs.v[i];
            float c0, c1, c2, c3;
            const uint32_t q0 = code(x.x, c0), q1 = code(x.y, c1), q2 = code(x.z, c2), q3 = code(x.w, c3);
            qs.q[i] = make_uchar4(static_cast<unsigned char>(q0), static_cast<unsigned char>(q1),
                                  static_cast<unsigned char>(q2), static_cast<unsigned char>(q3));
            tally(q0, c0), tally(q1, c1), tally(q2, c2), tally(q3, c3);
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const double sum = block256_sum_f64(s8[b], part, tid), cnt = block256_sum_f64(c8[b], part, tid);
            if (tid == 0 && b < n_bins) out[b] = sum, out[n_bins + b] = cnt;
        }
    } else {
        bin_sum[tid] = 0.0, bin_cnt[tid] = 0u;
        __syncthreads();
        for (int64_t i = tid; i < qs.n4; i += 256) {
            const float4 x = qs.v[i];
            float c0, c1, c2, c3;
            const uint32_t q0 = code(x.x, c0), q1 = code(x.y, c1), q2 = code(x.z, c2), q3 = code(x.w, c3);
            qs.q[i] = make_uchar4(static_cast<unsigned char>(q0), static_cast<unsigned char>(q1),
                                  static_cast<unsigned char>(q2), static_cast<unsigned char>(q3));
            atomicAdd(&bin_sum[q0], static_cast<double>(c0)), atomicAdd(&bin_cnt[q0], 1u);  // :614-617
            atomicAdd(&bin_sum[q1], static_cast<double>(c1)), atomicAdd(&bin_cnt[q1], 1u);
            atomicAdd(&bin_sum[q2], static_cast<double>(c2)), atomicAdd(&bin_cnt[q2], 1u);
            atomicAdd(&bin_sum[q3], static_cast<double>(c3)), atomicAdd(&bin_cnt[q3], 1u);
        }
        __syncthreads();
        if (tid < n_bins) out[tid] = bin_sum[tid], out[n_bins + tid] = static_cast<double>(bin_cnt[tid]);
    }
}

__global__ __launch_bounds__(256) void k_quant_tables(const tplr_tensor_desc* __restrict__ table, int k, int T, int S,
                                                      int n_bins, float range_in_sigmas,
                                                      const double* __restrict__ work, float* __restrict__ shift_out,
                                                      float* __restrict__ scale_out, float* __restrict__ lookup) {
    const int t = blockIdx.x, tid = threadIdx.x;
    const tplr_tensor_desc d = table[t];
    const int64_t n = static_cast<int64_t>(d.x_chunks) * d.y_chunks * k;
    if (tid < n_bins) {
        const double* bins = work + 2 * static_cast<int64_t>(T) * S + static_cast<int64_t>(t) * S * 2 * n_bins;
        double sum = 0.0, cnt = 0.0;
        for (int s = 0; s < S; ++s) sum += bins[s * 2 * n_bins + tid], cnt += bins[s * 2 * n_bins + n_bins + tid];
        lookup[static_cast<int64_t>(t) * n_bins + tid] = cnt > 0.0 ? static_cast<float>(sum / cnt) : 0.f;  // :619
    }
    if (tid == 0) {
        shift_out[t] = quant_shift(work, t, S, n);
        scale_out[t] = quant_scale(work, T, t, S, n, n_bins, range_in_sigmas);
    }
}

__global__ __launch_bounds__(256) void k_dequantize_batch(const uint8_t* __restrict__ q,
                                                          const float* __restrict__ lookup,
                                                          const float* __restrict__ shift, int n_bins, int k,
                                                          const tplr_tensor_desc* __restrict__ table, int n_tensors,
                                                          int64_t n4, float* __restrict__ val) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n4; i += stride) {
        const int64_t row = (i * 4) / k;  // k is a multiple of 4 here: the four codes share a row
        int lo = 0, hi = n_tensors;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table[mid].chunk_begin <= row)
                lo = mid;
            else
                hi = mid;
        }
        const uchar4 c = reinterpret_cast<const uchar4*>(q)[i];
        const float* lk = lookup + static_cast<int64_t>(lo) * n_bins;
        const float sh = shift[lo];
        float4 o;
        o.x = lk[c.x < n_bins ? c.x : n_bins - 1] + sh;
        o.y = lk[c.y < n_bins ? c.y : n_bins - 1] + sh;
        o.z = lk[c.z < n_bins ? c.z : n_bins - 1] + sh;
        o.w = lk[c.w < n_bins ? c.w : n_bins - 1] + sh;
        reinterpret_cast<float4*>(val)[i] = o;
    }
}

// generic rows (1-D tensors, un-chunked 2-D rows): exact source-order accumulation
__global__ __launch_bounds__(64) void k_scatter_rows(const uint8_t* __restrict__ idx12,
                                                     const int64_t* __restrict__ idx64,
                                                     const float* __restrict__ val, int64_t k_per_row,
                                                     int row_len, int reduce_mode, float* __restrict__ out,
                                                     int32_t* __restrict__ err) {
    __shared__ float acc[TPLR_MAX_ROW];
    __shared__ uint32_t cnt[TPLR_MAX_ROW];
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    for (int i = lane; i < row_len; i += 64) {
        acc[i] = 0.f;
        cnt[i] = 0;
    }
    __syncthreads();
    const uint8_t* irow = idx12 ? idx12 + row * (k_per_row + (k_per_row >> 1)) : nullptr;
    for (int64_t j0 = 0; j0 < k_per_row; j0 += 64) {
        const int64_t j = j0 + lane;
        int64_t ix = -1;
        float a = 0.f;
        if (j < k_per_row) {
            ix = idx12 ? static_cast<int64_t>(load_idx12(irow, static_cast<int>(j))) : idx64[row * k_per_row + j];
            a = val[row * k_per_row + j];
            if (ix < 0 || ix >= row_len) {
                if (err) atomicMax(err, ix < 0 || ix > 0x7fffffff ? 0x7fffffff : static_cast<int32_t>(ix));
                ix = -1;
            }
        }
        // rank among earlier lanes of this batch that hit the same destination
        const int me = static_cast<int>(ix);
        int rank = 0;
        for (int i = 0; i < 63; ++i) {
            const int other = __shfl(me, i);
            rank += (i < lane && other == me && me >= 0) ? 1 : 0;
        }
        int maxrank = rank;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int o = __shfl_xor(maxrank, off);
            maxrank = o > maxrank ? o : maxrank;
        }
        for (int r = 0; r <= maxrank; ++r) {
            if (me >= 0 && rank == r) {
                acc[me] += a;
                cnt[me] += 1;
            }
            __syncthreads();
        }
    }
    float* orow = out + row * row_len;
    for (int i = lane; i < row_len; i += 64) {
        const uint32_t c = cnt[i];
        const float s = acc[i];
        orow[i] = (reduce_mode == TPLR_REDUCE_MEAN && c > 1) ? s / static_cast<float>(c) : s;
    }
}

// =========================================================================================
// peer statistics
// =========================================================================================
struct ValPtrs {
    const float* val[TPLR_MAX_PEERS];
};

// Sum of squares of n values per peer in S slices: block (p, s) reduces the s-th of S equal runs
// and writes sumsq[p * S + s]; the consumer adds a peer's partial sums in order.  Eight
// independent accumulators per thread; the reduction order is fixed.
__global__ __launch_bounds__(1024) void k_peer_sumsq(const ValPtrs vp, int64_t n, int S, float* __restrict__ sumsq) {
    __shared__ float part[16];
    const int p = blockIdx.x / S, sl = blockIdx.x - p * S;
    const int64_t i0 = n * sl / S, i1 = n * (sl + 1) / S;
    const float* v = vp.val[p];
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int64_t i = i0 + threadIdx.x;
    for (; i + 7 * 1024 < i1; i += 8 * 1024) {
        float x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = v[i + u * 1024];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = __builtin_fmaf(x[u], x[u], acc[u]);
    }
    for (; i < i1; i += 1024) acc[0] = __builtin_fmaf(v[i], v[i], acc[0]);
    float s = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    s = wave_sum_f32(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int w = 0; w < 16; ++w) t += part[w];
        sumsq[blockIdx.x] = t;
    }
}

// Sum of squares of a tensor's part of a peer's values, in S slices: one block per (tensor,
// peer, slice), partial sums at sumsq[(t * P + p) * S + slice] (the consumer adds them in
// order).  A part starts at an even element (k is even), so it is read as float2.  The largest
// slice sets the duration of the launch, so a block keeps a lot in flight: 1024 threads with
// sixteen independent loads and accumulators each (128 KB per trip).  The reduction order is fixed.
__global__ __launch_bounds__(1024) void k_segment_sumsq(const ValPtrs vp, int P, int k, int S,
                                                        const tplr_tensor_desc* __restrict__ table,
                                                        float* __restrict__ sumsq) {
    constexpr int kT = 1024;
    __shared__ float part[kT / 64];
    // block = (tensor t, peer p, slice sl); a slice is a run of whole chunks
    const int tp = blockIdx.x / S, sl = blockIdx.x - tp * S;
    const int t = tp / P, p = tp - t * P;
    const tplr_tensor_desc d = table[t];
    const int64_t n_chunks = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const int64_t c0 = n_chunks * sl / S, c1 = n_chunks * (sl + 1) / S;
    // a slice is often no more than a few loads per lane (64 KB for a 2048 x 2048 parameter cut in two): four
    // independent streaming loads per trip, 16 bytes wide where rows of k values keep that alignment
    typedef float v2f __attribute__((ext_vector_type(2)));
    const float* base = vp.val[p] + (d.chunk_begin + c0) * k;
    const int64_t n = (c1 - c0) * k;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto sq4 = [](float a, v4f x) {
        return __builtin_fmaf(x.w, x.w, __builtin_fmaf(x.z, x.z, __builtin_fmaf(x.y, x.y, __builtin_fmaf(x.x, x.x, a))));
    };
    int64_t i = threadIdx.x;
    if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(base) & 15) == 0) {
        const v4f* v = reinterpret_cast<const v4f*>(base);
        const int64_t n4 = n >> 2;
        for (; i + 3 * kT < n4; i += 4 * kT) {
            v4f x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = __builtin_nontemporal_load(v + i + u * kT);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc[u] = sq4(acc[u], x[u]);
        }
        for (int u = 0; i < n4; i += kT, u = (u + 1) & 3) acc[u] = sq4(acc[u], __builtin_nontemporal_load(v + i));
    } else {
        const v2f* v = reinterpret_cast<const v2f*>(base);
        const int64_t n2 = n >> 1;
        for (; i + 3 * kT < n2; i += 4 * kT) {
            v2f x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = __builtin_nontemporal_load(v + i + u * kT);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc[u] = __builtin_fmaf(x[u].y, x[u].y, __builtin_fmaf(x[u].x, x[u].x, acc[u]));
        }
        for (; i < n2; i += kT) {
            const v2f x = __builtin_nontemporal_load(v + i);
            acc[0] = __builtin_fmaf(x.y, x.y, __builtin_fmaf(x.x, x.x, acc[0]));
        }
    }
    acc[0] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    const float s = wave_sum_f32(acc[0]);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < kT / 64; ++w) tot += part[w];
        sumsq[blockIdx.x] = tot;
    }
}

// Sum of squares of every row of k values of a flat payload: what a peer's norms are made of, taken once,
// when the payload arrives, so that the clip factors of a window cost a pass over one float per row instead
// of a second pass over the values.  The order of the additions is fixed: value j's square sits in lane j of
// a group of kW lanes (the power of two that holds k; zero where j >= k; rows longer than 64: lane j first adds
// the squares of values j, j + 64, ... in that order) and lane j adds lane j ^ off for off = kW/2 ... 1.
// 64 / kW rows per wave instruction, eight of them in flight per wave.
struct RowSumPtrs {
    float* out[TPLR_MAX_PEERS];
};
template <int kW>
__global__ __launch_bounds__(256) void k_row_sumsq(const ValPtrs vp, const RowSumPtrs op, int k, int64_t n_rows) {
    constexpr int kRows = 64 / kW;  // rows per trip of a wave
    constexpr int kFlight = 8;
    const int lane = threadIdx.x & 63;
    const int j = lane & (kW - 1);
    const float* __restrict__ val = vp.val[blockIdx.y];
    float* __restrict__ out = op.out[blockIdx.y];
    const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int64_t trips = (n_rows + kRows - 1) / kRows;
    for (int64_t t0 = wave * kFlight; t0 < trips; t0 += waves * kFlight) {
        float x[kFlight];
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
            const int64_t row = (t0 + u) * kRows + lane / kW;
            float acc = 0.f;
            if (row < n_rows) {
                if (kW < 64 || k <= 64) {
                    const float v = j < k ? __builtin_nontemporal_load(val + row * k + j) : 0.f;
                    acc = v * v;
                } else {
                    for (int e = j; e < k; e += 64) {
                        const float v = __builtin_nontemporal_load(val + row * k + e);
                        acc = __builtin_fmaf(v, v, acc);
                    }
                }
            }
            x[u] = acc;
        }
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
#pragma unroll
            for (int off = kW / 2; off > 0; off >>= 1) x[u] += __shfl_xor(x[u], off);
            const int64_t row = (t0 + u) * kRows + lane / kW;
            if (j == 0 && row < n_rows) out[row] = x[u];
        }
    }
}

// The same figures with 16-byte loads, for rows of k <= 64 values with k a multiple of four that start on
// 16-byte boundaries: kW / 4 lanes per row, lane m holds the squares of values 4m .. 4m + 3 (zero past k).  The
// tree above pairs value j with value j ^ off: for off >= 4 that is the same component of lane m ^ (off / 4),
// for off = 2 and 1 components of the lane itself - the same additions in the same order, so the same bits.
template <int kW>
__global__ __launch_bounds__(256) void k_row_sumsq_vec(const ValPtrs vp, const RowSumPtrs op, int k, int64_t n_rows) {
    constexpr int kLanes = kW / 4;      // lanes per row
    constexpr int kRows = 64 / kLanes;  // rows per trip of a wave
    constexpr int kFlight = 8;
    const int lane = threadIdx.x & 63;
    const int m = lane & (kLanes - 1);
    const float* __restrict__ val = vp.val[blockIdx.y];
    float* __restrict__ out = op.out[blockIdx.y];
    const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int64_t trips = (n_rows + kRows - 1) / kRows;
    const bool in_row = 4 * m < k;
    for (int64_t t0 = wave * kFlight; t0 < trips; t0 += waves * kFlight) {
        v4f x[kFlight];
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
            const int64_t row = (t0 + u) * kRows + lane / kLanes;
            x[u] = (v4f){0.f, 0.f, 0.f, 0.f};
            if (row < n_rows && in_row)
                x[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(val + row * k) + m);
        }
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
            v4f q = x[u] * x[u];
#pragma unroll
            for (int off = kLanes / 2; off > 0; off >>= 1) {
                q.x += __shfl_xor(q.x, off);
                q.y += __shfl_xor(q.y, off);
                q.z += __shfl_xor(q.z, off);
                q.w += __shfl_xor(q.w, off);
            }
            const float r = (q.x + q.z) + (q.y + q.w);
            const int64_t row = (t0 + u) * kRows + lane / kLanes;
            if (m == 0 && row < n_rows) out[row] = r;
        }
    }
}

// Partial sums over a tensor's rows of such per-row figures, in double: block (tensor t, peer p, slice s) adds
// the rows of slice s of tensor t (thread i the rows i, i + 256, ... in that order, then the fixed tree of
// block256_sum_f64) into partial[(t * P + p) * S + s].
struct RowSumConstPtrs {
    const float* in[TPLR_MAX_PEERS];
};
__global__ __launch_bounds__(256) void k_rowsum_partials(const RowSumConstPtrs rp, int P, int S,
                                                         const tplr_tensor_desc* __restrict__ table,
                                                         double* __restrict__ partial) {
    __shared__ double part[4];
    const int tp = blockIdx.x / S, sl = blockIdx.x - tp * S;
    const int t = tp / P, p = tp - t * P;
    const tplr_tensor_desc d = table[t];
    const int64_t n = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const int64_t c0 = n * sl / S, c1 = n * (sl + 1) / S;
    const float* __restrict__ s = rp.in[p] + d.chunk_begin;
    double acc = 0.0;
    int64_t i = c0 + threadIdx.x;
    for (; i + 768 < c1; i += 1024) {  // four independent loads in flight, added in the order of the rows
        const float a0 = s[i], a1 = s[i + 256], a2 = s[i + 512], a3 = s[i + 768];
        acc += static_cast<double>(a0);
        acc += static_cast<double>(a1);
        acc += static_cast<double>(a2);
        acc += static_cast<double>(a3);
    }
    for (; i < c1; i += 256) acc += static_cast<double>(s[i]);
    acc = block256_sum_f64(acc, part, threadIdx.x);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

// one block per tensor: scale[t][p] = min(1, med_t / (norm[t][p] + 1e-8))
// Partial: float (partial sums of squares added in float) or double (added in double, the norm rounded once)
template <typename Partial>
__global__ __launch_bounds__(128) void k_clip_scales(const Partial* __restrict__ norm, int P, int n_partials,
                                                     float* __restrict__ scale, float* __restrict__ median) {
    __shared__ float nv[TPLR_MAX_PEERS];
    __shared__ float med;
    const int i = threadIdx.x;
    const int64_t off = static_cast<int64_t>(blockIdx.x) * P;
    if (i < P) {
        if (n_partials > 0) {  // partial sums of squares, added in order
            const Partial* ps = norm + (off + i) * n_partials;
            Partial tot = 0;
            for (int s = 0; s < n_partials; ++s) tot += ps[s];
            if constexpr (sizeof(Partial) == 4)
                nv[i] = __builtin_sqrtf(tot);
            else
                nv[i] = static_cast<float>(__builtin_sqrt(tot));
        } else {
            nv[i] = static_cast<float>(norm[off + i]);
        }
    }
    __syncthreads();
    if (i < P) {
        // rank in a total order: ascending, NaN after everything, ties by peer - exactly one lane holds
        // the middle rank.  torch.median (:535) gives NaN as soon as one norm is NaN, and the lower
        // of the two middle values otherwise.
        int rank = 0;
        bool any_nan = false;
        const float mine = nv[i];
        const bool mine_nan = mine != mine;
        for (int j = 0; j < P; ++j) {
            const float other = nv[j];
            const bool other_nan = other != other;
            any_nan |= other_nan;
            const bool before = mine_nan ? (!other_nan || j < i) : (!other_nan && (other < mine || (other == mine && j < i)));
            rank += before ? 1 : 0;
        }
        if (rank == (P - 1) / 2) med = any_nan ? __builtin_nanf("") : mine;
    }
    __syncthreads();
    if (i < P) {
        const float f = med / (nv[i] + 1e-8f);
        scale[off + i] = f > 1.0f ? 1.0f : f;  // clamp(max=1); NaN propagates as in torch.clamp
    }
    if (i == 0 && median) median[blockIdx.x] = med;
}

// Per-tensor factor 1 / (||x_t|| + eps) from per-chunk sums of squares (as tplr_decode_aggregate_batch
// writes them): one block per tensor, the chunks' sums added in a fixed order.
__global__ __launch_bounds__(256) void k_tensor_rnorm(const float* __restrict__ sumsq,
                                                      const tplr_tensor_desc* __restrict__ table, float eps,
                                                      float* __restrict__ factor) {
    __shared__ double part[4];
    const tplr_tensor_desc d = table[blockIdx.x];
    const int64_t n = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const float* s = sumsq + d.chunk_begin;
    double acc = 0.0;
    {  // four independent loads in flight per thread: the largest tensors have tens of thousands of chunks
        int64_t i = threadIdx.x;
        for (; i + 768 < n; i += 1024) {
            const float a0 = s[i], a1 = s[i + 256], a2 = s[i + 512], a3 = s[i + 768];
            acc += (static_cast<double>(a0) + static_cast<double>(a1)) + (static_cast<double>(a2) + static_cast<double>(a3));
        }
        for (; i < n; i += 256) acc += static_cast<double>(s[i]);
    }
    acc = block256_sum_f64(acc, part, threadIdx.x);
    if (threadIdx.x == 0) factor[blockIdx.x] = 1.0f / (static_cast<float>(sqrt(acc)) + eps);
}

// x <- x * factor[t] for every chunk of a batch (the per-tensor normalisation that follows an aggregate):
// 16 KB read and written per chunk, persistent, one chunk's 64 row loads in flight ahead of its stores.
__global__ __launch_bounds__(64) void k_scale_chunks(const tplr_tensor_desc* __restrict__ table, int n_tensors,
                                                     int64_t total, const float* __restrict__ factor) {
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    Cursor c;
    tplr_tensor_desc none = {};
    cursor_seek(c, table, none, n_tensors, g0);
    for (int64_t g = g0; g < g1; ++g) {
        float v[64];
        load_chunk_cols(v, c, lane);
        const float f = factor[c.t];
#pragma unroll
        for (int r = 0; r < 64; ++r) v[r] *= f;
        store_chunk_cols(v, (float*)c.base, c.ld, c.y, c.xc, lane);
        if (g + 1 < g1) cursor_next(c, g + 1);
    }
}

// Per-chunk sum of squares of the peers' summed coefficients, from the payloads alone: nothing is transformed
// and no dense element is written.  The transform is orthonormal, so a tensor's L2 norm after the inverse
// transform is the norm of its summed coefficients, and a per-tensor normalisation can be folded into the
// factors of the one aggregate launch that follows instead of taking a pass of its own over the dense tensors.
// A unit is one peer's entries 64 m .. 64 m + 63 of the chunk (one wave instruction); units are taken kUnits
// at a time, the next round's payload requested before this round is scattered.  Sums are plain
// read-add-write through the claiming exchange (see tile_claim): entries of one instruction that name the
// same coefficient send the chunk through floating-point atomics instead.  The tile is read back and cleared
// 16 bytes per lane at a time, every lane adding its squares in a fixed order.
// kOneRound: k <= 64 and at most kUnits peers - unit i is peer i, one round per chunk, no unit arithmetic.
template <int kUnits, bool kOneRound>
__global__ __launch_bounds__(64) void k_aggregate_sumsq(const PeerPtrs pp, const float* __restrict__ scale, int P,
                                                        int k, const tplr_tensor_desc* __restrict__ table,
                                                        int n_tensors, int64_t total, float* __restrict__ sumsq) {
    __shared__ __align__(16) float tile[kChunk * kChunk];
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1);
    if (g0 >= g1) return;
    const int64_t idx_stride = k + (k >> 1);
    const int M = kOneRound ? 1 : (k + 63) >> 6;               // wave instructions per peer and chunk
    const int U = P * M;                                       // units per chunk
    const int nb = kOneRound ? 1 : (U + kUnits - 1) / kUnits;  // rounds per chunk
    float4* const tile4 = reinterpret_cast<float4*>(tile);
#pragma unroll
    for (int q = 0; q < 16; ++q) tile4[q * 64 + lane] = make_float4(0.f, 0.f, 0.f, 0.f);
    wave_lds_fence();

    uint32_t ix[2][kUnits];
    float a[2][kUnits];
    int t_of[2] = {0, 0};
    Cursor c;
    tplr_tensor_desc none = {};
    cursor_seek(c, table, none, n_tensors, g0);
    int64_t lg = g0;  // the round requested next: chunk and round number
    int lr = 0;
    auto unit_peer = [&](int u, int& m) -> int {  // wave-uniform
        if constexpr (kOneRound) {
            m = 0;
            return u;
        }
        const int p = u / M;
        m = u - p * M;
        return p;
    };
    auto request = [&](auto sel) {
        constexpr int s = decltype(sel)::value;
        if (lg >= g1) return;
        t_of[s] = c.t;
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            const int u = kOneRound ? i : lr * kUnits + i;
            if (u < U) {  // wave-uniform
                int m;
                const int p = unit_peer(u, m);
                const int j = m * 64 + lane;
                const int je = j < k ? j : 0;
                const gbyte* irow = (const gbyte*)pp.idx[p] + lg * idx_stride;
                ix[s][i] = *(const gu16*)(irow + (3 * (je >> 1) + (je & 1)));
                a[s][i] = ((const gfloat*)pp.val[p] + lg * k)[je];
            }
        }
        if (++lr == nb) {
            lr = 0;
            if (++lg < g1) cursor_next(c, lg);
        }
    };

    auto read_back = [&]() -> float {  // sum of squares of the tile, which it leaves cleared
        wave_lds_fence();
        float ss = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const float4 t = tile4[q * 64 + lane];
            ss = __builtin_fmaf(t.w, t.w, __builtin_fmaf(t.z, t.z, __builtin_fmaf(t.y, t.y, __builtin_fmaf(t.x, t.x, ss))));
            tile4[q * 64 + lane] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        wave_lds_fence();
        return wave_sum_f32(ss);
    };

    int64_t pg = g0;  // the round scattered next
    int pr = 0;
    uint32_t repeat = 0;
    auto scatter = [&](auto sel) {
        constexpr int s = decltype(sel)::value;
        const int t = t_of[s];
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
            const int u = kOneRound ? i : pr * kUnits + i;
            if (u < U) {  // wave-uniform
                int m;
                const int p = unit_peer(u, m);
                const int j = m * 64 + lane;
                const float sc = scale ? scale[static_cast<int64_t>(t) * P + p] : 1.0f;
                if (j < k) {
                    const uint32_t e = (j & 1) ? (ix[s][i] >> 4) : (ix[s][i] & 0xfffu);
                    const float cur = tile_claim(&tile[e]);
                    repeat = seen_mark(repeat, cur);
                    tile[e] = cur + a[s][i] * sc;
                }
            }
        }
        if (++pr < nb) return;
        // the chunk is complete
        float ss = read_back();
        if (__ballot(repeat == kClaimMark) != 0) {  // wave-uniform, false for top-k payloads
            for (int p = 0; p < P; ++p) {
                const float sc = scale ? scale[static_cast<int64_t>(t) * P + p] : 1.0f;
                const gbyte* irow = (const gbyte*)pp.idx[p] + pg * idx_stride;
                const gfloat* vrow = (const gfloat*)pp.val[p] + pg * k;
                for (int j = lane; j < k; j += 64) {
                    const uint32_t w = *(const gu16*)(irow + (3 * (j >> 1) + (j & 1)));
                    atomicAdd(&tile[(j & 1) ? (w >> 4) : (w & 0xfffu)], vrow[j] * sc);
                }
            }
            ss = read_back();
            repeat = 0;
        }
        if (lane == 0) sumsq[pg] = ss;
        pr = 0;
        ++pg;
    };

    request(std::integral_constant<int, 0>{});
    while (pg < g1) {
        request(std::integral_constant<int, 1>{});
        scatter(std::integral_constant<int, 0>{});
        if (pg >= g1) break;
        request(std::integral_constant<int, 0>{});
        scatter(std::integral_constant<int, 1>{});
    }
}

// From those sums: tensor t's factor 1 / (sqrt(sum of its entries) * pre + eps), and pre times that factor
// as the P aggregate factors of the tensor (pre = 1 / P makes the aggregate the normalised mean over P peers).
__global__ __launch_bounds__(256) void k_tensor_rnorm_scales(const float* __restrict__ sumsq,
                                                             const tplr_tensor_desc* __restrict__ table, float eps,
                                                             float pre, int P, float* __restrict__ factor,
                                                             float* __restrict__ scale) {
    __shared__ double part[4];
    __shared__ float f_all;
    const tplr_tensor_desc d = table[blockIdx.x];
    const int64_t n = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const float* s = sumsq + d.chunk_begin;
    double acc = 0.0;
    {  // four independent loads in flight per thread: the largest tensors have tens of thousands of chunks
        int64_t i = threadIdx.x;
        for (; i + 768 < n; i += 1024) {
            const float a0 = s[i], a1 = s[i + 256], a2 = s[i + 512], a3 = s[i + 768];
            acc += (static_cast<double>(a0) + static_cast<double>(a1)) + (static_cast<double>(a2) + static_cast<double>(a3));
        }
        for (; i < n; i += 256) acc += static_cast<double>(s[i]);
    }
    acc = block256_sum_f64(acc, part, threadIdx.x);
    if (threadIdx.x == 0) {
        const float f = 1.0f / (static_cast<float>(sqrt(acc)) * pre + eps);
        if (factor) factor[blockIdx.x] = f;
        f_all = f * pre;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += 256) scale[static_cast<int64_t>(blockIdx.x) * P + p] = f_all;
}

// What the caller of the aggregate looks at next, per tensor (src/tplr/neurons.py:380-385: L2 norm and mean of
// the decoded gradient; :411 and :438: is every element finite), from the two floats per chunk the aggregate
// kernel leaves when asked - no further pass over the dense tensors.  One workgroup per tensor; the chunks'
// figures are added in double, in a fixed order.  out[t]: {norm, mean, 1.0 if all finite else 0.0, sum of squares}.
// A chunk whose sum of squares (or sum) is not finite either holds a non-finite element or overflowed in
// fp32: its 4096 elements are read back and examined one by one, and where they are all finite their figures
// are formed again in double, so the flag is exact and the norm survives values near the top of the range.
// use_dct bit 1: the tensors of `table` do not hold the values the figures are about (an update subtracted them
// from its parameters): nothing is read back, and a figure that is not finite marks the tensor.
__global__ __launch_bounds__(256) void k_tensor_stats(const float* __restrict__ chunk_stats,
                                                      const tplr_tensor_desc* __restrict__ table, int use_dct,
                                                      float* __restrict__ out) {
    const bool figures_only = (use_dct & 2) != 0;
    use_dct &= 1;
    __shared__ double part[4];
    __shared__ int bad_any;
    const tplr_tensor_desc d = table[blockIdx.x];
    const int64_t n = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    if (threadIdx.x == 0) bad_any = 0;
    __syncthreads();
    double acc_ss = 0.0, acc_sm = 0.0;
    int bad = 0;
    const float2* cs = reinterpret_cast<const float2*>(chunk_stats) + d.chunk_begin;
    // one chunk's figures; not finite: the chunk is read back (rare)
    auto take = [&](int64_t i, float2 got) {
        double ss = static_cast<double>(got.x), sm = static_cast<double>(got.y);
        if (figures_only) {
            if (!isfinite(ss) || !isfinite(sm)) bad = 1;
        } else if (!isfinite(ss) || !isfinite(sm)) {
            const bool rows = use_dct || d.ld > 0;  // the (R, C) tensor itself, or chunk after chunk
            const int64_t y = i / d.x_chunks, x = i - y * d.x_chunks;
            const float* c0 = rows ? static_cast<const float*>(d.dense) + (y * 64) * d.ld + x * 64
                                   : static_cast<const float*>(d.dense) + i * 4096;
            const int64_t ld = rows ? d.ld : 64;
            ss = 0.0;
            sm = 0.0;
#pragma unroll 1
            for (int r = 0; r < 64; ++r)
#pragma unroll 1
                for (int c = 0; c < 64; ++c) {
                    const float v = c0[r * ld + c];
                    if (!isfinite(v)) bad = 1;
                    ss += static_cast<double>(v) * static_cast<double>(v);
                    sm += static_cast<double>(v);
                }
        }
        acc_ss += ss;
        acc_sm += sm;
    };
    {  // four independent loads in flight per thread: the largest tensors have tens of thousands of chunks
        int64_t i = threadIdx.x;
        for (; i + 768 < n; i += 1024) {
            const float2 g0 = cs[i], g1 = cs[i + 256], g2 = cs[i + 512], g3 = cs[i + 768];
            take(i, g0), take(i + 256, g1), take(i + 512, g2), take(i + 768, g3);
        }
        for (; i < n; i += 256) take(i, cs[i]);
    }
    if (bad) bad_any = 1;  // (every writer writes the same value)
    acc_ss = block256_sum_f64(acc_ss, part, threadIdx.x);
    __syncthreads();
    acc_sm = block256_sum_f64(acc_sm, part, threadIdx.x);
    __syncthreads();
    if (threadIdx.x == 0) {
        float* o = out + 4 * static_cast<int64_t>(blockIdx.x);
        o[0] = static_cast<float>(sqrt(acc_ss));
        o[1] = n > 0 ? static_cast<float>(acc_sm / (static_cast<double>(n) * 4096.0)) : 0.0f;
        o[2] = bad_any ? 0.0f : 1.0f;
        o[3] = static_cast<float>(acc_ss);
    }
}

// The 1-D parameters of a set (rows of 64 elements) decoded where they lie: what k_aggregate_rows leaves for a
// row, then the 64-point inverse transform and its scale exactly as k_dct1d applies them, written into the
// row's tensor.  One wave per row, a handful of rows per parameter: every peer's entries of the row are
// requested at once (32 peers to a round), so a row waits for one memory round trip instead of one per peer,
// and the row's transform runs on one lane (the same instruction sequence as on any lane of k_dct1d).
template <bool kUseDct>
__global__ __launch_bounds__(64) void k_decode_rows64(const PeerPtrs pp, const float* __restrict__ scale, int P, int k,
                                                      const tplr_tensor_desc* __restrict__ table, int n_tensors,
                                                      int reduce_mode, int32_t* __restrict__ err) {
    __shared__ float acc[64];
    __shared__ uint32_t cnt[64];
    __shared__ uint32_t tag[64];
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    acc[lane] = 0.f;
    cnt[lane] = 0;
    int t = 0;
    {  // the tensor this row belongs to: the last one that begins at or before it
        int lo = 0, hi = n_tensors;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table[mid].chunk_begin <= row)
                lo = mid;
            else
                hi = mid;
        }
        t = lo;
    }
    const tplr_tensor_desc d = table[t];
    wave_lds_fence();
    const int64_t idx_stride = k + (k >> 1);
    constexpr int kRound = 32;
    for (int p0 = 0; p0 < P; p0 += kRound) {
        int me[kRound];
        float a[kRound];
#pragma unroll
        for (int i = 0; i < kRound; ++i) {
            me[i] = -1;
            a[i] = 0.f;
            if (p0 + i < P && lane < k) {
                const int p = p0 + i;
                const gbyte* irow = (const gbyte*)pp.idx[p] + row * idx_stride;
                const gfloat* vrow = (const gfloat*)pp.val[p] + row * k;
                const float s = scale ? scale[static_cast<int64_t>(t) * P + p] : 1.0f;
                me[i] = static_cast<int>(load_idx12(irow, lane));
                a[i] = vrow[lane] * s;
            }
        }
#pragma unroll
        for (int i = 0; i < kRound; ++i) {
            if (p0 + i >= P) continue;  // wave-uniform
            int m = me[i];
            if (m >= 64) {
                if (err) atomicMax(err, m);
                m = -1;
            }
            // the usual case: the entries name distinct elements
            if (m >= 0) tag[m] = static_cast<uint32_t>(lane);
            wave_lds_fence();
            const bool clash = m >= 0 && tag[m] != static_cast<uint32_t>(lane);
            if (__ballot(clash) == 0) {
                if (m >= 0) {
                    acc[m] += a[i];
                    cnt[m] += 1;
                }
            } else {
                // rank among the earlier lanes that name the same element; one rank per turn
                int rank = 0;
                for (int l = 0; l < 63; ++l) {
                    const int other = __shfl(m, l);
                    rank += (l < lane && other == m && m >= 0) ? 1 : 0;
                }
                const int maxrank = static_cast<int>(wave_max_u32(static_cast<uint32_t>(rank)));
                for (int r = 0; r <= maxrank; ++r) {
                    if (m >= 0 && rank == r) {
                        acc[m] += a[i];
                        cnt[m] += 1;
                    }
                    wave_lds_fence();
                }
            }
            wave_lds_fence();
        }
    }
    const uint32_t c = cnt[lane];
    float v = acc[lane];
    v = (reduce_mode == TPLR_REDUCE_MEAN && c > 1) ? v / static_cast<float>(c) : v;
    if (kUseDct) {
        wave_lds_fence();
        acc[lane] = v;
        wave_lds_fence();
        if (lane == 0) {
            float w[64];
#pragma unroll
            for (int e = 0; e < 64; ++e) w[e] = acc[e];
            dct64_inv(w);
#pragma unroll
            for (int e = 0; e < 64; ++e) acc[e] = w[e] * 0.17677669529663687f;  // one pass is sqrt(32) times the orthonormal transform
        }
        wave_lds_fence();
        v = acc[lane];
    }
    static_cast<float*>(d.dense)[(row - d.chunk_begin) * 64 + lane] = v;
}

// Per-peer, per-tensor sums of squares of the values behind a payload of codes (quantiser of at most four
// bins), from the codes alone: a value is one of four, so the sum is four counts times four squares.  Block
// = (tensor, peer, slice) as in k_segment_sumsq, whose output layout this has; a code is two bits in a byte, and
// a 32-bit word's four codes are counted with three byte-sum instructions (bit 0 set, bit 1 set, both set).
// A code that the quantiser cannot have produced (>= n_bins) is reported through `bad` (atomic maximum of
// the offending byte): the reference's table lookup raises on it (src/tplr/compress.py:641).
struct CodePtrs {
    const uint8_t* code[TPLR_MAX_PEERS];
};
__global__ __launch_bounds__(256) void k_code_sumsq4(const CodePtrs cp, int P, int k, int S,
                                                     const tplr_tensor_desc* __restrict__ table, int n_bins,
                                                     const float* __restrict__ deq, float* __restrict__ sumsq,
                                                     int32_t* __restrict__ bad) {
    __shared__ uint32_t part[4][4];
    const int tp = blockIdx.x / S, sl = blockIdx.x - tp * S;
    const int t = tp / P, p = tp - t * P;
    const tplr_tensor_desc d = table[t];
    const int64_t n_chunks = static_cast<int64_t>(d.x_chunks) * d.y_chunks;
    const int64_t c0 = n_chunks * sl / S, c1 = n_chunks * (sl + 1) / S;
    const uint8_t* base = cp.code[p] + (d.chunk_begin + c0) * k;
    const int64_t n = (c1 - c0) * k;
    uint32_t n0 = 0, n1 = 0, n11 = 0, over = 0;
    auto word = [&](uint32_t w) {
        const uint32_t b0 = w & 0x01010101u, b1 = (w >> 1) & 0x01010101u;
        n0 = __builtin_amdgcn_sad_u8(b0, 0u, n0);
        n1 = __builtin_amdgcn_sad_u8(b1, 0u, n1);
        n11 = __builtin_amdgcn_sad_u8(b0 & b1, 0u, n11);
        over |= w & 0xfcfcfcfcu;
    };
    // bytes up to the first 16-byte boundary and after the last one go one at a time (a byte alone is a word
    // whose other codes are zero: they add to no count)
    const int64_t head = n < 16 ? n : ((16 - (reinterpret_cast<uintptr_t>(base) & 15)) & 15);
    const int64_t body = (n - head) >> 4;
    const int64_t tail0 = head + (body << 4);
    for (int64_t i = threadIdx.x; i < head; i += 256) word(base[i]);
    for (int64_t i = tail0 + threadIdx.x; i < n; i += 256) word(base[i]);
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const v4u* v = reinterpret_cast<const v4u*>(base + head);
    int64_t i = threadIdx.x;
    for (; i + 7 * 256 < body; i += 8 * 256) {  // eight independent loads in flight per lane
        v4u x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = __builtin_nontemporal_load(v + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; ++u) word(x[u].x), word(x[u].y), word(x[u].z), word(x[u].w);
    }
    for (; i < body; i += 256) {
        const v4u x = __builtin_nontemporal_load(v + i);
        word(x.x), word(x.y), word(x.z), word(x.w);
    }
    n0 = wave_sum_u32(n0), n1 = wave_sum_u32(n1), n11 = wave_sum_u32(n11);
    over = wave_max_u32(over);
    if ((threadIdx.x & 63) == 0) {
        uint32_t* o = part[threadIdx.x >> 6];
        o[0] = n0, o[1] = n1, o[2] = n11, o[3] = over;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint64_t a0 = 0, a1 = 0, a11 = 0;
        uint32_t ov = 0;
        for (int w = 0; w < 4; ++w) a0 += part[w][0], a1 += part[w][1], a11 += part[w][2], ov |= part[w][3];
        const uint64_t cnt[4] = {static_cast<uint64_t>(n) - a0 - a1 + a11, a0 - a11, a1 - a11, a11};
        const float* dq = deq + (static_cast<int64_t>(t) * P + p) * 4;
        double ss = 0.0;
        for (int b = 0; b < 4; ++b)
            if (cnt[b]) ss += static_cast<double>(cnt[b]) * static_cast<double>(dq[b]) * static_cast<double>(dq[b]);
        sumsq[blockIdx.x] = static_cast<float>(ss);
        int worst = 0;
        if (ov) worst = 255;  // (some byte of the slice has a bit beyond the two a code may use)
        for (int b = n_bins; b < 4; ++b)
            if (cnt[b]) worst = worst > b ? worst : b;
        if (worst && bad) atomicMax(bad, worst);
    }
}

// Plain streaming copy (16 bytes per lane per step, grid-stride).  It exists so that hardware
// traffic counters can be calibrated: it moves exactly n16 * 16 bytes each way.
__global__ __launch_bounds__(256) void k_calib_copy(const v4f* __restrict__ src, v4f* __restrict__ dst, int64_t n16) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Plain fill over a linear address range (16 bytes per lane per step): the write rate of the memory system with
// the friendliest access pattern there is, the figure the aggregate's chunk-pattern stores are held against.
// kPattern 0: grid-stride, neighbouring workgroups write neighbouring kilobytes; 1: the same with streaming stores;
// 2: every wave walks a contiguous span of its own, one kilobyte per step, as a persistent kernel would.
template <int kPattern>
__global__ __launch_bounds__(256) void k_calib_fill(v4f* __restrict__ dst, int64_t n16, float value) {
    const v4f v = {value, value, value, value};
    if constexpr (kPattern == 2) {
        const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
        const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
        const int64_t per = ((n16 + waves - 1) / waves + 63) & ~int64_t{63};
        const int64_t a = wave * per, b = a + per < n16 ? a + per : n16;
        for (int64_t i = a + (threadIdx.x & 63); i < b; i += 64) dst[i] = v;
    } else {
        const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
        for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n16; i += stride) {
            if constexpr (kPattern == 1)
                __builtin_nontemporal_store(v, dst + i);
            else
                dst[i] = v;
        }
    }
}

// The memory side of the fast aggregate alone: same grid, same chunk ranges, the same payload loads and the
// same 64 row stores per chunk, no scatter and no transform (what it stores is meaningless).  kGroup = 0: one
// two-byte index load per peer and chunk, as the kernels without the transform issue them; kGroup = 4 or 2:
// one four-byte load per peer and group of that many chunks, as the pipeline with the transform does.
template <int kGroup>
__global__ __launch_bounds__(64, 2) void k_calib_aggregate(const PeerPtrs pp, int P, int k,
                                                           const tplr_tensor_desc* __restrict__ table, int n_tensors,
                                                           int64_t total) {
    const int lane = threadIdx.x;
    int64_t g0, g1;
    my_range(total, g0, g1, kGroup ? kGroup : 1);
    if (g0 >= g1) return;
    const int64_t idx_stride = k + (k >> 1);
    const int le = lane < k ? lane : 0;
    const uint32_t lane_ioff = 3u * (static_cast<uint32_t>(le) >> 1) + (le & 1);
    constexpr int kU = 24;
    uint32_t ix[2][kU];
    float a[2][kU];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < kU; ++i) ix[s][i] = 0, a[s][i] = 0.f;
    auto load = [&](int s, int64_t g, auto with_group) {
        // (a group's lanes as the kernel places them: four bytes at 3 * lane, kept inside the rows of this launch)
        int64_t room = (total - g) * idx_stride;
        if (kGroup && room > kGroup * idx_stride) room = kGroup * idx_stride;
        room = room < 4 ? 0 : room - 4;
        const int64_t goff = 3 * lane < room ? 3 * lane : room;
#pragma unroll
        for (int i = 0; i < kU; ++i) {
            if (i < P) {  // wave-uniform
                const gbyte* irow = (const gbyte*)pp.idx[i] + g * idx_stride;
                const gfloat* vrow = (const gfloat*)pp.val[i] + g * k;
                if constexpr (kGroup == 0)
                    ix[s][i] = __builtin_nontemporal_load((const gu16*)(irow + lane_ioff));
                else if constexpr (decltype(with_group)::value)
                    ix[0][i] = __builtin_nontemporal_load((const gu32*)(irow + goff));
                a[s][i] = __builtin_nontemporal_load(vrow + le);
            }
        }
    };
    Cursor c;
    tplr_tensor_desc none = {};
    cursor_seek(c, table, none, n_tensors, g0);
    load(0, g0, std::true_type{});
    load(1, g0 + 1 < g1 ? g0 + 1 : g0, std::false_type{});
    auto chunk = [&](int64_t g, int s, auto with_group) {
        float x = 0.f;
#pragma unroll
        for (int i = 0; i < kU; ++i) x += a[s][i] + __builtin_bit_cast(float, ix[kGroup ? 0 : s][i]);
        load(s, g + 2 < g1 ? g + 2 : g1 - 1, with_group);
        float v[64];
#pragma unroll
        for (int r = 0; r < 64; ++r) v[r] = x + static_cast<float>(r);
        store_chunk_cols(v, (float*)c.base, c.ld, c.y, c.xc, lane);
        if (g + 1 < g1) cursor_next(c, g + 1);
    };
    // the payload requested while chunk g is stored is that of chunk g + 2: a group starts there every kGroup chunks
    if constexpr (kGroup == 4) {
        for (int64_t g = g0; g < g1; g += 4) {
            chunk(g, 0, std::false_type{});
            if (g + 1 < g1) chunk(g + 1, 1, std::false_type{});
            if (g + 2 < g1) chunk(g + 2, 0, std::true_type{});
            if (g + 3 < g1) chunk(g + 3, 1, std::false_type{});
        }
    } else {
        for (int64_t g = g0; g < g1; g += 2) {
            chunk(g, 0, std::true_type{});
            if (g + 1 < g1) chunk(g + 1, 1, std::false_type{});
        }
    }
}

// The same for the launches whose workgroups are teams of four waves: wave w takes chunks w, w + 4, ... of the
// team's range and the team meets at a barrier before every chunk's stores.  kGroup = 4 or 2 (with the transform):
// a group's index rows are four rows apart (lanes c k/2 .. take the row of the group's chunk c; cached loads);
// kGroup = 0 (without it): one two-byte index load per peer and chunk.
template <int kGroup>
__global__ __launch_bounds__(256, 2) void k_calib_aggregate_team(const PeerPtrs pp, int P, int k,
                                                                 const tplr_tensor_desc* __restrict__ table,
                                                                 int n_tensors, int64_t total) {
    constexpr int T = 4;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    int64_t t0, t1;
    my_range(total, t0, t1, T);
    if (t0 >= t1) return;
    const int64_t idx_stride = k + (k >> 1), idx_end = total * idx_stride;
    const int le = lane < k ? lane : 0;
    const uint32_t lane_ioff = 3u * (static_cast<uint32_t>(le) >> 1) + (le & 1);
    int lane_goff = 0;
    if constexpr (kGroup > 0) {
        const int half_k = k >> 1;
        int c = lane / half_k, q = lane - c * half_k;
        if (c >= kGroup) c = kGroup - 1, q = half_k - 1;
        lane_goff = c * T * static_cast<int>(idx_stride) + 3 * q;
    }
    constexpr int kU = kGroup > 0 ? 16 : 24;
    uint32_t ix[kU], ix2[2][kGroup > 0 ? 1 : kU];
    float a[2][kU];
#pragma unroll
    for (int i = 0; i < kU; ++i) {
        ix[i] = 0, a[0][i] = 0.f, a[1][i] = 0.f;
        if constexpr (kGroup == 0) ix2[0][i] = ix2[1][i] = 0;
    }
    const int64_t steps = (t1 - t0 + T - 1) / T;  // of the team; a wave past the end repeats its last chunk and stores nothing
    auto clampg = [&](int64_t g) { return g < t1 ? g : t1 - 1; };
    auto load_group = [&](int64_t g) {
        const int64_t want = clampg(g) * idx_stride + lane_goff;
        const int64_t from = want < idx_end - 4 ? want : idx_end - 4;
#pragma unroll
        for (int i = 0; i < kU; ++i)
            if (i < P) ix[i] = *(const gu32*)((const gbyte*)pp.idx[i] + from);
    };
    auto load_vals = [&](auto st, int64_t g) {
        constexpr int s = decltype(st)::value;
#pragma unroll
        for (int i = 0; i < kU; ++i)
            if (i < P) {
                if constexpr (kGroup > 0) {
                    a[s][i] = __builtin_nontemporal_load((const gfloat*)pp.val[i] + clampg(g) * k + le);
                } else {  // (as the kernel without the transform loads them: cached, two bytes of indices per chunk)
                    ix2[s][i] = *(const gu16*)((const gbyte*)pp.idx[i] + clampg(g) * idx_stride + lane_ioff);
                    a[s][i] = ((const gfloat*)pp.val[i] + clampg(g) * k)[le];
                }
            }
    };
    Cursor c;
    tplr_tensor_desc none = {};
    cursor_seek(c, table, none, n_tensors, clampg(t0 + w));
    if constexpr (kGroup > 0) load_group(t0 + w);
    load_vals(Index<0>{}, t0 + w);
    load_vals(Index<1>{}, t0 + w + T);
    auto body = [&](int64_t gb, auto st, bool with_group) {
        const int64_t g = gb + w;
        float x = 0.f;
#pragma unroll
        for (int i = 0; i < kU; ++i)
            x += a[decltype(st)::value][i] +
                 __builtin_bit_cast(float, kGroup > 0 ? ix[i] : ix2[decltype(st)::value][kGroup > 0 ? 0 : i]);
        if constexpr (kGroup > 0) {
            if (with_group) load_group(g + 2 * T);
        }
        load_vals(st, g + 2 * T);
        float v[64];
#pragma unroll
        for (int r = 0; r < 64; ++r) v[r] = x + static_cast<float>(r);
        __builtin_amdgcn_s_barrier();
        if (g < t1) store_chunk_cols(v, (float*)c.base, c.ld, c.y, c.xc, lane);
#pragma unroll
        for (int j = 1; j <= T; ++j)
            if (g + j < t1) cursor_next(c, g + j);
    };
    // (every wave of the team runs the same number of steps, and with them of barriers)
    for (int64_t s = 0; s < steps; s += (kGroup == 4 ? 4 : 2)) {
        const int64_t gb = t0 + s * T;
        body(gb, Index<0>{}, false);
        if (s + 1 < steps) body(gb + T, Index<1>{}, kGroup == 2);
        if constexpr (kGroup == 4) {
            if (s + 2 < steps) body(gb + 2 * T, Index<0>{}, true);
            if (s + 3 < steps) body(gb + 3 * T, Index<1>{}, false);
        }
    }
}

// Test aid: every compute unit's LDS filled with one word.  Two workgroups of 80 000 bytes fit a compute unit, and a
// grid of two per compute unit is one resident round, so the launch reaches (nearly) every LDS byte of the device.
// (`sink` may be null.)
__global__ __launch_bounds__(256, 2) void k_fill_lds(uint32_t word, uint32_t* __restrict__ sink) {
    __shared__ uint32_t all[20000];
    volatile uint32_t* const out = all;  // (LDS is dead when the kernel ends, as far as the optimiser knows)
    for (int i = threadIdx.x; i < 20000; i += 256) out[i] = word;
    // (stay for a fixed while, about 0.1 ms: the dispatcher then has to place every workgroup of the round on a slot
    // of its own instead of handing the slots of the first ones on)
    for (int i = 0; i < 32; ++i) __builtin_amdgcn_s_sleep(127);
    __syncthreads();
    uint32_t s = 0;
    for (int i = 255 - threadIdx.x; i < 20000; i += 256) s += out[i];
    if (sink && s == 0x12345678u) sink[0] = s;
}

}  // namespace tplr

// =========================================================================================
// C ABI
// =========================================================================================
using namespace tplr;

static inline int launch_status() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : static_cast<int>(e);
}

static inline unsigned grid8(int64_t n) { return static_cast<unsigned>(((n + 7) / 8) * 8); }

// persistent grids: exactly one resident set of workgroups of `threads` threads (one wave, or a team of
// waves), as the occupancy calculator reports it for the kernel at hand (registers or LDS bound it); a
// larger grid would leave a second, mostly empty round
template <typename Kernel>
static int persistent_grid(Kernel kernel, int64_t total, int threads = 64) {
    int n_cu = 256, per_cu = 0, dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        n_cu = v;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || per_cu < 1)
        per_cu = threads > 64 ? 2 : 4;
    int64_t g = static_cast<int64_t>(n_cu) * per_cu;
    g = g < 8 ? 8 : (g / 8) * 8;
    const int64_t need = ((total + 7) / 8) * 8;
    return static_cast<int>(need < g ? need : g);
}

// kTeam: waves per workgroup of the kernel (encode_team<> of its instantiation)
template <int kTeam = 1, typename Kernel>
static int launch_encode_as(Kernel kernel, const tplr_tensor_desc* d_desc, const tplr_tensor_desc& single,
                            int n_tensors, int64_t total, int k, uint8_t* d_idx12, float* d_val, void* stream,
                            const tplr_tensor_desc* d_grad_desc = nullptr, float decay = 0.f) {
    static int resident = 0;  // workgroups
    if (resident == 0) resident = persistent_grid(kernel, int64_t{1} << 40, 64 * kTeam);
    const int64_t need = (((total + kTeam - 1) / kTeam + 7) / 8) * 8;  // workgroups that have a chunk each, in eights
    const dim3 grid(static_cast<unsigned>(need < resident ? need : resident)), block(64 * kTeam);
    hipLaunchKernelGGL(kernel, grid, block, 0, static_cast<hipStream_t>(stream), d_desc, single, n_tensors, total, k,
                       d_idx12, d_val, d_grad_desc, decay);
    return launch_status();
}

// kTeam: waves per workgroup of the kernel (aggregate_team<> of its instantiation)
template <int kTeam = 1, typename Kernel>
static int launch_decode_as(Kernel kernel, const PeerPtrs& pp, const float* d_scale, int n_peers, int k,
                            const tplr_tensor_desc* d_desc, const tplr_tensor_desc& single, int n_tensors,
                            int64_t total, int reduce_mode, int normalise, float* d_sumsq, void* stream,
                            int64_t stride_idx = 0, int64_t stride_val = 0, const float* d_deq = nullptr,
                            int32_t* d_guard = nullptr) {
    static int resident = 0;  // workgroups; per kernel variant
    if (resident == 0) resident = persistent_grid(kernel, int64_t{1} << 40, 64 * kTeam);
    // a wave keeps one mark per chunk of its range (chunks to be done again on the exact path), so
    // one launch takes at most kMaxChunksPerWave chunks per wave: 68 GB of output on a whole device
    // (the margin covers the rounding of the slices and their alignment)
    const int64_t piece = static_cast<int64_t>(resident) * kTeam * (kMaxChunksPerWave - 8);
    for (int64_t first = 0; first < total; first += piece) {
        const int64_t count = total - first < piece ? total - first : piece;
        const int64_t need = (((count + kTeam - 1) / kTeam + 7) / 8) * 8;  // workgroups that have a chunk each, in eights
        const dim3 grid(static_cast<unsigned>(need < resident ? need : resident)), block(64 * kTeam);
        hipLaunchKernelGGL(kernel, grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale, n_peers, k, d_desc,
                           single, n_tensors, first, count, reduce_mode, normalise, d_sumsq, stride_idx, stride_val, d_deq,
                           d_guard);
    }
    return launch_status();
}

extern "C" {

int tplr_version(void) { return 100; }

const char* tplr_status_string(int status) {
    switch (status) {
        case 0: return "ok";
        case TPLR_E_BADARG: return "bad argument";
        case TPLR_E_ODD: return "number of indices must be even";
        case TPLR_E_SHAPE: return "dimension is not a multiple of the chunk size";
        case TPLR_E_TOOMANY: return "too many peers or row too long";
        case TPLR_E_WORKSPACE: return "workspace larger than the library's static scratch (tplr_static_work_bytes)";
        default: return status > 0 ? hipGetErrorString(static_cast<hipError_t>(status)) : "unknown status";
    }
}

int tplr_pack12(const int64_t* d_idx, int64_t n, uint8_t* d_packed, int32_t* d_err, void* stream) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!d_idx || !d_packed) return TPLR_E_BADARG;
    const int64_t n_pairs = n / 2, threads = (n_pairs + 3) / 4;
    hipLaunchKernelGGL(k_pack12, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_idx, n_pairs, d_packed, d_err);
    return launch_status();
}

int tplr_unpack12(const uint8_t* d_packed, int64_t n, int64_t* d_idx, void* stream) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!d_idx || !d_packed) return TPLR_E_BADARG;
    const int64_t n_pairs = n / 2, threads = (n_pairs + 3) / 4;
    hipLaunchKernelGGL(k_unpack12, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_packed, n_pairs, d_idx);
    return launch_status();
}

// (tplr_pack12_host, tplr_unpack12_host and tplr_gather_host touch host memory only: tplr_host.cpp)

static int check_2d(const void* a, const void* b, int64_t R, int64_t C) {
    if (!a || !b || R < 0 || C < 0) return TPLR_E_BADARG;
    if ((R % 64) || (C % 64)) return TPLR_E_SHAPE;
    return 0;
}

// chunk rows are addressed with 32-bit byte offsets (63 rows * ld * 4 bytes)
static inline bool ld_ok(int64_t ld) { return ld > 0 && ld <= (int64_t{1} << 23); }

int tplr_dct2d_fwd(const float* d_x, int64_t R, int64_t C, int64_t ld_x, float* d_coef, void* stream) {
    if (int s = check_2d(d_x, d_coef, R, C)) return s;
    if (ld_x < C) return TPLR_E_BADARG;
    if (!ld_ok(ld_x)) return TPLR_E_TOOMANY;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_dct2d_fwd, dim3(grid8(n)), dim3(64), 0, static_cast<hipStream_t>(stream), d_x, ld_x,
                       C / 64, n, d_coef);
    return launch_status();
}

int tplr_dct2d_inv(const float* d_coef, int64_t R, int64_t C, float* d_x, int64_t ld_x, void* stream) {
    if (int s = check_2d(d_x, d_coef, R, C)) return s;
    if (ld_x < C) return TPLR_E_BADARG;
    if (!ld_ok(ld_x)) return TPLR_E_TOOMANY;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_dct2d_inv, dim3(grid8(n)), dim3(64), 0, static_cast<hipStream_t>(stream), d_coef,
                       C / 64, n, d_x, ld_x);
    return launch_status();
}

int tplr_dct1d(const float* d_in, int64_t n_vec, int inverse, float* d_out, void* stream) {
    if (n_vec < 0) return TPLR_E_BADARG;
    if (n_vec == 0) return 0;
    if (!d_in || !d_out) return TPLR_E_BADARG;
    hipLaunchKernelGGL(k_dct1d, dim3(static_cast<unsigned>((n_vec + 63) / 64)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_in, n_vec, inverse, d_out);
    return launch_status();
}

int tplr_dct2d_dense(const float* d_in, int64_t R, int64_t C, int h, int w, const float* d_bh,
                     const float* d_bw, int in_chunked, int out_chunked, float* d_out, void* stream) {
    if (!d_in || !d_out || !d_bh || !d_bw || R < 0 || C < 0 || h < 1 || w < 1 || h > 64 || w > 64)
        return TPLR_E_BADARG;
    if ((R % h) || (C % w)) return TPLR_E_SHAPE;
    const int64_t n = (R / h) * (C / w);
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_dct2d_dense, dim3(static_cast<unsigned>(n)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_in, C, h, w, d_bh, d_bw, in_chunked, out_chunked, d_out);
    return launch_status();
}

int tplr_topk_pack(const float* d_coef, int64_t n_rows, int64_t row_len, int k, uint8_t* d_idx12,
                   float* d_val, void* stream) {
    if (n_rows < 0 || row_len < 1 || k < 2 || (k & 1) || k > row_len) return TPLR_E_BADARG;
    if (row_len > TPLR_MAX_ROW) return TPLR_E_TOOMANY;
    if (n_rows == 0) return 0;
    if (!d_coef || !d_idx12 || !d_val) return TPLR_E_BADARG;
    const int rl = static_cast<int>(row_len);
    if (k > kCandCap)
        hipLaunchKernelGGL(k_topk_rows_sorted, dim3(grid8(n_rows)), dim3(256), 0, static_cast<hipStream_t>(stream),
                           d_coef, n_rows, rl, k, d_idx12, d_val);
    else if (k > 32)
        hipLaunchKernelGGL(k_topk_rows<true>, dim3(grid8(n_rows)), dim3(64), 0,
                           static_cast<hipStream_t>(stream), d_coef, n_rows, rl, k, d_idx12, d_val);
    else
        hipLaunchKernelGGL(k_topk_rows<false>, dim3(grid8(n_rows)), dim3(64), 0,
                           static_cast<hipStream_t>(stream), d_coef, n_rows, rl, k, d_idx12, d_val);
    return launch_status();
}

static int launch_encode(const tplr_tensor_desc* d_desc, const tplr_tensor_desc& single, int n_tensors,
                         int64_t total, int k, int use_dct, uint8_t* d_idx12, float* d_val, void* stream) {
    if (k > 32) {
        if (use_dct)
            return launch_encode_as(k_encode_topk_pack<true, true>, d_desc, single, n_tensors, total, k, d_idx12, d_val, stream);
        return launch_encode_as<encode_team<false>()>(k_encode_topk_pack<true, false>, d_desc, single, n_tensors, total, k, d_idx12, d_val, stream);
    }
    if (use_dct)
        return launch_encode_as(k_encode_topk_pack<false, true>, d_desc, single, n_tensors, total, k, d_idx12, d_val, stream);
    return launch_encode_as<encode_team<false>()>(k_encode_topk_pack<false, false>, d_desc, single, n_tensors, total, k, d_idx12, d_val, stream);
}

int tplr_encode_topk_pack(const float* d_x, int64_t R, int64_t C, int64_t ld_x, int k, int use_dct,
                          uint8_t* d_idx12, float* d_val, void* stream) {
    if (int s = check_2d(d_x, d_val, R, C)) return s;
    if (!d_idx12 || ld_x < C || k < 2 || (k & 1) || k > kCandCap) return TPLR_E_BADARG;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    if (C / 64 > 0x7fffffff || R / 64 > 0x7fffffff || !ld_ok(ld_x)) return TPLR_E_TOOMANY;
    tplr_tensor_desc single;
    single.dense = const_cast<float*>(d_x);
    single.ld = ld_x;
    single.chunk_begin = 0;
    single.x_chunks = static_cast<int32_t>(C / 64);
    single.y_chunks = static_cast<int32_t>(R / 64);
    return launch_encode(nullptr, single, 1, n, k, use_dct, d_idx12, d_val, stream);
}

int tplr_encode_topk_pack_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, int k,
                                int use_dct, uint8_t* d_idx12, float* d_val, void* stream) {
    if (!d_desc || n_tensors < 1 || total_chunks < 0 || !d_idx12 || !d_val || k < 2 || (k & 1) || k > kCandCap)
        return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    return launch_encode(d_desc, none, n_tensors, total_chunks, k, use_dct, d_idx12, d_val, stream);
}

int tplr_encode_rows_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_groups, int k, int use_dct,
                           uint8_t* d_idx12, float* d_val, void* stream) {
    if (!d_desc || n_tensors < 1 || total_groups < 0 || !d_idx12 || !d_val || k < 2 || (k & 1) || k > 64)
        return TPLR_E_BADARG;
    if (total_groups == 0) return 0;
    if (total_groups > 0x7fffffff) return TPLR_E_TOOMANY;
    const dim3 grid(static_cast<unsigned>(total_groups)), block(64);
    if (use_dct)
        hipLaunchKernelGGL(k_encode_rows<true>, grid, block, 0, static_cast<hipStream_t>(stream), d_desc, n_tensors, k,
                           d_idx12, d_val);
    else
        hipLaunchKernelGGL(k_encode_rows<false>, grid, block, 0, static_cast<hipStream_t>(stream), d_desc, n_tensors, k,
                           d_idx12, d_val);
    return launch_status();
}

int tplr_ef_encode_topk_pack_batch(const tplr_tensor_desc* d_ef_desc, const tplr_tensor_desc* d_grad_desc,
                                   int n_tensors, int64_t total_chunks, float decay, int k, int use_dct,
                                   uint8_t* d_idx12, float* d_val, void* stream) {
    if (!d_ef_desc || !d_grad_desc || n_tensors < 1 || total_chunks < 0 || !d_idx12 || !d_val || k < 2 || (k & 1) ||
        k > kCandCap)
        return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    if (k > 32) {
        if (use_dct)
            return launch_encode_as<encode_team<true, true>()>(k_encode_topk_pack<true, true, true>, d_ef_desc, none, n_tensors, total_chunks, k,
                                    d_idx12, d_val, stream, d_grad_desc, decay);
        return launch_encode_as<encode_team<false, true>()>(k_encode_topk_pack<true, false, true>, d_ef_desc, none, n_tensors, total_chunks, k,
                                d_idx12, d_val, stream, d_grad_desc, decay);
    }
    if (use_dct)
        return launch_encode_as<encode_team<true, true>()>(k_encode_topk_pack<false, true, true>, d_ef_desc, none, n_tensors, total_chunks, k,
                                d_idx12, d_val, stream, d_grad_desc, decay);
    return launch_encode_as<encode_team<false, true>()>(k_encode_topk_pack<false, false, true>, d_ef_desc, none, n_tensors, total_chunks, k,
                            d_idx12, d_val, stream, d_grad_desc, decay);
}

int tplr_ef_step_batch(const tplr_tensor_desc* d_ef_desc, const tplr_tensor_desc* d_grad_desc, int n_tensors,
                       int64_t total_chunks, float decay, int k, uint8_t* d_idx12, float* d_val, void* stream) {
    if (!d_ef_desc || !d_grad_desc || n_tensors < 1 || total_chunks < 0 || !d_idx12 || !d_val || k < 2 || (k & 1))
        return TPLR_E_BADARG;
    if (k > 64) return TPLR_E_TOOMANY;
    if (total_chunks == 0) return 0;
    if (k > 32) {
        constexpr int kT = ef_team<true>();
        const int64_t teams = (((total_chunks + kT - 1) / kT + 7) / 8) * 8;  // workgroups that have a chunk each, in eights
        static int resident = 0;
        if (resident == 0) resident = persistent_grid(k_ef_step<true>, int64_t{1} << 40, 64 * kT);
        hipLaunchKernelGGL(k_ef_step<true>, dim3(static_cast<unsigned>(teams < resident ? teams : resident)), dim3(64 * kT), 0,
                           static_cast<hipStream_t>(stream), d_ef_desc, d_grad_desc, n_tensors, total_chunks, k, decay,
                           d_idx12, d_val);
    } else {
        static int resident = 0;
        constexpr int kT = ef_team<false>();
        const int64_t teams = (((total_chunks + kT - 1) / kT + 7) / 8) * 8;
        if (resident == 0) resident = persistent_grid(k_ef_step<false>, int64_t{1} << 40, 64 * kT);
        hipLaunchKernelGGL(k_ef_step<false>, dim3(static_cast<unsigned>(teams < resident ? teams : resident)), dim3(64 * kT), 0,
                           static_cast<hipStream_t>(stream), d_ef_desc, d_grad_desc, n_tensors, total_chunks, k, decay,
                           d_idx12, d_val);
    }
    return launch_status();
}

// dst <- dst - decode(decompress(payload)), every value of tensor t times d_factor[t] first (d_factor nullable)
static int subtract_decoded(const uint8_t* d_idx12, const float* d_val, const float* d_factor, int k,
                            const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, int use_dct,
                            int32_t* d_guard, void* stream) {
    if (!d_idx12 || !d_val || !d_desc || n_tensors < 1 || total_chunks < 0 || k < 2 || (k & 1)) return TPLR_E_BADARG;
    if (k > 64) return TPLR_E_TOOMANY;  // the register-resident decode path
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    if (!use_dct) {
        static int resident = 0;
        if (resident == 0) resident = persistent_grid(k_ef_subtract_sparse, int64_t{1} << 40);
        const int64_t need = ((total_chunks + 7) / 8) * 8;
        hipLaunchKernelGGL(k_ef_subtract_sparse, dim3(static_cast<unsigned>(need < resident ? need : resident)),
                           dim3(64), 0, static_cast<hipStream_t>(stream), d_idx12, d_val, k, d_desc, none, n_tensors,
                           total_chunks, d_factor, d_guard);
        return launch_status();
    }
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) pp.idx[p] = nullptr, pp.val[p] = nullptr;
    pp.idx[0] = d_idx12;
    pp.val[0] = d_val;
    // (one peer: the factor table (n_tensors, 1) is the aggregate's clip-factor table)
    return launch_decode_as<4>(k_decode_aggregate<true, 8, 4, true, true>, pp, d_factor, 1, k, d_desc, none, n_tensors,
                            total_chunks, TPLR_REDUCE_MEAN, 0, nullptr, stream, 0, 0, nullptr, d_guard);
}

int tplr_ef_subtract_batch(const uint8_t* d_idx12, const float* d_val, int k, const tplr_tensor_desc* d_ef_desc,
                           int n_tensors, int64_t total_chunks, int use_dct, void* stream) {
    return subtract_decoded(d_idx12, d_val, nullptr, k, d_ef_desc, n_tensors, total_chunks, use_dct, nullptr, stream);
}

int tplr_apply_decoded_batch(const uint8_t* d_idx12, const float* d_val, const float* d_factor, int k,
                             const tplr_tensor_desc* d_param_desc, int n_tensors, int64_t total_chunks, int use_dct,
                             int32_t* d_nonfinite, void* stream) {
    return subtract_decoded(d_idx12, d_val, d_factor, k, d_param_desc, n_tensors, total_chunks, use_dct, d_nonfinite,
                            stream);
}

int tplr_outer_step_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_factor, int n_peers,
                          int k, const tplr_tensor_desc* d_param_desc, int n_tensors, int64_t total_chunks,
                          float* d_chunk_stats, float* d_tensor_stats, int32_t* d_nonfinite, void* stream) {
    if (!h_idx12 || !h_val || !d_param_desc || n_peers < 1 || n_tensors < 1 || total_chunks < 0 || k < 4 || (k & 1))
        return TPLR_E_BADARG;
    if ((d_chunk_stats == nullptr) != (d_tensor_stats == nullptr)) return TPLR_E_BADARG;
    if (k > 64 || n_peers > 15) return TPLR_E_TOOMANY;  // the register-resident path with 4-bit counters
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    if (total_chunks > 0) {
        auto apart = [](const void* a, const void* b) {
            return static_cast<int64_t>(reinterpret_cast<intptr_t>(a) - reinterpret_cast<intptr_t>(b));
        };
        const int64_t si = n_peers > 1 ? apart(pp.idx[1], pp.idx[0]) : 0;
        const int64_t sv4 = n_peers > 1 ? apart(pp.val[1], pp.val[0]) : 0;
        bool strided = true;
        for (int p = 1; p < n_peers; ++p)
            strided = strided && apart(pp.idx[p], pp.idx[0]) == p * si && apart(pp.val[p], pp.val[0]) == p * sv4;
        tplr_tensor_desc none = {};
        const int options = d_chunk_stats ? 2 : 0;
        int st;
        if (n_peers <= 8 && strided)
            st = launch_decode_as<4>(k_decode_aggregate<true, 8, 4, true, true>, pp, d_factor, n_peers, k, d_param_desc, none,
                                  n_tensors, total_chunks, TPLR_REDUCE_MEAN, options, d_chunk_stats, stream, si, sv4 / 4,
                                  nullptr, d_nonfinite);
        else if (strided)
            st = launch_decode_as<4>(k_decode_aggregate<true, 16, 4, true, true>, pp, d_factor, n_peers, k, d_param_desc,
                                  none, n_tensors, total_chunks, TPLR_REDUCE_MEAN, options, d_chunk_stats, stream, si,
                                  sv4 / 4, nullptr, d_nonfinite);
        else
            st = launch_decode_as<4>(k_decode_aggregate<true, 16, 4, true, false>, pp, d_factor, n_peers, k, d_param_desc,
                                  none, n_tensors, total_chunks, TPLR_REDUCE_MEAN, options, d_chunk_stats, stream, 0, 0,
                                  nullptr, d_nonfinite);
        if (st) return st;
    }
    if (d_tensor_stats)
        hipLaunchKernelGGL(k_tensor_stats, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), d_chunk_stats, d_param_desc, 1 | 2, d_tensor_stats);
    return launch_status();
}

int tplr_outer_step_codes_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes, const float* d_deq,
                                const float* d_factor, int n_peers, int k, const tplr_tensor_desc* d_param_desc,
                                int n_tensors, int64_t total_chunks, float* d_chunk_stats, float* d_tensor_stats,
                                int32_t* d_nonfinite, void* stream) {
    if (!h_idx12 || !h_codes || !d_deq || !d_param_desc || n_peers < 1 || n_tensors < 1 || total_chunks < 0)
        return TPLR_E_BADARG;
    if ((d_chunk_stats == nullptr) != (d_tensor_stats == nullptr)) return TPLR_E_BADARG;
    if (k != 32 && k != 64) return TPLR_E_BADARG;   // the wide-load pipeline's two row lengths
    if (n_peers > 24) return TPLR_E_TOOMANY;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? reinterpret_cast<const float*>(h_codes[p]) : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    auto apart = [](const void* a, const void* b) {
        return static_cast<int64_t>(reinterpret_cast<intptr_t>(a) - reinterpret_cast<intptr_t>(b));
    };
    const int64_t si = n_peers > 1 ? apart(pp.idx[1], pp.idx[0]) : 0;
    const int64_t sv = n_peers > 1 ? apart(pp.val[1], pp.val[0]) : 0;
    bool wide = (reinterpret_cast<uintptr_t>(pp.val[0]) & 3) == 0 && (sv & 3) == 0 && sv >= 0 && si >= 0 &&
                (reinterpret_cast<uintptr_t>(pp.idx[0]) & 3) == 0 && (si & 3) == 0 && sv * n_peers < (int64_t{1} << 32) &&
                si * n_peers < (int64_t{1} << 32);
    for (int p = 1; p < n_peers; ++p)
        wide = wide && apart(pp.idx[p], pp.idx[0]) == p * si && apart(pp.val[p], pp.val[0]) == p * sv;
    if (!wide) return TPLR_E_SHAPE;  // the peers' payloads must be equally spaced, four-byte aligned (a staged window)
    if (total_chunks > 0) {
        tplr_tensor_desc none = {};
        const int options = d_chunk_stats ? 2 : 0;
        int st;
#define TPLR_OUTER_CODES(U, BITS)                                                                                       \
    (k == 64 ? launch_decode_as<4>(k_decode_aggregate<false, U, BITS, true, true, true, 64>, pp, d_factor, n_peers, k,      \
                                d_param_desc, none, n_tensors, total_chunks, TPLR_REDUCE_MEAN, options, d_chunk_stats,  \
                                stream, si, sv, d_deq, d_nonfinite)                                                     \
             : launch_decode_as<4>(k_decode_aggregate<false, U, BITS, true, true, true, 32>, pp, d_factor, n_peers, k,      \
                                d_param_desc, none, n_tensors, total_chunks, TPLR_REDUCE_MEAN, options, d_chunk_stats,  \
                                stream, si, sv, d_deq, d_nonfinite))
        if (n_peers <= 15)
            st = TPLR_OUTER_CODES(16, 4);
        else
            st = TPLR_OUTER_CODES(24, 5);
#undef TPLR_OUTER_CODES
        if (st) return st;
    }
    if (d_tensor_stats)
        hipLaunchKernelGGL(k_tensor_stats, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), d_chunk_stats, d_param_desc, 2, d_tensor_stats);
    return launch_status();
}

int tplr_ef_subtract_own_batch(const uint8_t* d_idx12, const float* d_sent, const float* d_own, int k,
                               const tplr_tensor_desc* d_ef_desc, int n_tensors, int64_t total_chunks, void* stream) {
    if (!d_idx12 || !d_sent || !d_own || !d_ef_desc || n_tensors < 1 || total_chunks < 0 || k < 2 || (k & 1))
        return TPLR_E_BADARG;
    if (k > 64) return TPLR_E_TOOMANY;
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    static int resident = 0;
    if (resident == 0) resident = persistent_grid(k_ef_overwrite_sparse, int64_t{1} << 40);
    const int64_t need = ((total_chunks + 7) / 8) * 8;
    hipLaunchKernelGGL(k_ef_overwrite_sparse, dim3(static_cast<unsigned>(need < resident ? need : resident)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_idx12, d_sent, d_own, k, d_ef_desc, none, n_tensors,
                       total_chunks);
    return launch_status();
}

static int launch_decode(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale, int n_peers,
                         int k, const tplr_tensor_desc* d_desc, const tplr_tensor_desc& single, int n_tensors,
                         int64_t total, int reduce_mode, int normalise, int use_dct, float* d_sumsq, void* stream,
                         const float* d_deq = nullptr) {
    // d_deq: h_val points at one-byte codes of a quantiser of at most four bins (see kCodes)
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    // register-resident fast path: k <= 64 and at most 24 peers; 4-bit counters up to 15 peers, 5-bit beyond
    const int units = (k > 64 || (normalise & 1)) ? 0 : n_peers <= 8 ? 8 : n_peers <= 15 ? 16 : n_peers <= 24 ? 24 : 0;
    // equally spaced payloads (one staged buffer per window): scalar addressing
    auto apart = [](const void* a, const void* b) {
        return static_cast<int64_t>(reinterpret_cast<intptr_t>(a) - reinterpret_cast<intptr_t>(b));
    };
    const int64_t si = n_peers > 1 ? apart(pp.idx[1], pp.idx[0]) : 0;       // bytes
    const int64_t sv4 = n_peers > 1 ? apart(pp.val[1], pp.val[0]) : 0;      // bytes, a multiple of 4
    const int64_t sv = sv4 / 4;
    bool strided = true;
    for (int p = 1; p < n_peers; ++p)
        strided = strided && apart(pp.idx[p], pp.idx[0]) == p * si && apart(pp.val[p], pp.val[0]) == p * sv4;
    if (d_deq) {
        if (use_dct || units == 0) return TPLR_E_TOOMANY;
        // wide loads take four aligned bytes of codes at a time, 32-bit lane offsets from peer 0's payload
        const bool wide_ok = (reinterpret_cast<uintptr_t>(pp.val[0]) & 3) == 0 && (sv4 & 3) == 0 && sv4 >= 0 && si >= 0 &&
                             (reinterpret_cast<uintptr_t>(pp.idx[0]) & 3) == 0 && (si & 3) == 0 &&
                             sv4 * n_peers < (int64_t{1} << 32) && si * n_peers < (int64_t{1} << 32);
#define TPLR_CODES_CASE(U, BITS)                                                                                    \
    case U:                                                                                                         \
        if (strided && wide_ok && k == 64)                                                                          \
            return launch_decode_as<4>(k_decode_aggregate<false, U, BITS, false, true, true, 64>, pp, d_scale, n_peers,  \
                                    k, d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream, si, \
                                    sv4, d_deq);                                                                    \
        if (strided && wide_ok && k == 32)                                                                          \
            return launch_decode_as<4>(k_decode_aggregate<false, U, BITS, false, true, true, 32>, pp, d_scale, n_peers,  \
                                    k, d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream, si, \
                                    sv4, d_deq);                                                                    \
        if (strided)                                                                                                \
            return launch_decode_as(k_decode_aggregate<false, U, BITS, false, true, true>, pp, d_scale, n_peers, k,   \
                                    d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream, si,    \
                                    sv4, d_deq);                                                                    \
        return launch_decode_as(k_decode_aggregate<false, U, BITS, false, false, true>, pp, d_scale, n_peers, k,      \
                                d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream, 0, 0, d_deq);
        switch (units) {
            TPLR_CODES_CASE(8, 4)
            TPLR_CODES_CASE(16, 4)
            TPLR_CODES_CASE(24, 5)
            default:
                return TPLR_E_TOOMANY;
        }
#undef TPLR_CODES_CASE
    }
#define TPLR_DECODE_CASE(U, BITS)                                                                                   \
    case U:                                                                                                         \
        if (strided)                                                                                                \
            return use_dct ? launch_decode_as<aggregate_team<true, U>()>(k_decode_aggregate<true, U, BITS, false, true>, pp, d_scale, n_peers,\
                                              k, d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq,  \
                                              stream, si, sv)                                                        \
                           : launch_decode_as<4>(k_decode_aggregate<false, U, BITS, false, true>, pp, d_scale, n_peers,\
                                              k, d_desc, single, n_tensors, total, reduce_mode, normalise, d_sumsq,  \
                                              stream, si, sv);                                                       \
        return use_dct ? launch_decode_as<aggregate_team<true, U>()>(k_decode_aggregate<true, U, BITS>, pp, d_scale, n_peers, k, d_desc,\
                                          single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream)         \
                       : launch_decode_as<4>(k_decode_aggregate<false, U, BITS>, pp, d_scale, n_peers, k, d_desc,     \
                                          single, n_tensors, total, reduce_mode, normalise, d_sumsq, stream);
    switch (units) {
        TPLR_DECODE_CASE(8, 4)
        TPLR_DECODE_CASE(16, 4)
        TPLR_DECODE_CASE(24, 5)
        default:
            break;
    }
#undef TPLR_DECODE_CASE
    return use_dct ? launch_decode_as(k_decode_aggregate<true, 0, 8>, pp, d_scale, n_peers, k, d_desc, single,
                                      n_tensors, total, reduce_mode, normalise, d_sumsq, stream)
                   : launch_decode_as(k_decode_aggregate<false, 0, 8>, pp, d_scale, n_peers, k, d_desc, single,
                                      n_tensors, total, reduce_mode, normalise, d_sumsq, stream);
}

static int check_decode(const void* a, const void* b, int n_peers, int k, int reduce_mode) {
    if (!a || !b || n_peers < 1 || k < 2 || (k & 1) || k > 4096 ||
        (reduce_mode != TPLR_REDUCE_MEAN && reduce_mode != TPLR_REDUCE_SUM))
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    return 0;
}

int tplr_decode_aggregate(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_peer_scale,
                          int n_peers, int k, int64_t R, int64_t C, int reduce_mode, int normalise, int use_dct,
                          float* d_out, int64_t ld_out, float* d_sumsq, void* stream) {
    if (int s = check_decode(h_idx12, h_val, n_peers, k, reduce_mode)) return s;
    if (!d_out || R < 0 || C < 0) return TPLR_E_BADARG;
    if ((R % 64) || (C % 64)) return TPLR_E_SHAPE;
    if ((use_dct || ld_out != 0) && ld_out < C) return TPLR_E_BADARG;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    if (C / 64 > 0x7fffffff || R / 64 > 0x7fffffff || (ld_out != 0 && !ld_ok(ld_out))) return TPLR_E_TOOMANY;
    tplr_tensor_desc single;
    single.dense = d_out;
    single.ld = ld_out;
    single.chunk_begin = 0;
    single.x_chunks = static_cast<int32_t>(C / 64);
    single.y_chunks = static_cast<int32_t>(R / 64);
    return launch_decode(h_idx12, h_val, d_peer_scale, n_peers, k, nullptr, single, 1, n, reduce_mode, normalise ? 1 : 0,
                         use_dct, d_sumsq, stream);
}

int tplr_decode_aggregate_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                                int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                                int64_t total_chunks, int reduce_mode, int normalise, int use_dct, float* d_sumsq,
                                void* stream) {
    if (int s = check_decode(h_idx12, h_val, n_peers, k, reduce_mode)) return s;
    if (!d_desc || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    return launch_decode(h_idx12, h_val, d_scale, n_peers, k, d_desc, none, n_tensors, total_chunks, reduce_mode,
                         normalise ? 1 : 0, use_dct, d_sumsq, stream);
}

int tplr_decode_aggregate_codes_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes, const float* d_deq,
                                      const float* d_scale, int n_peers, int k, const tplr_tensor_desc* d_desc,
                                      int n_tensors, int64_t total_chunks, int reduce_mode, float* d_sumsq,
                                      void* stream) {
    if (int s = check_decode(h_idx12, h_codes, n_peers, k, reduce_mode)) return s;
    if (!d_desc || !d_deq || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (k > 64 || n_peers > 24) return TPLR_E_TOOMANY;
    if (total_chunks == 0) return 0;
    tplr_tensor_desc none = {};
    return launch_decode(h_idx12, reinterpret_cast<const float* const*>(h_codes), d_scale, n_peers, k, d_desc, none,
                         n_tensors, total_chunks, reduce_mode, 0, 0, d_sumsq, stream, d_deq);
}

int tplr_decode_aggregate_codes_stats_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes,
                                            const float* d_deq, const float* d_scale, int n_peers, int k,
                                            const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks,
                                            int reduce_mode, float* d_chunk_stats, float* d_tensor_stats, void* stream) {
    if (int s = check_decode(h_idx12, h_codes, n_peers, k, reduce_mode)) return s;
    if (!d_desc || !d_deq || !d_chunk_stats || !d_tensor_stats || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (k > 64 || n_peers > 24) return TPLR_E_TOOMANY;
    if (total_chunks > 0) {
        tplr_tensor_desc none = {};
        if (int s = launch_decode(h_idx12, reinterpret_cast<const float* const*>(h_codes), d_scale, n_peers, k, d_desc, none,
                                  n_tensors, total_chunks, reduce_mode, 2, 0, d_chunk_stats, stream, d_deq))
            return s;
    }
    hipLaunchKernelGGL(k_tensor_stats, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_chunk_stats, d_desc, 0, d_tensor_stats);
    return launch_status();
}

int tplr_code_sumsq(const uint8_t* const* h_codes, int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                    int n_slices, int n_bins, const float* d_deq, float* d_sumsq, int32_t* d_bad, void* stream) {
    if (!h_codes || !d_desc || !d_deq || !d_sumsq || n_peers < 1 || n_tensors < 1 || k < 2 || (k & 1) || n_slices < 1 ||
        n_bins < 1 || n_bins > 4)
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS || n_slices > 4096) return TPLR_E_TOOMANY;
    CodePtrs cp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        cp.code[p] = p < n_peers ? h_codes[p] : nullptr;
        if (p < n_peers && !cp.code[p]) return TPLR_E_BADARG;
    }
    hipLaunchKernelGGL(k_code_sumsq4, dim3(static_cast<unsigned>(n_tensors) * n_peers * n_slices), dim3(256), 0,
                       static_cast<hipStream_t>(stream), cp, n_peers, k, n_slices, d_desc, n_bins, d_deq, d_sumsq, d_bad);
    return launch_status();
}

int tplr_decode_aggregate_stats_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                                      int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                                      int64_t total_chunks, int reduce_mode, int normalise, int use_dct,
                                      float* d_chunk_stats, float* d_tensor_stats, void* stream) {
    if (int s = check_decode(h_idx12, h_val, n_peers, k, reduce_mode)) return s;
    if (!d_desc || !d_chunk_stats || !d_tensor_stats || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (total_chunks > 0) {
        tplr_tensor_desc none = {};
        if (int s = launch_decode(h_idx12, h_val, d_scale, n_peers, k, d_desc, none, n_tensors, total_chunks, reduce_mode,
                                  (normalise ? 1 : 0) | 2, use_dct, d_chunk_stats, stream))
            return s;
    }
    hipLaunchKernelGGL(k_tensor_stats, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_chunk_stats, d_desc, use_dct, d_tensor_stats);
    return launch_status();
}

// Rows of any length up to TPLR_MAX_ROW from P peers' flat payloads: row g of the result takes, element
// by element, the sum (or the mean over the senders) of the peers' entries for row g, each peer's values
// times its factor for the tensor the row belongs to, added in peer order and, inside a peer, in entry
// order - the order scatter_reduce_ on the concatenation uses (src/tplr/compress.py:559-580).  One wave
// per row.  Entries of one peer that name the same element (a top-k has none) are added one after the
// other; an index outside the row is dropped and reported.
__global__ __launch_bounds__(64) void k_aggregate_rows(const PeerPtrs pp, const float* __restrict__ scale, int P, int k,
                                                       const tplr_tensor_desc* __restrict__ table, int n_tensors,
                                                       int row_len, int reduce_mode, float* __restrict__ out,
                                                       int32_t* __restrict__ err) {
    __shared__ float acc[TPLR_MAX_ROW];
    __shared__ uint32_t cnt[TPLR_MAX_ROW];
    __shared__ uint32_t tag[TPLR_MAX_ROW];
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    for (int i = lane; i < row_len; i += 64) {
        acc[i] = 0.f;
        cnt[i] = 0;
    }
    int t = 0;
    if (scale && table) {  // the tensor this row belongs to: the last one that begins at or before it
        int lo = 0, hi = n_tensors;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table[mid].chunk_begin <= row)
                lo = mid;
            else
                hi = mid;
        }
        t = lo;
    }
    wave_lds_fence();
    const int64_t idx_stride = k + (k >> 1);
    const int batches = (k + 63) >> 6;  // 64 entries at a time
    // turn `it` = (peer, batch of 64 entries): the entries of the next turn are requested before this
    // turn's are added, so that a row does not wait for one memory round trip per peer
    auto fetch = [&](int it, int& me, float& a) {
        me = -1;
        a = 0.f;
        if (it >= P * batches) return;
        const int p = it / batches, j = (it - p * batches) * 64 + lane;
        if (j < k) {
            const gbyte* irow = (const gbyte*)pp.idx[p] + row * idx_stride;
            const gfloat* vrow = (const gfloat*)pp.val[p] + row * k;
            const float s = scale ? scale[static_cast<int64_t>(t) * P + p] : 1.0f;
            me = static_cast<int>(load_idx12(irow, j));
            a = vrow[j] * s;
        }
    };
    int me_next;
    float a_next;
    fetch(0, me_next, a_next);
    for (int it = 0; it < P * batches; ++it) {
        int me = me_next;
        const float a = a_next;
        fetch(it + 1, me_next, a_next);
        if (me >= row_len) {
            if (err) atomicMax(err, me);
            me = -1;
        }
        // the usual case: the 64 entries name distinct elements
        if (me >= 0) tag[me] = static_cast<uint32_t>(lane);
        wave_lds_fence();
        const bool clash = me >= 0 && tag[me] != static_cast<uint32_t>(lane);
        if (__ballot(clash) == 0) {
            if (me >= 0) {
                acc[me] += a;
                cnt[me] += 1;
            }
        } else {
            // rank among the earlier lanes that name the same element; one rank per turn
            int rank = 0;
            for (int i = 0; i < 63; ++i) {
                const int other = __shfl(me, i);
                rank += (i < lane && other == me && me >= 0) ? 1 : 0;
            }
            int maxrank = rank;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const int o = __shfl_xor(maxrank, off);
                maxrank = o > maxrank ? o : maxrank;
            }
            for (int r = 0; r <= maxrank; ++r) {
                if (me >= 0 && rank == r) {
                    acc[me] += a;
                    cnt[me] += 1;
                }
                wave_lds_fence();
            }
        }
        wave_lds_fence();
    }
    float* orow = out + row * row_len;
    for (int i = lane; i < row_len; i += 64) {
        const uint32_t c = cnt[i];
        const float v = acc[i];
        orow[i] = (reduce_mode == TPLR_REDUCE_MEAN && c > 1) ? v / static_cast<float>(c) : v;
    }
}

int tplr_aggregate_rows(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale, int n_peers,
                        int k, const tplr_tensor_desc* d_desc, int n_tensors, int64_t n_rows, int64_t row_len,
                        int reduce_mode, float* d_out, int32_t* d_err, void* stream) {
    if (!h_idx12 || !h_val || !d_out || n_peers < 1 || n_rows < 0 || row_len < 1 || k < 2 || (k & 1) ||
        (reduce_mode != TPLR_REDUCE_MEAN && reduce_mode != TPLR_REDUCE_SUM) || (d_scale && (!d_desc || n_tensors < 1)))
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS || row_len > TPLR_MAX_ROW || k > TPLR_MAX_ROW || n_rows > 0x7fffffff) return TPLR_E_TOOMANY;
    if (n_rows == 0) return 0;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    hipLaunchKernelGGL(k_aggregate_rows, dim3(static_cast<unsigned>(n_rows)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), pp, d_scale, n_peers, k, d_desc, n_tensors,
                       static_cast<int>(row_len), reduce_mode, d_out, d_err);
    return launch_status();
}

int tplr_decode_rows_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale, int n_peers,
                           int k, const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_rows, int reduce_mode,
                           int use_dct, int32_t* d_err, void* stream) {
    if (!h_idx12 || !h_val || !d_desc || n_tensors < 1 || n_peers < 1 || total_rows < 0 || k < 2 || (k & 1) || k > 64 ||
        (reduce_mode != TPLR_REDUCE_MEAN && reduce_mode != TPLR_REDUCE_SUM))
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS || total_rows > 0x7fffffff) return TPLR_E_TOOMANY;
    if (total_rows == 0) return 0;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    const dim3 grid(static_cast<unsigned>(total_rows)), block(64);
    if (use_dct)
        hipLaunchKernelGGL(k_decode_rows64<true>, grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale, n_peers,
                           k, d_desc, n_tensors, reduce_mode, d_err);
    else
        hipLaunchKernelGGL(k_decode_rows64<false>, grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale, n_peers,
                           k, d_desc, n_tensors, reduce_mode, d_err);
    return launch_status();
}

// Momentum update and error-feedback subtraction on a flat run of values (the 1-D parameters, which do not
// go through the chunk kernels): a <- a * decay + b with two roundings, as mul_ then add_
// (src/tplr/neurons.py:151-152), or a <- a - b (:171).
__global__ __launch_bounds__(256) void k_flat_update(float* __restrict__ a, const float* __restrict__ b, int64_t n,
                                                     float decay, int subtract) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const float x = a[i], y = b[i];
        float r;
        if (subtract) {
            r = x - y;
        } else {
            const float m = x * decay;
            r = m + y;
        }
        a[i] = r;
    }
}

int tplr_flat_update(float* d_a, const float* d_b, int64_t n, float decay, int subtract, void* stream) {
    if (n < 0 || (n > 0 && (!d_a || !d_b))) return TPLR_E_BADARG;
    if (n == 0) return 0;
    int64_t blocks = (n + 255) / 256;
    blocks = blocks > 4096 ? 4096 : blocks;
    hipLaunchKernelGGL(k_flat_update, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       d_a, d_b, n, decay, subtract);
    return launch_status();
}

int tplr_scatter_rows(const uint8_t* d_idx12, const int64_t* d_idx64, const float* d_val, int64_t n_rows,
                      int64_t k_per_row, int64_t row_len, int reduce_mode, float* d_out, int32_t* d_err,
                      void* stream) {
    if (n_rows < 0 || k_per_row < 0 || row_len < 1 || (!d_idx12 == !d_idx64) || !d_val || !d_out ||
        (reduce_mode != TPLR_REDUCE_MEAN && reduce_mode != TPLR_REDUCE_SUM))
        return TPLR_E_BADARG;
    if (d_idx12 && (k_per_row & 1)) return TPLR_E_ODD;
    if (row_len > TPLR_MAX_ROW) return TPLR_E_TOOMANY;
    if (n_rows == 0) return 0;
    hipLaunchKernelGGL(k_scatter_rows, dim3(static_cast<unsigned>(n_rows)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_idx12, d_idx64, d_val, k_per_row,
                       static_cast<int>(row_len), reduce_mode, d_out, d_err);
    return launch_status();
}

int tplr_peer_sumsq(const float* const* h_val, int n_peers, int64_t n, int n_slices, float* d_sumsq, void* stream) {
    if (!h_val || !d_sumsq || n_peers < 1 || n < 0 || n_slices < 1 || n_slices > 4096) return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    ValPtrs vp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        vp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && !vp.val[p] && n > 0) return TPLR_E_BADARG;
    }
    hipLaunchKernelGGL(k_peer_sumsq, dim3(static_cast<unsigned>(n_peers) * n_slices), dim3(1024), 0,
                       static_cast<hipStream_t>(stream), vp, n, n_slices, d_sumsq);
    return launch_status();
}

int tplr_clip_scales(const float* d_norm, int n_peers, int n_partials, float* d_scale, float* d_median,
                     void* stream) {
    return tplr_clip_scales_batch(d_norm, 1, n_peers, n_partials, d_scale, d_median, stream);
}

int tplr_clip_scales_batch(const float* d_norm, int n_tensors, int n_peers, int n_partials, float* d_scale,
                           float* d_median, void* stream) {
    if (!d_norm || !d_scale || n_peers < 1 || n_tensors < 1 || n_partials < 0) return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    hipLaunchKernelGGL(k_clip_scales<float>, dim3(n_tensors), dim3(128), 0, static_cast<hipStream_t>(stream), d_norm,
                       n_peers, n_partials, d_scale, d_median);
    return launch_status();
}

int tplr_row_sumsq(const float* const* h_val, int n_peers, int k, int64_t n_rows, float* const* h_row_sumsq,
                   void* stream) {
    if (!h_val || !h_row_sumsq || n_peers < 1 || k < 1 || k > TPLR_MAX_ROW || n_rows < 0) return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    if (n_rows == 0) return 0;
    ValPtrs vp;
    RowSumPtrs op;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        vp.val[p] = p < n_peers ? h_val[p] : nullptr;
        op.out[p] = p < n_peers ? h_row_sumsq[p] : nullptr;
        if (p < n_peers && (!vp.val[p] || !op.out[p])) return TPLR_E_BADARG;
    }
    int w = 2;
    while (w < k && w < 64) w <<= 1;
    bool vec = w >= 4 && k <= 64 && (k & 3) == 0;
    for (int p = 0; p < n_peers; ++p) vec = vec && (reinterpret_cast<uintptr_t>(h_val[p]) & 15) == 0;
    const int rows_per_trip = vec ? 256 / w : 64 / w;
    const int64_t trips = (n_rows + rows_per_trip - 1) / rows_per_trip;
    // a wave takes eight trips per round; one resident round of four-wave workgroups is enough for a long list
    int64_t blocks = (trips + 31) / 32;
    const int64_t cap = (256 * 8 + n_peers - 1) / n_peers;
    blocks = blocks < 1 ? 1 : blocks > cap ? cap : blocks;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(n_peers)), block(256);
    const hipStream_t on = static_cast<hipStream_t>(stream);
    if (vec) {
        switch (w) {
            case 4: hipLaunchKernelGGL(k_row_sumsq_vec<4>, grid, block, 0, on, vp, op, k, n_rows); break;
            case 8: hipLaunchKernelGGL(k_row_sumsq_vec<8>, grid, block, 0, on, vp, op, k, n_rows); break;
            case 16: hipLaunchKernelGGL(k_row_sumsq_vec<16>, grid, block, 0, on, vp, op, k, n_rows); break;
            case 32: hipLaunchKernelGGL(k_row_sumsq_vec<32>, grid, block, 0, on, vp, op, k, n_rows); break;
            default: hipLaunchKernelGGL(k_row_sumsq_vec<64>, grid, block, 0, on, vp, op, k, n_rows); break;
        }
        return launch_status();
    }
    switch (w) {
        case 2: hipLaunchKernelGGL(k_row_sumsq<2>, grid, block, 0, on, vp, op, k, n_rows); break;
        case 4: hipLaunchKernelGGL(k_row_sumsq<4>, grid, block, 0, on, vp, op, k, n_rows); break;
        case 8: hipLaunchKernelGGL(k_row_sumsq<8>, grid, block, 0, on, vp, op, k, n_rows); break;
        case 16: hipLaunchKernelGGL(k_row_sumsq<16>, grid, block, 0, on, vp, op, k, n_rows); break;
        case 32: hipLaunchKernelGGL(k_row_sumsq<32>, grid, block, 0, on, vp, op, k, n_rows); break;
        default: hipLaunchKernelGGL(k_row_sumsq<64>, grid, block, 0, on, vp, op, k, n_rows); break;
    }
    return launch_status();
}

int tplr_clip_scales_rows(const float* const* h_row_sumsq, int n_peers, const tplr_tensor_desc* d_desc, int n_tensors,
                          int n_slices, double* d_partial, float* d_scale, float* d_median, void* stream) {
    if (!h_row_sumsq || !d_desc || !d_partial || !d_scale || n_peers < 1 || n_tensors < 1 || n_slices < 1)
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    if (static_cast<int64_t>(n_tensors) * n_peers * n_slices > 0x7fffffff) return TPLR_E_TOOMANY;
    RowSumConstPtrs rp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        rp.in[p] = p < n_peers ? h_row_sumsq[p] : nullptr;
        if (p < n_peers && !rp.in[p]) return TPLR_E_BADARG;
    }
    const hipStream_t on = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(k_rowsum_partials, dim3(static_cast<unsigned>(n_tensors) * n_peers * n_slices), dim3(256), 0, on,
                       rp, n_peers, n_slices, d_desc, d_partial);
    hipLaunchKernelGGL(k_clip_scales<double>, dim3(n_tensors), dim3(128), 0, on, d_partial, n_peers, n_slices, d_scale,
                       d_median);
    return launch_status();
}

int tplr_segment_sumsq(const float* const* h_val, int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                       int n_slices, float* d_sumsq, void* stream) {
    if (!h_val || !d_desc || !d_sumsq || n_peers < 1 || n_tensors < 1 || k < 2 || (k & 1) || n_slices < 1)
        return TPLR_E_BADARG;
    if (static_cast<int64_t>(n_tensors) * n_peers * n_slices > 0x7fffffff) return TPLR_E_TOOMANY;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    ValPtrs vp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        vp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && !vp.val[p]) return TPLR_E_BADARG;
    }
    hipLaunchKernelGGL(k_segment_sumsq, dim3(static_cast<unsigned>(n_tensors) * n_peers * n_slices), dim3(1024), 0,
                       static_cast<hipStream_t>(stream), vp, n_peers, k, n_slices, d_desc, d_sumsq);
    return launch_status();
}

int tplr_index_stats_batch(const uint8_t* const* h_idx12, int n_peers, int k, const tplr_tensor_desc* d_desc,
                           int n_tensors, int64_t total_rows, uint64_t* d_pair, uint64_t* d_dup, int32_t* d_max,
                           void* stream) {
    if (!h_idx12 || !d_desc || !d_pair || !d_dup || !d_max || n_peers < 1 || n_tensors < 1 || total_rows < 0 || k < 2 ||
        (k & 1) || k > 4096)
        return TPLR_E_BADARG;
    if (n_peers > kStatPeers) return TPLR_E_TOOMANY;
    if (total_rows == 0) return 0;
    IdxPtrs ip;
    for (int p = 0; p < kStatPeers; ++p) {
        ip.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        if (p < n_peers && !ip.idx[p]) return TPLR_E_BADARG;
    }
    const int64_t need = ((total_rows + 7) / 8) * 8;
    tplr_tensor_desc none = {};
    auto launch = [&](auto kernel, int& resident) {
        if (resident == 0) resident = persistent_grid(kernel, int64_t{1} << 40);
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(need < resident ? need : resident)), dim3(64), 0,
                           static_cast<hipStream_t>(stream), ip, n_peers, k, d_desc, none, n_tensors, total_rows,
                           reinterpret_cast<unsigned long long*>(d_pair), reinterpret_cast<unsigned long long*>(d_dup),
                           d_max);
    };
    static int resident[6] = {0, 0, 0, 0, 0, 0};
    if (k <= 32 && n_peers <= 16)
        launch(k_index_stats<2, 8, 8>, resident[0]);
    else if (k <= 32)
        launch(k_index_stats<2, 16, 8>, resident[1]);
    else if (k <= 64 && n_peers <= 16)
        launch(k_index_stats<1, 16, 8>, resident[2]);
    else if (k <= 64 && n_peers <= 24)
        launch(k_index_stats<1, 24, 6>, resident[3]);
    else if (k <= 64)
        launch(k_index_stats<1, 32, 0>, resident[4]);
    else
        launch(k_index_stats<0>, resident[5]);
    return launch_status();
}

struct DeqPtrs {
    const uint8_t* codes[TPLR_MAX_PEERS];
    float* out[TPLR_MAX_PEERS];
};

// One parameter's codes of P peers, each with its own lookup and shift: block row p serves peer p.
__global__ __launch_bounds__(256) void k_dequantize_peers(const DeqPtrs pp, int64_t n4,
                                                          const float* __restrict__ lookup,
                                                          const float* __restrict__ shift, int n_bins) {
    const int p = blockIdx.y;
    const uchar4* q = reinterpret_cast<const uchar4*>(pp.codes[p]);
    float4* o = reinterpret_cast<float4*>(pp.out[p]);
    const float* lk = lookup + static_cast<int64_t>(p) * n_bins;
    const float sh = shift[p];
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n4; i += stride) {
        const uchar4 c = q[i];
        float4 r;
        r.x = lk[c.x < n_bins ? c.x : n_bins - 1] + sh;
        r.y = lk[c.y < n_bins ? c.y : n_bins - 1] + sh;
        r.z = lk[c.z < n_bins ? c.z : n_bins - 1] + sh;
        r.w = lk[c.w < n_bins ? c.w : n_bins - 1] + sh;
        o[i] = r;
    }
}

int tplr_dequantize_peers(const uint8_t* const* h_codes, int n_peers, int64_t n, const float* d_lookup,
                          const float* d_shift, int n_bins, float* const* h_out, void* stream) {
    if (!h_codes || !h_out || !d_lookup || !d_shift || n_peers < 1 || n < 0 || (n & 3) || n_bins < 1 || n_bins > 256)
        return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    if (n == 0) return 0;
    DeqPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.codes[p] = p < n_peers ? h_codes[p] : nullptr;
        pp.out[p] = p < n_peers ? h_out[p] : nullptr;
        if (p < n_peers && (!pp.codes[p] || !pp.out[p] || (reinterpret_cast<uintptr_t>(pp.codes[p]) & 3) ||
                            (reinterpret_cast<uintptr_t>(pp.out[p]) & 15)))
            return TPLR_E_BADARG;
    }
    const int64_t n4 = n >> 2;
    int64_t bx = (n4 + 255) / 256;
    bx = bx > 2048 ? 2048 : bx;
    hipLaunchKernelGGL(k_dequantize_peers, dim3(static_cast<unsigned>(bx), static_cast<unsigned>(n_peers)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), pp, n4, d_lookup, d_shift, n_bins);
    return launch_status();
}

static int launch_quantize(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                           float range_in_sigmas, int n_slices, double* d_work, uint8_t* d_codes, float* d_shift,
                           float* d_scale, float* d_lookup, void* stream) {
    const dim3 grid(static_cast<unsigned>(n_tensors) * n_slices), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(k_quant_sum, grid, block, 0, st, d_val, k, d_desc, n_slices, d_work);
    hipLaunchKernelGGL(k_quant_sumsq, grid, block, 0, st, d_val, k, d_desc, n_tensors, n_slices, d_work);
    hipLaunchKernelGGL(k_quant_codes, grid, block, 0, st, d_val, k, d_desc, n_tensors, n_slices, n_bins, range_in_sigmas,
                       d_codes, d_work);
    hipLaunchKernelGGL(k_quant_tables, dim3(static_cast<unsigned>(n_tensors)), block, 0, st, d_desc, k, n_tensors,
                       n_slices, n_bins, range_in_sigmas, d_work, d_shift, d_scale, d_lookup);
    return launch_status();
}

static int check_quantize(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                          int n_slices, const uint8_t* d_codes, const float* d_shift, const float* d_scale,
                          const float* d_lookup) {
    if (!d_val || !d_desc || !d_codes || !d_shift || !d_scale || !d_lookup || n_tensors < 1 || k < 4 || (k & 3) ||
        n_bins < 1 || n_bins > 256 || n_slices < 1 || n_slices > 1024)
        return TPLR_E_BADARG;
    if ((reinterpret_cast<uintptr_t>(d_val) & 15) || (reinterpret_cast<uintptr_t>(d_codes) & 3)) return TPLR_E_BADARG;
    if (static_cast<int64_t>(n_tensors) * n_slices > 0x7fffffff) return TPLR_E_TOOMANY;
    return 0;
}

int tplr_quantize_batch(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                        float range_in_sigmas, int n_slices, double* d_work, uint8_t* d_codes, float* d_shift,
                        float* d_scale, float* d_lookup, void* stream) {
    if (!d_work || (reinterpret_cast<uintptr_t>(d_work) & 7)) return TPLR_E_BADARG;
    if (int s = check_quantize(d_val, k, d_desc, n_tensors, n_bins, n_slices, d_codes, d_shift, d_scale, d_lookup))
        return s;
    return launch_quantize(d_val, k, d_desc, n_tensors, n_bins, range_in_sigmas, n_slices, d_work, d_codes, d_shift,
                           d_scale, d_lookup, stream);
}

int tplr_dequantize_batch(const uint8_t* d_codes, const float* d_lookup, const float* d_shift, int n_bins, int k,
                          const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_rows, float* d_val,
                          void* stream) {
    if (!d_codes || !d_lookup || !d_shift || !d_desc || !d_val || n_bins < 1 || n_bins > 256 || k < 4 || (k & 3) ||
        n_tensors < 1 || total_rows < 0)
        return TPLR_E_BADARG;
    if ((reinterpret_cast<uintptr_t>(d_codes) & 3) || (reinterpret_cast<uintptr_t>(d_val) & 15)) return TPLR_E_BADARG;
    if (total_rows == 0) return 0;
    const int64_t n4 = total_rows * k / 4;
    const int64_t blocks = (n4 + 255) / 256;
    hipLaunchKernelGGL(k_dequantize_batch, dim3(static_cast<unsigned>(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_codes, d_lookup, d_shift, n_bins, k, d_desc, n_tensors, n4,
                       d_val);
    return launch_status();
}

int tplr_tensor_rnorm(const float* d_sumsq, const tplr_tensor_desc* d_desc, int n_tensors, float eps, float* d_factor,
                      void* stream) {
    if (!d_sumsq || !d_desc || !d_factor || n_tensors < 1) return TPLR_E_BADARG;
    hipLaunchKernelGGL(k_tensor_rnorm, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_sumsq, d_desc, eps, d_factor);
    return launch_status();
}

int tplr_scale_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, const float* d_factor,
                     void* stream) {
    if (!d_desc || !d_factor || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    static int resident = 0;
    if (resident == 0) resident = persistent_grid(k_scale_chunks, int64_t{1} << 40);
    const int64_t need = ((total_chunks + 7) / 8) * 8;
    hipLaunchKernelGGL(k_scale_chunks, dim3(static_cast<unsigned>(need < resident ? need : resident)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_desc, n_tensors, total_chunks, d_factor);
    return launch_status();
}

int tplr_aggregate_sumsq_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                               int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                               int64_t total_chunks, float* d_sumsq, void* stream) {
    if (int s = check_decode(h_idx12, h_val, n_peers, k, TPLR_REDUCE_SUM)) return s;
    if (!d_desc || !d_sumsq || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    static int resident = 0;  // (the instantiations differ in registers, not in LDS, which bounds them)
    if (resident == 0) resident = persistent_grid(k_aggregate_sumsq<16, true>, int64_t{1} << 40);
    const int64_t need = ((total_chunks + 7) / 8) * 8;
    const dim3 grid(static_cast<unsigned>(need < resident ? need : resident)), block(64);
    if (k <= 64 && n_peers <= 16)
        hipLaunchKernelGGL((k_aggregate_sumsq<16, true>), grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale,
                           n_peers, k, d_desc, n_tensors, total_chunks, d_sumsq);
    else if (k <= 64 && n_peers <= 32)
        hipLaunchKernelGGL((k_aggregate_sumsq<32, true>), grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale,
                           n_peers, k, d_desc, n_tensors, total_chunks, d_sumsq);
    else
        hipLaunchKernelGGL((k_aggregate_sumsq<16, false>), grid, block, 0, static_cast<hipStream_t>(stream), pp, d_scale,
                           n_peers, k, d_desc, n_tensors, total_chunks, d_sumsq);
    return launch_status();
}

int tplr_tensor_rnorm_scales(const float* d_sumsq, const tplr_tensor_desc* d_desc, int n_tensors, int n_peers,
                             float pre, float eps, float* d_factor, float* d_scale, void* stream) {
    if (!d_sumsq || !d_desc || !d_scale || n_tensors < 1 || n_peers < 1) return TPLR_E_BADARG;
    hipLaunchKernelGGL(k_tensor_rnorm_scales, dim3(static_cast<unsigned>(n_tensors)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_sumsq, d_desc, eps, pre, n_peers, d_factor, d_scale);
    return launch_status();
}

int tplr_calib_aggregate(const uint8_t* const* h_idx12, const float* const* h_val, int n_peers, int k, int use_dct,
                         const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, void* stream) {
    if (!d_desc || n_tensors < 1 || total_chunks < 0 || n_peers < 0 || k < 2 || (k & 1) || k > 64) return TPLR_E_BADARG;
    if (n_peers > 24) return TPLR_E_TOOMANY;
    if (n_peers > 0 && (!h_idx12 || !h_val)) return TPLR_E_BADARG;
    if (use_dct && k < 4) return TPLR_E_BADARG;  // (a group's four-byte loads need rows of at least four bytes)
    if (total_chunks == 0) return 0;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    static int resident = 0;
    if (resident == 0) resident = 4 * persistent_grid(k_decode_aggregate<true, 16, 4>, int64_t{1} << 40, 256);  // as many waves as the launch it stands in for
    const int64_t need = ((total_chunks + 7) / 8) * 8;
    const dim3 grid(static_cast<unsigned>(need < resident ? need : resident));
    const hipStream_t on = static_cast<hipStream_t>(stream);
    if (!use_dct || n_peers <= 16) {
        // (the launch it stands for runs teams of four waves)
        const int64_t teams = (((total_chunks + 3) / 4 + 7) / 8) * 8;
        const dim3 tgrid(static_cast<unsigned>(teams < resident / 4 ? teams : resident / 4));
        if (!use_dct)
            hipLaunchKernelGGL(k_calib_aggregate_team<0>, tgrid, dim3(256), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
        else if (k <= 32)
            hipLaunchKernelGGL(k_calib_aggregate_team<4>, tgrid, dim3(256), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
        else
            hipLaunchKernelGGL(k_calib_aggregate_team<2>, tgrid, dim3(256), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
        return launch_status();
    }
    if (!use_dct)
        hipLaunchKernelGGL(k_calib_aggregate<0>, grid, dim3(64), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
    else if (k <= 32)
        hipLaunchKernelGGL(k_calib_aggregate<4>, grid, dim3(64), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
    else
        hipLaunchKernelGGL(k_calib_aggregate<2>, grid, dim3(64), 0, on, pp, n_peers, k, d_desc, n_tensors, total_chunks);
    return launch_status();
}

int tplr_calib_encode(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, void* stream) {
    if (!d_desc || n_tensors < 1 || total_chunks < 0) return TPLR_E_BADARG;
    if (total_chunks == 0) return 0;
    static int resident = 0;
    if (resident == 0) resident = persistent_grid(k_encode_topk_pack<false, true>, int64_t{1} << 40);  // the grid it stands in for
    const int64_t need = ((total_chunks + 7) / 8) * 8;
    tplr_tensor_desc none = {};
    hipLaunchKernelGGL(k_calib_encode, dim3(static_cast<unsigned>(need < resident ? need : resident)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_desc, none, n_tensors, total_chunks,
                       static_cast<float*>(nullptr));
    return launch_status();
}

int tplr_calib_copy(const void* d_src, void* d_dst, int64_t n_bytes, void* stream) {
    if (!d_src || !d_dst || n_bytes < 0 || (n_bytes & 15)) return TPLR_E_BADARG;
    if ((reinterpret_cast<uintptr_t>(d_src) | reinterpret_cast<uintptr_t>(d_dst)) & 15) return TPLR_E_BADARG;
    if (n_bytes == 0) return 0;
    hipLaunchKernelGGL(k_calib_copy, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const v4f*>(d_src), static_cast<v4f*>(d_dst), n_bytes >> 4);
    return launch_status();
}

int tplr_debug_fill_lds(int word, void* stream) {
    int n_cu = 256, dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        n_cu = v;
    hipLaunchKernelGGL(k_fill_lds, dim3(static_cast<unsigned>(2 * n_cu)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t>(word), static_cast<uint32_t*>(nullptr));
    return launch_status();
}

int tplr_calib_fill(void* d_dst, int64_t n_bytes, int pattern, void* stream) {
    if (!d_dst || n_bytes < 0 || (n_bytes & 15) || pattern < 0 || pattern > 2) return TPLR_E_BADARG;
    if (reinterpret_cast<uintptr_t>(d_dst) & 15) return TPLR_E_BADARG;
    if (n_bytes == 0) return 0;
    const dim3 grid(256 * 8), block(256);  // one resident round: eight workgroups of four waves per CU
    const hipStream_t on = static_cast<hipStream_t>(stream);
    v4f* dst = static_cast<v4f*>(d_dst);
    if (pattern == 0)
        hipLaunchKernelGGL(k_calib_fill<0>, grid, block, 0, on, dst, n_bytes >> 4, 1.f);
    else if (pattern == 1)
        hipLaunchKernelGGL(k_calib_fill<1>, grid, block, 0, on, dst, n_bytes >> 4, 1.f);
    else
        hipLaunchKernelGGL(k_calib_fill<2>, grid, block, 0, on, dst, n_bytes >> 4, 1.f);
    return launch_status();
}

// ---- the quantiser without a caller-provided workspace ----------------------------------------
// The partial sums of tplr_quantize_batch live in a file-scope device array instead.  The array's
// name is a host-side handle, not a device address: its address on the current device comes from
// hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
}  // extern "C"

static __device__ __align__(256) double scratch[TPLR_STATIC_WORK_DOUBLES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_lock;
double* scratch_ptr[kMaxDevices];  // per device: every GPU holds its own copy of the array

// the array's address on the current device; nullptr with *status set when it cannot be had
double* scratch_on_current_device(int* status) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        *status = static_cast<int>(e);
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        *status = TPLR_E_TOOMANY;
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            *status = e != hipSuccess ? static_cast<int>(e) : TPLR_E_BADARG;
            return nullptr;
        }
        scratch_ptr[dev] = static_cast<double*>(p);
    }
    return scratch_ptr[dev];
}
}  // namespace

extern "C" {

int64_t tplr_static_work_bytes(void) { return static_cast<int64_t>(TPLR_STATIC_WORK_DOUBLES) * 8; }

int tplr_quantize_batch_static(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                               float range_in_sigmas, int n_slices, uint8_t* d_codes, float* d_shift, float* d_scale,
                               float* d_lookup, void* stream) {
    if (int s = check_quantize(d_val, k, d_desc, n_tensors, n_bins, n_slices, d_codes, d_shift, d_scale, d_lookup))
        return s;
    const int64_t need = static_cast<int64_t>(n_tensors) * n_slices * (2 + 2 * static_cast<int64_t>(n_bins));
    if (need > TPLR_STATIC_WORK_DOUBLES) return TPLR_E_WORKSPACE;
    int status = 0;
    double* work = scratch_on_current_device(&status);
    if (!work) return status;
    return launch_quantize(d_val, k, d_desc, n_tensors, n_bins, range_in_sigmas, n_slices, work, d_codes, d_shift,
                           d_scale, d_lookup, stream);
}

}  // extern "C"
