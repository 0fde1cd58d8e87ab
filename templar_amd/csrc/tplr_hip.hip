// libtplr_hip.so - gfx950 kernels and C ABI for templar's gradient codec.
// Reference semantics: src/tplr/compress.py (tplr 2.1.28); the entry points and what each
// replaces are documented in include/tplr_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

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
__device__ __forceinline__ void load_chunk_cols(float (&v)[64], const float* __restrict__ x, int64_t ld,
                                                int64_t y, int64_t xc, int lane) {
    const float* p = x + (y * 64) * ld + xc * 64 + lane;
#pragma unroll
    for (int r = 0; r < 64; ++r) v[r] = __builtin_nontemporal_load(p + r * ld);
}

__device__ __forceinline__ void store_chunk_cols(const float (&v)[64], float* __restrict__ x, int64_t ld,
                                                 int64_t y, int64_t xc, int lane) {
    float* p = x + (y * 64) * ld + xc * 64 + lane;
#pragma unroll
    for (int r = 0; r < 64; ++r) __builtin_nontemporal_store(v[r], p + r * ld);
}

// forward 2-D transform of the chunk held column-per-lane; result row-per-lane:
// v[d] = coef[lane][d], and the tile is left free
template <bool kUseDct>
__device__ __forceinline__ void chunk_forward(float (&v)[64], float* tile, int lane) {
    if (kUseDct) dct64_fwd(v);  // along rows k: v[b] = sum_k X[k][lane] F[k][b]
    regs_to_tile_cols(v, tile, lane);
    __syncthreads();
    tile_rows_to_regs(v, tile, lane);
    if (kUseDct) dct64_fwd(v);  // along columns l: v[d] = sum_l T[lane][l] F[l][d]
    __syncthreads();
}

// inverse: tile holds coef rows; result column-per-lane v[k] = x[k][lane]
template <bool kUseDct>
__device__ __forceinline__ void chunk_inverse(float (&v)[64], float* tile, int lane) {
    if (kUseDct) {
        tile_rows_to_regs(v, tile, lane);
        dct64_inv(v);  // along d: v[l] = sum_d Y[lane][d] F[l][d]
        __syncthreads();
        regs_to_tile_rows(v, tile, lane);
        __syncthreads();
    }
    tile_cols_to_regs(v, tile, lane);
    if (kUseDct) dct64_inv(v);  // along b: v[k] = sum_b Z[b][lane] F[k][b]
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
    float v[64];
    load_chunk_cols(v, x, ld, y, xc, lane);
    chunk_forward<true>(v, tile, lane);
    regs_to_tile_rows(v, tile, lane);
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
    chunk_inverse<true>(v, tile, lane);
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
    float v[64];
    tile_rows_to_regs(v, tile, lane);
    const Selected s = select_topk<kTwo>(v, tile, lane, k);
    emit_selected(s, lane, k, row, idx12, val);
}

template <bool kTwo, bool kUseDct>
__global__ __launch_bounds__(64) void k_encode_topk_pack(const float* __restrict__ x, int64_t ld, int64_t X,
                                                         int64_t n_chunks, int k, uint8_t* __restrict__ idx12,
                                                         float* __restrict__ val) {
    __shared__ __align__(16) float tile[kTileFloats];
    const int lane = threadIdx.x;
    const int64_t chunk = xcd_contiguous(blockIdx.x, gridDim.x);
    if (chunk >= n_chunks) return;
    const int64_t y = chunk / X, xc = chunk - y * X;
    float v[64];
    load_chunk_cols(v, x, ld, y, xc, lane);
    chunk_forward<kUseDct>(v, tile, lane);
    regs_to_tile_rows(v, tile, lane);
    __syncthreads();
    const Selected s = select_topk<kTwo>(v, tile, lane, k);
    emit_selected(s, lane, k, chunk, idx12, val);
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
__device__ __forceinline__ uint32_t load_idx12(const uint8_t* __restrict__ row, int j) {
    const uint8_t* b = row + 3 * (j >> 1) + (j & 1);
    const uint32_t w = b[0] | (static_cast<uint32_t>(b[1]) << 8);
    return (j & 1) ? (w >> 4) : (w & 0xfffu);
}

template <bool kUseDct>
__global__ __launch_bounds__(64) void k_decode_aggregate(const PeerPtrs pp, const float* __restrict__ scale,
                                                         int P, int k, int64_t X, int64_t n_chunks,
                                                         int reduce_mode, int normalise, float* __restrict__ out,
                                                         int64_t ld_out, float* __restrict__ sumsq) {
    __shared__ __align__(16) float tile[kTileFloats];
    __shared__ __align__(16) uint32_t cnt[1024];  // 4096 one-byte contribution counters
    const int lane = threadIdx.x;
    const int64_t chunk = xcd_contiguous(blockIdx.x, gridDim.x);
    if (chunk >= n_chunks) return;

    {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int c = 0; c < kTileFloats / 256; ++c) reinterpret_cast<float4*>(tile)[c * 64 + lane] = z;
        const uint4 zi = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < 4; ++c) reinterpret_cast<uint4*>(cnt)[c * 64 + lane] = zi;
    }
    __syncthreads();

    // A "unit" is one wave-wide batch of entries of this chunk: for k <= 64 it covers
    // G = 64 / k whole peers (lane -> peer g_lane, entry j_lane), for k > 64 one 64-entry
    // slice of one peer.  Peers are applied strictly in order (g loop below).
    const int G = k >= 64 ? 1 : 64 / k;
    const int S = (k + 63) >> 6;
    const int g_lane = k >= 64 ? 0 : lane / k;
    const int j_lane = k >= 64 ? lane : lane - g_lane * k;
    const int n_units = k >= 64 ? P * S : (P + G - 1) / G;
    const int64_t idx_row = chunk * (k + (k >> 1));
    const int64_t val_row = chunk * k;
    bool collide = false;

    auto entry = [&](int u, int& p, int& j) -> bool {
        if (k >= 64) {
            p = u / S;
            j = (u - p * S) * 64 + lane;
            return j < k;
        }
        p = u * G + g_lane;
        j = j_lane;
        return g_lane < G && p < P;
    };

    if (normalise) {
        // per-peer, per-chunk L2 normalisation (compress.py:541-545); simple, unbatched
        for (int p = 0; p < P; ++p) {
            float ss = 0.f;
            for (int j = lane; j < k; j += 64) {
                const float a = pp.val[p][val_row + j];
                ss += a * a;
            }
            const float nrm = __builtin_sqrtf(wave_sum_f32(ss)) + 1e-8f;
            for (int j0 = 0; j0 < k; j0 += 64) {
                const int j = j0 + lane;
                if (j < k) {
                    const uint32_t ix = load_idx12(pp.idx[p] + idx_row, j);
                    const float a = pp.val[p][val_row + j] / nrm;
                    atomicAdd(&tile[tile_pos(ix)], a);
                    const uint32_t sh = (ix & 3) * 8;
                    const uint32_t old = atomicAdd(&cnt[ix >> 2], 1u << sh);
                    collide |= ((old >> sh) & 0xffu) != 0;
                }
            }
        }
    } else {
        constexpr int kBatch = 8;
        for (int u0 = 0; u0 < n_units; u0 += kBatch) {
            uint32_t ix[kBatch];
            float a[kBatch];
            bool ok[kBatch];
#pragma unroll
            for (int t = 0; t < kBatch; ++t) {
                int p, j;
                ok[t] = (u0 + t < n_units) && entry(u0 + t, p, j);
                ix[t] = 0;
                a[t] = 0.f;
                if (ok[t]) {
                    ix[t] = load_idx12(pp.idx[p] + idx_row, j);
                    a[t] = pp.val[p][val_row + j];
                    if (scale) a[t] *= scale[p];
                }
            }
#pragma unroll
            for (int t = 0; t < kBatch; ++t) {
                if (u0 + t >= n_units) break;
                for (int g = 0; g < G; ++g) {
                    if (ok[t] && g_lane == g) {
                        atomicAdd(&tile[tile_pos(ix[t])], a[t]);
                        const uint32_t sh = (ix[t] & 3) * 8;
                        const uint32_t old = atomicAdd(&cnt[ix[t] >> 2], 1u << sh);
                        collide |= ((old >> sh) & 0xffu) != 0;
                    }
                }
            }
        }
    }
    __syncthreads();

    if (reduce_mode == TPLR_REDUCE_MEAN && __any(collide)) {
        // exactly one entry per destination claims the counter and divides the sum
        for (int u = 0; u < n_units; ++u) {
            int p, j;
            if (entry(u, p, j)) {
                const uint32_t ix = load_idx12(pp.idx[p] + idx_row, j);
                const uint32_t sh = (ix & 3) * 8;
                const uint32_t old = atomicAnd(&cnt[ix >> 2], ~(0xffu << sh));
                const uint32_t c = (old >> sh) & 0xffu;
                if (c > 1) {
                    float* t = &tile[tile_pos(ix)];
                    *t = *t / static_cast<float>(c);
                }
            }
        }
        __syncthreads();
    }

    if (kUseDct) {
        const int64_t y = chunk / X, xc = chunk - y * X;
        float v[64];
        chunk_inverse<true>(v, tile, lane);
        store_chunk_cols(v, out, ld_out, y, xc, lane);
        if (sumsq) {
            float ss = 0.f;
#pragma unroll
            for (int r = 0; r < 64; ++r) ss = __builtin_fmaf(v[r], v[r], ss);
            ss = wave_sum_f32(ss);
            if (lane == 0) sumsq[chunk] = ss;
        }
    } else {
        tile_to_flat(tile, out + chunk * 4096, lane);
        if (sumsq) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                const int q = c * 64 + lane;
                const float4 t = *reinterpret_cast<const float4*>(tile + (q >> 4) * kLd + ((q & 15) << 2));
                ss += t.x * t.x + t.y * t.y + t.z * t.z + t.w * t.w;
            }
            ss = wave_sum_f32(ss);
            if (lane == 0) sumsq[chunk] = ss;
        }
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

__global__ __launch_bounds__(1024) void k_peer_sumsq(const ValPtrs vp, int64_t n, float* __restrict__ sumsq) {
    __shared__ float part[16];
    const int p = blockIdx.x;
    const float* v = vp.val[p];
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) s = __builtin_fmaf(v[i], v[i], s);
    s = wave_sum_f32(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < 16; ++i) t += part[i];
        sumsq[p] = t;
    }
}

__global__ __launch_bounds__(128) void k_clip_scales(const float* __restrict__ norm, int P, int is_sumsq,
                                                     float* __restrict__ scale, float* __restrict__ median) {
    __shared__ float nv[TPLR_MAX_PEERS];
    __shared__ float med;
    const int i = threadIdx.x;
    if (i < P) nv[i] = is_sumsq ? __builtin_sqrtf(norm[i]) : norm[i];
    __syncthreads();
    if (i < P) {
        int rank = 0;
        const float mine = nv[i];
        for (int j = 0; j < P; ++j) rank += (nv[j] < mine || (nv[j] == mine && j < i)) ? 1 : 0;
        if (rank == (P - 1) / 2) med = mine;  // torch.median: lower of the two middles
    }
    __syncthreads();
    if (i < P) {
        const float f = med / (nv[i] + 1e-8f);
        scale[i] = f > 1.0f ? 1.0f : f;  // clamp(max=1); NaN propagates as in torch.clamp
    }
    if (i == 0 && median) *median = med;
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

extern "C" {

int tplr_version(void) { return 100; }

const char* tplr_status_string(int status) {
    switch (status) {
        case 0: return "ok";
        case TPLR_E_BADARG: return "bad argument";
        case TPLR_E_ODD: return "number of indices must be even";
        case TPLR_E_SHAPE: return "dimension is not a multiple of the chunk size";
        case TPLR_E_TOOMANY: return "too many peers or row too long";
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

int tplr_pack12_host(const int64_t* idx, int64_t n, uint8_t* packed, int64_t* bad) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!idx || !packed) return TPLR_E_BADARG;
    int64_t worst = 0;
    for (int64_t p = 0; p < n / 2; ++p) {
        const int64_t a = idx[2 * p], b = idx[2 * p + 1];
        worst = a > worst ? a : worst;
        worst = b > worst ? b : worst;
        const uint32_t w = (static_cast<uint32_t>(a) & 0xfffu) | ((static_cast<uint32_t>(b) & 0xfffu) << 12);
        packed[3 * p] = static_cast<uint8_t>(w);
        packed[3 * p + 1] = static_cast<uint8_t>(w >> 8);
        packed[3 * p + 2] = static_cast<uint8_t>(w >> 16);
    }
    if (bad) *bad = worst > 4095 ? worst : 0;
    return 0;
}

int tplr_unpack12_host(const uint8_t* packed, int64_t n, int64_t* idx) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!idx || !packed) return TPLR_E_BADARG;
    for (int64_t p = 0; p < n / 2; ++p) {
        const uint32_t w = packed[3 * p] | (static_cast<uint32_t>(packed[3 * p + 1]) << 8) |
                           (static_cast<uint32_t>(packed[3 * p + 2]) << 16);
        idx[2 * p] = w & 0xfffu;
        idx[2 * p + 1] = w >> 12;
    }
    return 0;
}

static int check_2d(const void* a, const void* b, int64_t R, int64_t C) {
    if (!a || !b || R < 0 || C < 0) return TPLR_E_BADARG;
    if ((R % 64) || (C % 64)) return TPLR_E_SHAPE;
    return 0;
}

int tplr_dct2d_fwd(const float* d_x, int64_t R, int64_t C, int64_t ld_x, float* d_coef, void* stream) {
    if (int s = check_2d(d_x, d_coef, R, C)) return s;
    if (ld_x < C) return TPLR_E_BADARG;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_dct2d_fwd, dim3(grid8(n)), dim3(64), 0, static_cast<hipStream_t>(stream), d_x, ld_x,
                       C / 64, n, d_coef);
    return launch_status();
}

int tplr_dct2d_inv(const float* d_coef, int64_t R, int64_t C, float* d_x, int64_t ld_x, void* stream) {
    if (int s = check_2d(d_x, d_coef, R, C)) return s;
    if (ld_x < C) return TPLR_E_BADARG;
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
    if (n_rows < 0 || row_len < 1 || k < 2 || (k & 1) || k > row_len || k > kCandCap) return TPLR_E_BADARG;
    if (row_len > TPLR_MAX_ROW) return TPLR_E_TOOMANY;
    if (n_rows == 0) return 0;
    if (!d_coef || !d_idx12 || !d_val) return TPLR_E_BADARG;
    const int rl = static_cast<int>(row_len);
    if (k > 32)
        hipLaunchKernelGGL(k_topk_rows<true>, dim3(grid8(n_rows)), dim3(64), 0,
                           static_cast<hipStream_t>(stream), d_coef, n_rows, rl, k, d_idx12, d_val);
    else
        hipLaunchKernelGGL(k_topk_rows<false>, dim3(grid8(n_rows)), dim3(64), 0,
                           static_cast<hipStream_t>(stream), d_coef, n_rows, rl, k, d_idx12, d_val);
    return launch_status();
}

int tplr_encode_topk_pack(const float* d_x, int64_t R, int64_t C, int64_t ld_x, int k, int use_dct,
                          uint8_t* d_idx12, float* d_val, void* stream) {
    if (int s = check_2d(d_x, d_val, R, C)) return s;
    if (!d_idx12 || ld_x < C || k < 2 || (k & 1) || k > kCandCap) return TPLR_E_BADARG;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    const dim3 grid(grid8(n)), block(64);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t X = C / 64;
    if (k > 32) {
        if (use_dct)
            hipLaunchKernelGGL((k_encode_topk_pack<true, true>), grid, block, 0, st, d_x, ld_x, X, n, k, d_idx12, d_val);
        else
            hipLaunchKernelGGL((k_encode_topk_pack<true, false>), grid, block, 0, st, d_x, ld_x, X, n, k, d_idx12, d_val);
    } else {
        if (use_dct)
            hipLaunchKernelGGL((k_encode_topk_pack<false, true>), grid, block, 0, st, d_x, ld_x, X, n, k, d_idx12, d_val);
        else
            hipLaunchKernelGGL((k_encode_topk_pack<false, false>), grid, block, 0, st, d_x, ld_x, X, n, k, d_idx12, d_val);
    }
    return launch_status();
}

int tplr_decode_aggregate(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_peer_scale,
                          int n_peers, int k, int64_t R, int64_t C, int reduce_mode, int normalise, int use_dct,
                          float* d_out, int64_t ld_out, float* d_sumsq, void* stream) {
    if (!h_idx12 || !h_val || !d_out || R < 0 || C < 0 || n_peers < 1 || k < 2 || (k & 1) || k > 4096 ||
        (reduce_mode != TPLR_REDUCE_MEAN && reduce_mode != TPLR_REDUCE_SUM))
        return TPLR_E_BADARG;
    if ((R % 64) || (C % 64)) return TPLR_E_SHAPE;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    if (use_dct && ld_out < C) return TPLR_E_BADARG;
    const int64_t n = (R / 64) * (C / 64);
    if (n == 0) return 0;
    PeerPtrs pp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        pp.idx[p] = p < n_peers ? h_idx12[p] : nullptr;
        pp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && (!pp.idx[p] || !pp.val[p])) return TPLR_E_BADARG;
    }
    const dim3 grid(grid8(n)), block(64);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (use_dct)
        hipLaunchKernelGGL(k_decode_aggregate<true>, grid, block, 0, st, pp, d_peer_scale, n_peers, k, C / 64, n,
                           reduce_mode, normalise, d_out, ld_out, d_sumsq);
    else
        hipLaunchKernelGGL(k_decode_aggregate<false>, grid, block, 0, st, pp, d_peer_scale, n_peers, k, C / 64, n,
                           reduce_mode, normalise, d_out, ld_out, d_sumsq);
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

int tplr_peer_sumsq(const float* const* h_val, int n_peers, int64_t n, float* d_sumsq, void* stream) {
    if (!h_val || !d_sumsq || n_peers < 1 || n < 0) return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    ValPtrs vp;
    for (int p = 0; p < TPLR_MAX_PEERS; ++p) {
        vp.val[p] = p < n_peers ? h_val[p] : nullptr;
        if (p < n_peers && !vp.val[p] && n > 0) return TPLR_E_BADARG;
    }
    hipLaunchKernelGGL(k_peer_sumsq, dim3(n_peers), dim3(1024), 0, static_cast<hipStream_t>(stream), vp, n,
                       d_sumsq);
    return launch_status();
}

int tplr_clip_scales(const float* d_norm, int n_peers, int is_sumsq, float* d_scale, float* d_median,
                     void* stream) {
    if (!d_norm || !d_scale || n_peers < 1) return TPLR_E_BADARG;
    if (n_peers > TPLR_MAX_PEERS) return TPLR_E_TOOMANY;
    hipLaunchKernelGGL(k_clip_scales, dim3(1), dim3(128), 0, static_cast<hipStream_t>(stream), d_norm, n_peers,
                       is_sumsq, d_scale, d_median);
    return launch_status();
}

}  // extern "C"
