/*
 * tplr_oracle.c - CPU restatement of templar's gradient codec (src/tplr/compress.py,
 * tplr 2.1.28), in plain C.
 *
 * THIS IS TEST INFRASTRUCTURE.  Only the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark may load it; the product (templar_amd) never does.
 *
 * Every function cites the lines of the reference it restates.  Floating-point
 * conventions: transforms accumulate in double against the closed-form basis and round
 * once per output, so the oracle is the mathematically defined result to within half an
 * ulp (the reference's own fp32 einsum and the device kernels both sit ~1e-7 relative
 * from it); sums of scattered values are kept in fp32 and in source order, exactly as
 * Tensor.scatter_reduce_ does on the CPU.
 *
 * Parity pins (tests/test_oracle.py): pack/unpack against the reference's inline
 * known-answer vectors and a brute-force bit model; divisor rule against its four known
 * answers and brute force; DCT against scipy.fft.dctn(norm="ortho"), orthonormality and
 * the reference's round-trip tolerance; top-k against torch.topk on tie-free data and a
 * brute-force sort; scatter-mean / median clip against torch.scatter_reduce_ and
 * torch.median and hand-built closed forms; quantiser against its closed form.
 * Nothing here is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* ---- pack_12bit_indices, src/tplr/compress.py:51-99 ------------------------------------
 * returns 0 ok, 1 = some index > 4095 (*bad receives the maximum), 2 = odd count */
int orc_pack12(const int64_t* idx, int64_t n, uint8_t* out, int64_t* bad) {
    int64_t mx = 0;
    for (int64_t i = 0; i < n; ++i) /* :64-66 max over all elements */
        if (i == 0 || idx[i] > mx) mx = idx[i];
    if (n > 0 && mx >= 4096) {
        if (bad) *bad = mx;
        return 1;
    }
    if (n % 2) return 2; /* :73-74 */
    for (int64_t p = 0; p < n / 2; ++p) {
        const int32_t a = (int32_t)idx[2 * p], b = (int32_t)idx[2 * p + 1]; /* :77 to(int32) */
        out[3 * p] = (uint8_t)(a & 0xFF);                                  /* :95 */
        out[3 * p + 1] = (uint8_t)(((a >> 8) & 0x0F) | ((b & 0x0F) << 4)); /* :96 */
        out[3 * p + 2] = (uint8_t)((b >> 4) & 0xFF);                       /* :97 */
    }
    return 0;
}

/* ---- unpack_12bit_indices, src/tplr/compress.py:102-142 --------------------------------- */
int orc_unpack12(const uint8_t* in, int64_t n, int64_t* idx) {
    if (n == 0) return 0;
    if (n % 2) return 2; /* :120-121 */
    for (int64_t p = 0; p < n / 2; ++p) {
        const int64_t b0 = in[3 * p], b1 = in[3 * p + 1], b2 = in[3 * p + 2];
        idx[2 * p] = b0 | ((b1 & 0x0F) << 8);            /* :136 */
        idx[2 * p + 1] = ((b1 >> 4) & 0x0F) | (b2 << 4); /* :137 */
    }
    return 0;
}

/* ---- _get_prime_divisors / _get_divisors / _get_smaller_split, :791-872 ------------------ */
static int cmp_i64(const void* a, const void* b) {
    const int64_t x = *(const int64_t*)a, y = *(const int64_t*)b;
    return x < y ? -1 : x > y;
}

/* writes the sorted divisors of n to out (capacity cap), returns their number */
int orc_divisors(int64_t n, int64_t* out, int cap) {
    int cnt = 0;
    if (n == 1) { /* :831-832 */
        if (cap > 0) out[0] = 1;
        return 1;
    }
    if (n < 1) return 0;
    int64_t primes[64];
    int np = 0;
    int64_t m = n;
    while (m % 2 == 0) { primes[np++] = 2; m /= 2; } /* :802-804 */
    while (m % 3 == 0) { primes[np++] = 3; m /= 3; } /* :805-807 */
    for (int64_t i = 5; i * i <= m; i += 6)           /* :808-814 */
        for (int s = 0; s < 2; ++s) {
            const int64_t k = i + 2 * s;
            while (m % k == 0) { primes[np++] = k; m /= k; }
        }
    if (m > 1) primes[np++] = m; /* :815-816 */
    out[cnt++] = 1;              /* :835 */
    int64_t last = 0, factor = 0;
    int slice = 0;
    for (int p = 0; p < np; ++p) { /* :840-848 */
        if (last != primes[p]) {
            slice = cnt;
            factor = primes[p];
        } else {
            factor *= primes[p];
        }
        for (int i = 0; i < slice && cnt < cap; ++i) out[cnt++] = out[i] * factor;
        last = primes[p];
    }
    qsort(out, (size_t)cnt, sizeof(int64_t), cmp_i64); /* :849 */
    return cnt;
}

int64_t orc_smaller_split(int64_t n, int64_t close_to) {
    int64_t d[4096];
    const int cnt = orc_divisors(n, d, 4096);
    for (int i = 0; i < cnt; ++i) { /* :865-871 */
        if (d[i] == close_to) return d[i];
        if (d[i] > close_to) return i == 0 ? d[i] : d[i - 1];
    }
    return n; /* :872 */
}

/* ---- DCT basis: what _dct(eye(n), "ortho") computes, :710-741 (closed form) --------------
 * f[i*n + k] = c_k cos(pi (2i+1) k / 2n), c_0 = sqrt(1/n), c_k = sqrt(2/n) */
void orc_dct_basis(int n, double* f) {
    for (int i = 0; i < n; ++i)
        for (int k = 0; k < n; ++k)
            f[i * n + k] = (k == 0 ? sqrt(1.0 / n) : sqrt(2.0 / n)) * cos(M_PI * (2 * i + 1) * k / (2.0 * n));
}

/* ---- ChunkingTransformer.encode, 2-D, :236-246 with einsum :203 --------------------------
 * x (R, C) row-major -> out (R/h, C/w, h, w); use_dct: out[y,x,b,d] = sum_kl X[k,l] F_h[k,b] F_w[l,d] */
void orc_encode2d(const float* x, int64_t R, int64_t C, int h, int w, int use_dct, float* out) {
    const int64_t Y = R / h, X = C / w;
    double *fh = NULL, *fw = NULL, *t = NULL;
    if (use_dct) {
        fh = (double*)malloc(sizeof(double) * h * h);
        fw = (double*)malloc(sizeof(double) * w * w);
        t = (double*)malloc(sizeof(double) * h * w);
        orc_dct_basis(h, fh);
        orc_dct_basis(w, fw);
    }
    for (int64_t y = 0; y < Y; ++y)
        for (int64_t xc = 0; xc < X; ++xc) {
            const float* src = x + (y * h) * C + xc * w; /* rearrange "(y h) (x w) -> y x h w", :244 */
            float* dst = out + (y * X + xc) * (int64_t)h * w;
            if (!use_dct) {
                for (int r = 0; r < h; ++r)
                    for (int c = 0; c < w; ++c) dst[r * w + c] = src[r * C + c];
                continue;
            }
            for (int b = 0; b < h; ++b)
                for (int l = 0; l < w; ++l) {
                    double acc = 0.0;
                    for (int k = 0; k < h; ++k) acc += (double)src[k * C + l] * fh[k * h + b];
                    t[b * w + l] = acc;
                }
            for (int b = 0; b < h; ++b)
                for (int d = 0; d < w; ++d) {
                    double acc = 0.0;
                    for (int l = 0; l < w; ++l) acc += t[b * w + l] * fw[l * w + d];
                    dst[b * w + d] = (float)acc;
                }
        }
    free(fh);
    free(fw);
    free(t);
}

/* ---- ChunkingTransformer.decode, 4-D, :271-281 with einsum :222 ---------------------------
 * coef (R/h, C/w, h, w) -> out (R, C); use_dct: out[k,l] = sum_bd Y[b,d] B_h[b,k] B_w[d,l], B = F^T */
void orc_decode2d(const float* coef, int64_t R, int64_t C, int h, int w, int use_dct, float* out) {
    const int64_t Y = R / h, X = C / w;
    double *fh = NULL, *fw = NULL, *t = NULL;
    if (use_dct) {
        fh = (double*)malloc(sizeof(double) * h * h);
        fw = (double*)malloc(sizeof(double) * w * w);
        t = (double*)malloc(sizeof(double) * h * w);
        orc_dct_basis(h, fh);
        orc_dct_basis(w, fw);
    }
    for (int64_t y = 0; y < Y; ++y)
        for (int64_t xc = 0; xc < X; ++xc) {
            const float* src = coef + (y * X + xc) * (int64_t)h * w;
            float* dst = out + (y * h) * C + xc * w; /* rearrange "y x h w -> (y h) (x w)", :281 */
            if (!use_dct) {
                for (int r = 0; r < h; ++r)
                    for (int c = 0; c < w; ++c) dst[r * C + c] = src[r * w + c];
                continue;
            }
            for (int b = 0; b < h; ++b)
                for (int l = 0; l < w; ++l) {
                    double acc = 0.0;
                    for (int d = 0; d < w; ++d) acc += (double)src[b * w + d] * fw[l * w + d];
                    t[b * w + l] = acc;
                }
            for (int k = 0; k < h; ++k)
                for (int l = 0; l < w; ++l) {
                    double acc = 0.0;
                    for (int b = 0; b < h; ++b) acc += t[b * w + l] * fh[k * h + b];
                    dst[k * C + l] = (float)acc;
                }
        }
    free(fh);
    free(fw);
    free(t);
}

/* 1-D tensors, :248-255 / :283-290: rows of w values, row @ F (inverse = 0) or row @ F^T */
void orc_dct1d(const float* in, int64_t n_vec, int w, int inverse, float* out) {
    double* f = (double*)malloc(sizeof(double) * w * w);
    orc_dct_basis(w, f);
    for (int64_t r = 0; r < n_vec; ++r)
        for (int d = 0; d < w; ++d) {
            double acc = 0.0;
            for (int l = 0; l < w; ++l)
                acc += (double)in[r * w + l] * (inverse ? f[d * w + l] : f[l * w + d]);
            out[r * w + d] = (float)acc;
        }
    free(f);
}

/* ---- TopKCompressor._clamp_topk, :352-367 ----------------------------------------------- */
int orc_clamp_topk(int64_t last_dim, int64_t topk) {
    int64_t k = topk < last_dim ? topk : last_dim;
    k = k > 2 ? k : 2;
    k -= k % 2;
    return (int)k;
}

/* ---- top-k by magnitude + gather, :409-412 -------------------------------------------------
 * Canonical order: descending |x|, lowest index first on exact ties, NaN above +inf (torch's
 * comparator ranks NaN largest).  For k*64 <= n this is the order torch.topk(sorted=False)
 * returns on the CPU when magnitudes are distinct; consumers only use the index set. */
static uint32_t mag_key(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    b &= 0x7fffffffu;
    return b > 0x7f800000u ? 0x7fffffffu : b;
}

void orc_topk_rows(const float* x, int64_t n_rows, int64_t n, int k, int64_t* idx, float* val) {
    uint64_t* key = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)n);
    for (int64_t r = 0; r < n_rows; ++r) {
        const float* row = x + r * n;
        for (int64_t i = 0; i < n; ++i)
            key[i] = ((uint64_t)mag_key(row[i]) << 32) | (uint64_t)(0xffffffffu - (uint32_t)i);
        /* partial selection sort: k is small */
        for (int j = 0; j < k; ++j) {
            int64_t best = j;
            for (int64_t i = j + 1; i < n; ++i)
                if (key[i] > key[best]) best = i;
            const uint64_t t = key[j];
            key[j] = key[best];
            key[best] = t;
            const int64_t ix = (int64_t)(0xffffffffu - (uint32_t)key[j]);
            idx[r * k + j] = ix;
            val[r * k + j] = row[ix]; /* gather of the signed values, :412 */
        }
    }
    free(key);
}

/* ---- TopKCompressor.decompress core, :452-474 ------------------------------------------------
 * out (n_rows, n) zeroed; for j in source order out[idx[j]] accumulates val[j] in fp32; every
 * touched position is divided by its contribution count (scatter_reduce_ "mean",
 * include_self=False).  mean = 0 gives the plain sum.  returns 1 on an out-of-range index. */
int orc_scatter_rows(const int64_t* idx, const float* val, int64_t n_rows, int64_t kk, int64_t n, int mean,
                     float* out) {
    int32_t* cnt = (int32_t*)malloc(sizeof(int32_t) * (size_t)n);
    for (int64_t r = 0; r < n_rows; ++r) {
        float* o = out + r * n;
        memset(o, 0, sizeof(float) * (size_t)n);
        memset(cnt, 0, sizeof(int32_t) * (size_t)n);
        for (int64_t j = 0; j < kk; ++j) {
            const int64_t ix = idx[r * kk + j];
            if (ix < 0 || ix >= n) {
                free(cnt);
                return 1;
            }
            o[ix] = o[ix] + val[r * kk + j];
            cnt[ix] += 1;
        }
        if (mean)
            for (int64_t i = 0; i < n; ++i)
                if (cnt[i] > 1) o[i] = o[i] / (float)cnt[i];
    }
    free(cnt);
    return 0;
}

/* ---- clip factors of batch_decompress, :526-535 and :553-556 ----------------------------------
 * norms[p] given; med = torch.median (lower middle); scale[p] = min(1, med / (norms[p] + 1e-8)) */
static int cmp_f32(const void* a, const void* b) {
    const float x = *(const float*)a, y = *(const float*)b;
    return x < y ? -1 : x > y;
}

float orc_clip_scales(const float* norms, int P, float* scale) {
    float* s = (float*)malloc(sizeof(float) * (size_t)P);
    memcpy(s, norms, sizeof(float) * (size_t)P);
    int any_nan = 0;
    for (int p = 0; p < P; ++p) any_nan |= norms[p] != norms[p];
    qsort(s, (size_t)P, sizeof(float), cmp_f32);
    /* torch.median (:535): the lower of the two middle values; NaN if any norm is NaN */
    const float med = any_nan ? NAN : s[(P - 1) / 2];
    free(s);
    for (int p = 0; p < P; ++p) {
        const float f = med / (norms[p] + 1e-8f);
        scale[p] = f > 1.0f ? 1.0f : f;
    }
    return med;
}

/* L2 norm of n values (torch.norm(v, p=2), :532-534); double accumulation */
float orc_norm2(const float* v, int64_t n) {
    double s = 0.0;
    for (int64_t i = 0; i < n; ++i) s += (double)v[i] * v[i];
    return (float)sqrt(s);
}

/* ---- batch_decompress + decode for 64x64-style chunk rows, :483-580 ---------------------------
 * P payloads of (n_rows, k) values and unpacked indices; per-peer scale (clip) or per-row L2
 * normalisation (:541-545); concatenation in peer order (:574-575); scatter-mean into
 * out (n_rows, n). */
int orc_batch_scatter(const int64_t* const* idx, const float* const* val, const float* scale, int P,
                      int64_t n_rows, int k, int64_t n, int normalise, int mean, float* out) {
    const int64_t kk = (int64_t)P * k;
    int64_t* ci = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n_rows * kk));
    float* cv = (float*)malloc(sizeof(float) * (size_t)(n_rows * kk));
    for (int64_t r = 0; r < n_rows; ++r)
        for (int p = 0; p < P; ++p) {
            float nrm = 0.f;
            if (normalise) {
                double s = 0.0;
                for (int j = 0; j < k; ++j) s += (double)val[p][r * k + j] * val[p][r * k + j];
                nrm = (float)sqrt(s) + 1e-8f;
            }
            for (int j = 0; j < k; ++j) {
                float v = val[p][r * k + j];
                if (normalise)
                    v = v / nrm;
                else if (scale)
                    v = v * scale[p];
                ci[r * kk + (int64_t)p * k + j] = idx[p][r * k + j];
                cv[r * kk + (int64_t)p * k + j] = v;
            }
        }
    const int rc = orc_scatter_rows(ci, cv, n_rows, kk, n, mean, out);
    free(ci);
    free(cv);
    return rc;
}

/* ---- _quantize_values / _dequantize_values, :582-644 -------------------------------------------
 * returns scale; lookup has n_bins entries; q has n entries */
static float round_half_even(float x) { return nearbyintf(x); }

float orc_quantize(const float* val, int64_t n, int n_bins, float range_in_sigmas, uint8_t* q, float* shift_out,
                   float* lookup) {
    const int offset = n_bins / 2; /* :593 */
    double s = 0.0;
    for (int64_t i = 0; i < n; ++i) s += val[i];
    const float shift = (float)(s / (double)n); /* :594 */
    double ss = 0.0;
    for (int64_t i = 0; i < n; ++i) {
        const float c = val[i] - shift; /* :595 */
        ss += (double)c * c;
    }
    const float std = (float)(sqrt(ss) / sqrt((double)(n - 1))); /* :597 */
    float scale = range_in_sigmas * std / (float)n_bins;          /* :598 */
    if (scale == 0.f || isnan(scale) || isinf(scale)) scale = 1.0f; /* :599-600 */
    double* sums = (double*)calloc((size_t)n_bins, sizeof(double));
    int64_t* counts = (int64_t*)calloc((size_t)n_bins, sizeof(int64_t));
    for (int64_t i = 0; i < n; ++i) {
        const float c = val[i] - shift;
        float r = round_half_even(c / scale + (float)offset); /* :604-605 */
        if (r < 0.f) r = 0.f;
        if (r > (float)(n_bins - 1)) r = (float)(n_bins - 1); /* :606 */
        q[i] = (uint8_t)r;
        sums[q[i]] += c; /* :614 */
        counts[q[i]] += 1;
    }
    for (int b = 0; b < n_bins; ++b) lookup[b] = counts[b] > 0 ? (float)(sums[b] / (double)counts[b]) : 0.f; /* :619 */
    free(sums);
    free(counts);
    *shift_out = shift;
    return scale;
}

void orc_dequantize(const uint8_t* q, int64_t n, const float* lookup, float shift, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = lookup[q[i]] + shift; /* :642 */
}
