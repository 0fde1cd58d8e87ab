/*
 * tplr_hip.h - C ABI of libtplr_hip.so, the gfx950 implementation of templar's
 * gradient codec (reference: src/tplr/compress.py, tplr 2.1.28).
 *
 * Conventions
 *   - every pointer named d_* is DEVICE memory owned by the caller; the library
 *     allocates nothing and keeps no state between calls (one exception, stated where
 *     it is declared: tplr_quantize_batch_static works in a static device array);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); all
 *     work is enqueued on it and the call returns without synchronising;
 *   - return value: 0 = ok, negative = TPLR_E_* (bad argument, nothing launched),
 *     positive = a hipError_t from the launch;
 *   - the persistent kernels' grid sizes (one resident round of workgroups, from the occupancy
 *     calculator) are worked out on an entry point's first call and kept per process in plain
 *     statics: the figure belongs to the device that was current then, and first calls racing
 *     on several threads merely compute it twice.  A process that drives GPUs of different sizes
 *     would launch the first one's grid on all of them (correct, since every kernel splits the
 *     work by its own grid size, but not a full round on the larger device);
 *   - "chunk" = one 64x64 fp32 tile of a 2-D tensor, stored row-major inside the
 *     chunked layout (Y, X, 64, 64); flat index inside a chunk = row*64 + col
 *     (reference: rearrange "y x h w -> y x (h w)", src/tplr/compress.py:402-403);
 *   - top-k output order is canonical: descending |value|, lowest flat index first
 *     on exact ties, every NaN ranking above +inf.  This is the order
 *     torch.topk(sorted=False) produces on the CPU for k*64 <= n when magnitudes
 *     are distinct (reference call: src/tplr/compress.py:409-411).
 */
#ifndef TPLR_HIP_H
#define TPLR_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPLR_E_BADARG   (-1) /* null pointer, negative size, unsupported k            */
#define TPLR_E_ODD      (-2) /* number of 12-bit indices is odd                        */
#define TPLR_E_SHAPE    (-3) /* dimension not a multiple of the chunk size             */
#define TPLR_E_TOOMANY  (-4) /* more peers / larger row than the kernel supports       */
#define TPLR_E_WORKSPACE (-5) /* needs more workspace than the library's static scratch */

#define TPLR_CHUNK        64   /* chunk edge handled by the factorised transform       */
#define TPLR_MAX_PEERS    128  /* peers per tplr_decode_aggregate call                 */
#define TPLR_MAX_ROW      4096 /* longest row the select / scatter kernels accept      */

/* reduce_mode of tplr_decode_aggregate / tplr_scatter_rows */
#define TPLR_REDUCE_MEAN  0    /* mean over the peers that sent the coefficient (reference) */
#define TPLR_REDUCE_SUM   1    /* plain sum                                             */

/* One 2-D fp32 tensor of a batch whose dimensions are multiples of 64.  A batch is the
 * concatenation of its tensors' chunk lists (tensor by tensor, chunks row-major); the
 * packed payload of a batch is indexed by that global chunk id: chunk g's indices are the
 * 3k/2 bytes at g*3k/2, its values the k floats at g*k. */
typedef struct tplr_tensor_desc {
    void*   dense;        /* the (R, C) tensor: input of encode, output of decode-aggregate */
    int64_t ld;           /* its row stride in elements                                     */
    int64_t chunk_begin;  /* id of its first chunk in the batch (running sum of x*y chunks) */
    int32_t x_chunks;     /* C / 64                                                         */
    int32_t y_chunks;     /* R / 64                                                         */
} tplr_tensor_desc;

/* Library / ABI version (major*10000 + minor*100 + patch). */
int tplr_version(void);

/* Text for a status code returned by any function below (static storage). */
const char* tplr_status_string(int status);

/* ---- 12-bit index packing ------------------------------------------------------
 * Replaces pack_12bit_indices (src/tplr/compress.py:51-99): pairs (i0,i1) become
 * b0 = i0 & 0xFF, b1 = (i0>>8 & 0xF) | (i1 & 0xF)<<4, b2 = i1>>4 & 0xFF.
 * n must be even (TPLR_E_ODD).  d_err (int32, caller-zeroed) receives, by atomic
 * max, the largest index value > 4095 seen (clamped to INT32_MAX), so the caller can
 * raise the reference's "exceeds 12-bit limit" error at its next synchronisation;
 * negative indices are packed by their low bits exactly as the reference does. */
int tplr_pack12(const int64_t* d_idx, int64_t n, uint8_t* d_packed, int32_t* d_err, void* stream);

/* Replaces unpack_12bit_indices (src/tplr/compress.py:102-142): n int64 indices
 * from 3n/2 bytes.  n must be even. */
int tplr_unpack12(const uint8_t* d_packed, int64_t n, int64_t* d_idx, void* stream);

/* The same two routines on HOST memory, for payloads that are validated before they are
 * moved to the device (unpack_12bit_indices is called on downloaded tensors by
 * src/tplr/comms.py:2599 and src/tplr/neurons.py:1361).  *bad (nullable) receives the
 * largest index > 4095, or 0. */
int tplr_pack12_host(const int64_t* idx, int64_t n, uint8_t* packed, int64_t* bad);
int tplr_unpack12_host(const uint8_t* packed, int64_t n, int64_t* idx);

/* Concatenates n_parts HOST buffers (h_src[i], h_bytes[i] bytes) into h_dst with n_threads host
 * threads (1..64), each copying an equal share of the bytes.  Turns one peer's per-parameter
 * payload tensors (the lists `state_dict.<name>idxs` / `<name>vals` that
 * src/tplr/comms.py:1938-1963 builds and neurons/validator.py:94-219 moves tensor by tensor)
 * into the flat payload the batch entry points read, inside a pinned buffer that then crosses to
 * the device in one copy.  Blocking; touches no device. */
int tplr_gather_host(const void* const* h_src, const int64_t* h_bytes, int64_t n_parts, void* h_dst,
                     int n_threads);

/* ---- chunked 2-D DCT ------------------------------------------------------------
 * Replaces ChunkingTransformer.encode(use_dct=True) for 2-D tensors whose chunk is
 * 64x64 (src/tplr/compress.py:236-246, einsum :203): d_x is (R, C) row-major with
 * row stride ld_x elements, d_coef is (R/64, C/64, 64, 64) contiguous,
 * coef[y,x] = F^T X[y,x] F with the orthonormal DCT-II basis. */
int tplr_dct2d_fwd(const float* d_x, int64_t R, int64_t C, int64_t ld_x, float* d_coef, void* stream);

/* Replaces ChunkingTransformer.decode(use_dct=True) (src/tplr/compress.py:271-281,
 * einsum :222): d_coef (R/64, C/64, 64, 64) -> d_x (R, C), x[y,x] = F coef[y,x] F^T. */
int tplr_dct2d_inv(const float* d_coef, int64_t R, int64_t C, float* d_x, int64_t ld_x, void* stream);

/* 1-D tensors (src/tplr/compress.py:248-255, :283-290): n_vec rows of 64 floats,
 * each row r <- r @ F (inverse = 0) or r @ F^T (inverse = 1). */
int tplr_dct1d(const float* d_in, int64_t n_vec, int inverse, float* d_out, void* stream);

/* Any chunk size h, w <= 64 (non-64 divisors chosen by _get_smaller_split,
 * src/tplr/compress.py:853-872; also einsum_2d / einsum_2d_t, :186-222, with arbitrary
 * bases): dense contraction out = Bh^T X Bw per (h, w) chunk with caller-supplied
 * d_bh (h, h) and d_bw (w, w), row-major.  Pass f_dict[h], f_dict[w] to encode and
 * b_dict[h], b_dict[w] to decode.  in_chunked / out_chunked select the layout of each
 * side: 0 = (R, C) row-major, 1 = (R/h, C/w, h, w) contiguous.  h = 1 gives the 1-D
 * form row @ Bw. */
int tplr_dct2d_dense(const float* d_in, int64_t R, int64_t C, int h, int w,
                     const float* d_bh, const float* d_bw, int in_chunked, int out_chunked,
                     float* d_out, void* stream);

/* ---- top-k select + value gather + 12-bit pack -----------------------------------
 * Replaces TopKCompressor.compress without quantisation (src/tplr/compress.py:402-416)
 * on n_rows rows of row_len fp32 coefficients (row_len = 4096 for 2-D chunks, 64 for
 * 1-D tensors, anything <= TPLR_MAX_ROW otherwise).  k even, 2 <= k <= row_len (k > 128 sorts the
 * whole row in LDS: exact, an order of magnitude slower than the select that serves k <= 128).
 * Outputs: d_idx12 = n_rows * k * 3/2 bytes, d_val = (n_rows, k) signed values.
 * This is the coefficient-input entry used for the bit-exact parity stage. */
int tplr_topk_pack(const float* d_coef, int64_t n_rows, int64_t row_len, int k,
                   uint8_t* d_idx12, float* d_val, void* stream);

/* Fused encode: tplr_dct2d_fwd (use_dct != 0) or plain chunking (use_dct == 0)
 * followed by tplr_topk_pack with row_len 4096, without writing the coefficients
 * to memory (src/tplr/neurons.py:155-159 calls encode then compress back to back).
 * k in {2,...,128}, even. */
int tplr_encode_topk_pack(const float* d_x, int64_t R, int64_t C, int64_t ld_x, int k, int use_dct,
                          uint8_t* d_idx12, float* d_val, void* stream);

/* The same over a whole gradient set in ONE launch (the per-parameter loop of
 * src/tplr/neurons.py:114-159 without its per-tensor kernel tails): d_desc is a DEVICE
 * array of n_tensors descriptors sorted by chunk_begin, total_chunks their chunk count;
 * outputs are the flat payload described at tplr_tensor_desc. */
int tplr_encode_topk_pack_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, int k,
                                int use_dct, uint8_t* d_idx12, float* d_val, void* stream);

/* The 1-D parameters of a set (norm vectors) in ONE launch: encode (rows of 64, the 64-point DCT-II of
 * every row when use_dct != 0, src/tplr/compress.py:248-255) followed by compress (top-k per row, :402-416)
 * for every tensor of d_desc, each read where it lies: `dense` = the tensor, x_chunks = its number of rows
 * (elements / 64), y_chunks = 1, chunk_begin = the id of its first row in the flat payload (row g: indices
 * at byte g*3k/2, values at float g*k).  total_groups = the sum over the tensors of ceil(rows / 64).
 * k even, 2 <= k <= 64.  Same bits as tplr_dct1d followed by tplr_topk_pack with row_len 64. */
int tplr_encode_rows_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_groups, int k, int use_dct,
                           uint8_t* d_idx12, float* d_val, void* stream);

/* ---- decode side -----------------------------------------------------------------
 * Fused TopKCompressor.batch_decompress + ChunkingTransformer.decode
 * (src/tplr/compress.py:483-580 then :259-292; caller: src/tplr/neurons.py:355-367).
 * For every chunk: unpack the 12-bit indices of n_peers payloads, multiply peer p's
 * values by d_peer_scale[p] (NULL = 1; the median-norm clip factors of
 * src/tplr/compress.py:553-556), or, when normalise != 0, divide them by their
 * per-chunk L2 norm + 1e-8 (:541-545); accumulate in peer order; divide every touched
 * coefficient by its number of contributions (scatter_reduce "mean",
 * include_self=False, :472-474) unless reduce_mode = TPLR_REDUCE_SUM; then apply the
 * inverse DCT (use_dct != 0, output (R, C) with row stride ld_out >= C); without it
 * (use_dct == 0) write either the dense coefficient tensor (R/64, C/64, 64, 64) (ld_out == 0:
 * what batch_decompress returns) or the (R, C) tensor with row stride ld_out >= C (what
 * decode(use_dct=False) makes of it, a pure re-layout, :281).
 * h_idx12 / h_val are HOST arrays of n_peers DEVICE pointers: payload p holds
 * n_chunks*k*3/2 index bytes and (n_chunks, k) values.  d_sumsq (nullable) receives
 * n_chunks partial sums of squares of the output, one per chunk.
 * A payload row may name a coefficient more than once (a top-k selection never does): every
 * entry is then added, in entry order, and counted, as scatter_reduce_ does; such chunks take
 * an exact, slower path inside the same launch. */
int tplr_decode_aggregate(const uint8_t* const* h_idx12, const float* const* h_val,
                          const float* d_peer_scale, int n_peers, int k,
                          int64_t R, int64_t C, int reduce_mode, int normalise, int use_dct,
                          float* d_out, int64_t ld_out, float* d_sumsq, void* stream);

/* The same over a whole gradient set in ONE launch (the per-parameter loop of
 * src/tplr/neurons.py:309-367): every peer's payload is flat over the batch
 * (tplr_tensor_desc), results go to each descriptor's `dense` tensor ((R, C) with row stride
 * ld; with use_dct == 0 a descriptor with ld == 0 receives the contiguous (R/64, C/64, 64, 64)
 * coefficient tensor instead); d_scale (nullable) holds
 * n_tensors x n_peers clip factors, d_sumsq (nullable) total_chunks partial sums. */
int tplr_decode_aggregate_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                                int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                                int64_t total_chunks, int reduce_mode, int normalise, int use_dct, float* d_sumsq,
                                void* stream);

/* Row-wise scatter for layouts that are not 64x64 chunks (1-D tensors, un-chunked
 * 2-D rows; TopKCompressor.decompress, src/tplr/compress.py:452-474): d_out is
 * (n_rows, row_len) zero-filled then d_val[r, j] * scale accumulated at d_idx[r, j]
 * in j order and averaged per destination.  Exactly one of d_idx12 (packed) and
 * d_idx64 (int64, as produced by unpack / batch concatenation) is non-NULL.
 * row_len <= TPLR_MAX_ROW.  d_err as in tplr_pack12: receives the largest
 * out-of-range index (>= row_len) seen; such entries are skipped. */
int tplr_scatter_rows(const uint8_t* d_idx12, const int64_t* d_idx64, const float* d_val,
                      int64_t n_rows, int64_t k_per_row, int64_t row_len, int reduce_mode,
                      float* d_out, int32_t* d_err, void* stream);

/* The same for P peers' flat payloads at once, without concatenating them: row g of d_out
 * (n_rows x row_len) takes the peers' entries for row g in peer order, peer p's values times
 * d_scale[t * n_peers + p], t the tensor of d_desc (chunk_begin = first row, as for the chunk
 * batches) that row g belongs to; d_scale NULL = no factors (then d_desc may be NULL).
 * Replaces batch_decompress (src/tplr/compress.py:483-580) for layouts that are not 64x64 chunks
 * - the 1-D parameters: rows of 64 - over a whole set of parameters in one launch.  k even;
 * d_err as above. */
int tplr_aggregate_rows(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale, int n_peers,
                        int k, const tplr_tensor_desc* d_desc, int n_tensors, int64_t n_rows, int64_t row_len,
                        int reduce_mode, float* d_out, int32_t* d_err, void* stream);

/* tplr_aggregate_rows for rows of 64 (the 1-D parameters) followed by decode (tplr_dct1d, inverse, when use_dct
 * != 0; src/tplr/compress.py:283-290) in ONE launch, every row written into its tensor where that lies:
 * d_desc as for tplr_encode_rows_batch (`dense` = the tensor, x_chunks = its rows, chunk_begin = the id of
 * its first row), total_rows the sum of the tensors' rows.  Same bits as the two calls it replaces.
 * k even, 2 <= k <= 64; d_err as for tplr_scatter_rows (indices >= 64 are skipped and reported). */
int tplr_decode_rows_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale, int n_peers,
                           int k, const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_rows, int reduce_mode,
                           int use_dct, int32_t* d_err, void* stream);

/* The elementwise steps of the miner's loop body on a flat run of n values (the 1-D parameters):
 * subtract == 0: d_a <- d_a * decay + d_b, two roundings, as mul_ then add_
 * (src/tplr/neurons.py:151-152); subtract != 0: d_a <- d_a - d_b (:171). */
int tplr_flat_update(float* d_a, const float* d_b, int64_t n, float decay, int subtract, void* stream);

/* ---- peer statistics (src/tplr/compress.py:526-535, :553-556) ---------------------
 * d_sumsq[p * n_slices + s] = sum of squares of the s-th of n_slices equal runs of payload p's
 * n values (h_val: HOST array of n_peers DEVICE pointers).  n_slices > 1 lets a few peers with
 * large payloads use the whole device; the consumer adds the partial sums in order. */
int tplr_peer_sumsq(const float* const* h_val, int n_peers, int64_t n, int n_slices, float* d_sumsq,
                    void* stream);

/* d_scale[p] = min(1, med / (norm_p + 1e-8)), med = lower median of the norms
 * (torch.median).  n_partials == 0: d_norm[p] is the norm itself; n_partials >= 1: d_norm holds
 * n_partials partial sums of squares per peer (peer-major), norm_p = sqrt of their sum taken in
 * order.  d_median (nullable) receives med. */
int tplr_clip_scales(const float* d_norm, int n_peers, int n_partials, float* d_scale, float* d_median,
                     void* stream);

/* Batch forms for flat payloads (the per-peer, per-parameter norms of src/tplr/neurons.py:346
 * and the clip of src/tplr/compress.py:526-556 for every parameter at once).
 * tplr_segment_sumsq: d_sumsq[(t * n_peers + p) * n_slices + s] = sum of squares of slice s of
 * peer p's values that belong to tensor t; a tensor's chunks are cut into n_slices runs so that
 * a few very large tensors still fill the device (n_slices = 1: one sum per tensor and peer).
 * tplr_clip_scales_batch: d_scale[t * n_peers + p] from the lower median over the peers of
 * tensor t, d_norm laid out as above with n_partials = n_slices (or 0 for plain norms). */
int tplr_segment_sumsq(const float* const* h_val, int n_peers, int k, const tplr_tensor_desc* d_desc,
                       int n_tensors, int n_slices, float* d_sumsq, void* stream);
int tplr_clip_scales_batch(const float* d_norm, int n_tensors, int n_peers, int n_partials, float* d_scale,
                           float* d_median, void* stream);

/* The same norms in two steps, so that the pass over the values is made once, when a payload arrives, and the
 * clip factors of a window (src/tplr/neurons.py:346, src/tplr/compress.py:526-556) cost one float per row:
 * tplr_row_sumsq: h_row_sumsq[p][r] = sum of squares of row r (k values, 1 <= k <= 4096) of peer p's flat values,
 * n_rows rows per peer (h_val, h_row_sumsq: HOST arrays of n_peers DEVICE pointers), one launch.  The additions
 * have a fixed order: a pairwise tree over the row's squares placed in the next power of two of lanes (rows
 * longer than 64: lane j first adds the squares of values j, j + 64, ...).
 * tplr_clip_scales_rows: d_scale[t * n_peers + p] = min(1, med_t / (norm_tp + 1e-8)) with norm_tp = sqrt of
 * the sum, in double and in a fixed order, of the row figures of tensor t (rows chunk_begin ... of d_desc;
 * x_chunks * y_chunks of them), med_t the lower median over the peers; d_median (nullable) receives med_t.
 * d_partial: workspace of n_tensors * n_peers * n_slices doubles (n_slices >= 1 cuts large tensors so that a
 * few of them still fill the device).  Two launches. */
int tplr_row_sumsq(const float* const* h_val, int n_peers, int k, int64_t n_rows, float* const* h_row_sumsq,
                   void* stream);
int tplr_clip_scales_rows(const float* const* h_row_sumsq, int n_peers, const tplr_tensor_desc* d_desc,
                          int n_tensors, int n_slices, double* d_partial, float* d_scale, float* d_median,
                          void* stream);

/* ---- miner side: error-feedback step (src/tplr/neurons.py:147-171) ------------------
 * The reference runs, per parameter: ef.mul_(decay); ef.add_(grad); encode(ef); compress;
 * decompress; decode; ef.sub_(decoded).  Two launches over a whole gradient set do the same:
 *
 * tplr_ef_encode_topk_pack_batch: for every chunk, ef <- ef * decay + grad (two roundings, as
 * mul_ then add_), written back in place, and the payload of the updated ef as in
 * tplr_encode_topk_pack_batch.  d_ef_desc and d_grad_desc are DEVICE arrays of n_tensors
 * descriptors with the same shapes and chunk_begin; `dense` points to the error-feedback
 * tensor and to the gradient respectively.  (A null round, neurons.py:148-149, is ef.zero_()
 * followed by the plain tplr_encode_topk_pack_batch.)
 *
 * tplr_ef_subtract_batch: ef <- ef - decode(decompress(payload)) (neurons.py:162-171).  d_val
 * holds the values the reference would decompress: the payload's own values, or the
 * de-quantised ones when the compressor quantises.  use_dct != 0: inverse transform per chunk,
 * k <= 64; use_dct == 0: only the k payload positions of each chunk change. */
int tplr_ef_encode_topk_pack_batch(const tplr_tensor_desc* d_ef_desc, const tplr_tensor_desc* d_grad_desc,
                                   int n_tensors, int64_t total_chunks, float decay, int k, int use_dct,
                                   uint8_t* d_idx12, float* d_val, void* stream);
int tplr_ef_subtract_batch(const uint8_t* d_idx12, const float* d_val, int k, const tplr_tensor_desc* d_ef_desc,
                           int n_tensors, int64_t total_chunks, int use_dct, void* stream);

/* tplr_ef_subtract_batch with use_dct == 0 for the step's own payload, i.e. d_idx12 and d_own as
 * tplr_ef_encode_topk_pack_batch (use_dct = 0) has just written them from these very tensors: a selected
 * position then holds the payload's own value, so ef - sent there is own - sent and the tensors are not read:
 * ef[position] <- d_own - d_sent, entry by entry (d_sent: what the reference would decompress - d_own itself
 * without a quantiser, the de-quantised values with one).  The same bits as tplr_ef_subtract_batch; every
 * row must name each position once, as a top-k selection does.  k <= 64. */
int tplr_ef_subtract_own_batch(const uint8_t* d_idx12, const float* d_sent, const float* d_own, int k,
                               const tplr_tensor_desc* d_ef_desc, int n_tensors, int64_t total_chunks, void* stream);

/* Both launches in one where nothing sits between them (no quantiser) and the chunks are transformed:
 * tplr_ef_encode_topk_pack_batch (use_dct = 1) followed by tplr_ef_subtract_batch (use_dct = 1) on the payload
 * it wrote - the same payload and the same tensors, bit for bit - with every chunk of the error-feedback
 * tensors read once and written once.  k even, 2 <= k <= 64. */
int tplr_ef_step_batch(const tplr_tensor_desc* d_ef_desc, const tplr_tensor_desc* d_grad_desc, int n_tensors,
                       int64_t total_chunks, float decay, int k, uint8_t* d_idx12, float* d_val, void* stream);

/* The validator's per-peer evaluation update (neurons/validator.py:3595-3737, update_model_with_gradient): per
 * parameter, the evaluated peer's values times its clip factor, decompress, decode, and
 * p.data.sub_(decoded, alpha = lr * eval_lr_factor) - here one launch over the whole set that reads and writes
 * every parameter once and never holds the dense gradient: param <- param - decode(decompress(payload)), every
 * value of tensor t times d_factor[t] first (pass alpha * clip factor; the transform is linear, so this differs
 * from scaling the decoded tensor by rounding only; NULL = 1).  The kernels are those of
 * tplr_ef_subtract_batch; k <= 64; repeated indices in a row as in decompress (the mean of those entries).
 * d_nonfinite (nullable): n_tensors ints, zeroed by the caller.  The reference tests the decoded gradient for
 * NaN and infinities before it touches the parameter and rejects the peer (validator.py:3646-3660, :3677-3680).
 * Here a chunk whose decoded values are not all finite is left unwritten - the parameter keeps its bits there -
 * and d_nonfinite[t] becomes 1 for its tensor; every other chunk is updated, so a caller that finds a flag set
 * rejects the peer and takes the update back with a second call with the factors negated (the same chunks are
 * skipped again).  NULL: no test, everything is subtracted. */
int tplr_apply_decoded_batch(const uint8_t* d_idx12, const float* d_val, const float* d_factor, int k,
                             const tplr_tensor_desc* d_param_desc, int n_tensors, int64_t total_chunks,
                             int use_dct, int32_t* d_nonfinite, void* stream);

/* The outer step over a whole window in one launch (src/tplr/neurons.py:309-447, outer_step, with the plain SGD
 * of neurons/trainer.py:128-130): per parameter the reference builds the dense gradient
 * decode(batch_decompress(P peers)), takes its norm and mean, tests isfinite().all() and, if that holds, lets
 * optimizer.step() compute p <- p - lr * grad - the dense gradient written, read three times and read again by
 * the optimiser.  Here param <- param - decode(aggregate of the peers' payloads), every value of peer p for
 * tensor t times d_factor[t * n_peers + p] first (pass lr * clip factor): the aggregate's fused launch whose
 * result is subtracted from the parameter's rows instead of stored, the gradient never written.  Chunks of 64x64
 * with the transform, k <= 64, n_peers <= 15; h_idx12, h_val as in tplr_decode_aggregate_batch.
 * d_nonfinite (nullable, n_tensors ints zeroed by the caller): as in tplr_apply_decoded_batch, a chunk whose
 * decoded values are not all finite is left unwritten and flags its tensor.  A caller that must leave such a
 * parameter untouched as a whole, as the reference does, makes every factor of a tensor it cannot vouch for a NaN
 * (then no chunk of it is written and the flag is set) and serves that tensor separately.
 * d_chunk_stats (2 floats per chunk) and d_tensor_stats (4 floats per tensor), both or neither: the decoded
 * values' {L2 norm, mean, 1.0 if every per-chunk figure is finite else 0.0, sum of squares} per tensor, i.e. the
 * figures of lr * grad when the factors carry lr. */
int tplr_outer_step_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_factor,
                          int n_peers, int k, const tplr_tensor_desc* d_param_desc, int n_tensors,
                          int64_t total_chunks, float* d_chunk_stats, float* d_tensor_stats, int32_t* d_nonfinite,
                          void* stream);

/* The same outer step straight from quantised payloads at templar's own settings (4-bin codes, chunks not
 * transformed, hparams/hparams.json): h_codes, d_deq as in tplr_decode_aggregate_codes_batch, d_factor[t * n_peers + p]
 * multiplies peer p's de-quantised values for tensor t (pass lr * clip factor).  The peers' payloads must be equally
 * spaced in memory and four-byte aligned, as a staged window lays them out (else TPLR_E_SHAPE); k = 32 or 64;
 * n_peers <= 24.  d_chunk_stats, d_tensor_stats, d_nonfinite as in tplr_outer_step_batch. */
int tplr_outer_step_codes_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes, const float* d_deq,
                                const float* d_factor, int n_peers, int k, const tplr_tensor_desc* d_param_desc,
                                int n_tensors, int64_t total_chunks, float* d_chunk_stats, float* d_tensor_stats,
                                int32_t* d_nonfinite, void* stream);

/* ---- validator side: checks on the packed index streams ------------------------------
 * For up to 32 peers whose flat payloads share one row layout (d_desc: n_tensors descriptors, of
 * which only chunk_begin, x_chunks and y_chunks are read; a parameter of n rows that are not
 * 64x64 chunks is one descriptor with x_chunks = n, y_chunks = 1), per tensor t:
 *   d_pair[(t * P + p) * P + q], p < q: entries of peer p that also occur in the same row of
 *       peer q, summed over the tensor's rows - `(a == b).any(-1).sum(-1)` summed over chunks in
 *       check_uid_index_overlap (src/tplr/neurons.py:1373-1378); divide by k * rows for its
 *       `mean_frac`;
 *   d_dup[t * P + p]: entries of peer p that repeat an earlier entry of their row;
 *   d_max[t * P + p]: largest index of peer p, for the bounds check of
 *       Comms.check_compressed_indices (src/tplr/comms.py:2573-2581).
 * The three arrays are accumulated into with atomics: the caller clears d_pair and d_dup to 0
 * and d_max to -1.  k even, at most 4096; indices are 12-bit by construction. */
int tplr_index_stats_batch(const uint8_t* const* h_idx12, int n_peers, int k, const tplr_tensor_desc* d_desc,
                           int n_tensors, int64_t total_rows, uint64_t* d_pair, uint64_t* d_dup, int32_t* d_max,
                           void* stream);

/* ---- payload staging: de-quantisation of a flat payload --------------------------------
 * TopKCompressor._dequantize_values (src/tplr/compress.py:637-643) for every parameter of one
 * peer's flat payload at once (the per-parameter loop of maybe_dequantize_values, :646-696,
 * src/tplr/neurons.py:325): d_val[i] = d_lookup[t * n_bins + d_codes[i]] + d_shift[t], t the
 * tensor that row i / k belongs to (d_desc: chunk_begin only).  k a multiple of 4, n_bins <= 256;
 * codes >= n_bins read the last bin (the reference would raise an index error). */
int tplr_dequantize_batch(const uint8_t* d_codes, const float* d_lookup, const float* d_shift, int n_bins, int k,
                          const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_rows, float* d_val,
                          void* stream);

/* The same arithmetic for ONE parameter's codes from n_peers peers, every peer with its own
 * lookup (d_lookup: n_peers x n_bins) and shift (d_shift: n_peers): the loop of
 * maybe_dequantize_values (src/tplr/compress.py:668-690) as it is called per parameter in
 * src/tplr/neurons.py:325, in one launch.  h_codes / h_out: host arrays of n_peers device pointers
 * (n codes in, n floats out, each; codes 4-byte and outputs 16-byte aligned).  n a multiple of 4. */
int tplr_dequantize_peers(const uint8_t* const* h_codes, int n_peers, int64_t n, const float* d_lookup,
                          const float* d_shift, int n_bins, float* const* h_out, void* stream);

/* TopKCompressor._quantize_values (src/tplr/compress.py:582-621) for every parameter of a flat
 * payload (the reference runs it per parameter inside compress, :419-421): per tensor t,
 * shift = mean of its values, scale = range_in_sigmas * std / n_bins (1 when that is 0, NaN or
 * infinite), d_codes[i] = clamp(round_half_even((v - shift) / scale + n_bins / 2), 0, n_bins - 1),
 * d_lookup[t * n_bins + b] = mean of the centred values coded b (0 for an unused bin).  Four
 * launches; every tensor is cut into n_slices (1..1024) runs of rows whose partial sums (double)
 * pass through d_work: n_tensors * n_slices * (2 + 2 * n_bins) doubles, contents irrelevant on
 * entry.  d_shift, d_scale: n_tensors floats.  k a multiple of 4, n_bins <= 256, d_val 16-byte
 * aligned; d_desc as above (chunk_begin and chunk counts). */
int tplr_quantize_batch(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                        float range_in_sigmas, int n_slices, double* d_work, uint8_t* d_codes, float* d_shift,
                        float* d_scale, float* d_lookup, void* stream);

/* The aggregate straight from quantised payloads, for a quantiser of at most four bins (templar runs
 * quantization_bins = 4, hparams/hparams.json) and chunks that are not transformed (use_dct = false): the
 * loop of maybe_dequantize_values over peers and parameters (src/tplr/compress.py:646-696,
 * src/tplr/neurons.py:325), the block norms (:346) and batch_decompress (:355-364) without ever writing the
 * fp32 values.  h_codes[p]: peer p's flat payload of one-byte codes (total_chunks * k bytes, chunk g's at g * k);
 * d_deq: (n_tensors, n_peers, 4) floats, d_deq[(t * n_peers + p) * 4 + c] = lookup[c] + shift of tensor t as
 * peer p sent them (:641-643; entries past the quantiser's bins are not read for valid codes).
 * tplr_code_sumsq: the sums of squares of the de-quantised values per (tensor, peer, slice), in the layout of
 * tplr_segment_sumsq and for the same consumer (tplr_clip_scales_batch), from four counts per slice;
 * *d_bad (caller-zeroed, nullable) receives by atomic maximum a code >= n_bins that was met (255 for any
 * byte above 3): the reference's lookup raises on such a code.
 * tplr_decode_aggregate_codes_batch: tplr_decode_aggregate_batch with use_dct = 0 and normalise = 0 whose
 * values are d_deq[..][code & 3] - the same bits as de-quantising first.  k <= 64, n_peers <= 24
 * (TPLR_E_TOOMANY beyond: de-quantise and call tplr_decode_aggregate_batch). */
int tplr_code_sumsq(const uint8_t* const* h_codes, int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                    int n_slices, int n_bins, const float* d_deq, float* d_sumsq, int32_t* d_bad, void* stream);
int tplr_decode_aggregate_codes_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes, const float* d_deq,
                                      const float* d_scale, int n_peers, int k, const tplr_tensor_desc* d_desc,
                                      int n_tensors, int64_t total_chunks, int reduce_mode, float* d_sumsq,
                                      void* stream);
/* tplr_decode_aggregate_codes_batch with the per-parameter statistics of tplr_decode_aggregate_stats_batch
 * (d_chunk_stats: 2 * total_chunks floats of scratch; d_tensor_stats: 4 floats per tensor). */
int tplr_decode_aggregate_codes_stats_batch(const uint8_t* const* h_idx12, const uint8_t* const* h_codes,
                                            const float* d_deq, const float* d_scale, int n_peers, int k,
                                            const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks,
                                            int reduce_mode, float* d_chunk_stats, float* d_tensor_stats, void* stream);

/* tplr_decode_aggregate_batch together with what its caller looks at next, per parameter
 * (src/tplr/neurons.py:380-385: L2 norm and mean of the decoded gradient for the fingerprint; :411 and
 * :438: the parameter is skipped unless every element is finite), without another pass over the dense
 * tensors: the aggregate leaves two floats per chunk in d_chunk_stats (2 * total_chunks floats, 8-byte aligned: sum of
 * squares and sum of the chunk's 4096 results) and one small launch turns them into
 * d_tensor_stats[4 t .. 4 t + 3] = {L2 norm, mean, 1.0 if every element is finite else 0.0, sum of squares}.
 * The flag is exact: a chunk whose figures are not finite is read back and examined element by element
 * (and, when its elements are all finite, summed again in double).  Norm and mean are sums in another
 * order than torch's: equal within fp32 rounding of the accumulation (1e-6 relative), non-finite when
 * the flag is 0.  Other arguments as tplr_decode_aggregate_batch. */
int tplr_decode_aggregate_stats_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                                      int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                                      int64_t total_chunks, int reduce_mode, int normalise, int use_dct,
                                      float* d_chunk_stats, float* d_tensor_stats, void* stream);

/* ---- per-tensor L2 normalisation of an aggregate ----------------------------------------------
 * The reference has no such step inside tplr.compress; the benchmark's aggregation workload words it
 * ("scatter-summed, inverse DCT, mean over peers, then L2-normalised per tensor"), and the per-chunk
 * d_sumsq output of tplr_decode_aggregate_batch exists for it.
 * tplr_tensor_rnorm: d_factor[t] = 1 / (sqrt(sum of tensor t's d_sumsq entries) + eps), the entries
 * added in a fixed order (d_desc: chunk_begin and chunk counts).
 * tplr_scale_batch: every element of tensor t times d_factor[t], in place (d_desc as for the aggregate). */
int tplr_tensor_rnorm(const float* d_sumsq, const tplr_tensor_desc* d_desc, int n_tensors, float eps, float* d_factor,
                      void* stream);
int tplr_scale_batch(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, const float* d_factor,
                     void* stream);

/* The same normalisation without a pass over the dense tensors.  The transform is orthonormal, so the L2
 * norm of a decoded tensor is the norm of its summed coefficients, which the payloads alone determine.
 * tplr_aggregate_sumsq_batch: d_sumsq[g] = sum over the coefficients of chunk g of (sum over the peers'
 * entries for that coefficient, each times d_scale[t * n_peers + p] when d_scale is given)^2; reads the
 * payloads only (arguments as tplr_decode_aggregate_batch, any even k up to 4096, repeated indices added
 * like any other entry).
 * tplr_tensor_rnorm_scales: d_factor[t] (optional) = 1 / (sqrt(sum of tensor t's d_sumsq entries) * pre + eps)
 * and d_scale[t * n_peers + p] = pre * d_factor[t] for every p: with pre = 1 / n_peers, the factors that make
 * tplr_decode_aggregate_batch in TPLR_REDUCE_SUM mode write mean-over-peers / (its L2 norm + eps) directly. */
int tplr_aggregate_sumsq_batch(const uint8_t* const* h_idx12, const float* const* h_val, const float* d_scale,
                               int n_peers, int k, const tplr_tensor_desc* d_desc, int n_tensors,
                               int64_t total_chunks, float* d_sumsq, void* stream);
int tplr_tensor_rnorm_scales(const float* d_sumsq, const tplr_tensor_desc* d_desc, int n_tensors, int n_peers,
                             float pre, float eps, float* d_factor, float* d_scale, void* stream);

/* tplr_quantize_batch for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc); it has no counterpart in the
 * reference.  Same arguments and results without d_work: the partial sums go through a static
 * device array inside the library, TPLR_STATIC_WORK_DOUBLES doubles (tplr_static_work_bytes()
 * bytes, about 8 MB, held on every GPU the library runs on until the process ends).  The call
 * allocates and frees nothing.  n_tensors * n_slices * (2 + 2 * n_bins) doubles must fit:
 * otherwise TPLR_E_WORKSPACE and nothing is launched.  Every call on a GPU uses that GPU's one
 * array, whose contents are irrelevant on entry: calls that overlap on one GPU (two streams, two
 * threads) race and must be serialised by the caller. */
#define TPLR_STATIC_WORK_DOUBLES (2048 * (2 + 2 * 256))
int64_t tplr_static_work_bytes(void);
int tplr_quantize_batch_static(const float* d_val, int k, const tplr_tensor_desc* d_desc, int n_tensors, int n_bins,
                               float range_in_sigmas, int n_slices, uint8_t* d_codes, float* d_shift,
                               float* d_scale, float* d_lookup, void* stream);

/* Measurement aid, no counterpart in the reference: a plain device-to-device copy of n_bytes
 * (a multiple of 16, both pointers 16-byte aligned) that moves exactly n_bytes each way.
 * Profilers' HBM traffic counters are scaled by what they report for this kernel. */
int tplr_calib_copy(const void* d_src, void* d_dst, int64_t n_bytes, void* stream);

/* Measurement aid, no counterpart in the reference: a plain fill of n_bytes (a multiple of 16, pointer 16-byte
 * aligned) over a linear address range with 16-byte stores, the write rate of the memory system under the
 * friendliest access pattern.  pattern 0: grid-stride (neighbouring workgroups write neighbouring kilobytes);
 * 1: the same with streaming stores; 2: every wave walks one contiguous span, as a persistent kernel would.
 * The aggregate's chunk-pattern fill (tplr_calib_aggregate with no peers) is held against it. */
int tplr_calib_fill(void* d_dst, int64_t n_bytes, int pattern, void* stream);

/* Test aid, no counterpart in the reference: fills the LDS of every compute unit with `word` (one resident round of
 * workgroups that write 80 000 bytes each).  LDS keeps its contents from kernel to kernel; the tests run the
 * aggregate kernels after it to show that nothing they read before writing it decides anything. */
int tplr_debug_fill_lds(int word, void* stream);

/* Measurement aid, no counterpart in the reference: the memory side of tplr_encode_topk_pack_batch alone.  Same
 * grid, same chunk ranges and the same 64 streaming row loads per chunk from the tensors of d_desc, without the
 * transform, the select and the payload stores.  Its duration is the time the memory system needs to hand the
 * encode its input in that access pattern - the ceiling the real kernel is held against. */
int tplr_calib_encode(const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, void* stream);

/* Measurement aid, no counterpart in the reference: the memory side of tplr_decode_aggregate_batch alone.
 * Same grid, same chunk ranges, the same streaming payload loads (n_peers <= 24, k <= 64) and the same 64 row
 * stores per chunk into the tensors of d_desc, without the scatter and the transform; what it stores is
 * meaningless.  use_dct selects whose loads it issues: with the transform the kernel fetches the packed indices
 * once per group of four (k <= 32) or two chunks, without it once per chunk.  Its duration is the time the
 * memory system needs for the aggregate's traffic in that access pattern - the ceiling the real kernel is held
 * against; n_peers = 0 gives the pure fill of the outputs.  k >= 4 with use_dct. */
int tplr_calib_aggregate(const uint8_t* const* h_idx12, const float* const* h_val, int n_peers, int k, int use_dct,
                         const tplr_tensor_desc* d_desc, int n_tensors, int64_t total_chunks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TPLR_HIP_H */
