/*
 * t5d — C ABI of the MI355X (gfx950) decode-step kernels for T5.1.1
 * encoder-decoder models.
 *
 * The reference (google-research/t5x) is pure Python/JAX and has no FFI of
 * its own; every entry point below replaces a JAX expression on the decode
 * path and cites it (paths relative to the reference checkout).  The Python
 * host code in t5x_amd/ binds this library with ctypes and keeps the
 * reference's call signatures (beam_search, temperature_sample,
 * predict_batch).
 *
 * Conventions
 *  - All pointers are DEVICE pointers unless the name ends in `_host`.
 *    The library never allocates, frees or copies device memory; the caller
 *    owns every buffer (PyTorch tensors in the Python binding).
 *  - `stream` is a hipStream_t passed as void*.  Calls only enqueue work; none
 *    synchronises.  A call is safe to record into a HIP graph.
 *  - Return value: 0 on success, a negative T5D_E* code otherwise;
 *    t5d_last_error() returns a message for the calling thread's last failure.
 *    Shapes are validated on the host before anything is launched.
 *  - Activation dtype: T5D_F32 or T5D_BF16.  bfloat16 values are rounded to
 *    nearest-even at the points where the reference casts to its activation
 *    dtype; all accumulation is float32.
 *  - Row-major, innermost dimension contiguous, unless stated otherwise.
 */
#ifndef T5D_H_
#define T5D_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { T5D_F32 = 0, T5D_BF16 = 1, T5D_I8 = 2 };

enum {
  T5D_OK = 0,
  T5D_EINVAL = -1,   /* bad shape / dtype / alignment / null pointer */
  T5D_EHIP = -2,     /* a HIP runtime call failed */
  T5D_ELIMIT = -3    /* size beyond what the kernels support */
};

/* GEMM epilogues. */
enum {
  T5D_EPI_NONE = 0,      /* C = A·W                                    */
  T5D_EPI_RESIDUAL = 1,  /* C = act(act(A·W) + residual)               */
  T5D_EPI_GEGLU = 2      /* C[:, f] = act(act(gelu(act(a0))) * act(a1)) */
};

/* Output layouts of t5d_gemm_rows. */
enum {
  T5D_OUT_ROWS = 0,        /* row-major [M, N] */
  T5D_OUT_HEADS_KEY = 1,   /* [B, H, 2, Ep, 32]: cross-attention keys */
  T5D_OUT_HEADS_VALUE = 2  /* [B, H, Ep/32, 64, 32]: cross-attention values */
};

int t5d_version(void);
const char* t5d_last_error(void);

/* Number of bytes t5d_pack_weight writes for a [K, N] kernel (padded to the
 * 32 x 16 MFMA tile grid).  w_dtype: T5D_BF16 or T5D_I8 (T5D_F32 kernels are
 * used unpacked). */
int64_t t5d_packed_weight_bytes(int w_dtype, int K, int N);

/* Repack a row-major [K, N] kernel (already cast to w_dtype) into the tile
 * order the bf16/int8 GEMM streams: tiles of 32(k) x 16(n), ordered
 * [n_tile][k_tile], each tile stored lane-major so that lane l of a wavefront
 * reads the 8 consecutive-k values W[32*kt + 8*(l/16) + j][16*nt + l%16],
 * j = 0..7, as one 16-byte (bf16) or 8-byte (int8) load.
 * geglu != 0: `src` is wi_0 and `src2` is wi_1 (each [K, N]); output column
 * 16*nt + c holds wi_0[:, 8*nt + c] for c < 8 and wi_1[:, 8*nt + c - 8]
 * otherwise, i.e. a packed [K, 2N] kernel whose tiles pair the two gates. */
int t5d_pack_weight(void* stream, int w_dtype, const void* src,
                    const void* src2, void* dst, int K, int N, int geglu);

/* Embedding row gather.  Replaces Embed.__call__ with one_hot=True
 * (t5x/examples/t5/layers.py:520-541): out[r, :] = table[ids[r], :]. */
int t5d_embed(void* stream, int dtype, const void* table, const int32_t* ids,
              void* out, int R, int d, int V);

/* T5 RMS LayerNorm (t5x/examples/t5/layers.py:683-702):
 * y = act(x * rsqrt(mean(x^2) + eps)); out = act(y * scale). */
int t5d_rmsnorm(void* stream, int dtype, const void* x, const void* scale,
                void* out, int R, int d, float eps);

/* Bias-free dense layer for few rows (DenseGeneral,
 * t5x/examples/t5/layers.py:364-414; MlpBlock gate product :460-474; the
 * residual adds of t5x/examples/t5/network.py:146,163,177).
 *   A [M, K] act dtype; W packed (bf16 / int8, see t5d_pack_weight) or
 *   row-major [K, N] float32 when dtype == T5D_F32.
 *   scales: per-output-channel float32 [N] for int8 weights, else NULL.
 *   out_dtype: dtype of C (T5D_F32 for the logits layer,
 *   t5x/examples/t5/network.py:286-291).
 *   T5D_EPI_GEGLU: W is a geglu-packed [K, 2F] kernel, N = 2F, C is [M, F].
 *   The kernels are laid out for M <= 128 (the weights stream once); more rows
 *   run as chunks of 128, each streaming the weights again.
 *   Which workgroup tile a shape runs on is internal (layers of 24 MB of
 *   weights and more with M >= 32 and K >= 2048 take large tiles of up to
 *   128 x 128, chosen so that the most loaded CU reads the fewest bytes);
 *   every tile splits and sums K the same way, so the result's bits do not
 *   depend on it.
 *   workspace/counters: reserved for plans that need scratch memory; no plan
 *   does (t5d_gemm_workspace_bytes returns 0 for every shape) and both may
 *   be NULL. */
int64_t t5d_gemm_workspace_bytes(int dtype, int w_dtype, int M, int K, int N);
int t5d_gemm(void* stream, int dtype, int w_dtype, int out_dtype,
             const void* A, const void* W, const float* scales,
             const void* residual, void* C, int M, int K, int N, int epilogue,
             void* workspace, int32_t* counters);

/* t5d_gemm on a large-tile kernel of the caller's choice (bfloat16
 * activations, M <= 128): a workgroup tile of mp*16 rows x nt*16 columns, K
 * split over k_parts workgroups.  (mp, nt) one of (2,3) (2,4) (2,5) (4,4)
 * (4,6) (4,8) (8,4) (8,5) (8,8).  k_parts > 1 needs the residual epilogue, a
 * workspace of k_parts*M*N*4 bytes, N a multiple of 8 and <= 16384: the
 * parts' float32 sums go there and a second kernel adds them in ascending
 * order and applies the epilogue.  The result does not depend on (mp, nt)
 * and equals t5d_gemm's bit for bit when k_parts == 1; it depends on k_parts
 * (summation order).  For tuning and for testing every kernel variant;
 * t5d_gemm picks the tile itself and never splits K. */
int t5d_gemm_tiled(void* stream, int dtype, int w_dtype, int out_dtype,
                   const void* A, const void* W, const float* scales,
                   const void* residual, void* C, int M, int K, int N,
                   int epilogue, void* workspace, int mp, int nt, int k_parts);

/* t5d_rmsnorm followed by t5d_gemm in one kernel (a pre-attention / pre-MLP
 * LayerNorm feeding its dense layer, t5x/examples/t5/network.py:134-139,
 * 166-171): the rows of A are normalised on their way into the matrix product,
 * with the same two roundings to bfloat16 as t5d_rmsnorm and the same
 * summation order of the product as t5d_gemm.  bfloat16 activations; packed
 * bfloat16 or int8 weights (scales: per-output-channel float32 [N] for int8,
 * else NULL); K a multiple of 64, <= 2048; epilogue NONE or GEGLU.
 * Very wide layers (bfloat16 weights, no epilogue, N >= 8192, K = 512, 768 or
 * 1024: the final LayerNorm + logits layer, t5x/examples/t5/network.py:274-291)
 * run on a kernel that keeps the normalised rows in LDS and streams only the
 * weights; there one wavefront sums all of K for its columns, so float32
 * results differ from t5d_rmsnorm + t5d_gemm by summation order (~1e-6
 * relative), deterministically.
 * float32 (activations, row-major [K, N] weights and outputs): any M, K, N;
 * the norm scale multiplies the weights as they are loaded and 1/rms the
 * finished sums, which differs from normalising first by a few float32 ulps. */
int t5d_norm_gemm(void* stream, int dtype, int w_dtype, int out_dtype,
                  const void* A, const void* norm_scale, float eps,
                  const void* W, const float* scales, void* C, int M, int K,
                  int N, int epilogue);

/* Bias-free dense layer over any number of rows (the encoder's DenseGeneral /
 * MlpBlock layers, t5x/examples/t5/layers.py:364-414,434-487, residual adds of
 * network.py:73,87, and the once-per-batch key / value projections of the
 * decoder's cross-attention, network.py:149-159).  bfloat16 activations;
 * W packed by t5d_pack_weight (bfloat16 or int8 + scales); epilogues as
 * t5d_gemm.  out_layout T5D_OUT_HEADS_KEY / T5D_OUT_HEADS_VALUE: row
 * m = b * E + e, column n = h * 64 + d is written to [B, H, 2, Ep, 32] at
 * [b, h, d / 32, e, d % 32] / to [B, H, Ep/32, 64, 32] at
 * [b, h, e / 32, d, e % 32] (the bfloat16 layouts t5d_cross_attention_step
 * and t5d_encoder_attention read; Ep a multiple of 32); positions e >= E of
 * those buffers are left untouched. */
int t5d_gemm_rows(void* stream, int w_dtype, const void* A, const void* W,
                  const float* scales, const void* residual, void* C,
                  int64_t M, int K, int N, int epilogue, int out_layout, int E,
                  int Ep);

/* t5d_gemm_rows with the workgroup tile of the caller's choice: tile 1 =
 * 256 rows x 128 columns (4 wavefronts, two workgroups per CU), tile 2 =
 * 256 x 256 and tile 3 = 256 x 192 (8 wavefronts, one workgroup per CU;
 * bfloat16 weights and K >= 64, otherwise tile 1 is used), tile 0 = what
 * t5d_gemm_rows picks from the shape.  Results have the same bits for every
 * tile.  For tuning and for testing every kernel at any size. */
int t5d_gemm_rows_tiled(void* stream, int w_dtype, const void* A,
                        const void* W, const float* scales,
                        const void* residual, void* C, int64_t M, int K, int N,
                        int epilogue, int out_layout, int E, int Ep, int tile);

/* The workgroup tile (1, 2 or 3, as in t5d_gemm_rows_tiled) that t5d_gemm_rows
 * uses for a shape: the cheapest by the rounds of workgroups each tile needs
 * on 256 CUs.  No device work; for tests and for reading a profile. */
int t5d_gemm_rows_tile(int w_dtype, int64_t M, int K, int N);

/* One step of cached decoder self-attention
 * (MultiHeadDotProductAttention decode branch,
 * t5x/examples/t5/layers.py:223-346, and dot_product_attention :52-129).
 *   qkv [R, 3*H*64]: query | key | value projections of the current token.
 *   cached_key / cached_value [R, H, 64, L] (the reference's cache layout,
 *   layers.py:231-241); column t = *cache_index receives the new key/value,
 *   then the query attends over columns 0..t.
 *   rel_bias [H, L] act dtype: rel_bias[h, n] is the decoder's relative
 *   position bias for distance n = t - j (RelativePositionBiases,
 *   layers.py:560-677, bidirectional=False).
 *   out [R, H*64].  *cache_index is read, not advanced. */
int t5d_self_attention_step(void* stream, int dtype, const void* qkv,
                            void* cached_key, void* cached_value,
                            const void* rel_bias, const int32_t* cache_index,
                            void* out, int R, int H, int L);

/* As t5d_self_attention_step for the B*beams rows of a beam search, but first
 * applying a beam gather that the caller deferred
 * (cache_gather_beams, t5x/decoding.py:1449-1457): row (b, e) attends over the
 * cache of row (b, pending_src[b, e]) and, if the item's beams were permuted,
 * that cache is written into slot (b, e).  After the call the caches equal
 * gather-then-step.  bfloat16 only; beams * ceil(L/128) <= 16.
 * pending_src may be NULL (no gather: plain t5d_self_attention_step).
 * pending_dst (optional, needs pending_src): row (b, e) keeps its cache in
 * slot (b, pending_dst[b, e]) instead of (b, e): what it read is copied there
 * unless that is where it read it, and the new column goes there.  Per item
 * pending_dst must be a permutation of 0..beams-1 and no slot that some row
 * writes without reading it may be read by another row.
 * value_blocked 1: cached_value is stored per (row, head) as
 * [L/32][64][32] (blocks of 32 positions, L a multiple of 32) instead of the
 * reference's [64][L]; 2: cached_key as well.  A caller that owns its caches
 * (a decode loop) gets loads of consecutive memory for them — a head's cache
 * is then read as whole 4 KB blocks up to the current length instead of the
 * first part of each of 64 rows — and converts when it hands the cache tree
 * out.  0: both in the reference layout.
 * value_blocked 3, the layout for a decode loop that owns its caches: a
 * (row, head) slot has (L + 32) * 64 elements in both caches;
 *   cached_key   [L + 32][64]: position-major (rows 0 .. L-1 in use), so the
 *                key a step appends is one full 128-byte line;
 *   cached_value [L/32 + 1][64][32]: finished blocks of 32 positions as with
 *                value_blocked 1, and in the last block (the tail) the
 *                positions of the block being filled, as [32][64]
 *                position-major; the step whose position completes a block
 *                writes the block and the tail starts over.
 * A reference-layout step appends a position as 64 separate 2-byte stores per
 * cache, each a partial cache line (measured: 2 of 14 us per launch at 128
 * rows x 12 heads, 21 of 73 us at 128 x 64); here it is two full lines.
 * Results have the same bits in every layout.  L a multiple of 32 and at
 * most 256 (128 for a pending_src without pending_dst); T5D_ELIMIT beyond. */
int t5d_self_attention_step_gather(void* stream, int dtype, const void* qkv,
                                   void* cached_key, void* cached_value,
                                   const void* rel_bias,
                                   const int32_t* cache_index, void* out,
                                   int B, int beams, int H, int L,
                                   const int32_t* pending_src,
                                   const int32_t* pending_dst,
                                   int value_blocked);

/* One step of encoder-decoder attention (t5x/examples/t5/network.py:149-159,
 * mask :366-370).  The reference re-projects K/V from the beam-expanded
 * encoder output every step; here they are projected once per batch item:
 *   float32: cross_key [B, H, E, 64] (head dim contiguous) and cross_value
 *   [B, H, 64, E] (positions contiguous), E a multiple of 4.
 *   bfloat16: cross_key [B, H, 2, E, 32] (dims 32 c .. 32 c + 31 of key e at
 *   [b, h, c, e, :]) and cross_value [B, H, E/32, 64, 32] (dim d of key
 *   32 j + p at [b, h, j, d, p]), E a multiple of 32: a 16-byte chunk is
 *   directly an MFMA operand of Q.K^T and P.V respectively, and the 64 chunks
 *   one wavefront load instruction fetches are 1 KB of consecutive memory.
 *   t5d_gemm_rows writes both (T5D_OUT_HEADS_KEY / T5D_OUT_HEADS_VALUE).
 *   K/V are shared by the item's `beams` rows (<= 8).
 *   enc_len [B]: number of leading valid (non-padding) encoder positions.
 *   q [B*beams, H*64] -> out [B*beams, H*64].
 *   units: NULL or the table of t5d_cross_attention_units (bfloat16). */
int t5d_cross_attention_step(void* stream, int dtype, const void* q,
                             const void* cross_key, const void* cross_value,
                             const int32_t* enc_len, void* out, int B,
                             int beams, int H, int E, const int32_t* units);

/* Work order for the bfloat16 cross-attention launches of one batch (no
 * counterpart in the reference; a scheduling aid).  A launch has one workgroup
 * per (item, head), and its work grows with the item's valid length; `units`
 * [B*H] tells workgroup p which (item, head) to take so that the CUs end up
 * evenly loaded: with at most two workgroups per CU the heaviest sit alone and
 * the others are paired heaviest with lightest, larger launches go by falling
 * length.  The entries also carry the valid length, so the table must be
 * rebuilt whenever enc_len changes.  Passing units = NULL to the attention
 * calls gives the natural order; results are identical either way.
 * B, H <= 256. */
int t5d_cross_attention_units(void* stream, const int32_t* enc_len, int B,
                              int H, int E, int32_t* units);

/* t5d_rmsnorm + the query projection (t5d_gemm) + t5d_cross_attention_step
 * in one kernel (pre_cross_attention_layer_norm, the `query` DenseGeneral and
 * the attention of t5x/examples/t5/network.py:149-159): every workgroup
 * normalises its batch item's rows of x and multiplies them with its head's
 * 64 columns of the packed query kernel while its K stream is in flight.
 *   x [B*beams, d] residual stream; ln_scale [d]; query_kernel: packed
 *   (t5d_pack_weight) [d, H*64] bfloat16 kernel.  bfloat16 only (K/V in the
 *   bfloat16 layouts above); E <= 512; d a multiple of 64, <= 1024. */
int t5d_cross_attention_step_norm_q(void* stream, int dtype, int w_dtype,
                                    const void* x, const void* ln_scale,
                                    float eps, const void* query_kernel,
                                    const void* cross_key,
                                    const void* cross_value,
                                    const int32_t* enc_len, void* out, int B,
                                    int beams, int H, int E, int d,
                                    const int32_t* units);

/* Encoder self-attention over whole sequences, bfloat16
 * (MultiHeadDotProductAttention without cache, t5x/examples/t5/layers.py:
 * 137-221,305-346, dot_product_attention :52-129, with the encoder's
 * bidirectional relative-position bias and padding mask,
 * t5x/examples/t5/network.py:47-96,325-328).
 *   q, k [B*E, *_stride]: head h in columns h*64 .. h*64+63 (row-major
 *   projections); v_t [B, H, Ep/32, 64, 32] (t5d_gemm_rows,
 *   T5D_OUT_HEADS_VALUE), Ep a multiple of 32;
 *   rel_bias [H, 2E-1] bfloat16 indexed by (key - query + E - 1);
 *   enc_len [B]: keys and queries at positions >= enc_len[b] are padding
 *   (masked with -1e10 as in the reference);
 *   valid_bits: NULL, or [B, (E + 31) / 32] words whose bit e says that
 *   position e of the item is valid (encoder_input_tokens > 0 element-wise,
 *   network.py:325-328: a padding token inside the text); positions at and
 *   beyond enc_len[b] (then: the last valid position + 1) are padding
 *   whatever their bits;
 *   out [B*E, H*64]. */
int t5d_encoder_attention(void* stream, const void* q, const void* k,
                          const void* v_t, const void* rel_bias,
                          const int32_t* enc_len, const uint32_t* valid_bits,
                          void* out, int B, int H, int E, int Ep, int q_stride,
                          int k_stride);

/* t5d_encoder_attention on the kernel of the caller's choice: variant 1 walks
 * the keys twice and forms every score twice (any E up to 2048), variant 2
 * keeps the scores of pass 1 in registers and shares K and V between the
 * wavefronts of a workgroup through LDS (E <= 512), variant 0 is what
 * t5d_encoder_attention picks (2 when E <= 512).  Same scores and
 * probabilities; the two sum a 32-key step's products in different orders, so
 * outputs agree to the last bfloat16 bit except for rare roundings.  For
 * testing both kernels on one shape. */
int t5d_encoder_attention_variant(void* stream, const void* q, const void* k,
                                  const void* v_t, const void* rel_bias,
                                  const int32_t* enc_len,
                                  const uint32_t* valid_bits, void* out, int B,
                                  int H, int E, int Ep, int q_stride,
                                  int k_stride, int variant);

/* The same attention in float32 (the dtype of the exactness tests), straight
 * from the fused projection: qkv [B*E, 3*H*64] holds q | k | v per row;
 * rel_bias [H, 2E-1] float32; enc_len / valid_bits as above; out
 * [B*E, H*64].  E <= 2048. */
int t5d_encoder_attention_f32(void* stream, const float* qkv,
                              const float* rel_bias, const int32_t* enc_len,
                              const uint32_t* valid_bits, float* out, int B,
                              int H, int E);

/* Add `delta` to n int32 values (cache_index += 1, layers.py:275). */
int t5d_add_i32(void* stream, int32_t* x, int n, int delta);

/* Beam-axis gather of cache tensors, in place
 * (cache_gather_beams, t5x/decoding.py:808-870; call site :1449-1457).
 *   cache: n_tensors tensors of [B, beams, inner, L] elements of elem_bytes,
 *   spaced tensor_stride_bytes apart; new[b, e] = old[b, beam_indices[b, e]].
 *   Only columns < *valid_len (or all L when valid_len is NULL) are moved;
 *   batch items whose indices are the identity are skipped. */
int t5d_cache_gather_beams(void* stream, void* cache, int64_t tensor_stride_bytes,
                           int n_tensors, int elem_bytes, int B, int beams,
                           int inner, int L, const int32_t* beam_indices,
                           const int32_t* valid_len, int valid_len_offset);

/* Beam-axis gather, out of place (gather_beams, t5x/decoding.py:873-915):
 * dst[b, e, :] = src[b, beam_indices[b, e], :], rows of inner_bytes bytes. */
int t5d_gather_beams(void* stream, const void* src, void* dst,
                     const int32_t* beam_indices, int B, int old_beams,
                     int new_beams, int64_t inner_bytes);

/* Exact top-k along the last axis (lax.top_k as used by
 * t5x/decoding.py:918-966,988,1426): values descending, ties toward the lower
 * index.  x [rows, n] float32 -> vals [rows, k], idx [rows, k]. k <= 64. */
int t5d_top_k(void* stream, const float* x, float* vals, int32_t* idx,
              int rows, int n, int k);

/* log_softmax over the vocabulary + prefix log-prob add + top-2K over
 * beam x vocab (t5x/decoding.py:1340-1366).
 *   logits [B*beams, V] f32, live_logprobs [B, beams] f32.
 *   topk_vals/topk_idx [B, k]: the k largest of
 *   (logits - max - lse) + live_logprobs over the flattened [beams*V] axis,
 *   flat index = beam*V + token.  row_max/row_lse [B*beams] are also written
 *   (max and log-sum-exp of the shifted row). k <= 16, beams*k <= 128.
 *   scratch: float32/int32 pairs, at least 2*B*beams*k*4 bytes. */
int t5d_beam_topk(void* stream, const float* logits,
                  const float* live_logprobs, float* topk_vals,
                  int32_t* topk_idx, float* row_max, float* row_lse,
                  void* scratch, int B, int beams, int V, int k);

/* t5d_beam_topk without the `scratch` argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  This entry point has no counterpart in
 * the reference.  The per-row candidates live in an array built into the
 * library (128 KiB on every GPU the library runs on, held until the process
 * ends), so B * beams * k must not exceed 16384; larger calls return
 * T5D_ELIMIT.  It calls no hipMalloc / hipFree.  The first call on a device
 * looks the array's address up (not a stream operation; make that call
 * outside a graph capture).  All calls on one GPU share the array: calls that
 * overlap on one GPU (different streams) race; the array keeps the previous
 * call's contents and every call overwrites the part it reads.
 * Results are bit-identical to t5d_beam_topk. */
int t5d_beam_topk_static(void* stream, const float* logits,
                         const float* live_logprobs, float* topk_vals,
                         int32_t* topk_idx, float* row_max, float* row_lse,
                         int B, int beams, int V, int k);

/* State of one beam search (t5x/decoding.py:1002-1021), device arrays. */
typedef struct {
  int32_t* cur_index;        /* scalar */
  float* live_logprobs;      /* [B, K] */
  float* finished_scores;    /* [B, K] */
  int32_t* live_seqs;        /* [B, K, S]  S = max_decode_len + 1 */
  int32_t* finished_seqs;    /* [B, K, S] */
  uint8_t* finished_flags;   /* [B, K] */
} t5d_beam_state;

/* Everything in the beam_search loop body after the top-2K
 * (t5x/decoding.py:1366-1506): prompt forcing, sequence gather + token write,
 * EOS handling, second top-K with flip, brevity-penalised finished pool merge.
 *   in/out: `cur` is read, `next` is written; they may be the same buffers
 *   (in-place update).  next.cur_index = cur.cur_index + 1.
 *   inputs [B, Lin] prompt tokens; initial_index [B];
 *   brevity [S + max(initial_index) + 1] f32: ((5+len)/6)^alpha by length.
 *   top_alive_indices [B, K] (out): source beam of each surviving beam, the
 *   argument of cache_gather_beams. */
int t5d_beam_update(void* stream, const t5d_beam_state* cur,
                    const t5d_beam_state* next, const float* topk_vals,
                    const int32_t* topk_idx, const int32_t* inputs,
                    const int32_t* initial_index, const float* brevity,
                    int32_t* top_alive_indices, int B, int K, int S, int Lin,
                    int V, int eos_id);

/* Loop condition of beam_search (t5x/decoding.py:1250-1300) evaluated on
 * `state`; writes 1 (continue) or 0 to *keep_going.
 *   min_brevity: ((5 + S)/6)^alpha; min_initial_index: min(initial_index). */
int t5d_beam_cond(void* stream, const t5d_beam_state* state, int B, int K,
                  int S, float min_brevity, float min_log_prob,
                  int max_decode_step, int min_initial_index,
                  int32_t* keep_going);

/* Token choice of one temperature_sample step (t5x/decoding.py:541-621 and
 * t5x/binary_search.py:167-227):
 *   temperature[r] <= 1e-4: argmax(logits[r]) (first occurrence);
 *   else scaled = logits / max(T, 1e-4); top-k mask (keep scaled >= k-th
 *   largest, others = -1e7) when topk > 0, or top-p mask (smallest set with
 *   probability mass >= topp, t5x/binary_search.py:230-299) when topp > 0;
 *   token = argmax(scaled + gumbel[r]);
 *   log-prob = log_softmax(rescale ? scaled : logits)[token]
 *   (0 for the greedy branch when rescale).
 *   logits, gumbel [R, V] f32 (gumbel may be NULL when every T <= 1e-4);
 *   temperature [R] f32; tokens [R] i32, logprobs [R] f32 (out).
 *   workspace: NULL, or t5d_sample_tokens_workspace_bytes(R) bytes of device
 *   memory of the caller's (4-byte aligned, contents irrelevant): with it a
 *   top-k choice (topk <= 64, rescale, R <= 128 rows of >= 4096 logits) runs
 *   as two launches — every row cut into 4 parts that list their own k
 *   largest, then one workgroup per row on those lists alone, which reads
 *   Gumbel noise only for the kept candidates — instead of one workgroup per
 *   row over everything (46 -> 13 us at 64 rows of 32128, k = 40).  The chosen
 *   tokens are the same; log-probs are summed in another order (both exact to
 *   float32 rounding). */
int64_t t5d_sample_tokens_workspace_bytes(int R);
int t5d_sample_tokens(void* stream, const float* logits, const float* gumbel,
                      const float* temperature, int32_t* tokens,
                      float* logprobs, int R, int V, int topk, float topp,
                      int rescale, void* workspace);

/* Bookkeeping of one temperature_sample step (t5x/decoding.py:631-700):
 * prompt teacher forcing, log-prob accumulation, sequence write at i+1, EOS
 * counting, `ended` update.  All arrays are updated in place.
 *   sequences [R, S] (S = L + 2); cur_index [R]; cur_token [R];
 *   ended [R] u8; log_prob [R]; max_decode_len [R]; initial_eos_count [R];
 *   *all_ended (out) = every row ended. */
int t5d_sample_update(void* stream, const int32_t* tokens,
                      const float* token_logprobs, int32_t* sequences,
                      int32_t* cur_index, int32_t* cur_token, uint8_t* ended,
                      float* log_prob, const int32_t* max_decode_len,
                      const int32_t* initial_eos_count, int32_t* all_ended,
                      int R, int S, int eos_id);

/* ids[r] = live_seqs[r, *cur_index]: the token each beam row feeds to the
 * decoder this step (t5x/decoding.py:1308-1312). live_seqs [R, S]. */
int t5d_gather_step_ids(void* stream, const int32_t* live_seqs,
                        const int32_t* cur_index, int32_t* ids, int R, int S);

/* ---- fused entry points --------------------------------------------------
 * One host call enqueues a whole decoder step / beam-search iteration, so the
 * host pays one FFI crossing per step instead of one per kernel, and the call
 * can be captured into a HIP graph once and replayed.
 * The structs hold device pointers and are read at call time only. */

typedef struct {
  /* norm scales [d] (act dtype); kernels packed with t5d_pack_weight (or
   * row-major float32), int8 scales or NULL */
  const void *ln_self, *qkv, *self_out, *ln_cross, *cross_q, *cross_out,
      *ln_mlp, *wi, *wo;
  const float *qkv_scales, *self_out_scales, *cross_q_scales,
      *cross_out_scales, *wi_scales, *wo_scales;
  void *cached_key, *cached_value;        /* [R, H, 64, L] */
  const void *cross_key;    /* as t5d_cross_attention_step takes them */
  const void *cross_value;
} t5d_layer;

typedef struct {
  int dtype, w_dtype;
  int d, H, F, V, L, E, NL;   /* emb, heads, mlp, vocab, cache len, enc len */
  int R, B, beams;            /* R = B * beams decoder rows */
  const void* embedding;      /* [V, d] act dtype */
  const void* rel_bias;       /* [H, L] act dtype, by distance */
  const void* ln_final;
  const void* logits_w;
  const float* logits_scales;
  const t5d_layer* layers;    /* HOST array of NL entries */
  int32_t* cache_index;       /* [NL] device, consecutive */
  const int32_t* enc_len;     /* [B] */
  /* optional [B*H]: t5d_cross_attention_units of enc_len (bfloat16 only) */
  const int32_t* cross_units;
  void *x, *x1, *x2, *xn;     /* [R, d] activations */
  void *qkv;                  /* [R, 3*H*64] */
  void *q, *ao;               /* [R, H*64] */
  void *h;                    /* [R, F] */
  float* logits;              /* [R, V] (out) */
  /* optional device flag: when non-NULL and 0, every kernel of the step
   * returns immediately (the step becomes a no-op) */
  const int32_t* gate;
  /* optional [B, beams] source slots of a deferred cache gather, applied
   * inside the self-attention kernels (t5d_self_attention_step_gather), and
   * optional destination slots (NULL: row e keeps slot e) */
  const int32_t* pending_src;
  const int32_t* pending_dst;
  /* the layers' cache layout, as value_blocked of
   * t5d_self_attention_step_gather (bfloat16; 0: the reference layout) */
  int value_blocked;
} t5d_model_step;

/* One decoder step for R rows (Decoder.__call__ with decode=True,
 * t5x/examples/t5/network.py:229-292, as driven by
 * _compute_logits_from_slice, t5x/models.py:484-515): ids [R] -> logits,
 * caches updated in place, every cache_index advanced by one. */
int t5d_decoder_step(void* stream, const t5d_model_step* model,
                     const int32_t* ids);

typedef struct {
  t5d_beam_state state;        /* updated in place */
  const int32_t* inputs;       /* [B, Lin] */
  const int32_t* initial_index;/* [B] */
  const float* brevity;        /* by length */
  int32_t* top_alive;          /* [B, K] */
  float* topk_vals;            /* [B, 2K] */
  int32_t* topk_idx;           /* [B, 2K] */
  float *row_max, *row_lse;    /* [R] */
  void* scratch;               /* 2*R*2K*4 bytes */
  int32_t* ids;                /* [R] */
  int32_t* keep_going;         /* loop flag; must equal model->gate */
  int S, Lin, eos_id;
  float min_brevity, min_log_prob;
  int max_decode_step, min_initial_index;
  void* kv_base;               /* first cache tensor [B, K, H, 64, L] */
  int64_t kv_tensor_stride_bytes;
  int n_kv_tensors;            /* 2 * NL when all layers share one block */
  /* non-zero: *keep_going is only read (as the gate); the caller runs
   * t5d_beam_cond itself, e.g. once over all slices of a batch that it steps
   * on separate streams */
  int skip_cond;
  /* optional, all three or none, [B, K] each: where the beams' cache rows
   * live.  cache_slot[b, e] = slot of beam e (identity before the first
   * iteration; updated in place).  Every iteration writes, for the next reader
   * of the cache, cache_src[b, e] = slot holding the rows of new beam e's
   * parent and cache_dst[b, e] = slot of new beam e: the first child of a
   * parent inherits its slot (a re-ranking of the beams moves nothing), further
   * children are copied into slots that no new beam reads.  With these set the
   * model's pending_src / pending_dst must be cache_src / cache_dst.  Beam
   * e's cache is then NOT in row e: after an iteration it is in row
   * cache_src[b, e], and from the next iteration's self-attention on in row
   * cache_dst[b, e] = cache_slot[b, e]. */
  int32_t *cache_slot, *cache_src, *cache_dst;
} t5d_beam_step;

/* One iteration of the beam_search loop body plus the loop condition
 * (t5x/decoding.py:1250-1506): gather ids, decoder step, log_softmax + top-2K,
 * bookkeeping, cache reorder over the valid prefix (done here, or deferred to
 * the next step's self-attention when model->pending_src == beam->top_alive,
 * which must then start as the identity, or == beam->cache_src with the slot
 * bookkeeping above), condition -> *keep_going.
 * Every kernel is gated on *keep_going, so iterations enqueued after the
 * condition turned false leave all state untouched. */
int t5d_beam_search_step(void* stream, const t5d_model_step* model,
                         const t5d_beam_step* beam);

typedef struct {
  int32_t* sequences;              /* [R, S], S = L + 2; updated in place */
  int32_t* cur_index;              /* [R] */
  int32_t* cur_token;              /* [R]: the ids the decoder step consumes */
  uint8_t* ended;                  /* [R] */
  float* log_prob;                 /* [R] */
  const int32_t* max_decode_len;   /* [R] */
  const int32_t* initial_eos_count;/* [R] */
  const float* temperature;        /* [R] */
  /* Gumbel noise for the coming steps, [noise_ring, R, V] f32: executed step n
   * reads slot n % noise_ring.  May be NULL when every temperature <= 1e-4. */
  const float* gumbel;
  int noise_ring;
  int32_t* step_count;             /* device counter of executed steps */
  int32_t* tokens;                 /* [R] scratch */
  float* token_logprobs;           /* [R] scratch */
  void* workspace;                 /* NULL or as t5d_sample_tokens takes it */
  int32_t* all_ended;              /* out: every row ended */
  int32_t* keep_going;             /* loop flag = !all_ended; == model->gate */
  int S, eos_id, topk, rescale;
  float topp;
} t5d_sample_step;

/* One iteration of the temperature_sample loop body plus its condition
 * (t5x/decoding.py:509-700): decoder step on cur_token, token choice
 * (t5d_sample_tokens), bookkeeping (t5d_sample_update); the layers' cache
 * indices and *step_count advance, *keep_going = !all_ended.  Every kernel is
 * gated by *keep_going, so iterations enqueued after the last row ended change
 * nothing.  Covers the loop without state / logit callbacks. */
int t5d_temperature_sample_step(void* stream, const t5d_model_step* model,
                                const t5d_sample_step* sample);

/* HIP graph capture on `stream` (must not be the null stream):
 * begin, enqueue any t5d calls, end -> executable graph; launch replays it. */
int t5d_graph_begin(void* stream);
int t5d_graph_end(void* stream, void** graph_exec);
int t5d_graph_launch(void* graph_exec, void* stream);
int t5d_graph_destroy(void* graph_exec);

#ifdef __cplusplus
}
#endif
#endif  /* T5D_H_ */
