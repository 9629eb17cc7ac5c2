/*
 * tqamd -- C ABI of the MI355X (gfx950) TurboQuant V3 KV-cache codec.
 *
 * Plain pointers and sizes only.  Every entry point returns an int status:
 *   0            success
 *   < 0          argument error (TQ_ERR_*), nothing was launched
 *   > 0          a hipError_t reported by the HIP runtime
 * No entry point allocates or frees device memory or synchronises the device;
 * work is enqueued on the caller's stream.  The library keeps no state between
 * calls apart from per-device launch parameters it looks up once and the
 * counters of tq_decompress_batched_noalloc (described there).
 *
 * Each declaration cites the line range of the upstream Python reference
 * (tonbistudio/turboquant-pytorch, turboquant/...) whose behaviour it replaces.
 */
#ifndef TQAMD_H
#define TQAMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TQ_ABI_VERSION 5

/* element types of K/V tensors */
enum { TQ_F32 = 0, TQ_F16 = 1, TQ_BF16 = 2 };

enum {
    TQ_OK = 0,
    TQ_ERR_NULL = -1,        /* a required pointer is NULL */
    TQ_ERR_BITS = -2,        /* bits outside 1..8 */
    TQ_ERR_HEAD_DIM = -3,    /* head_dim the kernels do not support (see tq_compress) */
    TQ_ERR_DTYPE = -4,       /* unknown element type */
    TQ_ERR_SIZE = -5,        /* negative / inconsistent size, stride or buffer too small */
    TQ_ERR_CODEBOOK = -6,    /* centroids not finite and strictly ascending */
    TQ_ERR_TABLE = -7,       /* table blob malformed (bad magic / version) */
    TQ_ERR_ALIGN = -8,       /* pointer or stride not aligned as required */
    TQ_ERR_NO_DEVICE = -9,   /* no usable HIP device */
    TQ_ERR_CAPACITY = -10    /* request larger than the fixed capacity of an entry point that allocates nothing */
};

int tq_abi_version(void);
const char *tq_status_string(int status);

/* Number of HIP devices visible (0 when there is none); never fails. */
int tq_device_count(void);

/*
 * Packed bytes per vector: ceil(head_dim / floor(8 / bits)).
 * Replaces the size arithmetic of MSECompressor.compress / memory_bytes,
 * compressors_v3.py:64-69 and :111-112.  Returns TQ_ERR_BITS for bits outside 1..8.
 */
int tq_bytes_per_vector(int head_dim, int bits);

/*
 * Decision thresholds of the nearest-centroid rule.  thresholds[i] (i < levels-1) is the
 * smallest float32 r for which |r - c[i+1]| < |r - c[i]| in float32 arithmetic, so that
 *     argmin_j |r - c[j]|  (first minimum on ties)  ==  #{ i : r >= thresholds[i] }
 * for every finite r.  Replaces the [N,D,L] broadcast + abs + argmin of
 * compressors_v3.py:60-61.  Host only.
 */
int tq_decision_thresholds(const float *centroids, int levels, float *thresholds);

/*
 * Codec table: everything a compressor instance keeps on the device, baked on the host
 * into one blob (rotation split into 16-bit MFMA operand tiles for both directions,
 * quantiser lookup grid, decode tables).  Replaces the device state built by
 * MSECompressor.__init__ (self.Pi, self.centroids), compressors_v3.py:37-43.
 *
 *   tq_table_bytes  size of the blob for (head_dim, bits); < 0 on error
 *   tq_table_build  fill `table_host` (host memory, tq_table_bytes long) from
 *                   Pi [head_dim*head_dim] row-major float32 (rotated = x @ Pi^T, as
 *                   turboquant.py:18-33 returns it) and centroids [2^bits] ascending.
 * The caller copies the blob to device memory (256-byte aligned) and passes that pointer
 * to the compress / decompress entry points.
 */
long long tq_table_bytes(int head_dim, int bits);
int tq_table_build(const float *Pi, const float *centroids, int head_dim, int bits,
                   void *table_host, size_t table_bytes);

/*
 * Checks a table blob in host memory against the (head_dim, bits) it is about to be used with: TQ_OK, or
 * TQ_ERR_TABLE (bad magic / version / size, or built for another head_dim or another bit width).  The launch
 * entry points cannot make this check (the blob they get is in device memory and `bits` selects the kernel):
 * a binding keeps `bits` next to every table pointer and calls this once per table, before the first launch.
 */
int tq_table_check(const void *table_host, size_t table_bytes, int head_dim, int bits);

/*
 * Host emulation of the kernels' quantiser lookup, bit for bit (same fused multiply-add,
 * same grid): idx[i] = code chosen for unit-sphere coordinate r[i].  For tests of the
 * table contents; the product path never calls it.
 */
int tq_table_quantize_host(const void *table_host, const float *r, long long n, uint8_t *idx);

/*
 * compress: K or V vectors -> packed codes + fp16 norms.
 * Replaces MSECompressor.compress, compressors_v3.py:46-81.
 *
 *   states      device pointer, `dtype` elements; vector n (0 <= n < rows*tokens) starts at
 *               element  (n / tokens) * row_stride + (n % tokens) * token_stride
 *               and its head_dim elements are contiguous.  A contiguous
 *               [B,H,S,D] tensor is rows=1, tokens=B*H*S, token_stride=D; a slice
 *               [:, :, :s, :] of one is rows=B*H, tokens=s, row_stride=S*D.
 *               Base address and strides must keep every vector 16-byte aligned (head dimensions that are
 *               not a multiple of 32: aligned to the element size).
 *   head_dim    128 runs the tuned kernels; tq_compress, tq_decompress and their batched forms also take
 *               every other head dimension from 8 to 256 (compressors_v3.py:37-43 accepts any head_dim):
 *               64 and 256 through kernels of their own, the rest through one pair of kernels that reads the
 *               dimension at run time and works on a dimension that is not a multiple of 32 as the next
 *               multiple (zero elements in, zero codes up to a whole byte out: compressors_v3.py:64-68).
 *               Everything else in this header (scores, weighted values, attention, token append, QJL signs)
 *               is 128 only.
 *   table_dev   device copy of the blob from tq_table_build
 *   idx_bytes   device, uint8, bytes_per_vector per packed slot
 *   vec_norms   device, one IEEE fp16 bit pattern per packed slot (norm of the fp32-widened vector)
 *   packed_row_stride
 *               vector n uses packed slot  (n / tokens) * packed_row_stride + (n % tokens)  of
 *               idx_bytes and vec_norms.  0 means `tokens`: the dense [rows*tokens] layout the
 *               reference returns.  A larger value appends to a preallocated per-row store
 *               [rows, capacity]: pass pointers already advanced to the first free token and
 *               packed_row_stride = capacity (the chunk list of generation_test_v2.py:109-126
 *               kept as one buffer).
 *   workspace   device memory of tq_workspace_bytes(1) bytes, 64-byte aligned, or NULL: the counters from which
 *               the blocks of a large single-row job of 16-bit elements draw runs of tiles in the order in which
 *               they become free (compute units that run slower take fewer, and all blocks end together; the
 *               results are the same bytes).  Same contract as the workspace of tq_decompress below: zero before
 *               its first use, left zero by every launch that completes, never shared by launches that can
 *               overlap in time.  NULL selects the fixed assignment of tiles to blocks.
 *   stream      hipStream_t (NULL = the default stream)
 */
int tq_compress(const void *states, int dtype, long long rows, long long tokens,
                long long row_stride, long long token_stride,
                const void *table_dev, int head_dim, int bits,
                uint8_t *idx_bytes, uint16_t *vec_norms, long long packed_row_stride,
                void *workspace, void *stream);

/*
 * decompress: packed codes + fp16 norms -> vectors of `out_dtype`.
 * Replaces MSECompressor.decompress, compressors_v3.py:84-105 (out_dtype = TQ_F32), and with
 * TQ_F16 / TQ_BF16 the fused `.to(dtype)` + torch.cat into the full-length K/V buffer of
 * TurboQuantV3.decompress_kv, compressors_v3.py:226-232: vector n is written at element
 *   (n / tokens) * row_stride + (n % tokens) * token_stride   of `out`
 * and read from packed slot (n / tokens) * packed_row_stride + (n % tokens) (0 = dense), which
 * also covers the loop over stored chunks of generation_test_v2.py:131-135.
 *
 *   workspace   device memory of tq_workspace_bytes(1) bytes, 64-byte aligned, or NULL.  It holds the
 *               counter from which the kernel's blocks draw their tiles in the order in which they
 *               become free, which keeps the output addresses written at any moment close together
 *               (measurably faster than a fixed assignment of tiles to blocks on large jobs; the
 *               results are the same bytes).  Contract: all zero before its first use; every launch
 *               that completes leaves it all zero again; two launches that can overlap in time
 *               (different streams) must not share one.  NULL selects the fixed assignment.
 */
#define TQ_MAX_JOBS 4096               /* most jobs one batched launch takes */
#define TQ_WORKSPACE_BYTES_PER_JOB 256
/* bytes of workspace for a launch of n_jobs jobs (n_jobs = 1 for tq_decompress); TQ_ERR_SIZE if n_jobs < 0 or > TQ_MAX_JOBS */
long long tq_workspace_bytes(int n_jobs);

int tq_decompress(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
                  long long rows, long long tokens,
                  const void *table_dev, int head_dim, int bits,
                  void *out, int out_dtype, long long row_stride, long long token_stride,
                  void *workspace, void *stream);

/*
 * Batched forms: one launch for many (layer, tensor) jobs, each with its own table.
 * Replaces the per-layer Python loop over TurboQuantV3.compress_kv / decompress_kv calls
 * (callers: generation_test_v2.py:65-78,109,121,135; validate_v3.py:71-84).
 * All jobs of one call share `bits` and `dtype` (group by width and launch once per group).
 * `jobs_host` is read for validation and launch sizing; `jobs_dev` is a device copy of the
 * same n_jobs records that the kernel reads -- the caller uploads it once and may reuse it
 * for every call with the same buffers (nothing is allocated here).
 * Both take a workspace of tq_workspace_bytes(n_jobs) bytes under the contract stated at
 * tq_decompress (job i uses bytes [i * TQ_WORKSPACE_BYTES_PER_JOB, ...)), or NULL; a compress and a
 * decompress launch that cannot overlap in time may share one.
 */
typedef struct tq_job {
    const void *states;        /* compress: input vectors;   decompress: output vectors   */
    uint8_t *idx_bytes;        /* compress: output;          decompress: input            */
    uint16_t *vec_norms;       /* compress: output;          decompress: input            */
    const void *table_dev;     /* this job's codec table                                 */
    long long rows, tokens;    /* vector n = (n / tokens, n % tokens)                     */
    long long row_stride;      /* elements, for `states`                                  */
    long long token_stride;    /* elements, for `states`                                  */
    int bits;                  /* 1..8, must match the table                              */
    int dtype;                 /* element type of `states`                                */
    long long packed_row_stride; /* packed slots per row of idx_bytes / vec_norms; 0 = tokens */
} tq_job;

int tq_compress_batched(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                        int head_dim, void *workspace, void *stream);
int tq_decompress_batched(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                          int head_dim, void *workspace, void *stream);

/*
 * V2 key path: MSE codes of (bits - 1) bits plus one QJL sign bit per coordinate of the quantisation residual, for the
 * unbiased inner-product estimate  <q, k> ~ <q, k_mse> + ||r|| * sqrt(pi/2) / D * <S q, sign(S r)>.
 * Replaces TurboQuantCompressorV2.compress / asymmetric_attention_scores, turboquant/compressors.py:84-158 (and the
 * two-stage quantiser TurboQuantProd.quantize / inner_product, turboquant/turboquant.py:134-192, whose arithmetic it is).
 * Stored per vector, as the reference's own memory accounting counts it (validate.py:121-127): packed MSE codes and
 * fp16 norm (tq_compress with mse_bits and the table of tq_table_build), 16 bytes of sign bits, fp16 residual norm.
 *
 *   tq_qjl_table_bytes / tq_qjl_table_build
 *                   host blob with Pi^T and S as MFMA operand tiles and the codebook, from Pi (row-major, as
 *                   tq_table_build takes it), S [head_dim * head_dim] row-major (projected = residual @ S^T,
 *                   compressors.py:49-52 and :116) and the 2^mse_bits centroids; upload it 256-byte aligned.
 *   tq_qjl_signs    second stage of compress (:107-117): from the input vectors (n_vec of them, token_stride elements
 *                   apart, 16-byte aligned) and the codes tq_compress wrote for them (dense [n_vec, G]):
 *                   residual = x - (centroids[codes] @ Pi) * ||x||  in float32,
 *                   sign_bytes[v][b] bit 7-k = (residual @ S^T)[8b + k] >= 0  (the 1-bit code packing of tq_compress),
 *                   residual_norm[v] = fp16(||residual||).
 * Scores need no entry point of their own: term 1 is tq_scores on the MSE codes with q_rot = Pi q, term 2 is tq_scores
 * on sign_bytes / residual_norm as a 1-bit store whose table was built from the identity rotation and the codebook
 * (-1, +1), with q_rot = sqrt(pi/2) / head_dim * S q.
 */
long long tq_qjl_table_bytes(int head_dim, int mse_bits);
int tq_qjl_table_build(const float *Pi, const float *S, const float *centroids, int head_dim, int mse_bits,
                       void *table_host, size_t table_bytes);
int tq_qjl_signs(const void *states, int dtype, long long n_vec, long long token_stride,
                 const uint8_t *idx_bytes, const void *qjl_table_dev, int head_dim, int mse_bits,
                 uint8_t *sign_bytes, uint16_t *residual_norm, void *stream);

/*
 * TurboQuantCompressorV2.compress (compressors.py:84-122) as one call: packed MSE codes and fp16 norms (what tq_compress
 * writes with mse_bits and `table_dev`), the 16 sign bytes and the fp16 residual norm of every vector (what tq_qjl_signs
 * writes).  The n_vec vectors lie token_stride elements apart; all four outputs are dense ([n_vec, G], [n_vec],
 * [n_vec, 16], [n_vec]).  For 16-bit inputs and codes of up to TQ_QJL_ONE_PASS_MAX_BITS bits the vectors are read once, by a
 * kernel that works on the residual in rotated coordinates ((Pi x)[k] - ||x|| centroid(code_k), projected by S Pi^T
 * from the table of tq_qjl_table_build); float32 inputs, wider codes and the last n_vec % 32 vectors of a job take
 * tq_compress followed by tq_qjl_signs.  Both forms write the same codes and norms; their sign bits agree wherever a
 * projection is further than 1e-5 of |S row| |residual| from zero.
 * The batched form is one launch for many (layer) jobs that share dtype and mse_bits; `jobs_dev` is a device copy of the
 * same records, uploaded once by the caller (the per-layer loop of validate.py:96-111).
 */
#define TQ_QJL_ONE_PASS_MAX_BITS 4
typedef struct tq_qjl_job {
    const void *states;          /* input vectors                                        */
    uint8_t *idx_bytes;          /* out: packed MSE codes, dense [n_vec, G]              */
    uint16_t *vec_norms;         /* out: fp16 norms [n_vec]                              */
    uint8_t *sign_bytes;         /* out: [n_vec, 16]                                     */
    uint16_t *residual_norm;     /* out: fp16 [n_vec]                                    */
    const void *table_dev;       /* tq_table_build(Pi, centroids, mse_bits)              */
    const void *qjl_table_dev;   /* tq_qjl_table_build(Pi, S, centroids, mse_bits)       */
    long long n_vec;
    long long token_stride;      /* elements                                             */
    int mse_bits;                /* 1..7, the same in all jobs of a call                 */
    int dtype;                   /* element type of `states`, the same in all jobs       */
} tq_qjl_job;
int tq_qjl_compress(const void *states, int dtype, long long n_vec, long long token_stride, const void *table_dev,
                    const void *qjl_table_dev, int head_dim, int mse_bits, uint8_t *idx_bytes, uint16_t *vec_norms,
                    uint8_t *sign_bytes, uint16_t *residual_norm, void *stream);
int tq_qjl_compress_batched(const tq_qjl_job *jobs_host, const tq_qjl_job *jobs_dev, int n_jobs, int head_dim, void *stream);
/*
 * Both terms of asymmetric_attention_scores (compressors.py:124-158) in one launch, from the packed form (dense buffers
 * of `rows` rows x `tokens` tokens) for any number of query tokens per row:
 *   scores[(r * n_queries + q) * tokens + t] = norm_t * q_rot[r][q] . centroids[codes_t] + residual_norm_t * q_sign[r][q] . signs_t
 * with q_rot = Pi q and q_sign = sqrt(pi/2) / head_dim * S q (float32 [rows, n_queries, head_dim], contiguous), `table_dev`
 * the codec table of the MSE stage.  rows <= 65535.
 */
int tq_qjl_scores(const uint8_t *idx_bytes, const uint16_t *vec_norms, const uint8_t *sign_bytes, const uint16_t *residual_norm,
                  long long rows, long long tokens, const void *table_dev, int head_dim, int mse_bits,
                  const float *q_rot, const float *q_sign, long long n_queries, float *scores, void *stream);

/*
 * tq_decompress_batched for callers that cannot allocate device memory and have no workspace to pass: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, checks and output bytes as tq_decompress_batched; the ticket counters live in a
 * device array inside the library (TQ_NOALLOC_MAX_JOBS * TQ_WORKSPACE_BYTES_PER_JOB = 128 KiB on each device
 * the library runs on, held until the process ends) and the words a call uses are cleared by a small kernel on
 * `stream` before the launch.  More than TQ_NOALLOC_MAX_JOBS jobs: TQ_ERR_CAPACITY, nothing is launched.  The
 * call allocates and frees nothing.  All calls on one device share the array: two calls that can overlap in
 * time on one device (different streams, different threads) race on the counters and must be serialised by
 * the caller.  The first call on a device looks the array's address up in the loaded code object; make that
 * call outside graph capture.
 */
#define TQ_NOALLOC_MAX_JOBS 512
int tq_decompress_batched_noalloc(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                                  int head_dim, void *stream);

/*
 * Decode-time attention on the packed cache, without de-quantising it.  Replaces, for single-token
 * decode steps, "de-quantise every stored chunk (generation_test_v2.py:131-135, compressors_v3.py:84-105)
 * and let the model multiply by the result" (score definition: validate_v3.py:87).
 * `rows` = batch * kv_heads packed rows of `tokens` tokens (slot of token t of row r:
 * r * packed_row_stride + t; 0 = tokens); query head (r * group + g) belongs to row r.
 *
 * tq_scores:   scores[(r*group + g) * scores_stride + t] = norm_t * sum_j q_rot[r][g][j] * centroid[code(t, j)]
 *              = q . k_hat_t  when  q_rot = Pi q  (times any softmax scale folded into q_rot).
 *              q_rot: device, float32 [rows, group, head_dim] contiguous; group <= 32.
 * tq_weighted_values:
 *              out_rot[r][g][j] = sum_t weights[(r*group + g) * weights_stride + t] * norm_t * centroid[code(t, j)],
 *              so that  sum_t w_t v_hat_t = out_rot[r][g] @ Pi.  group <= 8 per call.  The token range is
 *              cut into `splits` pieces summed in a fixed order; `partial` is caller-provided scratch of
 *              rows * splits * group * head_dim floats.  tq_weighted_values_splits suggests a split count.
 */
int tq_scores(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
              long long rows, long long tokens, const void *table_dev, int head_dim, int bits,
              const float *q_rot, int group, float *scores, long long scores_stride, void *stream);
int tq_weighted_values_splits(long long rows, long long tokens);
int tq_weighted_values(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
                       long long rows, long long tokens, const void *table_dev, int head_dim, int bits,
                       const float *weights, long long weights_stride, int group,
                       float *partial, int splits, float *out_rot, void *stream);

/*
 * The same attention in one pass over the packed keys and values (scores, softmax statistics and the
 * weighted value sums never leave the chip): for every (row, split of the token range, query head g)
 *   partial[((r * splits + s) * group + g) * 130 + {0, 1, 2..129}] =
 *       { m,  sum_t exp(score_t - m),  sum_t exp(score_t - m) * norm_t * centroid[code(t, j)] }
 * with score_t as tq_scores computes it (q_rot carries the softmax scale) and m a reference score of the split:
 * never above its largest score and at most 8 ln 2 below it (it follows the running maximum lazily).  The
 * rotated queries enter as one fp16 term per coordinate for keys of up to 4 bits (relative rounding 2^-12, the
 * precision the fp16 centroids of the decoded keys have) and as fp16 hi + lo for wider keys.  The caller merges the splits
 * (and any uncompressed tokens) by the usual log-sum-exp rule and multiplies the 128 sums by Pi of the value
 * codec.  Keys and values share rows, tokens and packed_row_stride; group <= 16.  Same replaced reference
 * lines as tq_scores / tq_weighted_values.  tq_attend_splits suggests a split count.
 */
int tq_attend_splits(long long rows, long long tokens);
/*
 * The two small ends of such a decode step, so that a layer costs three launches:
 *   tq_attend_prepare  q_rot[r][g] = scale * Pi_k q[r][g]  for the one query token of every head ([rows, group, 128]
 *                      elements of q_dtype), and the same {largest score, sum of exp, 128 weighted value sums} record
 *                      over the n_win (<= 512) uncompressed window tokens of every row (row r, token t at element
 *                      r * win_stride + t * 128 of k_win / v_win; plain, un-rotated space) -> part_w [rows, group, 130];
 *   tq_attend_merge    log-sum-exp merge of the splits' records (tq_attend_partials) and of the window's, rotation
 *                      of the packed part back by Pi_v, normalisation, cast -> out [rows, group, 128].
 * pi_k_t: device copy of the key codec's rotation, transposed (float32 [128,128], element [i][j] = Pi[j][i]);
 * pi_v: the value codec's rotation as MSECompressor keeps it (float32 [128,128] row-major).
 * k_win / v_win are 16-byte aligned and win_stride is a multiple of 8 (TQ_ERR_ALIGN otherwise).  group <= 16
 * in both.
 */
int tq_attend_prepare(const void *queries, int q_dtype, long long rows, int group, float scale,
                      const float *pi_k_t, const void *k_win, const void *v_win, int win_dtype,
                      long long n_win, long long win_stride, float *q_rot, float *part_w, void *stream);
int tq_attend_merge(const float *partial, int splits, const float *part_w, const float *pi_v,
                    long long rows, int group, void *out, int out_dtype, void *stream);
int tq_attend_partials(const uint8_t *k_idx, const uint16_t *k_norms, const uint8_t *v_idx, const uint16_t *v_norms,
                       long long packed_row_stride, long long rows, long long tokens,
                       const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                       const float *q_rot, int group, int splits, float *partial, void *stream);

/*
 * One decode step of a streaming cache layer as two calls (each chains the entry points above; for hosts
 * that pay per call).  Replaces the bookkeeping of V3Cache.update for one new token per sequence,
 * generation_test_v2.py:96-126, on a cache kept as one packed store [rows, capacity] plus a window buffer
 * [rows, win_cap, 128] per tensor.
 *
 * tq_append_token: if evict >= 0, window token `evict` of every row is compressed into packed slot
 * `packed_slot` of the row (tq_compress with rows x 1 token; k_idx .. v_norms are the bases of the stores,
 * packed_row_stride their capacity); then the new key / value vector of every row (row r at element
 * r * k_new_stride / r * v_new_stride) is written to window token `put`.  dtype is the element type of the
 * new vectors and of the window; win_stride = elements between rows of the window buffers.  Pointers are
 * 16-byte aligned, strides multiples of 16 bytes.
 *
 * tq_attend_step: tq_attend_prepare, tq_attend_partials (if tokens > 0, with `splits` splits) and
 * tq_attend_merge in a row; q_rot [rows, group, 128], part_w [rows, group, 130] and
 * partial [rows, splits, group, 130] are float32 scratch of the caller.  k_win / v_win point at the first
 * of the n_win window tokens.  tokens = 0 and n_win = 0 together: TQ_ERR_SIZE.
 */
int tq_append_token(const void *k_new, const void *v_new, int dtype, long long k_new_stride, long long v_new_stride,
                    void *k_win, void *v_win, long long win_stride, long long evict, long long put,
                    const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                    uint8_t *k_idx, uint16_t *k_norms, uint8_t *v_idx, uint16_t *v_norms,
                    long long packed_row_stride, long long packed_slot, long long rows, void *stream);
int tq_attend_step(const void *queries, int q_dtype, long long rows, int group, float scale,
                   const float *pi_k_t, const float *pi_v,
                   const void *k_win, const void *v_win, int win_dtype, long long n_win, long long win_stride,
                   const uint8_t *k_idx, const uint16_t *k_norms, const uint8_t *v_idx, const uint16_t *v_norms,
                   long long packed_row_stride, long long tokens,
                   const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                   float *q_rot, float *part_w, float *partial, int splits,
                   void *out, int out_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TQAMD_H */
