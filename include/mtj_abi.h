/*
 * mtj_abi.h - C ABI of the MI355X (gfx950) GPT-J forward/decode kernels.
 *
 * The reference (kingoflolz/mesh-transformer-jax) is pure Python on JAX: it has no FFI of its own,
 * so these entry points are what a binding for its generate path would bind.  Each one cites the
 * reference code whose XLA-generated kernels it replaces (paths relative to the reference checkout).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; nothing here allocates, frees or
 *     keeps a pointer after returning;
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*), never synchronises,
 *     and is safe to record into a HIP graph: per-step scalars (positions) are read from device memory;
 *   - return value: 0 on success, a negative MTJ_E* code otherwise; mtj_last_error() returns the
 *     message of the calling thread's last failure;
 *   - activations are float32 unless `dtype` says otherwise; `dtype` selects the storage type of
 *     weights / K,V cache / GEMM inputs: MTJ_F32 (exact path), MTJ_BF16 or MTJ_F16.  The reference multiplies
 *     float32 activations with bf16 weights (jnp.dot(f32, bf16)); the matrix cores want both operands in one
 *     16-bit type, and float16 holds every bf16 weight exactly (after a power-of-two scale, see
 *     mtj_pack_weight_cvt) while rounding an activation to 11 significant bits instead of bf16's 8, so the
 *     matrix-core paths of a bf16 model run in MTJ_F16;
 *   - conversions to MTJ_F16 saturate at +-65504;
 *   - "packed" weights are row-major [N_out, K_in] (K contiguous), i.e. the transpose of haiku's
 *     [in, out]; mtj_pack_weight builds them, with row/column offsets so that q|v|k|fc_in are
 *     concatenated along N and out|fc_out along K.
 */
#ifndef MTJ_ABI_H
#define MTJ_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MTJ_ABI_VERSION 4

enum { MTJ_F32 = 0, MTJ_BF16 = 1, MTJ_F16 = 2 };

enum {
  MTJ_OK = 0,
  MTJ_EINVAL = -1,   /* bad shape / argument (mirrors the reference's Python asserts) */
  MTJ_EALIGN = -2,   /* pointer or leading dimension not 16-byte aligned */
  MTJ_EDTYPE = -3,   /* unsupported dtype */
  MTJ_EHIP = -4,     /* HIP launch error, message holds hipGetErrorString */
  MTJ_ELIMIT = -5    /* size beyond what the kernel supports (e.g. LDS capacity) */
};

int mtj_version(void);
const char* mtj_last_error(void);

/* Epilogues of mtj_gemm / mtj_gemv. */
enum {
  MTJ_EPI_STORE = 0,  /* out[m, n] = acc (+ bias[n])                           (ProjectionShard linear, layers.py:559-563) */
  MTJ_EPI_RESID = 1,  /* x[m, n] += acc + bias[n], float32 in place            (layers.py:313 + transformer_shard.py:92,112) */
  MTJ_EPI_INPROJ = 2  /* fused q|v|k|fc_in: RoPE(q), RoPE(k) -> cache, v -> cache, gelu(fc_in + b1)
                         (layers.py:292-297, 261-273, 287-289, 325-326) */
};

/*
 * Geometry and destinations of the fused input projection.  Row m of the GEMM is token t = m % Tp of
 * sequence b = m / Tp, at absolute position pos = pos0[b] + t; rows with pos < 0 are left padding and
 * write nothing to the cache.  Output columns: [0,d) q, [d,2d) v, [2d,3d) k, [3d,3d+F) fc_in.
 * Precondition: every position is < max_pos.  A larger one is rotated with the LAST table row instead of reading
 * beyond the tables (memory safe, numerically wrong), so the caller sizes the tables for prompt + generated tokens.
 */
typedef struct {
  int32_t n_heads, d_head, rotary_dims; /* H, dh, r (r even, r <= dh)                                   */
  int32_t Tp;                           /* tokens per sequence in this call (1 at decode)              */
  int32_t Tcap;                         /* K/V window capacity in slots; slot = pos % Tcap             */
  int32_t max_pos;                      /* rows of the sin/cos tables                                  */
  const int32_t* pos0;                  /* [B] position of the first row of each sequence              */
  const float* sin_tab;                 /* [max_pos, r/2] float32, rounded once from float64           */
  const float* cos_tab;                 /* [max_pos, r/2]                                              */
  void* q;                              /* [B, H, Tp, dh] in q_dtype                                   */
  int32_t q_dtype;                      /* MTJ_F32 (decode attention reads float32 q) or a 16-bit type */
  int32_t kv_dtype;                     /* storage type of k_cache, v_cache and v_t                    */
  void* k_cache;                        /* [B, H, Tcap, dh] kv_dtype, rotated keys                     */
  void* v_cache;                        /* [B, H, Tcap, dh] kv_dtype                                   */
  void* v_t;                            /* optional [B, H, dh, ldvt] kv_dtype: V transposed, for prefill */
  int64_t ldvt;                         /* row length of v_t: >= Tp rounded up to a multiple of 64     */
  void* act;                            /* [M, ld_act]: gelu(fc_in) goes to columns [d, d+F)           */
  int64_t ld_act;
  int32_t act_dtype;                    /* MTJ_F32 or MTJ_BF16                                         */
} mtj_inproj;

/*
 * Per-range partial results of one-token attention, as mtj_attn_decode_partials leaves them and mtj_gemv consumes them:
 * partials[((b*H + h)*splits + s) * (dh + 4)] = {max, sum, -, -, V[dh]}; the attention output of a (sequence, head) is
 * sum_s exp(max_s - max) V_s / sum_s exp(max_s - max) sum_s.
 */
typedef struct {
  const float* partials;
  int32_t n_heads, d_head, splits;
} mtj_attn_merge;

/*
 * Transpose-pack a haiku [K, N] weight (row stride src_ld) into dst[(n_off + n) * K_total + k_off + k].
 * Replaces nothing in the reference; it is the layout change that lets q|v|k|fc_in (layers.py:249-256)
 * run as one GEMM and out|fc_out (layers.py:253-258) as another.
 */
int mtj_pack_weight(const void* src, int64_t src_ld, int64_t K, int64_t N, void* dst, int64_t K_total,
                    int64_t n_off, int64_t k_off, int dtype, void* stream);

/* mtj_pack_weight with a change of type: dst (dst_dtype) = src (src_dtype) * scale, rounded to nearest even
 * (saturating for MTJ_F16).  With src bf16, dst float16 and `scale` a power of two that brings the largest weight
 * of the matrix below 65504, every weight whose scaled magnitude is at least 2^-14 is represented exactly; smaller
 * ones are rounded to a multiple of 2^-24 (below 2^-40 of the largest weight).  The matching mtj_gemm call passes
 * alpha = 1 / scale. */
int mtj_pack_weight_cvt(const void* src, int64_t src_ld, int64_t K, int64_t N, void* dst, int64_t K_total,
                        int64_t n_off, int64_t k_off, int src_dtype, int dst_dtype, float scale, void* stream);

/* out[m, :] = W[tok[m], :] + b  (EmbeddingShard.__call__, layers.py:187-202: one_hot @ W + b).
 * W is the tree leaf itself, [V, d] in `dtype`; b float32 [d]; out float32 [M, d].
 * Token ids >= n_vocab give a zero row plus bias, as an all-zero one-hot row would. */
int mtj_embed(const int32_t* tok, int64_t M, const void* W, const float* b, int64_t n_vocab, int64_t d,
              int dtype, float* out, void* stream);

/* ReplicatedLayerNorm.__call__, layers.py:17-36 (biased variance, eps 1e-5 inside rsqrt).
 * x float32 [M, d] (row stride d); out [M, d] in out_dtype. */
int mtj_layernorm(const float* x, const float* scale, const float* offset, int64_t M, int64_t d,
                  void* out, int out_dtype, void* stream);

/* Rotary position embedding of projected q / k rows and the K/V window append, without the projection
 * (fixed_pos_embedding + apply_rotary_pos_emb inside self_attn, layers.py:128-148, 261-273; the window update of
 * decode_once, layers.py:325-326).  q, v, k float32 [M, H*dh] (any may be NULL and is then skipped); row m is token
 * m % Tp of sequence m / Tp at position pos0[b] + t, and goes where the fused input projection (MTJ_EPI_INPROJ) puts
 * it: q rotated into ip->q, k rotated into ip->k_cache, v into ip->v_cache (and ip->v_t when given); ip->act is not
 * used.  The module-level self_attn of the Python surface is built on it. */
int mtj_rope_append(const float* q, const float* v, const float* k, int64_t M, const mtj_inproj* ip, void* stream);

/* Per-row cross entropy of float32 logits [M, V] (row stride ld) against int32 targets [M]:
 * ProjectionShard.loss, layers.py:569-593, on one shard: loss = log(sum exp(l - max)) - (l[target] - max),
 * correct = (l[target] == max).  A target outside [0, V) selects nothing (loss = log-sum-exp), like an all-zero
 * one-hot row.  correct may be NULL. */
int mtj_xent(const float* logits, int64_t ld, const int32_t* target, int64_t M, int64_t V, float* loss,
             uint8_t* correct, void* stream);

/* C = alpha * A[M, K] (dtype, row stride lda) x W[N, K]^T (packed, dtype) with epilogue `epi`.
 * hk.Linear call sites: layers.py:249-258, 559.  MFMA kernel; bias is float32 [N] or NULL; alpha undoes the scale
 * of mtj_pack_weight_cvt (1 otherwise) and multiplies the float32 accumulator before anything else is applied.
 * STORE: out [M, ldo] in out_dtype.  RESID: out float32 [M, ldo].  INPROJ: `ip` non-NULL, bias = b1 [F].
 * K must be a multiple of 64 (32 for float32), A, W and the rows of A 16-byte aligned, and 256 rows of A or W must
 * span less than 1 GiB (MTJ_ELIMIT otherwise). */
int mtj_gemm(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
             int dtype, int epi, void* out, int64_t ldo, int out_dtype, const mtj_inproj* ip, float alpha,
             void* stream);

/* mtj_gemm for problems with few output tiles (batched decode; the out projection of a short prompt): when the
 * output has too few tiles to occupy the
 * chip, K is cut into ranges that run as separate workgroups, each storing a float32 partial tile into `work`,
 * and a second kernel adds the partials in a fixed order (results do not depend on scheduling) and applies the
 * epilogue.  STORE and RESID only.  `work` holds mtj_gemm_splitk_work_bytes() bytes (0: no split is used and the
 * call is mtj_gemm); out and bias must then be 16-byte aligned and ldo a multiple of 4.
 * Call sites: the out/fc_out projection of decode_once (layers.py:316-344) at batch > 1. */
int64_t mtj_gemm_splitk_work_bytes(int64_t M, int64_t N, int64_t K, int dtype);
int mtj_gemm_splitk(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                    int dtype, int epi, void* out, int64_t ldo, int out_dtype, void* work, int64_t work_bytes,
                    float alpha, void* stream);

/* mtj_gemm_splitk with the RESID epilogue, followed in the same launch by the LayerNorm of the rows it completes:
 * x [M, ldx] float32 += A x W^T + bias, then h [M, ldh] (h_dtype) = ReplicatedLayerNorm(x) with ln_scale / ln_offset
 * [N] (layers.py:17-36) - the LayerNorm of the next layer, or of the projection, that follows the residual add in
 * generate_once (transformer_shard.py:97-115).  `work` as for mtj_gemm_splitk; N <= 16384. */
int mtj_gemm_splitk_ln(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                       int dtype, float* x, int64_t ldx, void* work, int64_t work_bytes, const float* ln_scale,
                       const float* ln_offset, void* h, int64_t ldh, int h_dtype, float alpha, void* stream);

/* ProjectionShard.loss (layers.py:569-593) without the logits ever reaching memory: the rows of A are the
 * LayerNorm'd activations, logits = alpha * A x W^T + bias are formed tile by tile on the matrix cores and reduced in
 * the epilogue to (maximum, sum of exp(logit - maximum), logit of the target column) per row and column tile; a
 * second, tiny launch merges the tiles: loss[m] = log(sum exp(l - max)) - (l[target] - max), correct[m] =
 * (l[target] == max), exactly what mtj_xent computes from stored logits (a target outside [0, N) selects nothing).
 * `work`: mtj_gemm_xent_work_bytes(M, N, dtype) bytes (2 floats per row and column tile + 1 per row, against
 * 4 * N bytes per row for the logits themselves); correct may be NULL. */
int64_t mtj_gemm_xent_work_bytes(int64_t M, int64_t N, int dtype);
int mtj_gemm_xent(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                  int dtype, float alpha, const int32_t* target, float* loss, uint8_t* correct, void* work,
                  int64_t work_bytes, void* stream);

/* Batch-1 decode matrix-vector product: y = f(x) @ W^T with float32 activations and float32 accumulation
 * (jnp.dot(f32, bf16) semantics of hk.Linear at decode, layers.py:316-344).  x float32 [K].
 * If ln_scale != NULL the kernel first applies LayerNorm(x) (layers.py:17-36) - x then has K = d entries.
 * If am != NULL (no LayerNorm then) the first am->n_heads * am->d_head entries of the input are not read from x but
 * merged from the attention partials of batch row 0 (mtj_attn_decode_partials).
 * Same epilogues as mtj_gemm with M = 1; with MTJ_EPI_INPROJ, n_heads * Tcap * d_head, N and ld_act must be below 2^31. */
int mtj_gemv(const float* x, const float* ln_scale, const float* ln_offset, const void* W, const float* bias,
             int64_t N, int64_t K, int dtype, int epi, void* out, int out_dtype, const mtj_inproj* ip,
             const mtj_attn_merge* am, void* stream);

/* The out projection of a batch-1 decode layer with the one-token attention inside it (layers.py:275-285, 290, 313,
 * 316-344): out[N] += [attention(q, K/V window) | x[H*dh .. K)] @ W^T + bias, float32 in place.  The first workgroups
 * reduce the key ranges of the heads to partials while the weight stream of the launch starts; every workgroup
 * streams the columns of its rows that do not depend on the attention first, then waits (on an arrival counter in
 * `work`) for all partials, merges them and finishes its rows.  Compared with mtj_attn_decode_partials + mtj_gemv it
 * saves a launch and the exposed round trips of the attention.
 * Needs every workgroup resident at once: mtj_gemv_attn_supported() says whether the shape qualifies on the current
 * device (whole 8 KiB tiles on both sides of column H*dh, at most one workgroup per CU); MTJ_ELIMIT otherwise.
 * x float32 [K] (its first H*dh entries are not read); q float32 [H, dh]; caches [H, Tcap, dh] in kv_dtype; pos
 * int32 [1].  `work`: mtj_gemv_attn_work_bytes(H, dh) bytes, 128-byte aligned, zeroed by the caller ONCE before its
 * first use and then left alone (it holds a running arrival counter); launches sharing one `work` must not overlap
 * and must all have the same N.  The wait is bounded by real time (5 ms of the device's 100 MHz counter): a launch
 * whose workgroups are not all resident within that time (CUs masked off or held by other work) gives up and sets
 * word 2 (uint32) of `work`; its result and that of every later launch is then unusable, and later launches no
 * longer wait, until the caller has written 0 to that word (the arrival counter in words 0-1 must be left alone). */
int mtj_gemv_attn_supported(int64_t N, int64_t K, int dtype, int64_t H, int64_t dh, int kv_dtype, int64_t Tcap);
int64_t mtj_gemv_attn_work_bytes(int64_t H, int64_t dh);
int mtj_gemv_attn(const float* x, const void* W, const float* bias, int64_t N, int64_t K, int dtype, float* out,
                  const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t H, int64_t Tcap,
                  int64_t dh, int kv_dtype, void* work, void* stream);

/* Causal self-attention over a left-padded rectangle (self_attn + masks of get_init_decode_state,
 * layers.py:260-285, 347-366).  q [B,H,Tp,dh], k_cache [B,H,Tcap,dh] (rotated), v_t [B,H,dh,ldvt] with
 * ldvt >= Tp rounded up to a multiple of 64 (columns beyond the last key may hold anything);
 * out[m, h*dh + c] with row stride ld_out, dtype.  Scores are divided by sqrt(dh) after the dot;
 * masked keys contribute exactly 0 (exp(-1e10 - max) underflows in float32).  Padding rows get zeros.
 * key_limit (may be NULL): int32 [B]; query position p of sequence b sees keys 0 .. min(p, key_limit[b]) - the
 * additive mask (arange > ctx_length) * -1e10 of the evaluation path, transformer_shard.py:130. */
int mtj_attn_prefill(const void* q, const void* k_cache, const void* v_t, const int32_t* pos0, int64_t B,
                     int64_t H, int64_t Tp, int64_t Tcap, int64_t dh, int64_t ldvt, void* out, int64_t ld_out,
                     int dtype, const int32_t* key_limit, void* stream);

/* One-token attention over the K/V window (decode_once, layers.py:316-344): for sequence b the valid
 * slots are [0, min(pos[b]+1, Tcap)).  q float32 [B,H,dh]; caches in `dtype`; out [B, ld_out] in out_dtype
 * (columns h*dh + c).  The valid slots of a (sequence, head) are cut into mtj_attn_decode_splits(B, H, Tcap) equal key
 * ranges that run as separate workgroups; `work` (16-byte aligned, mtj_attn_decode_work_bytes(B, H, dh, Tcap) bytes)
 * holds their partial results (max, sum, weighted V) until a second launch merges them (no second launch when there
 * is one range); calls sharing one `work` must not overlap. */
int mtj_attn_decode_splits(int64_t B, int64_t H, int64_t Tcap);
int64_t mtj_attn_decode_work_bytes(int64_t B, int64_t H, int64_t dh, int64_t Tcap);
int mtj_attn_decode(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t B,
                    int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out, int out_dtype, int dtype,
                    void* work, void* stream);

/* The partial results of mtj_attn_decode without the merge: mtj_gemv merges them while it stages its input (the
 * attention output is consumed by the out projection only, layers.py:285), which saves a launch and a round trip
 * through memory per layer at batch 1.  *merge is filled for mtj_gemv. */
int mtj_attn_decode_partials(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t B,
                             int64_t H, int64_t Tcap, int64_t dh, int dtype, void* work, mtj_attn_merge* merge,
                             void* stream);

/* mtj_attn_decode for callers that cannot allocate or carry a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The partial results
 * live in a device array built into the library (MTJ_ATTN_DECODE_STATIC_BYTES per device, held until the process
 * ends: room for 4032 (sequence, head) pairs at d_head 256, e.g. batch 252 of a 16-head model); the call allocates nothing and returns MTJ_ELIMIT when mtj_attn_decode_work_bytes(B, H, dh, Tcap) exceeds
 * that.  Same arguments and results as mtj_attn_decode otherwise.  Every call on a device shares the array: calls
 * that overlap on one device (two streams, two threads) race; nothing checks for it.
 * Before the first capture on a device, call mtj_attn_decode_static_max_bytes() (or the entry point itself, eagerly,
 * once per shape) with that device current: the array's address is looked up at the first use on a device and the
 * kernels' attributes are set at their first launch, neither of which belongs inside a stream capture. */
#define MTJ_ATTN_DECODE_STATIC_BYTES (4 * 1024 * 1024)
int64_t mtj_attn_decode_static_max_bytes(void);
int mtj_attn_decode_static(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t B,
                           int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out, int out_dtype, int dtype,
                           void* stream);

/* Next-step embedding fused into the samplers: when `w` is non-NULL the sampler also writes
 * x_next[b, :] = w[token, :] + bias (EmbeddingShard of the token it just chose, layers.py:187-202), which is the
 * input of the next decode step (transformer_shard.py:107). */
typedef struct {
  const void* w;      /* [n_vocab, d] in dtype, or NULL */
  const float* bias;  /* [d] */
  float* x_next;      /* [B, d] */
  int64_t d;
  int32_t dtype;
} mtj_next_embed;

/* Greedy sampler through the reference's sampler contract (transformer_shard.py:203): lowest index among
 * maxima.  Writes tok[b], out_tokens[b * ld_tokens + (pos[b] - pos_start[b])], then pos[b] += 1. */
int mtj_sample_greedy(const float* logits, int64_t B, int64_t V, int32_t* tok, int32_t* out_tokens,
                      int64_t ld_tokens, int32_t* pos, const int32_t* pos_start, const mtj_next_embed* next,
                      void* stream);

/* The logits projection of a batch-1 decode step and the greedy sampler behind it in one launch
 * (transformer_shard.py:107-113 and :203): mtj_gemv with MTJ_EPI_STORE into float32 `logits` [N] followed by
 * mtj_sample_greedy(logits, 1, N, ...), same results bit for bit.  Every workgroup folds the best of its rows into
 * work[0] with a 64-bit atomic maximum and counts its arrival in work[128 bytes]; the workgroup that completes the
 * count does the sampler's part (tok, out_tokens, pos += 1, x_next) and puts both words back to 0 - no workgroup waits
 * for another.  `work`: 256 bytes, 256-byte aligned, zeroed once by the caller; launches that share it must not
 * overlap in time. */
int mtj_gemv_greedy(const float* x, const float* ln_scale, const float* ln_offset, const void* W, const float* bias,
                    int64_t N, int64_t K, int dtype, float* logits, int32_t* tok, int32_t* out_tokens,
                    int64_t ld_tokens, int32_t* pos, const int32_t* pos_start, const mtj_next_embed* next, void* work,
                    void* stream);

/* nucleaus_sample (sampling.py:10-44) with the Gumbel draw replaced by an inverse-CDF draw from
 * host-supplied uniforms: filter on the RAW logits (optional top_k, then top_p, float64 softmax and
 * running sum over the stable descending order, ties: higher id first), then weights
 * exp(filtered/temp - max) in float64 and the first token whose running weight exceeds u * total.
 * top_p, temp: float64 [B]; top_k: int32 [B] or NULL; uniforms: float64 [B, ld_u], column = step index.
 * keep_mask (optional) uint8 [B, V]: 1 where the filter left the logit untouched.
 * filtered (optional) float32 [B, V]: the filter's output.
 * One launch, one workgroup per row; the row is not sorted: the rank at which a running sum crosses its threshold is
 * found by selection, with the float64 weights accumulated exactly as 96-bit integers of 2^-62 (a decision differs
 * from a sequential float64 running sum only if that sum lies within 1.4e-14 of the threshold).  V <= 65536.
 * `work` (256-byte aligned, mtj_sample_work_bytes(B, V) = 256 bytes) is kept in the signature and not used. */
int64_t mtj_sample_work_bytes(int64_t B, int64_t V);
int mtj_sample_nucleus(const float* logits, int64_t B, int64_t V, const double* top_p, const double* temp,
                       const int32_t* top_k, const double* uniforms, int64_t ld_u, int32_t* tok,
                       int32_t* out_tokens, int64_t ld_tokens, int32_t* pos, const int32_t* pos_start,
                       uint8_t* keep_mask, float* filtered, void* work, const mtj_next_embed* next, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MTJ_ABI_H */
