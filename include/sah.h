/*
 * sah.h — C ABI of libsah_mi355.so: the MI355X (gfx950) kernels behind the
 * ResearchAttention decode path of sparse-attention-hub.
 *
 * The reference implementation is pure Python on torch and has no FFI of its
 * own; every entry point below therefore cites the reference *Python* function
 * whose body it replaces (paths relative to the reference checkout,
 * sparse_attention_hub/sparse_attention/...).
 *
 * Conventions
 *   - every pointer is a device pointer unless its comment says "host";
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*),
 *     never synchronises, never allocates, never frees;
 *   - return value 0 = success, negative = SAH_E* argument error (nothing was
 *     launched), positive = hipError_t from the launch;
 *   - sah_last_error() returns a thread-local description of the last failure;
 *   - calls may come from several threads; the library's only state of its own is a per-device record of the
 *     kernels whose dynamic-LDS limit has been raised and the optional timing registry of sah_timing_enable
 *     (both behind a mutex) and the fixed workspace of sah_sparse_attention_static (see there);
 *   - tensors are addressed by element strides, the innermost (head_dim)
 *     stride must be 1.
 *
 * Native sparse-mask layout ("rows"): the reference Mask
 * (utils/mask.py:10) is a dense (B,Hq,Lq,Lk) weight tensor or a flat int64
 * indices/ptr/data triple. The kernels use one row per (b, h, q):
 *     cols  [n_rows, cap]   int32  key columns of the active entries (unordered)
 *     cnt   [n_rows]        int32  number of valid entries of the row
 *     w     [n_rows, cap]   float  weight of each entry, or NULL (all 1.0)
 *     bitmap[n_rows, n_words] uint32  bit j of the row set <=> column j active
 * n_words = ceil(n_keys / 32). The Python Mask facade converts this to the
 * reference's flat int64 indices / ptr / data or to a dense tensor on demand.
 */
#ifndef SAH_H
#define SAH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout generation of this header. It changes whenever an argument struct gains, loses or reorders a field or an
 * entry point changes its signature, and never otherwise: a caller compares sah_version() with the SAH_VERSION it was
 * compiled (or, for a ctypes binding, written) against before its first call and refuses a library that differs,
 * because a struct of another generation would be read past its end. */
#define SAH_VERSION 4

enum {
  SAH_OK = 0,
  SAH_EINVAL = -1,      /* bad argument value / combination            */
  SAH_ENULL = -2,       /* required pointer is NULL                    */
  SAH_ESHAPE = -3,      /* shape the kernels do not support            */
  SAH_ECAPACITY = -4,   /* rows.cap or a workspace is too small        */
  SAH_EDTYPE = -5       /* unsupported dtype code                      */
};

/* element type codes */
enum { SAH_F32 = 0, SAH_BF16 = 1, SAH_F16 = 2 };

/* activation codes of the signature MLP (hashattention_top_k.py:210-215) */
enum { SAH_ACT_RELU = 0, SAH_ACT_SILU = 1, SAH_ACT_GELU = 2, SAH_ACT_TANH = 3 };

typedef struct sah_rows {
  int32_t* cols;
  int32_t* cnt;
  float* w;          /* may be NULL */
  uint32_t* bitmap;
  int32_t n_rows;    /* B * Hq * Lq */
  int32_t cap;       /* row pitch of cols / w */
  int32_t n_keys;    /* Lk */
  int32_t n_words;   /* row pitch of bitmap = ceil(Lk/32) */
} sah_rows;

int sah_version(void);
const char* sah_last_error(void);

/* Opt-in per-kernel timing for benchmarks; no counterpart in the reference (its
 * profile/profile_research_attention.py:273-319 times whole calls from Python).
 * While enabled every entry point brackets its kernel with a HIP event pair on
 * the caller's stream. sah_timing_collect waits for the recorded events, sums
 * the elapsed milliseconds per kernel name into names/counts/total_ms (host
 * arrays of `max` entries), clears the log and returns the number of names. */
int sah_timing_enable(int on);
int sah_timing_collect(const char** names, int* counts, float* total_ms, int max);

/* ---------------------------------------------------------------------------
 * Fused Sink + Local builder. Replaces SinkMasker.get_updated_mask_dense
 * (maskers/fixed/implementations/basic_fixed.py:354-363) and
 * LocalMasker.update_core (basic_fixed.py:48-67): columns [0, sink) and, for
 * query row q of Lq, columns [Lk-Lq-window+1+q, Lk-Lq+q]. Either part may be
 * switched off with 0. With fresh != 0 the rows are taken to be empty and are
 * initialised (cnt, bitmap and cols all written); otherwise the ranges are
 * merged into the existing rows (already-active columns keep their entry, and
 * a weighted entry that falls inside a range has its weight raised to 1.0 as
 * the reference's dense assignment `mask[...] = 1.0` does).
 * With clear_future != 0 every entry with column > Lk-Lq+q is removed first
 * (basic_fixed.py:60-66); a no-op when Lq == 1.
 * ------------------------------------------------------------------------- */
typedef struct sah_sink_local_args {
  sah_rows rows;
  int32_t lq;            /* query rows per (b,h): row r has q = r % lq */
  int32_t sink;          /* sink size, 0 = skip                         */
  int32_t window;        /* local window, 0 = skip                      */
  int32_t fresh;
  int32_t clear_future;
  void* stream;
} sah_sink_local_args;
int sah_sink_local_indices(const sah_sink_local_args* a);

/* ---------------------------------------------------------------------------
 * Dense <-> rows conversion. Replaces Mask.get_index_mask's dense scan
 * (utils/mask.py:553-573) and Mask.get_dense_mask's scatter (:595-609).
 * dense is [n_rows, n_keys] contiguous in `dtype`; an entry is active iff its
 * weight != 0. rows.w may be NULL for from_dense (weights dropped: caller
 * asserts they are all 1.0) and for to_dense (ones are written).
 * from_dense writes columns in ascending order and returns SAH_ECAPACITY
 * nowhere: rows whose population exceeds cap are truncated and their cnt is
 * still the true population, so the caller can detect it (cnt > cap).
 * ------------------------------------------------------------------------- */
typedef struct sah_dense_rows_args {
  sah_rows rows;
  void* dense;
  int32_t dtype;
  void* stream;
} sah_dense_rows_args;
int sah_rows_from_dense(const sah_dense_rows_args* a);
int sah_rows_to_dense(const sah_dense_rows_args* a);

/* ---------------------------------------------------------------------------
 * Hash signatures. Replaces HashAttentionTopKMasker._get_signatures /
 * _apply_single_layer (hashattention_top_k.py:203-253): per query head h,
 * x <- act(x W_i + b_i) for all but the last layer, x <- x W_L + b_L, then
 * sign(x) in {-1, 0, +1}. A signature is stored as a pair of uint32 planes
 * ("code", 8 bytes): bit e of word 0 = (x_e > 0), bit e of word 1 = (x_e != 0),
 * LSB first; at most 32 signature bits. (Exact zeros are common in bf16, and
 * the reference scores such a bit as 0.)
 * x is [B, Hx, L, D] with element strides; head h reads x head h / group
 * (group = Hq / Hx; keys pass Hx = Hkv, queries pass Hx = Hq, group = 1).
 * Layer i has W_i [Hq, d_in_i, d_out_i] and b_i [Hq, d_out_i], contiguous, in
 * `dtype`. With dtype = SAH_BF16 / SAH_F16 every layer output, bias add and
 * activation is rounded to that type exactly where torch would round it.
 * codes[((b*Hq + h) * code_pitch + code_offset + l) * 2 + {0,1}] receives
 * vector l (code_pitch and code_offset count codes, not words).
 * Wt (all layers or none): the same matrices transposed, which lets many vectors
 * at once (a prefill, the first decode call) go through the matrix cores when the
 * type is 16-bit, D and the hidden widths are multiples of 32 up to 128.
 * ------------------------------------------------------------------------- */
#define SAH_MAX_MLP_LAYERS 4
typedef struct sah_hash_sig_args {
  const void* x;
  int64_t xs_b, xs_h, xs_l;
  int32_t dtype;
  int32_t B, Hq, group, L, D;
  int32_t n_layers;
  const void* W[SAH_MAX_MLP_LAYERS];
  const void* bias[SAH_MAX_MLP_LAYERS];
  const void* Wt[SAH_MAX_MLP_LAYERS];  /* optional: W_i transposed, [Hq, d_out_i, d_in_i] */
  int32_t d_out[SAH_MAX_MLP_LAYERS];  /* d_in of layer 0 is D */
  int32_t act;
  uint32_t* codes;
  int64_t code_pitch;
  int64_t code_offset;
  void* stream;
} sah_hash_sig_args;
int sah_hash_signatures(const sah_hash_sig_args* a);
/* Two independent jobs (a decode step hashes its new keys and its queries) in one
 * launch when both are small; same results as two sah_hash_signatures calls. */
int sah_hash_signatures_pair(const sah_hash_sig_args* a, const sah_hash_sig_args* b);

/* ---------------------------------------------------------------------------
 * Signature top-k. Replaces the score half of
 * HashAttentionTopKMasker._compute_hashattention_score
 * (hashattention_top_k.py:365-370: scores = q_sig @ k_sig^T, already-active
 * columns pushed to the bottom),
 * TopKMasker._get_topk_indices_from_inactive_positions (fixed/base.py:74-85)
 * and the dense scatter + clamp-add merge that follows
 * (maskers/base.py:128-150, utils/mask.py:875-877).
 * With nz = q.nonzero & k.nonzero the score is
 *     popcount(nz) - 2 * popcount((q.positive ^ k.positive) & nz)
 * (= bits - 2 * Hamming distance when no signature entry is zero).
 * For row r = (b,h,q): rank columns j < n_keys by descending score of
 * qcodes[r] against kcodes[(b*Hq+h)*code_pitch + j], ties by lowest j,
 * columns whose bitmap bit is set ranking below every other column; the first
 * k of that order which are not yet active are appended to the row (ascending
 * j) with weight 1.0 and their bits are set.
 * ------------------------------------------------------------------------- */
typedef struct sah_hamming_topk_args {
  sah_rows rows;
  const uint32_t* kcodes;   /* 2 words per code */
  int64_t code_pitch;       /* in codes */
  const uint32_t* qcodes;   /* [n_rows] codes */
  int32_t lq;               /* row r uses key-code stream r / lq */
  int32_t k;
  void* stream;
} sah_hamming_topk_args;
int sah_hamming_topk(const sah_hamming_topk_args* a);

/* Signature scores with an additive attention mask
 * (hashattention_top_k.py:365-369): key of round_to_dtype(float(score) +
 * amask[b, h|0, q, j]) in the sortable-key form of sah_qk_scores, written at
 * keys_out[r * key_pitch + j]; feed sah_select_topk with the key of -inf as
 * excluded_key (fixed/base.py:80). amask may be NULL. */
typedef struct sah_hamming_scores_args {
  const uint32_t* kcodes;
  int64_t code_pitch;
  const uint32_t* qcodes;
  int32_t B, Hq, Lq, n_keys;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int32_t dtype;
  void* keys_out;
  int64_t key_pitch;
  void* stream;
} sah_hamming_scores_args;
int sah_hamming_scores(const sah_hamming_scores_args* a);

/* ---------------------------------------------------------------------------
 * Exact QK scores as sortable keys. Replaces OracleTopK.update_core's
 * `matmul(queries, keys^T)` (+ attention_mask) (oracle_top_k.py:70-72) without
 * repeat_kv: score = round_to_dtype(q[b,h,q,:] . K[b,h/group,j,:]), un-scaled,
 * then (+ amask, rounded again). Scores are written as order-preserving
 * unsigned keys (larger score => larger key; -0 == +0): uint16 for bf16/f16,
 * uint32 for f32, at keys_out[r * key_pitch + j].
 * amask is NULL or an additive mask [B, 1|Hq, Lq, >=Lk] in `dtype` with
 * element strides (stride 0 for a broadcast head).
 * ------------------------------------------------------------------------- */
typedef struct sah_qk_scores_args {
  const void* q;  int64_t qs_b, qs_h, qs_l;
  const void* k;  int64_t ks_b, ks_h, ks_l;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int32_t dtype;
  int32_t B, Hq, Hkv, Lq, Lk, D;
  void* keys_out;
  int64_t key_pitch;
  void* stream;
  /* Optional, 16-bit dtypes without amask only: [B*Hq*Lq][key_pitch] 16-bit words, what rounding the fp32 dot product
   * to `dtype` took away (fp32 dot - rounded score, itself rounded to `dtype`). The key orders the scores exactly as
   * torch's matmul output orders them; key and remainder together give the dot product to about 16 mantissa bits,
   * which lets the attention that follows skip K (sah_attention_args.score_keys / score_resid). NULL: not written. */
  void* resid_out;
} sah_qk_scores_args;
int sah_qk_scores(const sah_qk_scores_args* a);

/* ---------------------------------------------------------------------------
 * Generic top-k over sortable keys. Replaces `scores[prev != 0] = min;
 * torch.topk; scatter_(1.0)` (oracle_top_k.py:73-79, pq_top_k.py:513-537,
 * fixed/base.py:74-85) with the canonical tie rule "lowest column first".
 * Row r ranks candidates c in [0, n_cand) (column j = c + col_offset) by
 * descending key; active columns take `excluded_key` as their key. The first k
 * in that order that are not active are appended (ascending j), weight 1.0.
 * key_bits is 16 or 32. lds/work: none beyond static LDS.
 * ------------------------------------------------------------------------- */
typedef struct sah_select_topk_args {
  sah_rows rows;
  const void* keys;
  int64_t key_pitch;
  int32_t key_bits;
  int32_t n_cand;
  int32_t col_offset;
  int32_t k;
  uint32_t excluded_key;
  int32_t fresh;          /* != 0: the rows are taken to be empty and are first given the sink and local   */
  int32_t fresh_sink;     /* columns of one query per row - what sah_sink_local_indices(lq = 1, fresh = 1) */
  int32_t fresh_window;   /* writes - in the same launch when the keys are 16-bit and 16-byte aligned      */
  void* stream;
  int32_t skip_bitmap;    /* != 0: rows.bitmap need not be brought up to date (a caller that hands the rows */
                          /* to the attention only, which reads the column lists); honoured where it saves  */
                          /* work: by sah_select_topk_attention's one-kernel form                           */
} sah_select_topk_args;
int sah_select_topk(const sah_select_topk_args* a);

/* ---------------------------------------------------------------------------
 * Product quantisation (PQCache). A "group" is g = (b*Hkv + hk)*n_sub + s: one
 * sub-space s of one KV head; its vectors are K[b, hk, key_offset + n,
 * s*d_sub : (s+1)*d_sub] for n in [0, n_keys), read in `dtype`, used as fp32.
 * d_sub <= 16, n_cent <= 256 (codes are uint8).
 *
 * sah_pq_kmeans_assign: replaces pairwise_distance_batched + argmin
 * (maskers/fixed/implementations/utils/pq_utils.py:220-257, :353):
 * code = argmin_c sum_d (x[d] - centre[g,c,d])^2 in fp32, first minimum wins.
 * centres fp32 [n_groups, n_cent, d_sub]; codes uint8 laid out
 * [B, Hkv, code_pitch, n_sub], key n written at index code_offset + n.
 * With sums/counts non-NULL it also accumulates the per-centre fp32 sums
 * [n_groups, n_cent, d_sub] and int32 counts [n_groups, n_cent] of this
 * assignment (the one-hot sums of pq_utils.py:360-381; caller zeroes them).
 * With round_dist != 0 the distance follows PQCache._quantize_new_keys
 * (pq_top_k.py:388-404) instead, which works in the key dtype: each difference
 * and each square is rounded to `dtype`, the sum is accumulated in fp32 and
 * rounded to `dtype` (centres must already hold `dtype`-representable values).
 * skip_flag (optional): if *skip_flag != 0 the kernel does nothing; this is
 * how the Lloyd loop stops early without a host round trip.
 *
 * sah_pq_kmeans_update: replaces the centre update, empty-cluster reseed and
 * convergence test (pq_utils.py:372-432): centre = sum / max(count, 1); an
 * empty cluster takes vector reseed_idx[g*n_cent + c] of its group (the
 * reference draws these with torch.randint); shift2[g] = (sum_c ||new-old||)^2.
 * state is int32[4], zeroed by the caller before the first iteration:
 * when every group has shift2 < tol the kernel sets state[2] = 1 (the
 * skip_flag of later launches). centres are updated in place.
 *
 * sah_pq_adc_scores: replaces PQCache._compute_pq_scores
 * (pq_top_k.py:406-490): LUT[s][c] = round_to_dtype(q_sub . centre[g,c,:d_sub])
 * and score(n) = round_to_dtype(sum_s LUT[s][code[n,s]]) with fp32
 * accumulation; emitted as sortable keys like sah_qk_scores for candidates
 * n in [0, n_cand) at keys_out[r * key_pitch + n]. centres are the fp32
 * widening of the stored (`dtype`-rounded) centroids, [n_groups, n_cent, d_sub].
 * The table is read from LDS by the scoring kernel. Up to 65536 candidates every
 * workgroup computes its slab itself (one launch, `lut` is not touched); beyond that it
 * is built once per call in `lut` (caller's scratch of sah_pq_adc_lut_bytes(...) bytes).
 * ------------------------------------------------------------------------- */
/* Largest |element| of the keys [key_offset, key_offset + n_keys) of every (b, kv head), written as the bit
 * pattern of a float into *absmax_bits, which must be zero before the call. The Lloyd kernels below take their
 * per-centre sums in 64-bit fixed point, scaled by a power of two derived from this value: integer sums do not
 * depend on the order of the additions, so clustering the same keys twice gives the same centroids bit for bit
 * (the reference's one-hot sums, pq_utils.py:360-372, are reproducible too). */
typedef struct sah_pq_absmax_args {
  const void* k; int64_t ks_b, ks_h, ks_l;
  int32_t dtype;
  int32_t B, Hkv, D;
  int32_t key_offset, n_keys;
  uint32_t* absmax_bits;
  void* stream;
} sah_pq_absmax_args;
int sah_pq_keys_absmax(const sah_pq_absmax_args* a);

typedef struct sah_pq_assign_args {
  const void* k; int64_t ks_b, ks_h, ks_l;
  int32_t dtype;
  int32_t B, Hkv, n_sub, d_sub, n_cent;
  int32_t key_offset, n_keys;
  const float* centres;
  uint8_t* codes; int64_t code_pitch; int64_t code_offset;
  int64_t* sums; int32_t* counts;     /* [n_groups, n_cent, d_sub] fixed-point sums, [n_groups, n_cent]; both NULL: codes only */
  int32_t round_dist;
  const int32_t* skip_flag;
  void* stream;
  const uint32_t* absmax_bits;        /* from sah_pq_keys_absmax; needed when sums is not NULL */
} sah_pq_assign_args;
int sah_pq_kmeans_assign(const sah_pq_assign_args* a);

typedef struct sah_pq_update_args {
  const void* k; int64_t ks_b, ks_h, ks_l;
  int32_t dtype;
  int32_t B, Hkv, n_sub, d_sub, n_cent;
  int32_t key_offset;
  float* centres;
  const int64_t* sums; const int32_t* counts;
  const int32_t* reseed_idx;
  float* shift2;       /* [n_groups] */
  float tol;
  int32_t* state;      /* int32[4]: converged count, ticket, done flag, pending verdict */
  void* stream;
  const uint32_t* absmax_bits;        /* the value the assignment used */
} sah_pq_update_args;
int sah_pq_kmeans_update(const sah_pq_update_args* a);

typedef struct sah_pq_adc_args {
  const void* q; int64_t qs_b, qs_h, qs_l;
  int32_t dtype;
  int32_t B, Hq, Hkv, Lq, n_sub, d_sub, n_cent;
  const float* centres;
  const uint8_t* codes; int64_t code_pitch;
  int32_t n_cand;
  void* keys_out; int64_t key_pitch;
  void* lut; int64_t lut_bytes;   /* scratch: sah_pq_adc_lut_bytes(...) bytes */
  void* stream;
  const void* centres_narrow;     /* optional: the same centres [n_groups, n_cent, d_sub] in `dtype` (the form the
                                     reference stores, pq_top_k.py:246-254; `centres` is their widening). When given
                                     with a 16-bit dtype and d_sub a multiple of 8, the table is built from these:
                                     half the bytes, identical values */
} sah_pq_adc_args;
int64_t sah_pq_adc_lut_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lq, int32_t n_sub, int32_t n_cent, int32_t dtype);
int sah_pq_adc_scores(const sah_pq_adc_args* a);

/* ---------------------------------------------------------------------------
 * Masked-softmax attention over the gathered rows. Replaces
 * get_masked_attention_output (utils/mask_attention_utils.py:406-491):
 * z[j] = q.K[j] * scaling (+amask) in fp32, e[j] = exp(z[j] - m) / (w[j]+1e-6)
 * (unit_inv_w when rows.w is NULL), out = sum e V / (sum e [+ sink term,
 * apply_sink_bias :357-402]), written as out[b, q, h, :] in `dtype`
 * (contiguous (B, Lq, Hq, D)). With dense != 0 the rows are ignored and every
 * column j < Lk is used with weight 1 (the reference's treatment of an empty
 * or full Mask, utils/mask.py:733-735).
 * work: fp32 scratch of sah_sparse_attention_work_floats(...) floats (0 when whole
 * rows are handled by one workgroup each; work may then be NULL).
 * logits_out (optional, fp32 [n_rows, cap]) receives z[j] per entry and
 * stats_out (optional, fp32 [n_rows, 2]) the final (m, den) so that the dense
 * attention-weight tensor can be produced by sah_attention_weights.
 * ------------------------------------------------------------------------- */
typedef struct sah_attention_args {
  sah_rows rows;
  const void* q;  int64_t qs_b, qs_h, qs_l;
  const void* k;  int64_t ks_b, ks_h, ks_l;
  const void* v;  int64_t vs_b, vs_h, vs_l;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  const float* sinks;     /* [Hq] fp32 or NULL */
  int32_t dtype;
  int32_t B, Hq, Hkv, Lq, Lk, D;
  float scaling;
  float unit_inv_w;
  int32_t dense;
  int32_t closed_form;    /* != 0 (with dense = 0, Lq = 1, no additive mask): the rows' pointers are not read; */
  int32_t closed_sink;    /* every row's entries are the sink and local columns of its one query, weight 1.0,  */
  int32_t closed_window;  /* i.e. what sah_sink_local_indices(lq = 1, fresh = 1) would have written             */
  int32_t max_cnt;        /* upper bound of cnt[r] the grid is sized for */
  void* out;
  float* work; int64_t work_floats;
  float* logits_out;
  float* stats_out;
  void* stream;
  /* Training-mode dropout of the exp weights (torch.nn.functional.dropout in _compute_masked_exp_attention_weights,
   * utils/mask_attention_utils.py:234-238): with 0 < dropout_p < 1 the entry (mask row r, column j) is dropped
   * when word 0 of Philox4x32-10(counter (j, r, offset lo, offset hi), key (seed lo, seed hi)) is below
   * dropout_p * 2^32, and kept entries are scaled by 1 / (1 - dropout_p), in the numerator and in the denominator
   * (the sink term, where there is one, is not scaled). The reference draws from torch's generator: the stream
   * differs, the distribution does not. 0: no dropout. */
  float dropout_p;
  uint64_t dropout_seed;
  uint64_t dropout_offset;
  int32_t dropout_numerator_only; /* != 0: dropped entries leave the denominator as it is, i.e. dropout of the
                                     normalised probabilities, what the reference's dense path does
                                     (scaled_dot_product_attention with dropout_p, mask_attention_utils.py:40-52) */
  /* Optional: q.k of EVERY column of every mask row, [n_rows][score_pitch] each: the 16-bit score keys and the
   * remainders sah_qk_scores wrote for these q and k (keys_out / resid_out, no additive mask) - a chain whose selection
   * scored all keys exactly (OracleTopK, oracle_top_k.py:49-60) has them already. The kernels may then take a logit
   * from there ((score + remainder) * scaling: the fp32 dot product to about 16 mantissa bits) instead of reading the
   * K row again: half of the gather's bytes. amask, where given, is added as ever. Used when both are given, for
   * 16-bit tensors, head_dim 64 / 128 and no dropout; otherwise K is read. NULL: none. */
  const void* score_keys;
  const void* score_resid;
  int64_t score_pitch;
} sah_attention_args;
int64_t sah_sparse_attention_work_floats(int32_t n_rows, int32_t max_cnt, int32_t D);
int sah_sparse_attention(const sah_attention_args* a);

/* sah_sparse_attention for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same arguments
 * and results, except that a->work / a->work_floats are ignored: the partial results of the split form go
 * to a buffer of SAH_ATTENTION_STATIC_WORK_FLOATS floats (16 MiB) inside the library's device image, which
 * every GPU the library runs on holds until the process ends. A call that needs more (see
 * sah_sparse_attention_work_floats) returns SAH_ECAPACITY and launches nothing. The call allocates nothing
 * and records no kernel timing. All calls on one GPU share the buffer: calls that overlap on one GPU
 * (different streams, different threads) race; calls on one stream are ordered and safe. Nothing in the
 * buffer needs to start at zero: every launch writes each partial result before its merge kernel reads it. */
#define SAH_ATTENTION_STATIC_WORK_FLOATS (4 * 1024 * 1024)
int sah_sparse_attention_static(const sah_attention_args* a);

/* Dense attention probabilities (the second return value of
 * get_masked_attention_output, utils/mask_attention_utils.py:482-489):
 * weights[r, j] = round_to_dtype(exp(z - m) * inv_w / den) at the row's
 * entries; the caller zero-fills weights [n_rows, Lk] first. */
typedef struct sah_attention_weights_args {
  sah_rows rows;
  const float* logits;   /* [n_rows, cap] */
  const float* stats;    /* [n_rows, 2]   */
  float unit_inv_w;
  int32_t dense;         /* rows ignored: entry i is column i, pitch n_keys */
  int32_t dtype;
  void* weights;
  void* stream;
  float dropout_p;          /* the same three values the sah_sparse_attention call was given */
  uint64_t dropout_seed;
  uint64_t dropout_offset;
} sah_attention_weights_args;
int sah_attention_weights(const sah_attention_weights_args* a);

/* ---------------------------------------------------------------------------
 * Adaptive sampling (vAttention). Replaces the tensor work of
 * AdaptiveSamplingMasker.add_mask
 * (maskers/sampling/implementations/adaptive_sampling.py:183-302, 365-407) and
 * create_sampling_mask_with_per_head_budget (utils/mask_attention_utils.py:105-184).
 *
 * Both calls read the row's order-preserving score keys as written by
 * sah_qk_scores WITHOUT an additive mask (key of round_to_dtype(q.k), 16-bit for
 * bf16/f16, 32-bit for fp32); the numerators are recomputed from them as the
 * reference's torch ops round them in `dtype`:
 *     z[j] = round(round(s[j] * scaling) + amask[j]),  e[j] = round(exp(round(z[j] - max_j z[j]))).
 *
 * Random draws: Philox4x32-10 with key (seed lo, seed hi) and counter
 * (i / 4, row, offset lo, offset hi); draw i of a row is output word i % 4 and
 * maps to the column start + ((u * range) >> 32): uniform on [start, start+range),
 * with replacement, like torch.randint in the reference.
 *
 * sah_adaptive_budget, per row r:
 *   static_den = round(sum over the row's entries of round(e[col] * inv(w)))   (:370)
 *                with inv(w) = round(1 / round(w + 1e-6)); prev_empty != 0: plain
 *                sum of e over all keys (utils/mask_attention_utils.py:97-99);
 *   n_base draws; sigma = max(round(unbiased std of e over the draws), 1e-8)     (:251-264)
 *   sampled_den = round(sum over DISTINCT drawn columns of
 *                 round(e * inv(round(n_base / range))))                         (:266-278, :389)
 *   budget = clamp(trunc(clamp(round(round(round(ppf*sigma)*range /
 *            max(round(eps*(static_den+sampled_den)), 1e-8))^2), 1, range)), n_base, range)
 *                                                                           (:282-302, :394)
 *   prob   = round(budget / range)                                               (:397)
 * budget[r] int32, prob[r] float. stats (optional, [n_rows,4]) receives
 * static_den, sigma, the denominator estimate and max z for inspection.
 *
 * sah_adaptive_sample, per row r: budget[r] draws (use another `offset` than
 * the budget call); the distinct drawn columns are merged into the row as the
 * reference's dense merge does (utils/mask.py:875-877): a column already in the
 * row gets min(1, round(w + prob)), a new one is appended (ascending column
 * order) with weight prob; bitmap and cnt are updated. rows.w is required;
 * w_fresh != 0 says it holds garbage and every existing entry weighs 1.0.
 * Capacity: the row may grow by up to `range` entries; entries beyond rows.cap
 * are dropped, so size cap >= min(n_keys, cnt + range).
 * The sampling range is limited to what one workgroup's LDS bitmap holds
 * (1,179,648 columns).
 * ------------------------------------------------------------------------- */
typedef struct sah_adaptive_budget_args {
  sah_rows rows;
  const void* keys;       /* [n_rows, key_pitch] uint16 (bf16/f16) or uint32 (fp32) */
  int64_t key_pitch;
  const void* amask;      /* additive mask in `dtype`, or NULL */
  int64_t ms_b, ms_h, ms_l;
  int32_t dtype;
  int32_t Hq, Lq;         /* row r = (b * Hq + h) * Lq + q, for the amask strides */
  float scaling;
  int32_t start, range, n_base;
  float eps, delta_ppf;   /* delta_ppf = Phi^-1(1 - delta) */
  uint64_t seed, offset;
  int32_t prev_empty;
  int32_t* budget;        /* [n_rows] out */
  float* prob;            /* [n_rows] out */
  float* stats;           /* [n_rows, 4] out, or NULL */
  void* stream;
  int32_t max_in_rows;    /* != 0: the caller's promise that every row's largest key belongs to a column that  */
                          /* is already in the row (an exact top-k over these very keys has just run, with    */
                          /* k >= 1): the row maximum of adaptive_sampling.py:195-196 is then taken from the   */
                          /* row's entries instead of a pass over all n_keys keys. Ignored with an additive    */
                          /* mask, with prev_empty, and with scaling <= 0                                      */
} sah_adaptive_budget_args;
int sah_adaptive_budget(const sah_adaptive_budget_args* a);

typedef struct sah_adaptive_sample_args {
  sah_rows rows;
  const int32_t* budget;  /* [n_rows] */
  const float* prob;      /* [n_rows] */
  int32_t dtype;          /* mask dtype: rounding of w + prob */
  int32_t start, range;
  uint64_t seed, offset;
  int32_t w_fresh;
  void* stream;
} sah_adaptive_sample_args;
int sah_adaptive_sample(const sah_adaptive_sample_args* a);

/* ---------------------------------------------------------------------------
 * One decode step of a Sink + Local + HashAttentionTopK chain on rows that are
 * still empty, one query per row (Lq = 1, n_rows = B * Hq): the work of
 * sah_sink_local_indices (fresh = 1), sah_hash_signatures_pair(key_sig, query_sig)
 * and sah_hamming_topk, in this order, with the same results. Replaces, for a
 * decode call, SinkMasker / LocalMasker.add_mask (basic_fixed.py:354-363, :48-67),
 * HashAttentionTopKMasker._update_key_signatures and the query half of
 * _get_signatures (hashattention_top_k.py:203-305) and the score + top-k + merge
 * of :365-370 / fixed/base.py:74-85.
 * rows.cnt / rows.bitmap need no initialisation. query_sig: L = 1, codes =
 * [n_rows] query codes (written). key_sig: NULL or L = 0 when no key is new,
 * else the job that appends the newest key's code to the cache. kcodes /
 * code_pitch: the key-code stream of row r starts at kcodes + r * code_pitch
 * codes. When shapes allow (16-byte aligned code streams, layer widths powers of
 * two with d_in * d_out a multiple of 4096, the new key inside the local window)
 * everything runs in one kernel, otherwise as the three launches above.
 * A caller that consumes only the column lists (the attention kernel does) may
 * set skip_bitmap and save the write-back of the bitmap rows.
 * ------------------------------------------------------------------------- */
typedef struct sah_hash_decode_args {
  sah_rows rows;
  int32_t sink, window;
  const sah_hash_sig_args* query_sig;   /* host pointer */
  const sah_hash_sig_args* key_sig;     /* host pointer or NULL */
  const uint32_t* kcodes;
  int64_t code_pitch;
  int32_t k;
  int32_t skip_bitmap;                  /* != 0: rows.bitmap may be left stale (cols and cnt are complete) */
  /* Optional compact form of the same codes, kept up to date with sah_hash_compact_codes (all NULL / 0:
   * not offered). The single kernel then reads 4 bytes per column instead of 8: the sign plane, scored as
   * if no signature component were zero, and corrects the listed columns for which that is wrong. Same
   * results. Used only when no key is hashed inside this call (key_sig NULL or L = 0). */
  const uint32_t* pos_codes;            /* row r: pos_codes + r * pos_pitch; pos_pitch % 4 == 0, 16-byte aligned,
                                           readable up to ceil(n_keys / 256) * 256 + 6144 columns */
  int64_t pos_pitch;
  const uint32_t* exc;                  /* row r: exc + 4 * r * exc_cap; 16-byte entries, exc_cap >= 1024 */
  const int32_t* exc_cnt;               /* [n_rows] */
  int32_t exc_cap;
  uint32_t full_plane;                  /* non-zero plane of a key without zero components: (1 << bits) - 1 */
  void* stream;
} sah_hash_decode_args;
int sah_hash_decode_topk(const sah_hash_decode_args* a);

/* ---------------------------------------------------------------------------
 * Maintains the compact form of a key-code stream (no counterpart in the reference, whose
 * signatures are float tensors: hashattention_top_k.py:255-305 keeps (B, H, n, bits) values
 * in {-1, 0, +1}). For the columns [from, to) of every row: pos_codes gets the sign plane of
 * the two-plane code, and every column whose non-zero plane differs from full_plane is
 * appended to the row's exception list as the 16-byte entry (column, non-zero plane, sign
 * plane, 0); exc_cnt[r] counts them, also beyond exc_cap (the list has then overflowed and
 * readers fall back to the two-plane codes). exc_cnt must be zero before the first call;
 * call once per column range, in any order.
 * ------------------------------------------------------------------------- */
typedef struct sah_hash_compact_args {
  const uint32_t* codes;   /* two-plane codes, row r: codes + 2 * r * code_pitch */
  int64_t code_pitch;
  int32_t n_rows;
  int32_t from, to;
  uint32_t* pos_codes;
  int64_t pos_pitch;
  uint32_t* exc;
  int32_t exc_cap;
  int32_t* exc_cnt;
  uint32_t full_plane;
  void* stream;
} sah_hash_compact_args;
int sah_hash_compact_codes(const sah_hash_compact_args* a);

/* sah_hash_decode_topk(a) followed by sah_sparse_attention(t) on the same rows, with the same
 * results. When the single-kernel form of the former applies and the attention is the plain
 * decode case (one workgroup per row, Lq = 1, no additive mask, unit weights, no logits
 * output, head_dim 64 or 128, same stream and dtype) both run in ONE kernel: the workgroup
 * that selected a row goes straight on to gather that row's K / V, from a column list kept in
 * LDS (rows.cols / rows.cnt are still written). With fewer rows than compute units a row is given several
 * workgroups, as in sah_select_topk_attention (same `tickets`, same use of t->work; NULL tickets: one workgroup per
 * row or the separate calls). Otherwise the two calls are made. */
int sah_hash_decode_attention(const sah_hash_decode_args* a, const sah_attention_args* t, uint32_t* tickets);

/* ---------------------------------------------------------------------------
 * sah_select_topk followed by sah_sparse_attention over the same rows, with the same results up to the order of
 * the attention's sums. Replaces the tail of a chain with a scoring pass of its own - `topk; scatter_` and
 * get_masked_attention_output (oracle_top_k.py:73-79, pq_top_k.py:513-537, utils/mask_attention_utils.py:406-491).
 * When the selection is the 16-bit form with at most 65536 candidates and the attention is the plain decode case
 * (no additive mask, unit weights, no logits output, no dropout, head_dim 64 or 128, 2-byte dtype, same rows and
 * stream) both run in ONE kernel: every row is given several workgroups when there are fewer rows than compute
 * units; each finds the row's columns by itself, attends to its share of them, and the one that finishes last
 * merges the partial results, which meet in t->work (sah_sparse_attention_work_floats covers them).
 * tickets: rows.n_rows 32-bit words in which the workgroups of a row count their arrivals; zero before the first
 * call, left zero by every call (calls that share them must not overlap). NULL: rows are never given more than one
 * workgroup. rows.cols / rows.cnt / rows.bitmap are still written. Otherwise the two calls are made. */
int sah_select_topk_attention(const sah_select_topk_args* s, const sah_attention_args* t, uint32_t* tickets);

/* ---------------------------------------------------------------------------
 * What an additive attention mask holds. The reference adds the mask it is given to every score row
 * (hashattention_top_k.py:365-368, oracle_top_k.py:70-72) and to the attention logits
 * (utils/mask_attention_utils.py:221-225) whatever it contains; through HuggingFace it is the eager mask
 * (adapters/huggingface.py:311-319), which for a single decode query of an unpadded batch is all zeros. Adding
 * zeros changes nothing, so a caller that knows the mask is all zeros may pass NULL instead and skip its reads.
 * ORs into *flags (an int32 the caller has zeroed): SAH_AMASK_NONZERO if any of the first Lk columns of any row is not
 * 0, SAH_AMASK_GENERAL if any such value lies above the lowest finite value of `dtype` (i.e. is neither 0 nor a
 * "hidden column" marker such as finfo.min or -inf). Asynchronous like every call: read *flags after the stream has
 * reached this point. Mask shape (B, Hm, Lq, >= Lk), element strides ms_*, innermost stride 1. */
enum { SAH_AMASK_NONZERO = 1, SAH_AMASK_GENERAL = 2 };
typedef struct sah_amask_classify_args {
  const void* amask;
  int64_t ms_b, ms_h, ms_l;
  int32_t dtype;
  int32_t B, Hm, Lq, Lk;
  int32_t* flags;
  void* stream;
} sah_amask_classify_args;
int sah_amask_classify(const sah_amask_classify_args* a);

/* ---------------------------------------------------------------------------
 * One decode layer-step as a single call: runs, in this order and on the stream
 * each block names, every stage whose pointer is not NULL -
 *   sink_local -> (sig_a, sig_b as sah_hash_signatures_pair) -> compact -> hamming
 *   -> hash_decode -> qk -> pq_assign -> pq_adc -> select -> attention.
 * The blocks are the argument structures of the entry points above, unchanged;
 * a caller keeps them alive between steps and only patches the fields that move
 * (tensor pointers, key count). Replaces the per-masker Python dispatch of
 * ResearchAttention.custom_attention (research_attention/base.py:108-148) on the
 * decode path; stops at the first stage that fails and returns its code.
 * hash_decode directly followed by attention runs as sah_hash_decode_attention,
 * select directly followed by attention as sah_select_topk_attention.
 * ------------------------------------------------------------------------- */
typedef struct sah_chain_args {
  const sah_sink_local_args* sink_local;
  const sah_hash_sig_args* sig_a;
  const sah_hash_sig_args* sig_b;
  const sah_hamming_topk_args* hamming;
  const sah_hash_decode_args* hash_decode;
  const sah_qk_scores_args* qk;
  const sah_pq_assign_args* pq_assign;
  const sah_pq_adc_args* pq_adc;
  const sah_select_topk_args* select;
  const sah_attention_args* attention;
  const sah_hash_compact_args* compact;
  uint32_t* tickets;   /* of sah_select_topk_attention / sah_hash_decode_attention, or NULL */
} sah_chain_args;
int sah_run_chain(const sah_chain_args* a);

#ifdef __cplusplus
}
#endif
#endif /* SAH_H */
