// Masked-softmax attention over gathered KV rows (flash-decoding layout).
//
// HBM-bound: every selected key costs one K row and one V row (D * elem bytes
// each). A wavefront reads 64/LPK rows per load instruction, LPK = D/8 lanes per
// row with 8 elements (16 B for bf16, 32 B for fp32) per lane, so each row is
// one fully coalesced segment. grid = (splits, mask rows); each workgroup
// (4 waves) walks its slice of the row's column list in chunks of 256 keys with
// a two-phase softmax per chunk (all K loads, block max, all V loads) and an
// online rescale between chunks, then writes (m, l, acc[D]) to the workspace.
// A second small kernel merges the splits, applies the optional sink logit and
// writes out[b, q, h, :].
#include "sah_common.h"
#include "sah_attn.h"

#include <mutex>

// KEYED: the logits come from the score keys of an exact q.k scoring pass (P.score_keys); K is not read
template <int DT, int D, bool ROW, bool DROP, bool FULL, bool KEYED = false>
__global__ __launch_bounds__(ROW ? ATT_ROW_NT : ATT_NT, ROW ? 1 : 5) void k_sparse_attn(att_params P) {
  sah_touch_kernargs<sizeof(att_params)>();
  constexpr int NW = (ROW ? ATT_ROW_NT : ATT_NT) / SAH_WAVE;
  __shared__ float s_m[NW];
  __shared__ float s_l[NW];
  __shared__ float s_acc[NW][D];

  // Workgroup -> work mapping. The hardware deals consecutive workgroup ids round-robin to the 8
  // XCDs, each with its own L2. A tile is (GQA group, split); tile t runs on XCD t % 8 and the G
  // query heads of the group take adjacent slots of that XCD, so the K/V rows they have in common
  // (all sink/local rows, every row in dense mode) are fetched from HBM once and shared in L2,
  // while every XCD gets the same number of tiles.
  const int G = P.Hq / P.Hkv;
  const int slot = blockIdx.x / ATT_XCDS;
  const int tile = (slot / G) * ATT_XCDS + (int)(blockIdx.x % ATT_XCDS);
  const int n_groups = P.rows.n_rows / G;
  const int n_split = ROW ? 1 : P.n_split;
  if (tile >= n_groups * n_split) return;  // padding to a multiple of 8 tiles
  const int split = tile % n_split;
  const int gidx = tile / n_split;            // (b * Hkv + hk) * Lq + qi
  const int qi = gidx % P.Lq;
  const int hk = (gidx / P.Lq) % P.Hkv;
  const int b = gidx / (P.Lq * P.Hkv);
  const int h = hk * G + slot % G;
  const int r = (b * P.Hq + h) * P.Lq + qi;
  att_tile<DT, D, ROW, DROP, FULL, KEYED>(P, r, b, h, hk, qi, split, n_split, nullptr, -1, s_m, s_l, s_acc);
}

template <int DT, int D>
__global__ __launch_bounds__(D < 64 ? 64 : D) void k_attn_combine(const float* work, int n_split, int Hq, int Lq, int d_real,
                                                                  const float* sinks, void* out, float* stats) {
  __shared__ float s_m[ATT_MAX_SPLIT];
  __shared__ float s_l[ATT_MAX_SPLIT];
  att_combine_row<DT, D>(work, n_split, blockIdx.x, Hq, Lq, d_real, sinks, out, stats, s_m, s_l);
}

template <int DT>
__global__ __launch_bounds__(256) void k_attn_weights(sah_rows R, const float* logits, int64_t pitch,
                                                      const float* stats, float unit_inv_w, int dense, void* weights,
                                                      sah_dropout drop) {
  const int r = blockIdx.y;
  const float m = stats[2 * (int64_t)r];
  const float den = stats[2 * (int64_t)r + 1];
  int cnt = dense ? R.n_keys : R.cnt[r];
  if (!dense && cnt > R.cap) cnt = R.cap;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= cnt) return;
  int c = i;
  float iw = unit_inv_w;
  if (!dense) {
    c = R.cols[(int64_t)r * R.cap + i];
    if (R.w) iw = sah_round<DT>(1.0f / sah_round<DT>(R.w[(int64_t)r * R.cap + i] + 1e-6f));
    if (c < 0 || c >= R.n_keys) return;
  }
  if (drop.thresh) iw *= drop.factor(r, c);
  const float z = logits[(int64_t)r * pitch + i];
  const float p = (z == -INFINITY) ? 0.f : att_exp<DT>(z - m) * iw / den;
  sah_store<DT>(weights, (int64_t)r * R.n_keys + c, p);
}

// Splits per row, from an upper bound of the row lengths: enough workgroups to cover 256 CUs several times,
// at least one chunk and at most 11 chunks of keys each (the kernel divides every row's own length by it; the
// longest rows set the pace at the end of the launch, so their tiles must stay small: at 512 rows of 1300 to
// 130000 entries 32 -> 47 splits took the kernel from 513 to 501 us, 64 splits gained nothing more).
static int att_pick_split(int n_rows, int max_cnt) {
  int chunks = (max_cnt + ATT_CHUNK - 1) / ATT_CHUNK;
  if (chunks < 1) chunks = 1;
  int want = (4096 + n_rows - 1) / n_rows;  // target ~4096 workgroups
  const int for_length = (chunks + 10) / 11;
  if (want < for_length) want = for_length;
  int n_split = chunks < want ? chunks : want;
  if (n_split > ATT_MAX_SPLIT) n_split = ATT_MAX_SPLIT;
  const int cps = (chunks + n_split - 1) / n_split;  // chunks per split
  return (chunks + cps - 1) / cps;
}

// head_dim as the kernels see it: itself if it is 16, 32, 64 or 128, otherwise the next power of two (0: not supported)
static int att_pad_dim(int D) {
  if (D <= 0 || D % 8 || D > 256) return 0;
  int dp = 16;
  while (dp < D) dp *= 2;
  return dp;
}

// with the selection in the same kernel (sah_select_topk_attention): partial results of a row's parts and their tickets
int64_t selattn_work_floats(int n_rows, int D);

extern "C" int64_t sah_sparse_attention_work_floats(int32_t n_rows, int32_t max_cnt, int32_t D) {
  if (n_rows <= 0 || max_cnt < 0 || D <= 0) return 0;
  D = att_pad_dim(D) ? att_pad_dim(D) : D;
  const int64_t fused = selattn_work_floats(n_rows, D);
  if (att_use_row_form(n_rows, max_cnt)) return fused;
  int n_split = att_pick_split(n_rows, max_cnt);
  const int64_t split = (int64_t)n_rows * n_split * (D + 2);
  return split > fused ? split : fused;
}

template <int DT, int D, bool FULL>
static int att_launch(const sah_attention_args* a, const att_params& P, bool timing) {
  hipStream_t st = (hipStream_t)a->stream;
  const int G = a->Hq / a->Hkv;
  // the variant that takes the logits from score keys: 16-bit types, head_dim 64 / 128, no dropout
  constexpr bool CAN_KEY = DT != SAH_F32 && FULL && (D == 64 || D == 128);
  const bool keyed = CAN_KEY && P.score_keys && !P.drop.thresh;
  if (P.n_split == 0) {  // whole-row form
    sah_timed timed("k_sparse_attn", a->stream, timing);
    const int n_tiles = a->rows.n_rows / G;
    const int n_wg = (n_tiles + ATT_XCDS - 1) / ATT_XCDS * ATT_XCDS * G;
    if (P.drop.thresh) hipLaunchKernelGGL((k_sparse_attn<DT, D, true, true, FULL>), dim3(n_wg), dim3(ATT_ROW_NT), 0, st, P);
    else if (keyed) hipLaunchKernelGGL((k_sparse_attn<DT, D, true, false, FULL, CAN_KEY>), dim3(n_wg), dim3(ATT_ROW_NT), 0, st, P);
    else hipLaunchKernelGGL((k_sparse_attn<DT, D, true, false, FULL>), dim3(n_wg), dim3(ATT_ROW_NT), 0, st, P);
    return sah_launch_status("sah_sparse_attention");
  }
  int rc;
  {
    sah_timed timed("k_sparse_attn", a->stream, timing);
    const int n_tiles = (a->rows.n_rows / G) * P.n_split;
    const int n_wg = (n_tiles + ATT_XCDS - 1) / ATT_XCDS * ATT_XCDS * G;
    if (P.drop.thresh) hipLaunchKernelGGL((k_sparse_attn<DT, D, false, true, FULL>), dim3(n_wg), dim3(ATT_NT), 0, st, P);
    else if (keyed) hipLaunchKernelGGL((k_sparse_attn<DT, D, false, false, FULL, CAN_KEY>), dim3(n_wg), dim3(ATT_NT), 0, st, P);
    else hipLaunchKernelGGL((k_sparse_attn<DT, D, false, false, FULL>), dim3(n_wg), dim3(ATT_NT), 0, st, P);
    rc = sah_launch_status("sah_sparse_attention");
  }
  if (rc) return rc;
  sah_timed timed("k_attn_combine", a->stream, timing);
  hipLaunchKernelGGL((k_attn_combine<DT, D>), dim3(a->rows.n_rows), dim3(D < 64 ? 64 : D), 0, st,
                     (const float*)a->work, P.n_split, a->Hq, a->Lq, a->D, a->sinks, a->out, a->stats_out);
  return sah_launch_status("sah_sparse_attention(combine)");
}

template <int DT>
static int att_dispatch_d(const sah_attention_args* a, const att_params& P, bool timing) {
  switch (a->D) {
    case 16: return att_launch<DT, 16, true>(a, P, timing);
    case 32: return att_launch<DT, 32, true>(a, P, timing);
    case 64: return att_launch<DT, 64, true>(a, P, timing);
    case 128: return att_launch<DT, 128, true>(a, P, timing);
    default: break;
  }
  // any other multiple of 8 up to 256: the next power of two, the lanes beyond head_dim idle
  switch (att_pad_dim(a->D)) {
    case 16: return att_launch<DT, 16, false>(a, P, timing);
    case 32: return att_launch<DT, 32, false>(a, P, timing);
    case 64: return att_launch<DT, 64, false>(a, P, timing);
    case 128: return att_launch<DT, 128, false>(a, P, timing);
    case 256: return att_launch<DT, 256, false>(a, P, timing);
    default: return sah_fail(SAH_ESHAPE, "sah_sparse_attention: head_dim %d is not a multiple of 8 in [8, 256]", a->D);
  }
}

// checks of sah_sparse_attention and the kernels' parameter block (also used by the fused decode kernel)
int att_prepare(const sah_attention_args* a, att_params& P) {
  if (!a) return sah_fail(SAH_ENULL, "sah_sparse_attention: args is NULL");
  if (!a->q || !a->k || !a->v || !a->out) return sah_fail(SAH_ENULL, "sah_sparse_attention: NULL tensor");
  if (a->B <= 0 || a->Hq <= 0 || a->Hkv <= 0 || a->Lq <= 0 || a->Lk <= 0)
    return sah_fail(SAH_EINVAL, "sah_sparse_attention: non-positive dimension");
  if (a->Hq % a->Hkv) return sah_fail(SAH_EINVAL, "sah_sparse_attention: Hq %% Hkv != 0");
  if (a->rows.n_rows != a->B * a->Hq * a->Lq || a->rows.n_keys != a->Lk)
    return sah_fail(SAH_EINVAL, "sah_sparse_attention: rows shape does not match B*Hq*Lq x Lk");
  if (a->closed_form && (a->dense || a->Lq != 1 || a->closed_sink < 0 || a->closed_window < 0 || a->amask || a->logits_out))
    return sah_fail(SAH_EINVAL,
                    "sah_sparse_attention: closed_form needs Lq = 1, dense = 0, sink / window >= 0, no additive mask, no logits output");
  if (!a->dense && !a->closed_form) {
    int rc = sah_check_rows(a->rows, "sah_sparse_attention");
    if (rc) return rc;
  }
  const int es = a->dtype == SAH_F32 ? 4 : 2;
  const int64_t align = 8;  // elements: 8-element vector loads
  if (a->qs_b % align || a->qs_h % align || a->qs_l % align || a->ks_b % align || a->ks_h % align ||
      a->ks_l % align || a->vs_b % align || a->vs_h % align || a->vs_l % align)
    return sah_fail(SAH_ESHAPE, "sah_sparse_attention: strides must be multiples of 8 elements");
  if (((uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v) % (8 * es))
    return sah_fail(SAH_ESHAPE, "sah_sparse_attention: q/k/v base pointers must be %d-byte aligned", 8 * es);
  int max_cnt = a->dense ? a->Lk : a->max_cnt;
  P.closed_sink = P.closed_lo = P.closed_cnt = 0;
  if (a->closed_form) {
    // the columns k_sink_local would write for one query per row (basic_fixed.py:354-363, :48-67)
    const int s_hi = a->closed_sink < a->Lk ? a->closed_sink : a->Lk;
    int lo = a->closed_window > 0 ? a->Lk - a->closed_window : a->Lk;
    if (lo < 0) lo = 0;
    if (lo < s_hi) lo = s_hi;
    P.closed_sink = s_hi;
    P.closed_lo = lo;
    P.closed_cnt = s_hi + (a->closed_window > 0 ? a->Lk - lo : 0);
    max_cnt = P.closed_cnt;
  }
  if (max_cnt <= 0) return sah_fail(SAH_EINVAL, "sah_sparse_attention: max_cnt must be > 0");
  if (!a->dense && !a->closed_form && max_cnt > a->rows.cap) max_cnt = a->rows.cap;

  P.rows = a->rows;
  P.q = a->q; P.qs_b = a->qs_b; P.qs_h = a->qs_h; P.qs_l = a->qs_l;
  P.k = a->k; P.ks_b = a->ks_b; P.ks_h = a->ks_h; P.ks_l = a->ks_l;
  P.v = a->v; P.vs_b = a->vs_b; P.vs_h = a->vs_h; P.vs_l = a->vs_l;
  P.amask = a->amask; P.ms_b = a->ms_b; P.ms_h = a->ms_h; P.ms_l = a->ms_l;
  P.Hq = a->Hq; P.Hkv = a->Hkv; P.Lq = a->Lq; P.Lk = a->Lk;
  P.d_real = a->D;
  P.scaling = a->scaling; P.unit_inv_w = a->unit_inv_w;
  P.dense = a->dense ? 1 : (a->closed_form ? 2 : 0);
  P.n_split = att_use_row_form(a->rows.n_rows, max_cnt) ? 0 : att_pick_split(a->rows.n_rows, max_cnt);  // 0: whole rows
  P.work = a->work;
  P.sinks = a->sinks; P.out = a->out; P.stats = a->stats_out;
  P.logits_out = a->logits_out;
  P.logits_pitch = a->dense ? a->Lk : a->rows.cap;
  P.drop_num_only = a->dropout_numerator_only ? 1 : 0;
  P.score_keys = P.score_resid = nullptr;
  P.score_pitch = 0;
  if (a->score_keys && a->score_resid) {
    if (a->score_pitch < a->Lk) return sah_fail(SAH_EINVAL, "sah_sparse_attention: score_pitch < Lk");
    if (a->dtype != SAH_F32) {  // fp32 scores do not fit 16-bit keys: K is read as ever
      P.score_keys = (const uint16_t*)a->score_keys;
      P.score_resid = (const uint16_t*)a->score_resid;
      P.score_pitch = a->score_pitch;
    }
  }
  if (!sah_dropout_fill(a->dropout_p, a->dropout_seed, a->dropout_offset, P.drop))
    return sah_fail(SAH_EINVAL, "sah_sparse_attention: dropout_p %g not in [0, 1)", (double)a->dropout_p);
  if (!att_pad_dim(a->D)) return sah_fail(SAH_ESHAPE, "sah_sparse_attention: head_dim %d is not a multiple of 8 in [8, 256]", a->D);
  const int64_t need = (int64_t)a->rows.n_rows * P.n_split * (att_pad_dim(a->D) + 2);
  if (a->work_floats < need)
    return sah_fail(SAH_ECAPACITY, "sah_sparse_attention: work has %lld floats, need %lld", (long long)a->work_floats,
                    (long long)need);
  return SAH_OK;
}

static int att_dispatch(const sah_attention_args* a, const att_params& P, bool timing) {
  switch (a->dtype) {
    case SAH_F32: return att_dispatch_d<SAH_F32>(a, P, timing);
    case SAH_BF16: return att_dispatch_d<SAH_BF16>(a, P, timing);
    case SAH_F16: return att_dispatch_d<SAH_F16>(a, P, timing);
    default: return sah_fail(SAH_EDTYPE, "sah_sparse_attention: dtype %d", a->dtype);
  }
}

extern "C" int sah_sparse_attention(const sah_attention_args* a) {
  att_params P;
  const int rc = att_prepare(a, P);
  if (rc) return rc;
  return att_dispatch(a, P, true);
}

// ---------------------------------------------------------------------------
// The same call for callers that cannot allocate: the partial results of the split form go to a buffer that
// lives in the library's own device image instead of a workspace the caller would have to allocate.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float scratch[SAH_ATTENTION_STATIC_WORK_FLOATS];

// Device address of `scratch` on the current device. In host code the array's name is only a handle for
// hipGetSymbolAddress; every GPU has its own copy at its own address, looked up once per device.
static int att_static_work(float** out) {
  static std::mutex mu;
  static float* ptr[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sah_fail((int)e, "sah_sparse_attention_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= 64) return sah_fail(SAH_EINVAL, "sah_sparse_attention_static: device index %d not in [0, 64)", dev);
  std::lock_guard<std::mutex> lk(mu);
  if (!ptr[dev]) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return sah_fail(e != hipSuccess ? (int)e : SAH_ENULL, "sah_sparse_attention_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return SAH_OK;
}

extern "C" int sah_sparse_attention_static(const sah_attention_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_sparse_attention_static: args is NULL");
  sah_attention_args b = *a;
  int rc = att_static_work(&b.work);
  if (rc) return rc;
  b.work_floats = SAH_ATTENTION_STATIC_WORK_FLOATS;
  att_params P;
  rc = att_prepare(&b, P);
  if (rc == SAH_ECAPACITY)
    return sah_fail(SAH_ECAPACITY,
                    "sah_sparse_attention_static: this call needs %lld workspace floats, the built-in buffer holds %lld; "
                    "use sah_sparse_attention with a workspace of your own",
                    (long long)b.rows.n_rows * P.n_split * (b.D + 2), (long long)SAH_ATTENTION_STATIC_WORK_FLOATS);
  if (rc) return rc;
  return att_dispatch(&b, P, false);  // no kernel timing here: recording it creates events
}

extern "C" int sah_attention_weights(const sah_attention_weights_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_attention_weights: args is NULL");
  if (!a->logits || !a->stats || !a->weights) return sah_fail(SAH_ENULL, "sah_attention_weights: NULL tensor");
  if (a->rows.n_rows <= 0 || a->rows.n_keys <= 0) return sah_fail(SAH_EINVAL, "sah_attention_weights: empty rows");
  const int dense = a->dense ? 1 : 0;
  if (!dense) {
    int rc = sah_check_rows(a->rows, "sah_attention_weights");
    if (rc) return rc;
  }
  const int max_cnt = dense ? a->rows.n_keys : a->rows.cap;
  const int64_t pitch = dense ? a->rows.n_keys : a->rows.cap;
  dim3 g((max_cnt + 255) / 256, a->rows.n_rows), b(256);
  hipStream_t st = (hipStream_t)a->stream;
  sah_dropout drop;
  if (!sah_dropout_fill(a->dropout_p, a->dropout_seed, a->dropout_offset, drop))
    return sah_fail(SAH_EINVAL, "sah_attention_weights: dropout_p %g not in [0, 1)", (double)a->dropout_p);
  sah_timed timed("k_attn_weights", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_attn_weights<SAH_F32>, g, b, 0, st, a->rows, a->logits, pitch, a->stats, a->unit_inv_w, dense, a->weights, drop); break;
    case SAH_BF16: hipLaunchKernelGGL(k_attn_weights<SAH_BF16>, g, b, 0, st, a->rows, a->logits, pitch, a->stats, a->unit_inv_w, dense, a->weights, drop); break;
    case SAH_F16: hipLaunchKernelGGL(k_attn_weights<SAH_F16>, g, b, 0, st, a->rows, a->logits, pitch, a->stats, a->unit_inv_w, dense, a->weights, drop); break;
    default: return sah_fail(SAH_EDTYPE, "sah_attention_weights: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_attention_weights");
}

extern "C" int sah_run_chain(const sah_chain_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_run_chain: args is NULL");
  int rc = SAH_OK;
  if (a->sink_local && (rc = sah_sink_local_indices(a->sink_local))) return rc;
  if (a->sig_a && a->sig_b) {
    if ((rc = sah_hash_signatures_pair(a->sig_a, a->sig_b))) return rc;
  } else if (a->sig_a) {
    if ((rc = sah_hash_signatures(a->sig_a))) return rc;
  } else if (a->sig_b) {
    if ((rc = sah_hash_signatures(a->sig_b))) return rc;
  }
  if (a->compact && (rc = sah_hash_compact_codes(a->compact))) return rc;
  if (a->hamming && (rc = sah_hamming_topk(a->hamming))) return rc;
  if (a->hash_decode && a->attention && !a->qk && !a->pq_assign && !a->pq_adc && !a->select)
    return sah_hash_decode_attention(a->hash_decode, a->attention, a->tickets);  // one kernel when shapes allow
  if (a->hash_decode && (rc = sah_hash_decode_topk(a->hash_decode))) return rc;
  if (a->qk && (rc = sah_qk_scores(a->qk))) return rc;
  if (a->pq_assign && (rc = sah_pq_kmeans_assign(a->pq_assign))) return rc;
  if (a->pq_adc && (rc = sah_pq_adc_scores(a->pq_adc))) return rc;
  if (a->select && a->attention) return sah_select_topk_attention(a->select, a->attention, a->tickets);  // one kernel when shapes allow
  if (a->select && (rc = sah_select_topk(a->select))) return rc;
  if (a->attention && (rc = sah_sparse_attention(a->attention))) return rc;
  return SAH_OK;
}
