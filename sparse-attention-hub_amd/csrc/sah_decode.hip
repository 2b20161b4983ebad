// One decode step of a Sink + Local + HashAttentionTopK chain in a single kernel.
//
// One workgroup (1024 threads) per mask row (b, h), one query position. The row is built from
// scratch in LDS and registers:
//   1. sink and local columns in closed form: list entries written, bitmap row built in LDS
//      (never read from memory);
//   2. the two signature MLPs of the step, side by side: threads 0-511 hash the query of head h,
//      threads 512-1023 the newest key (its code goes to the signature cache; the column itself
//      lies inside the local window, so this step's selection never looks at it);
//   3. signature top-k of the not-yet-active columns (the SWAR selection), appended to the row.
// Against three separate launches this saves two kernel boundaries, the bitmap round trip through
// memory and the query-code round trip.
#include "sah_common.h"
#include "sah_attn.h"
#include "sah_hsw.h"
#include "sah_sig.h"

static_assert(ATT_ROW_NT == HSW_NT, "selection and whole-row attention share one workgroup");

// Threads per MLP job and weight-row slots per thread: the same geometry as the stand-alone signature
// kernel, so that both sum in the same order and produce the same bits.
#define HDEC_GROUP 512
#define HDEC_ROWS 4

// scratch of one signature job: the GEMV form or the matrix-core form
template <bool MF>
struct hdec_sig {
  typedef sig_gemv_lds<1, HDEC_GROUP> lds;
};
template <>
struct hdec_sig<true> {
  typedef sig_mfma_lds lds;
};

struct hdec_params {
  sah_rows R;
  sig_params job[2];  // 0: query, 1: newest key
  int has_key;
  const uint2* kcodes;
  int64_t pitch;
  int k;
  int sink, window;
  int update_bitmap;
  // compact code stream (all NULL / 0: the two-plane stream kcodes is scanned)
  const uint32_t* pos;
  int64_t pos_pitch;
  const uint4* exc;
  const int* exc_cnt;
  int exc_cap;
  uint32_t full_plane;
};

// The mask row r of one decode step; returns its entry count. s_cols (optional, LDS, R.cap ints): copy of the
// row's column list for a caller that continues with it in the same kernel (complete after its next barrier).
// CP: the codes are read in their compact form (one sign plane per column + exception list).
// SILU: both MLPs use SiLU and have the usual shape, 128 -> 128 -> 128 -> 32 (checked by the host): the matrix-core form
// then carries no other activation's code and knows every width at compile time
template <int DT, bool MF, bool CP, bool SILU = false>
__device__ __forceinline__ int hdec_row(const hdec_params& P, int r, hsw_lds& S, unsigned char* hdec_dyn, int* s_cols) {
  typedef typename hdec_sig<MF>::lds hdec_sig_lds;
  const sah_rows& R = P.R;
  const int tid = threadIdx.x;
  const int n = R.n_keys;
  const int n_ch = (n + 255) / 256;
  uint32_t* s_bm = (uint32_t*)hdec_dyn;
  uint32_t* s_key = s_bm + n_ch * 8;
  // the MLP scratch shares the space of the staged scores: the MLPs are over before staging starts
  hdec_sig_lds* s_sig = (hdec_sig_lds*)s_key;

  // ---- 1. sink + local, one query at position n - 1 (basic_fixed.py:354-363, :48-67)
  const int s_hi = P.sink < n ? P.sink : n;
  int lo = 0, hi = 0;
  if (P.window > 0) {
    lo = n - P.window;
    hi = n;
    if (lo < 0) lo = 0;
  }
  const int lo2 = lo > s_hi ? lo : s_hi;
  const int n_local = hi > lo2 ? hi - lo2 : 0;
  const int fixed = s_hi + n_local;
  // written while the loads requested below are on their way
  auto fixed_part = [&]() {
    int* cols = R.cols + (int64_t)r * R.cap;
    for (int i = tid; i < fixed && i < R.cap; i += HSW_NT) {
      cols[i] = i < s_hi ? i : lo2 + (i - s_hi);
      if (s_cols) s_cols[i] = i < s_hi ? i : lo2 + (i - s_hi);
      if (R.w) R.w[(int64_t)r * R.cap + i] = 1.0f;
    }
    for (int wi = tid; wi < n_ch * 8; wi += HSW_NT)
      s_bm[wi] = wi < R.n_words ? (sah_range_bits(wi, 0, s_hi) | sah_range_bits(wi, lo, hi)) : 0u;
  };

  // ---- 2. signatures of the query and of the newest key
  // uniform across the wave, and known to be: the job's parameters are then fetched by scalar loads
  const int job = __builtin_amdgcn_readfirstlane(tid / HDEC_GROUP);
  // without a new key the second group only takes the barriers
  const bool active = job == 0 || P.has_key != 0;
  const int Hq = P.job[0].Hq;
  // 2-byte weights: all layers requested up-front; fp32 rows are twice as wide, one layer at a time
  constexpr int PF = (DT == SAH_F32) ? 1 : SAH_MAX_MLP_LAYERS;
  // the first half of the row's codes is requested behind the MLP's own loads and arrives while it computes
  hsw_bufs_t<CP> buf;
  const uint2* kc = P.kcodes + (int64_t)r * P.pitch;
  hsw_compact cs;
  if constexpr (CP) {
    cs.pos = P.pos + (int64_t)r * P.pos_pitch;
    cs.exc = P.exc + (int64_t)r * P.exc_cap;
    cs.exc_cnt = P.exc_cnt + r;
    cs.full = kc;
    cs.exc_cap = P.exc_cap;
    cs.full_plane = P.full_plane;
  }
  // Compact stream with the matrix-core MLP: the waves that run the query's MLP (0-7) request their codes only
  // after it, so that no queue of code requests stands between them and their weights (issuing 8 more loads
  // per lane into the full memory pipe held their first layer up for 8K cycles); the idle half of the
  // workgroup requests its codes at once and scores them while the first half's are on their way.
  const bool early = !(MF && CP) || job != 0;
  auto prefetch = [&]() {
    if (early) {
      if constexpr (CP) hsw_prefetch(cs, n, buf);
      else hsw_prefetch(kc, n, buf);
    }
    fixed_part();
  };
  if constexpr (MF) {
    sig_mfma_block<DT, decltype(prefetch), SILU ? SAH_ACT_SILU : -1, SILU>(P.job[job], active, tid % HDEC_GROUP, r / Hq, r % Hq, 0, 1,
                                                                      P.job[0].n_layers, s_sig[job], prefetch);
  } else {
    sig_gemv_block<DT, 1, HDEC_GROUP, HDEC_ROWS, PF>(P.job[job], active, tid % HDEC_GROUP, r / Hq, r % Hq, 0, 1,
                                                      P.job[0].n_layers, s_sig[job], prefetch);
  }
  const uint2 q = s_sig[0].code[0];
  hsw_lds_init(S);
  __syncthreads();  // every thread holds q (and the bitmap is complete) before the scores overwrite the scratch

  // ---- 3. top-k over the remaining columns
  // the row's active columns are the sink and local ranges just built, nothing else
  return hsw_select_row<CP>(R, r, kc, q, P.k, fixed < R.cap ? fixed : R.cap, s_bm, s_key, S, buf, early, P.update_bitmap != 0,
                            s_cols, CP ? &cs : nullptr, s_hi, n_local > 0 ? lo2 : n);
}

template <int DT, bool MF, bool CP, bool SILU>
__global__ __launch_bounds__(HSW_NT) void k_hash_decode(hdec_params P) {
  sah_touch_kernargs<sizeof(hdec_params)>();
  __shared__ hsw_lds S;
  HIP_DYNAMIC_SHARED(unsigned char, hdec_dyn)
  hdec_row<DT, MF, CP, SILU>(P, blockIdx.x, S, hdec_dyn, nullptr);
}

// Selection and attention of a row in one workgroup: as soon as a row's columns are chosen its K / V rows are
// gathered, from a column list that never leaves LDS. No kernel boundary between the two halves: a CU whose row
// was selected early starts streaming while others still select, and the attention's start-up latency is paid
// while the memory system would otherwise idle. Workgroup -> row mapping as in k_sparse_attn (the query heads
// of a GQA group on one XCD).
// parts > 1 (fewer rows than CUs): every row is given `parts` workgroups. Each builds the whole row by itself (the
// same arithmetic, so the lists are identical and both write the same values to the row in memory), attends to its
// share of the list, and the one that arrives last merges the partial results (att_merge_parts).
template <int DT, bool MF, bool CP, int D, bool SILU>
__global__ __launch_bounds__(HSW_NT) void k_hash_decode_attn(hdec_params P, att_params A, int cols_offset, int parts, float* work,
                                                             uint32_t* tickets) {
  __shared__ hsw_lds S;
  __shared__ float s_m[HSW_NW];
  __shared__ float s_l[HSW_NW];
  __shared__ float s_acc[HSW_NW][D];
  __shared__ int s_last;
  HIP_DYNAMIC_SHARED(unsigned char, hdec_dyn)
  sah_touch_kernargs<sizeof(hdec_params) + sizeof(att_params) + 32>();
  const int G = A.Hq / A.Hkv;
  const int GP = G * parts;
  const int slot = blockIdx.x / ATT_XCDS;
  const int tile = (slot / GP) * ATT_XCDS + (int)(blockIdx.x % ATT_XCDS);  // b * Hkv + hk
  if (tile >= P.R.n_rows / G) return;  // padding to a multiple of 8 tiles
  const int within = slot % GP;
  const int part = within / G;
  const int hk = tile % A.Hkv;
  const int b = tile / A.Hkv;
  const int h = hk * G + within % G;
  const int r = b * A.Hq + h;
  int* s_cols = (int*)(hdec_dyn + cols_offset);
  const int cnt = hdec_row<DT, MF, CP, SILU>(P, r, S, hdec_dyn, s_cols);
  __syncthreads();  // the column list in LDS is complete
  // the whole-row attention over the list in LDS: no additive mask, no weights, no logits output on this path
  {
    constexpr int KPI = SAH_WAVE / (D / 8);
    const int wave = sah_wave_id();
    const int n_runs = HSW_NW * parts;
    const int per = (((cnt + n_runs - 1) / n_runs) + KPI - 1) / KPI * KPI;  // entries per wave
    const int first = (wave * parts + part) * per;
    const int bound = first + per < cnt ? first + per : cnt;
    att_wave_state st;
    st.clear();
    const float unit = A.unit_inv_w;
    att_walk<DT, D, false, true>(
        A, r, b, h, hk, 0, first, bound, SAH_WAVE, [&](int i) { return s_cols[i]; }, [&](int) { return unit; }, st);
    att_park<D, HSW_NW>(st, wave, s_m, s_l, s_acc);
    __syncthreads();
    float a, M, l;
    att_gather<DT, D, HSW_NW>(s_m, s_l, s_acc, a, M, l);
    if (parts == 1) att_store_row<DT, D>(A, r, b, h, 0, a, M, l);
    else att_merge_parts<DT, D>(A, r, b, h, 0, a, M, l, work, tickets + r, part, parts, s_last);
  }
}

static size_t hdec_lds_bytes(int n_keys) {
  const int n_ch = (n_keys + 255) / 256;
  const size_t a = sizeof(hdec_sig<false>::lds), b = sizeof(hdec_sig<true>::lds);
  const size_t bm = (size_t)n_ch * 8 * 4, key = (size_t)n_ch * 64 * 4, sig = 2 * (a > b ? a : b);
  return bm + (key > sig ? key : sig);
}

// both MLPs of the step with SiLU and the usual widths, in the matrix-core form: the kernel variant that knows it
static bool hdec_silu(const hdec_params& P) {
  for (int j = 0; j < (P.has_key ? 2 : 1); ++j) {
    const sig_params& J = P.job[j];
    if (J.act != SAH_ACT_SILU || J.D != 128 || J.n_layers != 3 || J.d_out[0] != 128 || J.d_out[1] != 128 || J.d_out[2] != 32)
      return false;
  }
  return true;
}

template <int DT, bool MF, bool CP, bool SILU>
static int hdec_launch_s(const sah_hash_decode_args* a, const hdec_params& P, size_t lds) {
  if (int rc = sah_allow_lds((const void*)k_hash_decode<DT, MF, CP, SILU>, 150 * 1024, "sah_hash_decode_topk")) return rc;
  sah_timed timed("k_hash_decode", a->stream);
  hipLaunchKernelGGL((k_hash_decode<DT, MF, CP, SILU>), dim3(a->rows.n_rows), dim3(HSW_NT), lds, (hipStream_t)a->stream, P);
  return sah_launch_status("sah_hash_decode_topk");
}

template <int DT, bool MF, bool CP>
static int hdec_launch_t(const sah_hash_decode_args* a, const hdec_params& P, size_t lds) {
  if constexpr (MF) {
    if (hdec_silu(P)) return hdec_launch_s<DT, MF, CP, true>(a, P, lds);
  }
  return hdec_launch_s<DT, MF, CP, false>(a, P, lds);
}

template <int DT, bool MF>
static int hdec_launch(const sah_hash_decode_args* a, const hdec_params& P, size_t lds) {
  return P.pos ? hdec_launch_t<DT, MF, true>(a, P, lds) : hdec_launch_t<DT, MF, false>(a, P, lds);
}

// Which form of the signature MLP the stand-alone launches would take for this step's jobs: the fused kernel
// must take the same one, so that both routes produce the same bits. 0: not fusable, 1: GEMV, 2: matrix cores.
static int hdec_sig_kind(const sah_hash_decode_args* a, bool has_key) {
  const sah_hash_sig_args* q = a->query_sig;
  const sah_hash_sig_args* kk = a->key_sig;
  const bool qm = sig_mfma_small_ok(q), km = has_key ? sig_mfma_small_ok(kk) : qm;
  if (qm && km) return 2;
  if (qm || km) return 0;
  if (!sig_gemv_ok(q, HDEC_GROUP, HDEC_ROWS)) return 0;
  if (has_key && !sig_gemv_ok(kk, HDEC_GROUP, HDEC_ROWS)) return 0;
  return 1;
}

// can the single-kernel form run this step?
static bool hdec_fusable(const sah_hash_decode_args* a) {
  const sah_hash_sig_args* q = a->query_sig;
  const sah_hash_sig_args* kk = a->key_sig;
  const int n = a->rows.n_keys;
  if (q->L != 1 || (int64_t)q->B * q->Hq != a->rows.n_rows) return false;
  if (hdec_sig_kind(a, kk && kk->L > 0) == 0) return false;
  if (kk && kk->L > 0) {
    if (kk->L != 1 || kk->B != q->B || kk->Hq != q->Hq || kk->n_layers != q->n_layers || kk->dtype != q->dtype) return false;
    if (kk->D != q->D || kk->act != q->act) return false;
    for (int l = 0; l < q->n_layers; ++l)
      if (kk->d_out[l] != q->d_out[l]) return false;
    // the new code is written while the row's codes are scanned: its column must be one the scan ignores
    if ((const uint32_t*)kk->codes == a->kcodes && kk->code_offset < n - a->window) return false;
  }
  if (hdec_lds_bytes(n) > 150 * 1024) return false;
  if (a->code_pitch % 2 || ((uintptr_t)a->kcodes % 16) || n < 4) return false;
  return true;
}

static int hdec_validate(const sah_hash_decode_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hash_decode_topk: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_hash_decode_topk");
  if (rc) return rc;
  if (!a->query_sig || !a->kcodes) return sah_fail(SAH_ENULL, "sah_hash_decode_topk: query_sig / kcodes is NULL");
  if (!a->query_sig->codes) return sah_fail(SAH_ENULL, "sah_hash_decode_topk: query_sig.codes is NULL");
  if (a->sink < 0 || a->window < 0 || a->k < 0) return sah_fail(SAH_EINVAL, "sah_hash_decode_topk: negative sink / window / k");
  if (a->code_pitch < a->rows.n_keys) return sah_fail(SAH_EINVAL, "sah_hash_decode_topk: code_pitch < n_keys");
  rc = sig_validate(a->query_sig);
  if (rc) return rc;
  const bool has_key = a->key_sig && a->key_sig->L > 0;
  if (has_key) {
    rc = sig_validate(a->key_sig);
    if (rc) return rc;
  }
  if (a->query_sig->L != 1 || (int64_t)a->query_sig->B * a->query_sig->Hq != a->rows.n_rows)
    return sah_fail(SAH_ESHAPE, "sah_hash_decode_topk: needs one query per row (Lq = 1, n_rows = B * Hq)");
  int64_t worst = (int64_t)a->sink + a->window + a->k;
  if (worst > a->rows.n_keys) worst = a->rows.n_keys;
  if (worst > a->rows.cap)
    return sah_fail(SAH_ECAPACITY, "sah_hash_decode_topk: cap %d < sink + window + k = %lld", a->rows.cap, (long long)worst);

  return SAH_OK;
}

// may the single kernel read the compact stream the caller offers? (if not it scans the two-plane stream)
static bool hdec_compact_ok(const sah_hash_decode_args* a) {
  if (!a->pos_codes || !a->exc || !a->exc_cnt) return false;
  if (a->key_sig && a->key_sig->L > 0) return false;  // a key hashed inside the kernel would miss its compact entry
  const int n_ch = (a->rows.n_keys + 255) / 256;
  const int cpw = (n_ch + HSW_NW - 1) / HSW_NW;
  if (a->pos_pitch % 4 || ((uintptr_t)a->pos_codes % 16) || a->pos_pitch < (int64_t)(HSW_NW * cpw + 2 * HSW_CBATCH) * 256) return false;
  if (a->exc_cap < HSW_NT || ((uintptr_t)a->exc % 16)) return false;
  return true;
}

static void hdec_fill(const sah_hash_decode_args* a, hdec_params& P) {
  const bool has_key = a->key_sig && a->key_sig->L > 0;
  P.R = a->rows;
  sig_fill(a->query_sig, P.job[0]);
  sig_fill(has_key ? a->key_sig : a->query_sig, P.job[1]);
  if (!has_key) P.job[1].codes = nullptr;
  P.has_key = has_key ? 1 : 0;
  P.kcodes = (const uint2*)a->kcodes;
  P.pitch = a->code_pitch;
  P.k = a->k;
  P.sink = a->sink;
  P.window = a->window;
  P.update_bitmap = a->skip_bitmap ? 0 : 1;
  const bool cp = hdec_compact_ok(a);
  P.pos = cp ? a->pos_codes : nullptr;
  P.pos_pitch = a->pos_pitch;
  P.exc = (const uint4*)a->exc;
  P.exc_cnt = a->exc_cnt;
  P.exc_cap = a->exc_cap;
  P.full_plane = a->full_plane;
}

extern "C" int sah_hash_decode_topk(const sah_hash_decode_args* a) {
  int rc = hdec_validate(a);
  if (rc) return rc;
  const bool has_key = a->key_sig && a->key_sig->L > 0;
  if (!hdec_fusable(a)) {
    // same step as three launches
    sah_sink_local_args sl;
    sl.rows = a->rows; sl.lq = 1; sl.sink = a->sink; sl.window = a->window; sl.fresh = 1; sl.clear_future = 0;
    sl.stream = a->stream;
    rc = sah_sink_local_indices(&sl);
    if (rc) return rc;
    rc = has_key ? sah_hash_signatures_pair(a->key_sig, a->query_sig) : sah_hash_signatures(a->query_sig);
    if (rc) return rc;
    sah_hamming_topk_args ht;
    ht.rows = a->rows; ht.kcodes = a->kcodes; ht.code_pitch = a->code_pitch; ht.qcodes = a->query_sig->codes;
    ht.lq = 1; ht.k = a->k; ht.stream = a->stream;
    return sah_hamming_topk(&ht);
  }

  hdec_params P;
  hdec_fill(a, P);
  const size_t lds = hdec_lds_bytes(a->rows.n_keys);
  const bool mf = hdec_sig_kind(a, has_key) == 2;
  switch (a->query_sig->dtype) {
    case SAH_F32: return hdec_launch<SAH_F32, false>(a, P, lds);
    case SAH_BF16: return mf ? hdec_launch<SAH_BF16, true>(a, P, lds) : hdec_launch<SAH_BF16, false>(a, P, lds);
    default: return mf ? hdec_launch<SAH_F16, true>(a, P, lds) : hdec_launch<SAH_F16, false>(a, P, lds);
  }
}

template <int DT, bool MF, bool CP, int D, bool SILU>
static int hdec_attn_launch_s(const sah_hash_decode_args* a, const hdec_params& P, const att_params& A, size_t lds, int cols_offset,
                              int parts, float* work, uint32_t* tickets) {
  if (int rc = sah_allow_lds((const void*)k_hash_decode_attn<DT, MF, CP, D, SILU>, 150 * 1024, "sah_hash_decode_attention")) return rc;
  const int G = A.Hq / A.Hkv;
  const int n_tiles = P.R.n_rows / G;
  const int n_wg = (n_tiles + ATT_XCDS - 1) / ATT_XCDS * ATT_XCDS * G * parts;
  sah_timed timed("k_hash_decode_attn", a->stream);
  hipLaunchKernelGGL((k_hash_decode_attn<DT, MF, CP, D, SILU>), dim3(n_wg), dim3(HSW_NT), lds, (hipStream_t)a->stream, P, A, cols_offset,
                     parts, work, tickets);
  return sah_launch_status("sah_hash_decode_attention");
}

template <int DT, bool MF, bool CP, int D>
static int hdec_attn_launch_t(const sah_hash_decode_args* a, const hdec_params& P, const att_params& A, size_t lds, int cols_offset,
                              int parts, float* work, uint32_t* tickets) {
  if constexpr (MF) {
    if (hdec_silu(P)) return hdec_attn_launch_s<DT, MF, CP, D, true>(a, P, A, lds, cols_offset, parts, work, tickets);
  }
  return hdec_attn_launch_s<DT, MF, CP, D, false>(a, P, A, lds, cols_offset, parts, work, tickets);
}

template <int DT, bool MF, int D>
static int hdec_attn_launch(const sah_hash_decode_args* a, const hdec_params& P, const att_params& A, size_t lds, int cols_offset,
                            int parts, float* work, uint32_t* tickets) {
  return P.pos ? hdec_attn_launch_t<DT, MF, true, D>(a, P, A, lds, cols_offset, parts, work, tickets)
               : hdec_attn_launch_t<DT, MF, false, D>(a, P, A, lds, cols_offset, parts, work, tickets);
}

extern "C" int sah_hash_decode_attention(const sah_hash_decode_args* a, const sah_attention_args* t, uint32_t* tickets) {
  if (!a || !t) return sah_fail(SAH_ENULL, "sah_hash_decode_attention: args is NULL");
  int rc = hdec_validate(a);
  if (rc) return rc;
  att_params A;
  rc = att_prepare(t, A);
  if (rc) return rc;
  const bool has_key = a->key_sig && a->key_sig->L > 0;
  const size_t cols_offset = (hdec_lds_bytes(a->rows.n_keys) + 15) & ~(size_t)15;
  const size_t lds = cols_offset + (size_t)a->rows.cap * 4;
  // rows fewer than CUs: several workgroups per row, if the caller brought the tickets and the workspace for it
  const int parts = att_row_parts(a->rows.n_rows);
  const bool shared_rows = parts > 1 && tickets && t->work && t->work_floats >= (int64_t)a->rows.n_rows * parts * (t->D + 2);
  const bool one_kernel =
      hdec_fusable(a) && (shared_rows || A.n_split == 0) && !t->dense && !t->closed_form && !t->amask && !t->logits_out && !t->rows.w && t->Lq == 1 &&
      t->dropout_p == 0.f &&
      t->rows.cols == a->rows.cols && t->rows.cnt == a->rows.cnt && t->rows.cap == a->rows.cap &&
      t->rows.n_rows == a->rows.n_rows && t->stream == a->stream && t->dtype == a->query_sig->dtype &&
      (t->D == 128 || t->D == 64) && lds <= 150 * 1024;
  if (!one_kernel) {
    if ((rc = sah_hash_decode_topk(a))) return rc;
    return sah_sparse_attention(t);
  }
  hdec_params P;
  hdec_fill(a, P);
  const bool mf = hdec_sig_kind(a, has_key) == 2;
#define SAH_HDA(DTC, MFC)                                                                    \
  (t->D == 128 ? hdec_attn_launch<DTC, MFC, 128>(a, P, A, lds, (int)cols_offset, shared_rows ? parts : 1, t->work, tickets)  \
               : hdec_attn_launch<DTC, MFC, 64>(a, P, A, lds, (int)cols_offset, shared_rows ? parts : 1, t->work, tickets))
  switch (t->dtype) {
    case SAH_F32: return SAH_HDA(SAH_F32, false);
    case SAH_BF16: return mf ? SAH_HDA(SAH_BF16, true) : SAH_HDA(SAH_BF16, false);
    default: return mf ? SAH_HDA(SAH_F16, true) : SAH_HDA(SAH_F16, false);
  }
#undef SAH_HDA
}

// ---------------------------------------------------------------------------
// Compact form of the key-code stream: sign planes and the list of columns with a zero component.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_hash_compact(const uint2* codes, int64_t code_pitch, int from, int to, uint32_t* pos,
                                                      int64_t pos_pitch, uint4* exc, int exc_cap, int* exc_cnt,
                                                      uint32_t full_plane) {
  const int r = blockIdx.y;
  const int j = from + blockIdx.x * 256 + threadIdx.x;
  if (j >= to) return;
  const uint2 c = codes[(int64_t)r * code_pitch + j];
  pos[(int64_t)r * pos_pitch + j] = c.x;
  if (c.y != full_plane) {
    const int slot = atomicAdd(&exc_cnt[r], 1);
    if (slot < exc_cap) exc[(int64_t)r * exc_cap + slot] = make_uint4((uint32_t)j, c.y, c.x, 0u);
  }
}

extern "C" int sah_hash_compact_codes(const sah_hash_compact_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hash_compact_codes: args is NULL");
  if (!a->codes || !a->pos_codes || !a->exc || !a->exc_cnt) return sah_fail(SAH_ENULL, "sah_hash_compact_codes: NULL buffer");
  if (a->n_rows <= 0 || a->n_rows > 65535) return sah_fail(SAH_ESHAPE, "sah_hash_compact_codes: n_rows %d not in [1, 65535]", a->n_rows);
  if (a->from < 0 || a->to < a->from) return sah_fail(SAH_EINVAL, "sah_hash_compact_codes: bad column range [%d, %d)", a->from, a->to);
  if (a->code_pitch < a->to || a->pos_pitch < a->to) return sah_fail(SAH_ECAPACITY, "sah_hash_compact_codes: pitch < to");
  if (a->exc_cap < 1 || ((uintptr_t)a->exc % 16)) return sah_fail(SAH_EINVAL, "sah_hash_compact_codes: exception list unaligned or empty");
  if (a->to == a->from) return SAH_OK;
  sah_timed timed("k_hash_compact", a->stream);
  hipLaunchKernelGGL(k_hash_compact, dim3((a->to - a->from + 255) / 256, a->n_rows), dim3(256), 0, (hipStream_t)a->stream,
                     (const uint2*)a->codes, a->code_pitch, a->from, a->to, a->pos_codes, a->pos_pitch, (uint4*)a->exc,
                     a->exc_cap, a->exc_cnt, a->full_plane);
  return sah_launch_status("sah_hash_compact_codes");
}
