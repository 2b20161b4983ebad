// Score-key top-k and the attention over the chosen rows in ONE kernel.
//
// The chains with a scoring pass of their own (OracleTopK: q.k of every key; PQCache: the ADC scores) end in
// "select the k best inactive columns of every row, then attend to the row". As two kernels that is a selection
// with one workgroup per mask row, a gather in split form and a merge kernel; with the 128 rows of a batch of 4
// half of the CUs idle through the selection, and a CU gathers K / V rows at a fixed rate however few of them work.
// Here every row is given `parts` workgroups (rows x parts ~ the number of CUs). Each of them finds the row's
// threshold by itself (the same arithmetic in every part; the score keys of a row are read `parts` times, from L2
// after the first: the parts of a KV group share a die) and builds the row's column list in LDS, then attends to its
// share of the list. The parts' partial results meet in the workspace; the part that
// arrives last merges them and writes the row. No part ever waits for another, so the grid cannot stall, and the
// hand-over uses device-scope atomic accesses, which need no cache write-back (sah_common.h).
#include "sah_common.h"
#include "sah_attn.h"
#include "sah_sel16.h"

static_assert(ATT_ROW_NT == SF_NT, "selection and whole-row attention share one workgroup");

struct selattn_params {
  sah_rows R;
  const uint16_t* keys;
  int64_t pitch;
  int n_cand, col_offset, k;
  uint32_t excluded_key;
  int fresh, sink, window;
  int write_bitmap;
  int parts;
  int cols_offset;  // of the column list inside the dynamic LDS
  const uint16_t* resid;  // KEYED: what the keys' rounding took away, laid out like `keys`
  float* work;        // [row][part][D + 2]
  uint32_t* tickets;  // [row], zero between kernels
};

// KEYED: the score keys are q.k itself, rounded as torch's matmul rounds it, and come with the remainders of that
// rounding (the exact scoring pass of OracleTopK): the walk takes its logits from there (two 2-byte reads per entry,
// of lines the selection has just pulled through the L2) and reads V rows only.
template <int DT, int D, int CPW, bool KEYED>
__global__ __launch_bounds__(SF_NT) void k_select16_attn(selattn_params P, att_params A) {
  sah_touch_kernargs<sizeof(selattn_params) + sizeof(att_params)>();
  constexpr int NW = SF_NT / SAH_WAVE;
  __shared__ sf_lds S;
  __shared__ float s_m[NW];
  __shared__ float s_l[NW];
  __shared__ float s_acc[NW][D];
  __shared__ int s_last;
  HIP_DYNAMIC_SHARED(unsigned char, sa_dyn)
  // Workgroup -> (row, part). Consecutive workgroup ids go round-robin to the 8 dies; a tile is a GQA group, tile t
  // runs on die t % 8 and all G x parts workgroups of the group take adjacent slots of that die: the sink / local K / V
  // rows the G heads have in common and the score keys the parts of a row have in common are fetched once per die.
  const int tid = threadIdx.x;
  const int G = A.Hq / A.Hkv;
  const int GP = G * P.parts;
  const int slot = blockIdx.x / ATT_XCDS;
  const int tile = (slot / GP) * ATT_XCDS + (int)(blockIdx.x % ATT_XCDS);  // (b * Hkv + hk) * Lq + qi
  if (tile >= P.R.n_rows / G) return;  // padding to a multiple of 8 tiles
  const int within = slot % GP;
  const int part = within / G;
  const int qi = tile % A.Lq;
  const int hk = (tile / A.Lq) % A.Hkv;
  const int b = tile / (A.Lq * A.Hkv);
  const int h = hk * G + within % G;
  const int r = (b * A.Hq + h) * A.Lq + qi;

  int* s_cols = (int*)(sa_dyn + P.cols_offset);
  int earlier = 0;
  const int cnt = sf_select_impl<CPW, true>(S, sa_dyn, P.R, r, P.keys + (int64_t)r * P.pitch, P.n_cand, P.col_offset,
                                            P.k < P.n_cand ? P.k : P.n_cand, P.excluded_key, P.fresh, P.sink, P.window,
                                            part == 0, P.write_bitmap != 0, &earlier, s_cols, part, P.parts);
  __syncthreads();  // the winners' part of the list is complete in LDS, and so is the bitmap row

  // This part's share of the row: its entries dealt to parts x 16 waves, a wave of part p taking every parts-th run.
  // The entries the row held before come first: the sink and local columns of one query in closed form (fresh rows),
  // or the row's list in memory.
  constexpr int KPI = SAH_WAVE / (D / 8);
  const int wave = sah_wave_id();
  const int n = P.R.n_keys;
  const int s_hi = P.sink < n ? P.sink : n;
  int lo = P.window > 0 ? n - P.window : n;
  if (lo < 0) lo = 0;
  const int lo2 = lo > s_hi ? lo : s_hi;
  const int* cols_mem = P.R.cols + (int64_t)r * P.R.cap;
  const int n_runs = NW * P.parts;
  const int per = (((cnt + n_runs - 1) / n_runs) + KPI - 1) / KPI * KPI;  // entries per run
  const int first = (wave * P.parts + part) * per;
  const int bound = first + per < cnt ? first + per : cnt;
  att_wave_state st;
  st.clear();
  const float unit = A.unit_inv_w;
  const uint16_t* krow = P.keys + (int64_t)r * P.pitch;
  const uint16_t* rrow = KEYED ? P.resid + (int64_t)r * P.pitch : nullptr;
  auto key_of = [&](int, int col) { return (uint32_t)krow[col] | ((uint32_t)rrow[col] << 16); };  // col_offset is 0
  if (KEYED && P.fresh)
    att_walk<DT, D, false, true>(
        A, r, b, h, hk, qi, first, bound, SAH_WAVE,
        [&](int i) { return i >= earlier ? s_cols[i] : (i < s_hi ? i : lo2 + (i - s_hi)); }, [&](int) { return unit; }, st, key_of);
  else if (KEYED)
    att_walk<DT, D, false, true>(
        A, r, b, h, hk, qi, first, bound, SAH_WAVE, [&](int i) { return i >= earlier ? s_cols[i] : cols_mem[i]; },
        [&](int) { return unit; }, st, key_of);
  else if (P.fresh)
    att_walk<DT, D, false, true>(
        A, r, b, h, hk, qi, first, bound, SAH_WAVE,
        [&](int i) { return i >= earlier ? s_cols[i] : (i < s_hi ? i : lo2 + (i - s_hi)); }, [&](int) { return unit; }, st);
  else
    att_walk<DT, D, false, true>(
        A, r, b, h, hk, qi, first, bound, SAH_WAVE, [&](int i) { return i >= earlier ? s_cols[i] : cols_mem[i]; },
        [&](int) { return unit; }, st);
  att_park<D, NW>(st, wave, s_m, s_l, s_acc);
  __syncthreads();
  if (part == 0 && P.write_bitmap) {  // the row's bitmap, complete in LDS since the barrier
    const uint32_t* s_bm = (const uint32_t*)sa_dyn;
    uint32_t* bm = P.R.bitmap + (int64_t)r * P.R.n_words;
    for (int i = tid; i < P.R.n_words; i += SF_NT) bm[i] = s_bm[i];
  }
  float a, M, l;
  att_gather<DT, D, NW>(s_m, s_l, s_acc, a, M, l);
  if (P.parts == 1) {
    att_store_row<DT, D>(A, r, b, h, qi, a, M, l);
    return;
  }
  // hand the partial result over; the part that arrives last merges
  att_merge_parts<DT, D>(A, r, b, h, qi, a, M, l, P.work, P.tickets + r, part, P.parts, s_last);
}

// floats of workspace the fused form needs for n_rows rows: the parts' partial results
int64_t selattn_work_floats(int n_rows, int D) {
  const int parts = att_row_parts(n_rows);
  if (parts == 1) return 0;
  return (int64_t)n_rows * parts * (D + 2);
}

template <int DT, int D, int CPW, bool KEYED>
static int selattn_launch(const sah_select_topk_args* s, const selattn_params& P, const att_params& A, size_t lds) {
  if (int rc = sah_allow_lds((const void*)k_select16_attn<DT, D, CPW, KEYED>, 150 * 1024, "sah_select_topk_attention")) return rc;
  const int G = A.Hq / A.Hkv;
  const int n_tiles = P.R.n_rows / G;
  const int n_wg = (n_tiles + ATT_XCDS - 1) / ATT_XCDS * ATT_XCDS * G * P.parts;
  sah_timed timed("k_select16_attn", s->stream);
  hipLaunchKernelGGL((k_select16_attn<DT, D, CPW, KEYED>), dim3(n_wg), dim3(SF_NT), lds, (hipStream_t)s->stream, P, A);
  return sah_launch_status("sah_select_topk_attention");
}

template <int DT, int D>
static int selattn_launch_c(const sah_select_topk_args* s, const selattn_params& P, const att_params& A, size_t lds, int cpw,
                            bool keyed) {
  if (keyed) return cpw <= 4 ? selattn_launch<DT, D, 4, true>(s, P, A, lds) : selattn_launch<DT, D, 8, true>(s, P, A, lds);
  return cpw <= 4 ? selattn_launch<DT, D, 4, false>(s, P, A, lds) : selattn_launch<DT, D, 8, false>(s, P, A, lds);
}

extern "C" int sah_select_topk_attention(const sah_select_topk_args* s, const sah_attention_args* t, uint32_t* tickets) {
  if (!s || !t) return sah_fail(SAH_ENULL, "sah_select_topk_attention: args is NULL");
  int rc = sel_validate(s, "sah_select_topk_attention");
  if (rc) return rc;
  att_params A;
  rc = att_prepare(t, A);
  if (rc) return rc;
  const int n_rows = s->rows.n_rows;
  const int cpw = sf_chunks_per_wave(s->n_cand);
  const size_t cols_offset = sf_hist_offset(s->rows.n_words);
  // the selection's keys are the attention's logits: the caller names the same array as the attention's score keys
  const bool keyed = t->score_keys && t->score_resid && t->score_keys == s->keys && t->score_pitch == s->key_pitch &&
                     s->col_offset == 0 && s->n_cand == s->rows.n_keys;
  const size_t lds = sf_lds_bytes(s->rows.n_words);
  const int parts = att_row_parts(n_rows);
  const int64_t need = selattn_work_floats(n_rows, t->D);
  int64_t worst = (int64_t)s->k + (s->fresh ? (int64_t)s->fresh_sink + s->fresh_window : (int64_t)s->rows.cap);
  if (worst > s->rows.cap) worst = s->rows.cap;
  const bool one_kernel =
      sel16_ok(s) && cpw <= 8 && (size_t)s->rows.cap * 4 <= sf_hist_bytes() && lds + 10 * 1024 <= 150 * 1024 && !s->rows.w &&
      !t->dense && !t->closed_form && !t->amask && !t->logits_out && !t->rows.w && t->dropout_p == 0.f &&
      t->rows.cols == s->rows.cols && t->rows.cnt == s->rows.cnt && t->rows.cap == s->rows.cap && t->rows.n_rows == n_rows &&
      t->stream == s->stream && (t->dtype == SAH_BF16 || t->dtype == SAH_F16) && (t->D == 128 || t->D == 64) &&
      // one workgroup per row pays when the rows are short enough for the whole-row form; several per row always
      // several workgroups per row read the row's count while one of them rewrites it: fresh rows only
      (parts > 1 ? (tickets && t->work && t->work_floats >= need && s->fresh) : worst <= 8192);
  if (!one_kernel) {
    if ((rc = sah_select_topk(s))) return rc;
    return sah_sparse_attention(t);
  }
  selattn_params P;
  P.R = s->rows;
  P.keys = (const uint16_t*)s->keys;
  P.pitch = s->key_pitch;
  P.n_cand = s->n_cand; P.col_offset = s->col_offset; P.k = s->k;
  P.excluded_key = s->excluded_key;
  P.fresh = s->fresh ? 1 : 0; P.sink = s->fresh_sink; P.window = s->fresh_window;
  P.write_bitmap = s->skip_bitmap ? 0 : 1;
  P.parts = parts;
  P.cols_offset = (int)cols_offset;
  P.resid = (const uint16_t*)t->score_resid;
  P.work = t->work;
  P.tickets = tickets;
#define SAH_SA(DTC) \
  (t->D == 128 ? selattn_launch_c<DTC, 128>(s, P, A, lds, cpw, keyed) : selattn_launch_c<DTC, 64>(s, P, A, lds, cpw, keyed))
  return t->dtype == SAH_BF16 ? SAH_SA(SAH_BF16) : SAH_SA(SAH_F16);
#undef SAH_SA
}
