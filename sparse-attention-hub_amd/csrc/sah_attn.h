// Masked-softmax attention over gathered KV rows: the device code shared by the stand-alone attention
// kernels and the fused decode kernel (selection + attention of a row in one workgroup).
#pragma once
#include "sah_common.h"

#define ATT_NT 256
#define ATT_NW (ATT_NT / SAH_WAVE)
#define ATT_ROW_NT 1024  // threads of the whole-row form
#define ATT_CHUNK (ATT_NT)  // keys per workgroup iteration: 64 per wave
#define ATT_XCDS 8           // accelerator complex dies of an MI355X, one L2 each
#define ATT_MAX_SPLIT 64

struct att_params {
  sah_rows rows;
  const void* q; int64_t qs_b, qs_h, qs_l;
  const void* k; int64_t ks_b, ks_h, ks_l;
  const void* v; int64_t vs_b, vs_h, vs_l;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int Hq, Hkv, Lq, Lk;
  int d_real;  // head_dim; the kernels' D is d_real padded to a power of two (lanes beyond d_real carry zeros)
  float scaling, unit_inv_w;
  int dense;
  int closed_sink, closed_lo, closed_cnt;  // dense == 2: entries [0, closed_sink) are columns [0, closed_sink), the rest start at closed_lo
  int n_split;
  const float* sinks;
  void* out;
  float* stats;
  float* work;
  float* logits_out;
  int64_t logits_pitch;
  sah_dropout drop;
  int drop_num_only;  // dropout leaves the softmax denominator alone (dropout of the normalised probabilities)
  const uint16_t* score_keys;   // [row][score_pitch]: q.k of every column as 16-bit score keys, or NULL
  const uint16_t* score_resid;  // ... and what the keys' rounding took away
  int64_t score_pitch;
};

// The logit source of a walk that reads K itself.
struct att_no_key {
  __device__ __forceinline__ uint32_t operator()(int, int) const { return 0u; }
};

// The dot product a (score key, remainder) pair stands for: the key is sah_sort_key of the dot product rounded to DT
// (low half of `kr`), the remainder what that rounding took away, in DT's bits (high half).
template <int DT>
__device__ __forceinline__ float att_key_score(uint32_t kr) {
  static_assert(DT != SAH_F32, "16-bit keys hold scores of 16-bit types");
  const uint32_t key = kr & 0xffffu;
  const uint32_t u = (key & 0x8000u) ? (key & 0x7fffu) : (~key & 0xffffu);
  if (DT == SAH_BF16) return sah_bits_to_float(u << 16) + sah_bits_to_float(kr & 0xffff0000u);
  return sah_f16_to_float((uint16_t)u) + sah_f16_to_float((uint16_t)(kr >> 16));
}

// exact expf for fp32 storage (1e-5 output tolerance), hardware exp2 path otherwise
template <int DT>
__device__ __forceinline__ float att_exp(float x) {
  return DT == SAH_F32 ? expf(x) : __expf(x);
}

template <int LPK>
__device__ __forceinline__ float att_group_sum(float v) {
  // sum over each aligned group of LPK lanes (LPK in {2,4,8,16,32})
  v += sah_dpp<0xB1>(v);
  if (LPK >= 4) v += sah_dpp<0x4E>(v);
  if (LPK >= 8) v += sah_dpp<0x141>(v);
  if (LPK >= 16) v += sah_dpp<0x140>(v);
  if (LPK >= 32) v += __shfl_xor(v, 16);
  return v;
}

// raw 8-element row slice as loaded (16 B for 2-byte types, 32 B for fp32)
template <int DT>
struct att_raw {
  uint4 lo;
  uint4 hi;  // only used for fp32
};

template <int DT>
__device__ __forceinline__ void att_load_raw(const char* p, att_raw<DT>& r) {
  r.lo = *(const uint4*)p;
  if (DT == SAH_F32) r.hi = *(const uint4*)(p + 16);
}

template <int DT>
__device__ __forceinline__ void att_unpack(const att_raw<DT>& r, float (&o)[8]) {
  const uint32_t w[4] = {r.lo.x, r.lo.y, r.lo.z, r.lo.w};
  if (DT == SAH_F32) {
    const uint32_t v[4] = {r.hi.x, r.hi.y, r.hi.z, r.hi.w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      o[t] = sah_bits_to_float(w[t]);
      o[4 + t] = sah_bits_to_float(v[t]);
    }
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (DT == SAH_BF16) {
        o[2 * t] = sah_bits_to_float(w[t] << 16);
        o[2 * t + 1] = sah_bits_to_float(w[t] & 0xffff0000u);
      } else {
        o[2 * t] = sah_f16_to_float((uint16_t)(w[t] & 0xffffu));
        o[2 * t + 1] = sah_f16_to_float((uint16_t)(w[t] >> 16));
      }
    }
  }
}

// merge the splits of one row: out = sum_s acc_s e^(m_s-M) / sum_s l_s e^(m_s-M).
// The (m, l) pairs go through LDS and each thread's partial values are requested together,
// so the merge costs about two memory round trips whatever the number of splits. Every thread of the
// workgroup calls it (one barrier inside); thread d < D produces output element d.
template <int DT, int D>
__device__ __forceinline__ void att_combine_row(const float* work, int n_split, int r, int Hq, int Lq, int d_real, const float* sinks,
                                                void* out, float* stats, float* s_m, float* s_l) {
  const int d = threadIdx.x;
  const float* w = work + (int64_t)r * n_split * (D + 2);
  if (d < n_split) {
    s_m[d] = w[(int64_t)d * (D + 2)];
    s_l[d] = w[(int64_t)d * (D + 2) + 1];
  }
  float part[ATT_MAX_SPLIT / 4];
  float a = 0.f;
  float M = -INFINITY, L = 0.f;
  for (int s0 = 0; s0 < n_split; s0 += ATT_MAX_SPLIT / 4) {
#pragma unroll
    for (int u = 0; u < ATT_MAX_SPLIT / 4; ++u) {
      const int sidx = s0 + u;
      part[u] = (sidx < n_split && d < D) ? w[(int64_t)sidx * (D + 2) + 2 + d] : 0.f;
    }
    if (s0 == 0) {
      __syncthreads();
      for (int sidx = 0; sidx < n_split; ++sidx) M = fmaxf(M, s_m[sidx]);
      for (int sidx = 0; sidx < n_split; ++sidx)
        if (s_m[sidx] != -INFINITY) L = fmaf(s_l[sidx], att_exp<DT>(s_m[sidx] - M), L);
    }
#pragma unroll
    for (int u = 0; u < ATT_MAX_SPLIT / 4; ++u) {
      const int sidx = s0 + u;
      if (sidx < n_split && s_m[sidx] != -INFINITY) a = fmaf(part[u], att_exp<DT>(s_m[sidx] - M), a);
    }
  }
  const int qi = r % Lq;
  const int h = (r / Lq) % Hq;
  const int b = r / (Lq * Hq);
  float Mf = M, den = L;
  if (sinks) {
    const float sk = sinks[h];
    Mf = fmaxf(M, sk);
    const float sc = (M == -INFINITY) ? 0.f : att_exp<DT>(M - Mf);
    a *= sc;
    den = L * sc + att_exp<DT>(sk - Mf);
  }
  if (d < d_real) sah_store<DT>(out, (((int64_t)b * Lq + qi) * Hq + h) * d_real + d, a / den);
  if (stats && d == 0) {
    stats[2 * (int64_t)r] = Mf;
    stats[2 * (int64_t)r + 1] = den;
  }
}

// A wave's online-softmax state: m uniform across the wave, l and acc per lane group (lane group = the D / 8
// lanes that share a key; a lane holds 8 elements of the accumulator).
struct att_wave_state {
  float acc[8];
  float l_run;
  float m_run;
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    l_run = 0.f;
    m_run = -INFINITY;
  }
};

// The K and V rows of one batch of a wave: UB iterations of SAH_WAVE / (D / 8) keys each, as loaded. id[u] is the
// column of the calling lane's key in iteration u (-1: none, the lane then reads row 0 and its result is dropped).
template <int DT, int UB>
struct att_batch {
  att_raw<DT> kr[UB], vr[UB];
  int id[UB];
};

// the calling lane's slice (8 elements) of the rows of head (b, hk): addresses, and the query's elements
// FULL: head_dim is D itself; otherwise D is head_dim padded to a power of two and the lanes of a key beyond head_dim
// load nothing and carry zeros
template <int DT, int D, bool FULL = true>
struct att_lane {
  static constexpr int LPK = D / 8;            // lanes per key
  static constexpr int KPI = SAH_WAVE / LPK;   // keys per wave iteration
  static constexpr int ES = (DT == SAH_F32) ? 4 : 2;
  const char* kbase;
  const char* vbase;
  int64_t krow, vrow;
  int sub, grp;  // which 8-element slice of the row, which key of the iteration
  bool live;     // this lane's slice lies inside head_dim
  __device__ __forceinline__ att_lane(const att_params& P, int b, int hk) {
    const int lane = threadIdx.x & (SAH_WAVE - 1);
    sub = lane % LPK;
    grp = lane / LPK;
    live = FULL || sub * 8 < P.d_real;
    kbase = (const char*)P.k + ((int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + sub * 8) * ES;
    vbase = (const char*)P.v + ((int64_t)b * P.vs_b + (int64_t)hk * P.vs_h + sub * 8) * ES;
    krow = P.ks_l * ES;
    vrow = P.vs_l * ES;
  }
  __device__ __forceinline__ void load_q(const att_params& P, int b, int h, int qi, float (&qv)[8]) const {
    if (FULL || live) {
      sah_load8<DT>(P.q, (int64_t)b * P.qs_b + (int64_t)h * P.qs_h + (int64_t)qi * P.qs_l + sub * 8, qv);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[e] = 0.f;
    }
  }
  // puts the batch's 2 * UB row loads on their way (KEYED: the logits are known, only the V rows are read)
  template <int UB, bool KEYED = false>
  __device__ __forceinline__ void request(att_batch<DT, UB>& B) const {
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int safe = B.id[u] >= 0 ? B.id[u] : 0;
      if (FULL || live) {
        if (!KEYED) att_load_raw<DT>(kbase + (int64_t)safe * krow, B.kr[u]);
        att_load_raw<DT>(vbase + (int64_t)safe * vrow, B.vr[u]);
      } else {
        B.kr[u].lo = B.kr[u].hi = B.vr[u].lo = B.vr[u].hi = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  }
  // the batch's logits (scaled, plus the additive mask; -inf for a lane without a key), and their maximum over the wave
  template <int UB, bool PLAIN = false>
  __device__ __forceinline__ float logits(const att_params& P, int64_t moff, const float (&qv)[8], const att_batch<DT, UB>& B,
                                          float (&z)[UB]) const {
    float mb = -INFINITY;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      float kf[8];
      att_unpack<DT>(B.kr[u], kf);
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) d = fmaf(qv[e], kf[e], d);
      d = att_group_sum<LPK>(d) * P.scaling;
      if (B.id[u] >= 0) {
        if (!PLAIN && P.amask) d += sah_load<DT>(P.amask, moff + B.id[u]);
      } else {
        d = -INFINITY;
      }
      z[u] = d;
      mb = fmaxf(mb, d);
    }
    // over the lane groups of the wave: m stays uniform across the wave
#pragma unroll
    for (int o = LPK; o < SAH_WAVE; o <<= 1) mb = fmaxf(mb, __shfl_xor(mb, o));
    return mb;
  }
  // the same from score keys: key[u] holds q.k of the lane's key in iteration u as (key, remainder)
  template <int UB, bool PLAIN = false>
  __device__ __forceinline__ float logits_of_keys(const att_params& P, int64_t moff, const uint32_t (&key)[UB],
                                                  const att_batch<DT, UB>& B, float (&z)[UB]) const {
    float mb = -INFINITY;
    if constexpr (DT != SAH_F32) {
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        float d = att_key_score<DT>(key[u]) * P.scaling;
        if (B.id[u] >= 0) {
          if (!PLAIN && P.amask) d += sah_load<DT>(P.amask, moff + B.id[u]);
        } else {
          d = -INFINITY;
        }
        z[u] = d;
        mb = fmaxf(mb, d);
      }
    }
#pragma unroll
    for (int o = LPK; o < SAH_WAVE; o <<= 1) mb = fmaxf(mb, __shfl_xor(mb, o));
    return mb;
  }
  // the online-softmax step of a batch: iw[u] is the inverse weight of the lane's key in iteration u
  // (iw_den: the inverse weights that enter the denominator - the same unless dropout spares it)
  template <int UB>
  __device__ __forceinline__ void accumulate(const att_batch<DT, UB>& B, const float (&z)[UB], float mb, const float (&iw)[UB],
                                             const float (&iw_den)[UB], att_wave_state& st) const {
    const float m_new = fmaxf(st.m_run, mb);
    if (m_new != -INFINITY) {
      const float rescale = (st.m_run == -INFINITY) ? 0.f : att_exp<DT>(st.m_run - m_new);
#pragma unroll
      for (int e = 0; e < 8; ++e) st.acc[e] *= rescale;
      st.l_run *= rescale;
      st.m_run = m_new;
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        float p = 0.f, pd = 0.f;
        if (z[u] != -INFINITY) {
          const float e = att_exp<DT>(z[u] - m_new);
          p = e * iw[u];
          pd = e * iw_den[u];
        }
        st.l_run += pd;
        float vf[8];
        att_unpack<DT>(B.vr[u], vf);
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[e] = fmaf(p, vf[e], st.acc[e]);
      }
    }
  }
};

// The calling wave attends to the entries first .. first + 63, first + stride .., all below `bound`, of row r:
// entry i is column col_of(i) (anything outside [0, Lk) is skipped) with inverse weight inv_w_of(i). Batches of UB
// iterations: the K and V rows of a batch are requested together, so 2 * UB row loads are in flight per lane.
// DROP: training-mode dropout of the exp weights (P.drop) is applied; a variant of its own, so that the decode path
// carries no trace of it. PLAIN: the caller knows that there is no additive mask and no logits output (the one-kernel
// decode step): their tests and code stay out. A caller whose column list lives in LDS hands col_of a pointer the
// compiler can see to be LDS: through a generic pointer every read of the list would be a flat load, which waits for
// all of the wave's outstanding row loads as well.
// key_of (anything but att_no_key): key_of(i, column) is q.k for entry i as score key (low half) and remainder (high
// half) - the caller has scored every column already (an exact-score top-k came before); K is then not read at all,
// and a batch holds twice as many V rows.
template <int DT, int D, bool DROP = false, bool PLAIN = false, bool FULL = true, typename ColOf, typename InvWOf,
          typename KeyOf = att_no_key>
__device__ __forceinline__ void att_walk(const att_params& P, int r, int b, int h, int hk, int qi, int first, int bound,
                                         int stride, ColOf col_of, InvWOf inv_w_of, att_wave_state& st, KeyOf key_of = KeyOf()) {
  typedef att_lane<DT, D, FULL> lane_t;
  constexpr bool KEYED = !std::is_same<KeyOf, att_no_key>::value;
  constexpr int KPI = lane_t::KPI;
  constexpr int IT = SAH_WAVE / KPI;    // iterations per 64-key wave slice
  constexpr int UB = IT < 4 ? IT : ((KEYED && IT >= 8) ? 8 : 4);   // iterations per batch
  const int lane = threadIdx.x & (SAH_WAVE - 1);
  const lane_t L(P, b, hk);
  const int64_t moff = (!PLAIN && P.amask) ? ((int64_t)b * P.ms_b + (int64_t)h * P.ms_h + (int64_t)qi * P.ms_l) : 0;
  float qv[8];
  L.load_q(P, b, h, qi, qv);

  for (int cbase = first; cbase < bound; cbase += stride) {
    // one column (and its inverse weight) per lane: this wave's next 64 keys
    const int my = cbase + lane;
    int idx_l = -1;
    uint32_t key_l = 0;
    float invw_l = P.unit_inv_w, invw_den_l = P.unit_inv_w;
    if (my < bound) {
      idx_l = col_of(my);
      invw_l = inv_w_of(my);
      if (idx_l < 0 || idx_l >= P.Lk) idx_l = -1;
      if (KEYED && idx_l >= 0) key_l = key_of(my, idx_l);
      invw_den_l = invw_l;
      if (DROP && idx_l >= 0) {
        invw_l *= P.drop.factor(r, idx_l);
        if (!P.drop_num_only) invw_den_l = invw_l;
      }
    }
#pragma unroll
    for (int ib = 0; ib < IT; ib += UB) {
      if (cbase + ib * KPI >= bound) break;  // uniform across the wave
      att_batch<DT, UB> B;
#pragma unroll
      for (int u = 0; u < UB; ++u) B.id[u] = __shfl(idx_l, (ib + u) * KPI + L.grp);
      L.template request<UB, KEYED>(B);
      float z[UB];
      float mb;
      if constexpr (KEYED) {
        uint32_t kz[UB];
#pragma unroll
        for (int u = 0; u < UB; ++u) kz[u] = (uint32_t)__shfl((int)key_l, (ib + u) * KPI + L.grp);
        mb = L.template logits_of_keys<UB, PLAIN>(P, moff, kz, B, z);
      } else {
        mb = L.template logits<UB, PLAIN>(P, moff, qv, B, z);
      }
      if (!PLAIN && P.logits_out && L.sub == 0) {
#pragma unroll
        for (int u = 0; u < UB; ++u) {
          const int pos = cbase + (ib + u) * KPI + L.grp;
          if (pos < bound) P.logits_out[(int64_t)r * P.logits_pitch + pos] = z[u];
        }
      }
      float iw[UB], iw_den[UB];
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        iw[u] = __shfl(invw_l, (ib + u) * KPI + L.grp);
        iw_den[u] = DROP ? __shfl(invw_den_l, (ib + u) * KPI + L.grp) : iw[u];
      }
      L.accumulate(B, z, mb, iw, iw_den, st);
    }
  }
}

// The calling wave's state, summed over its lane groups, into slot `slot` of the workgroup's partial results.
template <int D, int NS>
__device__ __forceinline__ void att_park(att_wave_state& st, int slot, float (&s_m)[NS], float (&s_l)[NS], float (&s_acc)[NS][D]) {
  constexpr int LPK = D / 8;
  const int lane = threadIdx.x & (SAH_WAVE - 1);
#pragma unroll
  for (int o = LPK; o < SAH_WAVE; o <<= 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[e] += __shfl_xor(st.acc[e], o);
    st.l_run += __shfl_xor(st.l_run, o);
  }
  if (lane < LPK) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_acc[slot][lane * 8 + e] = st.acc[e];
  }
  if (lane == 0) {
    s_l[slot] = st.l_run;
    s_m[slot] = st.m_run;
  }
}

// The workgroup's NS partial results (complete, a barrier passed) rescaled to a common max and summed: thread
// d < D gets element d of the numerator in `a`; every thread the max M and the denominator l.
template <int DT, int D, int NS>
__device__ __forceinline__ void att_gather(const float (&s_m)[NS], const float (&s_l)[NS], const float (&s_acc)[NS][D], float& a,
                                           float& M, float& l) {
  const int tid = threadIdx.x;
  M = s_m[0];
#pragma unroll
  for (int wv = 1; wv < NS; ++wv) M = fmaxf(M, s_m[wv]);
  float sc[NS];
#pragma unroll
  for (int wv = 0; wv < NS; ++wv) sc[wv] = (s_m[wv] == -INFINITY) ? 0.f : att_exp<DT>(s_m[wv] - M);
  a = 0.f;
  l = 0.f;
  if (tid < D) {
#pragma unroll
    for (int wv = 0; wv < NS; ++wv) a = fmaf(s_acc[wv][tid], sc[wv], a);
  }
#pragma unroll
  for (int wv = 0; wv < NS; ++wv) l = fmaf(s_l[wv], sc[wv], l);
}

// A complete row: normalise (with the optional sink logit, mask_attention_utils.py:357-402) and store
template <int DT, int D>
__device__ __forceinline__ void att_store_row(const att_params& P, int r, int b, int h, int qi, float a, float M, float l) {
  const int tid = threadIdx.x;
  float Mf = M, den = l;
  if (P.sinks) {
    const float sk = P.sinks[h];
    Mf = fmaxf(M, sk);
    const float rs = (M == -INFINITY) ? 0.f : att_exp<DT>(M - Mf);
    a *= rs;
    den = l * rs + att_exp<DT>(sk - Mf);
  }
  if (tid < P.d_real) sah_store<DT>(P.out, (((int64_t)b * P.Lq + qi) * P.Hq + h) * P.d_real + tid, a / den);
  if (P.stats && tid == 0) {
    P.stats[2 * (int64_t)r] = Mf;
    P.stats[2 * (int64_t)r + 1] = den;
  }
}

// A row attended to by `parts` workgroups, each holding the partial result (a for thread d < D, M, l) of its share:
// the partial results meet in `work` ([row][part][D + 2] floats) and the workgroup that arrives last (`ticket`: the
// row's arrival counter, zero between kernels) merges them, in part order whoever arrived last, and writes the row.
// Every thread of the workgroup calls it (two barriers inside); nobody waits for another workgroup. The hand-over
// uses device-scope atomic accesses, which need no cache write-back (sah_common.h).
#define ATT_MAX_PARTS 8
template <int DT, int D>
__device__ __forceinline__ void att_merge_parts(const att_params& P, int r, int b, int h, int qi, float a, float M, float l,
                                                float* work, uint32_t* ticket, int part, int parts, int& s_last) {
  const int tid = threadIdx.x;
  float* wrow = work + (int64_t)r * parts * (D + 2);
  float* mine = wrow + part * (D + 2);
  if (tid < D) sah_agent_store_f32(mine + 2 + tid, a);
  if (tid == 0) {
    sah_agent_store_f32(mine, M);
    sah_agent_store_f32(mine + 1, l);
  }
  sah_stores_done();
  __syncthreads();
  if (tid == 0) s_last = sah_last_arrival(ticket, (uint32_t)parts) ? 1 : 0;
  __syncthreads();
  if (!s_last) return;
  float pm[ATT_MAX_PARTS], pl[ATT_MAX_PARTS], pa[ATT_MAX_PARTS];
#pragma unroll
  for (int p = 0; p < ATT_MAX_PARTS; ++p) {
    const bool have = p < parts;
    pm[p] = have ? sah_agent_load_f32(wrow + p * (D + 2)) : -INFINITY;
    pl[p] = have ? sah_agent_load_f32(wrow + p * (D + 2) + 1) : 0.f;
    pa[p] = (have && tid < D) ? sah_agent_load_f32(wrow + p * (D + 2) + 2 + tid) : 0.f;
  }
  M = pm[0];
#pragma unroll
  for (int p = 1; p < ATT_MAX_PARTS; ++p) M = fmaxf(M, pm[p]);
  a = 0.f;
  l = 0.f;
#pragma unroll
  for (int p = 0; p < ATT_MAX_PARTS; ++p) {
    const float sc = (pm[p] == -INFINITY) ? 0.f : att_exp<DT>(pm[p] - M);
    a = fmaf(pa[p], sc, a);
    l = fmaf(pl[p], sc, l);
  }
  att_store_row<DT, D>(P, r, b, h, qi, a, M, l);
}

// workgroups per row of the kernels that select and attend in one launch: as many as it takes to give every CU a
// workgroup when there are fewer rows than CUs
static inline int att_row_parts(int n_rows) {
  int parts = 256 / n_rows;
  if (n_rows >= 192 || parts < 1) parts = 1;
  return parts > ATT_MAX_PARTS ? ATT_MAX_PARTS : parts;
}

// One tile of work of a workgroup. ROW = false: a workgroup of 4 waves handles one (row, split) tile and leaves (m, l, acc) in the workspace
//   for the merge kernel - the form for few or very uneven rows.
// ROW = true: a workgroup of 16 waves handles a whole row, every wave an equal share of the row's entries,
//   and merges the 16 partial results itself: no workspace, no second kernel, every CU gets the same
//   amount of work when there are at least as many rows as CUs.
template <int DT, int D, bool ROW, bool DROP = false, bool FULL = true, bool KEYED = false>
__device__ __forceinline__ void att_tile(const att_params& P, int r, int b, int h, int hk, int qi, int split, int n_split,
                                         const int* cols_known, int cnt_known,
                                         float (&s_m)[(ROW ? ATT_ROW_NT : ATT_NT) / SAH_WAVE],
                                         float (&s_l)[(ROW ? ATT_ROW_NT : ATT_NT) / SAH_WAVE],
                                         float (&s_acc)[(ROW ? ATT_ROW_NT : ATT_NT) / SAH_WAVE][D]) {
  constexpr int NW = (ROW ? ATT_ROW_NT : ATT_NT) / SAH_WAVE;
  constexpr int KPI = SAH_WAVE / (D / 8);   // keys per wave iteration
  const int tid = threadIdx.x;
  const int wave = sah_wave_id();

  // cnt_known >= 0: the caller holds the row's entry count (and `cols` may then point anywhere, LDS included)
  // P.dense: 0 = the rows' column lists, 1 = every key, 2 = the sink + local columns of one query in closed form
  int cnt = cnt_known >= 0 ? cnt_known : (P.dense == 1 ? P.Lk : (P.dense == 2 ? P.closed_cnt : P.rows.cnt[r]));
  if (!P.dense && cnt > P.rows.cap) cnt = P.rows.cap;
  // the row's own entry count decides the slices, so rows of very different lengths all spread evenly;
  // the host picks n_split from an upper bound only
  int first, bound, stride;  // this wave's slices start at first, first + stride, ... and stop at bound
  float* wout = nullptr;
  if constexpr (ROW) {
    const int per = (((cnt + NW - 1) / NW) + KPI - 1) / KPI * KPI;  // entries per wave
    first = wave * per;
    bound = first + per < cnt ? first + per : cnt;
    stride = SAH_WAVE;
  } else {
    const int row_chunks = (cnt + ATT_CHUNK - 1) / ATT_CHUNK;
    const int kps = ((row_chunks + n_split - 1) / n_split) * ATT_CHUNK;
    const int begin = split * kps;
    bound = begin + kps < cnt ? begin + kps : cnt;
    first = begin + wave * SAH_WAVE;
    stride = ATT_CHUNK;
    wout = P.work + ((int64_t)r * n_split + split) * (D + 2);
    if (begin >= bound) {
      if (tid == 0) {
        wout[0] = -INFINITY;
        wout[1] = 0.f;
      }
      return;
    }
  }

  const int* cols = cols_known ? cols_known : (P.dense ? nullptr : P.rows.cols + (int64_t)r * P.rows.cap);
  const float* wts = (!P.dense && P.rows.w) ? P.rows.w + (int64_t)r * P.rows.cap : nullptr;
  att_wave_state st;
  st.clear();
  auto col_of = [&](int i) {
    return P.dense == 1 ? i : (P.dense == 2 ? (i < P.closed_sink ? i : P.closed_lo + (i - P.closed_sink)) : cols[i]);
  };
  // the reference evaluates 1/(w + 1e-6) in the mask dtype (utils/mask.py:737-740)
  auto inv_w_of = [&](int i) { return wts ? sah_round<DT>(1.0f / sah_round<DT>(wts[i] + 1e-6f)) : P.unit_inv_w; };
  if constexpr (KEYED) {
    const uint16_t* krow = P.score_keys + (int64_t)r * P.score_pitch;
    const uint16_t* rrow = P.score_resid + (int64_t)r * P.score_pitch;
    att_walk<DT, D, DROP, false, FULL>(P, r, b, h, hk, qi, first, bound, stride, col_of, inv_w_of, st,
                                       [&](int, int col) { return (uint32_t)krow[col] | ((uint32_t)rrow[col] << 16); });
  } else {
    att_walk<DT, D, DROP, false, FULL>(P, r, b, h, hk, qi, first, bound, stride, col_of, inv_w_of, st);
  }

  // ---- reduce the lane groups of the wave, then the waves (rescaled to a common max)
  att_park<D, NW>(st, wave, s_m, s_l, s_acc);
  __syncthreads();
  float a, M, l;
  att_gather<DT, D, NW>(s_m, s_l, s_acc, a, M, l);
  if constexpr (ROW) {
    att_store_row<DT, D>(P, r, b, h, qi, a, M, l);
  } else {
    if (tid < D) wout[2 + tid] = a;
    if (tid == 0) {
      wout[0] = M;
      wout[1] = l;
    }
  }
}

// Whole-row form when every CU can be given rows of its own (or the rows are so short that splitting them
// only adds a second launch), and rows are not long enough for their spread in length to matter.
static inline bool att_use_row_form(int n_rows, int max_cnt) {
  return max_cnt <= 8192 && (n_rows >= 192 || max_cnt <= 1024);
}


// defined with the attention kernels: validation of a sah_sparse_attention call and its parameter block
int att_prepare(const sah_attention_args* a, att_params& P);
