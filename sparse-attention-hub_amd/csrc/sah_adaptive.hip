// Adaptive sampling (vAttention): per mask row, a budget from a base sample of the
// softmax numerators, then that many uniform draws merged into the row with their
// sampling probability as weight.
//
// Both kernels run one workgroup per mask row. The numerators e[j] are never
// stored: they are a pure function of the row's order-preserving score keys (the
// output of the QK scoring pass, 2 or 4 bytes per key), which stay L2-resident
// while a row is worked on. Random numbers come from Philox4x32-10 with the
// counter (block of 4 draws, row, call offset), so a row's draws do not depend
// on the launch geometry and a CPU restatement can reproduce them bit for bit.
#include "sah_common.h"

#define AD_NT 1024
#define AD_NW (AD_NT / SAH_WAVE)
#define AD_EPT 4          // entries of a row a thread keeps in registers
#define AD_MAX_LDS_WORDS 36864  // 144 KB bitmap: sampling range up to ~1.17 M keys

// uniform column of [start, start + range) from one 32-bit draw
__device__ __forceinline__ int ad_column(uint32_t u, int start, int range) { return start + (int)sah_mulhi(u, (uint32_t)range); }

// ---------------------------------------------------------------------------
// score keys -> numerators, rounded where the reference's torch ops round
// ---------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float ad_key_score(uint32_t k) {
  if (DT == SAH_F32) return sah_bits_to_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
  const uint32_t u = (k & 0x8000u) ? (k & 0x7fffu) : ((~k) & 0xffffu);
  return DT == SAH_BF16 ? sah_bf16_to_float((uint16_t)u) : sah_f16_to_float((uint16_t)u);
}

template <int DT>
struct ad_row {
  typedef typename std::conditional<DT == SAH_F32, uint32_t, uint16_t>::type key_t;
  const key_t* keys;
  const void* amask;  // additive mask row or NULL
  int64_t moff;
  float scaling;
  float zmax;
  // z and the numerator of column j whose score key the caller holds
  __device__ __forceinline__ float z_of(uint32_t key, int j) const {
    float s = sah_round<DT>(ad_key_score<DT>(key) * scaling);
    if (amask) s = sah_round<DT>(s + sah_load<DT>(amask, moff + j));
    return s;
  }
  __device__ __forceinline__ float e_of(uint32_t key, int j) const {
    return sah_round<DT>(expf(sah_round<DT>(z_of(key, j) - zmax)));
  }
  __device__ __forceinline__ float z(int j) const { return z_of(keys[j], j); }
  __device__ __forceinline__ float e(int j) const { return e_of(keys[j], j); }
};

__device__ __forceinline__ float ad_block_sum(float v, float* s_red) {
  v = sah_wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & (SAH_WAVE - 1)) == 0) s_red[threadIdx.x / SAH_WAVE] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < AD_NW; ++i) t += s_red[i];
  return t;
}

__device__ __forceinline__ float ad_block_max(float v, float* s_red) {
  v = sah_wave_max(v);
  __syncthreads();
  if ((threadIdx.x & (SAH_WAVE - 1)) == 0) s_red[threadIdx.x / SAH_WAVE] = v;
  __syncthreads();
  float t = s_red[0];
#pragma unroll
  for (int i = 1; i < AD_NW; ++i) t = fmaxf(t, s_red[i]);
  return t;
}

struct ad_budget_params {
  sah_rows rows;
  const void* keys; int64_t key_pitch;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int Hq, Lq;
  float scaling;
  int start, range, n_base;
  float eps, ppf;
  uint32_t k0, k1, o0, o1;
  int prev_empty;
  int max_in_rows;  // the caller's promise: every row's largest key belongs to a column already in the row
  int vec_keys;  // 1: every row of keys starts 16-byte aligned (vector loads in the row-maximum pass)
  int* budget;
  float* prob;
  float* stats;
};

template <int DT>
__global__ __launch_bounds__(AD_NT) void k_adaptive_budget(ad_budget_params P) {
  sah_touch_kernargs<sizeof(ad_budget_params)>();
  HIP_DYNAMIC_SHARED(uint32_t, s_bits)  // one bit per column of the sampling range (word aligned)
  __shared__ float s_red[AD_NW];
  const int tid = threadIdx.x;
  const int r = blockIdx.x;
  const int Lk = P.rows.n_keys;
  const int end = P.start + P.range;
  const int w0 = P.start >> 5;
  const int nw = ((end + 31) >> 5) - w0;

  ad_row<DT> row;
  row.keys = (const typename ad_row<DT>::key_t*)P.keys + (int64_t)r * P.key_pitch;
  row.amask = P.amask;
  row.moff = 0;
  if (P.amask) {
    const int qi = r % P.Lq, h = (r / P.Lq) % P.Hq, b = r / (P.Lq * P.Hq);
    row.moff = (int64_t)b * P.ms_b + (int64_t)h * P.ms_h + (int64_t)qi * P.ms_l;
  }
  row.scaling = P.scaling;
  row.zmax = 0.f;

  for (int i = tid; i < nw; i += AD_NT) s_bits[i] = 0u;

  // The row's entries, the first AD_EPT of every thread held in registers: they serve the row maximum (when the
  // caller promises that it is among them) and the static denominator from one fetch.
  int ent_c[AD_EPT];
  uint32_t ent_k[AD_EPT];
  int cnt = 0;
  const int* cols = P.rows.cols + (int64_t)r * P.rows.cap;
  if (!P.prev_empty) {
    cnt = P.rows.cnt[r];
    if (cnt > P.rows.cap) cnt = P.rows.cap;
  }
  // ---- row maximum of z over ALL keys (adaptive_sampling.py:195-196)
  float zm = -INFINITY;
  const bool from_entries = P.max_in_rows && !P.prev_empty && !P.amask && P.scaling > 0.f;
  if (from_entries) {
    // z is a non-decreasing function of the score and the keys keep the scores' order: the maximum is z of the
    // largest key, and an exact top-k over these keys has put that key's column into the row
    uint32_t best = 0u;
#pragma unroll
    for (int u = 0; u < AD_EPT; ++u) {
      const int i = tid + u * AD_NT;
      int c = i < cnt ? cols[i] : -1;
      if (c >= Lk) c = -1;
      ent_c[u] = c;
    }
#pragma unroll
    for (int u = 0; u < AD_EPT; ++u) {
      ent_k[u] = ent_c[u] >= 0 ? (uint32_t)row.keys[ent_c[u]] : 0u;  // key 0 is the smallest key
      best = ent_k[u] > best ? ent_k[u] : best;
    }
    for (int i = tid + AD_EPT * AD_NT; i < cnt; i += AD_NT) {
      const int c = cols[i];
      if (c < 0 || c >= Lk) continue;
      const uint32_t kc = (uint32_t)row.keys[c];
      best = kc > best ? kc : best;
    }
    zm = sah_round<DT>(ad_key_score<DT>(best) * row.scaling);
  } else if (!P.amask && P.vec_keys && P.scaling > 0.f) {
    // Without an additive mask z is a non-decreasing function of the score, and the keys keep the
    // scores' order: the row maximum is z of the largest key. 16 bytes of keys per load, integer max.
    constexpr int KPV = (DT == SAH_F32) ? 4 : 8;  // keys per 16-byte vector
    const uint4* kv = (const uint4*)row.keys;
    const int n_vec = Lk / KPV;
    uint32_t best = 0u;
    for (int base = 0; base < n_vec; base += 4 * AD_NT) {
      uint4 q[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * AD_NT + tid;
        q[u] = i < n_vec ? kv[i] : make_uint4(0u, 0u, 0u, 0u);  // key 0 is the smallest key
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          if (DT == SAH_F32) {
            best = w[t] > best ? w[t] : best;
          } else {
            const uint32_t lo = w[t] & 0xffffu, hi = w[t] >> 16;
            best = lo > best ? lo : best;
            best = hi > best ? hi : best;
          }
        }
      }
    }
    for (int j = n_vec * KPV + tid; j < Lk; j += AD_NT) {
      const uint32_t kj = (uint32_t)row.keys[j];
      best = kj > best ? kj : best;
    }
    float s = sah_round<DT>(ad_key_score<DT>(best) * row.scaling);
    zm = s;
  } else {
    for (int j = tid; j < Lk; j += AD_NT) zm = fmaxf(zm, row.z(j));
  }
  row.zmax = ad_block_max(zm, s_red);

  // ---- static denominator: numerators of the active entries times their inverse weight
  float part = 0.f;
  if (P.prev_empty) {
    for (int j = tid; j < Lk; j += AD_NT) part += row.e(j);
  } else {
    const float* w = P.rows.w ? P.rows.w + (int64_t)r * P.rows.cap : nullptr;
    auto add = [&](int i, int c, float num) {
      float iw = sah_round<DT>(1.0f / sah_round<DT>(1.0f + 1e-6f));
      if (w) iw = sah_round<DT>(1.0f / sah_round<DT>(w[i] + 1e-6f));
      part += sah_round<DT>(num * iw);
    };
    int i = tid;
    if (from_entries) {
#pragma unroll
      for (int u = 0; u < AD_EPT; ++u, i += AD_NT)
        if (ent_c[u] >= 0) add(i, ent_c[u], row.e_of(ent_k[u], ent_c[u]));
    }
    for (; i < cnt; i += AD_NT) {
      const int c = cols[i];
      if (c < 0 || c >= Lk) continue;
      add(i, c, row.e(c));
    }
  }
  const float static_den = sah_round<DT>(ad_block_sum(part, s_red));

  // ---- base sample: mean, unbiased std, and the set of distinct columns
  const int n_calls = (P.n_base + 3) >> 2;
  part = 0.f;
  float first_e[4] = {0.f, 0.f, 0.f, 0.f};  // numerators of the thread's first call (all of them up to 4096 draws)
  for (int c = tid; c < n_calls; c += AD_NT) {
    uint32_t u[4];
    sah_philox((uint32_t)c, (uint32_t)r, P.o0, P.o1, P.k0, P.k1, u);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (4 * c + t < P.n_base) {
        const int j = ad_column(u[t], P.start, P.range);
        const float ej = row.e(j);
        if (c == tid) first_e[t] = ej;
        part += ej;
        atomicOr(&s_bits[(j >> 5) - w0], 1u << (j & 31));
      }
    }
  }
  const float mean = ad_block_sum(part, s_red) / (float)P.n_base;
  part = 0.f;
  if (tid < n_calls) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (4 * tid + t < P.n_base) {
        const float d = first_e[t] - mean;
        part = fmaf(d, d, part);
      }
    }
  }
  for (int c = tid + AD_NT; c < n_calls; c += AD_NT) {
    uint32_t u[4];
    sah_philox((uint32_t)c, (uint32_t)r, P.o0, P.o1, P.k0, P.k1, u);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (4 * c + t < P.n_base) {
        const float d = row.e(ad_column(u[t], P.start, P.range)) - mean;
        part = fmaf(d, d, part);
      }
    }
  }
  const float var = ad_block_sum(part, s_red) / (float)(P.n_base - 1);
  float sigma = sah_round<DT>(sqrtf(var));
  sigma = fmaxf(sigma, sah_round<DT>(1e-8f));

  // ---- denominator estimate from the distinct base columns, each weighted 1/(nb/n + 1e-6)
  const float wb = sah_round<DT>((float)((double)P.n_base / (double)P.range));
  const float inv_b = sah_round<DT>(1.0f / sah_round<DT>(wb + 1e-6f));
  part = 0.f;
  for (int wi = tid; wi < nw; wi += AD_NT) {
    uint32_t m = s_bits[wi];
    while (m) {
      const int bit = __builtin_ctz(m);
      m &= m - 1;
      part += sah_round<DT>(row.e(((w0 + wi) << 5) + bit) * inv_b);
    }
  }
  const float sampled_den = sah_round<DT>(ad_block_sum(part, s_red));

  if (tid == 0) {
    // adaptive_sampling.py:282-302 and :394-397, every intermediate rounded to the tensor dtype
    const float est = sah_round<DT>(static_den + sampled_den);
    const float err = fmaxf(sah_round<DT>(P.eps * est), sah_round<DT>(1e-8f));
    const float num = sah_round<DT>(sah_round<DT>(P.ppf * sigma) * (float)P.range);
    const float ratio = sah_round<DT>(num / err);
    float sq = sah_round<DT>(ratio * ratio);
    const float hi = sah_round<DT>((float)P.range);
    if (!(sq >= 1.0f)) sq = 1.0f;  // also catches NaN the way clamp(min=) orders its compares
    if (sq > hi) sq = hi;
    long long b = (long long)sq;
    if (b < P.n_base) b = P.n_base;
    if (b > P.range) b = P.range;
    P.budget[r] = (int)b;
    P.prob[r] = sah_round<DT>((float)b / (float)P.range);
    if (P.stats) {
      float* s = P.stats + (int64_t)r * 4;
      s[0] = static_den;
      s[1] = sigma;
      s[2] = est;
      s[3] = row.zmax;
    }
  }
}

struct ad_sample_params {
  sah_rows rows;
  const int* budget;
  const float* prob;
  int start, range;
  uint32_t k0, k1, o0, o1;
  int w_fresh;
};

template <int DT>
__global__ __launch_bounds__(AD_NT) void k_adaptive_sample(ad_sample_params P) {
  sah_touch_kernargs<sizeof(ad_sample_params)>();
  HIP_DYNAMIC_SHARED(uint32_t, s_bits)
  __shared__ int s_scan[AD_NW + 1];
  const int tid = threadIdx.x;
  const int r = blockIdx.x;
  const int end = P.start + P.range;
  const int w0 = P.start >> 5;
  const int nw = ((end + 31) >> 5) - w0;
  const int cap = P.rows.cap;

  int cnt0 = P.rows.cnt[r];  // read before any barrier: thread 0 rewrites it at the end
  if (cnt0 > cap) cnt0 = cap;
  int budget = P.budget[r];
  if (budget > P.range) budget = P.range;
  const float p = P.prob[r];

  for (int i = tid; i < nw; i += AD_NT) s_bits[i] = 0u;
  __syncthreads();

  const int n_calls = (budget + 3) >> 2;
  for (int c = tid; c < n_calls; c += AD_NT) {
    uint32_t u[4];
    sah_philox((uint32_t)c, (uint32_t)r, P.o0, P.o1, P.k0, P.k1, u);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (4 * c + t < budget) {
        const int j = ad_column(u[t], P.start, P.range);
        atomicOr(&s_bits[(j >> 5) - w0], 1u << (j & 31));
      }
    }
  }
  __syncthreads();

  int* cols = P.rows.cols + (int64_t)r * cap;
  float* w = P.rows.w + (int64_t)r * cap;
  uint32_t* gbits = P.rows.bitmap + (int64_t)r * P.rows.n_words;

  // entries already in the row: clamp(w + p, 0, 1) when drawn (utils/mask.py:875-877)
  for (int i = tid; i < cnt0; i += AD_NT) {
    const int c = cols[i];
    float wv = P.w_fresh ? 1.0f : w[i];
    bool changed = P.w_fresh != 0;
    if (c >= P.start && c < end && ((s_bits[(c >> 5) - w0] >> (c & 31)) & 1u)) {
      wv = fminf(1.0f, sah_round<DT>(wv + p));
      changed = true;
    }
    if (changed) w[i] = wv;
  }

  // new columns: a wave owns a contiguous run of bitmap words. Counted per thread, positions from one block scan.
  const int wpt = (nw + AD_NT - 1) / AD_NT;
  const int wa = tid * wpt;
  int wb = wa + wpt;
  if (wb > nw) wb = nw;
  int mine = 0;
  for (int wi = wa; wi < wb; ++wi) mine += __builtin_popcount(s_bits[wi] & ~gbits[w0 + wi]);
  int total = 0;
  const int pos = cnt0 + sah_block_excl_scan<AD_NT>(mine, s_scan, &total);
  // Written wave by wave, 64 words at a time (lane i: word i of the group), one bit position after the other:
  // the lanes that hold bit b of their word store to consecutive entries, so every store instruction fills
  // whole cache lines. (A thread appending its own columns one after the other scatters each store over 64
  // lines; a row whose budget is most of the range writes tens of thousands of columns.) The list is unordered.
  const int lane = tid & (SAH_WAVE - 1);
  int out = __builtin_amdgcn_readfirstlane(pos);  // the wave's first entry
  const int wave_w0 = (tid - lane) * wpt;
  for (int g = 0; g < wpt; ++g) {
    const int wi = wave_w0 + g * SAH_WAVE + lane;
    uint32_t fresh = 0;
    if (wi < nw) {
      const uint32_t drawn = s_bits[wi];
      if (drawn) {
        const uint32_t old = gbits[w0 + wi];
        fresh = drawn & ~old;
        if (fresh) gbits[w0 + wi] = old | drawn;
      }
    }
    if (__ballot(fresh != 0) == 0) continue;  // uniform across the wave
    for (int bit = 0; bit < 32; ++bit) {
      const bool has = (fresh >> bit) & 1u;
      const uint64_t m = __ballot(has);
      if (m == 0) continue;
      if (has) {
        const int at = out + sah_lane_prefix(m);
        if (at < cap) cols[at] = ((w0 + wi) << 5) + bit;
      }
      out += __popcll(m);
    }
  }
  // every new entry carries the weight p: one contiguous fill instead of a second scatter
  for (int i = cnt0 + tid; i < cnt0 + total && i < cap; i += AD_NT) w[i] = p;
  if (tid == 0) {
    int c = cnt0 + total;
    P.rows.cnt[r] = c < cap ? c : cap;
  }
}

// ---------------------------------------------------------------------------
// host
// ---------------------------------------------------------------------------
static int ad_lds_words(int start, int range) { return ((start + range + 31) >> 5) - (start >> 5); }

static int ad_check_range(const sah_rows& rows, int start, int range, const char* what) {
  if (start < 0 || range < 2 || (int64_t)start + range > rows.n_keys)
    return sah_fail(SAH_EINVAL, "%s: sampling range [%d, %d) must hold >= 2 columns inside [0, %d)", what, start,
                    start + range, rows.n_keys);
  if (ad_lds_words(start, range) > AD_MAX_LDS_WORDS)
    return sah_fail(SAH_ESHAPE, "%s: sampling range %d exceeds the %d columns one workgroup's LDS bitmap holds", what,
                    range, AD_MAX_LDS_WORDS * 32);
  return SAH_OK;
}

template <int DT>
static int ad_budget_launch(const sah_adaptive_budget_args* a, const ad_budget_params& P) {
  int rc = sah_allow_lds((const void*)k_adaptive_budget<DT>, AD_MAX_LDS_WORDS * 4, "sah_adaptive_budget");
  if (rc) return rc;
  const size_t lds = (size_t)ad_lds_words(a->start, a->range) * 4;
  sah_timed timed("k_adaptive_budget", a->stream);
  hipLaunchKernelGGL(k_adaptive_budget<DT>, dim3(a->rows.n_rows), dim3(AD_NT), lds, (hipStream_t)a->stream, P);
  return sah_launch_status("sah_adaptive_budget");
}

extern "C" int sah_adaptive_budget(const sah_adaptive_budget_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_adaptive_budget: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_adaptive_budget", !a->prev_empty);
  if (rc) return rc;
  if (!a->keys || !a->budget || !a->prob) return sah_fail(SAH_ENULL, "sah_adaptive_budget: NULL keys / budget / prob");
  if (a->key_pitch < a->rows.n_keys) return sah_fail(SAH_EINVAL, "sah_adaptive_budget: key_pitch < n_keys");
  if (a->Hq <= 0 || a->Lq <= 0 || a->rows.n_rows % (a->Hq * a->Lq))
    return sah_fail(SAH_EINVAL, "sah_adaptive_budget: n_rows is not a multiple of Hq * Lq");
  rc = ad_check_range(a->rows, a->start, a->range, "sah_adaptive_budget");
  if (rc) return rc;
  if (a->n_base < 2) return sah_fail(SAH_EINVAL, "sah_adaptive_budget: n_base must be >= 2");
  ad_budget_params P;
  P.rows = a->rows;
  P.keys = a->keys; P.key_pitch = a->key_pitch;
  P.amask = a->amask; P.ms_b = a->ms_b; P.ms_h = a->ms_h; P.ms_l = a->ms_l;
  P.Hq = a->Hq; P.Lq = a->Lq;
  P.scaling = a->scaling;
  P.start = a->start; P.range = a->range; P.n_base = a->n_base;
  P.max_in_rows = a->max_in_rows;
  P.eps = a->eps; P.ppf = a->delta_ppf;
  P.k0 = (uint32_t)a->seed; P.k1 = (uint32_t)(a->seed >> 32);
  P.o0 = (uint32_t)a->offset; P.o1 = (uint32_t)(a->offset >> 32);
  P.prev_empty = a->prev_empty;
  {
    const int es = a->dtype == SAH_F32 ? 4 : 2;
    P.vec_keys = (((uintptr_t)a->keys % 16) == 0 && (a->key_pitch * es) % 16 == 0) ? 1 : 0;
  }
  P.budget = a->budget; P.prob = a->prob; P.stats = a->stats;
  switch (a->dtype) {
    case SAH_F32: return ad_budget_launch<SAH_F32>(a, P);
    case SAH_BF16: return ad_budget_launch<SAH_BF16>(a, P);
    case SAH_F16: return ad_budget_launch<SAH_F16>(a, P);
    default: return sah_fail(SAH_EDTYPE, "sah_adaptive_budget: dtype %d", a->dtype);
  }
}

template <int DT>
static int ad_sample_launch(const sah_adaptive_sample_args* a, const ad_sample_params& P) {
  int rc = sah_allow_lds((const void*)k_adaptive_sample<DT>, AD_MAX_LDS_WORDS * 4, "sah_adaptive_sample");
  if (rc) return rc;
  const size_t lds = (size_t)ad_lds_words(a->start, a->range) * 4;
  sah_timed timed("k_adaptive_sample", a->stream);
  hipLaunchKernelGGL(k_adaptive_sample<DT>, dim3(a->rows.n_rows), dim3(AD_NT), lds, (hipStream_t)a->stream, P);
  return sah_launch_status("sah_adaptive_sample");
}

extern "C" int sah_adaptive_sample(const sah_adaptive_sample_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_adaptive_sample: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_adaptive_sample");
  if (rc) return rc;
  if (!a->rows.w) return sah_fail(SAH_ENULL, "sah_adaptive_sample: rows.w is NULL (sampled entries carry weights)");
  if (!a->budget || !a->prob) return sah_fail(SAH_ENULL, "sah_adaptive_sample: NULL budget / prob");
  rc = ad_check_range(a->rows, a->start, a->range, "sah_adaptive_sample");
  if (rc) return rc;
  ad_sample_params P;
  P.rows = a->rows;
  P.budget = a->budget; P.prob = a->prob;
  P.start = a->start; P.range = a->range;
  P.k0 = (uint32_t)a->seed; P.k1 = (uint32_t)(a->seed >> 32);
  P.o0 = (uint32_t)a->offset; P.o1 = (uint32_t)(a->offset >> 32);
  P.w_fresh = a->w_fresh;
  switch (a->dtype) {
    case SAH_F32: return ad_sample_launch<SAH_F32>(a, P);
    case SAH_BF16: return ad_sample_launch<SAH_BF16>(a, P);
    case SAH_F16: return ad_sample_launch<SAH_F16>(a, P);
    default: return sah_fail(SAH_EDTYPE, "sah_adaptive_sample: dtype %d", a->dtype);
  }
}
