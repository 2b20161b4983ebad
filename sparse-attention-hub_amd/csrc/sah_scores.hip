// Exact QK scoring pass of OracleTopK: one stream over K per KV head serves up
// to 4 query vectors of that head's GQA group (the 4 query heads in decode), no
// repeat_kv copy. HBM-bound: Lk * D * elem bytes per (b, kv head).
//
// Layout as in the attention kernel: LPK = D/8 lanes per key row, 8 elements
// (one 16 B / 32 B vector load) per lane, DPP reduction inside the lane group.
// Scores are rounded to the storage type exactly where torch rounds them and
// emitted as order-preserving unsigned keys through an LDS tile so that the
// global writes are coalesced.
#include "sah_common.h"

#define SC_NT 256
#define SC_NW (SC_NT / SAH_WAVE)
#define SC_NQ 4          // query vectors per workgroup
#define SC_TILE 256      // keys per workgroup iteration
#define SC_ITERS 8       // tiles per workgroup => 2048 keys per workgroup

struct qk_params {
  const void* q; int64_t qs_b, qs_h, qs_l;
  const void* k; int64_t ks_b, ks_h, ks_l;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int B, Hq, Hkv, Lq, Lk;
  void* keys_out; int64_t key_pitch;
};

template <int LPK>
__device__ __forceinline__ float sc_group_sum(float v) {
  v += sah_dpp<0xB1>(v);
  if (LPK >= 4) v += sah_dpp<0x4E>(v);
  if (LPK >= 8) v += sah_dpp<0x141>(v);
  if (LPK >= 16) v += sah_dpp<0x140>(v);
  return v;
}

template <int DT, int D>
__global__ __launch_bounds__(SC_NT) void k_qk_scores(qk_params P) {
  constexpr int LPK = D / 8;
  constexpr int KPI = SAH_WAVE / LPK;
  constexpr int IT = SAH_WAVE / KPI;
  constexpr int ES = (DT == SAH_F32) ? 4 : 2;
  typedef typename std::conditional<DT == SAH_F32, uint32_t, uint16_t>::type key_t;
  __shared__ key_t s_out[SC_NQ][SC_TILE];

  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = tid / SAH_WAVE;
  const int sub = lane % LPK;
  const int grp = lane / LPK;
  const int G = P.Hq / P.Hkv;
  const int bhk = blockIdx.y;
  const int hk = bhk % P.Hkv;
  const int b = bhk / P.Hkv;
  const int v0 = blockIdx.z * SC_NQ;  // first query vector (of G*Lq) handled here
  const int nvec = G * P.Lq;

  float qv[SC_NQ][8];
  int row[SC_NQ];
  int64_t moff[SC_NQ];
#pragma unroll
  for (int i = 0; i < SC_NQ; ++i) {
    const int v = v0 + i;
    row[i] = -1;
    moff[i] = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[i][e] = 0.f;
    if (v < nvec) {
      const int h = hk * G + v / P.Lq;
      const int qi = v % P.Lq;
      row[i] = (b * P.Hq + h) * P.Lq + qi;
      sah_load8<DT>(P.q, (int64_t)b * P.qs_b + (int64_t)h * P.qs_h + (int64_t)qi * P.qs_l + sub * 8, qv[i]);
      if (P.amask) moff[i] = (int64_t)b * P.ms_b + (int64_t)h * P.ms_h + (int64_t)qi * P.ms_l;
    }
  }
  const char* kbase = (const char*)P.k + ((int64_t)b * P.ks_b + (int64_t)hk * P.ks_h) * ES;

  for (int iter = 0; iter < SC_ITERS; ++iter) {
    const int j0 = (blockIdx.x * SC_ITERS + iter) * SC_TILE;
    if (j0 >= P.Lk) break;  // uniform across the workgroup
    float kv[IT][8];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int j = j0 + wave * SAH_WAVE + it * KPI + grp;
      if (j < P.Lk) {
        sah_load8<DT>(kbase + (int64_t)j * P.ks_l * ES, sub * 8, kv[it]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kv[it][e] = 0.f;
      }
    }
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int jl = wave * SAH_WAVE + it * KPI + grp;  // key within the tile
      const int j = j0 + jl;
#pragma unroll
      for (int i = 0; i < SC_NQ; ++i) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) d = fmaf(qv[i][e], kv[it][e], d);
        d = sc_group_sum<LPK>(d);
        if (sub == (i % LPK) && j < P.Lk && row[i] >= 0) {
          float s = sah_round<DT>(d);
          if (P.amask) s = sah_round<DT>(s + sah_load<DT>(P.amask, moff[i] + j));
          s_out[i][jl] = (key_t)sah_sort_key<DT>(s);
        }
      }
    }
    __syncthreads();
    int nk = P.Lk - j0;
    if (nk > SC_TILE) nk = SC_TILE;
#pragma unroll
    for (int i = 0; i < SC_NQ; ++i) {
      if (row[i] >= 0 && tid < nk) ((key_t*)P.keys_out)[(int64_t)row[i] * P.key_pitch + j0 + tid] = s_out[i][tid];
    }
    __syncthreads();
  }
}

template <int DT, int D>
static int qk_launch(const sah_qk_scores_args* a, const qk_params& P) {
  const int G = a->Hq / a->Hkv;
  const int nvec = G * a->Lq;
  dim3 g((a->Lk + SC_TILE * SC_ITERS - 1) / (SC_TILE * SC_ITERS), a->B * a->Hkv, (nvec + SC_NQ - 1) / SC_NQ);
  sah_timed timed("k_qk_scores", a->stream);
  hipLaunchKernelGGL((k_qk_scores<DT, D>), g, dim3(SC_NT), 0, (hipStream_t)a->stream, P);
  return sah_launch_status("sah_qk_scores");
}

template <int DT>
static int qk_dispatch_d(const sah_qk_scores_args* a, const qk_params& P) {
  switch (a->D) {
    case 16: return qk_launch<DT, 16>(a, P);
    case 32: return qk_launch<DT, 32>(a, P);
    case 64: return qk_launch<DT, 64>(a, P);
    case 128: return qk_launch<DT, 128>(a, P);
    default: return sah_fail(SAH_ESHAPE, "sah_qk_scores: head_dim %d not in {16,32,64,128}", a->D);
  }
}

extern "C" int sah_qk_scores(const sah_qk_scores_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_qk_scores: args is NULL");
  if (!a->q || !a->k || !a->keys_out) return sah_fail(SAH_ENULL, "sah_qk_scores: NULL tensor");
  if (a->B <= 0 || a->Hq <= 0 || a->Hkv <= 0 || a->Lq <= 0 || a->Lk <= 0 || a->Hq % a->Hkv)
    return sah_fail(SAH_EINVAL, "sah_qk_scores: bad dimensions");
  if (a->key_pitch < a->Lk) return sah_fail(SAH_EINVAL, "sah_qk_scores: key_pitch < Lk");
  const int es = a->dtype == SAH_F32 ? 4 : 2;
  if (a->qs_b % 8 || a->qs_h % 8 || a->qs_l % 8 || a->ks_b % 8 || a->ks_h % 8 || a->ks_l % 8)
    return sah_fail(SAH_ESHAPE, "sah_qk_scores: strides must be multiples of 8 elements");
  if (((uintptr_t)a->q | (uintptr_t)a->k) % (8 * es))
    return sah_fail(SAH_ESHAPE, "sah_qk_scores: q/k base pointers must be %d-byte aligned", 8 * es);
  if ((int64_t)a->B * a->Hkv > 65535) return sah_fail(SAH_ESHAPE, "sah_qk_scores: B*Hkv > 65535");
  qk_params P;
  P.q = a->q; P.qs_b = a->qs_b; P.qs_h = a->qs_h; P.qs_l = a->qs_l;
  P.k = a->k; P.ks_b = a->ks_b; P.ks_h = a->ks_h; P.ks_l = a->ks_l;
  P.amask = a->amask; P.ms_b = a->ms_b; P.ms_h = a->ms_h; P.ms_l = a->ms_l;
  P.B = a->B; P.Hq = a->Hq; P.Hkv = a->Hkv; P.Lq = a->Lq; P.Lk = a->Lk;
  P.keys_out = a->keys_out; P.key_pitch = a->key_pitch;
  switch (a->dtype) {
    case SAH_F32: return qk_dispatch_d<SAH_F32>(a, P);
    case SAH_BF16: return qk_dispatch_d<SAH_BF16>(a, P);
    case SAH_F16: return qk_dispatch_d<SAH_F16>(a, P);
    default: return sah_fail(SAH_EDTYPE, "sah_qk_scores: dtype %d", a->dtype);
  }
}
