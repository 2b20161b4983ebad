// Exact QK scoring pass of OracleTopK: one stream over K per KV head serves up
// to 4 query vectors of that head's GQA group (the 4 query heads in decode), no
// repeat_kv copy. HBM-bound: Lk * D * elem bytes per (b, kv head).
//
// Layout as in the attention kernel: LPK = D/8 lanes per key row, 8 elements
// (one 16 B / 32 B vector load) per lane, DPP reduction inside the lane group.
// The dot products go through an LDS tile; at the copy-out they are rounded to the
// storage type exactly where torch rounds them and leave as order-preserving
// unsigned keys, in coalesced writes.
#include "sah_common.h"

#define SC_NT 256
#define SC_NW (SC_NT / SAH_WAVE)
#define SC_NQ 4          // query vectors per workgroup
#define SC_TILE 256      // keys per workgroup iteration
#ifndef SC_MIN_WGS
#define SC_MIN_WGS 4096  // workgroups wanted before a workgroup takes more than one tile
#endif
#define SC_ITERS 2       // most tiles per workgroup; one when that would leave CUs without work

struct qk_params {
  const void* q; int64_t qs_b, qs_h, qs_l;
  const void* k; int64_t ks_b, ks_h, ks_l;
  const void* amask; int64_t ms_b, ms_h, ms_l;
  int B, Hq, Hkv, Lq, Lk;
  int d_real;  // head_dim; the kernel's D is d_real padded to a power of two
  void* keys_out; int64_t key_pitch;
  void* resid_out;  // RES: what the rounding of each score took away, same layout as keys_out
  int iters;  // tiles of SC_TILE keys per workgroup
};

template <int LPK>
__device__ __forceinline__ float sc_group_sum(float v) {
  v += sah_dpp<0xB1>(v);
  if (LPK >= 4) v += sah_dpp<0x4E>(v);
  if (LPK >= 8) v += sah_dpp<0x141>(v);
  if (LPK >= 16) v += sah_dpp<0x140>(v);
  return v;
}

// One key row slice as loaded: 8 elements of a lane, not yet widened.
template <int DT>
struct sc_raw {
  uint4 a;
};
template <>
struct sc_raw<SAH_F32> {
  float4 a, b;
};

template <int DT>
__device__ __forceinline__ void sc_load(const char* p, sc_raw<DT>& r) {
  if constexpr (DT == SAH_F32) {
    r.a = ((const float4*)p)[0];
    r.b = ((const float4*)p)[1];
  } else {
    r.a = *(const uint4*)p;
  }
}

// the K stream is read once per step: a load that does not displace what the caches hold
template <int DT>
__device__ __forceinline__ void sc_load_stream(const char* p, sc_raw<DT>& r) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  if constexpr (DT == SAH_F32) {
    const u4 a = __builtin_nontemporal_load((const u4*)p);
    const u4 b = __builtin_nontemporal_load((const u4*)p + 1);
    r.a = make_float4(sah_bits_to_float(a.x), sah_bits_to_float(a.y), sah_bits_to_float(a.z), sah_bits_to_float(a.w));
    r.b = make_float4(sah_bits_to_float(b.x), sah_bits_to_float(b.y), sah_bits_to_float(b.z), sah_bits_to_float(b.w));
  } else {
    const u4 a = __builtin_nontemporal_load((const u4*)p);
    r.a = make_uint4(a.x, a.y, a.z, a.w);
  }
}

template <int DT>
__device__ __forceinline__ void sc_keep(sc_raw<DT>& r) {
  if constexpr (DT == SAH_F32) {
    sah_keep(r.a.x); sah_keep(r.a.y); sah_keep(r.a.z); sah_keep(r.a.w);
    sah_keep(r.b.x); sah_keep(r.b.y); sah_keep(r.b.z); sah_keep(r.b.w);
  } else {
    sah_keep(r.a.x); sah_keep(r.a.y); sah_keep(r.a.z); sah_keep(r.a.w);
  }
}

// partial dot product of the lane's 8 elements
template <int DT>
__device__ __forceinline__ float sc_dot(const sc_raw<DT>& q, const sc_raw<DT>& k) {
  if constexpr (DT == SAH_F32) {
    float d = q.a.x * k.a.x;
    d = fmaf(q.a.y, k.a.y, d); d = fmaf(q.a.z, k.a.z, d); d = fmaf(q.a.w, k.a.w, d);
    d = fmaf(q.b.x, k.b.x, d); d = fmaf(q.b.y, k.b.y, d); d = fmaf(q.b.z, k.b.z, d); d = fmaf(q.b.w, k.b.w, d);
    return d;
  } else {
    float d = sah_dot2<DT>(q.a.x, k.a.x, 0.f);
    d = sah_dot2<DT>(q.a.y, k.a.y, d);
    d = sah_dot2<DT>(q.a.z, k.a.z, d);
    return sah_dot2<DT>(q.a.w, k.a.w, d);
  }
}

// Sums four per-lane partials (one per query vector) over the LPK lanes of a key, leaving in lane `sub` the
// total of query 2*(sub&1) + ((sub>>1)&1): each exchange step halves what a lane still carries, so the four
// reductions cost 3 adds inside the quad instead of 8, plus one add per doubling of the group beyond 4 lanes.
template <int LPK>
__device__ __forceinline__ float sc_reduce4(float d0, float d1, float d2, float d3, int sub) {
  static_assert(LPK >= 4, "needs at least a quad per key");
  const bool odd = sub & 1;
  float x0 = odd ? d2 : d0, x1 = odd ? d3 : d1;
  const float y0 = odd ? d0 : d2, y1 = odd ? d1 : d3;
  x0 += sah_dpp<0xB1>(y0);  // lane ^ 1
  x1 += sah_dpp<0xB1>(y1);
  const bool up = sub & 2;
  float z = up ? x1 : x0;
  const float t = up ? x0 : x1;
  z += sah_dpp<0x4E>(t);    // lane ^ 2
  if (LPK == 8) z += __shfl_xor(z, 4);
  if (LPK == 16) {
    z += sah_dpp<0x124>(z);  // row_ror:4  (rotations keep the position inside the quad)
    z += sah_dpp<0x128>(z);  // row_ror:8
  }
  return z;
}

// AM: an additive attention mask is given (P.amask); without one the scoring loop holds no load but the rows'
// FULL: head_dim is D itself; otherwise D is head_dim padded to a power of two: the lanes of a key beyond head_dim
// carry a zero query slice (and re-read the row's first slice, so that no load sits behind a condition)
// RES: the remainder of every score's rounding goes out beside its key (16-bit types, no mask)
template <int DT, int D, bool AM, bool FULL, bool RES = false>
__global__ __launch_bounds__(SC_NT) void k_qk_scores(qk_params P) {
  sah_touch_kernargs<sizeof(qk_params)>();
  constexpr int LPK = D / 8;
  constexpr int KPI = SAH_WAVE / LPK;
  constexpr int IT = SAH_WAVE / KPI;
  constexpr int ES = (DT == SAH_F32) ? 4 : 2;
  constexpr bool FAST4 = LPK >= 4;  // transposing reduction of all four query vectors at once
  typedef typename std::conditional<DT == SAH_F32, uint32_t, uint16_t>::type key_t;
  // The tile holds the dot products as they come out of the reduction (fp32); rounding, key and remainder are made
  // at the copy-out, where every lane has one score per query vector - in the scoring loop only the few lanes that
  // end up with a total would work on them.
  __shared__ float s_out[SC_NQ][SC_TILE];
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  const int sub = lane % LPK;
  const int grp = lane / LPK;
  const int G = P.Hq / P.Hkv;
  const int bhk = blockIdx.y;
  const int hk = bhk % P.Hkv;
  const int b = bhk / P.Hkv;
  const int v0 = blockIdx.z * SC_NQ;  // first query vector (of G*Lq) handled here
  const int nvec = G * P.Lq;
  const bool in_dim = FULL || sub * 8 < P.d_real;
  const int sub_k = in_dim ? sub : 0;

  sc_raw<DT> qv[SC_NQ];
  int row[SC_NQ];
  int64_t moff[SC_NQ];
#pragma unroll
  for (int i = 0; i < SC_NQ; ++i) {
    int v = v0 + i;
    moff[i] = 0;
    // a slot beyond the group's query vectors repeats the last one: it computes and writes the same keys again
    if (v >= nvec) v = nvec - 1;
    const int h = hk * G + v / P.Lq;
    const int qi = v % P.Lq;
    sc_load<DT>((const char*)P.q + ((int64_t)b * P.qs_b + (int64_t)h * P.qs_h + (int64_t)qi * P.qs_l + sub_k * 8) * ES, qv[i]);
    if (!FULL && !in_dim) {
      if constexpr (DT == SAH_F32) {
        qv[i].a = make_float4(0.f, 0.f, 0.f, 0.f);
        qv[i].b = make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        qv[i].a = make_uint4(0u, 0u, 0u, 0u);
      }
    }
    row[i] = (b * P.Hq + h) * P.Lq + qi;
    if (AM) moff[i] = (int64_t)b * P.ms_b + (int64_t)h * P.ms_h + (int64_t)qi * P.ms_l;
  }
  const char* kbase = (const char*)P.k + ((int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + sub_k * 8) * ES;
  const int64_t krow = P.ks_l * ES;
  // which of the four totals this lane ends up with after sc_reduce4
  const int mine = FAST4 ? (2 * (sub & 1) + ((sub >> 1) & 1)) : 0;

  // A wave owns 64 consecutive keys of every tile and the matching columns of s_out: no workgroup
  // barrier anywhere. The rows come in half-slices of HB iterations through two register buffers;
  // the next half-slice is requested before the current one is scored, so every wave keeps
  // HB..2*HB row loads in flight all the time instead of alternating between loading and computing.
  // iterations per part of a wave's 64-key slice: half of it, a quarter for fp32 rows (twice the registers)
  constexpr int HB = (DT == SAH_F32 && IT >= 4) ? IT / 4 : (IT >= 2 ? IT / 2 : 1);
  constexpr int NH = IT / HB;                // parts per tile
  const int tile0 = blockIdx.x * P.iters;
  int n_tiles = (P.Lk - tile0 * SC_TILE + SC_TILE - 1) / SC_TILE;
  if (n_tiles > P.iters) n_tiles = P.iters;
  if (n_tiles <= 0) return;
  const int n_half = n_tiles * NH;
  auto request = [&](sc_raw<DT> (&buf)[HB], int hs) {
    const int j0 = (tile0 + hs / NH) * SC_TILE + wave * SAH_WAVE + (hs % NH) * HB * KPI;
#pragma unroll
    for (int it = 0; it < HB; ++it) {
      int j = j0 + it * KPI + grp;
      if (j > P.Lk - 1) j = P.Lk - 1;  // rows past the end re-read the last row
      sc_load_stream<DT>(kbase + (int64_t)j * krow, buf[it]);
    }
  };
  auto score = [&](sc_raw<DT> (&buf)[HB], int hs) {
    const int tile = tile0 + hs / NH;
    const int jl0 = wave * SAH_WAVE + (hs % NH) * HB * KPI;  // first key of the half-slice within the tile
#pragma unroll
    for (int it = 0; it < HB; ++it) sc_keep<DT>(buf[it]);
#pragma unroll
    for (int it = 0; it < HB; ++it) {
      const int jl = jl0 + it * KPI + grp;
      if constexpr (FAST4) {
        const float d = sc_reduce4<LPK>(sc_dot<DT>(qv[0], buf[it]), sc_dot<DT>(qv[1], buf[it]), sc_dot<DT>(qv[2], buf[it]),
                                         sc_dot<DT>(qv[3], buf[it]), sub);
        // keys past the row's end and dead query vectors park a value that the copy-out below never stores
        if (sub < 4) s_out[mine][jl] = d;
      } else {
#pragma unroll
        for (int i = 0; i < SC_NQ; ++i) {
          const float d = sc_group_sum<LPK>(sc_dot<DT>(qv[i], buf[it]));
          if (sub == (i % LPK)) s_out[i][jl] = d;
        }
      }
    }
    if (hs % NH == NH - 1) {
      // The wave's 64 keys of this tile are scored: write them out, one key per lane and query vector. No store
      // sits behind a condition (a lane past the row's end has scored the last key again, and writes it again): after
      // a store that may or may not have been issued, the compiler's waits for the row loads in flight are the
      // stricter of the two cases, and the two register buffers no longer overlap.
      sah_wave_lds_sync();
      int j = tile * SC_TILE + wave * SAH_WAVE + lane;
      if (j > P.Lk - 1) j = P.Lk - 1;
#pragma unroll
      for (int i = 0; i < SC_NQ; ++i) {
        const float d = s_out[i][wave * SAH_WAVE + lane];
        float s = sah_round<DT>(d);
        if (AM) s = sah_round<DT>(s + sah_load<DT>(P.amask, moff[i] + j));
        ((key_t*)P.keys_out)[(int64_t)row[i] * P.key_pitch + j] = (key_t)sah_sort_key<DT>(s);
        if constexpr (RES) {
          // the remainder of the rounding in DT's own bits (bf16: cut off, not rounded - it is a correction of a
          // correction; a score that rounds to infinity leaves none)
          const float rem = d - s;
          uint16_t rb;
          if (DT == SAH_BF16) rb = (uint16_t)(sah_float_to_bits(rem) >> 16);
          else rb = fabsf(s) < INFINITY ? (uint16_t)sah_float_to_f16(rem) : (uint16_t)0;
          ((uint16_t*)P.resid_out)[(int64_t)row[i] * P.key_pitch + j] = rb;
        }
      }
      sah_wave_lds_sync();  // the columns are free again for the next tile
    }
  };
  // No request of the steady state sits behind a condition: where a path with and a path without a request meet,
  // the compiler's wait for the buffer about to be scored is the stricter of the two, i.e. it also waits for the
  // loads just issued and the two buffers no longer overlap. The last one or two parts are a copy of their own.
  sc_raw<DT> ka[HB], kb[HB];
  request(ka, 0);
  int hs = 0;
  for (; hs + 2 < n_half; hs += 2) {
    request(kb, hs + 1);
    score(ka, hs);
    request(ka, hs + 2);
    score(kb, hs + 1);
  }
  if (hs + 1 < n_half) {
    request(kb, hs + 1);
    score(ka, hs);
    score(kb, hs + 1);
  } else {
    score(ka, hs);
  }
}

template <int DT, int D, bool FULL>
static int qk_launch(const sah_qk_scores_args* a, const qk_params& P) {
  const int G = a->Hq / a->Hkv;
  const int nvec = G * a->Lq;
  // enough workgroups for several waves per SIMD on all 256 CUs, as long as a workgroup keeps at least one tile
  const int64_t tiles = (a->Lk + SC_TILE - 1) / SC_TILE;
  const int64_t streams = (int64_t)a->B * a->Hkv * ((nvec + SC_NQ - 1) / SC_NQ);
  int iters = SC_ITERS;
  while (iters > 1 && streams * ((tiles + iters - 1) / iters) < SC_MIN_WGS) iters >>= 1;
  qk_params Q = P;
  Q.iters = iters;
  dim3 g((unsigned)((tiles + iters - 1) / iters), a->B * a->Hkv, (nvec + SC_NQ - 1) / SC_NQ);
  sah_timed timed("k_qk_scores", a->stream);
  constexpr bool CAN_RES = DT != SAH_F32 && FULL && (D == 64 || D == 128);
  if (a->amask) hipLaunchKernelGGL((k_qk_scores<DT, D, true, FULL>), g, dim3(SC_NT), 0, (hipStream_t)a->stream, Q);
  else if (CAN_RES && a->resid_out) hipLaunchKernelGGL((k_qk_scores<DT, D, false, FULL, CAN_RES>), g, dim3(SC_NT), 0, (hipStream_t)a->stream, Q);
  else hipLaunchKernelGGL((k_qk_scores<DT, D, false, FULL>), g, dim3(SC_NT), 0, (hipStream_t)a->stream, Q);
  return sah_launch_status("sah_qk_scores");
}

template <int DT>
static int qk_dispatch_d(const sah_qk_scores_args* a, const qk_params& P) {
  switch (a->D) {
    case 16: return qk_launch<DT, 16, true>(a, P);
    case 32: return qk_launch<DT, 32, true>(a, P);
    case 64: return qk_launch<DT, 64, true>(a, P);
    case 128: return qk_launch<DT, 128, true>(a, P);
    default: break;
  }
  // any other multiple of 8 below 128: the next power of two, the lanes beyond head_dim multiply zeros
  if (a->D <= 0 || a->D % 8 || a->D > 128)
    return sah_fail(SAH_ESHAPE, "sah_qk_scores: head_dim %d is not a multiple of 8 in [8, 128]", a->D);
  if (a->D < 16) return qk_launch<DT, 16, false>(a, P);
  if (a->D < 32) return qk_launch<DT, 32, false>(a, P);
  if (a->D < 64) return qk_launch<DT, 64, false>(a, P);
  return qk_launch<DT, 128, false>(a, P);
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
  P.d_real = a->D;
  P.keys_out = a->keys_out; P.key_pitch = a->key_pitch;
  P.resid_out = a->resid_out;
  if (a->resid_out && (a->amask || a->dtype == SAH_F32 || (a->D != 64 && a->D != 128)))
    return sah_fail(SAH_EINVAL, "sah_qk_scores: resid_out needs a 16-bit dtype, head_dim 64 or 128 and no additive mask");
  switch (a->dtype) {
    case SAH_F32: return qk_dispatch_d<SAH_F32>(a, P);
    case SAH_BF16: return qk_dispatch_d<SAH_BF16>(a, P);
    case SAH_F16: return qk_dispatch_d<SAH_F16>(a, P);
    default: return sah_fail(SAH_EDTYPE, "sah_qk_scores: dtype %d", a->dtype);
  }
}
