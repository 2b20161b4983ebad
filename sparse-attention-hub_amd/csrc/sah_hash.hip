// HashAttention bit signatures: per query head a small MLP (D -> hidden ... ->
// bits) followed by sign(), packed LSB-first into two uint32 planes per vector:
// "positive" and "non-zero" (in bf16 an exact zero is not rare, and the reference
// scores such a bit as 0, so it has to be representable).
//
// k_hash_sig_tile: one workgroup per (b, h, tile of TL vectors). The tile lives
// in LDS as fp32; thread e owns output feature e and streams W[h][:, e] (coalesced
// across threads) once per tile, so weight traffic is amortised over TL vectors.
// Rounding follows torch op by op when the storage type is 16-bit: the layer
// output, the bias add and the activation are each rounded to that type.
#include "sah_common.h"
#include "sah_sig.h"

#define SIG_NT 128
#define SIG_TL 16        // vectors per tile

template <int DT>
__global__ __launch_bounds__(SIG_NT) void k_hash_sig_tile(sig_params P) {
  __shared__ float s_a[SIG_TL][SIG_MAXD];
  __shared__ float s_b[SIG_TL][SIG_MAXD];
  const int tid = threadIdx.x;
  const int tile = blockIdx.x;
  const int bh = blockIdx.y;
  const int h = bh % P.Hq;
  const int b = bh / P.Hq;
  const int hx = h / P.group;
  const int l0 = tile * SIG_TL;
  int nl = P.L - l0;
  if (nl > SIG_TL) nl = SIG_TL;

  // stage the tile (zero rows beyond nl keep the arithmetic finite)
  for (int i = tid; i < SIG_TL * P.D; i += SIG_NT) {
    const int t = i / P.D, d = i % P.D;
    float v = 0.f;
    if (t < nl) v = sah_load<DT>(P.x, (int64_t)b * P.xs_b + (int64_t)hx * P.xs_h + (int64_t)(l0 + t) * P.xs_l + d);
    s_a[t][d] = v;
  }
  __syncthreads();

  float (*cur)[SIG_MAXD] = s_a;
  float (*nxt)[SIG_MAXD] = s_b;
  int din = P.D;
  for (int layer = 0; layer < P.n_layers; ++layer) {
    const int dout = P.d_out[layer];
    const bool last = (layer == P.n_layers - 1);
    const int64_t wbase = (int64_t)h * din * dout;
    for (int e = tid; e < dout; e += SIG_NT) {
      float acc[SIG_TL];
#pragma unroll
      for (int t = 0; t < SIG_TL; ++t) acc[t] = 0.f;
      for (int d = 0; d < din; ++d) {
        const float wv = sah_load<DT>(P.W[layer], wbase + (int64_t)d * dout + e);
#pragma unroll
        for (int t = 0; t < SIG_TL; ++t) acc[t] = fmaf(cur[t][d], wv, acc[t]);
      }
      const float bv = sah_load<DT>(P.bias[layer], (int64_t)h * dout + e);
#pragma unroll
      for (int t = 0; t < SIG_TL; ++t) {
        float y = sah_round<DT>(acc[t]);
        y = sah_round<DT>(y + bv);
        if (!last) y = sah_round<DT>(sig_act(P.act, y));
        nxt[t][e] = y;
      }
    }
    __syncthreads();
    float (*tmp)[SIG_MAXD] = cur;
    cur = nxt;
    nxt = tmp;
    din = dout;
  }

  // pack two planes per vector: bit e of .x = (y_e > 0), bit e of .y = (y_e != 0);
  // the first wave ballots one vector at a time
  if (tid < SAH_WAVE) {
    const int bits = din;  // <= 32, checked on the host
    for (int t = 0; t < nl; ++t) {
      const float y = (tid < bits) ? cur[t][tid] : 0.f;
      const uint64_t pos = __ballot(y > 0.f);
      const uint64_t nz = __ballot(y != 0.f);
      if (tid == 0) {
        uint2 c;
        c.x = (uint32_t)pos;
        c.y = (uint32_t)nz;
        ((uint2*)P.codes)[(int64_t)bh * P.code_pitch + P.code_offset + l0 + t] = c;
      }
    }
  }
}

#define GEMV_NT 512
#define GEMV_GV 4
#define GEMV_ROWS 4  // row slots per thread and layer (d_in * d_out / 8 / GEMV_NT <= 4)

struct sig_pair {
  sig_params p[2];
};

template <int DT, int GV>
__global__ __launch_bounds__(GEMV_NT) void k_hash_sig_gemv(sig_pair PP) {
  const sig_params& P = PP.p[blockIdx.z];
  if ((int)blockIdx.x * GV >= P.L) return;  // the two jobs may differ in vector count
  __shared__ sig_gemv_lds<GV, GEMV_NT> S;
  // fp32 weights are 32 B per row slot: prefetching every layer would not fit the registers
  constexpr int PF = (DT == SAH_F32) ? 1 : SAH_MAX_MLP_LAYERS;
  const int bh = blockIdx.y;
  const int l0 = blockIdx.x * GV;
  int nl = P.L - l0;
  if (nl > GV) nl = GV;
  sig_gemv_block<DT, GV, GEMV_NT, GEMV_ROWS, PF>(P, true, threadIdx.x, bh / P.Hq, bh % P.Hq, l0, nl, P.n_layers, S);
}

static int sig_launch_gemv(const sah_hash_sig_args* a, const sah_hash_sig_args* b2) {
  sig_pair PP;
  sig_fill(a, PP.p[0]);
  sig_fill(b2 ? b2 : a, PP.p[1]);
  const int maxL = (b2 && b2->L > a->L) ? b2->L : a->L;
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_hash_sig_gemv", a->stream);
  dim3 gb(GEMV_NT);
  if (maxL == 1) {  // decode: one vector per head and job
    dim3 gg(1, a->B * a->Hq, b2 ? 2 : 1);
    switch (a->dtype) {
      case SAH_F32: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_F32, 1>), gg, gb, 0, st, PP); break;
      case SAH_BF16: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_BF16, 1>), gg, gb, 0, st, PP); break;
      default: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_F16, 1>), gg, gb, 0, st, PP); break;
    }
  } else {
    dim3 gg((maxL + GEMV_GV - 1) / GEMV_GV, a->B * a->Hq, b2 ? 2 : 1);
    switch (a->dtype) {
      case SAH_F32: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_F32, GEMV_GV>), gg, gb, 0, st, PP); break;
      case SAH_BF16: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_BF16, GEMV_GV>), gg, gb, 0, st, PP); break;
      default: hipLaunchKernelGGL((k_hash_sig_gemv<SAH_F16, GEMV_GV>), gg, gb, 0, st, PP); break;
    }
  }
  return sah_launch_status("sah_hash_signatures");
}

static int sig_launch_one(const sah_hash_sig_args* a) {
  if (a->L <= 0) return SAH_OK;  // nothing to hash
  if (sig_gemv_ok(a, GEMV_NT, GEMV_ROWS)) return sig_launch_gemv(a, nullptr);
  sig_params P;
  sig_fill(a, P);
  dim3 g((a->L + SIG_TL - 1) / SIG_TL, a->B * a->Hq), b(SIG_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_hash_sig_tile", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_hash_sig_tile<SAH_F32>, g, b, 0, st, P); break;
    case SAH_BF16: hipLaunchKernelGGL(k_hash_sig_tile<SAH_BF16>, g, b, 0, st, P); break;
    default: hipLaunchKernelGGL(k_hash_sig_tile<SAH_F16>, g, b, 0, st, P); break;
  }
  return sah_launch_status("sah_hash_signatures");
}

extern "C" int sah_hash_signatures(const sah_hash_sig_args* a) {
  int rc = sig_validate(a);
  if (rc) return rc;
  return sig_launch_one(a);
}

// Two independent signature jobs (typically: the new keys of a decode step and its
// queries) in one launch when both are small; otherwise one launch each.
extern "C" int sah_hash_signatures_pair(const sah_hash_sig_args* a, const sah_hash_sig_args* b) {
  int rc = sig_validate(a);
  if (rc) return rc;
  rc = sig_validate(b);
  if (rc) return rc;
  if (a->L > 0 && b->L > 0 && sig_gemv_ok(a, GEMV_NT, GEMV_ROWS) && sig_gemv_ok(b, GEMV_NT, GEMV_ROWS) && a->dtype == b->dtype && a->stream == b->stream &&
      (int64_t)a->B * a->Hq == (int64_t)b->B * b->Hq)
    return sig_launch_gemv(a, b);
  rc = sig_launch_one(a);
  if (rc) return rc;
  return sig_launch_one(b);
}
