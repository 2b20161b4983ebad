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

#define SIG_NT 128
#define SIG_TL 16        // vectors per tile
#define SIG_MAXD 256     // widest layer supported

struct sig_params {
  const void* x; int64_t xs_b, xs_h, xs_l;
  int B, Hq, group, L, D;
  int n_layers;
  const void* W[SAH_MAX_MLP_LAYERS];
  const void* bias[SAH_MAX_MLP_LAYERS];
  int d_out[SAH_MAX_MLP_LAYERS];
  int act;
  uint32_t* codes; int64_t code_pitch, code_offset;
};

__device__ __forceinline__ float sig_act(int act, float v) {
  switch (act) {
    case SAH_ACT_RELU: return v > 0.f ? v : 0.f;
    case SAH_ACT_SILU: return v / (1.0f + expf(-v));
    case SAH_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    default: return tanhf(v);
  }
}

// 8 weights of one row as loaded: 16 B for 2-byte types, 32 B for fp32
template <int DT>
struct att_raw_w {
  uint4 lo;
  uint4 hi;
  __device__ __forceinline__ void load(const char* p) {
    lo = *(const uint4*)p;
    if (DT == SAH_F32) hi = *(const uint4*)(p + 16);
  }
  __device__ __forceinline__ void unpack(float (&o)[8]) const {
    const uint32_t w[4] = {lo.x, lo.y, lo.z, lo.w};
    if (DT == SAH_F32) {
      const uint32_t v[4] = {hi.x, hi.y, hi.z, hi.w};
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
};

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

// ---------------------------------------------------------------------------
// Decode path: a handful of vectors per head (one new key, one query). One
// workgroup per (b, h, group of up to GV vectors); the layer matrix W[h] (d_in x
// d_out, row-major) is read once with 16-byte loads: thread t owns 8 adjacent
// output columns (cg = t % CG) of the rows d = rg, rg + RG, ... (rg = t / CG), all
// of its row loads are in flight together, and the RG partial sums are reduced by
// wave shuffles and one pass through LDS. With 2-byte weights every layer is requested
// up-front (the weights do not depend on the activations): one memory round trip in all.
// Needs every layer width to be a power of two in [8, 256] and D % 8 == 0.
// ---------------------------------------------------------------------------
#define GEMV_NT 256
#define GEMV_NW (GEMV_NT / SAH_WAVE)
#define GEMV_GV 4


struct sig_pair {
  sig_params p[2];
};

#define GEMV_ROWS 8  // row slots per thread and layer (d_in * d_out / 8 / GEMV_NT <= 8)

// One layer: acc[t][e] = sum over this thread's row slots of x[t][d] * W[d][8 columns].
// Slots beyond the thread's real row count hold a clamped (valid) row and get weight 0.
template <int DT, int GV>
__device__ __forceinline__ void gemv_layer_fma(const att_raw_w<DT> (&raw)[GEMV_ROWS], int nrow, int rg, int RG,
                                               const float (*s_x)[SIG_MAXD], float (&acc)[GV][8]) {
#pragma unroll
  for (int i = 0; i < GEMV_ROWS; ++i) {
    float wv[8];
    raw[i].unpack(wv);
    const int d = rg + (i < nrow ? i : 0) * RG;
#pragma unroll
    for (int t = 0; t < GV; ++t) {
      const float xv = (i < nrow) ? s_x[t][d] : 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[t][e] = fmaf(xv, wv[e], acc[t][e]);
    }
  }
}

template <int DT, int GV>
__global__ __launch_bounds__(GEMV_NT) void k_hash_sig_gemv(sig_pair PP) {
  const sig_params& P = PP.p[blockIdx.z];
  if ((int)blockIdx.x * GV >= P.L) return;  // the two jobs may differ in vector count
  __shared__ float s_x[GV][SIG_MAXD];
  __shared__ float s_part[GEMV_NW][GV][SIG_MAXD];
  __shared__ float s_bias[SAH_MAX_MLP_LAYERS][SIG_MAXD];
  constexpr int ES = (DT == SAH_F32) ? 4 : 2;
  // fp32 weights are 32 B per row slot: prefetching every layer would not fit the registers
  constexpr int PF = (DT == SAH_F32) ? 1 : SAH_MAX_MLP_LAYERS;
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = tid / SAH_WAVE;
  const int bh = blockIdx.y;
  const int h = bh % P.Hq;
  const int b = bh / P.Hq;
  const int hx = h / P.group;
  const int l0 = blockIdx.x * GV;
  int nl = P.L - l0;
  if (nl > GV) nl = GV;

  // The weights do not depend on the activations: request every layer's rows (and biases)
  // now, so the three layers cost one memory round trip instead of three.
  att_raw_w<DT> raw[PF][GEMV_ROWS];
  auto fetch_layer = [&](int layer, int din, att_raw_w<DT> (&dst)[GEMV_ROWS]) {
    const int dout = P.d_out[layer];
    const int CG = dout / 8, RG = GEMV_NT / CG;
    const int cg = tid % CG, rg = tid / CG;
    const int nrow = din / RG;
    const char* wbase = (const char*)P.W[layer] + ((int64_t)h * din * dout + cg * 8) * ES;
#pragma unroll
    for (int i = 0; i < GEMV_ROWS; ++i) {
      const int d = rg + (i < nrow ? i : 0) * RG;
      dst[i].load(wbase + (int64_t)d * dout * ES);
    }
    if (tid < dout) s_bias[layer][tid] = sah_load<DT>(P.bias[layer], (int64_t)h * dout + tid);
  };
  if (PF > 1) {
    int din0 = P.D;
#pragma unroll
    for (int layer = 0; layer < PF; ++layer) {
      if (layer < P.n_layers) {
        fetch_layer(layer, din0, raw[layer]);
        din0 = P.d_out[layer];
      }
    }
  }

  for (int i = tid; i < GV * P.D; i += GEMV_NT) {
    const int t = i / P.D, d = i % P.D;
    float v = 0.f;
    if (t < nl) v = sah_load<DT>(P.x, (int64_t)b * P.xs_b + (int64_t)hx * P.xs_h + (int64_t)(l0 + t) * P.xs_l + d);
    s_x[t][d] = v;
  }
  __syncthreads();

  int din = P.D;
#pragma unroll
  for (int layer = 0; layer < SAH_MAX_MLP_LAYERS; ++layer) {
    if (layer >= P.n_layers) break;
    const int dout = P.d_out[layer];
    const bool last = (layer == P.n_layers - 1);
    const int CG = dout / 8;            // column groups (power of two, <= 32)
    const int RG = GEMV_NT / CG;        // row groups
    const int cg = tid % CG, rg = tid / CG;
    const int nrow = din / RG;          // real rows of this thread: 1, 2, 4 or 8
    float acc[GV][8];
#pragma unroll
    for (int t = 0; t < GV; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[t][e] = 0.f;
    if (PF > 1) {
      gemv_layer_fma<DT, GV>(raw[layer < PF ? layer : 0], nrow, rg, RG, s_x, acc);
    } else {
      fetch_layer(layer, din, raw[0]);
      gemv_layer_fma<DT, GV>(raw[0], nrow, rg, RG, s_x, acc);
    }
    // lanes of a wave that share cg differ by multiples of CG
    for (int o = CG; o < SAH_WAVE; o <<= 1) {
#pragma unroll
      for (int t = 0; t < GV; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[t][e] += __shfl_xor(acc[t][e], o);
    }
    if (lane < CG) {
#pragma unroll
      for (int t = 0; t < GV; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) s_part[wave][t][cg * 8 + e] = acc[t][e];
    }
    __syncthreads();
    // dout <= 256 => CG <= 32 < 64, so every wave holds all column groups
    for (int i = tid; i < GV * dout; i += GEMV_NT) {
      const int t = i / dout, e = i % dout;
      float y = 0.f;
#pragma unroll
      for (int wv2 = 0; wv2 < GEMV_NW; ++wv2) y += s_part[wv2][t][e];
      y = sah_round<DT>(y);
      y = sah_round<DT>(y + s_bias[layer][e]);
      if (!last) y = sah_round<DT>(sig_act(P.act, y));
      s_x[t][e] = y;
    }
    __syncthreads();
    din = dout;
  }

  if (tid < SAH_WAVE) {
    const int bits = din;
    for (int t = 0; t < nl; ++t) {
      const float y = (tid < bits) ? s_x[t][tid] : 0.f;
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

static bool sig_gemv_ok(const sah_hash_sig_args* a) {
  if (a->L > 64 || a->D % 8 || a->D > SIG_MAXD) return false;
  int din = a->D;
  for (int i = 0; i < a->n_layers; ++i) {
    const int dout = a->d_out[i];
    if (dout < 8 || dout > 256 || (dout & (dout - 1))) return false;
    const int rows_per_thread = (int)((int64_t)din * dout / (8 * GEMV_NT));
    if ((int64_t)din * dout % (8 * GEMV_NT) || (rows_per_thread != 1 && rows_per_thread != 2 && rows_per_thread != 4 &&
                                                 rows_per_thread != 8))
      return false;
    const int es = a->dtype == SAH_F32 ? 4 : 2;
    if (((uintptr_t)a->W[i]) % (8 * es)) return false;
    din = dout;
  }
  return true;
}

static int sig_validate(const sah_hash_sig_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hash_signatures: args is NULL");
  if (!a->x || !a->codes) return sah_fail(SAH_ENULL, "sah_hash_signatures: x / codes is NULL");
  if (a->B <= 0 || a->Hq <= 0 || a->group <= 0 || a->D <= 0 || a->Hq % a->group)
    return sah_fail(SAH_EINVAL, "sah_hash_signatures: bad B/Hq/group/D");
  if (a->n_layers < 1 || a->n_layers > SAH_MAX_MLP_LAYERS)
    return sah_fail(SAH_ESHAPE, "sah_hash_signatures: n_layers %d not in [1, %d]", a->n_layers, SAH_MAX_MLP_LAYERS);
  if (a->D > SIG_MAXD) return sah_fail(SAH_ESHAPE, "sah_hash_signatures: D %d > %d", a->D, SIG_MAXD);
  for (int i = 0; i < a->n_layers; ++i) {
    if (!a->W[i] || !a->bias[i]) return sah_fail(SAH_ENULL, "sah_hash_signatures: layer %d weights are NULL", i);
    if (a->d_out[i] <= 0 || a->d_out[i] > SIG_MAXD)
      return sah_fail(SAH_ESHAPE, "sah_hash_signatures: layer %d width %d not in [1, %d]", i, a->d_out[i], SIG_MAXD);
  }
  if (a->d_out[a->n_layers - 1] > 32)
    return sah_fail(SAH_ESHAPE, "sah_hash_signatures: %d signature bits do not fit one 32-bit plane", a->d_out[a->n_layers - 1]);
  if (a->act < SAH_ACT_RELU || a->act > SAH_ACT_TANH) return sah_fail(SAH_EINVAL, "sah_hash_signatures: activation %d", a->act);
  if (a->L > 0 && a->code_pitch < a->code_offset + a->L) return sah_fail(SAH_ECAPACITY, "sah_hash_signatures: code_pitch too small");
  if ((int64_t)a->B * a->Hq > 65535) return sah_fail(SAH_ESHAPE, "sah_hash_signatures: B*Hq > 65535");
  if (a->dtype != SAH_F32 && a->dtype != SAH_BF16 && a->dtype != SAH_F16) return sah_fail(SAH_EDTYPE, "sah_hash_signatures: dtype %d", a->dtype);
  return SAH_OK;
}

static void sig_fill(const sah_hash_sig_args* a, sig_params& P) {
  P.x = a->x; P.xs_b = a->xs_b; P.xs_h = a->xs_h; P.xs_l = a->xs_l;
  P.B = a->B; P.Hq = a->Hq; P.group = a->group; P.L = a->L; P.D = a->D;
  P.n_layers = a->n_layers;
  for (int i = 0; i < SAH_MAX_MLP_LAYERS; ++i) {
    P.W[i] = a->W[i]; P.bias[i] = a->bias[i]; P.d_out[i] = a->d_out[i];
  }
  P.act = a->act;
  P.codes = a->codes; P.code_pitch = a->code_pitch; P.code_offset = a->code_offset;
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
  if (sig_gemv_ok(a)) return sig_launch_gemv(a, nullptr);
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
  if (a->L > 0 && b->L > 0 && sig_gemv_ok(a) && sig_gemv_ok(b) && a->dtype == b->dtype && a->stream == b->stream &&
      (int64_t)a->B * a->Hq == (int64_t)b->B * b->Hq)
    return sig_launch_gemv(a, b);
  rc = sig_launch_one(a);
  if (rc) return rc;
  return sig_launch_one(b);
}
