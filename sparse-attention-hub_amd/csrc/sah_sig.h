// Signature MLP of HashAttention: parameter block, activation, and the block-level GEMV used by the
// decode kernels (stand-alone and fused with the top-k selection).
#pragma once
#include "sah_common.h"

#define SIG_MAXD 256     // widest layer supported

struct sig_params {
  const void* x; int64_t xs_b, xs_h, xs_l;
  int B, Hq, group, L, D;
  int n_layers;
  const void* W[SAH_MAX_MLP_LAYERS];
  const void* bias[SAH_MAX_MLP_LAYERS];
  const void* Wt[SAH_MAX_MLP_LAYERS];
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

// The activations with the hardware exponential and reciprocal: for the bulk kernel, whose results are
// rounded to a 16-bit type right after (relative error ~1e-6 against 4e-3 of a bf16 step).
__device__ __forceinline__ float sig_act_fast(int act, float v) {
  switch (act) {
    case SAH_ACT_RELU: return v > 0.f ? v : 0.f;
    case SAH_ACT_SILU: return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    case SAH_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    default: {
      const float e = __expf(-2.0f * fabsf(v));  // tanh |v| = (1 - e) / (1 + e)
      const float t = (1.0f - e) * __builtin_amdgcn_rcpf(1.0f + e);
      return v < 0.f ? -t : t;
    }
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


// ---------------------------------------------------------------------------
// Decode path: a handful of vectors per head (one new key, one query). A group of NT threads handles
// (b, h, up to GV vectors); the layer matrix W[h] (d_in x d_out, row-major) is read once with 16-byte
// loads: thread t owns 8 adjacent output columns (cg = t % CG) of the rows d = rg, rg + RG, ...
// (rg = t / CG), all of its row loads are in flight together, and the RG partial sums are reduced by
// wave shuffles and one pass through LDS. With PF == SAH_MAX_MLP_LAYERS every layer is requested
// up-front (the weights do not depend on the activations): one memory round trip in all.
// Needs every layer width to be a power of two in [8, 256], D % 8 == 0 and
// d_in * d_out / (8 * NT) in {1, 2, 4, ..., ROWS} for every layer.
// ---------------------------------------------------------------------------
template <int GV, int NT>
struct sig_gemv_lds {
  float x[GV][SIG_MAXD];
  float part[NT / SAH_WAVE][GV][SIG_MAXD];
  float bias[SAH_MAX_MLP_LAYERS][SIG_MAXD];
  uint2 code[GV];
};

// One layer: acc[t][e] = sum over this thread's row slots of x[t][d] * W[d][8 columns].
// Slots beyond the thread's real row count hold a clamped (valid) row and get weight 0.
template <int DT, int GV, int ROWS>
__device__ __forceinline__ void gemv_layer_fma(const att_raw_w<DT> (&raw)[ROWS], int nrow, int rg, int RG,
                                               const float (*s_x)[SIG_MAXD], float (&acc)[GV][8]) {
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
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

// The MLP for vectors l0 .. l0 + nl - 1 of head (b, h), run by the NT threads of a group (`tid` = index
// in the group, the group is a whole number of waves). Every thread of the workgroup must call it, because
// it contains workgroup barriers (2 + 2 * n_layers of them): threads outside any group pass active = false
// and only take the barriers. The packed codes land in S.code[t] (valid on return)
// and, when P.codes is not NULL, in the code stream.
struct sig_no_hook {
  __device__ __forceinline__ void operator()() const {}
};

// `after_requests` runs once every load of the MLP has been requested and before the first result is waited
// for: the place for a caller to put loads of its own on their way without delaying the MLP's.
template <int DT, int GV, int NT, int ROWS, int PF, typename Hook = sig_no_hook>
__device__ __forceinline__ void sig_gemv_block(const sig_params& P, bool active, int tid, int b, int h, int l0, int nl,
                                               int n_layers, sig_gemv_lds<GV, NT>& S, Hook after_requests = Hook()) {
  constexpr int ES = (DT == SAH_F32) ? 4 : 2;
  constexpr int NW = NT / SAH_WAVE;
  constexpr int LOG_NT = 31 - __builtin_clz(NT);
  static_assert((NT & (NT - 1)) == 0, "NT must be a power of two");
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SAH_WAVE);  // tid: the caller's numbering of the block's threads
  const int hx = active ? h / P.group : 0;
  const int D = active ? P.D : 8;

  // Every width is a power of two here, so the thread -> (column group, row group) maps are shifts and masks:
  // layer geometry from d_out: CG = d_out / 8 column groups, RG = NT / CG row groups, d_in / RG rows per thread
  auto log2_cg = [&](int layer) { return 31 - __builtin_clz(P.d_out[layer]) - 3; };

  // Loads are requested in the order they are needed - the input vector and the biases (parked in LDS before
  // the first barrier), then the weight rows layer by layer - and none of them sits behind a branch, so they
  // are all in flight together.
  att_raw_w<DT> raw[PF][ROWS];
  auto fetch_layer = [&](int layer, int din, att_raw_w<DT> (&dst)[ROWS]) {
    const int dout = P.d_out[layer];
    const int lcg = log2_cg(layer);
    const int RG = NT >> lcg;
    const int cg = tid & ((1 << lcg) - 1), rg = tid >> lcg;
    const int nrow = din >> (LOG_NT - lcg);
    const char* wbase = (const char*)P.W[layer] + ((int64_t)h * din * dout + cg * 8) * ES;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = rg + (i < nrow ? i : 0) * RG;
      dst[i].load(wbase + (int64_t)d * dout * ES);
    }
  };
  auto fetch_bias = [&](int layer) -> float {  // threads beyond the width re-read element 0
    const int dout = P.d_out[layer];
    return sah_load<DT>(P.bias[layer], (int64_t)h * dout + (tid < dout ? tid : 0));
  };
  auto x_at = [&](int i) -> float {  // element i of the GV x D tile; rows beyond nl re-read the last vector
    int t = 0, d = i;
    if (GV > 1) {
      t = i / D;
      d = i - t * D;
    }
    if (t > nl - 1) t = nl - 1;
    return sah_load<DT>(P.x, (int64_t)b * P.xs_b + (int64_t)hx * P.xs_h + (int64_t)(l0 + t) * P.xs_l + d);
  };
  float xr = 0.f;
  float bias_r[PF];
  if (active) {
    xr = x_at(tid < GV * D ? tid : 0);
    if (PF > 1) {
#pragma unroll
      for (int layer = 0; layer < PF; ++layer) bias_r[layer] = layer < n_layers ? fetch_bias(layer) : 0.f;
      int din0 = D;
#pragma unroll
      for (int layer = 0; layer < PF; ++layer) {
        if (layer < n_layers) {
          fetch_layer(layer, din0, raw[layer]);
          din0 = P.d_out[layer];
        }
      }
    }
  }
  after_requests();
  if (active) {
    if (tid < GV * D) {
      if (GV > 1) S.x[tid / D][tid % D] = (tid / D < nl) ? xr : 0.f;
      else S.x[0][tid] = xr;
    }
    for (int i = tid + NT; i < GV * D; i += NT) S.x[i / D][i % D] = (i / D < nl) ? x_at(i) : 0.f;
    if (PF > 1) {
#pragma unroll
      for (int layer = 0; layer < PF; ++layer)
        if (layer < n_layers && tid < P.d_out[layer]) S.bias[layer][tid] = bias_r[layer];
    }
  }
  __syncthreads();

  int din = D;
#pragma unroll
  for (int layer = 0; layer < SAH_MAX_MLP_LAYERS; ++layer) {
    if (layer >= n_layers) break;
    const int dout = active ? P.d_out[layer] : 8;
    const bool last = (layer == n_layers - 1);
    const int lcg = 31 - __builtin_clz(dout) - 3;
    const int CG = 1 << lcg;            // column groups (power of two, <= 32)
    const int RG = NT >> lcg;           // row groups
    const int cg = tid & (CG - 1), rg = tid >> lcg;
    if (active) {
      const int nrow = din >> (LOG_NT - lcg);  // real rows of this thread: 1, 2, ... ROWS
      float acc[GV][8];
#pragma unroll
      for (int t = 0; t < GV; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[t][e] = 0.f;
      if (PF > 1) {
        gemv_layer_fma<DT, GV, ROWS>(raw[layer < PF ? layer : 0], nrow, rg, RG, S.x, acc);
      } else {
        if (tid < dout) S.bias[layer][tid] = fetch_bias(layer);  // read after this layer's barrier
        fetch_layer(layer, din, raw[0]);
        gemv_layer_fma<DT, GV, ROWS>(raw[0], nrow, rg, RG, S.x, acc);
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
          for (int e = 0; e < 8; ++e) S.part[wave][t][cg * 8 + e] = acc[t][e];
      }
    }
    __syncthreads();
    if (active) {
      // dout <= 256 => CG <= 32 < 64, so every wave holds all column groups
      const int ldout = lcg + 3;
      for (int i = tid; i < (GV << ldout); i += NT) {
        const int t = i >> ldout, e = i & (dout - 1);
        float y = 0.f;
#pragma unroll
        for (int wv2 = 0; wv2 < NW; ++wv2) y += S.part[wv2][t][e];
        y = sah_round<DT>(y);
        y = sah_round<DT>(y + S.bias[layer][e]);
        if (!last) y = sah_round<DT>(sig_act(P.act, y));
        S.x[t][e] = y;
      }
    }
    __syncthreads();
    din = dout;
  }

  if (active && tid < SAH_WAVE) {
    const int bits = din;
    for (int t = 0; t < nl; ++t) {
      const float y = (tid < bits) ? S.x[t][tid] : 0.f;
      const uint64_t pos = __ballot(y > 0.f);
      const uint64_t nz = __ballot(y != 0.f);
      if (tid == 0) {
        uint2 c;
        c.x = (uint32_t)pos;
        c.y = (uint32_t)nz;
        S.code[t] = c;
        if (P.codes) ((uint2*)P.codes)[((int64_t)b * P.Hq + h) * P.code_pitch + P.code_offset + l0 + t] = c;
      }
    }
  }
  __syncthreads();  // S.code is visible to the whole workgroup
}

// ---------------------------------------------------------------------------
// The same decode-size job on the matrix cores: up to 16 vectors of one head per call, 512 threads.
// Transposed, Y^T = W^T X^T: wave w owns the 16 output features 16 w .. 16 w + 15 of every layer, its slice of
// W^T (16 rows, k contiguous: one 16-byte load per lane and 32-element k-step, every layer requested up-front)
// is the A operand, the vectors (in LDS, 16-bit) are the B operand, and column j of the result is vector j.
// One barrier per layer. Needs 16-bit storage, W^T, D and the hidden widths multiples of 32 up to 128.
// ---------------------------------------------------------------------------
#define SMB_NT 512
#define SMB_MAXW 128
#define SMB_MAXK (SMB_MAXW / 32)
#define SMB_PITCH (SMB_MAXW + 8)  // 16-bit elements per LDS row: 16 B of padding against bank conflicts

struct sig_mfma_lds {
  uint16_t x[2][16][SMB_PITCH];  // inputs of the layers after the first, double buffered
  float y[16][32];               // last layer's outputs
  uint2 code[16];
};

// `after_requests` runs once every load of the MLP has been requested: the place for a caller to put loads of
// its own on their way without delaying the MLP's.
// ACT >= 0: the activation is that one, whatever P.act says (the caller has checked): the other three, GELU's error
// function among them, then stay out of the kernel's code; ACT < 0: P.act decides at run time. STD: the job has the usual
// HashAttention shape (inputs of 128, layers of 128, 128 and 32 outputs; the caller has checked): every width is then a
// compile-time constant, no load hides behind a branch, and the waits before a layer's matrix instructions count exactly
// the loads that layer needs instead of "everything outstanding". Same arithmetic either way.
template <int DT, typename Hook = sig_no_hook, int ACT = -1, bool STD = false>
__device__ __forceinline__ void sig_mfma_block(const sig_params& P, bool active, int tid, int b, int h, int l0, int nl,
                                               int n_layers, sig_mfma_lds& S, Hook after_requests = Hook()) {
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SAH_WAVE);  // tid: the caller's numbering of the block's threads
  const int i16 = lane & 15;  // row of A, column (vector) of B and C
  const int g = lane >> 4;    // k-group of the operands, row group of C
  const int hx = active ? h / P.group : 0;
  const int D = STD ? 128 : (active ? P.D : 32);
  const int NL = STD ? 3 : n_layers;
  auto dw = [&](int l) -> int { return STD ? (l < 2 ? 128 : 32) : P.d_out[l]; };  // width of layer l
  const int act = ACT >= 0 ? ACT : (active ? P.act : 0);
  const int f0 = 16 * wave + 4 * g;  // this lane's 4 output features of every layer: f0 .. f0 + 3

  // ---- first requests, only what the first layer needs, so that it can start as early as possible: the
  // vector itself straight into the B operand (no LDS round, no barrier), the biases (8 bytes per lane and
  // layer), this wave's slice of the first W^T. Raw loads and wave-uniform conditions only.
  uint4 bop0[SMB_MAXK];
  uint2 bias_raw[SAH_MAX_MLP_LAYERS];
  uint4 wr[SAH_MAX_MLP_LAYERS][SMB_MAXK];
  auto request_weights = [&](int l) {
    if (l < NL && 16 * wave < dw(l)) {  // a wave skips the layers it has no rows of
      const int dout = dw(l);
      const int din = l == 0 ? D : dw(l - 1);
      int row = 16 * wave + i16;
      if (row > dout - 1) row = dout - 1;  // rows beyond the width repeat the last one; their results are dropped
      const uint16_t* wrow = (const uint16_t*)P.Wt[l] + ((int64_t)h * dout + row) * din + 8 * g;
#pragma unroll
      for (int s = 0; s < SMB_MAXK; ++s)
        if (32 * s < din) wr[l][s] = *(const uint4*)(wrow + 32 * s);
    }
  };
  if (active) {
    const int t = i16 < nl ? i16 : nl - 1;  // columns beyond nl repeat the last vector (computed and dropped)
    const uint16_t* xrow = (const uint16_t*)P.x + (int64_t)b * P.xs_b + (int64_t)hx * P.xs_h + (int64_t)(l0 + t) * P.xs_l + 8 * g;
#pragma unroll
    for (int s = 0; s < SMB_MAXK; ++s)
      if (32 * s < D) bop0[s] = *(const uint4*)(xrow + 32 * s);
#pragma unroll
    for (int l = 0; l < SAH_MAX_MLP_LAYERS; ++l) {
      const int ll = l < NL ? l : 0;
      const int dout = dw(ll);
      bias_raw[l] = *(const uint2*)((const uint16_t*)P.bias[ll] + (int64_t)h * dout + (f0 + 4 <= dout ? f0 : 0));
    }
    request_weights(0);
  }

  int din = D;
#pragma unroll
  for (int l = 0; l < SAH_MAX_MLP_LAYERS; ++l) {
    if (l >= NL) break;
    const int dout = STD ? dw(l) : (active ? P.d_out[l] : 16);
    const bool last = (l == NL - 1);
    sah_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const bool mine = active && 16 * wave < dout;
    if (mine) {
#pragma unroll
      for (int s = 0; s < SMB_MAXK; ++s) {
        if (32 * s < din) {
          const uint4 bop = l == 0 ? bop0[s] : *(const uint4*)&S.x[l & 1][i16][32 * s + 8 * g];
          acc = sah_mfma_16x16x32<DT>(wr[l][s], bop, acc);
        }
      }
    }
    if (l == 0) {
      // the rest goes out behind the first layer's operands: it has the first layer's epilogue and a barrier
      // to arrive in
      __builtin_amdgcn_sched_barrier(0);
      if (active) {
#pragma unroll
        for (int k = 1; k < SAH_MAX_MLP_LAYERS; ++k) request_weights(k);
      }
      after_requests();
      __builtin_amdgcn_sched_barrier(0);
    }
    if (mine) {
      // lane (vector i16, group g) holds the features f0 + v
      const uint32_t braw[2] = {bias_raw[l].x, bias_raw[l].y};
      float y[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const uint16_t bb = (uint16_t)(braw[v >> 1] >> (16 * (v & 1)));
        const float bv = (f0 + 4 <= dout) ? ((DT == SAH_BF16) ? sah_bf16_to_float(bb) : sah_f16_to_float(bb)) : 0.f;
        y[v] = sah_round<DT>(sah_round<DT>(acc[v]) + bv);
      }
      if (!last) {
        if (f0 + 4 <= dout) {
          const uint2 packed = make_uint2(sah_pack2_hw<DT>(sig_act_fast(act, y[0]), sig_act_fast(act, y[1])),
                                          sah_pack2_hw<DT>(sig_act_fast(act, y[2]), sig_act_fast(act, y[3])));
          *(uint2*)&S.x[(l + 1) & 1][i16][f0] = packed;
        }
      } else if (f0 < 32) {
#pragma unroll
        for (int v = 0; v < 4; ++v) S.y[i16][f0 + v] = (f0 + 4 <= dout) ? y[v] : 0.f;
      }
    }
    __syncthreads();
    din = dout;
  }

  if (active && tid < SAH_WAVE) {
    const int bits = din;
    for (int t = 0; t < nl; ++t) {
      const float y = (tid < bits && tid < 32) ? S.y[t][tid] : 0.f;
      const uint64_t pos = __ballot(y > 0.f);
      const uint64_t nz = __ballot(y != 0.f);
      if (tid == 0) {
        uint2 c;
        c.x = (uint32_t)pos;
        c.y = (uint32_t)nz;
        S.code[t] = c;
        if (P.codes) ((uint2*)P.codes)[((int64_t)b * P.Hq + h) * P.code_pitch + P.code_offset + l0 + t] = c;
      }
    }
  }
  __syncthreads();  // S.code is visible to the whole workgroup
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// can the block-level GEMV with `nt` threads and `max_rows` row slots per thread run this job?
static inline bool sig_gemv_ok(const sah_hash_sig_args* a, int nt, int max_rows) {
  if (a->L > 64 || a->D % 8 || a->D > SIG_MAXD) return false;
  int din = a->D;
  for (int i = 0; i < a->n_layers; ++i) {
    const int dout = a->d_out[i];
    if (dout < 8 || dout > 256 || (dout & (dout - 1))) return false;
    const int rows_per_thread = (int)((int64_t)din * dout / (8 * nt));
    if ((int64_t)din * dout % (8 * nt) || rows_per_thread < 1 || rows_per_thread > max_rows ||
        (rows_per_thread & (rows_per_thread - 1)))
      return false;
    const int es = a->dtype == SAH_F32 ? 4 : 2;
    if (((uintptr_t)a->W[i]) % (8 * es)) return false;
    din = dout;
  }
  return true;
}

// can the matrix-core form of the decode-size job (sig_mfma_block) run this?
static inline bool sig_mfma_small_ok(const sah_hash_sig_args* a) {
  if (a->dtype != SAH_BF16 && a->dtype != SAH_F16) return false;
  if (a->L > 64 || a->D % 32 || a->D > SMB_MAXW) return false;
  if (a->xs_b % 8 || a->xs_h % 8 || a->xs_l % 8 || ((uintptr_t)a->x % 16)) return false;
  int din = a->D;
  for (int l = 0; l < a->n_layers; ++l) {
    if (!a->Wt[l] || ((uintptr_t)a->Wt[l] % 16)) return false;
    const bool last = l == a->n_layers - 1;
    if (last ? (a->d_out[l] > 32 || a->d_out[l] % 4) : (a->d_out[l] % 32 || a->d_out[l] > SMB_MAXW)) return false;
    if ((uintptr_t)a->bias[l] % 8) return false;
    din = a->d_out[l];
  }
  (void)din;
  return true;
}

static inline int sig_validate(const sah_hash_sig_args* a) {
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

static inline void sig_fill(const sah_hash_sig_args* a, sig_params& P) {
  P.x = a->x; P.xs_b = a->xs_b; P.xs_h = a->xs_h; P.xs_l = a->xs_l;
  P.B = a->B; P.Hq = a->Hq; P.group = a->group; P.L = a->L; P.D = a->D;
  P.n_layers = a->n_layers;
  for (int i = 0; i < SAH_MAX_MLP_LAYERS; ++i) {
    P.W[i] = a->W[i]; P.bias[i] = a->bias[i]; P.Wt[i] = a->Wt[i]; P.d_out[i] = a->d_out[i];
  }
  P.act = a->act;
  P.codes = a->codes; P.code_pitch = a->code_pitch; P.code_offset = a->code_offset;
}

