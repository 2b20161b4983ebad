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

// ---------------------------------------------------------------------------
// Bulk path on the matrix cores (a prefill, the first decode call of a layer: every key of the context).
// Per head the MLP is three small GEMMs; computed transposed, Y^T = W^T X^T, so that the vectors are the
// columns (N) of every product: a wave owns 32 vectors, the matrix-core result of one layer - lane j + 32 g
// holds, for vector j, the features 8 (v / 4) + 4 g + v % 4 of each 32-feature tile - is, after bias and
// activation, already laid out as the B operand of the next layer if the k-slots of a 16-feature step are
// taken in the order [0-3][8-11] (g = 0), [4-7][12-15] (g = 1). The A operand (W^T, staged once per workgroup
// in LDS, rows padded against bank conflicts) is stored in exactly that order for the layers after the
// first, so no value ever moves between lanes until the sign bits are packed.
// Needs 16-bit storage, D and the hidden widths multiples of 32 and at most 128, W^T given.
// ---------------------------------------------------------------------------
#define SGM_NT 512
#define SGM_NW (SGM_NT / SAH_WAVE)
#define SGM_TILE (32 * SGM_NW)  // vectors per workgroup tile
#define SGM_MAXW 128            // widest layer
#define SGM_MAXK (SGM_MAXW / 16)
#define SGM_MAXM (SGM_MAXW / 32)
#define SGM_PAD 8               // elements of padding per LDS row: 16 B

// ACT: the activation, fixed at compile time (one kernel each: with the choice left to run time the four epilogues,
// GELU's error function included, end up inside the hot loop and the code outgrows the instruction cache)
template <int DT, int ACT>
__global__ __launch_bounds__(SGM_NT, 4) void k_hash_sig_mfma(sig_params P, int n_chunks, int tiles_per_wg) {
  HIP_DYNAMIC_SHARED(unsigned char, sgm_dyn)
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  const int i32 = lane & 31;  // row of A / column of B and C
  const int g = lane >> 5;    // k-group of the operands, row group of C
  // the heads of one KV group are neighbours in the grid: they read the same vectors, which then hit in L2
  int idx = blockIdx.x;
  const int hq = idx % P.group;
  idx /= P.group;
  const int chunk = idx % n_chunks;
  idx /= n_chunks;
  const int Hx = P.Hq / P.group;
  const int hx = idx % Hx;
  const int b = idx / Hx;
  const int h = hx * P.group + hq;

  // ---- stage W^T (and the biases as fp32) in LDS
  // (offsets, not pointers: a pointer that has been through an array is a generic one to the compiler, and every read
  // through it a flat load, which also waits for the wave's outstanding global loads)
  int w_off[SAH_MAX_MLP_LAYERS];
  int pitch[SAH_MAX_MLP_LAYERS];
  int w_elems = 0;
  uint16_t* const s_w0 = (uint16_t*)sgm_dyn;
  {
    int din = P.D;
    for (int l = 0; l < P.n_layers; ++l) {
      w_off[l] = w_elems;
      pitch[l] = din + SGM_PAD;
      w_elems += ((P.d_out[l] + 31) & ~31) * pitch[l];
      din = P.d_out[l];
    }
  }
  float* s_bias = (float*)((uint16_t*)sgm_dyn + ((w_elems + 1) & ~1));
  {
    int din = P.D;
    for (int l = 0; l < P.n_layers; ++l) {
      const int dout = P.d_out[l];
      const int rows = (dout + 31) & ~31;
      const int upr = din >> 2;  // 8-byte units per row
      const uint16_t* wt = (const uint16_t*)P.Wt[l] + (int64_t)h * dout * din;
      for (int u = tid; u < rows * upr; u += SGM_NT) {
        const int row = u / upr, c4 = u - row * upr;
        const int blk = c4 >> 2, sub = c4 & 3;
        // layers after the first: the 4-element groups of a 16-block are kept as [0-3][8-11][4-7][12-15]
        const int dsub = (l > 0 && (sub == 1 || sub == 2)) ? (sub ^ 3) : sub;
        uint2 val = make_uint2(0u, 0u);
        if (row < dout) val = *(const uint2*)(wt + (int64_t)row * din + c4 * 4);
        *(uint2*)(s_w0 + w_off[l] + row * pitch[l] + blk * 16 + dsub * 4) = val;
      }
      for (int e = tid; e < SGM_MAXW; e += SGM_NT)
        s_bias[l * SGM_MAXW + e] = e < dout ? sah_load<DT>(P.bias[l], (int64_t)h * dout + e) : 0.f;
      din = dout;
    }
  }
  __syncthreads();

  const char* xbase = (const char*)P.x + ((int64_t)b * P.xs_b + (int64_t)hx * P.xs_h + 8 * g) * 2;
  uint2* codes = (uint2*)P.codes + ((int64_t)b * P.Hq + h) * P.code_pitch + P.code_offset;

  for (int t = 0; t < tiles_per_wg; ++t) {
    const int v0 = (chunk * tiles_per_wg + t) * SGM_TILE + wave * 32;  // first vector of this wave
    if (v0 >= P.L) break;                                               // uniform across the wave
    int vec = v0 + i32;
    const bool live = vec < P.L;
    if (!live) vec = P.L - 1;  // computed and dropped
    // B operand of the first layer: 8 consecutive elements of the vector per 16-element step
    uint4 bop[SGM_MAXK];
    const char* xrow = xbase + (int64_t)vec * P.xs_l * 2;
    const int k0 = P.D >> 4;
#pragma unroll
    for (int s = 0; s < SGM_MAXK; ++s) bop[s] = s < k0 ? *(const uint4*)(xrow + s * 32) : make_uint4(0u, 0u, 0u, 0u);

    int ksteps = k0;
#pragma unroll
    for (int l = 0; l < SAH_MAX_MLP_LAYERS; ++l) {
      if (l >= P.n_layers) break;
      const bool last = (l == P.n_layers - 1);
      const int mt = (P.d_out[l] + 31) >> 5;
      const uint16_t* wl = s_w0 + w_off[l] + i32 * pitch[l] + 8 * g;
      const float* bl = s_bias + l * SGM_MAXW + 4 * g;
      // one 32-row tile of the layer's output: 32x32x16 steps over the input, accumulator from zero
      auto tile = [&](int q) {
        sah_f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int s = 0; s < SGM_MAXK; ++s) {
          if (s < ksteps) {
            const uint4 a = *(const uint4*)(wl + q * 32 * pitch[l] + s * 16);
            acc = sah_mfma_32x32x16<DT>(a, bop[s], acc);
          }
        }
        return acc;
      };
      if (!last) {
        // bias, activation, rounding as torch rounds them; the result is the next layer's B operand. Two tiles at a
        // time: their accumulators, this layer's operand and the next one's are all that is live (four waves per SIMD)
        uint4 nxt[SGM_MAXK];
#pragma unroll
        for (int q = 0; q < SGM_MAXM; ++q) {
          float y[16];
          if (q < mt) {
            sah_f32x16 acc = tile(q);
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4) {
              const float4 b4 = *(const float4*)(bl + q * 32 + 8 * v4);  // four biases in one read
              const float bb[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                float z = sah_round<DT>(acc[4 * v4 + t]);
                z = sah_round<DT>(z + bb[t]);
                y[4 * v4 + t] = sig_act_fast(ACT, z);  // rounded by the packing below
              }
            }
          } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = 0.f;
          }
          nxt[2 * q] = make_uint4(sah_pack2_hw<DT>(y[0], y[1]), sah_pack2_hw<DT>(y[2], y[3]), sah_pack2_hw<DT>(y[4], y[5]),
                                  sah_pack2_hw<DT>(y[6], y[7]));
          nxt[2 * q + 1] = make_uint4(sah_pack2_hw<DT>(y[8], y[9]), sah_pack2_hw<DT>(y[10], y[11]), sah_pack2_hw<DT>(y[12], y[13]),
                                      sah_pack2_hw<DT>(y[14], y[15]));
        }
#pragma unroll
        for (int s = 0; s < SGM_MAXK; ++s) bop[s] = nxt[s];
        ksteps = 2 * mt;
      } else {
        // sign planes: this lane holds 16 of the vector's bits, lane ^ 32 the other 16
        sah_f32x16 acc0 = tile(0);
        uint32_t pos = 0u, nz = 0u;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float z = sah_round<DT>(acc0[v]);
          z = sah_round<DT>(z + bl[8 * (v >> 2) + (v & 3)]);
          const int bit = 8 * (v >> 2) + 4 * g + (v & 3);
          pos |= (z > 0.f ? 1u : 0u) << bit;
          nz |= (z != 0.f ? 1u : 0u) << bit;
        }
        pos |= __shfl_xor(pos, 32);
        nz |= __shfl_xor(nz, 32);
        if (g == 0 && live) codes[v0 + i32] = make_uint2(pos, nz);
      }
    }
  }
}

static size_t sgm_lds_bytes(const sah_hash_sig_args* a) {
  size_t elems = 0;
  int din = a->D;
  for (int l = 0; l < a->n_layers; ++l) {
    elems += (size_t)((a->d_out[l] + 31) & ~31) * (din + SGM_PAD);
    din = a->d_out[l];
  }
  elems = (elems + 1) & ~(size_t)1;
  return elems * 2 + (size_t)a->n_layers * SGM_MAXW * 4;
}

// can the matrix-core kernel run this job?
static bool sig_mfma_ok(const sah_hash_sig_args* a) {
  if (a->dtype != SAH_BF16 && a->dtype != SAH_F16) return false;
  if (a->L < 128) return false;  // a few vectors per head: the small forms are the better fit
  if (a->D % 32 || a->D > SGM_MAXW) return false;
  if (a->xs_b % 8 || a->xs_h % 8 || a->xs_l % 8 || ((uintptr_t)a->x % 16)) return false;
  for (int l = 0; l < a->n_layers; ++l) {
    if (!a->Wt[l] || ((uintptr_t)a->Wt[l] % 8)) return false;
    const bool last = l == a->n_layers - 1;
    if (last ? a->d_out[l] > 32 : (a->d_out[l] % 32 || a->d_out[l] > SGM_MAXW)) return false;
  }
  return sgm_lds_bytes(a) <= 150 * 1024;
}

template <int DT, int ACT>
static int sig_launch_mfma_a(const sah_hash_sig_args* a, const sig_params& P) {
  if (int rc = sah_allow_lds((const void*)k_hash_sig_mfma<DT, ACT>, 150 * 1024, "sah_hash_signatures")) return rc;
  const int n_tiles = (a->L + SGM_TILE - 1) / SGM_TILE;
  const int tiles_per_wg = n_tiles < 8 ? n_tiles : 8;   // the staged weights serve up to 8 tiles
  const int n_chunks = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
  const int64_t n_wg = (int64_t)a->B * a->Hq * n_chunks;
  if (n_wg > 0x7fffffff) return sah_fail(SAH_ESHAPE, "sah_hash_signatures: too many workgroups");
  sah_timed timed("k_hash_sig_mfma", a->stream);
  hipLaunchKernelGGL((k_hash_sig_mfma<DT, ACT>), dim3((unsigned)n_wg), dim3(SGM_NT), sgm_lds_bytes(a), (hipStream_t)a->stream, P,
                     n_chunks, tiles_per_wg);
  return sah_launch_status("sah_hash_signatures");
}

template <int DT>
static int sig_launch_mfma_t(const sah_hash_sig_args* a, const sig_params& P) {
  switch (a->act) {
    case SAH_ACT_RELU: return sig_launch_mfma_a<DT, SAH_ACT_RELU>(a, P);
    case SAH_ACT_SILU: return sig_launch_mfma_a<DT, SAH_ACT_SILU>(a, P);
    case SAH_ACT_GELU: return sig_launch_mfma_a<DT, SAH_ACT_GELU>(a, P);
    default: return sig_launch_mfma_a<DT, SAH_ACT_TANH>(a, P);
  }
}

// decode-size jobs on the matrix cores: up to 16 vectors of one head per workgroup
template <int DT>
__global__ __launch_bounds__(SMB_NT) void k_hash_sig_small_mfma(sig_pair PP) {
  sah_touch_kernargs<(sizeof(sig_pair) < 1024 ? sizeof(sig_pair) : 1024)>();
  const sig_params& P = PP.p[blockIdx.z];
  if ((int)blockIdx.x * 16 >= P.L) return;  // the two jobs may differ in vector count
  __shared__ sig_mfma_lds S;
  const int bh = blockIdx.y;
  const int l0 = blockIdx.x * 16;
  int nl = P.L - l0;
  if (nl > 16) nl = 16;
  sig_mfma_block<DT>(P, true, threadIdx.x, bh / P.Hq, bh % P.Hq, l0, nl, P.n_layers, S);
}

static int sig_launch_gemv(const sah_hash_sig_args* a, const sah_hash_sig_args* b2) {
  sig_pair PP;
  sig_fill(a, PP.p[0]);
  sig_fill(b2 ? b2 : a, PP.p[1]);
  const int maxL = (b2 && b2->L > a->L) ? b2->L : a->L;
  hipStream_t st = (hipStream_t)a->stream;
  if (sig_mfma_small_ok(a) && (!b2 || sig_mfma_small_ok(b2))) {
    sah_timed timed("k_hash_sig_small_mfma", a->stream);
    dim3 gg((maxL + 15) / 16, a->B * a->Hq, b2 ? 2 : 1);
    if (a->dtype == SAH_BF16) hipLaunchKernelGGL(k_hash_sig_small_mfma<SAH_BF16>, gg, dim3(SMB_NT), 0, st, PP);
    else hipLaunchKernelGGL(k_hash_sig_small_mfma<SAH_F16>, gg, dim3(SMB_NT), 0, st, PP);
    return sah_launch_status("sah_hash_signatures");
  }
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
  if (sig_mfma_ok(a)) {
    sig_params P;
    sig_fill(a, P);
    return a->dtype == SAH_BF16 ? sig_launch_mfma_t<SAH_BF16>(a, P) : sig_launch_mfma_t<SAH_F16>(a, P);
  }
  if (sig_mfma_small_ok(a) || sig_gemv_ok(a, GEMV_NT, GEMV_ROWS)) return sig_launch_gemv(a, nullptr);
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
  const bool both_mfma = sig_mfma_small_ok(a) && sig_mfma_small_ok(b);
  const bool both_gemv = !sig_mfma_small_ok(a) && !sig_mfma_small_ok(b) && sig_gemv_ok(a, GEMV_NT, GEMV_ROWS) &&
                         sig_gemv_ok(b, GEMV_NT, GEMV_ROWS);
  if (a->L > 0 && b->L > 0 && (both_mfma || both_gemv) && a->dtype == b->dtype && a->stream == b->stream &&
      (int64_t)a->B * a->Hq == (int64_t)b->B * b->Hq)
    return sig_launch_gemv(a, b);
  rc = sig_launch_one(a);
  if (rc) return rc;
  return sig_launch_one(b);
}
