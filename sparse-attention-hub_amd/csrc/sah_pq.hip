// PQCache kernels: batched Lloyd iteration (assignment + centre update) over
// the sub-vectors of the key cache, quantisation of newly appended keys, and
// asymmetric-distance (ADC) scoring through an LDS-resident lookup table.
//
// A group g = (b*Hkv + hk)*n_sub + s is one sub-space of one KV head. The
// assignment kernel keeps the group's centres (n_cent x d_sub fp32, <= 16 KB) in
// LDS, one thread per key, and accumulates the per-centre sums in LDS before a
// single flush of global atomics per workgroup, so no (b, n, k, d) tensor ever
// exists. Blocks are ordered sub-space-fastest so the n_sub workgroups that read
// different 16 B slices of the same key rows run next to each other and share
// the rows in L2.
#include "sah_common.h"

#define PQ_NT 256
#define PQ_MAX_D 17  // widest sub-vector of the kernels that keep a key in registers: 16 plus the extra coordinate of
                     // inner-product search done as L2 search; wider sub-vectors (up to PQM_MAX_D) take the matrix-core
                     // assignment and the one-centre-per-thread quantisation
#define PQ_MAX_CENT 256
#define PQ_TILES 8  // key tiles of PQ_NT per workgroup

// Per-centre sums of the Lloyd update are kept in 64-bit fixed point, so that their value does not depend on the
// order in which threads and workgroups add to them (floating-point atomics would make two runs on the same keys
// differ in a centroid's last bits). The scale is a power of two picked from the largest |key element|:
// |x| * scale < 2^41, which leaves room for 2^20 keys per centre and costs nothing in precision (a float has 24
// significant bits).
__device__ __forceinline__ float pq_sum_scale(uint32_t absmax_bits) {
  const float m = sah_bits_to_float(absmax_bits);
  if (!(m > 0.f) || !(m < INFINITY)) return 1.f;
  int e;
  frexpf(m, &e);  // m = f * 2^e, f in [0.5, 1)
  int sh = 40 - e;
  sh = sh < -100 ? -100 : (sh > 100 ? 100 : sh);
  return ldexpf(1.0f, sh);
}
__device__ __forceinline__ void pq_sum_add(long long* p, float x, float scale) {
  atomicAdd((unsigned long long*)p, (unsigned long long)__float2ll_rn(x * scale));
}

struct pq_assign_params {
  const void* k; int64_t ks_b, ks_h, ks_l;
  int Hkv, n_sub, d_sub, n_cent;
  int key_offset, n_keys;
  const float* centres;
  uint8_t* codes; int64_t code_pitch, code_offset;
  long long* sums; int* counts;
  const uint32_t* absmax_bits;
  int round_dist;
  const int* skip_flag;
};

template <int DT>
__global__ __launch_bounds__(PQ_NT) void k_pq_assign(pq_assign_params P) {
  __shared__ float s_c[PQ_MAX_CENT * PQ_MAX_D];
  __shared__ long long s_sum[PQ_MAX_CENT * PQ_MAX_D];
  __shared__ int s_cnt[PQ_MAX_CENT];
  if (P.skip_flag && *P.skip_flag) return;
  const float sum_scale = P.sums ? pq_sum_scale(*P.absmax_bits) : 1.f;
  const int tid = threadIdx.x;
  const int s = blockIdx.x % P.n_sub;
  const int tg = blockIdx.x / P.n_sub;
  const int bh = blockIdx.y;  // b*Hkv + hk
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int g = bh * P.n_sub + s;
  const int d_sub = P.d_sub, n_cent = P.n_cent;
  const int cd = n_cent * d_sub;

  for (int i = tid; i < cd; i += PQ_NT) {
    s_c[i] = P.centres[(int64_t)g * cd + i];
    s_sum[i] = 0;
  }
  for (int i = tid; i < n_cent; i += PQ_NT) s_cnt[i] = 0;
  __syncthreads();

  const int64_t kbase = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)s * d_sub;
  for (int t = 0; t < PQ_TILES; ++t) {
    const int n = (tg * PQ_TILES + t) * PQ_NT + tid;
    if (n >= P.n_keys) continue;
    float x[PQ_MAX_D];
    const int64_t off = kbase + (int64_t)(P.key_offset + n) * P.ks_l;
#pragma unroll
    for (int d = 0; d < PQ_MAX_D; ++d) x[d] = (d < d_sub) ? sah_load<DT>(P.k, off + d) : 0.f;
    int best = 0;
    float bd = INFINITY;
    for (int c = 0; c < n_cent; ++c) {
      const float* cc = s_c + c * d_sub;
      float dist = 0.f;
      if (P.round_dist) {
#pragma unroll
        for (int d = 0; d < PQ_MAX_D; ++d) {
          if (d < d_sub) {
            const float df = sah_round<DT>(x[d] - cc[d]);
            dist += sah_round<DT>(df * df);
          }
        }
        dist = sah_round<DT>(dist);
      } else {
#pragma unroll
        for (int d = 0; d < PQ_MAX_D; ++d) {
          if (d < d_sub) {
            const float df = x[d] - cc[d];
            dist = fmaf(df, df, dist);
          }
        }
      }
      if (dist < bd) {
        bd = dist;
        best = c;
      }
    }
    P.codes[(((int64_t)bh * P.code_pitch) + P.code_offset + n) * P.n_sub + s] = (uint8_t)best;
    if (P.sums) {
#pragma unroll
      for (int d = 0; d < PQ_MAX_D; ++d)
        if (d < d_sub) pq_sum_add(&s_sum[best * d_sub + d], x[d], sum_scale);
      atomicAdd(&s_cnt[best], 1);
    }
  }
  if (!P.sums) return;
  __syncthreads();
  for (int c = tid; c < n_cent; c += PQ_NT) {
    const int cn = s_cnt[c];
    if (cn) {
      atomicAdd(&P.counts[(int64_t)g * n_cent + c], cn);
      for (int d = 0; d < d_sub; ++d)
        atomicAdd((unsigned long long*)&P.sums[(int64_t)g * cd + c * d_sub + d], (unsigned long long)s_sum[c * d_sub + d]);
    }
  }
}

// Quantisation of a handful of keys (a decode step appends one): the work of one key and sub-space is a
// 256-way argmin, so the centres take the threads - one centre per thread, read straight from memory - and
// the keys take the grid. Same distances, same order of operations and the same lowest-index rule as the
// one-thread-per-key kernel above.
template <int DT>
__global__ __launch_bounds__(PQ_NT) void k_pq_assign_few(pq_assign_params P) {
  sah_touch_kernargs<sizeof(pq_assign_params)>();
  __shared__ float s_d[PQ_NT / SAH_WAVE];
  __shared__ int s_i[PQ_NT / SAH_WAVE];
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  const int s = blockIdx.x;
  const int bh = blockIdx.y;
  const int n = blockIdx.z;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int g = bh * P.n_sub + s;
  const int d_sub = P.d_sub, n_cent = P.n_cent;
  const int64_t off = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)s * d_sub + (int64_t)(P.key_offset + n) * P.ks_l;
  float dist = INFINITY;
  int best = 0x7fffffff;
  for (int c = tid; c < n_cent; c += PQ_NT) {
    const float* cc = P.centres + ((int64_t)g * n_cent + c) * d_sub;
    float dd = 0.f;
    if (P.round_dist) {
      for (int d = 0; d < d_sub; ++d) {
        const float df = sah_round<DT>(sah_load<DT>(P.k, off + d) - cc[d]);
        dd += sah_round<DT>(df * df);
      }
      dd = sah_round<DT>(dd);
    } else {
      for (int d = 0; d < d_sub; ++d) {
        const float df = sah_load<DT>(P.k, off + d) - cc[d];
        dd = fmaf(df, df, dd);
      }
    }
    if (dd < dist) {  // c ascends: the first minimum is kept
      dist = dd;
      best = c;
    }
  }
  // smallest distance, lowest centre among equals
#pragma unroll
  for (int o = 1; o < SAH_WAVE; o <<= 1) {
    const float od = __shfl_xor(dist, o);
    const int oi = __shfl_xor(best, o);
    if (od < dist || (od == dist && oi < best)) {
      dist = od;
      best = oi;
    }
  }
  if (lane == 0) {
    s_d[wave] = dist;
    s_i[wave] = best;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < PQ_NT / SAH_WAVE; ++w) {
      if (s_d[w] < dist || (s_d[w] == dist && s_i[w] < best)) {
        dist = s_d[w];
        best = s_i[w];
      }
    }
    P.codes[(((int64_t)bh * P.code_pitch) + P.code_offset + n) * P.n_sub + s] = (uint8_t)best;
  }
}

// A block of new keys (up to a few hundred) against frozen centres: one workgroup per (sub-space, batch x KV head)
// stages the group's centres in LDS once; a wave takes every 4th key, its lanes share the centres out
// (lane, lane + 64, ...), and the argmin of a key is a wave reduction: no workgroup barrier per key. Same
// arithmetic per (key, centre) pair as k_pq_assign_few, same "first minimum" rule.
#define PQB_NT 1024
template <int DT>
__global__ __launch_bounds__(PQB_NT) void k_pq_assign_block(pq_assign_params P) {
  sah_touch_kernargs<sizeof(pq_assign_params)>();
  __shared__ float s_c[PQ_MAX_CENT * PQ_MAX_D];
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = tid / SAH_WAVE;
  const int s = blockIdx.x;
  const int bh = blockIdx.y;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int g = bh * P.n_sub + s;
  const int d_sub = P.d_sub, n_cent = P.n_cent;
  // centres transposed, s_c[d][c]: the lanes of a wave (consecutive centres) read consecutive words
  for (int i = tid; i < n_cent * d_sub; i += PQB_NT) {
    const int c = i / d_sub, d = i - c * d_sub;
    s_c[d * n_cent + c] = P.centres[(int64_t)g * n_cent * d_sub + i];
  }
  // this wave's keys (every 16th), up to four of them requested before the first is used
  constexpr int NW = PQB_NT / SAH_WAVE;
  constexpr int KB = 4;
  const int64_t key0 = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)s * d_sub;
  auto load_key = [&](int n, float (&x)[PQ_MAX_D]) {
    const int64_t off = key0 + (int64_t)(P.key_offset + n) * P.ks_l;
#pragma unroll
    for (int d = 0; d < PQ_MAX_D; ++d) x[d] = d < d_sub ? sah_load<DT>(P.k, off + d) : 0.f;
  };
  __syncthreads();
  for (int n0 = wave; n0 < P.n_keys; n0 += KB * NW) {
    float xs[KB][PQ_MAX_D];
#pragma unroll
    for (int u = 0; u < KB; ++u) {
      const int n = n0 + u * NW;
      load_key(n < P.n_keys ? n : n0, xs[u]);
    }
#pragma unroll
    for (int u = 0; u < KB; ++u) {
      const int n = n0 + u * NW;
      if (n >= P.n_keys) break;  // uniform across the wave
      const float (&x)[PQ_MAX_D] = xs[u];
      float dist = INFINITY;
      int best = 0x7fffffff;
      for (int c = lane; c < n_cent; c += SAH_WAVE) {
        float dd = 0.f;
        if (P.round_dist) {
#pragma unroll
          for (int d = 0; d < PQ_MAX_D; ++d) {
            if (d < d_sub) {
              const float df = sah_round<DT>(x[d] - s_c[d * n_cent + c]);
              dd += sah_round<DT>(df * df);
            }
          }
          dd = sah_round<DT>(dd);
        } else {
#pragma unroll
          for (int d = 0; d < PQ_MAX_D; ++d) {
            if (d < d_sub) {
              const float df = x[d] - s_c[d * n_cent + c];
              dd = fmaf(df, df, dd);
            }
          }
        }
        if (dd < dist) {  // c ascends: the first minimum is kept
          dist = dd;
          best = c;
        }
      }
#pragma unroll
      for (int o = 1; o < SAH_WAVE; o <<= 1) {
        const float od = __shfl_xor(dist, o);
        const int oi = __shfl_xor(best, o);
        if (od < dist || (od == dist && oi < best)) {
          dist = od;
          best = oi;
        }
      }
      if (lane == 0) P.codes[(((int64_t)bh * P.code_pitch) + P.code_offset + n) * P.n_sub + s] = (uint8_t)best;
    }
  }
}

// ---------------------------------------------------------------------------
// Lloyd assignment on the matrix cores. argmin_c ||x - c||^2 = argmin_c (||c||^2 - 2 x.c): the key x centre
// contraction is an fp32 MFMA (32 centres x 32 keys x 2 dims per instruction) whose accumulator starts at
// ||c||^2 and whose A operand is -2 c, so the accumulator IS the quantity to minimise. A lane owns one key
// (column) and, per centre tile, 16 centres (rows) in ascending order: the running argmin needs no cross-lane
// work until the two lanes of a key are merged at the end. Centres (pre-scaled, in operand order) and their
// norms sit in LDS; per-centre sums for the update step are accumulated in LDS and flushed once.
// The expansion rounds differently from the difference form of the reference ((A - B)^2 summed,
// pq_utils.py:220-257): a key whose two nearest centres tie to the last bits may take the other one.
// ---------------------------------------------------------------------------
#define PQM_NT 256
#define PQM_NW (PQM_NT / SAH_WAVE)
#define PQM_KEY_TILES 16  // 32-key tiles per wave and workgroup: 2048 keys per workgroup
#define PQM_MAX_D 128     // widest sub-vector of the matrix-core assignment (64 k-steps)
#define PQM_FUSED_LDS (80 * 1024)  // operands + sums up to this much LDS: sums in the same kernel, two workgroups a CU

// LDS of the assignment kernel: A operands, centre norms and, when the sums are fused, the fixed-point sums and counts
static size_t pqm_lds_bytes(int n_cent, int d_sub, int ks, bool sums) {
  const size_t n_tiles = (size_t)(n_cent + 31) / 32;
  size_t bytes = n_tiles * 64 * ks * 4 + n_tiles * 32 * 4;
  if (sums) bytes += (size_t)n_cent * d_sub * 8 + (size_t)n_cent * 4;
  return bytes;
}

// (two waves per SIMD at least: with at most 256 registers a wave the compiler keeps the accumulators in ordinary
// vector registers, which the minimum search reads directly)
// KS k-steps of two dimensions each: sub-vectors of up to 2 KS dimensions (the operands beyond d_sub are zero).
// SUMS: the per-centre sums of the update step are accumulated here (P.sums given and the LDS holds them).
template <int DT, int KS, bool SUMS>
__global__ __launch_bounds__(PQM_NT, 2) void k_pq_assign_mfma(pq_assign_params P) {
  HIP_DYNAMIC_SHARED(unsigned char, pqm_dyn)
  if (P.skip_flag && *P.skip_flag) return;
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  const int j = lane & 31, g = lane >> 5;
  const int s_idx = blockIdx.x % P.n_sub;
  const int tg = blockIdx.x / P.n_sub;
  const int bh = blockIdx.y;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int grp = bh * P.n_sub + s_idx;
  const int n_cent = P.n_cent, d_sub = P.d_sub;
  const int n_tiles = (n_cent + 31) >> 5;
  const float* cbase = P.centres + (int64_t)grp * n_cent * d_sub;
  // -2 c as the A operand: element (k-step s, half g, centre row i of tile t). Four k-steps of a row sit together
  // and consecutive rows follow each other, so that a wave's 16-byte reads are conflict-free whatever KS is.
  float* s_a = (float*)pqm_dyn;                                    // [tile][g][s / 4][i][s % 4]   (KS = 2: [tile][g][i][s])
  float* s_cn = s_a + (size_t)n_tiles * 64 * KS;                   // ||c||^2, [tile][g][v]
  long long* s_sum = (long long*)(s_cn + (size_t)n_tiles * 32);    // [centre][d]      (SUMS only; 8-byte aligned: both
  int* s_cnt = (int*)(s_sum + (size_t)n_cent * d_sub);             // [centre]          sizes above are multiples of 8)
  const float sum_scale = SUMS ? pq_sum_scale(*P.absmax_bits) : 1.f;
  constexpr int SQ = KS >= 4 ? 4 : KS;  // k-steps per 16-byte (8-byte) group

  for (int idx = tid; idx < n_tiles * 64 * KS; idx += PQM_NT) {
    const int s4 = idx % SQ, i = (idx / SQ) & 31, q = (idx / (SQ * 32)) % (KS / SQ), gg = (idx / (SQ * 32 * (KS / SQ))) & 1,
              t = idx / (64 * KS);
    const int c = t * 32 + i, d = 2 * (q * SQ + s4) + gg;
    s_a[idx] = (c < n_cent && d < d_sub) ? -2.0f * cbase[c * d_sub + d] : 0.f;
  }
  for (int idx = tid; idx < n_tiles * 32; idx += PQM_NT) {
    const int v = idx & 15, gg = (idx >> 4) & 1, t = idx >> 5;
    const int c = t * 32 + 8 * (v >> 2) + 4 * gg + (v & 3);
    float nn = INFINITY;  // centres beyond n_cent never win
    if (c < n_cent) {
      nn = 0.f;
      for (int d = 0; d < d_sub; ++d) nn = fmaf(cbase[c * d_sub + d], cbase[c * d_sub + d], nn);
    }
    s_cn[idx] = nn;
  }
  if (SUMS) {
    for (int i = tid; i < n_cent * d_sub; i += PQM_NT) s_sum[i] = 0;
    for (int i = tid; i < n_cent; i += PQM_NT) s_cnt[i] = 0;
  }
  __syncthreads();

  const int64_t kbase = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)s_idx * d_sub;
  for (int kt = 0; kt < PQM_KEY_TILES; ++kt) {
    const int n0 = ((tg * PQM_KEY_TILES + kt) * PQM_NW + wave) * 32;
    if (n0 >= P.n_keys) break;  // uniform across the wave
    const int n = n0 + j;
    const bool valid = n < P.n_keys;
    const int64_t off = kbase + (int64_t)(P.key_offset + (valid ? n : P.n_keys - 1)) * P.ks_l;
    float xs[KS];  // this lane's dims 2 s + g of its key
#pragma unroll
    for (int s = 0; s < KS; ++s) xs[s] = (2 * s + g < d_sub) ? sah_load<DT>(P.k, off + 2 * s + g) : 0.f;
    float best = INFINITY;
    int bidx = 0;
    // accumulator of centre tile t: seeded with the norms, then the KS matrix instructions
    auto product = [&](sah_f32x16& acc, int t) {
      const float4* cn4 = (const float4*)(s_cn + (t * 2 + g) * 16);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const float4 c4 = cn4[q4];
        acc[4 * q4] = c4.x; acc[4 * q4 + 1] = c4.y; acc[4 * q4 + 2] = c4.z; acc[4 * q4 + 3] = c4.w;
      }
      if constexpr (KS >= 4) {
        const float4* ap = (const float4*)(s_a + (size_t)(t * 2 + g) * 32 * KS) + j;
#pragma unroll
        for (int q = 0; q < KS / 4; ++q) {
          const float4 a4 = ap[q * 32];
          acc = sah_mfma_32x32x2_f32(a4.x, xs[4 * q], acc);
          acc = sah_mfma_32x32x2_f32(a4.y, xs[4 * q + 1], acc);
          acc = sah_mfma_32x32x2_f32(a4.z, xs[4 * q + 2], acc);
          acc = sah_mfma_32x32x2_f32(a4.w, xs[4 * q + 3], acc);
        }
      } else {
        const float* ap = s_a + ((t * 2 + g) * 32 + j) * KS;
#pragma unroll
        for (int s = 0; s < KS; ++s) acc = sah_mfma_32x32x2_f32(ap[s], xs[s], acc);
      }
    };
    // the tile's first minimum and its accumulator slot (constants), then one comparison with the best so far:
    // bidx holds 16 t + slot until the end
    auto take_min = [&](const sah_f32x16& acc, int t) {
      float m = acc[0];
      int mv = 0;
#pragma unroll
      for (int v = 1; v < 16; ++v) {  // ascending centre index: the first minimum is kept
        if (acc[v] < m) {
          m = acc[v];
          mv = v;
        }
      }
      if (m < best) {
        best = m;
        bidx = t * 16 + mv;
      }
    };
    // Two accumulators: while the matrix unit works on one tile, the vector unit takes the minimum of the tile
    // before (48 vector instructions against 4 matrix instructions of 16 passes: about the same time).
    sah_f32x16 acc0, acc1;
    product(acc0, 0);
    int t = 0;
    for (; t + 2 < n_tiles; t += 2) {
      product(acc1, t + 1);
      take_min(acc0, t);
      product(acc0, t + 2);
      take_min(acc1, t + 1);
    }
    if (t + 1 < n_tiles) {
      product(acc1, t + 1);
      take_min(acc0, t);
      take_min(acc1, t + 1);
    } else {
      take_min(acc0, t);
    }
    bidx = (bidx >> 4) * 32 + 8 * ((bidx >> 2) & 3) + 4 * g + (bidx & 3);  // tile, slot -> centre
    const float ob = __shfl_xor(best, 32);
    const int oi = __shfl_xor(bidx, 32);
    if (ob < best || (ob == best && oi < bidx)) {
      best = ob;
      bidx = oi;
    }
    if (valid) {
      if (g == 0) P.codes[(((int64_t)bh * P.code_pitch) + P.code_offset + n) * P.n_sub + s_idx] = (uint8_t)bidx;
      if (SUMS) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
          if (2 * s + g < d_sub) pq_sum_add(&s_sum[bidx * d_sub + 2 * s + g], xs[s], sum_scale);
        if (g == 0) atomicAdd(&s_cnt[bidx], 1);
      }
    }
  }
  if (!SUMS) return;
  __syncthreads();
  for (int c = tid; c < n_cent; c += PQM_NT) {
    const int cn = s_cnt[c];
    if (cn) {
      atomicAdd(&P.counts[(int64_t)grp * n_cent + c], cn);
      for (int d = 0; d < d_sub; ++d)
        atomicAdd((unsigned long long*)&P.sums[(int64_t)grp * n_cent * d_sub + c * d_sub + d], (unsigned long long)s_sum[c * d_sub + d]);
    }
  }
}

// Per-centre sums and counts from the codes an assignment wrote, for shapes whose sums do not fit beside the
// assignment's operands in LDS. One workgroup takes 2048 keys of a group; consecutive threads take consecutive
// dimensions of a key, so their LDS atomics fall into consecutive words of one centre's row.
#define PQS_NT 1024
#define PQS_KEYS 2048
#define PQS_MAX_SUMS 16384  // fixed-point sums a workgroup keeps in LDS (128 KB): wider groups are split by dimension
// grid.z splits the dimensions into slices of d_chunk; slice 0 also counts the members
template <int DT>
__global__ __launch_bounds__(PQS_NT) void k_pq_sums(pq_assign_params P, int d_chunk) {
  HIP_DYNAMIC_SHARED(unsigned char, pqs_dyn)
  if (P.skip_flag && *P.skip_flag) return;
  const int tid = threadIdx.x;
  const int s_idx = blockIdx.x % P.n_sub;
  const int tg = blockIdx.x / P.n_sub;
  const int bh = blockIdx.y;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int grp = bh * P.n_sub + s_idx;
  const int n_cent = P.n_cent, d_sub = P.d_sub;
  const int d0 = blockIdx.z * d_chunk;
  const int dn = d_sub - d0 < d_chunk ? d_sub - d0 : d_chunk;
  long long* s_sum = (long long*)pqs_dyn;                  // [centre][dn]
  int* s_cnt = (int*)(s_sum + (size_t)n_cent * d_chunk);
  const float sum_scale = pq_sum_scale(*P.absmax_bits);
  for (int i = tid; i < n_cent * dn; i += PQS_NT) s_sum[i] = 0;
  for (int i = tid; i < n_cent; i += PQS_NT) s_cnt[i] = 0;
  __syncthreads();
  const int first = tg * PQS_KEYS;
  const int count = P.n_keys - first < PQS_KEYS ? P.n_keys - first : PQS_KEYS;
  const int64_t kbase = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)s_idx * d_sub + d0;
  for (int idx = tid; idx < count * dn; idx += PQS_NT) {
    const int n = first + idx / dn, d = idx % dn;
    const int code = P.codes[(((int64_t)bh * P.code_pitch) + P.code_offset + n) * P.n_sub + s_idx];
    pq_sum_add(&s_sum[code * dn + d], sah_load<DT>(P.k, kbase + (int64_t)(P.key_offset + n) * P.ks_l + d), sum_scale);
    if (d == 0) atomicAdd(&s_cnt[code], 1);
  }
  __syncthreads();
  for (int i = tid; i < n_cent * dn; i += PQS_NT) {
    const int c = i / dn, d = i % dn;
    if (s_cnt[c])
      atomicAdd((unsigned long long*)&P.sums[(int64_t)grp * n_cent * d_sub + c * d_sub + d0 + d], (unsigned long long)s_sum[i]);
  }
  if (blockIdx.z == 0)
    for (int c = tid; c < n_cent; c += PQS_NT)
      if (s_cnt[c]) atomicAdd(&P.counts[(int64_t)grp * n_cent + c], s_cnt[c]);
}

template <int DT, int KS>
static int pq_launch_mfma_ks(const sah_pq_assign_args* a, const pq_assign_params& P, bool fused, size_t lds) {
  const int per_wg = PQM_NW * 32 * PQM_KEY_TILES;
  dim3 g(((a->n_keys + per_wg - 1) / per_wg) * a->n_sub, a->B * a->Hkv), blk(PQM_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_pq_assign_mfma", a->stream);
  if (fused) {
    if (int rc = sah_allow_lds((const void*)k_pq_assign_mfma<DT, KS, true>, 160 * 1024, "sah_pq_kmeans_assign")) return rc;
    hipLaunchKernelGGL((k_pq_assign_mfma<DT, KS, true>), g, blk, lds, st, P);
  } else {
    if (int rc = sah_allow_lds((const void*)k_pq_assign_mfma<DT, KS, false>, 160 * 1024, "sah_pq_kmeans_assign")) return rc;
    hipLaunchKernelGGL((k_pq_assign_mfma<DT, KS, false>), g, blk, lds, st, P);
  }
  return sah_launch_status("sah_pq_kmeans_assign");
}

template <int DT>
static int pq_launch_mfma(const sah_pq_assign_args* a, const pq_assign_params& P) {
  int ks = 2;
  while (2 * ks < a->d_sub) ks *= 2;  // 2, 4, 8, 16, 32, 64 k-steps: sub-vectors of up to 4 ... 128 dimensions
  const bool want_sums = a->sums != nullptr;
  const bool fused = want_sums && pqm_lds_bytes(a->n_cent, a->d_sub, ks, true) <= PQM_FUSED_LDS;
  const size_t lds = pqm_lds_bytes(a->n_cent, a->d_sub, ks, fused);
  int rc;
  switch (ks) {
    case 2: rc = pq_launch_mfma_ks<DT, 2>(a, P, fused, lds); break;
    case 4: rc = pq_launch_mfma_ks<DT, 4>(a, P, fused, lds); break;
    case 8: rc = pq_launch_mfma_ks<DT, 8>(a, P, fused, lds); break;
    case 16: rc = pq_launch_mfma_ks<DT, 16>(a, P, fused, lds); break;
    case 32: rc = pq_launch_mfma_ks<DT, 32>(a, P, fused, lds); break;
    default: rc = pq_launch_mfma_ks<DT, 64>(a, P, fused, lds); break;
  }
  if (rc || !want_sums || fused) return rc;
  // the sums from the codes just written, in a launch of their own
  int d_chunk = a->d_sub;
  while (a->n_cent * d_chunk > PQS_MAX_SUMS) d_chunk = (d_chunk + 1) / 2;
  const size_t lds_s = (size_t)a->n_cent * d_chunk * 8 + (size_t)a->n_cent * 4;
  if ((rc = sah_allow_lds((const void*)k_pq_sums<DT>, 160 * 1024, "sah_pq_kmeans_assign"))) return rc;
  dim3 g(((a->n_keys + PQS_KEYS - 1) / PQS_KEYS) * a->n_sub, a->B * a->Hkv, (a->d_sub + d_chunk - 1) / d_chunk), blk(PQS_NT);
  sah_timed timed("k_pq_sums", a->stream);
  hipLaunchKernelGGL(k_pq_sums<DT>, g, blk, lds_s, (hipStream_t)a->stream, P, d_chunk);
  return sah_launch_status("sah_pq_kmeans_assign(sums)");
}

struct pq_update_params {
  const void* k; int64_t ks_b, ks_h, ks_l;
  int Hkv, n_sub, d_sub, n_cent, key_offset;
  float* centres;
  const long long* sums; const int* counts;
  const uint32_t* absmax_bits;
  const int* reseed_idx;
  float* shift2;
  float tol;
  int* state;
  int n_groups;
};

template <int DT>
__global__ __launch_bounds__(PQ_NT) void k_pq_update(pq_update_params P) {
  __shared__ float s_red[PQ_NT / SAH_WAVE];
  if (P.state[2]) return;
  const int tid = threadIdx.x;
  const int g = blockIdx.x;
  const int s = g % P.n_sub;
  const int bh = g / P.n_sub;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int d_sub = P.d_sub, n_cent = P.n_cent;
  float move = 0.f;
  if (tid < n_cent) {
    const int c = tid;
    const int cn = P.counts[(int64_t)g * n_cent + c];
    float* cc = P.centres + ((int64_t)g * n_cent + c) * d_sub;
    const long long* ss = P.sums + ((int64_t)g * n_cent + c) * d_sub;
    const double unscale = 1.0 / ((double)pq_sum_scale(*P.absmax_bits) * (double)(cn > 0 ? cn : 1));
    float acc = 0.f;
    int64_t roff = 0;
    if (cn == 0) {
      const int ridx = P.reseed_idx[(int64_t)g * n_cent + c];
      roff = (int64_t)b * P.ks_b + (int64_t)hk * P.ks_h + (int64_t)(P.key_offset + ridx) * P.ks_l + (int64_t)s * d_sub;
    }
    for (int d = 0; d < d_sub; ++d) {
      const float nv = (cn > 0) ? (float)((double)ss[d] * unscale) : sah_load<DT>(P.k, roff + d);
      const float df = nv - cc[d];
      acc = fmaf(df, df, acc);
      cc[d] = nv;
    }
    move = sqrtf(acc);
  }
  move = sah_wave_sum(move);
  if ((tid & (SAH_WAVE - 1)) == 0) s_red[tid / SAH_WAVE] = move;
  __syncthreads();
  if (tid == 0) {
    float tot = 0.f;
    for (int i = 0; i < PQ_NT / SAH_WAVE; ++i) tot += s_red[i];
    const float sh2 = tot * tot;
    P.shift2[g] = sh2;
    if (sh2 < P.tol) atomicAdd(&P.state[0], 1);
    __threadfence();
    const int ticket = atomicAdd(&P.state[1], 1);
    if (ticket == P.n_groups - 1) {
      // last group of this iteration: publish the verdict and reset the counters
      const int conv = atomicAdd(&P.state[0], 0);
      P.state[3] = (conv == P.n_groups) ? 1 : 0;
      P.state[0] = 0;
      P.state[1] = 0;
    }
  }
}

// state[3] -> state[2] is promoted by a separate one-thread kernel so that every
// group of the iteration in flight still sees the old flag.
__global__ void k_pq_promote(int* state) {
  if (threadIdx.x == 0 && blockIdx.x == 0 && state[3]) state[2] = 1;
}

struct pq_adc_params {
  const void* q; int64_t qs_b, qs_h, qs_l;
  int Hq, Hkv, Lq, n_sub, d_sub, n_cent;
  const float* centres;
  const void* centres_narrow;  // the same values in the storage type, or NULL
  const uint8_t* codes; int64_t code_pitch;
  int n_cand;
  void* keys_out; int64_t key_pitch;
};

#define ADC_MAX_LUT 4096  // n_sub * n_cent
#define ADC_NT 1024       // threads of the scoring kernel
#define ADC_KEYS 4096     // candidates per workgroup of the scoring kernel
#define ADC_MAX_HEAD_DIM 512  // widest query vector a workgroup stages in LDS when it builds its own table
#define ADC_OWN_LUT_WGS 16 // up to this many workgroups per KV head each build the lookup table themselves

// Lookup table of one decode step: lut[bh][vg][s][c][i] = round(q_v . centre[bh][s][c]) for the NQ query vectors
// v = vg * NQ + i of the KV head's group, in the storage type (fp32: NQ = 2, 16-bit: NQ = 4, i.e. 8 bytes per
// (s, c): one LDS read serves all the query vectors a workgroup scores).
// NQ dot products -> one 8-byte table entry, each rounded to the storage type
template <int DT, int NQ>
__device__ __forceinline__ uint2 pq_pack_entry(const float (&acc)[NQ]) {
  float val[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) val[i] = sah_round<DT>(acc[i]);
  uint2 pk;
  if (DT == SAH_F32) {
    pk.x = sah_float_to_bits(val[0]);
    pk.y = sah_float_to_bits(val[1]);
  } else if (DT == SAH_BF16) {
    pk.x = (uint32_t)sah_float_to_bf16(val[0]) | ((uint32_t)sah_float_to_bf16(val[1]) << 16);
    pk.y = (uint32_t)sah_float_to_bf16(val[NQ > 2 ? 2 : 0]) | ((uint32_t)sah_float_to_bf16(val[NQ > 2 ? 3 : 0]) << 16);
  } else {
    pk.x = (uint32_t)sah_float_to_f16(val[0]) | ((uint32_t)sah_float_to_f16(val[1]) << 16);
    pk.y = (uint32_t)sah_float_to_f16(val[NQ > 2 ? 2 : 0]) | ((uint32_t)sah_float_to_f16(val[NQ > 2 ? 3 : 0]) << 16);
  }
  return pk;
}

// One table entry: the NQ rounded dot products of sub-space s, centre c, packed into 8 bytes.
template <int DT>
__device__ __forceinline__ uint2 pq_lut_entry(const pq_adc_params& P, int b, int hk, int bh, int vg, int s, int c) {
  constexpr int NQ = (DT == SAH_F32) ? 2 : 4;
  const int G = P.Hq / P.Hkv;
  const int nvec = G * P.Lq;
  const int d_sub = P.d_sub;
  const float* cc = P.centres + (((int64_t)bh * P.n_sub + s) * P.n_cent + c) * d_sub;
  float val[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int v = vg * NQ + i;
    val[i] = 0.f;
    if (v < nvec) {
      const int h = hk * G + v / P.Lq, qi = v % P.Lq;
      const int64_t qo = (int64_t)b * P.qs_b + (int64_t)h * P.qs_h + (int64_t)qi * P.qs_l + (int64_t)s * d_sub;
      float acc = 0.f;
      for (int d = 0; d < d_sub; ++d) acc = fmaf(sah_load<DT>(P.q, qo + d), cc[d], acc);
      val[i] = acc;
    }
  }
  return pq_pack_entry<DT>(val);
}

template <int DT>
__global__ __launch_bounds__(PQ_NT) void k_pq_lut(pq_adc_params P, void* lut) {
  constexpr int NQ = (DT == SAH_F32) ? 2 : 4;
  const int s = blockIdx.x;
  const int bh = blockIdx.y;
  const int vg = blockIdx.z;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int nvec = (P.Hq / P.Hkv) * P.Lq;
  const int n_vg = (nvec + NQ - 1) / NQ;
  for (int c = threadIdx.x; c < P.n_cent; c += PQ_NT) {
    const int64_t e = (((int64_t)bh * n_vg + vg) * P.n_sub + s) * P.n_cent + c;
    ((uint2*)lut)[e] = pq_lut_entry<DT>(P, b, hk, bh, vg, s, c);
  }
}

// Scores of ADC_KEYS candidates for the NQ query vectors of one group: one 16-wave workgroup, the table in LDS
// as 8-byte entries per (s, c) (two floats for fp32, four packed 16-bit values otherwise: the entries are rounded to
// the storage type anyway, and the LDS reads are what bounds this kernel), one thread per candidate. A lookup is
// one LDS read, NQ widenings (a shift or a mask for bf16) and NQ additions. (The packed dot-product instruction
// against (1, 0) would widen and add in one operation, but its sum is not always the correctly rounded one: one
// addition in 800 differed in the last bit.) OWN_LUT: the workgroup computes its table itself
// (every workgroup of a KV head repeats that work, which is cheaper than a launch of its own as long as a head is
// covered by a few dozen workgroups); otherwise the entries k_pq_lut wrote are copied in.
template <int DT, bool OWN_LUT>
__global__ __launch_bounds__(ADC_NT) void k_pq_adc(pq_adc_params P, const void* lut) {
  sah_touch_kernargs<sizeof(pq_adc_params) + 8>();
  constexpr int NQ = (DT == SAH_F32) ? 2 : 4;
  typedef typename std::conditional<DT == SAH_F32, uint32_t, uint16_t>::type key_t;
  typedef uint2 entry_t;
  HIP_DYNAMIC_SHARED(unsigned char, adc_dyn)
  const int tid = threadIdx.x;
  const int bh = blockIdx.y;
  const int vg = blockIdx.z;
  const int hk = bh % P.Hkv;
  const int b = bh / P.Hkv;
  const int G = P.Hq / P.Hkv;
  const int nvec = G * P.Lq;
  const int n_vg = (nvec + NQ - 1) / NQ;
  const int n_sub = P.n_sub, n_cent = P.n_cent;
  const int lut_n = n_sub * n_cent;
  entry_t* s_lut = (entry_t*)adc_dyn;                      // lut_n entries
  float* s_q = (float*)(adc_dyn + (size_t)lut_n * sizeof(entry_t));  // NQ x ADC_MAX_HEAD_DIM (OWN_LUT only)

  int row[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int v = vg * NQ + i;
    row[i] = -1;
    if (v < nvec) row[i] = (b * P.Hq + hk * G + v / P.Lq) * P.Lq + v % P.Lq;
  }
  // rounded to the storage type by the hardware converters (round to nearest even, as the software rounding)
  auto store_entry = [&](int i, const float (&val)[NQ]) {
    if constexpr (NQ == 2) s_lut[i] = make_uint2(sah_float_to_bits(val[0]), sah_float_to_bits(val[1]));
    else s_lut[i] = make_uint2(sah_pack2_hw<DT>(val[0], val[1]), sah_pack2_hw<DT>(val[2], val[3]));
  };
  // 16 one-byte codes per candidate = one 16-byte load: all of the thread's candidates are requested before
  // anything else and arrive while the table is built
  constexpr int T = ADC_KEYS / ADC_NT;
  const bool wide = n_sub == 16 && ((uintptr_t)P.codes & 15) == 0;
  uint4 cw[T];
  if (wide) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      int n = blockIdx.x * ADC_KEYS + t * ADC_NT + tid;
      if (n >= P.n_cand) n = P.n_cand - 1;
      cw[t] = *(const uint4*)(P.codes + ((int64_t)bh * P.code_pitch + n) * 16);
    }
  }
  if (OWN_LUT) {
    // the group's query vectors once into LDS (as floats), then every thread builds lut_n / ADC_NT entries
    // from one centre each: the centre's d_sub floats from memory, the query elements as LDS broadcasts
    const int d_sub = P.d_sub;
    const int D = n_sub * d_sub;
    for (int i = tid; i < NQ * D; i += ADC_NT) {
      const int qn = i / D, e = i % D;
      const int v = vg * NQ + qn;
      float x = 0.f;
      if (v < nvec) {
        const int h = hk * G + v / P.Lq, qi = v % P.Lq;
        x = sah_load<DT>(P.q, (int64_t)b * P.qs_b + (int64_t)h * P.qs_h + (int64_t)qi * P.qs_l + e);
      }
      s_q[qn * ADC_MAX_HEAD_DIM + e] = x;
    }
    __syncthreads();
    const bool pow2 = (n_cent & (n_cent - 1)) == 0;  // the usual case (2^bits centres): no integer division per entry
    const int shift = 31 - __builtin_clz(n_cent);
    int first = tid;  // first entry the general loop below still has to build
    if (DT != SAH_F32 && P.centres_narrow && d_sub == 8 && pow2 && n_cent >= SAH_WAVE) {
      // Sub-vectors of 8 in 16-bit storage. A wave takes whole sub-spaces (wave w: s = w, w + 16, ...), so the
      // query elements of a sub-space are read from LDS once per wave and lane instead of once per entry (those
      // broadcast reads were most of the table's cost); a lane builds the entries of centres lane, lane + 64, ...:
      // one 16-byte load per centre, up to four of them requested together.
      const int lane = tid & (SAH_WAVE - 1);
      constexpr int LE = 4;
      for (int s = sah_wave_id(); s < n_sub; s += ADC_NT / SAH_WAVE) {
        float qv[NQ][8];
#pragma unroll
        for (int qn = 0; qn < NQ; ++qn) {
          const float4 q0 = *(const float4*)&s_q[qn * ADC_MAX_HEAD_DIM + s * 8];
          const float4 q1 = *(const float4*)&s_q[qn * ADC_MAX_HEAD_DIM + s * 8 + 4];
          qv[qn][0] = q0.x; qv[qn][1] = q0.y; qv[qn][2] = q0.z; qv[qn][3] = q0.w;
          qv[qn][4] = q1.x; qv[qn][5] = q1.y; qv[qn][6] = q1.z; qv[qn][7] = q1.w;
        }
        for (int c0 = lane; c0 < n_cent; c0 += LE * SAH_WAVE) {
          uint4 raw[LE];
#pragma unroll
          for (int u = 0; u < LE; ++u) {
            int c = c0 + u * SAH_WAVE;
            if (c >= n_cent) c = n_cent - 1;
            raw[u] = *(const uint4*)((const uint16_t*)P.centres_narrow + (((int64_t)bh * n_sub + s) * n_cent + c) * 8);
          }
#pragma unroll
          for (int u = 0; u < LE; ++u) {
            const int c = c0 + u * SAH_WAVE;
            if (c < n_cent) {
              const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
              float cv[8];
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                if (DT == SAH_BF16) {
                  cv[2 * t] = sah_bits_to_float(w[t] << 16);
                  cv[2 * t + 1] = sah_bits_to_float(w[t] & 0xffff0000u);
                } else {
                  cv[2 * t] = sah_f16_to_float((uint16_t)(w[t] & 0xffffu));
                  cv[2 * t + 1] = sah_f16_to_float((uint16_t)(w[t] >> 16));
                }
              }
              float acc[NQ];
#pragma unroll
              for (int qn = 0; qn < NQ; ++qn) {
                float a = 0.f;
#pragma unroll
                for (int d = 0; d < 8; ++d) a = fmaf(qv[qn][d], cv[d], a);
                acc[qn] = a;
              }
              store_entry(s * n_cent + c, acc);
            }
          }
        }
      }
      first = lut_n;
    }
    for (int i = first; i < lut_n; i += ADC_NT) {
      const int s = pow2 ? i >> shift : i / n_cent;
      const int c = pow2 ? i & (n_cent - 1) : i % n_cent;
      const float* cc = P.centres + (((int64_t)bh * n_sub + s) * n_cent + c) * d_sub;
      float acc[NQ];
#pragma unroll
      for (int qn = 0; qn < NQ; ++qn) acc[qn] = 0.f;
      if (DT != SAH_F32 && P.centres_narrow) {
        // the centres in their 16-bit storage form: every workgroup of a KV head reads the whole codebook of the
        // head, so halving its bytes halves the larger part of this kernel's memory traffic
        for (int d = 0; d < d_sub; d += 8) {
          float cv[8];
          sah_load8<DT>(P.centres_narrow, (((int64_t)bh * n_sub + s) * n_cent + c) * d_sub + d, cv);
#pragma unroll
          for (int qn = 0; qn < NQ; ++qn) {
            const float4 q0 = *(const float4*)&s_q[qn * ADC_MAX_HEAD_DIM + s * d_sub + d];
            const float4 q1 = *(const float4*)&s_q[qn * ADC_MAX_HEAD_DIM + s * d_sub + d + 4];
            acc[qn] = fmaf(q0.x, cv[0], acc[qn]);
            acc[qn] = fmaf(q0.y, cv[1], acc[qn]);
            acc[qn] = fmaf(q0.z, cv[2], acc[qn]);
            acc[qn] = fmaf(q0.w, cv[3], acc[qn]);
            acc[qn] = fmaf(q1.x, cv[4], acc[qn]);
            acc[qn] = fmaf(q1.y, cv[5], acc[qn]);
            acc[qn] = fmaf(q1.z, cv[6], acc[qn]);
            acc[qn] = fmaf(q1.w, cv[7], acc[qn]);
          }
        }
      } else if ((d_sub & 3) == 0) {
        // 16-byte reads of the centre and of the staged queries (the same fused multiply-adds in the same order)
        for (int d = 0; d < d_sub; d += 4) {
          const float4 cv = *(const float4*)(cc + d);
#pragma unroll
          for (int qn = 0; qn < NQ; ++qn) {
            const float4 qv = *(const float4*)&s_q[qn * ADC_MAX_HEAD_DIM + s * d_sub + d];
            acc[qn] = fmaf(qv.x, cv.x, acc[qn]);
            acc[qn] = fmaf(qv.y, cv.y, acc[qn]);
            acc[qn] = fmaf(qv.z, cv.z, acc[qn]);
            acc[qn] = fmaf(qv.w, cv.w, acc[qn]);
          }
        }
      } else {
        for (int d = 0; d < d_sub; ++d) {
          const float cv = cc[d];
#pragma unroll
          for (int qn = 0; qn < NQ; ++qn) acc[qn] = fmaf(s_q[qn * ADC_MAX_HEAD_DIM + s * d_sub + d], cv, acc[qn]);
        }
      }
      store_entry(i, acc);
    }
  } else {
    const uint2* slab = (const uint2*)lut + ((int64_t)bh * n_vg + vg) * lut_n;
    for (int i = tid; i < lut_n; i += ADC_NT) s_lut[i] = slab[i];
  }
  __syncthreads();

  float acc[NQ];
  auto add = [&](int s, int c) {
    const entry_t e = s_lut[s * n_cent + c];
    if constexpr (NQ == 2) {
      acc[0] += sah_bits_to_float(e.x);
      acc[1] += sah_bits_to_float(e.y);
    } else if constexpr (DT == SAH_BF16) {
      acc[0] += sah_bits_to_float(e.x << 16);
      acc[1] += sah_bits_to_float(e.x & 0xffff0000u);
      acc[2] += sah_bits_to_float(e.y << 16);
      acc[3] += sah_bits_to_float(e.y & 0xffff0000u);
    } else {
      acc[0] += sah_f16_to_float((uint16_t)(e.x & 0xffffu));
      acc[1] += sah_f16_to_float((uint16_t)(e.x >> 16));
      acc[2] += sah_f16_to_float((uint16_t)(e.y & 0xffffu));
      acc[3] += sah_f16_to_float((uint16_t)(e.y >> 16));
    }
  };
  auto store = [&](int n) {
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      if (row[i] >= 0)
        ((key_t*)P.keys_out)[(int64_t)row[i] * P.key_pitch + n] = (key_t)sah_sort_key<DT>(sah_round<DT>(acc[i]));
    }
  };
  if (wide) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int n = blockIdx.x * ADC_KEYS + t * ADC_NT + tid;
      const uint32_t w4[4] = {cw[t].x, cw[t].y, cw[t].z, cw[t].w};
#pragma unroll
      for (int i = 0; i < NQ; ++i) acc[i] = 0.f;
#pragma unroll
      for (int s = 0; s < 16; ++s) add(s, (int)((w4[s >> 2] >> (8 * (s & 3))) & 0xffu));
      if (n < P.n_cand) store(n);
    }
    return;
  }
  const bool words = (n_sub & 3) == 0 && ((P.code_pitch * n_sub) & 3) == 0 && ((uintptr_t)P.codes & 3) == 0;
  for (int t = 0; t < T; ++t) {
    const int n = blockIdx.x * ADC_KEYS + t * ADC_NT + tid;
    if (n >= P.n_cand) continue;
    const uint8_t* code = P.codes + ((int64_t)bh * P.code_pitch + n) * n_sub;
#pragma unroll
    for (int i = 0; i < NQ; ++i) acc[i] = 0.f;
    if (words) {
      for (int s4 = 0; s4 < n_sub; s4 += 4) {
        const uint32_t w = *(const uint32_t*)(code + s4);
        add(s4, (int)(w & 0xffu));
        add(s4 + 1, (int)((w >> 8) & 0xffu));
        add(s4 + 2, (int)((w >> 16) & 0xffu));
        add(s4 + 3, (int)(w >> 24));
      }
    } else {
      for (int s = 0; s < n_sub; ++s) add(s, (int)code[s]);
    }
    store(n);
  }
}

// dynamic LDS of k_pq_adc: the table (8 bytes per entry) and, for OWN_LUT, the staged query vectors
template <int DT>
static size_t adc_lds_bytes(int lut_n) {
  constexpr int NQ = (DT == SAH_F32) ? 2 : 4;
  return (size_t)lut_n * 8 + (size_t)NQ * ADC_MAX_HEAD_DIM * 4;
}

template <int DT, bool OWN_LUT>
static int adc_launch(const pq_adc_params& P, const void* lut, dim3 g, hipStream_t st) {
  if (int rc = sah_allow_lds((const void*)k_pq_adc<DT, OWN_LUT>, 150 * 1024, "sah_pq_adc_scores")) return rc;
  hipLaunchKernelGGL((k_pq_adc<DT, OWN_LUT>), g, dim3(ADC_NT), adc_lds_bytes<DT>(P.n_sub * P.n_cent), st, P, lut);
  return SAH_OK;
}

static int pq_check_common(const char* what, int B, int Hkv, int n_sub, int d_sub, int n_cent) {
  if (B <= 0 || Hkv <= 0 || n_sub <= 0) return sah_fail(SAH_EINVAL, "%s: bad B/Hkv/n_sub", what);
  if (d_sub <= 0 || d_sub > PQM_MAX_D) return sah_fail(SAH_ESHAPE, "%s: d_sub %d not in [1, %d]", what, d_sub, PQM_MAX_D);
  if (n_cent <= 0 || n_cent > PQ_MAX_CENT) return sah_fail(SAH_ESHAPE, "%s: n_cent %d not in [1, %d]", what, n_cent, PQ_MAX_CENT);
  if ((int64_t)B * Hkv > 65535) return sah_fail(SAH_ESHAPE, "%s: B*Hkv > 65535", what);
  return SAH_OK;
}

// Largest |element| of the keys [key_offset, key_offset + n_keys) of every (b, kv head), as float bits (non-negative
// floats order like their bit patterns, so an integer atomic max does it). *out must be zero before the launch.
template <int DT>
__global__ __launch_bounds__(PQ_NT) void k_pq_absmax(const void* k, int64_t ks_b, int64_t ks_h, int64_t ks_l, int Hkv, int D,
                                                     int key_offset, int n_keys, uint32_t* out) {
  const int bh = blockIdx.y;
  const int64_t base = (int64_t)(bh / Hkv) * ks_b + (int64_t)(bh % Hkv) * ks_h;
  const int64_t total = (int64_t)n_keys * D;
  uint32_t best = 0u;
  for (int64_t i = (int64_t)blockIdx.x * PQ_NT + threadIdx.x; i < total; i += (int64_t)gridDim.x * PQ_NT) {
    const int n = (int)(i / D), d = (int)(i % D);
    const uint32_t bits = sah_float_to_bits(sah_load<DT>(k, base + (int64_t)(key_offset + n) * ks_l + d)) & 0x7fffffffu;
    if (bits <= 0x7f800000u) best = bits > best ? bits : best;  // NaN is skipped
  }
#pragma unroll
  for (int o = 1; o < SAH_WAVE; o <<= 1) {
    const uint32_t other = (uint32_t)__shfl_xor((int)best, o);
    best = other > best ? other : best;
  }
  if ((threadIdx.x & (SAH_WAVE - 1)) == 0 && best) atomicMax(out, best);
}

extern "C" int sah_pq_keys_absmax(const sah_pq_absmax_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_pq_keys_absmax: args is NULL");
  if (!a->k || !a->absmax_bits) return sah_fail(SAH_ENULL, "sah_pq_keys_absmax: NULL tensor");
  if (a->B <= 0 || a->Hkv <= 0 || a->D <= 0 || a->key_offset < 0 || a->n_keys < 0 || (int64_t)a->B * a->Hkv > 65535)
    return sah_fail(SAH_EINVAL, "sah_pq_keys_absmax: bad B/Hkv/D/key range");
  if (a->n_keys == 0) return SAH_OK;
  const int64_t total = (int64_t)a->n_keys * a->D;
  int gx = (int)((total + PQ_NT * 16 - 1) / (PQ_NT * 16));
  gx = gx < 1 ? 1 : (gx > 64 ? 64 : gx);
  dim3 g(gx, a->B * a->Hkv), blk(PQ_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_pq_absmax", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_pq_absmax<SAH_F32>, g, blk, 0, st, a->k, a->ks_b, a->ks_h, a->ks_l, a->Hkv, a->D, a->key_offset, a->n_keys, a->absmax_bits); break;
    case SAH_BF16: hipLaunchKernelGGL(k_pq_absmax<SAH_BF16>, g, blk, 0, st, a->k, a->ks_b, a->ks_h, a->ks_l, a->Hkv, a->D, a->key_offset, a->n_keys, a->absmax_bits); break;
    case SAH_F16: hipLaunchKernelGGL(k_pq_absmax<SAH_F16>, g, blk, 0, st, a->k, a->ks_b, a->ks_h, a->ks_l, a->Hkv, a->D, a->key_offset, a->n_keys, a->absmax_bits); break;
    default: return sah_fail(SAH_EDTYPE, "sah_pq_keys_absmax: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_pq_keys_absmax");
}

extern "C" int sah_pq_kmeans_assign(const sah_pq_assign_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_pq_kmeans_assign: args is NULL");
  int rc = pq_check_common("sah_pq_kmeans_assign", a->B, a->Hkv, a->n_sub, a->d_sub, a->n_cent);
  if (rc) return rc;
  if (!a->k || !a->centres || !a->codes) return sah_fail(SAH_ENULL, "sah_pq_kmeans_assign: NULL tensor");
  if ((a->sums == nullptr) != (a->counts == nullptr)) return sah_fail(SAH_EINVAL, "sah_pq_kmeans_assign: sums and counts go together");
  if (a->sums && !a->absmax_bits) return sah_fail(SAH_ENULL, "sah_pq_kmeans_assign: sums need absmax_bits (sah_pq_keys_absmax)");
  if (a->n_keys <= 0) return SAH_OK;
  if (a->key_offset < 0 || a->code_offset < 0 || a->code_pitch < a->code_offset + a->n_keys)
    return sah_fail(SAH_ECAPACITY, "sah_pq_kmeans_assign: code_pitch %lld < code_offset %lld + n_keys %d",
                    (long long)a->code_pitch, (long long)a->code_offset, a->n_keys);
  pq_assign_params P;
  P.k = a->k; P.ks_b = a->ks_b; P.ks_h = a->ks_h; P.ks_l = a->ks_l;
  P.Hkv = a->Hkv; P.n_sub = a->n_sub; P.d_sub = a->d_sub; P.n_cent = a->n_cent;
  P.key_offset = a->key_offset; P.n_keys = a->n_keys;
  P.centres = a->centres;
  P.codes = a->codes; P.code_pitch = a->code_pitch; P.code_offset = a->code_offset;
  P.sums = (long long*)a->sums; P.counts = a->counts;
  P.absmax_bits = a->absmax_bits;
  P.round_dist = a->round_dist;
  P.skip_flag = a->skip_flag;
  hipStream_t st = (hipStream_t)a->stream;
  const bool wide = a->d_sub > PQ_MAX_D;  // no kernel keeps such a key in registers
  if (wide && a->round_dist && a->sums)
    return sah_fail(SAH_ESHAPE, "sah_pq_kmeans_assign: rounded distances with sums need d_sub <= %d", PQ_MAX_D);
  if ((!a->sums && !a->skip_flag && a->n_keys <= 32) || (wide && a->round_dist)) {
    // new keys of a decode step (or, for wide sub-vectors, any number of keys against frozen centres)
    for (int first = 0; first < a->n_keys; first += 32768) {
      pq_assign_params Q = P;
      Q.key_offset += first; Q.code_offset += first;
      Q.n_keys = a->n_keys - first < 32768 ? a->n_keys - first : 32768;
      dim3 gf(a->n_sub, a->B * a->Hkv, Q.n_keys), blk(PQ_NT);
      sah_timed timed("k_pq_assign_few", a->stream);
      switch (a->dtype) {
        case SAH_F32: hipLaunchKernelGGL(k_pq_assign_few<SAH_F32>, gf, blk, 0, st, Q); break;
        case SAH_BF16: hipLaunchKernelGGL(k_pq_assign_few<SAH_BF16>, gf, blk, 0, st, Q); break;
        case SAH_F16: hipLaunchKernelGGL(k_pq_assign_few<SAH_F16>, gf, blk, 0, st, Q); break;
        default: return sah_fail(SAH_EDTYPE, "sah_pq_kmeans_assign: dtype %d", a->dtype);
      }
      if (int rc2 = sah_launch_status("sah_pq_kmeans_assign")) return rc2;
    }
    return SAH_OK;
  }
  if (!wide && !a->sums && !a->skip_flag && a->n_keys <= 512) {  // a block of new keys of a decode plan
    dim3 gb(a->n_sub, a->B * a->Hkv), blk(PQB_NT);
    sah_timed timed("k_pq_assign_block", a->stream);
    switch (a->dtype) {
      case SAH_F32: hipLaunchKernelGGL(k_pq_assign_block<SAH_F32>, gb, blk, 0, st, P); break;
      case SAH_BF16: hipLaunchKernelGGL(k_pq_assign_block<SAH_BF16>, gb, blk, 0, st, P); break;
      case SAH_F16: hipLaunchKernelGGL(k_pq_assign_block<SAH_F16>, gb, blk, 0, st, P); break;
      default: return sah_fail(SAH_EDTYPE, "sah_pq_kmeans_assign: dtype %d", a->dtype);
    }
    return sah_launch_status("sah_pq_kmeans_assign");
  }
  if (!a->round_dist && (wide || (a->n_keys >= 1024 && (a->d_sub == 4 || a->d_sub == 8 || a->d_sub == 16)))) {
    // Lloyd iterations over a whole context: the contraction goes to the matrix cores
    switch (a->dtype) {
      case SAH_F32: return pq_launch_mfma<SAH_F32>(a, P);
      case SAH_BF16: return pq_launch_mfma<SAH_BF16>(a, P);
      case SAH_F16: return pq_launch_mfma<SAH_F16>(a, P);
      default: return sah_fail(SAH_EDTYPE, "sah_pq_kmeans_assign: dtype %d", a->dtype);
    }
  }
  const int per_wg = PQ_NT * PQ_TILES;
  dim3 g(((a->n_keys + per_wg - 1) / per_wg) * a->n_sub, a->B * a->Hkv), blk(PQ_NT);
  sah_timed timed("k_pq_assign", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_pq_assign<SAH_F32>, g, blk, 0, st, P); break;
    case SAH_BF16: hipLaunchKernelGGL(k_pq_assign<SAH_BF16>, g, blk, 0, st, P); break;
    case SAH_F16: hipLaunchKernelGGL(k_pq_assign<SAH_F16>, g, blk, 0, st, P); break;
    default: return sah_fail(SAH_EDTYPE, "sah_pq_kmeans_assign: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_pq_kmeans_assign");
}

extern "C" int sah_pq_kmeans_update(const sah_pq_update_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_pq_kmeans_update: args is NULL");
  int rc = pq_check_common("sah_pq_kmeans_update", a->B, a->Hkv, a->n_sub, a->d_sub, a->n_cent);
  if (rc) return rc;
  if (!a->k || !a->centres || !a->sums || !a->counts || !a->reseed_idx || !a->shift2 || !a->state || !a->absmax_bits)
    return sah_fail(SAH_ENULL, "sah_pq_kmeans_update: NULL tensor");
  pq_update_params P;
  P.k = a->k; P.ks_b = a->ks_b; P.ks_h = a->ks_h; P.ks_l = a->ks_l;
  P.Hkv = a->Hkv; P.n_sub = a->n_sub; P.d_sub = a->d_sub; P.n_cent = a->n_cent; P.key_offset = a->key_offset;
  P.centres = a->centres; P.sums = (const long long*)a->sums; P.counts = a->counts; P.reseed_idx = a->reseed_idx;
  P.absmax_bits = a->absmax_bits;
  P.shift2 = a->shift2; P.tol = a->tol; P.state = a->state;
  P.n_groups = a->B * a->Hkv * a->n_sub;
  dim3 g(P.n_groups), blk(PQ_NT);
  hipStream_t st = (hipStream_t)a->stream;
  {
    sah_timed timed("k_pq_update", a->stream);
    switch (a->dtype) {
      case SAH_F32: hipLaunchKernelGGL(k_pq_update<SAH_F32>, g, blk, 0, st, P); break;
      case SAH_BF16: hipLaunchKernelGGL(k_pq_update<SAH_BF16>, g, blk, 0, st, P); break;
      case SAH_F16: hipLaunchKernelGGL(k_pq_update<SAH_F16>, g, blk, 0, st, P); break;
      default: return sah_fail(SAH_EDTYPE, "sah_pq_kmeans_update: dtype %d", a->dtype);
    }
  }
  rc = sah_launch_status("sah_pq_kmeans_update");
  if (rc) return rc;
  hipLaunchKernelGGL(k_pq_promote, dim3(1), dim3(SAH_WAVE), 0, st, a->state);
  return sah_launch_status("sah_pq_kmeans_update(promote)");
}

extern "C" int64_t sah_pq_adc_lut_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lq, int32_t n_sub, int32_t n_cent,
                                        int32_t dtype) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Lq <= 0 || n_sub <= 0 || n_cent <= 0 || Hq % Hkv) return 0;
  const int nq = dtype == SAH_F32 ? 2 : 4;
  const int n_vg = ((Hq / Hkv) * Lq + nq - 1) / nq;
  return (int64_t)B * Hkv * n_vg * n_sub * n_cent * 8;
}

extern "C" int sah_pq_adc_scores(const sah_pq_adc_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_pq_adc_scores: args is NULL");
  int rc = pq_check_common("sah_pq_adc_scores", a->B, a->Hkv, a->n_sub, a->d_sub, a->n_cent);
  if (rc) return rc;
  if (!a->q || !a->centres || !a->codes || !a->keys_out) return sah_fail(SAH_ENULL, "sah_pq_adc_scores: NULL tensor");
  if (a->Hq <= 0 || a->Lq <= 0 || a->Hq % a->Hkv) return sah_fail(SAH_EINVAL, "sah_pq_adc_scores: bad Hq/Lq");
  if (a->n_sub * a->n_cent > ADC_MAX_LUT) return sah_fail(SAH_ESHAPE, "sah_pq_adc_scores: n_sub*n_cent > %d", ADC_MAX_LUT);
  if (a->n_cand <= 0) return SAH_OK;
  if (a->code_pitch < a->n_cand || a->key_pitch < a->n_cand) return sah_fail(SAH_ECAPACITY, "sah_pq_adc_scores: pitch < n_cand");
  pq_adc_params P;
  P.q = a->q; P.qs_b = a->qs_b; P.qs_h = a->qs_h; P.qs_l = a->qs_l;
  P.Hq = a->Hq; P.Hkv = a->Hkv; P.Lq = a->Lq; P.n_sub = a->n_sub; P.d_sub = a->d_sub; P.n_cent = a->n_cent;
  P.centres = a->centres; P.codes = a->codes; P.code_pitch = a->code_pitch; P.n_cand = a->n_cand;
  P.centres_narrow = (a->dtype != SAH_F32 && a->d_sub % 8 == 0 && ((uintptr_t)a->centres_narrow % 16) == 0) ? a->centres_narrow : nullptr;
  P.keys_out = a->keys_out; P.key_pitch = a->key_pitch;
  const int nvec = (a->Hq / a->Hkv) * a->Lq;
  const int nq = a->dtype == SAH_F32 ? 2 : 4;
  const int n_vg = (nvec + nq - 1) / nq;
  if (n_vg > 65535) return sah_fail(SAH_ESHAPE, "sah_pq_adc_scores: too many query vectors per KV head");
  hipStream_t st = (hipStream_t)a->stream;
  const int wgs_per_head = (a->n_cand + ADC_KEYS - 1) / ADC_KEYS;
  dim3 g(wgs_per_head, a->B * a->Hkv, n_vg), blk(PQ_NT);
  if (wgs_per_head <= ADC_OWN_LUT_WGS && a->n_sub * a->d_sub <= ADC_MAX_HEAD_DIM) {
    // short contexts: no table in memory, no second launch
    sah_timed timed("k_pq_adc", a->stream);
    switch (a->dtype) {
      case SAH_F32: rc = adc_launch<SAH_F32, true>(P, nullptr, g, st); break;
      case SAH_BF16: rc = adc_launch<SAH_BF16, true>(P, nullptr, g, st); break;
      case SAH_F16: rc = adc_launch<SAH_F16, true>(P, nullptr, g, st); break;
      default: return sah_fail(SAH_EDTYPE, "sah_pq_adc_scores: dtype %d", a->dtype);
    }
    if (rc) return rc;
    return sah_launch_status("sah_pq_adc_scores");
  }
  const int64_t need = (int64_t)a->B * a->Hkv * n_vg * a->n_sub * a->n_cent * 8;
  if (!a->lut || a->lut_bytes < need)
    return sah_fail(SAH_ECAPACITY, "sah_pq_adc_scores: lut holds %lld bytes, need %lld", (long long)(a->lut ? a->lut_bytes : 0),
                    (long long)need);
  {
    dim3 gl(a->n_sub, a->B * a->Hkv, n_vg);
    sah_timed timed("k_pq_lut", a->stream);
    switch (a->dtype) {
      case SAH_F32: hipLaunchKernelGGL(k_pq_lut<SAH_F32>, gl, blk, 0, st, P, a->lut); break;
      case SAH_BF16: hipLaunchKernelGGL(k_pq_lut<SAH_BF16>, gl, blk, 0, st, P, a->lut); break;
      case SAH_F16: hipLaunchKernelGGL(k_pq_lut<SAH_F16>, gl, blk, 0, st, P, a->lut); break;
      default: return sah_fail(SAH_EDTYPE, "sah_pq_adc_scores: dtype %d", a->dtype);
    }
    rc = sah_launch_status("sah_pq_adc_scores(lut)");
    if (rc) return rc;
  }
  sah_timed timed("k_pq_adc", a->stream);
  switch (a->dtype) {
    case SAH_F32: rc = adc_launch<SAH_F32, false>(P, a->lut, g, st); break;
    case SAH_BF16: rc = adc_launch<SAH_BF16, false>(P, a->lut, g, st); break;
    default: rc = adc_launch<SAH_F16, false>(P, a->lut, g, st); break;
  }
  if (rc) return rc;
  return sah_launch_status("sah_pq_adc_scores");
}
