// Signature (Hamming) top-k of one mask row, SWAR form: shared by the stand-alone kernel and the
// fused decode kernel.
#pragma once
#include "sah_common.h"

// signature score of the reference, sum_e q_e k_e with q_e, k_e in {-1, 0, +1}:
// popc(nz) - 2 popc((q ^ k) & nz), nz = bits where both are non-zero; in [-32, 32]
__device__ __forceinline__ int sig_score(uint2 q, uint2 k) {
  const uint32_t nz = q.y & k.y;
  return __popc(nz) - 2 * __popc((q.x ^ k.x) & nz);
}

// ---------------------------------------------------------------------------
// Signature top-k, SWAR form. Scores fit a byte (score + 33 in [1, 65], 0 = column already
// active or out of range), so a lane handles 4 consecutive columns as one 32-bit word:
//   P0  each lane loads its 4 codes (32 B, whole wave: 2 KB contiguous; in the compact form of the stream 16 B of
//       sign planes, with the few columns that have a zero component corrected afterwards), scores them, zeroes
//       the already-active ones with a nibble of the bitmap row and parks the word in LDS;
//   P1  the threshold T: P0 has already counted the columns at or above 8 probe thresholds, one more
//       pass over the staged bytes counts the 3 inside the bracket (byte-parallel compares);
//   P2  per-lane bit masks "above T" / "equal T" of the lane's columns, per-wave counts of both;
//   P3  write: a wave scan of per-lane counts, every lane appends the set bits of its mask; ties are
//       taken lowest column first until `need` are used (the one wave where the budget runs out ranks
//       its ties in column order); new bits are OR-ed into the LDS copy of the bitmap row, which is
//       written back once at the end.
// Active columns hold byte 0 and T >= 1 whenever k inactive columns exist, so P2/P3 never
// look at the bitmap again.
// ---------------------------------------------------------------------------
#define HSW_NT 1024
#define HSW_NW (HSW_NT / SAH_WAVE)
#define HSW_BATCH 2  // 256-column chunks per register buffer in P0 (two buffers in flight)

// per byte b < 128 of w: 0x80 if b >= t (t in [0, 128]) else 0
__device__ __forceinline__ uint32_t swar_ge(uint32_t w, uint32_t t) {
  return ((w | 0x80808080u) - t * 0x01010101u) & 0x80808080u;
}

#define HSW_GC 8      // chunks per mask group of P2 / P3: 8 x 4 columns of a lane = one 32-bit mask
#define HSW_PROBES 8  // thresholds counted while the scores are staged
// Probe i: 32, 36, ... 60. Scores + 33 lie in [1, 65] around 33, and a top-k of less than half the row has its
// threshold above that, so these eight bracket it to 4 values in the usual case; below 32 a second set
// (4, 8, ... 28) is counted from the staged bytes, from 60 up the last bracket is resolved in one 7-way pass.
__host__ __device__ constexpr uint32_t hsw_probe_at(int i) { return 32u + 4u * (uint32_t)i; }

struct hsw_lds {
  int gt[HSW_NW];
  int eq[HSW_NW];
  int probe[HSW_PROBES];  // workgroup totals of the coarse and of the fine counts: one LDS atomic per wave and
  int fine[HSW_PROBES];   // counter, read back by everyone after the barrier; zeroed by hsw_lds_init
  int low[HSW_PROBES];    // the second probe set (thresholds below 32), counted only when the first one misses
};

// Clears the counters of `S`. To be called by every thread before the barrier that precedes hsw_select_row.
__device__ __forceinline__ void hsw_lds_init(hsw_lds& S) {
  if (threadIdx.x < HSW_PROBES) {
    S.probe[threadIdx.x] = 0;
    S.fine[threadIdx.x] = 0;
    S.low[threadIdx.x] = 0;
  }
}

// LDS words the row needs: bitmap (padded to whole chunks) and one byte per column
__host__ __device__ inline size_t hsw_lds_bytes(int n_keys) {
  const int n_ch = (n_keys + 255) / 256;
  return (size_t)n_ch * 8 * 4 + (size_t)n_ch * 64 * 4;
}

// Compact form of a row's code stream, for rows whose keys almost never have a zero signature component: one
// 32-bit sign plane per column (`pos`, 4 B instead of 8), scored as if every component were non-zero, plus the
// list of the columns for which that is not true (`exc`: column, non-zero plane, sign plane, unused), whose
// scores are corrected after staging. *exc_cnt entries exist; a count above exc_cap means the list overflowed,
// and every column is then checked against the two-plane stream `full`.
struct hsw_compact {
  const uint32_t* pos;   // this row's sign planes; readable up to (16 * chunks per wave + 8) * 256 columns
  const uint4* exc;      // this row's exception entries (exc_cap >= HSW_NT of them allocated)
  const int* exc_cnt;    // this row's exception count
  const uint2* full;     // this row's two-plane codes
  int exc_cap;
  uint32_t full_plane;   // non-zero plane of a key without zero components
};

#define HSW_CBATCH 4  // compact stream: 256-column chunks per register buffer (16 B per lane and chunk)

// Register buffers of the staging pass: two batches of HSW_BATCH chunks (4 codes = 32 B per lane and chunk),
// or, for the compact stream, two batches of HSW_CBATCH chunks (4 sign planes = 16 B) and the row's first
// exception entry per thread.
template <bool CP>
struct hsw_bufs_t {
  uint4 a0[HSW_BATCH], a1[HSW_BATCH], b0[HSW_BATCH], b1[HSW_BATCH];
};
template <>
struct hsw_bufs_t<true> {
  uint4 a[HSW_CBATCH], b[HSW_CBATCH];
  uint4 exc_first;
  int exc_n;
};
typedef hsw_bufs_t<false> hsw_bufs;

// wave `wave` stages the chunks [c0, c1) of a row of n columns
__device__ __forceinline__ void hsw_wave_chunks(int n, int wave, int& c0, int& c1) {
  const int n_ch = (n + 255) / 256;
  const int cpw = (n_ch + HSW_NW - 1) / HSW_NW;
  c0 = wave * cpw;
  c1 = c0 + cpw;
  if (c1 > n_ch) c1 = n_ch;
}

__device__ __forceinline__ void hsw_request(const uint2* kc, int n, int lane, uint4 (&ra)[HSW_BATCH], uint4 (&rb)[HSW_BATCH],
                                            int c0) {
#pragma unroll
  for (int u = 0; u < HSW_BATCH; ++u) {
    const int j0 = ((c0 + u) * SAH_WAVE + lane) * 4;
    // clamp to the last full group of 4 codes: out-of-range lanes re-read valid memory
    int jl = j0;
    if (jl + 4 > n) jl = n >= 4 ? ((n - 4) & ~1) : 0;
    const uint4* p = (const uint4*)(kc + jl);
    ra[u] = p[0];
    rb[u] = p[1];
  }
}

// Requests the first two batches of the calling wave ahead of hsw_select_row(..., prefetched = true): the codes
// do not depend on the query, so a caller that still has to compute the query code can have them on their way.
__device__ __forceinline__ void hsw_prefetch(const uint2* kc, int n, hsw_bufs& buf) {
  const int lane = threadIdx.x & (SAH_WAVE - 1);
  int c0, c1;
  hsw_wave_chunks(n, sah_wave_id(), c0, c1);
  (void)c1;  // no conditions: a request past the row's end re-reads valid memory and is never scored
  hsw_request(kc, n, lane, buf.a0, buf.a1, c0);
  hsw_request(kc, n, lane, buf.b0, buf.b1, c0 + HSW_BATCH);
}

__device__ __forceinline__ void hsw_request_c(const uint32_t* pos, int lane, uint4 (&rc)[HSW_CBATCH], int c0) {
#pragma unroll
  for (int u = 0; u < HSW_CBATCH; ++u) rc[u] = *(const uint4*)(pos + ((c0 + u) * SAH_WAVE + lane) * 4);
}

// the same for the compact stream: the calling wave's first 8 chunks (a row of up to 32768 columns completely),
// the row's exception count and the calling thread's first exception entry
__device__ __forceinline__ void hsw_prefetch(const hsw_compact& cs, int n, hsw_bufs_t<true>& buf) {
  const int lane = threadIdx.x & (SAH_WAVE - 1);
  int c0, c1;
  hsw_wave_chunks(n, sah_wave_id(), c0, c1);
  (void)c1;
  hsw_request_c(cs.pos, lane, buf.a, c0);
  hsw_request_c(cs.pos, lane, buf.b, c0 + HSW_CBATCH);
  buf.exc_n = *cs.exc_cnt;
  buf.exc_first = cs.exc[threadIdx.x];
}

// Top-k of row r over the not-yet-active columns. On entry `s_bm` (n_ch * 8 words of dynamic LDS, zero
// padded) holds the row's bitmap, hsw_lds_init(S) has run, and every thread of the workgroup has passed a
// barrier after both; cnt0 entries of R.cols are already in place. On exit the selected columns are appended (in no
// particular order) and cnt is updated; with update_bitmap also the bitmap row (LDS copy and global).
// Returns the row's new entry count (every thread). s_cols: optional LDS copy of the row's column list (cap entries):
// the appended columns are mirrored there for a caller that goes on to use them in the same kernel (the mirror
// is complete only after the caller's next barrier).
// CP: the row's codes come in the compact form `cs` (kc is not used).
// active_below / active_from (both >= 0): the caller knows that the row's active columns are exactly
// [0, active_below) and [active_from, n) (the sink and local columns of a fresh decode row); chunks that lie between
// the two ranges then skip the bitmap test of every word.
template <bool CP = false>
__device__ __forceinline__ int hsw_select_row(const sah_rows& R, int r, const uint2* kc, const uint2 q, int k, int cnt0,
                                              uint32_t* s_bm, uint32_t* s_key, hsw_lds& S, hsw_bufs_t<CP>& buf,
                                              bool prefetched = false, bool update_bitmap = true, int* s_cols = nullptr,
                                              const hsw_compact* cs = nullptr, int active_below = -1, int active_from = -1) {
  int* s_gt = S.gt;
  int* s_eq = S.eq;
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  const int n = R.n_keys;
  const int n_ch = (n + 255) / 256;            // chunks of 256 columns = 64 words
  int my_c0, my_c1;
  hsw_wave_chunks(n, wave, my_c0, my_c1);
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;
  if (k > n) k = n;

  // ---- P0: score and stage --------------------------------------------------
  // While the codes stream in the ALUs are idle: count, on the side, the columns at or above each of
  // HSW_PROBES coarse thresholds, so that P1 only has to resolve the last 3 bits of the threshold.
  int pc[HSW_PROBES];
#pragma unroll
  for (int i = 0; i < HSW_PROBES; ++i) pc[i] = 0;
  // what staging a word has in common: zero the bytes of already-active columns, park the word, count the probes
  const bool ranges_known = active_below >= 0 && active_from >= 0;
  // may chunk c hold an active column? (uniform across the wave)
  auto chunk_may_be_active = [&](int c) { return !ranges_known || c * 256 < active_below || (c + 1) * 256 > active_from; };
  auto stage = [&](uint32_t word, int wi, bool check) {
    uint32_t kw = word;
    if (check) {
      const int j0 = wi * 4;
      // Most chunks of a long row hold no active column at all: uniform test, the expansion is skipped
      const uint32_t nib = (s_bm[j0 >> 5] >> (j0 & 31)) & 0xFu;  // nibble -> byte mask
      if (__ballot(nib != 0)) {
        const uint32_t one = (nib | (nib << 7) | (nib << 14) | (nib << 21)) & 0x01010101u;
        kw = word & ~((one << 8) - one);
      }
    }
    s_key[wi] = kw;
    const uint32_t x = kw | 0x80808080u;
#pragma unroll
    for (int i = 0; i < HSW_PROBES; ++i) pc[i] += __popc((x - hsw_probe_at(i) * 0x01010101u) & 0x80808080u);
  };
  if constexpr (CP) {
    // ---- compact stream: every component taken as non-zero, score = popc(q.y) - 2 popc((q.x ^ k.x) & q.y)
    const uint32_t s_full = (uint32_t)__popc(q.y) + 33u;
    const uint32_t s_full4 = s_full * 0x01010101u;
    // a query without zero components (the usual case) needs no mask on the differing bits; uniform
    const bool q_dense = q.y == 0xFFFFFFFFu;
    // four scores as the bytes of a word: the four mismatch counts are packed first, then one multiply-add turns
    // them into scores (a count is at most popc(q.y), so no byte borrows from its neighbour)
    auto word_of = [&](const uint4& k4) {
      uint32_t m0 = q.x ^ k4.x, m1 = q.x ^ k4.y, m2 = q.x ^ k4.z, m3 = q.x ^ k4.w;
      if (!q_dense) {
        m0 &= q.y; m1 &= q.y; m2 &= q.y; m3 &= q.y;
      }
      const uint32_t p4 = (uint32_t)__popc(m0) | ((uint32_t)__popc(m1) << 8) | ((uint32_t)__popc(m2) << 16) | ((uint32_t)__popc(m3) << 24);
      return s_full4 - 2u * p4;
    };
    auto score_c = [&](uint4 (&rc)[HSW_CBATCH], int c0) {
#pragma unroll
      for (int u = 0; u < HSW_CBATCH; ++u) {
        sah_keep(rc[u].x); sah_keep(rc[u].y); sah_keep(rc[u].z); sah_keep(rc[u].w);
      }
#pragma unroll
      for (int u = 0; u < HSW_CBATCH; ++u) {
        if (c0 + u >= my_c1) break;
        const int wi = (c0 + u) * SAH_WAVE + lane;
        const int j0 = wi * 4;
        uint32_t word = word_of(rc[u]);
        // ragged tail: the stream is readable beyond the row, what lies there scores nothing
        if (j0 + 4 > n) word = j0 < n ? word & ((1u << (8 * (n - j0))) - 1u) : 0u;
        stage(word, wi, chunk_may_be_active(c0 + u));
      }
    };
    if (!prefetched) {
      buf.exc_n = *cs->exc_cnt;
      buf.exc_first = cs->exc[tid];
      if (my_c0 < my_c1) hsw_request_c(cs->pos, lane, buf.a, my_c0);
    }
    for (int c0 = my_c0; c0 < my_c1; c0 += 2 * HSW_CBATCH) {
      const bool more_b = c0 + HSW_CBATCH < my_c1;          // uniform across the wave
      if (more_b && !(prefetched && c0 == my_c0)) hsw_request_c(cs->pos, lane, buf.b, c0 + HSW_CBATCH);
      score_c(buf.a, c0);
      if (c0 + 2 * HSW_CBATCH < my_c1) hsw_request_c(cs->pos, lane, buf.a, c0 + 2 * HSW_CBATCH);
      if (more_b) score_c(buf.b, c0 + HSW_CBATCH);
    }
    // ---- the columns with a zero component: exact score from both planes, staged byte and probe counts corrected
    __syncthreads();  // every word is staged
    unsigned char* s_byte = (unsigned char*)s_key;
    auto patch = [&](int col, uint32_t kx, uint32_t ky) {
      if (col < n && !((s_bm[col >> 5] >> (col & 31)) & 1u)) {
        const uint32_t s_new = (uint32_t)(sig_score(q, make_uint2(kx, ky)) + 33);
        const uint32_t s_old = s_byte[col];
        s_byte[col] = (unsigned char)s_new;
#pragma unroll
        for (int i = 0; i < HSW_PROBES; ++i)
          pc[i] += (int)(s_new >= hsw_probe_at(i)) - (int)(s_old >= hsw_probe_at(i));
      }
    };
    const int n_exc = __builtin_amdgcn_readfirstlane(buf.exc_n);
    if (n_exc <= cs->exc_cap) {
      for (int e = tid; e < n_exc; e += HSW_NT) {
        const uint4 en = e == tid ? buf.exc_first : cs->exc[e];
        patch((int)en.x, en.z, en.y);
      }
    } else {  // the list overflowed: every column from the two-plane stream
      for (int col = tid; col < n; col += HSW_NT) {
        const uint2 c = cs->full[col];
        if (c.y != cs->full_plane) patch(col, c.x, c.y);
      }
    }
  } else {
    // Two register buffers of HSW_BATCH chunks each: the next batch is requested before the current one is
    // scored, so the memory pipe stays busy while the ALUs work.
    auto score = [&](uint4 (&ra)[HSW_BATCH], uint4 (&rb)[HSW_BATCH], int c0) {
#pragma unroll
      for (int u = 0; u < HSW_BATCH; ++u) {
        sah_keep(ra[u].x); sah_keep(ra[u].y); sah_keep(ra[u].z); sah_keep(ra[u].w);
        sah_keep(rb[u].x); sah_keep(rb[u].y); sah_keep(rb[u].z); sah_keep(rb[u].w);
      }
#pragma unroll
      for (int u = 0; u < HSW_BATCH; ++u) {
        if (c0 + u >= my_c1) break;
        const int wi = (c0 + u) * SAH_WAVE + lane;
        const int j0 = wi * 4;
        uint32_t word;
        if (j0 + 4 <= n) {
          const uint32_t s0 = (uint32_t)(sig_score(q, make_uint2(ra[u].x, ra[u].y)) + 33);
          const uint32_t s1 = (uint32_t)(sig_score(q, make_uint2(ra[u].z, ra[u].w)) + 33);
          const uint32_t s2 = (uint32_t)(sig_score(q, make_uint2(rb[u].x, rb[u].y)) + 33);
          const uint32_t s3 = (uint32_t)(sig_score(q, make_uint2(rb[u].z, rb[u].w)) + 33);
          word = s0 | (s1 << 8) | (s2 << 16) | (s3 << 24);
        } else {
          word = 0;  // ragged tail: the few columns of the last, partial group
          for (int t = 0; t < 4; ++t)
            if (j0 + t < n) word |= (uint32_t)(sig_score(q, kc[j0 + t]) + 33) << (8 * t);
        }
        stage(word, wi, chunk_may_be_active(c0 + u));
      }
    };
    if (!prefetched && my_c0 < my_c1) hsw_request(kc, n, lane, buf.a0, buf.a1, my_c0);
    for (int c0 = my_c0; c0 < my_c1; c0 += 2 * HSW_BATCH) {
      const bool more_b = c0 + HSW_BATCH < my_c1;          // uniform across the wave
      if (more_b && !(prefetched && c0 == my_c0)) hsw_request(kc, n, lane, buf.b0, buf.b1, c0 + HSW_BATCH);
      score(buf.a0, buf.a1, c0);
      if (c0 + 2 * HSW_BATCH < my_c1) hsw_request(kc, n, lane, buf.a0, buf.a1, c0 + 2 * HSW_BATCH);
      if (more_b) score(buf.b0, buf.b1, c0 + HSW_BATCH);
    }
  }
  // Wave totals, two counters to a register as signed 16-bit fields: a wave stages at most 64 * 4 * 35 columns,
  // and the corrections a wave's lanes made (to columns anywhere in the row) can take its total a little below
  // zero; only the workgroup's totals are counts.
#pragma unroll
  for (int i = 0; i < HSW_PROBES; i += 2) {
    const int t = sah_wave_sum_i((int)((uint32_t)pc[i] + ((uint32_t)pc[i + 1] << 16)));
    const int lo = (int)(int16_t)(t & 0xFFFF);
    if (lane == 0) {
      atomicAdd(&S.probe[i], lo);
      atomicAdd(&S.probe[i + 1], (t - lo) >> 16);
    }
  }
  __syncthreads();

  // ---- P1: largest T with count(key >= T) >= k --------------------------------
  // counts fall as the threshold rises, so the thresholds that still reach k form a prefix
  const int n_w = n_ch * SAH_WAVE;
  const int tot = lane < HSW_PROBES ? S.probe[lane] : 0;
  const int n_pass = __popcll(__ballot(lane < HSW_PROBES && tot >= k));
  uint32_t base;   // T is in [base, base + n_f + 1)
  int n_f;         // fine thresholds base + 1 .. base + n_f to count: 3, or 7 in the top bracket
  int next_probe;  // count(key >= base + n_f + 1)
  if (n_pass >= 1 && n_pass < HSW_PROBES) {
    base = hsw_probe_at(n_pass - 1);
    n_f = 3;
    next_probe = __shfl(tot, n_pass);
  } else if (n_pass == HSW_PROBES) {
    base = hsw_probe_at(HSW_PROBES - 1);  // 60: scores end at 65, so count(key >= 68) = 0
    n_f = 7;
    next_probe = 0;
  } else {
    // T < 32: the second probe set, thresholds 4, 8, ... 28, from the staged bytes
    int lc[7];
#pragma unroll
    for (int j = 0; j < 7; ++j) lc[j] = 0;
    for (int i = tid; i < n_w; i += HSW_NT) {
      const uint32_t x = s_key[i] | 0x80808080u;
#pragma unroll
      for (int j = 0; j < 7; ++j) lc[j] += __popc((x - (uint32_t)(4 * (j + 1)) * 0x01010101u) & 0x80808080u);
    }
#pragma unroll
    for (int j = 0; j < 7; j += 2) {
      const uint32_t t = (uint32_t)sah_wave_sum_i(lc[j] + ((j + 1 < 7 ? lc[j + 1] : 0) << 16));
      if (lane == 0) {
        atomicAdd(&S.low[j], (int)(t & 0xFFFFu));
        if (j + 1 < 7) atomicAdd(&S.low[j + 1], (int)(t >> 16));
      }
    }
    __syncthreads();
    const int ltot = lane < 7 ? S.low[lane] : 0;
    const int n_low = __popcll(__ballot(lane < 7 && ltot >= k));
    base = 4u * (uint32_t)n_low;
    n_f = 3;
    next_probe = n_low < 7 ? __shfl(ltot, n_low) : __shfl(tot, 0);
  }
  int fc[7];
#pragma unroll
  for (int j = 0; j < 7; ++j) fc[j] = 0;
  if (n_f == 3) {  // uniform across the workgroup
    for (int i = tid; i < n_w; i += HSW_NT) {
      const uint32_t x = s_key[i] | 0x80808080u;
#pragma unroll
      for (int j = 0; j < 3; ++j) fc[j] += __popc((x - (base + 1u + j) * 0x01010101u) & 0x80808080u);
    }
  } else {
    for (int i = tid; i < n_w; i += HSW_NT) {
      const uint32_t x = s_key[i] | 0x80808080u;
#pragma unroll
      for (int j = 0; j < 7; ++j) fc[j] += __popc((x - (base + 1u + j) * 0x01010101u) & 0x80808080u);
    }
  }
#pragma unroll
  for (int j = 0; j < 7; j += 2) {
    if (j < n_f) {
      const uint32_t t = (uint32_t)sah_wave_sum_i(fc[j] + ((j + 1 < 7 ? fc[j + 1] : 0) << 16));
      if (lane == 0) {
        atomicAdd(&S.fine[j], (int)(t & 0xFFFFu));
        if (j + 1 < 7) atomicAdd(&S.fine[j + 1], (int)(t >> 16));
      }
    }
  }
  __syncthreads();
  const int ftot = lane < n_f ? S.fine[lane] : 0;
  const int n_fine = __popcll(__ballot(lane < n_f && ftot >= k));
  const uint32_t T = base + (uint32_t)n_fine;
  const int above = n_fine < n_f ? __shfl(ftot, n_fine) : next_probe;      // count(key >= T + 1)
  // T == 0: fewer than k inactive columns exist; take them all, byte-0 "ties" emit nothing
  const int need = (T == 0) ? 0 : k - above;

  // ---- P2: per-lane masks and per-wave counts ---------------------------------------
  // A lane's columns of 8 chunks are one 32-bit mask (bit 8 t + u: column t of the lane's word in chunk
  // c + u), built with byte-parallel compares: `above T` and `equal T`. The first group's masks stay in
  // registers for P3 (a row of up to 32768 columns has no second group).
  auto group_masks = [&](int cg, uint32_t& m_gt, uint32_t& m_eq) {
    uint32_t ge = 0;
    m_gt = 0;
#pragma unroll
    for (int u = 0; u < HSW_GC; ++u) {
      if (cg + u < my_c1) {  // uniform across the wave
        const uint32_t x = s_key[(cg + u) * SAH_WAVE + lane] | 0x80808080u;
        // bit 7 of every byte of the difference is the flag; it moves to bit u of its byte
        m_gt |= ((x - (T + 1u) * 0x01010101u) >> (7 - u)) & (0x01010101u << u);
        ge |= ((x - T * 0x01010101u) >> (7 - u)) & (0x01010101u << u);
      }
    }
    m_eq = ge & ~m_gt;
  };
  const int n_grp = (my_c1 - my_c0 + HSW_GC - 1) / HSW_GC;  // uniform across the wave; <= 0 for a wave without chunks
  uint32_t mg0 = 0, me0 = 0;
  int lane_gt = 0, lane_eq = 0;
  for (int g = 0; g < n_grp; ++g) {
    uint32_t m_gt, m_eq;
    group_masks(my_c0 + g * HSW_GC, m_gt, m_eq);
    lane_gt += __popc(m_gt);
    lane_eq += __popc(m_eq);
    if (g == 0) {
      mg0 = m_gt;
      me0 = m_eq;
    }
  }
  const uint32_t n_both = (uint32_t)sah_wave_sum_i(lane_gt + (lane_eq << 16));
  const int n_gt = (int)(n_both & 0xFFFFu);
  const int n_eq = (int)(n_both >> 16);
  if (lane == 0) {
    s_gt[wave] = n_gt;
    s_eq[wave] = n_eq;
  }
  __syncthreads();
  // lane w < 16 holds wave w's counts: two wave scans give every wave's tie and output offsets
  int tie_base, out_base, total_out;
  {
    const int eq_w = lane < HSW_NW ? s_eq[lane] : 0;
    const int gt_w = lane < HSW_NW ? s_gt[lane] : 0;
    const int tie_incl = sah_wave_incl_scan(eq_w);
    int take = need - (tie_incl - eq_w);
    if (take < 0) take = 0;
    if (take > eq_w) take = eq_w;
    const int out_incl = sah_wave_incl_scan(gt_w + take);
    tie_base = __builtin_amdgcn_readlane(tie_incl - eq_w, wave);
    out_base = __builtin_amdgcn_readlane(out_incl - gt_w - take, wave);
    total_out = __builtin_amdgcn_readlane(out_incl, SAH_WAVE - 1);
  }

  // ---- P3: write ----------------------------------------------------------------------
  // The list of a row is unordered. Per group of 8 chunks a lane's winners are the set bits of one mask: one
  // wave scan of the per-lane counts places them, and a lane walks its own bits (a few per lane, so the walk
  // is as long as the busiest lane's count, not the number of chunks). A wave whose ties are all taken or all
  // dropped needs nothing else; the one wave in which the tie budget runs out first walks its chunks in
  // column order to keep the lowest ties.
  int* cols = R.cols + (int64_t)r * R.cap;
  float* wts = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  const bool ties_all = (tie_base + n_eq <= need);   // every tie of this wave is taken
  const bool ties_none = (tie_base >= need);         // none is
  int out_pos = cnt0 + out_base;
  int tie_run = tie_base;
  for (int g = 0; g < n_grp; ++g) {
    const int cg = my_c0 + g * HSW_GC;
    uint32_t m_gt = mg0, m_eq = me0;
    if (g > 0) group_masks(cg, m_gt, m_eq);
    uint32_t sel = m_gt;
    if (ties_all) {
      sel |= m_eq;
    } else if (!ties_none) {
      uint32_t kept = 0;
#pragma unroll
      for (int u = 0; u < HSW_GC; ++u) {
        if (cg + u < my_c1 && tie_run < need) {            // uniform across the wave
          const uint32_t e = m_eq & (0x01010101u << u);    // this lane's ties in chunk cg + u
          const int ne = __popc(e);
          const int incl = sah_wave_incl_scan(ne);
          int allowed = need - (tie_run + incl - ne);      // ties in lower chunks and lower lanes come first
          if (allowed >= ne) {
            kept |= e;
          } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) {                  // keep only the lowest `allowed` ties
              const uint32_t bit = e & (1u << (8 * t + u));
              if (bit && allowed > 0) {
                kept |= bit;
                --allowed;
              }
            }
          }
          tie_run += __builtin_amdgcn_readlane(incl, SAH_WAVE - 1);
        }
      }
      sel |= kept;
    }
    const int ns = __popc(sel);
    const int incl = sah_wave_incl_scan(ns);
    int pos = out_pos + incl - ns;
    out_pos += __builtin_amdgcn_readlane(incl, SAH_WAVE - 1);
    if (update_bitmap) {
#pragma unroll
      for (int u = 0; u < HSW_GC; ++u) {
        const uint32_t x = (sel >> u) & 0x01010101u;
        const uint32_t nib = (x | (x >> 7) | (x >> 14) | (x >> 21)) & 0xFu;
        const int j0 = ((cg + u) * SAH_WAVE + lane) * 4;
        if (nib) atomicOr(&s_bm[j0 >> 5], nib << (j0 & 31));
      }
    }
    const int col0 = (cg * SAH_WAVE + lane) * 4;
    while (sel) {
      const int b = __ffs(sel) - 1;
      sel &= sel - 1;
      const int col = col0 + (b & 7) * (4 * SAH_WAVE) + (b >> 3);
      if (pos < R.cap) {
        cols[pos] = col;
        if (wts) wts[pos] = 1.0f;
        if (s_cols) s_cols[pos] = col;
      }
      ++pos;
    }
  }
  int cnt_new = cnt0 + total_out;
  if (tid == 0) R.cnt[r] = cnt_new;
  if (cnt_new > R.cap) cnt_new = R.cap;
  if (!update_bitmap) return cnt_new;
  __syncthreads();
  for (int i = tid; i < R.n_words; i += HSW_NT) bm[i] = s_bm[i];
  return cnt_new;
}

