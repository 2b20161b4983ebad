// Row-wise top-k over 16-bit sortable keys (bf16 / fp16 scores), eight candidates per lane.
//
// One workgroup of 1024 threads per mask row. A lane owns eight consecutive candidates of a
// 512-candidate chunk: one 16-byte load brings their keys, one byte of the bitmap row tells
// which of them are already active. The k-th largest key is found byte by byte. Rows of up to 64
// keys per thread: the high byte from the row's largest key and packed-compare counts of the few
// bins below it (float scores: the k-th largest key lies within a bin or two of the largest), the
// low byte from a small histogram that only the keys of that bin touch. Longer rows, or a threshold
// further down: two 256-bin histogram levels (high byte with one counter per lane and bin, then the
// low byte of the keys inside the chosen bin). Either way the pass count is fixed: threshold, count,
// write; rows of up to 131072 candidates stay in registers from the first pass on.
// Winners above the threshold are written by every wave independently; only the wave that
// holds the last accepted tie walks its candidates in column order, which keeps the
// canonical rule "equal keys: lowest column first" at the cost of one ordered wave.
// The output list is unordered inside a row (its order is still a pure function of the
// inputs), as the attention kernel does not need sorted columns.
#pragma once
#include "sah_common.h"

#define SF_NT 1024
#define SF_NW (SF_NT / SAH_WAVE)
#define SF_CHUNK 512  // candidates a wave covers with one load per lane
#define SF_BATCH 4    // chunks a wave has in flight
#define SF_COPIES 64  // counters per bin: one per lane
static_assert(SF_COPIES == 64, "sf_pick reads one row of 16 lanes x 4 counters per bin");
#define SF_COPIES2 8  // counters per bin of the low-byte histogram of the short path
#define SF_TOP_BINS 4 // high-byte bins below the row's largest key that the short path looks at
static_assert(SF_TOP_BINS % 2 == 0, "the short path counts its bins in pairs");

struct sf_lds {
  int part[SF_NW];
  int eq[SF_NW];
  int gt[SF_NW];  // FUSED: keys above the threshold per wave
  int out[SF_NW];
  int top[SF_TOP_BINS];  // short path: candidates at or above each of the top high-byte bins
  int sel_bin, sel_need;
};

struct sf_chunk {
  uint32_t k[4];   // eight effective keys: candidate p in the low half of k[p], candidate p + 4 in the high half
  uint32_t excl;   // bit t: candidate t is already active (ranks with the excluded key, emits nothing)
  uint32_t valid;  // bit t: candidate t exists
};

// flag bits p and p + 4 -> the two 16-bit masks of word p
__device__ __forceinline__ uint32_t sf_mask2(uint32_t flags, int p) {
  return ((0u - ((flags >> p) & 1u)) & 0xffffu) | ((0u - ((flags >> (p + 4)) & 1u)) & 0xffff0000u);
}
// split mask (bit p: low half of word p, bit 16 + p: high half) -> one bit per candidate
__device__ __forceinline__ uint32_t sf_join(uint32_t split) { return (split | (split >> 12)) & 0xffu; }

// active / existing flags of the eight candidates starting at `cand`
__device__ __forceinline__ void sf_flags(const uint32_t* s_bm, int n_words, int cand, int n_cand, int col_offset,
                                         uint32_t& excl, uint32_t& valid) {
  int nv = n_cand - cand;
  nv = nv < 0 ? 0 : (nv > 8 ? 8 : nv);
  valid = (1u << nv) - 1u;
  const int col = cand + col_offset;
  int wi = col >> 5;
  wi = wi < n_words ? wi : n_words - 1;  // s_bm has one zero word of padding behind the row
  const uint64_t two = ((uint64_t)s_bm[wi + 1] << 32) | s_bm[wi];
  excl = (uint32_t)(two >> (col & 31)) & valid;
}

// keys straight from memory -> effective keys (active candidates take `ek2`, missing ones 0),
// re-paired so that one packed compare yields mask bits in candidate order
__device__ __forceinline__ void sf_effective(sf_chunk& c, uint4 raw, uint32_t ek2) {
  c.k[0] = (raw.x & 0xffffu) | (raw.z << 16);
  c.k[1] = (raw.x >> 16) | (raw.z & 0xffff0000u);
  c.k[2] = (raw.y & 0xffffu) | (raw.w << 16);
  c.k[3] = (raw.y >> 16) | (raw.w & 0xffff0000u);
  if (c.excl) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t me = sf_mask2(c.excl, p);
      c.k[p] = (c.k[p] & ~me) | (ek2 & me);
    }
  }
  if (c.valid != 0xffu) {
#pragma unroll
    for (int p = 0; p < 4; ++p) c.k[p] &= sf_mask2(c.valid, p);
  }
}

// k-th largest bin of a 256-bin histogram of [256][SF_COPIES] counters; all SF_NT threads call.
// Wave w owns the 16 bins 255 - 16w .. 240 - 16w. One 16-byte read per lane covers four
// bins (a row of 16 lanes per bin, 1 KB contiguous per instruction, no bank conflict); the
// row sums become wave-uniform scalars, so the scan over the wave's bins is scalar work.
__device__ __forceinline__ void sf_pick(const uint32_t* hist, int k, sf_lds& S, int& bin, int& need) {
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = tid / SAH_WAVE;
  int cnt[16];  // cnt[4 * i + row]: bin 255 - (16 * wave + 4 * i + row)
  int wave_total = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int b = 255 - (16 * wave + 4 * i + (lane >> 4));
    const uint4 q = *(const uint4*)(hist + b * SF_COPIES + (lane & 15) * 4);
    int v = (int)(q.x + q.y + q.z + q.w);
    v += sah_dpp_i<0xB1, 0xF, true>(v);   // quad_perm [1,0,3,2]
    v += sah_dpp_i<0x4E, 0xF, true>(v);   // quad_perm [2,3,0,1]
    v += sah_dpp_i<0x141, 0xF, true>(v);  // row_half_mirror
    v += sah_dpp_i<0x140, 0xF, true>(v);  // row_mirror
#pragma unroll
    for (int row = 0; row < 4; ++row) {
      cnt[4 * i + row] = __builtin_amdgcn_readlane(v, 16 * row);
      wave_total += cnt[4 * i + row];
    }
  }
  if (lane == 0) S.part[wave] = wave_total;
  __syncthreads();
  int above = 0;
#pragma unroll
  for (int w = 0; w < SF_NW; ++w) above += w < wave ? S.part[w] : 0;
  if (above < k && k <= above + wave_total) {  // wave-uniform: the bin lies in this wave's range
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (above < k && k <= above + cnt[j] && lane == 0) {
        S.sel_bin = 255 - (16 * wave + j);
        S.sel_need = k - above;
      }
      above += cnt[j];
    }
  }
  __syncthreads();
  bin = S.sel_bin;
  need = S.sel_need;
}

// The same for the short path's histogram of [SF_COPIES2][256] counters (copy-major: the counters of a bin are 1 KB
// apart), by ONE wave: lane l sums the copies of the four bins 252 - 4 l .. 255 - 4 l (one 16-byte read per copy,
// consecutive lanes at consecutive addresses), a wave scan gives the candidates in all bins from its own up, and the
// first lane that reaches k holds the bin. One barrier; the other waves only wait for it.
__device__ __forceinline__ void sf_pick8(const uint32_t* hist, int k, sf_lds& S, int& bin, int& need) {
  const int tid = threadIdx.x;
  if (tid < SAH_WAVE) {
    const int lo = 4 * (SAH_WAVE - 1 - tid);  // this lane's bins: lo .. lo + 3
    uint4 c = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int cp = 0; cp < SF_COPIES2; ++cp) {
      const uint4 q = *(const uint4*)(hist + cp * 256 + lo);
      c.x += q.x; c.y += q.y; c.z += q.z; c.w += q.w;
    }
    const int mine = (int)(c.x + c.y + c.z + c.w);
    const int incl = sah_wave_incl_scan(mine);  // candidates in the bins lo .. 255
    const uint64_t reach = __ballot(incl >= k);
    if (reach) {  // always: the caller's k is at most the histogram's total
      const int l = __builtin_ctzll(reach);
      if (tid == l) {
        int above = incl - mine;
        const int cnt[4] = {(int)c.w, (int)c.z, (int)c.y, (int)c.x};  // bins lo + 3, lo + 2, lo + 1, lo
        int bsel = lo, nsel = k - above;
        bool found = false;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (!found && k <= above + cnt[j]) {
            found = true;
            bsel = lo + 3 - j;
            nsel = k - above;
          }
          above += cnt[j];
        }
        S.sel_bin = bsel;
        S.sel_need = nsel;
      }
    }
  }
  __syncthreads();
  bin = S.sel_bin;
  need = S.sel_need;
}

// the `allowed` lowest set bits of an 8-bit mask
__device__ __forceinline__ uint32_t sf_lowest(uint32_t m, int allowed) {
  uint32_t take = 0;
  while (allowed > 0 && m) {
    const uint32_t b = m & (0u - m);
    take |= b;
    m ^= b;
    --allowed;
  }
  return take;
}

// CPW > 0: a wave keeps the effective keys of its (at most CPW) chunks in registers through
// all passes; CPW == 0: rows too long for that re-read their keys from memory in every pass.
// to_memory = false: the row's list, count and bitmap in memory are left alone (another workgroup writes them).
// Returns the row's entry count after the call; *first_new = the count before it.
//
// FUSED: the caller attends to the chosen columns in the same kernel, as one of `parts` workgroups that each run this
// selection for the row. The winners are written to the list s_cols (LDS; it may lie over the histograms, which are
// dead by then) at the positions they take in the row's list - complete after the caller's next barrier, entries
// [*first_new, return value); the entries before are the caller's to fill in or to derive. The row in memory: every
// part writes the columns of its own candidate chunks (chunk c belongs to part c % parts), part 0 (to_memory) also
// the count; the bitmap row is left complete in LDS (at the start of dyn) for part 0 to copy out after that barrier.
template <int CPW, bool FUSED = false>
__device__ __forceinline__ int sf_select_impl(sf_lds& S, unsigned char* dyn, const sah_rows& R, int r,
                                              const uint16_t* keys, int n_cand, int col_offset, int k,
                                              uint32_t excluded_key, int fresh, int sink, int window,
                                              bool to_memory, bool write_bitmap, int* first_new, int* s_cols, int part,
                                              int parts) {
  constexpr bool REG = CPW > 0;
  constexpr int NREG = REG ? CPW : 1;
  static_assert(!FUSED || (REG && CPW <= 8), "the fused form keeps a row's keys and its emission masks in registers");
  // The short way to the threshold (below) costs four packed compares per key word and pays up to 64 keys per
  // thread; longer rows amortise the histograms' fixed cost better (512 x 131072: 134 us against 107)
  constexpr bool SHORT = REG && CPW <= 8;
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  // rows of more than 64 keys per thread: a scalar wave index keeps the chunk bases of all passes out of the vector
  // registers (they were spilled); shorter rows are 0.2 us faster with the plain one
  const int wave = (CPW == 0 || CPW > 8) ? sah_wave_id() : tid / SAH_WAVE;
  const int n_chunks = (n_cand + SF_CHUNK - 1) / SF_CHUNK;
  const int cpw = (n_chunks + SF_NW - 1) / SF_NW;  // <= CPW when REG (the host picks CPW)
  const int c0 = wave * cpw;
  const int c1 = c0 + cpw < n_chunks ? c0 + cpw : n_chunks;

  // Histograms: SF_COPIES counters per bin, indexed by lane, so that the lanes of one atomic
  // instruction never meet on an address however few bins the keys fall into (the high byte
  // of a float key is sign + exponent: a handful of bins hold everything).
  uint32_t* s_bm = (uint32_t*)dyn;                     // n_words + 2
  uint32_t* s_h1 = s_bm + ((R.n_words + 2 + 3) & ~3);  // high byte: [256][SF_COPIES]
  uint32_t* s_h2 = s_h1 + 256 * SF_COPIES;             // low byte inside the chosen bin
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;
  const uint32_t ek = excluded_key & 0xffffu;
  const uint32_t ek2 = ek * 0x00010001u;

  auto raw_load = [&](int c) -> uint4 {
    int cand = c * SF_CHUNK + lane * 8;
    if (cand >= n_cand) cand = 0;  // a group with no candidate: any valid address will do
    return *(const uint4*)(keys + cand);
  };
  auto effective = [&](int c, uint4 raw) -> uint4 {
    sf_chunk ch;
    sf_flags(s_bm, R.n_words, c * SF_CHUNK + lane * 8, n_cand, col_offset, ch.excl, ch.valid);
    sf_effective(ch, raw, ek2);
    return make_uint4(ch.k[0], ch.k[1], ch.k[2], ch.k[3]);
  };

  // Counters that must be zero at the first barrier. Rows held in registers try the short path first (see
  // below), which needs the top-bin counts and a low-byte histogram of SF_COPIES2 counters per bin; the two
  // histograms of SF_COPIES counters per bin (128 KB, slow to clear and to scan) are cleared by the long path
  // itself when it is taken.
  auto clear_counters = [&]() {
    if (SHORT) {
      if (tid < SF_TOP_BINS) S.top[tid] = 0;
      for (int i = tid; i < 256 * SF_COPIES2 / 4; i += SF_NT) ((uint4*)s_h2)[i] = make_uint4(0u, 0u, 0u, 0u);
    } else {
      for (int i = tid; i < 2 * 256 * SF_COPIES / 4; i += SF_NT) ((uint4*)s_h1)[i] = make_uint4(0u, 0u, 0u, 0u);
    }
  };
  uint4 kreg[NREG];
  if (REG) {
    // the key loads go out first and land while the bitmap row and the counters are set up
#pragma unroll
    for (int u = 0; u < NREG; ++u) kreg[u] = raw_load(c0 + u);
  }
  int cnt0;
  if (fresh) {
    // rows still empty: the sink and local columns of one query per row in closed form, as
    // k_sink_local would have left them (basic_fixed.py:354-363, :48-67), without a launch of their own
    const int n = R.n_keys;
    const int s_hi = sink < n ? sink : n;
    int lo = 0, hi = 0;
    if (window > 0) {
      lo = n - window;
      hi = n;
      if (lo < 0) lo = 0;
    }
    const int lo2 = lo > s_hi ? lo : s_hi;
    const int fixed = s_hi + (hi > lo2 ? hi - lo2 : 0);
    int* cols0 = R.cols + (int64_t)r * R.cap;
    if (to_memory) {
      for (int i = tid; i < fixed && i < R.cap; i += SF_NT) {
        cols0[i] = i < s_hi ? i : lo2 + (i - s_hi);
        if (R.w) R.w[(int64_t)r * R.cap + i] = 1.0f;
      }
    }
    cnt0 = fixed < R.cap ? fixed : R.cap;
    clear_counters();
    for (int i = tid; i < R.n_words + 2; i += SF_NT)
      s_bm[i] = i < R.n_words ? (sah_range_bits(i, 0, s_hi) | sah_range_bits(i, lo, hi)) : 0u;
  } else {
    cnt0 = R.cnt[r];  // read before the first barrier: rewritten at the end
    if (cnt0 > R.cap) cnt0 = R.cap;
    // clear the counters first: these stores do not wait for the loads above, the bitmap copy does
    clear_counters();
    for (int i = tid; i < R.n_words + 2; i += SF_NT) s_bm[i] = i < R.n_words ? bm[i] : 0u;
  }
  __syncthreads();
  if (REG) {
#pragma unroll
    for (int u = 0; u < NREG; ++u) kreg[u] = effective(c0 + u, kreg[u]);
  }

  // run f(c, keys) over this wave's chunks in ascending order
  auto for_chunks = [&](auto&& f) {
    if (REG) {
#pragma unroll
      for (int u = 0; u < NREG; ++u)
        if (c0 + u < c1) {
          // opaque to the optimiser: values derived from the keys in one pass are not kept
          // alive for the next, they are cheaper to recompute than to hold in registers
          sah_keep(kreg[u].x), sah_keep(kreg[u].y), sah_keep(kreg[u].z), sah_keep(kreg[u].w);
          const uint32_t kk[4] = {kreg[u].x, kreg[u].y, kreg[u].z, kreg[u].w};
          f(c0 + u, kk);
        }
    } else {
      for (int cb = c0; cb < c1; cb += SF_BATCH) {
        uint4 raw[SF_BATCH];
#pragma unroll
        for (int u = 0; u < SF_BATCH; ++u) raw[u] = raw_load(cb + u < c1 ? cb + u : c1 - 1);
#pragma unroll
        for (int u = 0; u < SF_BATCH; ++u)
          if (cb + u < c1) {
            const uint4 e = effective(cb + u, raw[u]);
            const uint32_t kk[4] = {e.x, e.y, e.z, e.w};
            f(cb + u, kk);
          }
      }
    }
  };
  // the same with the chunk's register slot as third argument (REG only; 0 otherwise)
  auto for_chunks_slot = [&](auto&& f) {
    if (REG) {
#pragma unroll
      for (int u = 0; u < NREG; ++u)
        if (c0 + u < c1) {
          sah_keep(kreg[u].x), sah_keep(kreg[u].y), sah_keep(kreg[u].z), sah_keep(kreg[u].w);
          const uint32_t kk[4] = {kreg[u].x, kreg[u].y, kreg[u].z, kreg[u].w};
          f(c0 + u, kk, u);
        }
    } else {
      for_chunks([&](int c, const uint32_t (&kk)[4]) { f(c, kk, 0); });
    }
  };
  auto key_of = [](const uint32_t (&kk)[4], int t) -> uint32_t {
    return t < 4 ? (kk[t] & 0xffffu) : (kk[t - 4] >> 16);
  };
  // ---- threshold: the k-th largest key, as (high byte b1, low byte b2) ---------------------------
  uint32_t* my_h1 = s_h1 + (lane & (SF_COPIES - 1));
  uint32_t* my_h2 = s_h2 + (lane & (SF_COPIES - 1));
  int b1 = 0, need1 = 0, b2 = 0, need = 0;
  bool short_path = false;
  if (SHORT) {
    // Short path. Scores are floats: the high byte of a key is sign + seven exponent bits, and the k-th largest
    // key of a row lies within a few such bins of the largest. The row's largest key, then the counts of the
    // keys at or above the bottom of the SF_TOP_BINS bins below it (packed 16-bit compares, no histogram),
    // give b1 whenever it is one of those bins; otherwise the long path runs.
    uint32_t m2 = 0;
    for_chunks([&](int, const uint32_t (&kk)[4]) {
#pragma unroll
      for (int p = 0; p < 4; ++p) m2 = sah_pk_max_u16(m2, kk[p]);
    });
    uint32_t m = (m2 & 0xffffu) > (m2 >> 16) ? (m2 & 0xffffu) : (m2 >> 16);
#pragma unroll
    for (int o = 1; o < SAH_WAVE; o <<= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)m, o);
      m = other > m ? other : m;
    }
    if (lane == 0) S.part[wave] = (int)m;
    __syncthreads();
    uint32_t row_max = 0;
#pragma unroll
    for (int w = 0; w < SF_NW; ++w) row_max = (uint32_t)S.part[w] > row_max ? (uint32_t)S.part[w] : row_max;
    const int b_max = (int)(row_max >> 8);
    // bin b_max - j has its bottom at key (b_max - j) << 8; bin 0 is left to the long path (a compare against
    // "below zero" does not exist). Two bins at a time: the threshold is nearly always in the largest key's own
    // bin or the next, and the second pair is counted only when it is not.
    auto bottom = [&](int jj) -> uint32_t {
      const int bj = b_max - jj;
      return bj >= 1 ? (uint32_t)((bj << 8) - 1) * 0x00010001u : 0xffffffffu;  // nothing is above 0xffff
    };
    int above = 0;
    for (int j0 = 0; j0 < SF_TOP_BINS && !short_path; j0 += 2) {  // uniform across the workgroup
      const uint32_t lim0 = bottom(j0), lim1 = bottom(j0 + 1);
      uint32_t pc0 = 0, pc1 = 0;
      for_chunks([&](int, const uint32_t (&kk)[4]) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          pc0 += sah_pk_gt01_u16(kk[p], lim0);
          pc1 += sah_pk_gt01_u16(kk[p], lim1);
        }
      });
      // both counts in one wave sum: a wave holds at most 64 * 8 * CPW <= 4096 candidates
      const int both = sah_wave_sum_i((int)((pc0 & 0xffffu) + (pc0 >> 16) + (((pc1 & 0xffffu) + (pc1 >> 16)) << 16)));
      if (lane == 0) {
        atomicAdd(&S.top[j0], both & 0xffff);
        atomicAdd(&S.top[j0 + 1], (int)((uint32_t)both >> 16));
      }
      __syncthreads();
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int c = S.top[j0 + jj];  // candidates in the bins b_max .. b_max - (j0 + jj)
        if (!short_path && b_max - (j0 + jj) >= 1 && c >= k) {
          short_path = true;
          b1 = b_max - (j0 + jj);
          need1 = k - above;
        }
        above = c;
      }
    }
  }
  if (short_path) {
    // low byte inside bin b1: only the keys of that bin touch the histogram
    uint32_t* my_h = s_h2 + (lane & (SF_COPIES2 - 1)) * 256;
    for_chunks([&](int, const uint32_t (&kk)[4]) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const uint32_t key = key_of(kk, t);
        if ((int)(key >> 8) == b1) atomicAdd(&my_h[key & 0xffu], 1u);
      }
    });
    __syncthreads();
    sf_pick8(s_h2, need1, S, b2, need);
  } else {
    if (SHORT) {  // the short path left these untouched
      for (int i = tid; i < 2 * 256 * SF_COPIES / 4; i += SF_NT) ((uint4*)s_h1)[i] = make_uint4(0u, 0u, 0u, 0u);
      __syncthreads();
    }
    // ---- pass 1: histogram of the high byte
    for_chunks([&](int, const uint32_t (&kk)[4]) {
#pragma unroll
      for (int t = 0; t < 8; ++t) atomicAdd(&my_h1[(key_of(kk, t) >> 8) * SF_COPIES], 1u);
    });
    __syncthreads();
    sf_pick(s_h1, k, S, b1, need1);
    // ---- pass 2: histogram of the low byte inside bin b1
    for_chunks([&](int, const uint32_t (&kk)[4]) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const uint32_t key = key_of(kk, t);
        atomicAdd(&my_h2[(key & 0xffu) * SF_COPIES], (int)(key >> 8) == b1 ? 1u : 0u);
      }
    });
    __syncthreads();
    sf_pick(s_h2, need1, S, b2, need);
  }
  const uint32_t T = ((uint32_t)b1 << 8) | (uint32_t)b2;
  // Active candidates carry the excluded key. While that ranks below the threshold they are
  // neither winners nor ties and their flags are not needed again; otherwise (a row with
  // fewer than k better inactive candidates) they take rank but are never emitted.
  const bool slow = ek >= T;

  // 8-bit masks of one chunk: emittable keys above the threshold, ties, active candidates
  const uint32_t T2 = T * 0x00010001u;
  auto masks = [&](int c, const uint32_t (&kk)[4], uint32_t& gt, uint32_t& eq, uint32_t& ex) {
    uint32_t g = 0, n = 0;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      g |= sah_pk_gt01_u16(kk[p], T2) << p;
      n |= sah_pk_ne01_u16(kk[p], T2) << p;
    }
    gt = sf_join(g);
    eq = sf_join(~n & 0x000f000fu);
    ex = 0;
    if (slow) {
      uint32_t valid;
      sf_flags(s_bm, R.n_words, c * SF_CHUNK + lane * 8, n_cand, col_offset, ex, valid);
      eq &= valid;  // a missing candidate has key 0, which ties when T is 0
      gt &= ~ex;
    }
  };

  // ---- pass 3: winners and ties per lane and wave --------------------------------------------
  // Rows held in registers keep the two masks of every chunk (16 bits, two chunks to a register) for the passes
  // below, which then do not compare a key again; not when active candidates may rank (their flags come from LDS).
  // (up to 64 keys per thread: beyond that the registers are full)
  constexpr bool KEEP = REG && CPW <= 8;
  constexpr int NPM = KEEP ? (NREG + 1) / 2 : 1;
  const bool stored = KEEP && !slow;  // uniform across the workgroup
  uint32_t pm[NPM];
#pragma unroll
  for (int i = 0; i < NPM; ++i) pm[i] = 0;
  int n_gt = 0, n_eq = 0;
  for_chunks_slot([&](int c, const uint32_t (&kk)[4], int u) {
    uint32_t gt, eq, ex;
    masks(c, kk, gt, eq, ex);
    n_gt += __popc(gt);
    n_eq += __popc(eq);
    if (KEEP) pm[u >> 1] |= (gt | (eq << 8)) << (16 * (u & 1));
  });
  const int wave_eq = sah_wave_sum_i(n_eq);
  if (lane == 0) S.eq[wave] = wave_eq;
  if constexpr (FUSED) {
    const int wave_gt = sah_wave_sum_i(n_gt);
    if (lane == 0) S.gt[wave] = wave_gt;
  }
  __syncthreads();
  int tie_base = 0;
#pragma unroll
  for (int w = 0; w < SF_NW; ++w) tie_base += w < wave ? S.eq[w] : 0;
  // 0: no tie of this wave is taken, 1: all are, 2: the boundary lies inside the wave
  const int mode = tie_base >= need ? 0 : (tie_base + wave_eq <= need ? 1 : 2);

  // emission mask of a chunk; `tie_run` counts the wave's ties seen so far (mode 2 only)
  int tie_run = tie_base;
  auto emit_mask = [&](int c, const uint32_t (&kk)[4], int u) -> uint32_t {
    uint32_t gt, eq, ex;
    if (stored) {
      const uint32_t both = pm[KEEP ? u >> 1 : 0] >> (16 * (u & 1));
      gt = both & 0xffu;
      eq = (both >> 8) & 0xffu;
      ex = 0;
    } else {
      masks(c, kk, gt, eq, ex);
    }
    uint32_t take = 0;
    if (mode == 1) take = eq;
    if (mode == 2) {
      const int ne = __popc(eq);
      const int incl = sah_wave_incl_scan(ne);
      take = sf_lowest(eq, need - tie_run - (incl - ne));
      tie_run += __builtin_amdgcn_readlane(incl, SAH_WAVE - 1);
    }
    return gt | (take & ~ex);
  };

  if constexpr (FUSED) {
    // ---- the winners into the LDS list (all of them, at the positions they take in the row's list) and, for the
    // chunks of this part, into the row in memory. Every wave's number of winners follows from the counts exchanged
    // at the tie barrier (its keys above the threshold plus the ties it may take), so the positions need no second
    // barrier - unless active candidates may rank (`slow`), whose ties cannot be counted ahead.
    uint32_t em_all[(NREG + 3) / 4];  // emission masks of the wave's chunks, 8 bits each
#pragma unroll
    for (int i = 0; i < (NREG + 3) / 4; ++i) em_all[i] = 0;
    int mine_all = 0;
    for_chunks_slot([&](int c, const uint32_t (&kk)[4], int u) {
      const uint32_t em = emit_mask(c, kk, u);
      em_all[u >> 2] |= em << (8 * (u & 3));
      mine_all += __popc(em);
    });
    const int incl_a = sah_wave_incl_scan(mine_all);
    int out_base = 0, total = 0;
    if (!slow) {
      int ties_before = 0;
#pragma unroll
      for (int w = 0; w < SF_NW; ++w) {
        int take = need - ties_before;
        take = take < 0 ? 0 : (take > S.eq[w] ? S.eq[w] : take);
        const int v = S.gt[w] + take;
        out_base += w < wave ? v : 0;
        total += v;
        ties_before += S.eq[w];
      }
    } else {
      if (lane == SAH_WAVE - 1) S.out[wave] = incl_a;
      __syncthreads();
      for (int w = 0; w < SF_NW; ++w) {
        const int v = S.out[w];
        out_base += w < wave ? v : 0;
        total += v;
      }
    }
    int* cols = R.cols + (int64_t)r * R.cap;
    int pos = cnt0 + out_base + incl_a - mine_all;
#pragma unroll
    for (int u = 0; u < NREG; ++u) {
      const int c = c0 + u;
      if (c < c1) {
        uint32_t em = (em_all[u >> 2] >> (8 * (u & 3))) & 0xffu;
        const int col0 = c * SF_CHUNK + lane * 8 + col_offset;
        if (em && to_memory && write_bitmap) {
          atomicOr(&s_bm[col0 >> 5], em << (col0 & 31));
          if ((col0 & 31) > 24) atomicOr(&s_bm[(col0 >> 5) + 1], em >> (32 - (col0 & 31)));
        }
        const bool my_chunk = c % parts == part;
        while (em) {
          const int t = __builtin_ctz(em);
          em &= em - 1;
          if (pos < R.cap) {
            s_cols[pos] = col0 + t;
            if (my_chunk) cols[pos] = col0 + t;
          }
          ++pos;
        }
      }
    }
    if (to_memory && tid == 0) R.cnt[r] = cnt0 + total;
    // (part 0 writes the bitmap row, complete in LDS after the caller's next barrier, back to memory)
    if (first_new) *first_new = cnt0;
    const int after = cnt0 + total;
    return after < R.cap ? after : R.cap;
  }
  // what each lane emits: known from the counts, except where ties are cut or may be active
  int mine = n_gt + (mode == 1 ? n_eq : 0);
  if (mode == 2 || slow) {
    mine = 0;
    for_chunks_slot([&](int c, const uint32_t (&kk)[4], int u) { mine += __popc(emit_mask(c, kk, u)); });
  }
  const int incl = sah_wave_incl_scan(mine);
  if (lane == SAH_WAVE - 1) S.out[wave] = incl;
  __syncthreads();
  int out_base = 0, total = 0;
  for (int w = 0; w < SF_NW; ++w) {
    const int v = S.out[w];
    out_base += w < wave ? v : 0;
    total += v;
  }

  // ---- pass 4: write ---------------------------------------------------------------------------
  int* cols = R.cols + (int64_t)r * R.cap;
  float* wgt = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  int pos = cnt0 + out_base + incl - mine;
  tie_run = tie_base;
  for_chunks_slot([&](int c, const uint32_t (&kk)[4], int u) {
    uint32_t em = emit_mask(c, kk, u);
    if (em) {
      const int col0 = c * SF_CHUNK + lane * 8 + col_offset;
      if (to_memory && write_bitmap) {
        atomicOr(&s_bm[col0 >> 5], em << (col0 & 31));
        if ((col0 & 31) > 24) atomicOr(&s_bm[(col0 >> 5) + 1], em >> (32 - (col0 & 31)));
      }
      while (em) {
        const int t = __builtin_ctz(em);
        em &= em - 1;
        if (pos < R.cap) {
          if (to_memory) {
            cols[pos] = col0 + t;
            if (wgt) wgt[pos] = 1.0f;
          }
        }
        ++pos;
      }
    }
  });
  __syncthreads();
  if (to_memory) {
    if (write_bitmap && (total > 0 || fresh))
      for (int i = tid; i < R.n_words; i += SF_NT) bm[i] = s_bm[i];
    if (tid == 0) R.cnt[r] = cnt0 + total;
  }
  if (first_new) *first_new = cnt0;
  const int after = cnt0 + total;
  return after < R.cap ? after : R.cap;
}

// The stand-alone form: the row's list, count and bitmap in memory are extended.
template <int CPW>
__device__ __forceinline__ int sf_select_row(sf_lds& S, unsigned char* dyn, const sah_rows& R, int r,
                                             const uint16_t* keys, int n_cand, int col_offset, int k,
                                             uint32_t excluded_key, int fresh, int sink, int window) {
  return sf_select_impl<CPW>(S, dyn, R, r, keys, n_cand, col_offset, k, excluded_key, fresh, sink, window, true, true, nullptr,
                             nullptr, 0, 1);
}

// dynamic LDS bytes of one launch
static inline size_t sf_lds_bytes(int n_words) {
  return (size_t)((n_words + 2 + 3) & ~3) * 4 + (size_t)2 * 256 * SF_COPIES * 4;
}
// chunks per wave of a row of n_cand candidates
static inline int sf_chunks_per_wave(int n_cand) {
  const int n_chunks = (n_cand + SF_CHUNK - 1) / SF_CHUNK;
  return (n_chunks + SF_NW - 1) / SF_NW;
}

// byte offset, inside the dynamic LDS of sf_select_row, of the region its histograms occupy (dead once the threshold
// is known): where a caller may keep the row's column list
static inline size_t sf_hist_offset(int n_words) { return (size_t)((n_words + 2 + 3) & ~3) * 4; }
static inline size_t sf_hist_bytes() { return (size_t)2 * 256 * SF_COPIES * 4; }

// argument checks of sah_select_topk (defined with it), for entry points that run the same selection
int sel_validate(const sah_select_topk_args* a, const char* who);
// may this call take the eight-keys-per-lane kernel? (16-bit keys, aligned rows, the LDS fits)
static inline bool sel16_ok(const sah_select_topk_args* a) {
  return a->key_bits == 16 && a->key_pitch % 8 == 0 && ((uintptr_t)a->keys % 16) == 0 && sf_lds_bytes(a->rows.n_words) <= 150 * 1024;
}
