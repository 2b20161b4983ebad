// Row-wise top-k selection with the canonical tie rule "lowest column first".
//
// One workgroup (1024 threads = 16 waves) per mask row. Keys are unsigned and
// order-preserving (larger = better); already-active columns take a caller
// chosen key so they rank exactly where the reference's `scores[prev != 0] =
// min` puts them. The k-th key is found by MSB-first radix select with an LDS
// histogram per digit; the winners are then written in ascending column order
// by a wave-ordered compaction (ballot + mbcnt inside a wave, one LDS exchange
// across the 16 waves), which is what makes ties resolve to the lowest column.
// Each wave owns 64-column aligned chunks, so the bitmap words it updates are
// touched by no other wave and need no atomics.
#include "sah_common.h"
#include "sah_hsw.h"
#include "sah_sel16.h"

#define SEL_NT 1024
#define SEL_NW (SEL_NT / SAH_WAVE)
#define SEL_DIGIT_BITS 13
#define SEL_BINS (1 << SEL_DIGIT_BITS)

// ---- key sources -----------------------------------------------------------
// A source splits "fetch" (one global load, issued in batches) from "key" (ALU only).
struct key_src_mem16 {
  typedef uint32_t raw_t;
  const uint16_t* keys;  // row base, indexed by candidate
  __device__ __forceinline__ raw_t fetch(int cand) const { return keys[cand]; }
  __device__ __forceinline__ uint32_t key(raw_t r) const { return r; }
  __device__ __forceinline__ static void keep(raw_t& r) { sah_keep(r); }
};
struct key_src_mem32 {
  typedef uint32_t raw_t;
  const uint32_t* keys;
  __device__ __forceinline__ raw_t fetch(int cand) const { return keys[cand]; }
  __device__ __forceinline__ uint32_t key(raw_t r) const { return r; }
  __device__ __forceinline__ static void keep(raw_t& r) { sah_keep(r); }
};
struct key_src_hamming {
  typedef uint2 raw_t;
  const uint2* kcodes;  // code stream base: (positive plane, non-zero plane) per key
  uint2 qcode;
  __device__ __forceinline__ raw_t fetch(int cand) const { return kcodes[cand]; }
  // score + 33 in [1, 65], so every real column outranks the excluded key 0
  __device__ __forceinline__ uint32_t key(raw_t r) const { return (uint32_t)(sig_score(qcode, r) + 33); }
  __device__ __forceinline__ static void keep(raw_t& r) {
    sah_keep(r.x);
    sah_keep(r.y);
  }
};

struct sel_shared {
  int scan[SEL_NW + 1];
  int wave_gt[SEL_NW];
  int wave_eq[SEL_NW];
  int wave_out[SEL_NW];
  int wave_tie[SEL_NW];
  uint32_t digit;
  int need;
  int total_out;
};

#define SEL_LOAD_BATCH 16  // 64-column chunks requested together in the staging pass

// Dynamic LDS layout of one row: [histogram 4*nbins][bitmap row 4*n_words][staged keys].
// The bitmap row and (when they fit) the effective keys of all candidates are staged once,
// with SEL_LOAD_BATCH chunks of loads in flight per wave, so that the digit passes and the
// two compaction passes run out of LDS instead of re-reading global memory.
struct sel_layout {
  int hist_bins;      // bins of the widest digit
  int stage_keys;     // 1: effective keys are staged in LDS
};

// sum of one int per thread over the block; every thread gets the total
__device__ __forceinline__ int sel_block_sum(int v, int* scratch) {
  v = sah_wave_sum_i(v);
  __syncthreads();
  if ((threadIdx.x & (SAH_WAVE - 1)) == 0) scratch[threadIdx.x / SAH_WAVE] = v;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int i = 0; i < SEL_NW; ++i) t += scratch[i];
  return t;
}

// KEYBITS: number of significant key bits (7, 16 or 32); STG: LDS type of a staged key
template <typename SRC, int KEYBITS, typename STG>
__device__ __forceinline__ void select_row(sel_shared& S, unsigned char* dyn, sel_layout L, const sah_rows& R, int r,
                                           const SRC& src, int n_cand, int col_offset, int k, uint32_t excluded_key) {
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  uint32_t* hist = (uint32_t*)dyn;
  uint32_t* s_bm = hist + L.hist_bins;
  STG* staged = (STG*)(s_bm + R.n_words);
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;

  // 64-column aligned chunks of the candidate range, split contiguously over waves
  const int c_first = col_offset / SAH_WAVE;
  const int c_last = (col_offset + n_cand - 1) / SAH_WAVE;
  const int n_chunks = c_last - c_first + 1;
  const int cpw = (n_chunks + SEL_NW - 1) / SEL_NW;
  const int my_c0 = c_first + wave * cpw;
  int my_c1 = my_c0 + cpw;
  if (my_c1 > c_last + 1) my_c1 = c_last + 1;
  const int col_base = c_first * SAH_WAVE;  // staged[] is indexed by col - col_base

  // read before any barrier: thread 0 overwrites the count at the very end
  int cnt0 = R.cnt[r];
  if (cnt0 > R.cap) cnt0 = R.cap;
  for (int i = tid; i < R.n_words; i += SEL_NT) s_bm[i] = bm[i];
  __syncthreads();

  // effective key of a column: straight from global memory (clamped address)
  auto eff_key_global = [&](int col, bool& valid, bool& excl) -> uint32_t {
    const int cand = col - col_offset;
    valid = (cand >= 0 && cand < n_cand);
    const int cc = valid ? cand : 0;
    const int cl = valid ? col : col_offset;
    const uint32_t key = src.key(src.fetch(cc));
    excl = valid && ((s_bm[cl >> 5] >> (cl & 31)) & 1u);
    return valid ? (excl ? excluded_key : key) : 0u;
  };
  // one batch of SEL_LOAD_BATCH chunks: every global load is issued before the first use
  auto load_batch = [&](int c0, uint32_t (&key)[SEL_LOAD_BATCH], bool (&valid)[SEL_LOAD_BATCH]) {
    typename SRC::raw_t raw[SEL_LOAD_BATCH];
#pragma unroll
    for (int u = 0; u < SEL_LOAD_BATCH; ++u) {
      const int cand = (c0 + u) * SAH_WAVE + lane - col_offset;
      valid[u] = (c0 + u < my_c1) && cand >= 0 && cand < n_cand;
      raw[u] = src.fetch(valid[u] ? cand : 0);
    }
#pragma unroll
    for (int u = 0; u < SEL_LOAD_BATCH; ++u) SRC::keep(raw[u]);
#pragma unroll
    for (int u = 0; u < SEL_LOAD_BATCH; ++u) {
      const int col = (c0 + u) * SAH_WAVE + lane;
      const int cl = valid[u] ? col : col_offset;
      const bool excl = (s_bm[cl >> 5] >> (cl & 31)) & 1u;
      key[u] = valid[u] ? (excl ? excluded_key : src.key(raw[u])) : 0u;
    }
  };
  auto eff_key = [&](int col, bool& valid, bool& excl) -> uint32_t {
    if (!L.stage_keys) return eff_key_global(col, valid, excl);
    const int cand = col - col_offset;
    valid = (cand >= 0 && cand < n_cand);
    const int cl = valid ? col : col_offset;
    excl = valid && ((s_bm[cl >> 5] >> (cl & 31)) & 1u);
    return valid ? (uint32_t)staged[cl - col_base] : 0u;
  };

  if (k > n_cand) k = n_cand;
  int need = k;
  uint32_t prefix = 0;
  int bits_done = 0;

  if (KEYBITS == 7 && L.stage_keys) {
    // ---- byte keys staged in LDS: bisection on the threshold, no atomics ------
    // (a 65-value histogram would serialise on a handful of LDS addresses)
    const int n_bytes = n_chunks * SAH_WAVE;
    for (int c0 = my_c0; c0 < my_c1; c0 += SEL_LOAD_BATCH) {
      uint32_t key[SEL_LOAD_BATCH];
      bool valid[SEL_LOAD_BATCH];
      load_batch(c0, key, valid);
#pragma unroll
      for (int u = 0; u < SEL_LOAD_BATCH; ++u)
        if (c0 + u < my_c1) staged[(c0 + u) * SAH_WAVE + lane - col_base] = (STG)key[u];  // 0 outside the range
    }
    __syncthreads();
    const uint32_t* words = (const uint32_t*)staged;
    const int n_w = n_bytes / 4;
    auto count_ge = [&](uint32_t t) -> int {
      // bytes are < 128: (b | 0x80) - t keeps bit 7 exactly when b >= t, without borrows
      int c = 0;
      const uint32_t tt = t * 0x01010101u;
      for (int i = tid; i < n_w; i += SEL_NT) c += __popc(((words[i] | 0x80808080u) - tt) & 0x80808080u);
      return sel_block_sum(c, S.scan);
    };
    uint32_t T7 = 0;
    for (int bit = 6; bit >= 0; --bit) {
      const uint32_t cand = T7 | (1u << bit);
      if (count_ge(cand) >= k) T7 = cand;
    }
    const int above = (T7 >= 127u) ? 0 : count_ge(T7 + 1);
    prefix = T7;
    need = k - above;
    bits_done = KEYBITS;
  }
  // ---- radix select of the k-th largest key --------------------------------
  while (bits_done < KEYBITS) {
    int wd = KEYBITS - bits_done;
    if (wd > SEL_DIGIT_BITS) wd = SEL_DIGIT_BITS;
    const int sh = KEYBITS - bits_done - wd;
    const int nb = 1 << wd;
    for (int i = tid; i < nb; i += SEL_NT) hist[i] = 0;
    __syncthreads();
    if (bits_done == 0) {
      // first pass: batched global loads, stage the keys, histogram of the top digit
      for (int c0 = my_c0; c0 < my_c1; c0 += SEL_LOAD_BATCH) {
        uint32_t key[SEL_LOAD_BATCH];
        bool valid[SEL_LOAD_BATCH];
        load_batch(c0, key, valid);
#pragma unroll
        for (int u = 0; u < SEL_LOAD_BATCH; ++u) {
          if (valid[u]) {
            const int col = (c0 + u) * SAH_WAVE + lane;
            if (L.stage_keys) staged[col - col_base] = (STG)key[u];
            atomicAdd(&hist[(key[u] >> sh) & (uint32_t)(nb - 1)], 1u);
          }
        }
      }
    } else {
      for (int c = my_c0; c < my_c1; ++c) {
        const int col = c * SAH_WAVE + lane;
        bool valid, excl;
        const uint32_t key = eff_key(col, valid, excl);
        if (valid && ((key >> (sh + wd)) == prefix)) atomicAdd(&hist[(key >> sh) & (uint32_t)(nb - 1)], 1u);
      }
    }
    __syncthreads();
    // descending scan over digits: thread t owns the t-th highest group of bins
    const int per = (nb + SEL_NT - 1) / SEL_NT;  // bins per thread (1 or 8)
    const int hi_bin = nb - 1 - tid * per;       // my highest bin
    int mine = 0;
    for (int i = 0; i < per; ++i) {
      const int bin = hi_bin - i;
      if (bin >= 0) mine += (int)hist[bin];
    }
    int total;
    const int above = sah_block_excl_scan<SEL_NT>(mine, S.scan, &total);
    if (above < need && need <= above + mine) {
      int run = above;
      for (int i = 0; i < per; ++i) {
        const int bin = hi_bin - i;
        if (bin < 0) break;
        const int cbin = (int)hist[bin];
        if (need <= run + cbin) {
          S.digit = (uint32_t)bin;
          S.need = need - run;
          break;
        }
        run += cbin;
      }
    }
    __syncthreads();
    prefix = (prefix << wd) | S.digit;
    need = S.need;
    bits_done += wd;
    __syncthreads();
  }
  const uint32_t T = prefix;  // k-th largest key; `need` ties at T are taken, lowest column first

  // ---- per-wave counts: keys above T that will be emitted, ties, emitted ties ----
  // Ties are consumed in column order; an already-active tie uses up rank but emits nothing,
  // so a wave first learns how many ties precede it, then counts the ties it will emit.
  int n_gt = 0, n_eq = 0;
  for (int c = my_c0; c < my_c1; ++c) {
    const int col = c * SAH_WAVE + lane;
    bool valid, excl;
    const uint32_t key = eff_key(col, valid, excl);
    n_gt += __popcll(__ballot(valid && !excl && key > T));
    n_eq += __popcll(__ballot(valid && key == T));
  }
  if (lane == 0) {
    S.wave_gt[wave] = n_gt;
    S.wave_eq[wave] = n_eq;
  }
  __syncthreads();
  if (tid == 0) {
    int tie_run = 0;
    for (int wv = 0; wv < SEL_NW; ++wv) {
      S.wave_tie[wv] = tie_run;
      tie_run += S.wave_eq[wv];
    }
  }
  __syncthreads();
  int tie_rank = S.wave_tie[wave];
  int emit_ties = 0;
  if (tie_rank < need && n_eq > 0) {
    for (int c = my_c0; c < my_c1; ++c) {
      const int col = c * SAH_WAVE + lane;
      bool valid, excl;
      const uint32_t key = eff_key(col, valid, excl);
      const bool is_tie = valid && key == T;
      const uint64_t tm = __ballot(is_tie);
      const bool take = is_tie && !excl && (tie_rank + sah_lane_prefix(tm) < need);
      emit_ties += __popcll(__ballot(take));
      tie_rank += __popcll(tm);
    }
  }
  __syncthreads();  // wave_eq is re-used below
  if (lane == 0) S.wave_eq[wave] = emit_ties;
  __syncthreads();
  if (tid == 0) {
    int out_run = 0;
    for (int wv = 0; wv < SEL_NW; ++wv) {
      S.wave_out[wv] = out_run;
      out_run += S.wave_gt[wv] + S.wave_eq[wv];
    }
    S.total_out = out_run;
  }
  __syncthreads();

  // ---- ordered compaction ----------------------------------------------------
  int* cols = R.cols + (int64_t)r * R.cap;
  float* w = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  int out_pos = cnt0 + S.wave_out[wave];
  tie_rank = S.wave_tie[wave];
  for (int c = my_c0; c < my_c1; ++c) {
    const int col = c * SAH_WAVE + lane;
    bool valid, excl;
    const uint32_t key = eff_key(col, valid, excl);
    const bool is_tie = valid && key == T;
    const uint64_t tm = __ballot(is_tie);
    const bool sel = valid && !excl && (key > T || (is_tie && (tie_rank + sah_lane_prefix(tm) < need)));
    const uint64_t sm = __ballot(sel);
    if (sel) {
      const int pos = out_pos + sah_lane_prefix(sm);
      if (pos < R.cap) {
        cols[pos] = col;
        if (w) w[pos] = 1.0f;
      }
    }
    if (sm) {
      // this wave owns words 2c and 2c+1 of the row: plain read-modify-write
      const int w0 = c * 2;
      if (lane == 0 && (uint32_t)sm) bm[w0] = s_bm[w0] | (uint32_t)sm;
      if (lane == 32 && (uint32_t)(sm >> 32) && w0 + 1 < R.n_words) bm[w0 + 1] = s_bm[w0 + 1] | (uint32_t)(sm >> 32);
    }
    out_pos += __popcll(sm);
    tie_rank += __popcll(tm);
  }
  if (tid == 0) R.cnt[r] = cnt0 + S.total_out;
}

// dynamic LDS bytes and staging decision for one launch
static size_t sel_plan(int key_bits, int stage_bytes, int n_words, int n_cand, int col_offset, sel_layout* L) {
  const int wd = key_bits < SEL_DIGIT_BITS ? key_bits : SEL_DIGIT_BITS;
  L->hist_bins = 1 << wd;
  size_t fixed = (size_t)L->hist_bins * 4 + (size_t)n_words * 4;
  const int c_first = col_offset / SAH_WAVE;
  const int c_last = (col_offset + n_cand - 1) / SAH_WAVE;
  size_t stage = (size_t)(c_last - c_first + 1) * SAH_WAVE * stage_bytes;
  const size_t budget = 150 * 1024;  // of the 160 KB LDS of a CU, minus the static part
  L->stage_keys = (fixed + stage <= budget) ? 1 : 0;
  return fixed + (L->stage_keys ? stage : 0);
}

template <int KB>
__global__ __launch_bounds__(SEL_NT) void k_select_topk(sah_rows R, sel_layout L, const void* keys, int64_t pitch,
                                                        int n_cand, int col_offset, int k, uint32_t excluded_key) {
  __shared__ sel_shared S;
  HIP_DYNAMIC_SHARED(unsigned char, sel_dyn)
  const int r = blockIdx.x;
  if (KB == 16) {
    key_src_mem16 src{(const uint16_t*)keys + (int64_t)r * pitch};
    select_row<key_src_mem16, 16, uint16_t>(S, sel_dyn, L, R, r, src, n_cand, col_offset, k, excluded_key);
  } else {
    key_src_mem32 src{(const uint32_t*)keys + (int64_t)r * pitch};
    select_row<key_src_mem32, 32, uint32_t>(S, sel_dyn, L, R, r, src, n_cand, col_offset, k, excluded_key);
  }
}

__global__ __launch_bounds__(SEL_NT) void k_hamming_topk(sah_rows R, sel_layout L, const uint2* kcodes, int64_t pitch,
                                                         const uint2* qcodes, int lq, int k) {
  __shared__ sel_shared S;
  HIP_DYNAMIC_SHARED(unsigned char, sel_dyn)
  const int r = blockIdx.x;
  key_src_hamming src{kcodes + (int64_t)(r / lq) * pitch, qcodes[r]};
  select_row<key_src_hamming, 7, uint8_t>(S, sel_dyn, L, R, r, src, R.n_keys, 0, k, 0u);
}

__global__ __launch_bounds__(HSW_NT) void k_hamming_topk_swar(sah_rows R, const uint2* kcodes, int64_t pitch,
                                                              const uint2* qcodes, int lq, int k) {
  __shared__ hsw_lds S;
  HIP_DYNAMIC_SHARED(unsigned char, hsw_dyn)
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int n_ch = (R.n_keys + 255) / 256;
  uint32_t* s_bm = (uint32_t*)hsw_dyn;   // n_words (+ padding to a chunk)
  uint32_t* s_key = s_bm + n_ch * 8;     // n_ch * 64 words
  const uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;
  int cnt0 = R.cnt[r];  // read before the first barrier: the row's last thread rewrites it at the end
  if (cnt0 > R.cap) cnt0 = R.cap;
  for (int i = tid; i < n_ch * 8; i += HSW_NT) s_bm[i] = i < R.n_words ? bm[i] : 0u;
  hsw_lds_init(S);
  __syncthreads();
  hsw_bufs buf;
  hsw_select_row(R, r, kcodes + (int64_t)(r / lq) * pitch, qcodes[r], k, cnt0, s_bm, s_key, S, buf);
}

template <int CPW>
__global__ __launch_bounds__(SF_NT) void k_select16(sah_rows R, const uint16_t* keys, int64_t pitch, int n_cand,
                                                    int col_offset, int k, uint32_t excluded_key, int fresh, int sink,
                                                    int window) {
  sah_touch_kernargs<sizeof(sah_rows) + 56>();
  __shared__ sf_lds S;
  HIP_DYNAMIC_SHARED(unsigned char, sf_dyn)
  const int r = blockIdx.x;
  sf_select_row<CPW>(S, sf_dyn, R, r, keys + (int64_t)r * pitch, n_cand, col_offset, k < n_cand ? k : n_cand,
                     excluded_key, fresh, sink, window);
}

// kernels may use up to 160 KB of LDS; HIP needs to be told once per kernel
template <typename K>
static int sel_allow_lds(K kernel, size_t bytes, const char* what) {
  if (bytes <= 48 * 1024) return SAH_OK;
  return sah_allow_lds((const void*)kernel, 160 * 1024 - 1024, what);
}

// Signature scores as sortable float keys, for callers that pass an additive
// attention mask: score = round_to_dtype(float(sig_score) + amask).
template <int DT>
__global__ __launch_bounds__(256) void k_hamming_scores(const uint2* kcodes, int64_t code_pitch, const uint2* qcodes,
                                                        int Hq, int Lq, int n_keys, const void* amask,
                                                        int64_t ms_b, int64_t ms_h, int64_t ms_l, void* keys_out,
                                                        int64_t key_pitch) {
  typedef typename std::conditional<DT == SAH_F32, uint32_t, uint16_t>::type key_t;
  const int r = blockIdx.y;
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= n_keys) return;
  const int qi = r % Lq;
  const int h = (r / Lq) % Hq;
  const int b = r / (Lq * Hq);
  float s = (float)sig_score(qcodes[r], kcodes[(int64_t)(r / Lq) * code_pitch + j]);
  if (amask) s = sah_round<DT>(s + sah_load<DT>(amask, (int64_t)b * ms_b + (int64_t)h * ms_h + (int64_t)qi * ms_l + j));
  ((key_t*)keys_out)[(int64_t)r * key_pitch + j] = (key_t)sah_sort_key<DT>(s);
}

extern "C" int sah_hamming_scores(const sah_hamming_scores_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hamming_scores: args is NULL");
  if (!a->kcodes || !a->qcodes || !a->keys_out) return sah_fail(SAH_ENULL, "sah_hamming_scores: NULL tensor");
  if (a->B <= 0 || a->Hq <= 0 || a->Lq <= 0 || a->n_keys <= 0)
    return sah_fail(SAH_EINVAL, "sah_hamming_scores: bad dimensions");
  if (a->code_pitch < a->n_keys || a->key_pitch < a->n_keys) return sah_fail(SAH_ECAPACITY, "sah_hamming_scores: pitch < n_keys");
  const int n_rows = a->B * a->Hq * a->Lq;
  if (n_rows > 65535) return sah_fail(SAH_ESHAPE, "sah_hamming_scores: more than 65535 rows");
  dim3 g((a->n_keys + 255) / 256, n_rows), blk(256);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_hamming_scores", a->stream);
#define SAH_HS_LAUNCH(DTC)                                                                                          \
  hipLaunchKernelGGL(k_hamming_scores<DTC>, g, blk, 0, st, (const uint2*)a->kcodes, a->code_pitch,                  \
                     (const uint2*)a->qcodes, a->Hq, a->Lq, a->n_keys, a->amask, a->ms_b, a->ms_h, a->ms_l,        \
                     a->keys_out, a->key_pitch)
  switch (a->dtype) {
    case SAH_F32: SAH_HS_LAUNCH(SAH_F32); break;
    case SAH_BF16: SAH_HS_LAUNCH(SAH_BF16); break;
    case SAH_F16: SAH_HS_LAUNCH(SAH_F16); break;
    default: return sah_fail(SAH_EDTYPE, "sah_hamming_scores: dtype %d", a->dtype);
  }
#undef SAH_HS_LAUNCH
  return sah_launch_status("sah_hamming_scores");
}

int sel_validate(const sah_select_topk_args* a, const char* who) {
  if (!a) return sah_fail(SAH_ENULL, "%s: args is NULL", who);
  int rc = sah_check_rows(a->rows, who);
  if (rc) return rc;
  if (!a->keys) return sah_fail(SAH_ENULL, "%s: keys is NULL", who);
  if (a->key_bits != 16 && a->key_bits != 32) return sah_fail(SAH_EINVAL, "%s: key_bits must be 16 or 32", who);
  if (a->n_cand <= 0 || a->col_offset < 0 || (int64_t)a->col_offset + a->n_cand > a->rows.n_keys)
    return sah_fail(SAH_EINVAL, "%s: candidate range [%d, %d) outside [0, %d)", who, a->col_offset,
                    a->col_offset + a->n_cand, a->rows.n_keys);
  if (a->k <= 0) return sah_fail(SAH_EINVAL, "%s: k must be > 0", who);
  if (a->key_pitch < a->n_cand) return sah_fail(SAH_EINVAL, "%s: key_pitch < n_cand", who);
  if (a->fresh && (a->fresh_sink < 0 || a->fresh_window < 0))
    return sah_fail(SAH_EINVAL, "%s: fresh_sink / fresh_window must be >= 0", who);
  if (a->fresh) {
    int64_t worst = (int64_t)a->fresh_sink + a->fresh_window;
    if (worst > a->rows.n_keys) worst = a->rows.n_keys;
    if (worst > a->rows.cap)
      return sah_fail(SAH_ECAPACITY, "%s: cap %d < sink+window %lld", who, a->rows.cap, (long long)worst);
  }
  return SAH_OK;
}

extern "C" int sah_select_topk(const sah_select_topk_args* a) {
  int rc = sel_validate(a, "sah_select_topk");
  if (rc) return rc;
  hipStream_t st = (hipStream_t)a->stream;
  if (sel16_ok(a)) {
    // eight keys per lane: needs 16-byte aligned key rows
    const size_t lds = sf_lds_bytes(a->rows.n_words);
    const int cpw = sf_chunks_per_wave(a->n_cand);
    sah_timed timed("k_select_topk", a->stream);
#define SAH_SEL16(CPW)                                                                                      \
  do {                                                                                                      \
    rc = sel_allow_lds(k_select16<CPW>, lds, "sah_select_topk");                                            \
    if (rc) return rc;                                                                                      \
    hipLaunchKernelGGL(k_select16<CPW>, dim3(a->rows.n_rows), dim3(SF_NT), lds, st, a->rows,                \
                       (const uint16_t*)a->keys, a->key_pitch, a->n_cand, a->col_offset, a->k, a->excluded_key, \
                       a->fresh ? 1 : 0, a->fresh_sink, a->fresh_window);                                   \
  } while (0)
    if (cpw <= 4) SAH_SEL16(4);
    else if (cpw <= 8) SAH_SEL16(8);
    else if (cpw <= 16) SAH_SEL16(16);
    else SAH_SEL16(0);
#undef SAH_SEL16
    return sah_launch_status("sah_select_topk");
  }
  if (a->fresh) {
    // the general kernel starts from rows in memory: build the sink + local rows with their own launch
    sah_sink_local_args sl = {a->rows, 1, a->fresh_sink, a->fresh_window, 1, 0, a->stream};
    rc = sah_sink_local_indices(&sl);
    if (rc) return rc;
  }
  sel_layout L;
  const size_t lds = sel_plan(a->key_bits, a->key_bits / 8, a->rows.n_words, a->n_cand, a->col_offset, &L);
  if (lds > 159 * 1024) return sah_fail(SAH_ESHAPE, "sah_select_topk: %d keys need %zu bytes of LDS", a->rows.n_keys, lds);
  rc = a->key_bits == 16 ? sel_allow_lds(k_select_topk<16>, lds, "sah_select_topk")
                         : sel_allow_lds(k_select_topk<32>, lds, "sah_select_topk");
  if (rc) return rc;
  sah_timed timed("k_select_topk", a->stream);
  if (a->key_bits == 16)
    hipLaunchKernelGGL(k_select_topk<16>, dim3(a->rows.n_rows), dim3(SEL_NT), lds, st, a->rows, L, a->keys,
                       a->key_pitch, a->n_cand, a->col_offset, a->k, a->excluded_key);
  else
    hipLaunchKernelGGL(k_select_topk<32>, dim3(a->rows.n_rows), dim3(SEL_NT), lds, st, a->rows, L, a->keys,
                       a->key_pitch, a->n_cand, a->col_offset, a->k, a->excluded_key);
  return sah_launch_status("sah_select_topk");
}

extern "C" int sah_hamming_topk(const sah_hamming_topk_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hamming_topk: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_hamming_topk");
  if (rc) return rc;
  if (!a->kcodes || !a->qcodes) return sah_fail(SAH_ENULL, "sah_hamming_topk: codes are NULL");
  if (a->lq <= 0 || a->rows.n_rows % a->lq) return sah_fail(SAH_EINVAL, "sah_hamming_topk: lq must divide n_rows");
  if (a->k <= 0) return sah_fail(SAH_EINVAL, "sah_hamming_topk: k must be > 0");
  if (a->code_pitch < a->rows.n_keys) return sah_fail(SAH_EINVAL, "sah_hamming_topk: code_pitch < n_keys");
  {
    // SWAR kernel: bitmap row + one byte per column in LDS; needs 16-byte aligned code streams
    const int n_ch = (a->rows.n_keys + 255) / 256;
    const size_t lds = (size_t)n_ch * 8 * 4 + (size_t)n_ch * 64 * 4;
    if (lds <= 150 * 1024 && a->code_pitch % 2 == 0 && ((uintptr_t)a->kcodes % 16) == 0 && a->rows.n_keys >= 4) {
      rc = sel_allow_lds(k_hamming_topk_swar, lds, "sah_hamming_topk");
      if (rc) return rc;
      sah_timed timed("k_hamming_topk", a->stream);
      hipLaunchKernelGGL(k_hamming_topk_swar, dim3(a->rows.n_rows), dim3(HSW_NT), lds, (hipStream_t)a->stream, a->rows,
                         (const uint2*)a->kcodes, a->code_pitch, (const uint2*)a->qcodes, a->lq, a->k);
      return sah_launch_status("sah_hamming_topk");
    }
  }
  sel_layout L;
  const size_t lds = sel_plan(7, 1, a->rows.n_words, a->rows.n_keys, 0, &L);
  if (lds > 159 * 1024) return sah_fail(SAH_ESHAPE, "sah_hamming_topk: %d keys need %zu bytes of LDS", a->rows.n_keys, lds);
  rc = sel_allow_lds(k_hamming_topk, lds, "sah_hamming_topk");
  if (rc) return rc;
  sah_timed timed("k_hamming_topk", a->stream);
  hipLaunchKernelGGL(k_hamming_topk, dim3(a->rows.n_rows), dim3(SEL_NT), lds, (hipStream_t)a->stream, a->rows, L,
                     (const uint2*)a->kcodes, a->code_pitch, (const uint2*)a->qcodes, a->lq, a->k);
  return sah_launch_status("sah_hamming_topk");
}
