// Sparse-mask row builders: fused Sink+Local index generation and dense<->rows
// conversion. Integer work; one workgroup per mask row, bitmap kept coherent
// with the column list so later maskers can test membership in O(1).
#include "sah_common.h"

static thread_local char g_err[512];
char* sah_err_buf() { return g_err; }

// ---------------------------------------------------------------------------
// opt-in kernel timing
// ---------------------------------------------------------------------------
#include <mutex>
#include <string>
#include <vector>
namespace {
struct timing_rec {
  const char* name;
  hipEvent_t a, b;
};
std::mutex g_tmu;
bool g_timing = false;
std::vector<timing_rec> g_recs;
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_pool;
}  // namespace

bool sah_timing_enabled() { return g_timing; }

void sah_timing_begin(const char* name, hipStream_t st) {
  std::lock_guard<std::mutex> lk(g_tmu);
  timing_rec r;
  r.name = name;
  if (!g_pool.empty()) {
    r.a = g_pool.back().first;
    r.b = g_pool.back().second;
    g_pool.pop_back();
  } else {
    if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) return;
  }
  (void)hipEventRecord(r.a, st);
  g_recs.push_back(r);
}

void sah_timing_end(hipStream_t st) {
  std::lock_guard<std::mutex> lk(g_tmu);
  if (!g_recs.empty()) (void)hipEventRecord(g_recs.back().b, st);
}

extern "C" int sah_timing_enable(int on) {
  std::lock_guard<std::mutex> lk(g_tmu);
  g_timing = on != 0;
  return SAH_OK;
}

// Waits for the recorded events, adds up the time per kernel name and clears the log.
// names: out array of `max` pointers to static strings; returns the number of distinct kernels.
extern "C" int sah_timing_collect(const char** names, int* counts, float* total_ms, int max) {
  std::lock_guard<std::mutex> lk(g_tmu);
  int n = 0;
  for (auto& r : g_recs) {
    float ms = 0.f;
    if (hipEventSynchronize(r.b) == hipSuccess && hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess) {
      int i = 0;
      for (; i < n; ++i)
        if (names[i] == r.name) break;
      if (i == n) {
        if (n >= max) continue;
        names[n] = r.name;
        counts[n] = 0;
        total_ms[n] = 0.f;
        ++n;
      }
      counts[i] += 1;
      total_ms[i] += ms;
    }
    g_pool.push_back({r.a, r.b});
  }
  g_recs.clear();
  return n;
}

int sah_allow_lds(const void* kernel, size_t bytes, const char* what) {
  static std::mutex mu;
  static std::vector<std::pair<const void*, int>> done;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sah_fail((int)e, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  std::lock_guard<std::mutex> lk(mu);
  for (const auto& d : done)
    if (d.first == kernel && d.second == dev) return SAH_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return sah_fail((int)e, "%s: cannot raise the dynamic LDS limit: %s", what, hipGetErrorString(e));
  done.emplace_back(kernel, dev);
  return SAH_OK;
}

extern "C" int sah_version(void) { return SAH_VERSION; }
extern "C" const char* sah_last_error(void) { return g_err; }

#define ROWS_NT 256
#define ROWS_MAX_WORDS 8192  // LDS bitmap row of from_dense: 32 KB => Lk <= 262144

// Append, in ascending column order, every column whose bit is in `want(wi)`
// but not yet in the row's bitmap; returns the new count. All threads call.
template <int NT, typename F>
__device__ __forceinline__ int rows_append_new_bits(const sah_rows& R, int r, int cnt, int w_begin,
                                                    int w_end, int* s_scan, F want) {
  int* cols = R.cols + (int64_t)r * R.cap;
  float* w = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;
  for (int base = w_begin; base < w_end; base += NT) {
    const int wi = base + (int)threadIdx.x;
    uint32_t nw = 0, old = 0;
    if (wi < w_end) {
      old = bm[wi];
      nw = want(wi) & ~old;
    }
    int total;
    int pos = cnt + sah_block_excl_scan<NT>(__popc(nw), s_scan, &total);
    if (nw) {
      bm[wi] = old | nw;
      while (nw) {
        int b = __ffs((int)nw) - 1;
        nw &= nw - 1;
        if (pos < R.cap) {
          cols[pos] = wi * 32 + b;
          if (w) w[pos] = 1.0f;
        }
        ++pos;
      }
    }
    cnt += total;
  }
  return cnt;
}

__global__ __launch_bounds__(ROWS_NT) void k_sink_local(sah_rows R, int lq, int sink, int window,
                                                        int fresh, int clear_future) {
  __shared__ int s_scan[ROWS_NT / SAH_WAVE + 1];
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int q = r % lq;
  const int Lk = R.n_keys;
  const int last = Lk - lq + q;  // last column this query row may see
  int lo = 0, hi = 0;            // local range [lo, hi)
  if (window > 0) {
    lo = last - window + 1;
    hi = last + 1;
    if (lo < 0) lo = 0;
  }
  int s_hi = sink < Lk ? sink : Lk;  // sink range [0, s_hi)
  if (clear_future && s_hi > last + 1) s_hi = last + 1;

  int* cols = R.cols + (int64_t)r * R.cap;
  float* w = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;

  if (fresh) {
    const int lo2 = lo > s_hi ? lo : s_hi;
    const int n_local = hi > lo2 ? hi - lo2 : 0;
    const int total = s_hi + n_local;
    for (int i = tid; i < total && i < R.cap; i += ROWS_NT) {
      cols[i] = i < s_hi ? i : lo2 + (i - s_hi);
      if (w) w[i] = 1.0f;
    }
    for (int wi = tid; wi < R.n_words; wi += ROWS_NT)
      bm[wi] = sah_range_bits(wi, 0, s_hi) | sah_range_bits(wi, lo, hi);
    if (tid == 0) R.cnt[r] = total;
    return;
  }

  int cnt = R.cnt[r];
  if (cnt > R.cap) cnt = R.cap;

  if (clear_future && lq > 1) {
    // stable in-place compaction of the entries with column <= last
    int kept = 0;
    for (int base = 0; base < cnt; base += ROWS_NT) {
      const int i = base + tid;
      int c = -1;
      float wv = 1.0f;
      if (i < cnt) {
        c = cols[i];
        if (w) wv = w[i];
      }
      const int keep = (c >= 0 && c <= last) ? 1 : 0;
      int total;
      int pos = kept + sah_block_excl_scan<ROWS_NT>(keep, s_scan, &total);
      __syncthreads();  // every read of this chunk is done before any write
      if (keep) {
        cols[pos] = c;
        if (w) w[pos] = wv;
      }
      kept += total;
    }
    cnt = kept;
    for (int wi = tid; wi < R.n_words; wi += ROWS_NT) {
      uint32_t allow = sah_range_bits(wi, 0, last + 1);
      uint32_t old = bm[wi];
      if (old & ~allow) bm[wi] = old & allow;
    }
    __syncthreads();
  }

  if (w) {
    for (int i = tid; i < cnt; i += ROWS_NT) {
      int c = cols[i];
      if (c < s_hi || (c >= lo && c < hi)) w[i] = 1.0f;
    }
  }

  auto want = [=](int wi) { return sah_range_bits(wi, 0, s_hi) | sah_range_bits(wi, lo, hi); };
  if (s_hi > 0) cnt = rows_append_new_bits<ROWS_NT>(R, r, cnt, 0, (s_hi + 31) / 32, s_scan, want);
  if (hi > lo) {
    int wb = lo / 32;
    const int sink_words = (s_hi + 31) / 32;
    if (s_hi > 0 && wb < sink_words) wb = sink_words;  // words below were already merged
    const int we = (hi + 31) / 32;
    if (wb < we) cnt = rows_append_new_bits<ROWS_NT>(R, r, cnt, wb, we, s_scan, want);
  }
  if (tid == 0) R.cnt[r] = cnt;
}

extern "C" int sah_sink_local_indices(const sah_sink_local_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_sink_local_indices: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_sink_local_indices");
  if (rc) return rc;
  if (a->lq <= 0 || a->rows.n_rows % a->lq != 0)
    return sah_fail(SAH_EINVAL, "sah_sink_local_indices: lq must divide n_rows");
  if (a->sink < 0 || a->window < 0) return sah_fail(SAH_EINVAL, "sah_sink_local_indices: negative size");
  if (a->fresh) {
    int64_t worst = (int64_t)(a->sink < a->rows.n_keys ? a->sink : a->rows.n_keys) + a->window;
    if (worst > a->rows.n_keys) worst = a->rows.n_keys;
    if (worst > a->rows.cap)
      return sah_fail(SAH_ECAPACITY, "sah_sink_local_indices: cap %d < sink+window %lld", a->rows.cap,
                      (long long)worst);
  }
  sah_timed timed("k_sink_local", a->stream);
  hipLaunchKernelGGL(k_sink_local, dim3(a->rows.n_rows), dim3(ROWS_NT), 0, (hipStream_t)a->stream, a->rows,
                     a->lq, a->sink, a->window, a->fresh, a->clear_future);
  return sah_launch_status("sah_sink_local_indices");
}

// ---------------------------------------------------------------------------
// dense -> rows
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(ROWS_NT) void k_rows_from_dense(sah_rows R, const void* dense) {
  __shared__ int s_scan[ROWS_NT / SAH_WAVE + 1];
  __shared__ uint32_t s_bm[ROWS_MAX_WORDS];
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  constexpr int NW = ROWS_NT / SAH_WAVE;
  const int Lk = R.n_keys;
  const int64_t rowoff = (int64_t)r * Lk;
  uint32_t* bm = R.bitmap + (int64_t)r * R.n_words;

  const int n_chunks = (Lk + SAH_WAVE - 1) / SAH_WAVE;
  for (int c = wave; c < n_chunks; c += NW) {
    const int j = c * SAH_WAVE + lane;
    float v = 0.f;
    if (j < Lk) v = sah_load<DT>(dense, rowoff + j);
    uint64_t m = __ballot(v != 0.f);
    if (lane == 0) {
      s_bm[2 * c] = (uint32_t)m;
      bm[2 * c] = (uint32_t)m;
    }
    if (lane == 32 && 2 * c + 1 < R.n_words) {
      s_bm[2 * c + 1] = (uint32_t)(m >> 32);
      bm[2 * c + 1] = (uint32_t)(m >> 32);
    }
  }
  __syncthreads();

  int* cols = R.cols + (int64_t)r * R.cap;
  float* w = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  int cnt = 0;
  for (int base = 0; base < R.n_words; base += ROWS_NT) {
    const int wi = base + tid;
    uint32_t nw = wi < R.n_words ? s_bm[wi] : 0u;
    int total;
    int pos = cnt + sah_block_excl_scan<ROWS_NT>(__popc(nw), s_scan, &total);
    while (nw) {
      int b = __ffs((int)nw) - 1;
      nw &= nw - 1;
      if (pos < R.cap) {
        const int col = wi * 32 + b;
        cols[pos] = col;
        if (w) w[pos] = sah_load<DT>(dense, rowoff + col);
      }
      ++pos;
    }
    cnt += total;
  }
  if (tid == 0) R.cnt[r] = cnt;
}

template <int DT>
__global__ __launch_bounds__(ROWS_NT) void k_rows_to_dense(sah_rows R, void* dense) {
  const int r = blockIdx.x;
  int cnt = R.cnt[r];
  if (cnt > R.cap) cnt = R.cap;
  const int* cols = R.cols + (int64_t)r * R.cap;
  const float* w = R.w ? R.w + (int64_t)r * R.cap : nullptr;
  const int64_t rowoff = (int64_t)r * R.n_keys;
  for (int i = threadIdx.x; i < cnt; i += ROWS_NT) {
    const int c = cols[i];
    if (c >= 0 && c < R.n_keys) sah_store<DT>(dense, rowoff + c, w ? w[i] : 1.0f);
  }
}

extern "C" int sah_rows_from_dense(const sah_dense_rows_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_rows_from_dense: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_rows_from_dense");
  if (rc) return rc;
  if (!a->dense) return sah_fail(SAH_ENULL, "sah_rows_from_dense: dense is NULL");
  if (a->rows.n_words > ROWS_MAX_WORDS)
    return sah_fail(SAH_ESHAPE, "sah_rows_from_dense: n_keys %d exceeds %d", a->rows.n_keys, ROWS_MAX_WORDS * 32);
  dim3 g(a->rows.n_rows), b(ROWS_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_rows_from_dense", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_rows_from_dense<SAH_F32>, g, b, 0, st, a->rows, (const void*)a->dense); break;
    case SAH_BF16: hipLaunchKernelGGL(k_rows_from_dense<SAH_BF16>, g, b, 0, st, a->rows, (const void*)a->dense); break;
    case SAH_F16: hipLaunchKernelGGL(k_rows_from_dense<SAH_F16>, g, b, 0, st, a->rows, (const void*)a->dense); break;
    default: return sah_fail(SAH_EDTYPE, "sah_rows_from_dense: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_rows_from_dense");
}

extern "C" int sah_rows_to_dense(const sah_dense_rows_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_rows_to_dense: args is NULL");
  int rc = sah_check_rows(a->rows, "sah_rows_to_dense");
  if (rc) return rc;
  if (!a->dense) return sah_fail(SAH_ENULL, "sah_rows_to_dense: dense is NULL");
  dim3 g(a->rows.n_rows), b(ROWS_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_rows_to_dense", a->stream);
  switch (a->dtype) {
    case SAH_F32: hipLaunchKernelGGL(k_rows_to_dense<SAH_F32>, g, b, 0, st, a->rows, a->dense); break;
    case SAH_BF16: hipLaunchKernelGGL(k_rows_to_dense<SAH_BF16>, g, b, 0, st, a->rows, a->dense); break;
    case SAH_F16: hipLaunchKernelGGL(k_rows_to_dense<SAH_F16>, g, b, 0, st, a->rows, a->dense); break;
    default: return sah_fail(SAH_EDTYPE, "sah_rows_to_dense: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_rows_to_dense");
}

// ---------------------------------------------------------------------------
// What an additive attention mask holds, so that the host can tell once per forward pass whether the mask of a
// decode step is all zeros (HuggingFace's eager mask of an unpadded single-token step) and drop it for every layer.
// ---------------------------------------------------------------------------
#define AMC_NT 256
#define AMC_PER_THREAD 8

template <int DT>
__global__ __launch_bounds__(AMC_NT) void k_amask_classify(const void* amask, int64_t ms_b, int64_t ms_h, int64_t ms_l, int Hm,
                                                           int Lq, int Lk, float lowest, int* flags) {
  const int row = blockIdx.y;  // (b * Hm + h) * Lq + q
  const int q = row % Lq, h = (row / Lq) % Hm, b = row / (Lq * Hm);
  const int64_t base = b * ms_b + h * ms_h + q * ms_l;
  const int c0 = (blockIdx.x * AMC_NT + threadIdx.x) * AMC_PER_THREAD;
  int f = 0;
#pragma unroll
  for (int i = 0; i < AMC_PER_THREAD; ++i) {
    const int c = c0 + i;
    if (c < Lk) {
      const float x = sah_load<DT>(amask, base + c);
      if (x != 0.f) f |= (x <= lowest) ? SAH_AMASK_NONZERO : (SAH_AMASK_NONZERO | SAH_AMASK_GENERAL);  // NaN: general
    }
  }
  if (__ballot(f != 0)) {
    // one atomic per wave that saw anything
    for (int m = 32; m >= 1; m >>= 1) f |= __shfl_xor(f, m);
    if ((threadIdx.x & (SAH_WAVE - 1)) == 0) atomicOr(flags, f);
  }
}

extern "C" int sah_amask_classify(const sah_amask_classify_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_amask_classify: args is NULL");
  if (!a->amask || !a->flags) return sah_fail(SAH_ENULL, "sah_amask_classify: amask / flags is NULL");
  if (a->B <= 0 || a->Hm <= 0 || a->Lq <= 0 || a->Lk <= 0) return sah_fail(SAH_EINVAL, "sah_amask_classify: B, Hm, Lq, Lk must be > 0");
  const int64_t rows = (int64_t)a->B * a->Hm * a->Lq;
  if (rows > 65535) return sah_fail(SAH_ESHAPE, "sah_amask_classify: %lld mask rows exceed 65535", (long long)rows);
  const dim3 g((unsigned)((a->Lk + AMC_NT * AMC_PER_THREAD - 1) / (AMC_NT * AMC_PER_THREAD)), (unsigned)rows), blk(AMC_NT);
  hipStream_t st = (hipStream_t)a->stream;
  sah_timed timed("k_amask_classify", a->stream);
  // "as low as the lowest finite value of the dtype" (what HuggingFace's masks put on a hidden column) or -inf
  switch (a->dtype) {
    case SAH_F32:
      hipLaunchKernelGGL(k_amask_classify<SAH_F32>, g, blk, 0, st, a->amask, a->ms_b, a->ms_h, a->ms_l, a->Hm, a->Lq, a->Lk,
                         -3.4028234663852886e38f, a->flags);
      break;
    case SAH_BF16:
      hipLaunchKernelGGL(k_amask_classify<SAH_BF16>, g, blk, 0, st, a->amask, a->ms_b, a->ms_h, a->ms_l, a->Hm, a->Lq, a->Lk,
                         -3.3895313892515355e38f, a->flags);
      break;
    case SAH_F16:
      hipLaunchKernelGGL(k_amask_classify<SAH_F16>, g, blk, 0, st, a->amask, a->ms_b, a->ms_h, a->ms_l, a->Hm, a->Lq, a->Lk, -65504.0f,
                         a->flags);
      break;
    default: return sah_fail(SAH_EDTYPE, "sah_amask_classify: dtype %d", a->dtype);
  }
  return sah_launch_status("sah_amask_classify");
}
