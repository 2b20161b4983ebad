// Shared device/host helpers for the gfx950 kernels of libsah_mi355.so.
// Wavefront = 64 lanes; a DPP "row" = 16 lanes; LDS = 160 KB per CU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <type_traits>

#include "../../include/sah.h"

#define SAH_WAVE 64

// ---------------------------------------------------------------------------
// host side: error reporting
// ---------------------------------------------------------------------------
char* sah_err_buf();  // thread-local, 512 bytes

static inline int sah_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(sah_err_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}

// Opt-in per-kernel timing with HIP events on the launch stream (see sah_timing_* in
// include/sah.h). A scope brackets one kernel launch; it costs nothing when disabled.
bool sah_timing_enabled();
void sah_timing_begin(const char* name, hipStream_t st);
void sah_timing_end(hipStream_t st);
struct sah_timed {
  hipStream_t st;
  bool on;
  // allow = false: never time (entry points that must not create events)
  sah_timed(const char* name, void* stream, bool allow = true) : st((hipStream_t)stream), on(allow && sah_timing_enabled()) {
    if (on) sah_timing_begin(name, st);
  }
  ~sah_timed() {
    if (on) sah_timing_end(st);
  }
};

static inline int sah_launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    return sah_fail((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
  }
  return SAH_OK;
}

// A kernel that wants more than 48 KB of dynamic LDS needs hipFuncAttributeMaxDynamicSharedMemorySize raised
// once per (kernel, device). Thread-safe; remembers what has been done (defined with the row builders).
int sah_allow_lds(const void* kernel, size_t bytes, const char* what);

static inline int sah_check_rows(const sah_rows& r, const char* what, bool need_cols = true) {
  if (r.n_rows <= 0 || r.n_keys <= 0) return sah_fail(SAH_EINVAL, "%s: rows.n_rows/n_keys must be > 0", what);
  if (r.n_words != (r.n_keys + 31) / 32) return sah_fail(SAH_EINVAL, "%s: rows.n_words != ceil(n_keys/32)", what);
  if (!r.cnt || !r.bitmap) return sah_fail(SAH_ENULL, "%s: rows.cnt / rows.bitmap is NULL", what);
  if (need_cols && (!r.cols || r.cap <= 0)) return sah_fail(SAH_ENULL, "%s: rows.cols is NULL or cap <= 0", what);
  return SAH_OK;
}

// The calling wave's index in its (one-dimensional) workgroup, in a scalar register: loops and conditions on it
// compile to scalar branches instead of execution-mask bookkeeping.
__device__ __forceinline__ int sah_wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x / SAH_WAVE)); }

// ---------------------------------------------------------------------------
// device side: kernel arguments
// ---------------------------------------------------------------------------
// A kernel's arguments live in memory and are fetched by scalar loads where the code first needs them. Each
// first touch of a 64-byte line is a round trip of about 500 cycles, and the compiler chains them (a load, a
// wait, the next load ...) along the kernel's control flow: 5 to 6 round trips before the first vector load of a
// kernel with a 700-byte argument block. Called first thing in a kernel, this reads one word of every line of
// the first BYTES of the block in ONE batch; the real loads that follow hit the scalar cache.
template <int BYTES>
__device__ __forceinline__ void sah_touch_kernargs() {
  static_assert(BYTES <= 1024, "at most 16 lines");
#if defined(__HIP_DEVICE_COMPILE__)
  typedef const int __attribute__((address_space(4))) karg_int;
  karg_int* p = (karg_int*)__builtin_amdgcn_kernarg_segment_ptr();
  // word o of line i, or of line 0 again when the block is shorter; one sink for all of them, so that every
  // load is issued before the one wait
#define SAH_KARG(i) p[(64 * (i) < BYTES ? 16 * (i) : 0)]
  asm volatile("" ::"s"(SAH_KARG(0)), "s"(SAH_KARG(1)), "s"(SAH_KARG(2)), "s"(SAH_KARG(3)), "s"(SAH_KARG(4)), "s"(SAH_KARG(5)),
               "s"(SAH_KARG(6)), "s"(SAH_KARG(7)), "s"(SAH_KARG(8)), "s"(SAH_KARG(9)), "s"(SAH_KARG(10)), "s"(SAH_KARG(11)),
               "s"(SAH_KARG(12)), "s"(SAH_KARG(13)), "s"(SAH_KARG(14)), "s"(SAH_KARG(15)));
#undef SAH_KARG
#endif
}

// ---------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3")
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t sah_mulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }

__device__ __forceinline__ void sah_philox(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                           uint32_t (&out)[4]) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t hi0 = sah_mulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = sah_mulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// Dropout of the exp weights: what an entry's weight is multiplied by (0, or 1 / (1 - p)). thresh = p * 2^32.
struct sah_dropout {
  uint32_t thresh;  // 0: off
  float scale;
  uint32_t k0, k1, o0, o1;
  __device__ __forceinline__ float factor(int row, int col) const {
    uint32_t u[4];
    sah_philox((uint32_t)col, (uint32_t)row, o0, o1, k0, k1, u);
    return u[0] < thresh ? 0.f : scale;
  }
};
// host side: from the entry point's three arguments; false when p is outside [0, 1)
static inline bool sah_dropout_fill(float p, uint64_t seed, uint64_t offset, sah_dropout& d) {
  d.thresh = 0; d.scale = 1.f; d.k0 = d.k1 = d.o0 = d.o1 = 0;
  if (!(p >= 0.f) || !(p < 1.f)) return false;
  if (p == 0.f) return true;
  const double t = (double)p * 4294967296.0;
  d.thresh = t >= 4294967295.0 ? 0xffffffffu : (uint32_t)t;
  if (d.thresh == 0) d.thresh = 1;
  d.scale = 1.0f / (1.0f - p);
  d.k0 = (uint32_t)seed; d.k1 = (uint32_t)(seed >> 32);
  d.o0 = (uint32_t)offset; d.o1 = (uint32_t)(offset >> 32);
  return true;
}

// ---------------------------------------------------------------------------
// device side: dtype helpers (bf16 / f16 handled as raw bits, fp32 arithmetic)
// ---------------------------------------------------------------------------
__device__ __forceinline__ float sah_bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t sah_float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float sah_bf16_to_float(uint16_t h) { return sah_bits_to_float(((uint32_t)h) << 16); }

// round-to-nearest-even fp32 -> bf16 (what torch's .to(bfloat16) does): the hardware converter, one instruction
// and no branch (a NaN stays a NaN)
__device__ __forceinline__ uint16_t sah_float_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

__device__ __forceinline__ float sah_f16_to_float(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ uint16_t sah_float_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// value of `f` after a round trip through storage type DT
template <int DT>
__device__ __forceinline__ float sah_round(float f) {
  if (DT == SAH_BF16) return (float)(__bf16)f;
  if (DT == SAH_F16) return (float)(_Float16)f;
  return f;
}

// two values rounded to the 16-bit storage type DT and packed, lo in the low half
template <int DT>
__device__ __forceinline__ uint32_t sah_pack2_hw(float lo, float hi) {
  if (DT == SAH_BF16) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    const v2 p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
  }
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  const v2 p = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, p);
}

template <int DT>
__device__ __forceinline__ float sah_load(const void* p, int64_t i) {
  if (DT == SAH_BF16) return sah_bf16_to_float(((const uint16_t*)p)[i]);
  if (DT == SAH_F16) return sah_f16_to_float(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

template <int DT>
__device__ __forceinline__ void sah_store(void* p, int64_t i, float f) {
  if (DT == SAH_BF16) ((uint16_t*)p)[i] = sah_float_to_bf16(f);
  else if (DT == SAH_F16) ((uint16_t*)p)[i] = sah_float_to_f16(f);
  else ((float*)p)[i] = f;
}

// 8 consecutive elements starting at element index i (i % 8 == 0, 16-byte
// aligned for 2-byte types, 32-byte for fp32) -> 8 floats
template <int DT>
__device__ __forceinline__ void sah_load8(const void* p, int64_t i, float (&o)[8]) {
  if (DT == SAH_F32) {
    const float4* f = (const float4*)((const float*)p + i);
    float4 a = f[0], b = f[1];
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    uint4 u = *(const uint4*)((const uint16_t*)p + i);
    uint32_t w[4] = {u.x, u.y, u.z, u.w};
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

// order-preserving key of a score already rounded to DT: larger score => larger
// unsigned key; -0 and +0 map to the same key (torch compares them equal).
template <int DT>
__device__ __forceinline__ uint32_t sah_sort_key(float score) {
  if (DT == SAH_F32) {
    uint32_t u = sah_float_to_bits(score);
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  } else {
    uint32_t u = (DT == SAH_BF16) ? sah_float_to_bf16(score) : sah_float_to_f16(score);
    if (u == 0x8000u) u = 0;
    return (u & 0x8000u) ? ((~u) & 0xffffu) : (u | 0x8000u);
  }
}

// c + a.lo * b.lo + a.hi * b.hi for two packed 16-bit pairs of storage type DT (bf16 or f16),
// products and sum in fp32: one instruction on the device
template <int DT>
__device__ __forceinline__ float sah_dot2(uint32_t a, uint32_t b, float c) {
#if defined(__HIP_DEVICE_COMPILE__)
  if (DT == SAH_BF16) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, a), __builtin_bit_cast(bf2, b), c, false);
  } else {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), c, false);
  }
#else
  if (DT == SAH_BF16) {
    return c + sah_bits_to_float(a << 16) * sah_bits_to_float(b << 16) +
           sah_bits_to_float(a & 0xffff0000u) * sah_bits_to_float(b & 0xffff0000u);
  }
  return c + sah_f16_to_float((uint16_t)(a & 0xffffu)) * sah_f16_to_float((uint16_t)(b & 0xffffu)) +
         sah_f16_to_float((uint16_t)(a >> 16)) * sah_f16_to_float((uint16_t)(b >> 16));
#endif
}

// D = A (32 x 16) * B (16 x 32) + C on the matrix cores, 16-bit inputs, fp32 accumulation. Per lane 8 packed
// elements of A and of B and 16 of C (layouts checked on the hardware):
//   A[i][k]: lane i + 32 g holds k = 8 g .. 8 g + 7;   B[k][j]: lane j + 32 g holds k = 8 g .. 8 g + 7;
//   C[i][j]: lane j + 32 g, element v holds i = 8 (v / 4) + 4 g + v % 4.
typedef float sah_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 sah_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 sah_f16x8 __attribute__((ext_vector_type(8)));
template <int DT>
__device__ __forceinline__ sah_f32x16 sah_mfma_32x32x16(uint4 a, uint4 b, sah_f32x16 c) {
  if (DT == SAH_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(sah_bf16x8, a), __builtin_bit_cast(sah_bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(sah_f16x8, a), __builtin_bit_cast(sah_f16x8, b), c, 0, 0, 0);
}

// D = A (32 x 2) * B (2 x 32) + C in fp32 (layouts checked on the hardware): A[i][k]: lane i + 32 k;
// B[k][j]: lane j + 32 k; C as for the 32 x 32 x 16 form above.
__device__ __forceinline__ sah_f32x16 sah_mfma_32x32x2_f32(float a, float b, sah_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// D = A (16 x 32) * B (32 x 16) + C, 16-bit inputs, fp32 accumulation (layouts checked on the hardware):
//   A[i][k]: lane i + 16 g holds k = 8 g .. 8 g + 7 (g = 0..3);   B[k][j]: lane j + 16 g likewise;
//   C[i][j]: lane j + 16 g, element v holds i = 4 g + v.
typedef float sah_f32x4 __attribute__((ext_vector_type(4)));
template <int DT>
__device__ __forceinline__ sah_f32x4 sah_mfma_16x16x32(uint4 a, uint4 b, sah_f32x4 c) {
  if (DT == SAH_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sah_bf16x8, a), __builtin_bit_cast(sah_bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sah_f16x8, a), __builtin_bit_cast(sah_f16x8, b), c, 0, 0, 0);
}

// Pins a loaded value at this point of the program: the load that produced it must have
// been issued (and is waited for) here, so the compiler can neither sink it into a later
// branch nor serialise a batch of independent loads one wait at a time.
__device__ __forceinline__ void sah_keep(uint32_t& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#endif
}
__device__ __forceinline__ void sah_keep(float& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#endif
}

// Two unsigned 16-bit compares per instruction pair, for keys packed two to a word.
// Result per half: 1 where a > b, else 0 (saturating packed subtract, then min with 1).
__device__ __forceinline__ uint32_t sah_pk_gt01_u16(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t d;
  asm("v_pk_sub_u16 %0, %1, %2 clamp" : "=v"(d) : "v"(a), "v"(b));
  asm("v_pk_min_u16 %0, %1, %2" : "=v"(d) : "v"(d), "v"(0x00010001u));
  return d;
#else
  return ((a & 0xffffu) > (b & 0xffffu) ? 1u : 0u) | ((a >> 16) > (b >> 16) ? 0x10000u : 0u);
#endif
}
// larger of the two unsigned 16-bit halves, per half
__device__ __forceinline__ uint32_t sah_pk_max_u16(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t d;
  asm("v_pk_max_u16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
#else
  const uint32_t lo = (a & 0xffffu) > (b & 0xffffu) ? (a & 0xffffu) : (b & 0xffffu);
  const uint32_t hi = (a >> 16) > (b >> 16) ? (a >> 16) : (b >> 16);
  return lo | (hi << 16);
#endif
}
// Result per half: 1 where a != b, else 0
__device__ __forceinline__ uint32_t sah_pk_ne01_u16(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t d;
  asm("v_pk_min_u16 %0, %1, %2" : "=v"(d) : "v"(a ^ b), "v"(0x00010001u));
  return d;
#else
  return ((a ^ b) & 0xffffu ? 1u : 0u) | ((a ^ b) >> 16 ? 0x10000u : 0u);
#endif
}

// ---------------------------------------------------------------------------
// Hand-over between workgroups of one kernel, without a cache write-back.
// An MI355X has eight L2 caches (one per die). A device-scope release fence makes a workgroup's ordinary stores
// visible to the other dies by writing the whole L2 back, which costs more than the kernels here run for. The
// accesses below are device-scope *atomic* loads / stores / read-modify-writes (relaxed): they bypass the
// non-coherent cache levels by themselves, so data handed over with them needs no fence, only the wait that orders
// a workgroup's stores before its arrival ticket:
//   producer: sah_agent_store_* the data; sah_stores_done(); __syncthreads(); one thread calls sah_last_arrival
//   consumer: (the workgroup that arrived last) __syncthreads(); sah_agent_load_* the data
// Nobody ever waits for another workgroup: the last one to arrive does the common work.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void sah_agent_store_f32(float* p, float v) {
#if defined(__HIP_DEVICE_COMPILE__)
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
  *(volatile float*)p = v;
#endif
}
__device__ __forceinline__ float sah_agent_load_f32(const float* p) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
  return *(const volatile float*)p;
#endif
}
// every store this thread has issued has reached its point of coherence
__device__ __forceinline__ void sah_stores_done() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}
// Arrival ticket of one of `n` workgroups that share `word` (zero before the first of them arrives): returns true for
// the one that arrives last, which also puts the word back to zero for the next kernel that uses it. One atomic
// read-modify-write per workgroup, no retry loop: eight workgroups arriving together do not queue behind each other.
__device__ __forceinline__ bool sah_last_arrival(uint32_t* word, uint32_t n) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t before = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (before + 1u != n) return false;
  __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
#else
  const uint32_t before = __atomic_fetch_add(word, 1u, __ATOMIC_RELAXED);
  if (before + 1u != n) return false;
  __atomic_store_n(word, 0u, __ATOMIC_RELAXED);
  return true;
#endif
}

// Orders the LDS traffic of ONE wave: what its lanes wrote before is visible to its lanes after.
// For LDS regions that a single wave owns; costs a wait on the wave's own LDS queue, no workgroup barrier.
__device__ __forceinline__ void sah_wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------
// device side: cross-lane helpers
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float sah_dpp(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// sum over each aligned group of 16 lanes (one DPP row); every lane gets the sum
__device__ __forceinline__ float sah_row16_sum(float v) {
  v += sah_dpp<0xB1>(v);   // quad_perm [1,0,3,2]
  v += sah_dpp<0x4E>(v);   // quad_perm [2,3,0,1]
  v += sah_dpp<0x141>(v);  // row_half_mirror
  v += sah_dpp<0x140>(v);  // row_mirror
  return v;
}

__device__ __forceinline__ float sah_wave_sum(float v) {
  v = sah_row16_sum(v);
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

__device__ __forceinline__ float sah_wave_max(float v) {
  v = fmaxf(v, sah_dpp<0xB1>(v));
  v = fmaxf(v, sah_dpp<0x4E>(v));
  v = fmaxf(v, sah_dpp<0x141>(v));
  v = fmaxf(v, sah_dpp<0x140>(v));
  v = fmaxf(v, __shfl_xor(v, 16));
  v = fmaxf(v, __shfl_xor(v, 32));
  return v;
}

template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ int sah_dpp_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xF, BOUND);
}

// inclusive scan of one int per lane across the wave, all in DPP (no LDS traffic):
// Hillis-Steele inside each row of 16 lanes, then the row totals are carried across rows
__device__ __forceinline__ int sah_wave_incl_scan(int v) {
  v += sah_dpp_i<0x111, 0xF, true>(v);   // row_shr:1, lanes without a source add 0
  v += sah_dpp_i<0x112, 0xF, true>(v);   // row_shr:2
  v += sah_dpp_i<0x114, 0xF, true>(v);   // row_shr:4
  v += sah_dpp_i<0x118, 0xF, true>(v);   // row_shr:8
  v += sah_dpp_i<0x142, 0xA, false>(v);  // row_bcast:15 into rows 1 and 3
  v += sah_dpp_i<0x143, 0xC, false>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// sum over the wave; every lane gets it
__device__ __forceinline__ int sah_wave_sum_i(int v) {
  return __builtin_amdgcn_readlane(sah_wave_incl_scan(v), SAH_WAVE - 1);
}

// number of set bits of `m` at lane positions below the calling lane
__device__ __forceinline__ int sah_lane_prefix(uint64_t m) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
}

// Exclusive scan of one int per thread across a block of NT threads
// (NT % 64 == 0, NT <= 1024). `wsum` is LDS scratch of NT/64 + 1 ints. All
// threads must call. Returns the exclusive prefix; *total receives the sum.
template <int NT>
__device__ __forceinline__ int sah_block_excl_scan(int v, int* wsum, int* total) {
  constexpr int NW = NT / SAH_WAVE;
  const int lane = threadIdx.x & (SAH_WAVE - 1);
  const int wave = sah_wave_id();
  int incl = sah_wave_incl_scan(v);
  __syncthreads();  // protect wsum from a previous use
  if (lane == SAH_WAVE - 1) wsum[wave] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int i = 0; i < NW; ++i) {
      int t = wsum[i];
      wsum[i] = run;
      run += t;
    }
    wsum[NW] = run;
  }
  __syncthreads();
  *total = wsum[NW];
  return wsum[wave] + incl - v;
}

// bits of 32-bit word `wi` that fall inside column range [lo, hi)
__device__ __forceinline__ uint32_t sah_range_bits(int wi, int lo, int hi) {
  int base = wi * 32;
  int a = lo - base, b = hi - base;
  if (b <= 0 || a >= 32) return 0u;
  if (a < 0) a = 0;
  if (b > 32) b = 32;
  uint32_t upto_b = (b == 32) ? 0xffffffffu : ((1u << b) - 1u);
  uint32_t upto_a = (a == 0) ? 0u : ((1u << a) - 1u);
  return upto_b & ~upto_a;
}
