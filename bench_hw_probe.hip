// Bench-only measurement aid (loaded by `bench.py --hw-probe`, no part of libsah_mi355.so or of its ABI): what this GPU
// gives to the access pattern of the exact-score pass (a long read stream, alone and with 1/32 of its volume written
// back) and to the instruction mix of the Lloyd assignment (matrix instructions, vector instructions, both
// interleaved). The roofline fractions of k_qk_scores and k_pq_assign_mfma are judged against these figures.
//   kind 0  a read stream of `bytes` bytes (64 KB per workgroup, 1 KB per wave instruction, non-temporal loads);
//   kind 1  the same with 1/32 of the volume written to dst, as four 128-byte stores to four rows per 16 KB read;
//   kind 2  the same volume written as one 512-byte store per 16 KB;
//   kind 3  `workgroups` workgroups of 4 waves, `iters` iterations of four dependent 32x32x2 fp32 matrix instructions;
//   kind 4  the same loop with 48 vector instructions instead;
//   kind 5  both, interleaved.
// Returns 0, or -1 for arguments outside these bounds: bytes a multiple of 65536, dst_bytes >= bytes / 32 (kinds
// 0-2; kind 0 writes nothing) or >= 4 (kinds 3-5), iters in [1, 16384], workgroups in [1, 4096].
#include <hip/hip_runtime.h>
#include <cstdint>

#define PR_WAVE 64
typedef float pr_f32x16 __attribute__((ext_vector_type(16)));
#define PR_NT 256
#define PR_CHUNK 65536  // bytes a workgroup reads: a wave its quarter, as two batches of eight 1 KB loads

// kind 0: read only. kind 1: after each 16 KB a wave writes four 128-byte pieces to four rows `pitch` bytes apart
// (the 2-byte keys of 64 columns for the four query heads of a group). kind 2: the same 512 bytes as one store.
template <int KIND>
__global__ __launch_bounds__(PR_NT) void k_probe_stream(const char* src, char* dst, int64_t pitch) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & (PR_WAVE - 1), wave = threadIdx.x / PR_WAVE;
  const int64_t at = (int64_t)blockIdx.x * PR_CHUNK + (int64_t)wave * (PR_CHUNK / 4);
  const char* p = src + at + lane * 16;
  uint32_t acc = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    u4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load((const u4*)(p + h * 8192 + u * 1024));
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  const int64_t oo = at / 32;  // 512 bytes of output for these 16 KB
  if (KIND == 1) {
#pragma unroll
    for (int r = 0; r < 4; ++r) *((uint16_t*)(dst + r * pitch + oo / 4) + lane) = (uint16_t)(acc + r);
  } else if (KIND == 2) {
    *((uint64_t*)(dst + oo) + lane) = (uint64_t)acc;
  } else if (acc == 0x12345678u) {
    dst[0] = (char)acc;  // keeps the loads alive
  }
}

// kind 3: four dependent 32x32x2 fp32 matrix instructions per iteration (one centre tile of the Lloyd assignment);
// kind 4: 48 vector instructions per iteration on four dependent chains (its minimum search); kind 5: both, interleaved
template <int KIND>
__global__ __launch_bounds__(PR_NT, 2) void k_probe_issue(float* out, int iters, float a, float b) {
  pr_f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = (float)threadIdx.x;
  float v0 = a, v1 = b, v2 = a + 1.f, v3 = b + 1.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (KIND != 4) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
      if (KIND != 3) {
#pragma unroll
        for (int q = 0; q < 3; ++q) {
          v0 = fmaf(v0, a, b); v1 = fmaf(v1, a, b); v2 = fmaf(v2, a, b); v3 = fmaf(v3, a, b);
        }
      }
    }
  }
  float r = v0 + v1 + v2 + v3;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += acc[i];
  if (r == 12345.678f) out[0] = r;
}

extern "C" int bench_hw_probe(int kind, const void* src, int64_t bytes, void* dst, int64_t dst_bytes, int iters,
                              int workgroups, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (kind >= 0 && kind <= 2) {
    if (!src || !dst) return -1;
    if (bytes < PR_CHUNK || bytes % PR_CHUNK || bytes / PR_CHUNK > 0x7fffffff) return -1;
    if (((uintptr_t)src | (uintptr_t)dst) & 15) return -1;
    if (dst_bytes < bytes / 32) return -1;
    const dim3 g((unsigned)(bytes / PR_CHUNK)), blk(PR_NT);
    const int64_t pitch = bytes / 128;  // four rows, a quarter of the written volume each
    if (kind == 0) hipLaunchKernelGGL(k_probe_stream<0>, g, blk, 0, st, (const char*)src, (char*)dst, pitch);
    else if (kind == 1) hipLaunchKernelGGL(k_probe_stream<1>, g, blk, 0, st, (const char*)src, (char*)dst, pitch);
    else hipLaunchKernelGGL(k_probe_stream<2>, g, blk, 0, st, (const char*)src, (char*)dst, pitch);
    return hipGetLastError() == hipSuccess ? 0 : -2;
  }
  if (kind >= 3 && kind <= 5) {
    if (!dst || dst_bytes < 4) return -1;
    if (iters <= 0 || iters > (1 << 14) || workgroups <= 0 || workgroups > 4096) return -1;
    const dim3 g((unsigned)workgroups), blk(PR_NT);
    if (kind == 3) hipLaunchKernelGGL(k_probe_issue<3>, g, blk, 0, st, (float*)dst, iters, 1.0f, 0.5f);
    else if (kind == 4) hipLaunchKernelGGL(k_probe_issue<4>, g, blk, 0, st, (float*)dst, iters, 1.0f, 0.5f);
    else hipLaunchKernelGGL(k_probe_issue<5>, g, blk, 0, st, (float*)dst, iters, 1.0f, 0.5f);
    return hipGetLastError() == hipSuccess ? 0 : -2;
  }
  return -1;
}
