// Measurement aid, not part of the decode path: what this GPU gives to the access pattern of the exact-score
// pass (a long read stream, alone and with 1/32 of its volume written back) and to the instruction mix of the
// Lloyd assignment (matrix instructions, vector instructions, both interleaved). The roofline fractions of
// k_qk_scores and k_pq_assign_mfma are judged against these figures.
#include "sah_common.h"

#define PR_NT 256
#define PR_CHUNK 65536  // bytes a workgroup reads: a wave its quarter, as two batches of eight 1 KB loads

// kind 0: read only. kind 1: after each 16 KB a wave writes four 128-byte pieces to four rows `pitch` bytes apart
// (the 2-byte keys of 64 columns for the four query heads of a group). kind 2: the same 512 bytes as one store.
template <int KIND>
__global__ __launch_bounds__(PR_NT) void k_probe_stream(const char* src, char* dst, int64_t pitch) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & (SAH_WAVE - 1), wave = threadIdx.x / SAH_WAVE;
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
  sah_f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = (float)threadIdx.x;
  float v0 = a, v1 = b, v2 = a + 1.f, v3 = b + 1.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (KIND != 4) acc = sah_mfma_32x32x2_f32(a, b, acc);
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

extern "C" int sah_hw_probe(const sah_hw_probe_args* a) {
  if (!a) return sah_fail(SAH_ENULL, "sah_hw_probe: args is NULL");
  hipStream_t st = (hipStream_t)a->stream;
  if (a->kind >= 0 && a->kind <= 2) {
    if (!a->src || !a->dst) return sah_fail(SAH_ENULL, "sah_hw_probe: NULL src / dst");
    if (a->bytes < PR_CHUNK || a->bytes % PR_CHUNK || a->bytes / PR_CHUNK > 0x7fffffff)
      return sah_fail(SAH_EINVAL, "sah_hw_probe: bytes must be a multiple of %d", PR_CHUNK);
    if (((uintptr_t)a->src | (uintptr_t)a->dst) & 15) return sah_fail(SAH_ESHAPE, "sah_hw_probe: src / dst must be 16-byte aligned");
    if (a->dst_bytes < a->bytes / 32) return sah_fail(SAH_EINVAL, "sah_hw_probe: dst_bytes < bytes / 32");
    const dim3 g((unsigned)(a->bytes / PR_CHUNK)), blk(PR_NT);
    const int64_t pitch = a->bytes / 128;  // four rows, a quarter of the written volume each
    if (a->kind == 0) hipLaunchKernelGGL(k_probe_stream<0>, g, blk, 0, st, (const char*)a->src, (char*)a->dst, pitch);
    else if (a->kind == 1) hipLaunchKernelGGL(k_probe_stream<1>, g, blk, 0, st, (const char*)a->src, (char*)a->dst, pitch);
    else hipLaunchKernelGGL(k_probe_stream<2>, g, blk, 0, st, (const char*)a->src, (char*)a->dst, pitch);
    return sah_launch_status("sah_hw_probe");
  }
  if (a->kind >= 3 && a->kind <= 5) {
    if (!a->dst || a->dst_bytes < 4) return sah_fail(SAH_ENULL, "sah_hw_probe: dst must hold a float");
    if (a->iters <= 0 || a->iters > (1 << 20) || a->workgroups <= 0 || a->workgroups > (1 << 16))
      return sah_fail(SAH_EINVAL, "sah_hw_probe: iters in [1, 2^20], workgroups in [1, 2^16]");
    const dim3 g((unsigned)a->workgroups), blk(PR_NT);
    if (a->kind == 3) hipLaunchKernelGGL(k_probe_issue<3>, g, blk, 0, st, (float*)a->dst, a->iters, 1.0f, 0.5f);
    else if (a->kind == 4) hipLaunchKernelGGL(k_probe_issue<4>, g, blk, 0, st, (float*)a->dst, a->iters, 1.0f, 0.5f);
    else hipLaunchKernelGGL(k_probe_issue<5>, g, blk, 0, st, (float*)a->dst, a->iters, 1.0f, 0.5f);
    return sah_launch_status("sah_hw_probe");
  }
  return sah_fail(SAH_EINVAL, "sah_hw_probe: kind %d not in 0..5", a->kind);
}
