// What the machine gives: the rate at which a kernel can read and copy device memory, and the rate of the
// bfloat16 matrix-core instruction. bench.py times these once and prints them beside the published peaks that
// its roofline fractions are taken against (the reference has no counterpart; its instruments are wall-clock
// log lines, example/examples/llm_engine_example.rs:59,127,149).
#include "common.h"

// A workgroup reads a contiguous part of the buffer, 32 KB at a time: every thread has eight 16-byte loads in
// flight. (With the grid striding over the buffer and four loads in flight the same chip gives 5.6 TB/s instead
// of 6.3: neighbouring workgroups then sit in different pages of memory all the time.) The loads are marked
// non-temporal, as the kernels' loads of what they read once are: the caches then keep nothing of the stream, and the
// same read runs at 6.7 TB/s instead of 6.3.
typedef unsigned int measure_u32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void measure_read_kernel(const uint4* __restrict__ src, long n16,
                                                           unsigned* __restrict__ sink) {
  constexpr int U = 8;
  unsigned acc = 0;
  const long per = n16 / gridDim.x;
  const long begin = (long)blockIdx.x * per, end = blockIdx.x == gridDim.x - 1 ? n16 : begin + per;
  long i = begin + threadIdx.x;
  for (; i + (U - 1) * 256 < end; i += U * 256) {
    measure_u32x4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const measure_u32x4_t*>(src + i + u * 256));
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < end; i += 256) {
    const measure_u32x4_t a = __builtin_nontemporal_load(reinterpret_cast<const measure_u32x4_t*>(src + i));
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;   // never, for the buffers bench.py fills; keeps the loads alive
}

__global__ __launch_bounds__(256) void measure_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                           long n16) {
  const long stride = (long)gridDim.x * 256;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Four independent accumulators per wave, so that the matrix pipe always has an instruction to issue.
__global__ __launch_bounds__(256) void measure_mfma_kernel(float* __restrict__ sink, int iters) {
  bf16x8_t a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(float)(threadIdx.x % 7);
    b[i] = (__bf16)(float)(threadIdx.x % 5);
  }
  f32x4_t c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c3, 0, 0, 0);
  }
  const float s = c0[0] + c1[1] + c2[2] + c3[3];
  if (s == -1.f) sink[0] = s;
}

// Reads ``bytes`` (a multiple of 16) from src once.
extern "C" int lmsf_measure_read(const void* src, long bytes, void* sink, hipStream_t stream) {
  LMSF_CHECK(src && sink && bytes > 0 && bytes % 16 == 0 && lmsf_aligned16(src), "measure_read: bad arguments");
  const int cus = lmsf_compute_units();
  hipLaunchKernelGGL(measure_read_kernel, dim3((cus > 0 ? cus : 256) * 16), dim3(256), 0, stream, (const uint4*)src,
                     bytes / 16, (unsigned*)sink);
  LMSF_LAUNCH_CHECK("measure_read");
  return 0;
}

extern "C" int lmsf_measure_copy(const void* src, void* dst, long bytes, hipStream_t stream) {
  LMSF_CHECK(src && dst && bytes > 0 && bytes % 16 == 0 && lmsf_aligned16(src) && lmsf_aligned16(dst),
             "measure_copy: bad arguments");
  const int cus = lmsf_compute_units();
  hipLaunchKernelGGL(measure_copy_kernel, dim3((cus > 0 ? cus : 256) * 8), dim3(256), 0, stream, (const uint4*)src,
                     (uint4*)dst, bytes / 16);
  LMSF_LAUNCH_CHECK("measure_copy");
  return 0;
}

// ``iters`` rounds of four 16x16x32 bfloat16 matrix instructions in every wave of ``blocks`` workgroups of four
// waves; returns the number of floating-point operations that is (2 * 16 * 16 * 32 an instruction), or 0.
extern "C" double lmsf_measure_mfma(void* sink, int iters, int blocks, hipStream_t stream) {
  if (!sink || iters <= 0 || blocks <= 0) {
    lmsf_set_error("measure_mfma: bad arguments");
    return 0.0;
  }
  hipLaunchKernelGGL(measure_mfma_kernel, dim3(blocks), dim3(256), 0, stream, (float*)sink, iters);
  if (hipGetLastError() != hipSuccess) {
    lmsf_set_error("measure_mfma: launch failed");
    return 0.0;
  }
  return (double)blocks * 4.0 * iters * 4.0 * 2.0 * 16 * 16 * 32;
}
