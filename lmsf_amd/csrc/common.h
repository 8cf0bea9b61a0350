// Shared helpers of the gfx950 kernels: element types, wave64 reductions, argument checks.
//
// Every entry point is extern "C", takes raw device pointers and a hipStream_t, validates
// its arguments on the host before it launches anything, and returns 0 on success. On failure
// it returns non-zero and lmsf_last_error() gives the reason; nothing is launched then.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define LMSF_WAVE 64

// dtype codes shared with the Python side
enum { LMSF_F32 = 0, LMSF_BF16 = 1 };

typedef uint16_t bf16_t;  // raw bfloat16 bits

// operand and accumulator registers of the bfloat16 matrix-core instructions
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

void lmsf_set_error(const char* fmt, ...);
int lmsf_compute_units();   // of the current device

#define LMSF_CHECK(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      lmsf_set_error(__VA_ARGS__);       \
      return 1;                          \
    }                                    \
  } while (0)

#define LMSF_LAUNCH_CHECK(name)                                             \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      lmsf_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                             \
    }                                                                       \
  } while (0)

// ---------------------------------------------------------------- element conversion

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return *reinterpret_cast<const bf16_t*>(&b);
}
// two values in one register, a in the low half
typedef __bf16 lmsf_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float lmsf_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  const lmsf_f32x2_t v = {a, b};
  const lmsf_bf16x2_t r = __builtin_convertvector(v, lmsf_bf16x2_t);
  return *reinterpret_cast<const uint32_t*>(&r);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// A bfloat16 product [M, N] left as float32 partial sums over parts of K: element (m, n) is the sum over
// s = 0 .. n_split-1, in that order, of part[(s * M + m) * N + n], plus bias[n] (bias may be null), rounded
// to bfloat16: the value that the reduction kernel of the product would have stored. Kernels that take one
// do that reduction while they load their operand. N is a multiple of 4 and part is 16-byte aligned.
struct LmsfPartialSum {
  const float* part;
  const bf16_t* bias;
  int n_split, M, N;
};
__device__ __forceinline__ float partial_sum_value(const LmsfPartialSum& p, int m, int n) {
  float s = 0.f;
  for (int i = 0; i < p.n_split; ++i) s += p.part[((long)i * p.M + m) * p.N + n];
  if (p.bias) s += bf16_to_f32(p.bias[n]);
  return bf16_to_f32(f32_to_bf16(s));
}
// four neighbours (n a multiple of 4)
__device__ __forceinline__ void partial_sum_value4(const LmsfPartialSum& p, int m, int n, float* x) {
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int i = 0; i < p.n_split; ++i) {
    const float4 v = *reinterpret_cast<const float4*>(p.part + ((long)i * p.M + m) * p.N + n);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  x[0] = s.x; x[1] = s.y; x[2] = s.z; x[3] = s.w;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (p.bias) x[e] += bf16_to_f32(p.bias[n + e]);
    x[e] = bf16_to_f32(f32_to_bf16(x[e]));
  }
}

// What a fused QKV product needs for its rotary-embedding-and-cache-write epilogue beside its own arguments.
struct RopeCacheArgs {
  const int* positions;    // [M]
  const float* table;      // [max_pos, d] = [cos(d/2) | sin(d/2)]
  const int* slots;        // [M]: page * page_size + offset of the token in the cache, negative: not stored
  bf16_t* k_pages;         // [pages, nkv, page_size, d]
  bf16_t* v_pages;         // [pages, nkv, d, page_size]
  int nh, nkv, d, ps;
};

// 16-byte vectors: 4 floats or 8 bfloat16
template <typename T> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  float4 v;
  __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
  __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
  __device__ __forceinline__ float raw(int i) const { return get(i); }   // element i as stored
  __device__ __forceinline__ void set(int i, float f) {
    if (i == 0) v.x = f; else if (i == 1) v.y = f; else if (i == 2) v.z = f; else v.w = f;
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  __device__ __forceinline__ void load(const bf16_t* p) { v = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void store(bf16_t* p) const { *reinterpret_cast<uint4*>(p) = v; }
  __device__ __forceinline__ float get(int i) const {
    uint32_t w = (i >> 1) == 0 ? v.x : (i >> 1) == 1 ? v.y : (i >> 1) == 2 ? v.z : v.w;
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  __device__ __forceinline__ bf16_t raw(int i) const {                    // element i as stored
    uint32_t w = (i >> 1) == 0 ? v.x : (i >> 1) == 1 ? v.y : (i >> 1) == 2 ? v.z : v.w;
    return (bf16_t)((i & 1) ? (w >> 16) : (w & 0xffffu));
  }
  __device__ __forceinline__ void set(int i, float f) {
    uint32_t b = f32_to_bf16(f);
    uint32_t* w = (i >> 1) == 0 ? &v.x : (i >> 1) == 1 ? &v.y : (i >> 1) == 2 ? &v.z : &v.w;
    *w = (i & 1) ? ((*w & 0x0000ffffu) | (b << 16)) : ((*w & 0xffff0000u) | b);
  }
};

// One rotation pair of the rotary embedding, x' = x cos - y sin, y' = y cos + x sin, with the roundings
// pinned (a product, then one fused multiply-add), so that every kernel that rotates gives the same bits.
__device__ __forceinline__ void rope_rotate(float x, float y, float c, float s, float* xr, float* yr) {
  *xr = __fmaf_rn(x, c, -__fmul_rn(y, s));
  *yr = __fmaf_rn(y, c, __fmul_rn(x, s));
}

// ---------------------------------------------------------------- wave64 and block reductions

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LMSF_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LMSF_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads (a multiple of 64); every thread gets the result.
// ``red`` is LDS scratch of at least 16 floats. Safe to call repeatedly with the same scratch.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int nw = (blockDim.x + LMSF_WAVE - 1) / LMSF_WAVE;
  if (nw == 1) return v;
  const int w = threadIdx.x / LMSF_WAVE, l = threadIdx.x % LMSF_WAVE;
  __syncthreads();
  if (l == 0) red[w] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int nw = (blockDim.x + LMSF_WAVE - 1) / LMSF_WAVE;
  if (nw == 1) return v;
  const int w = threadIdx.x / LMSF_WAVE, l = threadIdx.x % LMSF_WAVE;
  __syncthreads();
  if (l == 0) red[w] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
  return r;
}

static inline bool lmsf_aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }
static inline int lmsf_elem_size(int dtype) { return dtype == LMSF_F32 ? 4 : 2; }
