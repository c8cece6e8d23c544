// Shared helpers of the gfx950 kernel library: element types, reductions over a
// 64-wide wavefront, error reporting to the Python side.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define TK_WAVE 64

enum TkDtype { TK_F32 = 0, TK_BF16 = 1 };

typedef __hip_bfloat16 bf16_t;

// Entry points are the only symbols a library exports.
#define TK_API extern "C" __attribute__((visibility("default")))

// Every entry point returns 0 or a negative code; the text is read with tk_last_error().
void tk_set_error(const char* fmt, ...);

#define TK_REQUIRE(cond, ...)        \
  do {                               \
    if (!(cond)) {                   \
      tk_set_error(__VA_ARGS__);     \
      return -1;                     \
    }                                \
  } while (0)

#define TK_CHECK_LAUNCH(name)                                                \
  do {                                                                       \
    hipError_t e__ = hipGetLastError();                                      \
    if (e__ != hipSuccess) {                                                 \
      tk_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));   \
      return -2;                                                             \
    }                                                                        \
  } while (0)

// Layout of a page of the cache (P tokens of one kv head, head size d), chosen so that
// the lanes of a wavefront that feed the matrix cores read consecutive memory:
//   keys   [d / 8][P][8]   the 8-element pieces of the P keys, piece by piece
//   values [P / 4][d][4]   groups of 4 tokens, for each the d rows of 4 values
// A page of kv head h of page `page` starts at ((page * nkv + h) * P * d).
#define TK_KEY_PIECE 8
#define TK_VALUE_QUAD 4
__host__ __device__ __forceinline__ size_t key_offset(int P, int in_page, int e) {
  return ((size_t)(e / TK_KEY_PIECE) * P + in_page) * TK_KEY_PIECE + (e % TK_KEY_PIECE);
}
__host__ __device__ __forceinline__ size_t value_offset(int d, int in_page, int e) {
  return ((size_t)(in_page / TK_VALUE_QUAD) * d + e) * TK_VALUE_QUAD + (in_page % TK_VALUE_QUAD);
}

// One rotation of a pair by (cos, sin) in 32-bit, written out in fused multiply-adds so that
// every kernel that rotates gets the same bits whatever the compiler would contract.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float& o1, float& o2) {
  o1 = __fmaf_rn(x1, c, -__fmul_rn(x2, s));
  o2 = __fmaf_rn(x2, c, __fmul_rn(x1, s));
}

template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return __bfloat162float(v); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return __float2bfloat16(v); }

// Round a 32-bit value to the storage type and back: the place where the
// reference's tensors are materialised in the engine dtype.
template <typename T>
__device__ __forceinline__ float round_to(float v) { return to_f32<T>(from_f32<T>(v)); }

// silu(gate) * up as the engine's storage type sees it: both operands and the activation
// rounded to bfloat16, the product left in 32-bit for the caller to round.
__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
  const float gr = round_to<bf16_t>(g), ur = round_to<bf16_t>(u);
  const float s = round_to<bf16_t>(gr / (1.0f + expf(-gr)));
  return s * ur;
}

// Accesses that are coherent across the chip's dies (each has an L2 of its own): relaxed
// atomics of agent scope, which the compiler turns into loads that go around, and stores that
// write through, the caches.  Data that one workgroup of a running kernel writes and another
// reads moves through these; no cache-wide write-back or invalidation is needed then.
__device__ __forceinline__ uint64_t shared_load64(const void* p) {
  return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void shared_store64(void* p, uint64_t v) {
  __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void shared_store16(void* p, uint16_t v) {
  __hip_atomic_store((uint16_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = TK_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TK_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = TK_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TK_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS; the order of the additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const int wave = threadIdx.x / TK_WAVE;
  const int nwaves = (blockDim.x + TK_WAVE - 1) / TK_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const int wave = threadIdx.x / TK_WAVE;
  const int nwaves = (blockDim.x + TK_WAVE - 1) / TK_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}
