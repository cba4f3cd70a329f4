// Device helpers shared by the kernel files of layer-list models: the bfloat16 storage type and its
// conversions, wave and block reductions on 64-lane waves, dot products of two rows over a wave, and the
// host-side launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdexcept>
#include <string>

#include "../kernels/wave_shuffle.h"

namespace omx {
namespace stack {

struct bf16 {
  uint16_t v;
};
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
// round to nearest even, as torch's float -> bfloat16 conversion
__device__ __forceinline__ uint16_t f2bf(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16* p) { return bf2f(p->v); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16* p, float v) { p->v = f2bf(v); }

// butterfly reductions on DPP / permlane exchanges (wave_shuffle.h): no LDS round trip per dependent step
__device__ __forceinline__ float wave_sum(float v) {
  v += xor_shfl<32>(v);
  v += xor_shfl<16>(v);
  v += xor_shfl<8>(v);
  v += xor_shfl<4>(v);
  v += xor_shfl<2>(v);
  v += xor_shfl<1>(v);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, xor_shfl<32>(v));
  v = fmaxf(v, xor_shfl<16>(v));
  v = fmaxf(v, xor_shfl<8>(v));
  v = fmaxf(v, xor_shfl<4>(v));
  v = fmaxf(v, xor_shfl<2>(v));
  v = fmaxf(v, xor_shfl<1>(v));
  return v;
}
// sum over a block of 256 threads; every thread gets the result. red: 4 floats of LDS
__device__ __forceinline__ float block_sum256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}
__device__ __forceinline__ float silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + expf(-z)); }

static inline void check(bool ok, const char* what) {
  if (!ok) throw std::runtime_error(std::string("stack kernels: ") + what);
}
static inline void launched(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) throw std::runtime_error(std::string("stack kernels: ") + what + ": " + hipGetErrorString(e));
}

// ------------------------------------------------------------------------------------------------
// dot product of two rows over a wave: 16-byte loads when both rows allow it
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ w, const T* __restrict__ x, int K, int lane, bool vec);
template <>
__device__ __forceinline__ float wave_dot<bf16>(const bf16* __restrict__ w, const bf16* __restrict__ x, int K, int lane,
                                                bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int k = lane * 8; k < K; k += 512) {
      const u32x4 a = *(const u32x4*)(w + k), b = *(const u32x4*)(x + k);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc += __uint_as_float(a[i] << 16) * __uint_as_float(b[i] << 16);
        acc += __uint_as_float(a[i] & 0xffff0000u) * __uint_as_float(b[i] & 0xffff0000u);
      }
    }
  } else {
    for (int k = lane; k < K; k += 64) acc += ld(w + k) * ld(x + k);
  }
  return wave_sum(acc);
}
template <>
__device__ __forceinline__ float wave_dot<float>(const float* __restrict__ w, const float* __restrict__ x, int K, int lane,
                                                 bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int k = lane * 4; k < K; k += 256) {
      const f32x4 a = *(const f32x4*)(w + k), b = *(const f32x4*)(x + k);
      acc += a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
  } else {
    for (int k = lane; k < K; k += 64) acc += w[k] * x[k];
  }
  return wave_sum(acc);
}
template <typename T>
static inline bool vec_ok(const void* p, long long ld_elems, int K) {
  const int per = 16 / (int)sizeof(T);
  return K % per == 0 && ld_elems % per == 0 && ((uintptr_t)p & 15) == 0;
}


}  // namespace stack
}  // namespace omx
