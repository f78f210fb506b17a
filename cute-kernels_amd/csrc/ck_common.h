// Shared device/host helpers for libck_mi355.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "debug_options.h"
#include <stdio.h>

#include "ck_mi355.h"

namespace ck {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- error plumbing -------------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define CK_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      ::ck::set_error(__VA_ARGS__);      \
      return CK_ERR_ARG;                 \
    }                                    \
  } while (0)

#define CK_CHECK_LAUNCH(name)                                                      \
  do {                                                                             \
    hipError_t err__ = hipGetLastError();                                          \
    if (err__ != hipSuccess) {                                                     \
      ::ck::set_error("%s: launch failed: %s", name, hipGetErrorString(err__));    \
      return CK_ERR_LAUNCH;                                                        \
    }                                                                              \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- 16-bit float element types -------------------------------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

// 16 bytes moved as one 128-bit access.
struct __attribute__((aligned(16))) vec16 {
  uint32_t w[4];
};

template <typename T>
struct Elem;  // upcast / downcast through fp32, round-to-nearest-even

template <>
struct Elem<float> {
  static constexpr int per16 = 4;
  static constexpr int code = CK_F32;
  __device__ static inline float up(float v) { return v; }
  __device__ static inline float down(float v) { return v; }
};
template <>
struct Elem<bf16_t> {
  static constexpr int per16 = 8;
  static constexpr int code = CK_BF16;
  __device__ static inline float up(bf16_t v) { return static_cast<float>(v); }
  __device__ static inline bf16_t down(float v) { return static_cast<bf16_t>(v); }
};
template <>
struct Elem<f16_t> {
  static constexpr int per16 = 8;
  static constexpr int code = CK_F16;
  __device__ static inline float up(f16_t v) { return static_cast<float>(v); }
  __device__ static inline f16_t down(float v) { return static_cast<f16_t>(v); }
};

template <typename T>
union Pack16 {
  vec16 v;
  T e[Elem<T>::per16];
};

__device__ inline vec16 load16(const void* p) { return *reinterpret_cast<const vec16*>(p); }
__device__ inline void store16(void* p, const vec16& v) { *reinterpret_cast<vec16*>(p) = v; }
// Streaming variants for data that is touched once: non-temporal accesses do not displace reusable lines from the caches
// (measured on a 1 GiB read: 6.9 TB/s against 6.4 TB/s with plain loads).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline vec16 load16_nt(const void* p) {
  const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  vec16 v;
  v.w[0] = t.x;
  v.w[1] = t.y;
  v.w[2] = t.z;
  v.w[3] = t.w;
  return v;
}
__device__ inline void store16_nt(void* p, const vec16& v) {
  const u32x4_t t = {v.w[0], v.w[1], v.w[2], v.w[3]};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(p));
}
__device__ inline vec16 zero16() {
  vec16 z;
  z.w[0] = z.w[1] = z.w[2] = z.w[3] = 0u;
  return z;
}

// ---- wave / block reductions ----------------------------------------------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Sum over a block of NT threads (NT multiple of 64). `scratch` has NT/64 floats of LDS. All threads get the sum.
template <int NT>
__device__ inline float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  constexpr int NW = NT / kWave;
  if constexpr (NW == 1) return v;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();  // protect scratch reuse across calls
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += scratch[i];
  return t;
}

// sigmoid in fp32 with the exponent argument clamped like cute_kernels/include/activations.h:9-19
__device__ inline float sigmoid_f32(float x) {
  const float xc = fminf(fmaxf(x, -88.3762626647949f), 88.3762626647949f);
  return 1.0f / (1.0f + expf(-xc));
}
// same, on the hardware exp2 / reciprocal units (relative error ~1e-6): for results that are rounded to 16 bits anyway
__device__ inline float sigmoid_fast(float x) {
  const float xc = fminf(fmaxf(x, -88.3762626647949f), 88.3762626647949f);
  return __builtin_amdgcn_rcpf(1.0f + __expf(-xc));  // v_rcp_f32: 1 ulp, one instruction (a rounded division is ten)
}

// tanh-approximated GELU, 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3) (torch.nn.GELU("tanh"), the non-GLU
// activation of the reference's layer test, tests/test_commons.py:85-86), written as x * sigmoid(2u); and its derivative
// sigmoid(2u) + x * sigmoid(2u) (1 - sigmoid(2u)) * 2 du/dx
__device__ inline float gelu_tanh_fast(float x) {
  const float u2 = 1.5957691216057308f * (x + 0.044715f * x * x * x);
  return x * sigmoid_fast(u2);
}
__device__ inline float gelu_tanh_grad_fast(float x) {
  const float u2 = 1.5957691216057308f * (x + 0.044715f * x * x * x);
  const float s = sigmoid_fast(u2);
  return s + x * s * (1.f - s) * 1.5957691216057308f * (1.f + 0.134145f * x * x);
}

// fp32 tensors get the accurate form, 16-bit tensors the fast one
template <typename T>
__device__ inline float sigmoid_for(float x) {
  if constexpr (sizeof(T) == 4) return sigmoid_f32(x);
  else return sigmoid_fast(x);
}

#define CK_DISPATCH_FLOAT(dtype, NAME, ...)                       \
  switch (dtype) {                                                \
    case CK_F32: {                                                \
      using scalar_t = float;                                     \
      __VA_ARGS__;                                                \
    } break;                                                      \
    case CK_F16: {                                                \
      using scalar_t = ::ck::f16_t;                               \
      __VA_ARGS__;                                                \
    } break;                                                      \
    case CK_BF16: {                                               \
      using scalar_t = ::ck::bf16_t;                              \
      __VA_ARGS__;                                                \
    } break;                                                      \
    default:                                                      \
      ::ck::set_error("%s: unsupported dtype code %d", NAME, (int)(dtype)); \
      return CK_ERR_ARG;                                          \
  }

#define CK_DISPATCH_HALF(dtype, NAME, ...)                        \
  switch (dtype) {                                                \
    case CK_F16: {                                                \
      using scalar_t = ::ck::f16_t;                               \
      __VA_ARGS__;                                                \
    } break;                                                      \
    case CK_BF16: {                                               \
      using scalar_t = ::ck::bf16_t;                              \
      __VA_ARGS__;                                                \
    } break;                                                      \
    default:                                                      \
      ::ck::set_error("%s: only f16 / bf16 are supported (dtype code %d)", NAME, (int)(dtype)); \
      return CK_ERR_ARG;                                          \
  }

}  // namespace ck
