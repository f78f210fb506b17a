// Softmax over the last dimension, forward / backward, fp32 math:
//   y = softmax(x * multiplier);   d_x = multiplier * y * (d_y - sum_h(d_y * y)).
//
// A row is owned by TPR = 64 lanes (one wave) or 256 (the block). Rows of up to 4 chunks per lane stay in registers
// between the reductions and the write (x is read once); longer rows run the online form (running maximum and rescaled
// sum in one pass, second pass to write).
#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;

template <typename T, int P>
struct Vals {
  float f[P];
  __device__ static inline Vals load(const T* p, bool once) {
    Vals v;
    if constexpr (P == 1) {
      v.f[0] = Elem<T>::up(*p);
    } else {
      Pack16<T> k;
      k.v = once ? load16_nt(p) : load16(p);
#pragma unroll
      for (int i = 0; i < P; ++i) v.f[i] = Elem<T>::up(k.e[i]);
    }
    return v;
  }
  __device__ inline void store(T* p) const {
    if constexpr (P == 1) {
      *p = Elem<T>::down(f[0]);
    } else {
      Pack16<T> k;
#pragma unroll
      for (int i = 0; i < P; ++i) k.e[i] = Elem<T>::down(f[i]);
      store16_nt(p, k.v);
    }
  }
};

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

template <int TPR>
__device__ inline float row_sum(float v, float* scratch) {
  if constexpr (TPR == kWave) return wave_sum(v);
  return block_sum<kBlock>(v, scratch);
}
template <int TPR>
__device__ inline float row_max(float v, float* scratch) {
  v = wave_max(v);
  if constexpr (TPR == kWave) return v;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
#pragma unroll
  for (int i = 1; i < kBlock / kWave; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

constexpr float kNegInf = -__builtin_huge_valf();

// chunks: H / P. NC > 0 requires chunks <= NC * TPR.
template <typename T, int P, int TPR, int NC>
__global__ __launch_bounds__(kBlock) void softmax_fwd_kernel(const T* __restrict__ x, float multiplier, int64_t B, int H,
                                                              int chunks, T* __restrict__ out) {
  __shared__ float scratch[kBlock / kWave];
  constexpr int ROWS = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  // TPR == kBlock: all threads of the block share the row, so the trip count is block-uniform (the reductions synchronise)
  for (int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR; row < B; row += (int64_t)gridDim.x * ROWS) {
    const T* xr = x + row * H;
    T* yr = out + row * H;
    if constexpr (NC > 0) {
      Vals<T, P> v[NC];
      float m = kNegInf;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          v[c] = Vals<T, P>::load(xr + (int64_t)ch * P, true);
#pragma unroll
          for (int i = 0; i < P; ++i) {
            v[c].f[i] *= multiplier;
            m = fmaxf(m, v[c].f[i]);
          }
        }
      }
      m = row_max<TPR>(m, scratch);
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        if (c * TPR + lane < chunks) {
#pragma unroll
          for (int i = 0; i < P; ++i) {
            v[c].f[i] = expf(v[c].f[i] - m);
            s += v[c].f[i];
          }
        }
      }
      s = row_sum<TPR>(s, scratch);
      const float inv = 1.0f / s;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
#pragma unroll
          for (int i = 0; i < P; ++i) v[c].f[i] *= inv;
          v[c].store(yr + (int64_t)ch * P);
        }
      }
    } else {
      float m = kNegInf, s = 0.f;  // online: s is the sum of exp(x - m) for the running maximum m
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vals<T, P> v = Vals<T, P>::load(xr + (int64_t)ch * P, false);
        float cm = m;
#pragma unroll
        for (int i = 0; i < P; ++i) cm = fmaxf(cm, v.f[i] * multiplier);
        s *= expf(m - cm);  // exp(-inf - finite) = 0 on the first chunk
        m = cm;
#pragma unroll
        for (int i = 0; i < P; ++i) s += expf(v.f[i] * multiplier - m);
      }
      const float row_m = row_max<TPR>(m, scratch);
      s = row_sum<TPR>(m == kNegInf ? 0.f : s * expf(m - row_m), scratch);
      const float inv = 1.0f / s;
      for (int ch = lane; ch < chunks; ch += TPR) {
        Vals<T, P> v = Vals<T, P>::load(xr + (int64_t)ch * P, false);  // second read: L1 / L2
#pragma unroll
        for (int i = 0; i < P; ++i) v.f[i] = expf(v.f[i] * multiplier - row_m) * inv;
        v.store(yr + (int64_t)ch * P);
      }
    }
  }
}

template <typename T, int P, int TPR, int NC>
__global__ __launch_bounds__(kBlock) void softmax_bwd_kernel(const T* __restrict__ y, const T* __restrict__ d_y,
                                                              float multiplier, int64_t B, int H, int chunks,
                                                              T* __restrict__ d_x) {
  __shared__ float scratch[kBlock / kWave];
  constexpr int ROWS = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  for (int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR; row < B; row += (int64_t)gridDim.x * ROWS) {
    const T* yr = y + row * H;
    const T* gr = d_y + row * H;
    T* dxr = d_x + row * H;
    float dot = 0.f;
    if constexpr (NC > 0) {
      Vals<T, P> yv[NC], gv[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          yv[c] = Vals<T, P>::load(yr + (int64_t)ch * P, true);
          gv[c] = Vals<T, P>::load(gr + (int64_t)ch * P, true);
#pragma unroll
          for (int i = 0; i < P; ++i) dot += yv[c].f[i] * gv[c].f[i];
        }
      }
      dot = row_sum<TPR>(dot, scratch);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          Vals<T, P> o;
#pragma unroll
          for (int i = 0; i < P; ++i) o.f[i] = multiplier * yv[c].f[i] * (gv[c].f[i] - dot);
          o.store(dxr + (int64_t)ch * P);
        }
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vals<T, P> yv = Vals<T, P>::load(yr + (int64_t)ch * P, false);
        const Vals<T, P> gv = Vals<T, P>::load(gr + (int64_t)ch * P, false);
#pragma unroll
        for (int i = 0; i < P; ++i) dot += yv.f[i] * gv.f[i];
      }
      dot = row_sum<TPR>(dot, scratch);
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vals<T, P> yv = Vals<T, P>::load(yr + (int64_t)ch * P, false);
        const Vals<T, P> gv = Vals<T, P>::load(gr + (int64_t)ch * P, false);
        Vals<T, P> o;
#pragma unroll
        for (int i = 0; i < P; ++i) o.f[i] = multiplier * yv.f[i] * (gv.f[i] - dot);
        o.store(dxr + (int64_t)ch * P);
      }
    }
  }
}

struct Plan {
  int tpr, nc, P, chunks;
};
template <typename T>
Plan make_plan(int H, bool aligned) {
  Plan p;
  p.P = (aligned && H % Elem<T>::per16 == 0) ? Elem<T>::per16 : 1;
  p.chunks = H / p.P;
  p.tpr = p.chunks <= 2 * kWave ? kWave : kBlock;
  const int per_lane = (p.chunks + p.tpr - 1) / p.tpr;
  p.nc = per_lane <= 1 ? 1 : (per_lane <= 2 ? 2 : (per_lane <= 4 ? 4 : 0));
  return p;
}

}  // namespace
}  // namespace ck

using namespace ck;

#define CK_SM_DISPATCH(KERNEL)                                   \
  do {                                                           \
    if (plan.P == 1) {                                           \
      if (plan.tpr == kWave) {                                   \
        if (plan.nc == 1) KERNEL(1, kWave, 1);                   \
        else KERNEL(1, kWave, 2);                                \
      } else {                                                   \
        if (plan.nc == 4) KERNEL(1, kBlock, 4);                  \
        else if (plan.nc > 0) KERNEL(1, kBlock, 2);              \
        else KERNEL(1, kBlock, 0);                               \
      }                                                          \
    } else {                                                     \
      constexpr int PV = Elem<scalar_t>::per16;                  \
      if (plan.tpr == kWave) {                                   \
        if (plan.nc == 1) KERNEL(PV, kWave, 1);                  \
        else KERNEL(PV, kWave, 2);                               \
      } else {                                                   \
        if (plan.nc == 4) KERNEL(PV, kBlock, 4);                 \
        else if (plan.nc > 0) KERNEL(PV, kBlock, 2);             \
        else KERNEL(PV, kBlock, 0);                              \
      }                                                          \
    }                                                            \
  } while (0)

#define CK_SM_FWD(PP, TPR, NC)                                                                                     \
  hipLaunchKernelGGL((softmax_fwd_kernel<scalar_t, PP, TPR, NC>), dim3((unsigned)blocks), dim3(kBlock), 0, s,       \
                     static_cast<const scalar_t*>(x), multiplier, B, (int)H, plan.chunks, static_cast<scalar_t*>(out))
#define CK_SM_BWD(PP, TPR, NC)                                                                                     \
  hipLaunchKernelGGL((softmax_bwd_kernel<scalar_t, PP, TPR, NC>), dim3((unsigned)blocks), dim3(kBlock), 0, s,       \
                     static_cast<const scalar_t*>(y), static_cast<const scalar_t*>(d_y), multiplier, B, (int)H,     \
                     plan.chunks, static_cast<scalar_t*>(d_x))

extern "C" int ck_softmax_fwd(const void* x, float multiplier, int64_t B, int32_t H, void* out, int32_t dtype,
                              void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "ck_softmax_fwd: bad sizes B=%lld H=%d", (long long)B, H);
  if (B == 0) return CK_OK;
  CK_REQUIRE(x && out, "ck_softmax_fwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_softmax_fwd", {
    const Plan plan = make_plan<scalar_t>(H, aligned16(x) && aligned16(out));
    int64_t blocks = ceil_div(B, (int64_t)(kBlock / plan.tpr));
    if (blocks > 16384) blocks = 16384;
    CK_SM_DISPATCH(CK_SM_FWD);
  });
  CK_CHECK_LAUNCH("ck_softmax_fwd");
  return CK_OK;
}

extern "C" int ck_softmax_bwd(const void* y, const void* d_y, float multiplier, int64_t B, int32_t H, void* d_x,
                              int32_t dtype, void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "ck_softmax_bwd: bad sizes B=%lld H=%d", (long long)B, H);
  if (B == 0) return CK_OK;
  CK_REQUIRE(y && d_y && d_x, "ck_softmax_bwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_softmax_bwd", {
    const Plan plan = make_plan<scalar_t>(H, aligned16(y) && aligned16(d_y) && aligned16(d_x));
    int64_t blocks = ceil_div(B, (int64_t)(kBlock / plan.tpr));
    if (blocks > 16384) blocks = 16384;
    CK_SM_DISPATCH(CK_SM_BWD);
  });
  CK_CHECK_LAUNCH("ck_softmax_bwd");
  return CK_OK;
}
