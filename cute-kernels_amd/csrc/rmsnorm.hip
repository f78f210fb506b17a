// RMSNorm forward / backward. fp32 math; y = x * rstd * w is rounded once (F.rms_norm numerics).
//
// A row is owned by TPR = 64 (one wave) or 256 (one block) lanes, each lane on consecutive 16-byte chunks; rows whose
// chunks fit NC per lane stay in registers between the reduction and the write (NC = 0: re-read, served by L1/L2).
// Backward is persistent: every row owner walks a strided set of rows and keeps its share of d_weight in registers,
// then writes one fp32 partial row; a second small kernel sums the partial rows in a fixed order (no float atomics).
#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;

template <typename T, int P>
struct Vec {
  float f[P];
  __device__ static inline Vec load(const T* p) {
    Vec v;
    if constexpr (P == 1) {
      v.f[0] = Elem<T>::up(*p);
    } else {
      Pack16<T> k;
      k.v = load16(p);
#pragma unroll
      for (int i = 0; i < P; ++i) v.f[i] = Elem<T>::up(k.e[i]);
    }
    return v;
  }
  __device__ static inline Vec ones() {
    Vec v;
#pragma unroll
    for (int i = 0; i < P; ++i) v.f[i] = 1.0f;
    return v;
  }
  __device__ inline void store(T* p) const {
    if constexpr (P == 1) {
      *p = Elem<T>::down(f[0]);
    } else {
      Pack16<T> k;
#pragma unroll
      for (int i = 0; i < P; ++i) k.e[i] = Elem<T>::down(f[i]);
      store16(p, k.v);
    }
  }
};

template <int TPR>
__device__ inline float row_sum(float v, float* scratch) {
  if constexpr (TPR == kWave) return wave_sum(v);
  return block_sum<kBlock>(v, scratch);
}

// chunks: H / P. NC > 0 requires chunks <= NC * TPR.
template <typename T, int P, int TPR, int NC>
__global__ __launch_bounds__(kBlock) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                              float eps, int64_t B, int H, int chunks,
                                                              T* __restrict__ out, float* __restrict__ rstd_out) {
  __shared__ float scratch[kBlock / kWave];
  constexpr int ROWS = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  const int64_t row_stride = (int64_t)gridDim.x * ROWS;
  const float inv_h = 1.0f / (float)H;
  // TPR == kBlock: all threads of the block share the row, so the loop trip count is block-uniform (block_sum barriers)
  for (int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR; row < B; row += row_stride) {
    const T* xr = x + row * H;
    T* yr = out + row * H;
    float ss = 0.f;
    if constexpr (NC > 0) {
      Vec<T, P> xv[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          xv[c] = Vec<T, P>::load(xr + (int64_t)ch * P);
#pragma unroll
          for (int i = 0; i < P; ++i) ss += xv[c].f[i] * xv[c].f[i];
        }
      }
      ss = row_sum<TPR>(ss, scratch);
      const float rs = rsqrtf(ss * inv_h + eps);
      if (rstd_out != nullptr && lane == 0) rstd_out[row] = rs;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
          Vec<T, P> y;
#pragma unroll
          for (int i = 0; i < P; ++i) y.f[i] = xv[c].f[i] * rs * wv.f[i];
          y.store(yr + (int64_t)ch * P);
        }
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> v = Vec<T, P>::load(xr + (int64_t)ch * P);
#pragma unroll
        for (int i = 0; i < P; ++i) ss += v.f[i] * v.f[i];
      }
      ss = row_sum<TPR>(ss, scratch);
      const float rs = rsqrtf(ss * inv_h + eps);
      if (rstd_out != nullptr && lane == 0) rstd_out[row] = rs;
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> v = Vec<T, P>::load(xr + (int64_t)ch * P);
        const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
        Vec<T, P> y;
#pragma unroll
        for (int i = 0; i < P; ++i) y.f[i] = v.f[i] * rs * wv.f[i];
        y.store(yr + (int64_t)ch * P);
      }
    }
  }
}

// d_x = rstd * (d_y * w) - x * rstd^3 / H * sum_h(d_y * w * x);  d_w[h] = sum_rows d_y * x * rstd.
// partial: [workers, H] fp32; worker = row owner index. NC == 0 accumulates d_w straight into its partial row.
template <typename T, int P, int TPR, int NC>
__global__ __launch_bounds__(kBlock) void rmsnorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                              const T* __restrict__ d_out, const float* __restrict__ rstd,
                                                              float eps, int64_t B, int H, int chunks,
                                                              T* __restrict__ d_x, float* __restrict__ partial) {
  __shared__ float scratch[kBlock / kWave];
  constexpr int ROWS = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  const int64_t worker = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;
  const int64_t row_stride = (int64_t)gridDim.x * ROWS;
  const float inv_h = 1.0f / (float)H;
  float* my_partial = partial ? partial + worker * H : nullptr;

  Vec<T, P> dw[NC > 0 ? NC : 1];
#pragma unroll
  for (int c = 0; c < (NC > 0 ? NC : 1); ++c)
#pragma unroll
    for (int i = 0; i < P; ++i) dw[c].f[i] = 0.f;
  if constexpr (NC == 0) {
    if (my_partial != nullptr) {  // same lane -> element mapping as the accumulation below
      for (int ch = lane; ch < chunks; ch += TPR)
#pragma unroll
        for (int i = 0; i < P; ++i) my_partial[(int64_t)ch * P + i] = 0.f;
    }
  }

  // with TPR == 64 the waves of a block may run different trip counts; nothing below synchronises the block then
  for (int64_t row = worker; row < B; row += row_stride) {
    const T* xr = x + row * H;
    const T* gr = d_out + row * H;
    T* dxr = d_x + row * H;
    float dot = 0.f, ss = 0.f;
    if constexpr (NC > 0) {
      Vec<T, P> xv[NC], gv[NC];  // gv holds d_y * w
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          xv[c] = Vec<T, P>::load(xr + (int64_t)ch * P);
          gv[c] = Vec<T, P>::load(gr + (int64_t)ch * P);
          const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
#pragma unroll
          for (int i = 0; i < P; ++i) {
            ss += xv[c].f[i] * xv[c].f[i];
            dot += gv[c].f[i] * wv.f[i] * xv[c].f[i];
          }
        }
      }
      dot = row_sum<TPR>(dot, scratch);
      float rs;
      if (rstd != nullptr) {
        rs = rstd[row];
      } else {
        ss = row_sum<TPR>(ss, scratch);
        rs = rsqrtf(ss * inv_h + eps);
      }
      const float coef = dot * rs * rs * rs * inv_h;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
          Vec<T, P> o;
#pragma unroll
          for (int i = 0; i < P; ++i) {
            o.f[i] = rs * gv[c].f[i] * wv.f[i] - coef * xv[c].f[i];
            dw[c].f[i] += gv[c].f[i] * xv[c].f[i] * rs;
          }
          o.store(dxr + (int64_t)ch * P);
        }
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> xv = Vec<T, P>::load(xr + (int64_t)ch * P);
        const Vec<T, P> gv = Vec<T, P>::load(gr + (int64_t)ch * P);
        const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
#pragma unroll
        for (int i = 0; i < P; ++i) {
          ss += xv.f[i] * xv.f[i];
          dot += gv.f[i] * wv.f[i] * xv.f[i];
        }
      }
      dot = row_sum<TPR>(dot, scratch);
      float rs;
      if (rstd != nullptr) {
        rs = rstd[row];
      } else {
        ss = row_sum<TPR>(ss, scratch);
        rs = rsqrtf(ss * inv_h + eps);
      }
      const float coef = dot * rs * rs * rs * inv_h;
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> xv = Vec<T, P>::load(xr + (int64_t)ch * P);
        const Vec<T, P> gv = Vec<T, P>::load(gr + (int64_t)ch * P);
        const Vec<T, P> wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
        Vec<T, P> o;
#pragma unroll
        for (int i = 0; i < P; ++i) {
          o.f[i] = rs * gv.f[i] * wv.f[i] - coef * xv.f[i];
          if (my_partial != nullptr) my_partial[(int64_t)ch * P + i] += gv.f[i] * xv.f[i] * rs;  // lane-private slots
        }
        o.store(dxr + (int64_t)ch * P);
      }
    }
  }
  if constexpr (NC > 0) {
    if (my_partial != nullptr) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
#pragma unroll
          for (int i = 0; i < P; ++i) my_partial[(int64_t)ch * P + i] = dw[c].f[i];
        }
      }
    }
  }
}

// d_weight[h] = sum over the partial rows, in a fixed order. A block owns 64 columns; its 4 waves each sum a quarter of
// the rows (reads are 256-byte coalesced), then the quarters are added through LDS.
__global__ __launch_bounds__(kBlock) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int64_t workers,
                                                                    int H, float* __restrict__ d_weight) {
  __shared__ float part[kBlock / kWave][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int h = blockIdx.x * kWave + lane;
  float s = 0.f;
  if (h < H) {
    for (int64_t w = wave; w < workers; w += kBlock / kWave) s += partial[w * H + h];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && h < H) {
    float t = 0.f;
#pragma unroll
    for (int g = 0; g < kBlock / kWave; ++g) t += part[g][lane];
    d_weight[h] = t;
  }
}

constexpr int64_t kMaxWorkers = 2048;

struct Plan {
  int tpr;      // lanes per row
  int nc;       // chunks cached per lane (0 = streaming)
  int P;        // elements per access
  int chunks;
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

inline int64_t workers_for(int64_t B, int tpr) {
  const int rows_per_block = kBlock / tpr;
  int64_t w = B < kMaxWorkers ? B : kMaxWorkers;
  if (tpr == kBlock && w > kMaxWorkers / 2) w = kMaxWorkers / 2;
  return round_up(w, rows_per_block);
}

}  // namespace
}  // namespace ck

using namespace ck;

#define CK_RMS_DISPATCH(KERNEL, ...)                                                          \
  do {                                                                                        \
    if (plan.P == 1) {                                                                        \
      if (plan.tpr == kWave) {                                                                \
        if (plan.nc == 1) KERNEL(1, kWave, 1, __VA_ARGS__);                                   \
        else if (plan.nc == 2) KERNEL(1, kWave, 2, __VA_ARGS__);                              \
        else KERNEL(1, kWave, 0, __VA_ARGS__);                                                \
      } else {                                                                                \
        KERNEL(1, kBlock, 0, __VA_ARGS__);                                                    \
      }                                                                                       \
    } else {                                                                                  \
      constexpr int PV = Elem<scalar_t>::per16;                                               \
      if (plan.tpr == kWave) {                                                                \
        if (plan.nc == 1) KERNEL(PV, kWave, 1, __VA_ARGS__);                                  \
        else KERNEL(PV, kWave, 2, __VA_ARGS__);                                               \
      } else {                                                                                \
        if (plan.nc == 1) KERNEL(PV, kBlock, 1, __VA_ARGS__);                                 \
        else if (plan.nc == 2) KERNEL(PV, kBlock, 2, __VA_ARGS__);                            \
        else if (plan.nc == 4) KERNEL(PV, kBlock, 4, __VA_ARGS__);                            \
        else KERNEL(PV, kBlock, 0, __VA_ARGS__);                                              \
      }                                                                                       \
    }                                                                                         \
  } while (0)

#define CK_RMS_FWD(PP, TPR, NC, dummy)                                                                              \
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<scalar_t, PP, TPR, NC>), dim3((unsigned)blocks), dim3(kBlock), 0, s,        \
                     static_cast<const scalar_t*>(x), static_cast<const scalar_t*>(weight), eps, B, (int)H,          \
                     plan.chunks, static_cast<scalar_t*>(out), rstd)

extern "C" int ck_rmsnorm_fwd(const void* x, const void* weight, float eps, int64_t B, int32_t H, void* out,
                              float* rstd, int32_t dtype, void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "ck_rmsnorm_fwd: bad sizes B=%lld H=%d", (long long)B, H);
  if (B == 0) return CK_OK;
  CK_REQUIRE(x && out, "ck_rmsnorm_fwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_rmsnorm_fwd", {
    const bool aligned = aligned16(x) && aligned16(out) && (weight == nullptr || aligned16(weight));
    const Plan plan = make_plan<scalar_t>(H, aligned);
    const int rows_per_block = kBlock / plan.tpr;
    int64_t blocks = ceil_div(B, rows_per_block);
    if (blocks > 8192) blocks = 8192;
    CK_RMS_DISPATCH(CK_RMS_FWD, 0);
  });
  CK_CHECK_LAUNCH("ck_rmsnorm_fwd");
  return CK_OK;
}

#define CK_RMS_BWD(PP, TPR, NC, dummy)                                                                              \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<scalar_t, PP, TPR, NC>), dim3((unsigned)blocks), dim3(kBlock), 0, s,        \
                     static_cast<const scalar_t*>(x), static_cast<const scalar_t*>(weight),                          \
                     static_cast<const scalar_t*>(d_out), rstd, eps, B, (int)H, plan.chunks,                         \
                     static_cast<scalar_t*>(d_x), d_weight_partial)

extern "C" int64_t ck_rmsnorm_bwd_partial_rows(int64_t B) {
  if (B <= 0) return 0;
  return round_up(B < kMaxWorkers ? B : kMaxWorkers, kBlock / kWave);
}

extern "C" int ck_rmsnorm_bwd(const void* x, const void* weight, const void* d_out, const float* rstd, float eps,
                              int64_t B, int32_t H, void* d_x, float* d_weight_partial, float* d_weight, int32_t dtype,
                              void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "ck_rmsnorm_bwd: bad sizes B=%lld H=%d", (long long)B, H);
  CK_REQUIRE((weight == nullptr) == (d_weight == nullptr) && (weight == nullptr) == (d_weight_partial == nullptr),
             "ck_rmsnorm_bwd: weight, d_weight and d_weight_partial must be given together");
  if (B == 0) {
    if (d_weight != nullptr) {  // no rows: the sum over zero partial rows is zero
      hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((unsigned)ceil_div(H, kWave)), dim3(kBlock), 0,
                         static_cast<hipStream_t>(stream), d_weight_partial, (int64_t)0, (int)H, d_weight);
      CK_CHECK_LAUNCH("ck_rmsnorm_bwd");
    }
    return CK_OK;
  }
  CK_REQUIRE(x && d_out && d_x, "ck_rmsnorm_bwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_rmsnorm_bwd", {
    const bool aligned = aligned16(x) && aligned16(d_out) && aligned16(d_x) && (weight == nullptr || aligned16(weight));
    const Plan plan = make_plan<scalar_t>(H, aligned);
    const int rows_per_block = kBlock / plan.tpr;
    const int64_t workers = workers_for(B, plan.tpr);
    const int64_t blocks = workers / rows_per_block;
    CK_RMS_DISPATCH(CK_RMS_BWD, 0);
    if (d_weight != nullptr) {
      hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((unsigned)ceil_div(H, kWave)), dim3(kBlock), 0, s,
                         d_weight_partial, workers, (int)H, d_weight);
    }
  });
  CK_CHECK_LAUNCH("ck_rmsnorm_bwd");
  return CK_OK;
}
