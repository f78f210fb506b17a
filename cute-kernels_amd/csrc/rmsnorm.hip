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
  // for rows that are read exactly once (non-temporal)
  __device__ static inline Vec load_once(const T* p) {
    Vec v;
    if constexpr (P == 1) {
      v.f[0] = Elem<T>::up(*p);
    } else {
      Pack16<T> k;
      k.v = load16_nt(p);
#pragma unroll
      for (int i = 0; i < P; ++i) v.f[i] = Elem<T>::up(k.e[i]);
    }
    return v;
  }
  // a 16-byte chunk fetched earlier (P > 1)
  __device__ static inline Vec unpack(const vec16& raw) {
    Vec v;
    Pack16<T> k;
    k.v = raw;
#pragma unroll
    for (int i = 0; i < P; ++i) v.f[i] = Elem<T>::up(k.e[i]);
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
      store16_nt(p, k.v);
    }
  }
};

// Residual-add fusion (both optional, all-null = plain RMSNorm).
// forward: added = round(round(x * multiplier) + residual) is written out and normalised (multiplier == 1: no scaling);
// backward: d_added_total = d(norm input) + d_added; d_residual = d_added_total, d_x = d_added_total * multiplier.
template <typename T>
struct FwdFuse {
  const T* residual;
  T* added;
  float multiplier;
};
template <typename T>
struct BwdFuse {
  const T* d_added;
  T* d_residual;
  float multiplier;
};

template <typename T>
__device__ inline float round_to(float v) {
  return Elem<T>::up(Elem<T>::down(v));
}

template <int TPR>
__device__ inline float row_sum(float v, float* scratch) {
  if constexpr (TPR == kWave) return wave_sum(v);
  return block_sum<kBlock>(v, scratch);
}

// chunks: H / P. NC > 0 requires chunks <= NC * TPR.
template <typename T, int P, int TPR, int NC>
__global__ __launch_bounds__(kBlock) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                              float eps, int64_t B, int H, int chunks,
                                                              T* __restrict__ out, float* __restrict__ rstd_out,
                                                              const FwdFuse<T> fuse) {
  __shared__ float scratch[kBlock / kWave];
  constexpr int ROWS = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  const int64_t row_stride = (int64_t)gridDim.x * ROWS;
  const float inv_h = 1.0f / (float)H;
  // Cached rows in 16-byte chunks: the next row (and its residual row) is fetched, packed, before this row's reduction
  // and stores; a lane's weight chunks are the same in every row and are fetched once. Rows of four chunks per lane
  // would pay for the extra registers with occupancy (measured slower), so they load in place.
  constexpr bool kPrefetch = NC > 0 && NC <= 2 && P > 1;
  vec16 next_x[kPrefetch ? NC : 1], next_r[kPrefetch ? NC : 1], w_raw[kPrefetch ? NC : 1];
  auto fetch = [&](int64_t r) {
    if constexpr (kPrefetch) {
      if (r < B) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int ch = c * TPR + lane;
          if (ch < chunks) {
            next_x[c] = load16_nt(x + r * H + (int64_t)ch * P);
            if (fuse.residual != nullptr) next_r[c] = load16_nt(fuse.residual + r * H + (int64_t)ch * P);
          }
        }
      }
    }
  };
  if constexpr (kPrefetch) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int ch = c * TPR + lane;
      if (weight != nullptr && ch < chunks) w_raw[c] = load16(weight + (int64_t)ch * P);
    }
  }
  const int64_t first_row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;
  fetch(first_row);
  // TPR == kBlock: all threads of the block share the row, so the loop trip count is block-uniform (block_sum barriers)
  for (int64_t row = first_row; row < B; row += row_stride) {
    const T* xr = x + row * H;
    T* yr = out + row * H;
    const T* rr = fuse.residual ? fuse.residual + row * H : nullptr;
    T* ar = fuse.residual ? fuse.added + row * H : nullptr;
    // the row to normalise: x, or the freshly written sum with the residual stream
    auto add_residual = [&](Vec<T, P>& v, const Vec<T, P>& r, int ch) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        float t = v.f[i];
        if (fuse.multiplier != 1.0f) t = round_to<T>(__fmul_rn(t, fuse.multiplier));  // never contracted into an fma
        v.f[i] = round_to<T>(__fadd_rn(t, r.f[i]));
      }
      v.store(ar + (int64_t)ch * P);
    };
    auto load_x = [&](int ch) {
      // cached rows (NC > 0) are read once; streaming rows come back for the second pass
      Vec<T, P> v = NC > 0 ? Vec<T, P>::load_once(xr + (int64_t)ch * P) : Vec<T, P>::load(xr + (int64_t)ch * P);
      if (rr != nullptr) add_residual(v, Vec<T, P>::load_once(rr + (int64_t)ch * P), ch);
      return v;
    };
    float ss = 0.f;
    if constexpr (NC > 0) {
      Vec<T, P> xv[NC];
      if constexpr (kPrefetch) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int ch = c * TPR + lane;
          if (ch < chunks) {
            xv[c] = Vec<T, P>::unpack(next_x[c]);
            if (rr != nullptr) add_residual(xv[c], Vec<T, P>::unpack(next_r[c]), ch);
          }
        }
        fetch(row + row_stride);  // the packed registers are free again: the next row is in flight from here on
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          if (c * TPR + lane < chunks) {
#pragma unroll
            for (int i = 0; i < P; ++i) ss += xv[c].f[i] * xv[c].f[i];
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int ch = c * TPR + lane;
          if (ch < chunks) {
            xv[c] = load_x(ch);
#pragma unroll
            for (int i = 0; i < P; ++i) ss += xv[c].f[i] * xv[c].f[i];
          }
        }
      }
      ss = row_sum<TPR>(ss, scratch);
      const float rs = rsqrtf(ss * inv_h + eps);
      if (rstd_out != nullptr && lane == 0) rstd_out[row] = rs;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          Vec<T, P> wv;
          if constexpr (kPrefetch) wv = weight ? Vec<T, P>::unpack(w_raw[c]) : Vec<T, P>::ones();
          else wv = weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
          Vec<T, P> y;
#pragma unroll
          for (int i = 0; i < P; ++i) y.f[i] = xv[c].f[i] * rs * wv.f[i];
          y.store(yr + (int64_t)ch * P);
        }
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> v = load_x(ch);
#pragma unroll
        for (int i = 0; i < P; ++i) ss += v.f[i] * v.f[i];
      }
      ss = row_sum<TPR>(ss, scratch);
      const float rs = rsqrtf(ss * inv_h + eps);
      if (rstd_out != nullptr && lane == 0) rstd_out[row] = rs;
      const T* again = rr != nullptr ? ar : xr;  // this lane's own writes, or x (L1 / L2 serve the second read)
      for (int ch = lane; ch < chunks; ch += TPR) {
        const Vec<T, P> v = Vec<T, P>::load(again + (int64_t)ch * P);
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
                                                              T* __restrict__ d_x, float* __restrict__ partial,
                                                              const BwdFuse<T> fuse) {
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

  // Cached rows in 16-byte chunks: the next row's x and d_y are fetched (packed, 4 registers a chunk) before this row's
  // reductions and stores, so that a row owner always has a row of loads in flight.
  constexpr bool kPrefetch = NC > 0 && P > 1;
  vec16 next_x[kPrefetch ? NC : 1], next_g[kPrefetch ? NC : 1], w_raw[kPrefetch ? NC : 1];
  float next_rs = 0.f;
  if constexpr (kPrefetch) {  // a lane sees the same weight chunks in every row: fetched once (loads return in order, so
                              // a weight or rstd load issued behind the prefetch would wait for the whole next row)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int ch = c * TPR + lane;
      if (weight != nullptr && ch < chunks) w_raw[c] = load16(weight + (int64_t)ch * P);
    }
  }
  auto weight_chunk = [&](int c, int ch) {
    if constexpr (kPrefetch) return weight ? Vec<T, P>::unpack(w_raw[c]) : Vec<T, P>::ones();
    else return weight ? Vec<T, P>::load(weight + (int64_t)ch * P) : Vec<T, P>::ones();
  };
  auto fetch = [&](int64_t r) {
    if constexpr (kPrefetch) {
      if (r < B) {
        if (rstd != nullptr) next_rs = rstd[r];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int ch = c * TPR + lane;
          if (ch < chunks) {
            next_x[c] = load16_nt(x + r * H + (int64_t)ch * P);
            next_g[c] = load16_nt(d_out + r * H + (int64_t)ch * P);
          }
        }
      }
    }
  };
  fetch(worker);

  // with TPR == 64 the waves of a block may run different trip counts; nothing below synchronises the block then
  for (int64_t row = worker; row < B; row += row_stride) {
    const T* xr = x + row * H;
    const T* gr = d_out + row * H;
    T* dxr = d_x + row * H;
    // o = gradient w.r.t. the normalised row; with the fusion add the residual stream's gradient, emit both outputs
    auto finish = [&](Vec<T, P>& o, int ch) {
      if (fuse.d_added != nullptr) {
        const Vec<T, P> a = Vec<T, P>::load_once(fuse.d_added + row * H + (int64_t)ch * P);
#pragma unroll
        for (int i = 0; i < P; ++i) o.f[i] += a.f[i];
      }
      if (fuse.d_residual != nullptr) o.store(fuse.d_residual + row * H + (int64_t)ch * P);
      if (fuse.multiplier != 1.0f) {
#pragma unroll
        for (int i = 0; i < P; ++i) o.f[i] = round_to<T>(o.f[i]) * fuse.multiplier;
      }
      o.store(dxr + (int64_t)ch * P);
    };
    float dot = 0.f, ss = 0.f;
    if constexpr (kPrefetch) {
      // this row's chunks stay packed (4 registers each) and are unpacked in both passes: fewer live registers than
      // holding them as floats, which keeps four waves per SIMD next to the prefetched row
      vec16 cur_x[NC], cur_g[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        cur_x[c] = next_x[c];
        cur_g[c] = next_g[c];
      }
      const float saved_rs = next_rs;
      fetch(row + row_stride);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          const Vec<T, P> xv = Vec<T, P>::unpack(cur_x[c]), gv = Vec<T, P>::unpack(cur_g[c]), wv = weight_chunk(c, ch);
#pragma unroll
          for (int i = 0; i < P; ++i) {
            ss += xv.f[i] * xv.f[i];
            dot += gv.f[i] * wv.f[i] * xv.f[i];
          }
        }
      }
      dot = row_sum<TPR>(dot, scratch);
      float rs;
      if (rstd != nullptr) {
        rs = saved_rs;
      } else {
        ss = row_sum<TPR>(ss, scratch);
        rs = rsqrtf(ss * inv_h + eps);
      }
      const float coef = dot * rs * rs * rs * inv_h;
#pragma unroll
      for (int c = 0; c < NC; ++c) {  // the compiler must not carry the first pass's unpacked floats over the reductions
        asm volatile("" : "+v"(cur_x[c].w[0]), "+v"(cur_x[c].w[1]), "+v"(cur_x[c].w[2]), "+v"(cur_x[c].w[3]));
        asm volatile("" : "+v"(cur_g[c].w[0]), "+v"(cur_g[c].w[1]), "+v"(cur_g[c].w[2]), "+v"(cur_g[c].w[3]));
      }
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          const Vec<T, P> xv = Vec<T, P>::unpack(cur_x[c]), gv = Vec<T, P>::unpack(cur_g[c]), wv = weight_chunk(c, ch);
          Vec<T, P> o;
#pragma unroll
          for (int i = 0; i < P; ++i) {
            o.f[i] = rs * gv.f[i] * wv.f[i] - coef * xv.f[i];
            dw[c].f[i] += gv.f[i] * xv.f[i] * rs;
          }
          finish(o, ch);
        }
      }
    } else if constexpr (NC > 0) {
      Vec<T, P> xv[NC], gv[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          xv[c] = Vec<T, P>::load_once(xr + (int64_t)ch * P);
          gv[c] = Vec<T, P>::load_once(gr + (int64_t)ch * P);
          const Vec<T, P> wv = weight_chunk(c, ch);
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
          const Vec<T, P> wv = weight_chunk(c, ch);
          Vec<T, P> o;
#pragma unroll
          for (int i = 0; i < P; ++i) {
            o.f[i] = rs * gv[c].f[i] * wv.f[i] - coef * xv[c].f[i];
            dw[c].f[i] += gv[c].f[i] * xv[c].f[i] * rs;
          }
          finish(o, ch);
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
        finish(o, ch);
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

// d_weight[h] = sum over the partial rows, in a fixed order. A block owns 64 columns; its 16 waves each sum a sixteenth
// of the rows (256-byte coalesced reads, 8 independent partial sums so that 8 loads are in flight per wave), then the
// sixteen results are added through LDS.
constexpr int kReduceBlock = 1024, kReduceWaves = kReduceBlock / kWave, kReduceUnroll = 8;
__global__ __launch_bounds__(kReduceBlock) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int64_t workers,
                                                                          int H, float* __restrict__ d_weight) {
  __shared__ float part[kReduceWaves][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int h = blockIdx.x * kWave + lane;
  float s = 0.f;
  if (h < H) {
    float acc[kReduceUnroll];
#pragma unroll
    for (int u = 0; u < kReduceUnroll; ++u) acc[u] = 0.f;
    int64_t w = wave;
    for (; w + (kReduceUnroll - 1) * kReduceWaves < workers; w += kReduceUnroll * kReduceWaves) {
#pragma unroll
      for (int u = 0; u < kReduceUnroll; ++u) acc[u] += partial[(w + u * kReduceWaves) * H + h];
    }
    for (; w < workers; w += kReduceWaves) acc[0] += partial[w * H + h];
#pragma unroll
    for (int u = 0; u < kReduceUnroll; ++u) s += acc[u];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && h < H) {
    float t = 0.f;
#pragma unroll
    for (int g = 0; g < kReduceWaves; ++g) t += part[g][lane];
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

// CUs of the current device (256 on an MI355X), looked up once per device.
inline int compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// Persistent row owners of the backward kernel. One block per row (wide rows): a whole number of blocks per CU, fewer
// the wider the row -- measured at 65,536 rows, plain backward (2 streams in, 1 out), % of 8 TB/s at 1 / 2 / 3 / 4 blocks
// per CU: H = 2,048: 45 / 71 / 77 / 73; H = 4,096: 60 / 74 / 67 / 65; H = 8,192: 75 / 73 / 66 / 72; counts that are not a
// multiple of the CU count lose 5-10 points to the ragged last wave of blocks. With the residual fusion (3 streams in, 2
// out) the curve is flat (68-70 % at 2-4 per CU) and 3 / 4 per CU are kept.
// `added_only`: the residual stream's gradient comes in but one buffer takes both outputs (3 streams in, 1 out):
// 65,536 x 4,096 419 / 369 / 380 us at 2 / 3 / 4 per CU, 16,384 x 8,192 195 / 235 / 204.
inline int64_t workers_for(int64_t B, int tpr, int H, bool fused, bool added_only = false) {
  const int rows_per_block = kBlock / tpr;
  int64_t w = B < kMaxWorkers ? B : kMaxWorkers;
  if (tpr == kBlock) {
    const int per_cu = fused ? (H < 3072 ? 3 : 4) : added_only ? (H < 6144 ? 3 : 2) : (H < 3072 ? 3 : 2);
    const int64_t cap = (int64_t)per_cu * compute_units();
    if (w > cap) w = cap;
    if (w > kMaxWorkers / 2) w = kMaxWorkers / 2;
  }
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
                     plan.chunks, static_cast<scalar_t*>(out), rstd, fuse)

static int rmsnorm_fwd_impl(const char* name, const void* x, const void* residual, const void* weight, float eps,
                            float multiplier, int64_t B, int32_t H, void* out, void* added, float* rstd, int32_t dtype,
                            void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "%s: bad sizes B=%lld H=%d", name, (long long)B, H);
  if (B == 0) return CK_OK;
  CK_REQUIRE(x && out, "%s: NULL argument", name);
  CK_REQUIRE((residual == nullptr) == (added == nullptr), "%s: residual and added must be given together", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, name, {
    const bool aligned = aligned16(x) && aligned16(out) && (weight == nullptr || aligned16(weight)) &&
                         (residual == nullptr || (aligned16(residual) && aligned16(added)));
    const Plan plan = make_plan<scalar_t>(H, aligned);
    const int rows_per_block = kBlock / plan.tpr;
    int64_t blocks = ceil_div(B, rows_per_block);
    if (blocks > 8192) blocks = 8192;
    const FwdFuse<scalar_t> fuse = {static_cast<const scalar_t*>(residual), static_cast<scalar_t*>(added), multiplier};
    CK_RMS_DISPATCH(CK_RMS_FWD, 0);
  });
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int ck_rmsnorm_fwd(const void* x, const void* weight, float eps, int64_t B, int32_t H, void* out,
                              float* rstd, int32_t dtype, void* stream) {
  return rmsnorm_fwd_impl("ck_rmsnorm_fwd", x, nullptr, weight, eps, 1.0f, B, H, out, nullptr, rstd, dtype, stream);
}

extern "C" int ck_fused_residual_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, float eps,
                                                 float multiplier, int64_t B, int32_t H, void* out, void* added,
                                                 float* rstd, int32_t dtype, void* stream) {
  const char* name = "ck_fused_residual_add_rmsnorm_fwd";
  CK_REQUIRE(B == 0 || (residual && added), "%s: residual and added are required", name);
  return rmsnorm_fwd_impl(name, x, residual, weight, eps, multiplier, B, H, out, added, rstd, dtype, stream);
}

#define CK_RMS_BWD(PP, TPR, NC, dummy)                                                                              \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<scalar_t, PP, TPR, NC>), dim3((unsigned)blocks), dim3(kBlock), 0, s,        \
                     static_cast<const scalar_t*>(x), static_cast<const scalar_t*>(weight),                          \
                     static_cast<const scalar_t*>(d_out), rstd, eps, B, (int)H, plan.chunks,                         \
                     static_cast<scalar_t*>(d_x), d_weight_partial, fuse)

extern "C" int64_t ck_rmsnorm_bwd_partial_rows(int64_t B) {
  if (B <= 0) return 0;
  return round_up(B < kMaxWorkers ? B : kMaxWorkers, kBlock / kWave);
}

static int rmsnorm_bwd_impl(const char* name, const void* x, const void* weight, const void* d_out, const void* d_added,
                            const float* rstd, float eps, float multiplier, int64_t B, int32_t H, void* d_x,
                            void* d_residual, float* d_weight_partial, float* d_weight, int32_t dtype, void* stream) {
  CK_REQUIRE(B >= 0 && H >= 1, "%s: bad sizes B=%lld H=%d", name, (long long)B, H);
  CK_REQUIRE((weight == nullptr) == (d_weight == nullptr) && (weight == nullptr) == (d_weight_partial == nullptr),
             "%s: weight, d_weight and d_weight_partial must be given together", name);
  if (B == 0) {
    if (d_weight != nullptr) {  // no rows: the sum over zero partial rows is zero
      hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((unsigned)ceil_div(H, kWave)), dim3(kReduceBlock), 0,
                         static_cast<hipStream_t>(stream), d_weight_partial, (int64_t)0, (int)H, d_weight);
      CK_CHECK_LAUNCH(name);
    }
    return CK_OK;
  }
  CK_REQUIRE(x && d_out && d_x, "%s: NULL argument", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, name, {
    const bool aligned = aligned16(x) && aligned16(d_out) && aligned16(d_x) && (weight == nullptr || aligned16(weight)) &&
                         (d_added == nullptr || aligned16(d_added)) && (d_residual == nullptr || aligned16(d_residual));
    const Plan plan = make_plan<scalar_t>(H, aligned);
    const int rows_per_block = kBlock / plan.tpr;
    const int64_t workers = workers_for(B, plan.tpr, (int)H, d_residual != nullptr, d_added != nullptr);
    const int64_t blocks = workers / rows_per_block;
    const BwdFuse<scalar_t> fuse = {static_cast<const scalar_t*>(d_added), static_cast<scalar_t*>(d_residual), multiplier};
    CK_RMS_DISPATCH(CK_RMS_BWD, 0);
    if (d_weight != nullptr) {
      hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((unsigned)ceil_div(H, kWave)), dim3(kReduceBlock), 0, s,
                         d_weight_partial, workers, (int)H, d_weight);
    }
  });
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int ck_rmsnorm_bwd(const void* x, const void* weight, const void* d_out, const float* rstd, float eps,
                              int64_t B, int32_t H, void* d_x, float* d_weight_partial, float* d_weight, int32_t dtype,
                              void* stream) {
  return rmsnorm_bwd_impl("ck_rmsnorm_bwd", x, weight, d_out, nullptr, rstd, eps, 1.0f, B, H, d_x, nullptr,
                          d_weight_partial, d_weight, dtype, stream);
}

extern "C" int ck_fused_residual_add_rmsnorm_bwd(const void* added, const void* weight, const void* d_out,
                                                 const void* d_added, const float* rstd, float eps, float multiplier,
                                                 int64_t B, int32_t H, void* d_x, void* d_residual,
                                                 float* d_weight_partial, float* d_weight, int32_t dtype, void* stream) {
  const char* name = "ck_fused_residual_add_rmsnorm_bwd";
  CK_REQUIRE(B == 0 || d_residual != nullptr, "%s: d_residual is required", name);
  CK_REQUIRE(d_residual != d_x || multiplier == 1.0f, "%s: d_x and d_residual may be one buffer only when multiplier is 1", name);
  // multiplier == 1: both gradients are the same values; a caller that passes one buffer for both gets one store
  return rmsnorm_bwd_impl(name, added, weight, d_out, d_added, rstd, eps, multiplier, B, H, d_x,
                          d_residual == d_x ? nullptr : d_residual, d_weight_partial, d_weight, dtype, stream);
}
