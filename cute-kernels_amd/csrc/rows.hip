// Token-row movement: gather, gated combine (+ d_gates), padded grouped copy with transpose, batched transpose.
// All of it is HBM-bound byte shuffling: 128-bit accesses, consecutive lanes on consecutive 16-byte chunks of a row,
// 64x64 tiles staged through LDS wherever a transpose is needed so that both the read and the write side stay coalesced.
#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;

template <typename T>
__device__ inline vec16 scale16(const vec16& v, float c) {
  Pack16<T> p;
  p.v = v;
#pragma unroll
  for (int i = 0; i < Elem<T>::per16; ++i) p.e[i] = Elem<T>::down(Elem<T>::up(p.e[i]) * c);
  return p.v;
}

// out[n, :] = src[idx[n] / fan_out, :] * coeff[idx[n]]
template <typename T>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(const T* __restrict__ src, const int32_t* __restrict__ idx,
                                                              const T* __restrict__ coeff, int fan_out, int64_t num_rows,
                                                              int chunks_per_row, T* __restrict__ out) {
  constexpr int P = Elem<T>::per16;
  const int64_t total = num_rows * chunks_per_row;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x; c < total; c += stride) {
    const int64_t n = c / chunks_per_row;
    const int ch = (int)(c - n * chunks_per_row);
    const int32_t slot = idx[n];
    const int64_t srow = slot / fan_out;
    vec16 v = load16(src + (srow * chunks_per_row + ch) * P);
    if (coeff != nullptr) {
      // the product is rounded to the tensor dtype, as the reference's gather does (kernels.py:268-273)
      v = scale16<T>(v, Elem<T>::up(coeff[slot]));
    }
    store16_nt(out + c * P, v);
  }
}

// out[t, :] = sum_j gates[t, j] * expanded[t, j, :]
template <typename T>
__global__ __launch_bounds__(kBlock) void combine_rows_kernel(const T* __restrict__ expanded, const T* __restrict__ gates,
                                                               int64_t T_tokens, int k, int chunks_per_row,
                                                               T* __restrict__ out) {
  constexpr int P = Elem<T>::per16;
  const int64_t total = T_tokens * chunks_per_row;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x; c < total; c += stride) {
    const int64_t t = c / chunks_per_row;
    const int ch = (int)(c - t * chunks_per_row);
    float acc[P];
#pragma unroll
    for (int i = 0; i < P; ++i) acc[i] = 0.f;
    for (int j = 0; j < k; ++j) {
      Pack16<T> p;
      p.v = load16_nt(expanded + ((t * k + j) * chunks_per_row + ch) * P);  // read once
      const float g = gates ? Elem<T>::up(gates[t * k + j]) : 1.0f;
#pragma unroll
      for (int i = 0; i < P; ++i) acc[i] += g * Elem<T>::up(p.e[i]);
    }
    Pack16<T> o;
#pragma unroll
    for (int i = 0; i < P; ++i) o.e[i] = Elem<T>::down(acc[i]);
    store16_nt(out + c * P, o.v);
  }
}

// d_gates[t, j] = <expanded[t, j, :], grad_out[t, :]>, one wave per (t, j)
template <typename T, typename OUT>
__global__ __launch_bounds__(kBlock) void gate_grad_kernel(const T* __restrict__ expanded, const T* __restrict__ grad_out,
                                                            int64_t pairs, int k, int chunks_per_row,
                                                            OUT* __restrict__ d_gates) {
  constexpr int P = Elem<T>::per16;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t pair = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (pair >= pairs) return;
  const int64_t t = pair / k;
  float acc = 0.f;
  for (int ch = lane; ch < chunks_per_row; ch += kWave) {
    Pack16<T> a, b;
    a.v = load16_nt(expanded + (pair * chunks_per_row + ch) * P);  // read once
    b.v = load16(grad_out + (t * chunks_per_row + ch) * P);
#pragma unroll
    for (int i = 0; i < P; ++i) acc += Elem<T>::up(a.e[i]) * Elem<T>::up(b.e[i]);
  }
  acc = wave_sum(acc);
  if (lane == 0) d_gates[pair] = Elem<OUT>::down(acc);
}

// ---- 64x64 tiles of 16-bit elements through LDS ---------------------------------------------------------------
constexpr int kTile = 64;
constexpr int kTileStride = kTile + 2;  // in elements: 33 words per row, so column reads spread over the banks

// Writes tile^T: dst[(c0 + c) * ld + r0 + r] = tile[r][c] for r < 64 (rows valid up to rows_ok), c < cols_ok.
// Each thread assembles 16-byte chunks along r. Requires r0 % 8 == 0, ld % 8 == 0.
template <typename T>
__device__ inline void store_tile_transposed(const T (*tile)[kTileStride], T* __restrict__ dst, int64_t ld, int64_t r0,
                                             int64_t c0, int cols_ok, int64_t r_limit) {
#pragma unroll
  for (int q = 0; q < (kTile * kTile / 8) / kBlock; ++q) {
    const int chunk = q * kBlock + threadIdx.x;
    const int c = chunk >> 3, rc = (chunk & 7) * 8;
    if (c < cols_ok && r0 + rc < r_limit) {
      Pack16<T> p;
#pragma unroll
      for (int i = 0; i < 8; ++i) p.e[i] = tile[rc + i][c];
      store16_nt(dst + (c0 + c) * ld + r0 + rc, p.v);  // multi-GB outputs: written once, read by a later kernel
    }
  }
}

template <typename T>
__device__ inline void fill_tile_chunk(T (*tile)[kTileStride], int r, int cchunk, const vec16& v) {
  uint32_t* w = reinterpret_cast<uint32_t*>(&tile[r][cchunk * 8]);
  w[0] = v.w[0];
  w[1] = v.w[1];
  w[2] = v.w[2];
  w[3] = v.w[3];
}

// grid: (ceil(H / 64), max_rows / 64). Valid padded rows gather a (scaled) token row; pad rows of live tiles are zero.
template <typename T>
__global__ __launch_bounds__(kBlock) void group_rows_padded_kernel(
    const T* __restrict__ src, const T* __restrict__ coeff, int fan_out, int H, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ seg_starts, const uint32_t* __restrict__ counts, const int32_t* __restrict__ tile_expert,
    int align, T* __restrict__ grouped, T* __restrict__ grouped_t, int64_t ld_t) {
  __shared__ T tile[kTile][kTileStride];
  const int64_t p0 = (int64_t)blockIdx.y * kTile;
  const int e = tile_expert[p0 / align];
  if (e < 0) return;  // past the last segment: nothing reads these rows
  const int64_t valid_end = (int64_t)seg_starts[e] + counts[e];
  const int h0 = blockIdx.x * kTile;
#pragma unroll
  for (int q = 0; q < (kTile * kTile / 8) / kBlock; ++q) {
    const int chunk = q * kBlock + threadIdx.x;
    const int r = chunk >> 3, cc = chunk & 7;
    const int64_t p = p0 + r;
    const int h = h0 + cc * 8;
    vec16 v = zero16();
    if (p < valid_end && h < H) {
      if (fan_out > 0) {
        const int32_t slot = row_slot[p];
        v = load16(src + (int64_t)(slot / fan_out) * H + h);
        if (coeff != nullptr) v = scale16<T>(v, Elem<T>::up(coeff[slot]));
      } else {  // src is already padded-grouped: row p maps to itself
        v = load16(src + p * H + h);
      }
    }
    if (grouped != nullptr && h < H) store16_nt(grouped + p * H + h, v);
    if (grouped_t != nullptr) fill_tile_chunk(tile, r, cc, v);
  }
  if (grouped_t == nullptr) return;
  __syncthreads();
  store_tile_transposed<T>(tile, grouped_t, ld_t, p0, h0, min(kTile, H - h0), p0 + kTile);
}

// SwiGLU backward over padded grouped rows, with the transposed copy the weight-gradient GEMM consumes:
//   d_pre[p, :] = swiglu_bwd(pre[p, :], d_act[p, :]) for valid rows;  d_pre_t = d_pre^T with zeros in pad rows.
// grid: (ceil(I / 64), max_rows / 64); pre / d_pre are [max_rows, 2I] packed [up | gate], d_act is [max_rows, I].
template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_grouped_kernel(
    const T* __restrict__ pre, const T* __restrict__ d_act, int I, const int32_t* __restrict__ seg_starts,
    const uint32_t* __restrict__ counts, const int32_t* __restrict__ tile_expert, int align, T* __restrict__ d_pre,
    T* __restrict__ d_pre_t, int64_t ld_t, int act_kind) {
  __shared__ T tile_up[kTile][kTileStride];
  __shared__ T tile_gate[kTile][kTileStride];
  const int64_t p0 = (int64_t)blockIdx.y * kTile;
  const int e = tile_expert[p0 / align];
  if (e < 0) return;
  const int64_t valid_end = (int64_t)seg_starts[e] + counts[e];
  const int c0 = blockIdx.x * kTile;
  const int64_t two_i = 2 * (int64_t)I;
#pragma unroll
  for (int q = 0; q < (kTile * kTile / 8) / kBlock; ++q) {
    const int chunk = q * kBlock + threadIdx.x;
    const int r = chunk >> 3, cc = chunk & 7;
    const int64_t p = p0 + r;
    const int c = c0 + cc * 8;
    Pack16<T> du, dg;
    du.v = zero16();
    dg.v = zero16();
    if (p < valid_end && c < I) {
      Pack16<T> u, g, dy;
      u.v = load16_nt(pre + p * two_i + c);  // all three are read once
      g.v = load16_nt(pre + p * two_i + I + c);
      dy.v = load16_nt(d_act + p * I + c);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float gf = Elem<T>::up(g.e[i]), uf = Elem<T>::up(u.e[i]), dyf = Elem<T>::up(dy.e[i]);
        const float sg = sigmoid_for<T>(gf);
        if (act_kind == CK_ACT_GLU) {  // act = up * sigmoid(gate)
          dg.e[i] = Elem<T>::down(dyf * uf * sg * (1.0f - sg));
          du.e[i] = Elem<T>::down(dyf * sg);
        } else {  // act = up * gate * sigmoid(gate)
          const float gsg = gf * sg;
          dg.e[i] = Elem<T>::down(dyf * uf * (sg + gsg * (1.0f - sg)));
          du.e[i] = Elem<T>::down(dyf * gsg);
        }
      }
      store16_nt(d_pre + p * two_i + c, du.v);
      store16_nt(d_pre + p * two_i + I + c, dg.v);
    }
    if (d_pre_t != nullptr) {
      fill_tile_chunk(tile_up, r, cc, du.v);
      fill_tile_chunk(tile_gate, r, cc, dg.v);
    }
  }
  if (d_pre_t == nullptr) return;
  __syncthreads();
  const int cols_ok = min(kTile, I - c0);
  store_tile_transposed<T>(tile_up, d_pre_t, ld_t, p0, c0, cols_ok, p0 + kTile);
  store_tile_transposed<T>(tile_gate, d_pre_t, ld_t, p0, (int64_t)I + c0, cols_ok, p0 + kTile);
}

// Whole-row forms of the two kernels above for callers that take no transposed copy (the weight-gradient GEMM reads
// row-major operands): consecutive lanes walk consecutive 16-byte chunks of a row, so a wave touches 1 KiB of each
// stream at a time instead of 64 rows x 128 bytes. Same results as the tiled kernels, pad rows included.
template <typename T>
__global__ __launch_bounds__(kBlock) void group_rows_stream_kernel(
    const T* __restrict__ src, const T* __restrict__ coeff, int fan_out, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ seg_starts, const uint32_t* __restrict__ counts, const int32_t* __restrict__ tile_expert,
    int align, int64_t max_rows, int chunks_per_row, T* __restrict__ grouped) {
  constexpr int P = Elem<T>::per16;  // elements per 16-byte chunk
  const int64_t total = max_rows * chunks_per_row;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x; c < total; c += stride) {
    const int64_t p = c / chunks_per_row;
    const int ch = (int)(c - p * chunks_per_row);
    const int e = tile_expert[p / align];
    if (e < 0) continue;  // past the last segment: nothing reads these rows
    vec16 v = zero16();
    if (p < (int64_t)seg_starts[e] + counts[e]) {
      if (fan_out > 0) {
        const int32_t slot = row_slot[p];
        v = load16(src + ((int64_t)(slot / fan_out) * chunks_per_row + ch) * P);
        if (coeff != nullptr) v = scale16<T>(v, Elem<T>::up(coeff[slot]));
      } else {
        v = load16(src + c * P);
      }
    }
    store16_nt(grouped + c * P, v);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_stream_kernel(
    const T* __restrict__ pre, const T* __restrict__ d_act, int chunks_per_row, const int32_t* __restrict__ seg_starts,
    const uint32_t* __restrict__ counts, const int32_t* __restrict__ tile_expert, int align, int64_t max_rows,
    T* __restrict__ d_pre, int act_kind) {
  const int64_t total = max_rows * chunks_per_row;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int I = chunks_per_row * 8;
  for (int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x; c < total; c += stride) {
    const int64_t p = c / chunks_per_row;
    const int col = (int)(c - p * chunks_per_row) * 8;
    const int e = tile_expert[p / align];
    if (e < 0 || p >= (int64_t)seg_starts[e] + counts[e]) continue;  // pad rows of d_pre are left as they are
    const int64_t up_at = p * 2 * I + col;
    Pack16<T> u, g, dy, du, dg;
    u.v = load16_nt(pre + up_at);  // all three are read once
    g.v = load16_nt(pre + up_at + I);
    dy.v = load16_nt(d_act + c * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float gf = Elem<T>::up(g.e[i]), uf = Elem<T>::up(u.e[i]), dyf = Elem<T>::up(dy.e[i]);
      const float sg = sigmoid_for<T>(gf);
      if (act_kind == CK_ACT_GLU) {  // act = up * sigmoid(gate)
        dg.e[i] = Elem<T>::down(dyf * uf * sg * (1.0f - sg));
        du.e[i] = Elem<T>::down(dyf * sg);
      } else {  // act = up * gate * sigmoid(gate)
        const float gsg = gf * sg;
        dg.e[i] = Elem<T>::down(dyf * uf * (sg + gsg * (1.0f - sg)));
        du.e[i] = Elem<T>::down(dyf * gsg);
      }
    }
    store16_nt(d_pre + up_at, du.v);
    store16_nt(d_pre + up_at + I, dg.v);
  }
}

// dst[b, c, r] = src[b, r, c]; grid: (ceil(cols/64), ceil(rows/64), batch); rows % 8 == 0 and cols % 8 == 0
template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_batched_kernel(const T* __restrict__ src, int rows, int cols,
                                                                    T* __restrict__ dst) {
  __shared__ T tile[kTile][kTileStride];
  const int64_t boff = (int64_t)blockIdx.z * rows * cols;
  const int r0 = blockIdx.y * kTile, c0 = blockIdx.x * kTile;
#pragma unroll
  for (int q = 0; q < (kTile * kTile / 8) / kBlock; ++q) {
    const int chunk = q * kBlock + threadIdx.x;
    const int r = chunk >> 3, cc = chunk & 7;
    vec16 v = zero16();
    if (r0 + r < rows && c0 + cc * 8 < cols) v = load16_nt(src + boff + (int64_t)(r0 + r) * cols + c0 + cc * 8);
    fill_tile_chunk(tile, r, cc, v);
  }
  __syncthreads();
  store_tile_transposed<T>(tile, dst + boff, rows, r0, c0, min(kTile, cols - c0), rows);
}

inline unsigned grid_for(int64_t work_items, int per_thread) {
  int64_t b = ceil_div(work_items, (int64_t)kBlock * per_thread);
  if (b < 1) b = 1;
  if (b > 65535 * 16) b = 65535 * 16;
  return (unsigned)b;
}


// ---- expert biases (the reference's Experts_Torch applies one bias row per expert: torch_implementation.py:20-22,42) ----
// y[r, :] += bias[e(r), :]. Grouped rows: e(r) is the expert of the row's tile, pad rows are skipped. Token-order rows
// (row_expert != nullptr): e(r) = row_expert[r], negative = skip.
template <typename T>
__global__ __launch_bounds__(kBlock) void add_expert_bias_kernel(T* __restrict__ y, int64_t rows, int N,
                                                                  const T* __restrict__ bias,
                                                                  const int32_t* __restrict__ row_expert,
                                                                  const int32_t* __restrict__ seg_starts,
                                                                  const uint32_t* __restrict__ counts,
                                                                  const int32_t* __restrict__ tile_expert, int align) {
  const int chunks = N / 8;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    int e;
    if (row_expert != nullptr) {
      e = row_expert[r];
    } else {
      e = tile_expert[r / align];
      if (e >= 0 && r >= (int64_t)seg_starts[e] + counts[e]) e = -1;
    }
    if (e < 0) continue;
    for (int ch = blockIdx.x * kBlock + threadIdx.x; ch < chunks; ch += gridDim.x * kBlock) {
      Pack16<T> v, b;
      v.v = load16(y + r * N + ch * 8);
      b.v = load16(bias + (int64_t)e * N + ch * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) v.e[i] = Elem<T>::down(Elem<T>::up(v.e[i]) + Elem<T>::up(b.e[i]));
      store16(y + r * N + ch * 8, v.v);
    }
  }
}

// d_bias[e, :] = sum over the rows of expert e of d_y (padded grouped rows), fp32 accumulation in a fixed order.
// grid (ceil(N / 64), E); a block owns 64 columns, its 4 waves split the rows, 8 loads in flight per wave.
template <typename T>
__global__ __launch_bounds__(kBlock) void expert_bias_grad_kernel(const T* __restrict__ d_y, int N,
                                                                   const int32_t* __restrict__ seg_starts,
                                                                   const uint32_t* __restrict__ counts,
                                                                   T* __restrict__ d_bias) {
  __shared__ float part[kBlock / kWave][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int e = blockIdx.y, col = blockIdx.x * kWave + lane;
  const int64_t first = seg_starts[e], last = first + counts[e];
  float s = 0.f;
  if (col < N) {
    constexpr int U = 8, W = kBlock / kWave;
    float acc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) acc[u] = 0.f;
    int64_t r = first + wave;
    for (; r + (U - 1) * W < last; r += U * W) {
#pragma unroll
      for (int u = 0; u < U; ++u) acc[u] += Elem<T>::up(d_y[(r + u * W) * N + col]);
    }
    for (; r < last; r += W) acc[0] += Elem<T>::up(d_y[r * N + col]);
#pragma unroll
    for (int u = 0; u < U; ++u) s += acc[u];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && col < N) {
    float t = 0.f;
#pragma unroll
    for (int g = 0; g < kBlock / kWave; ++g) t += part[g][lane];
    d_bias[(int64_t)e * N + col] = Elem<T>::down(t);
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_gather_rows(const void* src, const int32_t* idx, const void* coeff, int32_t fan_out, int64_t num_rows,
                              int32_t H, void* out, int32_t dtype, void* stream) {
  CK_REQUIRE(num_rows >= 0 && H >= 1 && fan_out >= 1, "ck_gather_rows: bad sizes rows=%lld H=%d fan_out=%d",
             (long long)num_rows, H, fan_out);
  if (num_rows == 0) return CK_OK;
  CK_REQUIRE(src && idx && out, "ck_gather_rows: NULL argument");
  CK_REQUIRE(aligned16(src) && aligned16(out), "ck_gather_rows: src/out must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_gather_rows", {
    constexpr int P = Elem<scalar_t>::per16;
    CK_REQUIRE(H % P == 0, "ck_gather_rows: H=%d is not a multiple of %d", H, P);
    const int cpr = H / P;
    hipLaunchKernelGGL((gather_rows_kernel<scalar_t>), dim3(grid_for(num_rows * cpr, 2)), dim3(kBlock), 0, s,
                       static_cast<const scalar_t*>(src), idx, static_cast<const scalar_t*>(coeff), (int)fan_out,
                       num_rows, cpr, static_cast<scalar_t*>(out));
  });
  CK_CHECK_LAUNCH("ck_gather_rows");
  return CK_OK;
}

extern "C" int ck_combine_rows(const void* expanded, const void* gates, int64_t T, int32_t k, int32_t H, void* out,
                               const void* grad_out, void* d_gates_out, int32_t dtype, void* stream) {
  CK_REQUIRE(T >= 0 && k >= 1 && H >= 1, "ck_combine_rows: bad sizes T=%lld k=%d H=%d", (long long)T, k, H);
  if (T == 0) return CK_OK;
  CK_REQUIRE(expanded != nullptr && aligned16(expanded), "ck_combine_rows: expanded is NULL or misaligned");
  CK_REQUIRE(out != nullptr || d_gates_out != nullptr, "ck_combine_rows: nothing to compute");
  CK_REQUIRE(d_gates_out == nullptr || grad_out != nullptr, "ck_combine_rows: d_gates_out needs grad_out");
  CK_REQUIRE((out == nullptr || aligned16(out)) && (grad_out == nullptr || aligned16(grad_out)),
             "ck_combine_rows: out/grad_out must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_combine_rows", {
    constexpr int P = Elem<scalar_t>::per16;
    CK_REQUIRE(H % P == 0, "ck_combine_rows: H=%d is not a multiple of %d", H, P);
    const int cpr = H / P;
    if (out != nullptr) {
      hipLaunchKernelGGL((combine_rows_kernel<scalar_t>), dim3(grid_for(T * cpr, 1)), dim3(kBlock), 0, s,
                         static_cast<const scalar_t*>(expanded), static_cast<const scalar_t*>(gates), T, (int)k, cpr,
                         static_cast<scalar_t*>(out));
    }
    if (d_gates_out != nullptr) {
      const int64_t pairs = T * k;
      hipLaunchKernelGGL((gate_grad_kernel<scalar_t, scalar_t>), dim3((unsigned)ceil_div(pairs, kBlock / kWave)), dim3(kBlock),
                         0, s, static_cast<const scalar_t*>(expanded), static_cast<const scalar_t*>(grad_out), pairs,
                         (int)k, cpr, static_cast<scalar_t*>(d_gates_out));
    }
  });
  CK_CHECK_LAUNCH("ck_combine_rows");
  return CK_OK;
}

extern "C" int ck_gate_grad_f32(const void* expanded, const void* grad_out, int64_t T, int32_t k, int32_t H,
                                float* d_gates, int32_t dtype, void* stream) {
  CK_REQUIRE(T >= 0 && k >= 1 && H >= 1, "ck_gate_grad_f32: bad sizes T=%lld k=%d H=%d", (long long)T, k, H);
  if (T == 0) return CK_OK;
  CK_REQUIRE(expanded && grad_out && d_gates, "ck_gate_grad_f32: NULL argument");
  CK_REQUIRE(aligned16(expanded) && aligned16(grad_out), "ck_gate_grad_f32: expanded / grad_out must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_gate_grad_f32", {
    constexpr int P = Elem<scalar_t>::per16;
    CK_REQUIRE(H % P == 0, "ck_gate_grad_f32: H=%d is not a multiple of %d", H, P);
    const int64_t pairs = T * k;
    hipLaunchKernelGGL((gate_grad_kernel<scalar_t, float>), dim3((unsigned)ceil_div(pairs, kBlock / kWave)), dim3(kBlock), 0,
                       s, static_cast<const scalar_t*>(expanded), static_cast<const scalar_t*>(grad_out), pairs, (int)k,
                       H / P, d_gates);
  });
  CK_CHECK_LAUNCH("ck_gate_grad_f32");
  return CK_OK;
}

extern "C" int ck_group_rows_padded(const void* src, const void* coeff, int32_t fan_out, int32_t H,
                                    const int32_t* row_slot, const int32_t* seg_starts, const uint32_t* counts,
                                    const int32_t* tile_expert, int32_t align, int64_t max_rows, void* grouped,
                                    void* grouped_t, int64_t ld_t, int32_t dtype, void* stream) {
  CK_REQUIRE(H >= 8 && H % 8 == 0, "ck_group_rows_padded: H=%d must be a positive multiple of 8", H);
  CK_REQUIRE(fan_out >= 0 && (fan_out > 0 || coeff == nullptr), "ck_group_rows_padded: fan_out=%d (0 takes no coeff)", fan_out);
  CK_REQUIRE(align >= kTile && align % kTile == 0, "ck_group_rows_padded: align=%d must be a multiple of %d", align, kTile);
  CK_REQUIRE(max_rows >= 0 && max_rows % align == 0, "ck_group_rows_padded: max_rows=%lld is not a multiple of align",
             (long long)max_rows);
  if (max_rows == 0) return CK_OK;
  CK_REQUIRE(src && row_slot && seg_starts && counts && tile_expert, "ck_group_rows_padded: NULL argument");
  CK_REQUIRE(grouped || grouped_t, "ck_group_rows_padded: nothing to write");
  CK_REQUIRE(grouped_t == nullptr || (ld_t >= max_rows && ld_t % 8 == 0),
             "ck_group_rows_padded: ld_t=%lld must be >= max_rows and a multiple of 8", (long long)ld_t);
  CK_REQUIRE(aligned16(src) && (!grouped || aligned16(grouped)) && (!grouped_t || aligned16(grouped_t)),
             "ck_group_rows_padded: pointers must be 16-byte aligned");
  CK_REQUIRE(max_rows / kTile <= 65535, "ck_group_rows_padded: too many rows for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)ceil_div(H, kTile), (unsigned)(max_rows / kTile));
  if (grouped_t == nullptr) {  // the row-major copy alone: also for fp32 rows
    CK_DISPATCH_FLOAT(dtype, "ck_group_rows_padded", {
      constexpr int P = Elem<scalar_t>::per16;
      CK_REQUIRE(H % P == 0, "ck_group_rows_padded: H=%d must be a multiple of %d", H, P);
      hipLaunchKernelGGL((group_rows_stream_kernel<scalar_t>), dim3(grid_for(max_rows * (H / P), 2)), dim3(kBlock), 0, s,
                         static_cast<const scalar_t*>(src), static_cast<const scalar_t*>(coeff), (int)fan_out, row_slot,
                         seg_starts, counts, tile_expert, (int)align, max_rows, (int)(H / P),
                         static_cast<scalar_t*>(grouped));
    });
    CK_CHECK_LAUNCH("ck_group_rows_padded");
    return CK_OK;
  }
  CK_DISPATCH_HALF(dtype, "ck_group_rows_padded", {
    hipLaunchKernelGGL((group_rows_padded_kernel<scalar_t>), grid, dim3(kBlock), 0, s,
                       static_cast<const scalar_t*>(src), static_cast<const scalar_t*>(coeff), (int)fan_out, (int)H,
                       row_slot, seg_starts, counts, tile_expert, (int)align, static_cast<scalar_t*>(grouped),
                       static_cast<scalar_t*>(grouped_t), ld_t);
  });
  CK_CHECK_LAUNCH("ck_group_rows_padded");
  return CK_OK;
}

extern "C" int ck_swiglu_bwd_grouped(const void* pre, const void* d_act, int32_t I, const int32_t* seg_starts,
                                     const uint32_t* counts, const int32_t* tile_expert, int32_t align,
                                     int64_t max_rows, void* d_pre, void* d_pre_t, int64_t ld_t, int32_t act_kind,
                                     int32_t dtype, void* stream) {
  CK_REQUIRE(I >= 8 && I % 8 == 0, "ck_swiglu_bwd_grouped: I=%d must be a positive multiple of 8", I);
  CK_REQUIRE(act_kind == CK_ACT_SWIGLU || act_kind == CK_ACT_GLU, "ck_swiglu_bwd_grouped: unknown act_kind %d", act_kind);
  CK_REQUIRE(align >= kTile && align % kTile == 0, "ck_swiglu_bwd_grouped: align=%d must be a multiple of %d", align, kTile);
  CK_REQUIRE(max_rows >= 0 && max_rows % align == 0, "ck_swiglu_bwd_grouped: max_rows=%lld is not a multiple of align",
             (long long)max_rows);
  if (max_rows == 0) return CK_OK;
  CK_REQUIRE(pre && d_act && d_pre && seg_starts && counts && tile_expert, "ck_swiglu_bwd_grouped: NULL argument");
  CK_REQUIRE(d_pre_t == nullptr || (ld_t >= max_rows && ld_t % 8 == 0),
             "ck_swiglu_bwd_grouped: ld_t=%lld must be >= max_rows and a multiple of 8", (long long)ld_t);
  CK_REQUIRE(aligned16(pre) && aligned16(d_act) && aligned16(d_pre) && (!d_pre_t || aligned16(d_pre_t)),
             "ck_swiglu_bwd_grouped: pointers must be 16-byte aligned");
  CK_REQUIRE(max_rows / kTile <= 65535, "ck_swiglu_bwd_grouped: too many rows for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)ceil_div(I, kTile), (unsigned)(max_rows / kTile));
  if (d_pre_t == nullptr) {
    CK_DISPATCH_HALF(dtype, "ck_swiglu_bwd_grouped", {
      hipLaunchKernelGGL((swiglu_bwd_stream_kernel<scalar_t>), dim3(grid_for(max_rows * (I / 8), 1)), dim3(kBlock), 0, s,
                         static_cast<const scalar_t*>(pre), static_cast<const scalar_t*>(d_act), (int)(I / 8), seg_starts,
                         counts, tile_expert, (int)align, max_rows, static_cast<scalar_t*>(d_pre), (int)act_kind);
    });
    CK_CHECK_LAUNCH("ck_swiglu_bwd_grouped");
    return CK_OK;
  }
  CK_DISPATCH_HALF(dtype, "ck_swiglu_bwd_grouped", {
    hipLaunchKernelGGL((swiglu_bwd_grouped_kernel<scalar_t>), grid, dim3(kBlock), 0, s,
                       static_cast<const scalar_t*>(pre), static_cast<const scalar_t*>(d_act), (int)I, seg_starts, counts,
                       tile_expert, (int)align, static_cast<scalar_t*>(d_pre), static_cast<scalar_t*>(d_pre_t), ld_t,
                       (int)act_kind);
  });
  CK_CHECK_LAUNCH("ck_swiglu_bwd_grouped");
  return CK_OK;
}

extern "C" int ck_transpose_batched(const void* src, int64_t batch, int32_t rows, int32_t cols, void* dst,
                                    int32_t dtype, void* stream) {
  CK_REQUIRE(batch >= 0 && rows >= 8 && cols >= 8 && rows % 8 == 0 && cols % 8 == 0,
             "ck_transpose_batched: rows=%d cols=%d must be positive multiples of 8", rows, cols);
  if (batch == 0) return CK_OK;
  CK_REQUIRE(src && dst && aligned16(src) && aligned16(dst), "ck_transpose_batched: NULL or misaligned pointer");
  CK_REQUIRE(batch <= 65535 && ceil_div(rows, kTile) <= 65535, "ck_transpose_batched: grid too large");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)ceil_div(cols, kTile), (unsigned)ceil_div(rows, kTile), (unsigned)batch);
  CK_DISPATCH_HALF(dtype, "ck_transpose_batched", {
    hipLaunchKernelGGL((transpose_batched_kernel<scalar_t>), grid, dim3(kBlock), 0, s,
                       static_cast<const scalar_t*>(src), (int)rows, (int)cols, static_cast<scalar_t*>(dst));
  });
  CK_CHECK_LAUNCH("ck_transpose_batched");
  return CK_OK;
}

extern "C" int ck_add_expert_bias(void* y, int64_t rows, int32_t N, const void* bias, const int32_t* row_expert,
                                  const ck_segments* seg, int32_t dtype, void* stream) {
  const char* name = "ck_add_expert_bias";
  CK_REQUIRE(rows >= 0 && N >= 8 && N % 8 == 0, "%s: N=%d must be a positive multiple of 8", name, N);
  if (rows == 0) return CK_OK;
  CK_REQUIRE(y && bias && aligned16(y) && aligned16(bias), "%s: NULL or misaligned pointer", name);
  CK_REQUIRE(row_expert != nullptr || seg != nullptr, "%s: give row_expert (token-order rows) or seg (grouped rows)", name);
  CK_REQUIRE(row_expert != nullptr || (seg->seg_starts && seg->counts && seg->tile_expert && seg->align >= 1 &&
                                        rows <= seg->max_rows),
             "%s: seg is incomplete or has fewer rows than y", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)ceil_div(N / 8, kBlock), (unsigned)(rows < 65535 ? rows : 65535));
  CK_DISPATCH_HALF(dtype, name, {
    hipLaunchKernelGGL((add_expert_bias_kernel<scalar_t>), grid, dim3(kBlock), 0, s, static_cast<scalar_t*>(y), rows, (int)N,
                       static_cast<const scalar_t*>(bias), row_expert, row_expert ? nullptr : seg->seg_starts,
                       row_expert ? nullptr : seg->counts, row_expert ? nullptr : seg->tile_expert,
                       row_expert ? 1 : seg->align);
  });
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int ck_expert_bias_grad(const void* d_y, int32_t N, const ck_segments* seg, void* d_bias, int32_t dtype,
                                   void* stream) {
  const char* name = "ck_expert_bias_grad";
  CK_REQUIRE(N >= 1, "%s: N=%d must be positive", name, N);
  CK_REQUIRE(seg && seg->seg_starts && seg->counts && seg->num_experts >= 1 && seg->num_experts <= 65535,
             "%s: seg is incomplete (or more than 65535 experts)", name);
  CK_REQUIRE(d_bias != nullptr && (seg->max_rows == 0 || d_y != nullptr), "%s: NULL argument", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)ceil_div(N, kWave), (unsigned)seg->num_experts);
  CK_DISPATCH_FLOAT(dtype, name, {
    hipLaunchKernelGGL((expert_bias_grad_kernel<scalar_t>), grid, dim3(kBlock), 0, s, static_cast<const scalar_t*>(d_y),
                       (int)N, seg->seg_starts, seg->counts, static_cast<scalar_t*>(d_bias));
  });
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}
