// Stand-alone SwiGLU forward / backward: out = up * gate * sigmoid(gate), fp32 math, one rounding on the way out.
// Row-strided operands so that the [up | gate] halves of a packed tensor are consumed in place.
#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;

// N elements moved as one access: N = Elem<T>::per16 (128-bit) on the aligned fast path, N = 1 otherwise.
template <typename T, int N>
struct Chunk {
  T e[N];
  __device__ static inline Chunk load(const T* p) {
    Chunk c;
    if constexpr (N == 1) {
      c.e[0] = *p;
    } else {
      Pack16<T> k;
      k.v = load16_nt(p);  // streaming: every element is read once
#pragma unroll
      for (int i = 0; i < N; ++i) c.e[i] = k.e[i];
    }
    return c;
  }
  __device__ inline void store(T* p) const {
    if constexpr (N == 1) {
      *p = e[0];
    } else {
      Pack16<T> k;
#pragma unroll
      for (int i = 0; i < N; ++i) k.e[i] = e[i];
      store16_nt(p, k.v);
    }
  }
};

template <typename T, int P>
__global__ __launch_bounds__(kBlock) void swiglu_fwd_kernel(const T* __restrict__ gate, int64_t gate_stride,
                                                             const T* __restrict__ up, int64_t up_stride,
                                                             T* __restrict__ out, int64_t out_stride, int64_t rows,
                                                             int64_t chunks_per_row, int tpr_log2) {
  // 2^tpr_log2 threads share a row (chunk index = lane within the row, strided), the block's remaining threads take
  // further rows: no division per chunk, and short rows still fill the block. A flat tensor is one long row.
  const int tpr = 1 << tpr_log2;
  const int lane_in_row = threadIdx.x & (tpr - 1);
  const int64_t rows_per_block = kBlock >> tpr_log2;
  for (int64_t r = (int64_t)blockIdx.y * rows_per_block + (threadIdx.x >> tpr_log2); r < rows;
       r += (int64_t)gridDim.y * rows_per_block) {
    for (int64_t ch = (int64_t)blockIdx.x * tpr + lane_in_row; ch < chunks_per_row; ch += (int64_t)gridDim.x * tpr) {
      const int64_t col = ch * P;
      const Chunk<T, P> g = Chunk<T, P>::load(gate + r * gate_stride + col);
      const Chunk<T, P> u = Chunk<T, P>::load(up + r * up_stride + col);
      Chunk<T, P> o;
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const float gf = Elem<T>::up(g.e[i]);
        o.e[i] = Elem<T>::down(Elem<T>::up(u.e[i]) * gf * sigmoid_for<T>(gf));
      }
      o.store(out + r * out_stride + col);
    }
  }
}

template <typename T, int P>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_kernel(const T* __restrict__ gate, int64_t gate_stride,
                                                             const T* __restrict__ up, int64_t up_stride,
                                                             const T* __restrict__ d_out, int64_t d_out_stride,
                                                             T* __restrict__ d_gate, int64_t d_gate_stride,
                                                             T* __restrict__ d_up, int64_t d_up_stride, int64_t rows,
                                                             int64_t chunks_per_row, int tpr_log2) {
  const int tpr = 1 << tpr_log2;
  const int lane_in_row = threadIdx.x & (tpr - 1);
  const int64_t rows_per_block = kBlock >> tpr_log2;
  for (int64_t r = (int64_t)blockIdx.y * rows_per_block + (threadIdx.x >> tpr_log2); r < rows;
       r += (int64_t)gridDim.y * rows_per_block) {
    for (int64_t ch = (int64_t)blockIdx.x * tpr + lane_in_row; ch < chunks_per_row; ch += (int64_t)gridDim.x * tpr) {
      const int64_t col = ch * P;
      const Chunk<T, P> g = Chunk<T, P>::load(gate + r * gate_stride + col);
      const Chunk<T, P> u = Chunk<T, P>::load(up + r * up_stride + col);
      const Chunk<T, P> dy = Chunk<T, P>::load(d_out + r * d_out_stride + col);
      Chunk<T, P> dg, du;
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const float gf = Elem<T>::up(g.e[i]), uf = Elem<T>::up(u.e[i]), dyf = Elem<T>::up(dy.e[i]);
        const float sg = sigmoid_for<T>(gf);
        const float gsg = gf * sg;
        dg.e[i] = Elem<T>::down(dyf * uf * (sg + gsg * (1.0f - sg)));
        du.e[i] = Elem<T>::down(dyf * gsg);
      }
      dg.store(d_gate + r * d_gate_stride + col);
      du.store(d_up + r * d_up_stride + col);
    }
  }
}

template <typename T>
bool view_vector_ok(const void* p, int64_t stride, int64_t rows) {
  return aligned16(p) && (rows == 1 || stride % Elem<T>::per16 == 0);
}

// Launch shape for rows x chunks_per_row chunks: threads per row = smallest power of two covering the row (at most the
// block), grid.y over row groups, grid.x over the chunks of long rows (a flat tensor is one row). The slices of a row
// are the fast grid dimension, so blocks that run together walk memory in address order (with rows as the fast dimension
// they touched 4 KiB pieces of thousands of rows at once: 5.35 -> 5.7 TB/s for the backward pass at 32,768 x 14,336).
struct Shape {
  dim3 grid;
  int tpr_log2;
};
inline Shape shape_for(int64_t rows, int64_t chunks_per_row) {
  Shape s;
  s.tpr_log2 = 0;
  while ((1 << s.tpr_log2) < kBlock && (1 << s.tpr_log2) < chunks_per_row) ++s.tpr_log2;
  const int64_t rows_per_block = kBlock >> s.tpr_log2;
  int64_t gx = ceil_div(rows, rows_per_block);
  if (gx > 65535) gx = 65535;
  // long rows: split them over grid.x, one chunk per thread (many small blocks stream fastest here: 6.1 TB/s against
  // 5.7 with two chunks and 5.5 with four for the backward pass at 32,768 x 14,336), at most 2^20 blocks
  int64_t gy = 1;
  if (s.tpr_log2 == 8) {
    gy = ceil_div(chunks_per_row, (int64_t)kBlock);
    const int64_t most = ceil_div((int64_t)1 << 20, gx);
    if (gy > most) gy = most;
    if (gy < 1) gy = 1;
    if (gy > 65535) gy = 65535;
  }
  s.grid = dim3((unsigned)gy, (unsigned)gx);
  return s;
}

// d_pre = d_act * gelu'(pre) for the tanh-approximated GELU, over a flat range: the backward of the activation that the
// grouped GEMM's CK_EPI_GELU_TANH epilogue applies
template <typename T, int P>
__global__ __launch_bounds__(kBlock) void gelu_tanh_bwd_kernel(const T* __restrict__ pre, const T* __restrict__ d_act,
                                                                T* __restrict__ d_pre, int64_t chunks) {
  for (int64_t ch = (int64_t)blockIdx.x * kBlock + threadIdx.x; ch < chunks; ch += (int64_t)gridDim.x * kBlock) {
    const Chunk<T, P> x = Chunk<T, P>::load(pre + ch * P);
    const Chunk<T, P> g = Chunk<T, P>::load(d_act + ch * P);
    Chunk<T, P> o;
#pragma unroll
    for (int i = 0; i < P; ++i) o.e[i] = Elem<T>::down(Elem<T>::up(g.e[i]) * gelu_tanh_grad_fast(Elem<T>::up(x.e[i])));
    o.store(d_pre + ch * P);
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_swiglu_fwd(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                             int64_t out_stride, int64_t rows, int64_t cols, int32_t dtype, void* stream) {
  CK_REQUIRE(rows >= 0 && cols >= 0, "ck_swiglu_fwd: negative size");
  if (rows == 0 || cols == 0) return CK_OK;
  CK_REQUIRE(gate && up && out, "ck_swiglu_fwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_swiglu_fwd", {
    constexpr int P = Elem<scalar_t>::per16;
    const scalar_t* g = static_cast<const scalar_t*>(gate);
    const scalar_t* u = static_cast<const scalar_t*>(up);
    scalar_t* o = static_cast<scalar_t*>(out);
    const bool vec = view_vector_ok<scalar_t>(gate, gate_stride, rows) && view_vector_ok<scalar_t>(up, up_stride, rows) &&
                     view_vector_ok<scalar_t>(out, out_stride, rows) && (cols % P == 0 || rows == 1);
    int64_t done = 0;  // columns covered by the 128-bit kernel
    if (vec && cols >= P) {
      done = cols / P * P;
      const Shape sh = shape_for(rows, done / P);
      hipLaunchKernelGGL((swiglu_fwd_kernel<scalar_t, P>), sh.grid, dim3(kBlock), 0, s, g, gate_stride, u, up_stride, o,
                         out_stride, rows, done / P, sh.tpr_log2);
    }
    if (done < cols) {  // misaligned views, or the ragged end of a flat tensor
      const int64_t rest = cols - done;
      const Shape sh = shape_for(rows, rest);
      hipLaunchKernelGGL((swiglu_fwd_kernel<scalar_t, 1>), sh.grid, dim3(kBlock), 0, s, g + done, gate_stride, u + done,
                         up_stride, o + done, out_stride, rows, rest, sh.tpr_log2);
    }
  });
  CK_CHECK_LAUNCH("ck_swiglu_fwd");
  return CK_OK;
}

extern "C" int ck_swiglu_bwd(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride,
                             const void* d_out, int64_t d_out_stride, void* d_gate, int64_t d_gate_stride, void* d_up,
                             int64_t d_up_stride, int64_t rows, int64_t cols, int32_t dtype, void* stream) {
  CK_REQUIRE(rows >= 0 && cols >= 0, "ck_swiglu_bwd: negative size");
  if (rows == 0 || cols == 0) return CK_OK;
  CK_REQUIRE(gate && up && d_out && d_gate && d_up, "ck_swiglu_bwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, "ck_swiglu_bwd", {
    constexpr int P = Elem<scalar_t>::per16;
    const scalar_t* g = static_cast<const scalar_t*>(gate);
    const scalar_t* u = static_cast<const scalar_t*>(up);
    const scalar_t* dy = static_cast<const scalar_t*>(d_out);
    scalar_t* dg = static_cast<scalar_t*>(d_gate);
    scalar_t* du = static_cast<scalar_t*>(d_up);
    const bool vec = view_vector_ok<scalar_t>(gate, gate_stride, rows) && view_vector_ok<scalar_t>(up, up_stride, rows) &&
                     view_vector_ok<scalar_t>(d_out, d_out_stride, rows) &&
                     view_vector_ok<scalar_t>(d_gate, d_gate_stride, rows) &&
                     view_vector_ok<scalar_t>(d_up, d_up_stride, rows) && (cols % P == 0 || rows == 1);
    int64_t done = 0;
    if (vec && cols >= P) {
      done = cols / P * P;
      const Shape sh = shape_for(rows, done / P);
      hipLaunchKernelGGL((swiglu_bwd_kernel<scalar_t, P>), sh.grid, dim3(kBlock), 0, s, g, gate_stride, u, up_stride, dy,
                         d_out_stride, dg, d_gate_stride, du, d_up_stride, rows, done / P, sh.tpr_log2);
    }
    if (done < cols) {
      const int64_t rest = cols - done;
      const Shape sh = shape_for(rows, rest);
      hipLaunchKernelGGL((swiglu_bwd_kernel<scalar_t, 1>), sh.grid, dim3(kBlock), 0, s, g + done, gate_stride, u + done,
                         up_stride, dy + done, d_out_stride, dg + done, d_gate_stride, du + done, d_up_stride, rows, rest,
                         sh.tpr_log2);
    }
  });
  CK_CHECK_LAUNCH("ck_swiglu_bwd");
  return CK_OK;
}

extern "C" int ck_gelu_tanh_bwd(const void* pre, const void* d_act, void* d_pre, int64_t n, int32_t dtype, void* stream) {
  CK_REQUIRE(n >= 0, "ck_gelu_tanh_bwd: negative size");
  if (n == 0) return CK_OK;
  CK_REQUIRE(pre && d_act && d_pre, "ck_gelu_tanh_bwd: NULL argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_HALF(dtype, "ck_gelu_tanh_bwd", {
    constexpr int P = Elem<scalar_t>::per16;
    const scalar_t* x = static_cast<const scalar_t*>(pre);
    const scalar_t* g = static_cast<const scalar_t*>(d_act);
    scalar_t* o = static_cast<scalar_t*>(d_pre);
    const bool vec = ((reinterpret_cast<uintptr_t>(pre) | reinterpret_cast<uintptr_t>(d_act) | reinterpret_cast<uintptr_t>(d_pre)) & 15) == 0;
    const int64_t done = vec ? n / P * P : 0;
    auto grid_for = [](int64_t chunks) {
      const int64_t blocks = (chunks + kBlock - 1) / kBlock;
      return dim3((unsigned)(blocks < 256 * 16 ? blocks : 256 * 16));
    };
    if (done > 0) hipLaunchKernelGGL((gelu_tanh_bwd_kernel<scalar_t, P>), grid_for(done / P), dim3(kBlock), 0, s, x, g, o, done / P);
    if (done < n)
      hipLaunchKernelGGL((gelu_tanh_bwd_kernel<scalar_t, 1>), grid_for(n - done), dim3(kBlock), 0, s, x + done, g + done, o + done, n - done);
  });
  CK_CHECK_LAUNCH("ck_gelu_tanh_bwd");
  return CK_OK;
}
