// Grouped GEMMs of the expert layer for fp32 tensors: v_mfma_f32_32x32x2_f32, i.e. fp32 products and fp32 accumulation
// (the reference's Triton kernels take fp32 operands through TF32 -- cute_kernels/kernels/scattermoe/
// triton_implementation/kernels.py:131,218; full fp32 is the more accurate reading of the same arithmetic). fp32 is the
// dtype of the reference's test grid (tests/test_commons.py:26-27), not of the benchmarks: these kernels are plain
// 64 x 64 tiles staged through LDS, one 32 x 32 block per wave, and share the padded grouped layout, the gather and the
// scatter conventions of the 16-bit kernels.
#include "ck_common.h"

namespace ck {
namespace {

constexpr int TM = 64, TN = 64, TK = 16, NT = 256;

struct F32Params {
  const float* a;
  const float* w;
  const float* bias;
  float* y;
  int64_t w_expert_stride;
  int w_is_kn;  // 0: w [E, N, K] (forward); 1: w [E, K, N] (input gradient: the forward's weight read as stored)
  int a_gather_div, scatter;
  int N, K, align, n_tiles;
  const int32_t* seg_starts;
  const uint32_t* counts;
  const int32_t* tile_expert;
  const int32_t* row_slot;
  const int32_t* row_slot_out;
};

__device__ inline f32x16 zero_acc() {
  f32x16 c;
#pragma unroll
  for (int v = 0; v < 16; ++v) c[v] = 0.f;
  return c;
}

// one K slab of 16 from LDS: lane l feeds row / column l % 32 and contraction index l / 32 of each x2 step
__device__ inline void mfma_slab(const float (*As)[TK + 1], const float (*Bs)[TK + 1], int arow, int brow, int khalf, f32x16& acc) {
#pragma unroll
  for (int kk = 0; kk < TK / 2; ++kk) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[arow][2 * kk + khalf], Bs[brow][2 * kk + khalf], acc, 0, 0, 0);
}

// y[out_row(p), :] = a[a_row(p), :] @ W_e (+ bias_e) for every valid padded row p
__global__ __launch_bounds__(NT) void grouped_gemm_f32_kernel(const F32Params prm) {
  __shared__ float As[TM][TK + 1], Bs[TN][TK + 1];
  __shared__ int64_t a_rows[TM], out_rows[TM];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int mt = blockIdx.x / prm.n_tiles, nt = blockIdx.x % prm.n_tiles;
  const int64_t p0 = (int64_t)mt * TM;
  const int e = prm.tile_expert[p0 / prm.align];
  if (e < 0) return;
  const int64_t valid_end = (int64_t)prm.seg_starts[e] + prm.counts[e];
  if (p0 >= valid_end) return;  // a tile of pad rows
  if (tid < TM) {
    const int64_t p = p0 + tid;
    const bool ok = p < valid_end;
    a_rows[tid] = ok ? (prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p) : -1;
    out_rows[tid] = ok ? (prm.scatter ? (int64_t)prm.row_slot_out[p] : p) : -1;
  }
  __syncthreads();
  const float* w = prm.w + (int64_t)e * prm.w_expert_stride;
  const int n0 = nt * TN;
  f32x16 acc = zero_acc();
  for (int k0 = 0; k0 < prm.K; k0 += TK) {
    {  // A: 64 rows x 16 k, four consecutive k per thread (K % 4 == 0)
      const int r = tid >> 2, kq = (tid & 3) * 4;
      float4 v = {0.f, 0.f, 0.f, 0.f};
      if (a_rows[r] >= 0 && k0 + kq < prm.K) v = *reinterpret_cast<const float4*>(prm.a + a_rows[r] * prm.K + k0 + kq);
      As[r][kq] = v.x;
      As[r][kq + 1] = v.y;
      As[r][kq + 2] = v.z;
      As[r][kq + 3] = v.w;
    }
    if (!prm.w_is_kn) {  // w[n, k]: four consecutive k per thread
      const int n = tid >> 2, kq = (tid & 3) * 4;
      float4 v = {0.f, 0.f, 0.f, 0.f};
      if (n0 + n < prm.N && k0 + kq < prm.K) v = *reinterpret_cast<const float4*>(w + (int64_t)(n0 + n) * prm.K + k0 + kq);
      Bs[n][kq] = v.x;
      Bs[n][kq + 1] = v.y;
      Bs[n][kq + 2] = v.z;
      Bs[n][kq + 3] = v.w;
    } else {  // w[k, n]: four consecutive n per thread (N % 4 == 0)
      const int k = tid >> 4, nq = (tid & 15) * 4;
      float4 v = {0.f, 0.f, 0.f, 0.f};
      if (k0 + k < prm.K && n0 + nq < prm.N) v = *reinterpret_cast<const float4*>(w + (int64_t)(k0 + k) * prm.N + n0 + nq);
      Bs[nq][k] = v.x;
      Bs[nq + 1][k] = v.y;
      Bs[nq + 2][k] = v.z;
      Bs[nq + 3][k] = v.w;
    }
    __syncthreads();
    mfma_slab(As, Bs, wm * 32 + (lane & 31), wn * 32 + (lane & 31), lane >> 5, acc);
    __syncthreads();
  }
  // lane l holds column l % 32 and rows 8 (v / 4) + 4 (l / 32) + v % 4 of the wave's 32 x 32 block
  const int n = n0 + wn * 32 + (lane & 31);
  if (n >= prm.N) return;
  const float b = prm.bias != nullptr ? prm.bias[(int64_t)e * prm.N + n] : 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int r = wm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
    const int64_t orow = out_rows[r];
    if (orow >= 0) prm.y[orow * prm.N + n] = acc[v] + b;
  }
}

// dw[e] = a[rows of e]^T @ b[rows of e]; a [max_rows, M], b [max_rows, N] padded grouped rows; grid (tiles, E)
__global__ __launch_bounds__(NT) void grouped_gemm_dw_f32_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                  int M, int N, int n_tiles,
                                                                  const int32_t* __restrict__ seg_starts,
                                                                  const uint32_t* __restrict__ counts,
                                                                  float* __restrict__ dw) {
  __shared__ float As[TM][TK + 1], Bs[TN][TK + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int e = blockIdx.y;
  const int m0 = (blockIdx.x / n_tiles) * TM, n0 = (blockIdx.x % n_tiles) * TN;
  const int64_t start = seg_starts[e];
  const int cnt = (int)counts[e];
  f32x16 acc = zero_acc();
  for (int r0 = 0; r0 < cnt; r0 += TK) {
    const int r = tid >> 4, cq = (tid & 15) * 4;  // 16 rows x 64 columns of each operand, four columns per thread
    float4 va = {0.f, 0.f, 0.f, 0.f}, vb = {0.f, 0.f, 0.f, 0.f};
    if (r0 + r < cnt) {
      if (m0 + cq < M) va = *reinterpret_cast<const float4*>(a + (start + r0 + r) * M + m0 + cq);
      if (n0 + cq < N) vb = *reinterpret_cast<const float4*>(b + (start + r0 + r) * N + n0 + cq);
    }
    As[cq][r] = va.x;
    As[cq + 1][r] = va.y;
    As[cq + 2][r] = va.z;
    As[cq + 3][r] = va.w;
    Bs[cq][r] = vb.x;
    Bs[cq + 1][r] = vb.y;
    Bs[cq + 2][r] = vb.z;
    Bs[cq + 3][r] = vb.w;
    __syncthreads();
    mfma_slab(As, Bs, wm * 32 + (lane & 31), wn * 32 + (lane & 31), lane >> 5, acc);
    __syncthreads();
  }
  const int n = n0 + wn * 32 + (lane & 31);
  if (n >= N) return;
  float* out = dw + (int64_t)e * M * N;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m0 + wm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
    if (m < M) out[(int64_t)m * N + n] = acc[v];  // experts without rows get exact zeros
  }
}

int check_seg(const ck_segments* seg, const char* name) {
  CK_REQUIRE(seg && seg->seg_starts && seg->counts && seg->tile_expert && seg->row_slot, "%s: seg is incomplete", name);
  CK_REQUIRE(seg->align >= TM && seg->align % TM == 0 && seg->max_rows >= 0 && seg->max_rows % seg->align == 0 && seg->num_experts >= 1,
             "%s: align=%d must be a multiple of %d and max_rows a multiple of align", name, seg->align, TM);
  return CK_OK;
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_grouped_gemm_f32(const float* a, int32_t a_gather_div, const float* w, int32_t w_is_kn, int32_t N,
                                   int32_t K, const ck_segments* seg, int32_t scatter, float* y, const float* bias,
                                   void* stream) {
  const char* name = "ck_grouped_gemm_f32";
  if (int rc = check_seg(seg, name)) return rc;
  CK_REQUIRE(N >= 4 && K >= 4 && N % 4 == 0 && K % 4 == 0, "%s: N=%d and K=%d must be positive multiples of 4", name, N, K);
  CK_REQUIRE(a_gather_div >= 0, "%s: a_gather_div=%d is negative", name, a_gather_div);
  if (seg->max_rows == 0) return CK_OK;
  CK_REQUIRE(a && w && y && aligned16(a) && aligned16(w), "%s: NULL or misaligned pointer", name);
  F32Params prm = {};
  prm.a = a;
  prm.w = w;
  prm.bias = bias;
  prm.y = y;
  prm.w_expert_stride = (int64_t)N * K;
  prm.w_is_kn = w_is_kn != 0;
  prm.a_gather_div = a_gather_div;
  prm.scatter = scatter != 0;
  prm.N = N;
  prm.K = K;
  prm.align = seg->align;
  prm.n_tiles = (int)ceil_div(N, TN);
  prm.seg_starts = seg->seg_starts;
  prm.counts = seg->counts;
  prm.tile_expert = seg->tile_expert;
  prm.row_slot = seg->row_slot;
  prm.row_slot_out = seg->row_slot_out != nullptr ? seg->row_slot_out : seg->row_slot;
  const int64_t blocks = seg->max_rows / TM * prm.n_tiles;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  hipLaunchKernelGGL(grouped_gemm_f32_kernel, dim3((unsigned)blocks), dim3(NT), 0, static_cast<hipStream_t>(stream), prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int ck_grouped_gemm_dw_f32(const float* a, const float* b, int32_t M, int32_t N, const ck_segments* seg,
                                      float* dw, void* stream) {
  const char* name = "ck_grouped_gemm_dw_f32";
  if (int rc = check_seg(seg, name)) return rc;
  CK_REQUIRE(M >= 4 && N >= 4 && M % 4 == 0 && N % 4 == 0, "%s: M=%d and N=%d must be positive multiples of 4", name, M, N);
  CK_REQUIRE(seg->num_experts <= 65535, "%s: more than 65535 experts", name);
  CK_REQUIRE(dw != nullptr && (seg->max_rows == 0 || (a && b && aligned16(a) && aligned16(b))), "%s: NULL or misaligned pointer", name);
  const int n_tiles = (int)ceil_div(N, TN);
  const int64_t tiles = ceil_div(M, TM) * n_tiles;
  CK_REQUIRE(tiles < (int64_t)0x7fffffff, "%s: grid too large", name);
  hipLaunchKernelGGL(grouped_gemm_dw_f32_kernel, dim3((unsigned)tiles, (unsigned)seg->num_experts), dim3(NT), 0,
                     static_cast<hipStream_t>(stream), a, b, (int)M, (int)N, n_tiles, seg->seg_starts, seg->counts, dw);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}
