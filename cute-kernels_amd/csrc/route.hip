// Router: top-k over the logits of one token + softmax over the k selected logits, and its backward.
//
// A token is owned by a group of G lanes (a power of two, chosen on the host); each lane keeps ceil(E / G) logits in registers as
// 64-bit keys (order-preserving float bits in the high word, ~expert index in the low word), so "largest value, lowest
// expert index on ties" is a plain integer max that a butterfly of lane shuffles reduces in log2(G) steps.
#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxPerLane = 16;  // E <= 64 * 16
constexpr int kMaxTopK = 32;

__device__ inline uint32_t float_order_bits(float v) {
  if (v != v) return 0xffffffffu;  // NaN sorts above everything, as torch does
  v += 0.0f;                       // -0.0 -> +0.0 so that the two zeros tie
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

template <typename T, int PER>
__global__ __launch_bounds__(kBlock) void route_topk_softmax_kernel(const T* __restrict__ logits, int64_t T_tokens,
                                                                     int E, int k, int G, int32_t* __restrict__ selected,
                                                                     float* __restrict__ gates, T* __restrict__ topk_values) {
  const int lane_in_group = threadIdx.x & (G - 1);
  const int64_t token = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / G;
  const bool live = token < T_tokens;
  const T* row = logits + (live ? token : 0) * (int64_t)E;

  uint64_t key[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int e = p * G + lane_in_group;  // consecutive lanes read consecutive experts
    key[p] = 0ull;                        // below every real key (real keys have a non-zero low word or high word)
    if (live && e < E) {
      const float v = Elem<T>::up(row[e]);
      key[p] = ((uint64_t)float_order_bits(v) << 32) | (uint32_t)(0xffffffffu - (uint32_t)e);
    }
  }

  float vmax = 0.f, denom = 0.f;
  for (int j = 0; j < k; ++j) {
    uint64_t best = 0ull;
#pragma unroll
    for (int p = 0; p < PER; ++p) best = key[p] > best ? key[p] : best;
    for (int off = G >> 1; off > 0; off >>= 1) {
      const uint32_t lo = __shfl_xor((uint32_t)best, off, kWave);
      const uint32_t hi = __shfl_xor((uint32_t)(best >> 32), off, kWave);
      const uint64_t other = ((uint64_t)hi << 32) | lo;
      best = other > best ? other : best;
    }
    const uint32_t e = 0xffffffffu - (uint32_t)best;
#pragma unroll
    for (int p = 0; p < PER; ++p)
      if (key[p] == best) key[p] = 0ull;  // keys are unique (they embed the expert index)
    float v = 0.f;
    if (live) v = Elem<T>::up(row[e < (uint32_t)E ? e : 0]);
    if (j == 0) vmax = v;
    const float ex = expf(v - vmax);
    denom += ex;
    if (live && lane_in_group == 0) {
      gates[token * k + j] = ex;  // normalised below by the same lane
      selected[token * k + j] = (int32_t)e;
      if (topk_values) topk_values[token * k + j] = Elem<T>::down(v);
    }
  }
  if (live && lane_in_group == 0) {
    for (int j = 0; j < k; ++j) gates[token * k + j] = gates[token * k + j] / denom;
  }
}

// d_values = g * (d_g - sum_i g_i d_g_i); scattered into an otherwise zero row of d_logits. One group of G lanes per token.
// d_gates_rounded (optional): the gradient as it arrived in the 16-bit type. Where it is d_gates rounded to that type,
// the unrounded d_gates is used, elsewhere (something scaled or replaced the gradient on its way) the value that arrived.
template <typename T>
__global__ __launch_bounds__(kBlock) void route_bwd_kernel(const float* __restrict__ gates, const float* __restrict__ d_gates,
                                                            const T* __restrict__ d_gates_rounded,
                                                            const int32_t* __restrict__ selected, int64_t T_tokens, int E,
                                                            int k, T* __restrict__ d_logits) {
  const int64_t token = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (token >= T_tokens) return;
  const int lane = threadIdx.x & (kWave - 1);
  auto d_gate = [&](int j) {
    const float exact = d_gates[token * k + j];
    if (d_gates_rounded == nullptr) return exact;
    const float arrived = Elem<T>::up(d_gates_rounded[token * k + j]);
    return Elem<T>::up(Elem<T>::down(exact)) == arrived ? exact : arrived;
  };
  float dot = 0.f;
  for (int j = 0; j < k; ++j) dot += gates[token * k + j] * d_gate(j);
  for (int e = lane; e < E; e += kWave) {
    float d = 0.f;
    for (int j = 0; j < k; ++j) {
      if (selected[token * k + j] == e) {
        const float g = gates[token * k + j];
        d += g * (d_gate(j) - dot);
      }
    }
    d_logits[token * (int64_t)E + e] = Elem<T>::down(d);
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_route_topk_softmax(const void* logits, int32_t dtype, int64_t T, int32_t E, int32_t k,
                                     int32_t* selected, float* gates, void* topk_values, void* stream) {
  CK_REQUIRE(E >= 1 && E <= kWave * kMaxPerLane, "ck_route_topk_softmax: E=%d outside [1, %d]", E, kWave * kMaxPerLane);
  CK_REQUIRE(k >= 1 && k <= E && k <= kMaxTopK, "ck_route_topk_softmax: k=%d outside [1, min(E, %d)]", k, kMaxTopK);
  CK_REQUIRE(T >= 0, "ck_route_topk_softmax: T is negative");
  if (T == 0) return CK_OK;
  CK_REQUIRE(logits && selected && gates, "ck_route_topk_softmax: logits, selected and gates are required");
  // Lanes per token: as few as keep at most 8 logits per lane (fewer lanes = fewer shuffle rounds per selection and more
  // tokens per wave; measured at T = 65,536, E = 128, k = 8: 85 us with a whole wave per token). Wide rows fall back to
  // whole waves with up to 16 logits per lane.
  int G = 1;
  while (G < kWave && (E + G - 1) / G > 8) G <<= 1;
  const int per = (E + G - 1) / G;
  const int64_t blocks = ceil_div(T * G, kBlock);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CK_LAUNCH_ROUTE(PER)                                                                                      \
  hipLaunchKernelGGL((route_topk_softmax_kernel<scalar_t, PER>), dim3((unsigned)blocks), dim3(kBlock), 0, s,      \
                     static_cast<const scalar_t*>(logits), T, (int)E, (int)k, G, selected, gates,                 \
                     static_cast<scalar_t*>(topk_values))
  CK_DISPATCH_FLOAT(dtype, "ck_route_topk_softmax", {
    if (per == 1) CK_LAUNCH_ROUTE(1);
    else if (per == 2) CK_LAUNCH_ROUTE(2);
    else if (per <= 4) CK_LAUNCH_ROUTE(4);
    else if (per <= 8) CK_LAUNCH_ROUTE(8);
    else CK_LAUNCH_ROUTE(16);
  });
#undef CK_LAUNCH_ROUTE
  CK_CHECK_LAUNCH("ck_route_topk_softmax");
  return CK_OK;
}

static int route_bwd_impl(const char* name, const float* gates, const float* d_gates, const void* d_gates_rounded,
                          const int32_t* selected, int64_t T, int32_t E, int32_t k, void* d_logits, int32_t dtype,
                          void* stream) {
  CK_REQUIRE(E >= 1 && k >= 1 && k <= E && T >= 0, "%s: bad sizes T=%lld E=%d k=%d", name, (long long)T, E, k);
  if (T == 0) return CK_OK;
  CK_REQUIRE(gates && d_gates && selected && d_logits, "%s: NULL argument", name);
  const int64_t blocks = ceil_div(T, kBlock / kWave);
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_FLOAT(dtype, name, {
    hipLaunchKernelGGL((route_bwd_kernel<scalar_t>), dim3((unsigned)blocks), dim3(kBlock), 0, s, gates, d_gates,
                       static_cast<const scalar_t*>(d_gates_rounded), selected, T, (int)E, (int)k,
                       static_cast<scalar_t*>(d_logits));
  });
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int ck_route_topk_softmax_bwd(const float* gates, const float* d_gates, const int32_t* selected, int64_t T,
                                         int32_t E, int32_t k, void* d_logits, int32_t dtype, void* stream) {
  return route_bwd_impl("ck_route_topk_softmax_bwd", gates, d_gates, nullptr, selected, T, E, k, d_logits, dtype, stream);
}

extern "C" int ck_route_topk_softmax_bwd_exact(const float* gates, const float* d_gates_exact, const void* d_gates,
                                               const int32_t* selected, int64_t T, int32_t E, int32_t k, void* d_logits,
                                               int32_t dtype, void* stream) {
  const char* name = "ck_route_topk_softmax_bwd_exact";
  CK_REQUIRE(T == 0 || d_gates != nullptr, "%s: d_gates is required", name);
  CK_REQUIRE(dtype != CK_F32, "%s: d_gates of a 16-bit type (fp32 gradients go to ck_route_topk_softmax_bwd)", name);
  return route_bwd_impl(name, gates, d_gates_exact, d_gates, selected, T, E, k, d_logits, dtype, stream);
}
