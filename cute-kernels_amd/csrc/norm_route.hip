// RMSNorm fused ahead of the router: one pass over x that writes the normalised rows, rstd, the router logits
// gate(rmsnorm(x)) and, for the quantised-expert path, the e4m3 rows with their per-row scales.
//
// Replaces, as one kernel: rmsnorm_forward_triton (cute_kernels/kernels/rmsnorm/triton_implementation/forward.py:14-53),
// the router's nn.Linear (cute_kernels/kernels/scattermoe/torch_implementation.py:122-124) and the per-row quantiser
// ahead of the fp8 expert GEMMs.
//
// A workgroup (4 waves) owns 16 rows and keeps them in registers from the first load to the last store: wave w holds
// columns [w H/4, (w+1) H/4) of the 16 rows, already in the operand layout of v_mfma_f32_16x16x32 (lane l: row l % 16,
// four 8-element pieces per 128-column step, 32 columns apart). Sum of squares -> rstd (shuffles inside a
// wave, LDS across the four waves), y = round((x * rstd) * w) in place, stores of y (and of the e4m3 row after a second
// reduction for the row maximum), then the logits: the normalised 16-bit values are the first MFMA operand's partner,
// the gate weight's rows stream from L2 straight into the other operand's registers (lane l: expert 16 j + l % 16, the
// same columns -- the contraction only needs both operands to agree on which column sits where), each wave
// accumulates its quarter of the contraction, and the four partial [16 x E] blocks are summed through LDS in a fixed
// order. x is read once; the gate weight (E x H, at most 1 MiB; re-ordered first by a small kernel so that those loads are
// contiguous) is read once per 16 rows from L2, which is what bounds the kernel at E = 128, H = 4096 (three workgroups per
// CU overlap one's loads and stores with the others' MFMAs).
// The logits are those of the 16-bit normalised rows, exactly what a linear layer applied to the stored y computes
// (fp32 accumulation, another summation order).
#include "gemm_common.h"

namespace ck {
namespace {

constexpr int kRows = 16;            // rows per workgroup: one MFMA row block
constexpr int kWaves = 4, kNT = kWaves * kWave;
constexpr int kMaxExperts = 128;
constexpr float kE4M3Max = 448.0f;

template <typename T>
__device__ inline float dot2_acc(uint32_t pair, float acc);  // acc + lo * lo + hi * hi of a packed pair
template <>
__device__ inline float dot2_acc<bf16_t>(uint32_t pair, float acc) {
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  const v2bf v = __builtin_bit_cast(v2bf, pair);
  return __builtin_amdgcn_fdot2_f32_bf16(v, v, acc, false);
}
template <>
__device__ inline float dot2_acc<f16_t>(uint32_t pair, float acc) {
  typedef _Float16 v2h __attribute__((ext_vector_type(2)));
  const v2h v = __builtin_bit_cast(v2h, pair);
  return __builtin_amdgcn_fdot2(v, v, acc, false);
}
__device__ inline uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  typedef unsigned short v2us __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2us, a), __builtin_bit_cast(v2us, b)));
}
template <typename T>
__device__ inline float half_bits_to_float(uint32_t bits) {
  return Elem<T>::up(__builtin_bit_cast(T, (unsigned short)bits));
}

// The gate weight in the order the main kernel's lanes consume it: packed[j][w][t][s][lane] = the 8 elements
// G[16 j + lane % 16][w H/4 + 128 t + 32 s + 8 (lane / 16) ..], so that every load instruction of a wave reads 1 KiB of
// consecutive bytes. Read as stored, the 16 rows of one instruction lie a whole row pitch apart (8 KiB at H = 4096): they
// fall into the same L2 channel and every CU asks for the same lines at once, which measured 10 TB/s chip-wide instead
// of the 30+ TB/s L2 delivers on consecutive lines. Experts past E repeat the last one (their logits are not stored).
template <typename T>
__global__ __launch_bounds__(256) void pack_gate_kernel(const T* __restrict__ gate_w, int E, int H, T* __restrict__ packed) {
  const int S = H / 512;
  const int64_t pieces = (int64_t)((E + 15) / 16) * 4 * S * 4 * kWave;
  for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < pieces; p += (int64_t)gridDim.x * blockDim.x) {
    const int lane = (int)(p % kWave);
    int64_t rest = p / kWave;
    const int s = (int)(rest % 4);
    rest /= 4;
    const int t = (int)(rest % S);
    rest /= S;
    const int w = (int)(rest % 4);
    const int j = (int)(rest / 4);
    const int e = min(16 * j + (lane & 15), E - 1);
    const int col = w * (H / 4) + 128 * t + 32 * s + 8 * (lane >> 4);
    store16(packed + p * 8, load16(gate_w + (int64_t)e * H + col));
  }
}

// S: 128-column steps per wave (H = 512 S); W: with a norm weight
template <typename T, int S, bool W>
__global__ __launch_bounds__(kNT, 3) void rmsnorm_route_kernel(const T* __restrict__ x, const T* __restrict__ norm_w,
                                                                const T* __restrict__ gate_packed, float eps, int64_t B, int E,
                                                                T* __restrict__ y, float* __restrict__ rstd_out,
                                                                T* __restrict__ logits, uint8_t* __restrict__ x8,
                                                                float* __restrict__ scale8) {
  constexpr int H = 512 * S;
  __shared__ float part[kWaves][kRows][kMaxExperts];  // partial logits of the four column quarters
  __shared__ float red[2][kWaves][kRows];             // per-wave row sums of squares / row maxima
  __shared__ __attribute__((aligned(16))) T w_lds[W ? H : 8];  // the norm weight: read by all 16 rows of every wave
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane & 15, q = lane >> 4;
  const int64_t row0 = (int64_t)blockIdx.x * kRows;
  const int64_t row = row0 + r;
  const bool row_ok = row < B;
  const int64_t row_ld = row_ok ? row : B - 1;  // rows past the end re-read the last row; nothing of theirs is stored
  // this lane's first column; step t adds 128 t, piece s adds 32 s: the four lanes of a row then cover 64 contiguous
  // bytes with every load / store instruction (the operand layout of the MFMA itself)
  const int col0 = wave * (H / 4) + 8 * q;

  if constexpr (W) {
    for (int c = tid; c < H / 8; c += kNT) *reinterpret_cast<vec16*>(&w_lds[8 * c]) = load16(norm_w + 8 * c);
  }  // visible after the barrier of the rstd reduction

  // ---- the 16 x H/4 block of x, in registers
  vec16 xa[S][4];
  const T* xr = x + row_ld * H + col0;
#pragma unroll
  for (int t = 0; t < S; ++t)
#pragma unroll
    for (int s = 0; s < 4; ++s) xa[t][s] = load16_nt(xr + t * 128 + 32 * s);

  // ---- rstd; the sum of squares straight from the packed pairs (v_dot2_f32_bf16 / v_dot2_f32_f16)
  float ss = 0.f;
#pragma unroll
  for (int t = 0; t < S; ++t)
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) ss = dot2_acc<T>(xa[t][s].w[i], ss);
  ss += __shfl_xor(ss, 16, kWave);
  ss += __shfl_xor(ss, 32, kWave);
  if (q == 0) red[0][wave][r] = ss;
  __syncthreads();
  ss = red[0][0][r] + red[0][1][r] + red[0][2][r] + red[0][3][r];
  const float rs = rsqrtf(ss * (1.0f / (float)H) + eps);
  if (rstd_out != nullptr && wave == 0 && q == 0 && row_ok) rstd_out[row] = rs;

  // ---- y = round((x * rstd) * w), in place; the row maximum for the e4m3 scale is taken on the packed bit patterns
  // (magnitudes of 16-bit floats order like unsigned integers)
  uint32_t amax_bits = 0;
#pragma unroll
  for (int t = 0; t < S; ++t) {
    vec16 wv[4];
    if constexpr (W) {
#pragma unroll
      for (int s = 0; s < 4; ++s) wv[s] = *reinterpret_cast<const vec16*>(&w_lds[col0 + t * 128 + 32 * s]);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      Pack16<T> p, w;
      p.v = xa[t][s];
      if constexpr (W) w.v = wv[s];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v0 = Elem<T>::up(p.e[2 * i]) * rs, v1 = Elem<T>::up(p.e[2 * i + 1]) * rs;
        if constexpr (W) {
          v0 *= Elem<T>::up(w.e[2 * i]);
          v1 *= Elem<T>::up(w.e[2 * i + 1]);
        }
        const uint32_t packed = pack_pair<T>(v0, v1);
        xa[t][s].w[i] = packed;
        amax_bits = pk_max_u16(amax_bits, packed & 0x7fff7fffu);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // step by step: four weight pieces and their temporaries live at a time
  }
  if (row_ok) {
    T* yr = y + row * H + col0;
#pragma unroll
    for (int t = 0; t < S; ++t)
#pragma unroll
      for (int s = 0; s < 4; ++s) store16(yr + t * 128 + 32 * s, xa[t][s]);  // cached: L2 merges the 64-byte halves of a line
  }

  // ---- e4m3 row and scale, as ck_quant_rows_e4m3 computes them from the stored y
  if (x8 != nullptr) {
    float amax = fmaxf(half_bits_to_float<T>(amax_bits & 0xffffu), half_bits_to_float<T>(amax_bits >> 16));
    amax = fmaxf(amax, __shfl_xor(amax, 16, kWave));
    amax = fmaxf(amax, __shfl_xor(amax, 32, kWave));
    if (q == 0) red[1][wave][r] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[1][0][r], red[1][1][r]), fmaxf(red[1][2][r], red[1][3][r]));
    const float inv = amax > 0.f ? kE4M3Max / amax : 1.0f;
    if (wave == 0 && q == 0 && row_ok) scale8[row] = amax > 0.f ? amax / kE4M3Max : 1.0f;
    if (row_ok) {
      uint8_t* qr = x8 + row * H + col0;
#pragma unroll
      for (int t = 0; t < S; ++t) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {  // 8 elements -> 8 bytes; the four lanes of a row write 32 contiguous bytes
          Pack16<T> a;
          a.v = xa[t][s];
          int lo = 0, hi = 0;
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(a.e[0]) * inv, Elem<T>::up(a.e[1]) * inv, lo, false);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(a.e[2]) * inv, Elem<T>::up(a.e[3]) * inv, lo, true);
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(a.e[4]) * inv, Elem<T>::up(a.e[5]) * inv, hi, false);
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(a.e[6]) * inv, Elem<T>::up(a.e[7]) * inv, hi, true);
          *reinterpret_cast<uint2*>(qr + t * 128 + 32 * s) = uint2{(uint32_t)lo, (uint32_t)hi};
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- logits: block j of 16 experts at a time; gate-weight rows go from L2 into the second operand's registers,
  // one step (4 pieces = 64 bytes per lane) ahead of the MFMAs that use them
  const int n_blocks = (E + 15) / 16;
  auto load_gate = [&](int j, int t, vec16 (&g)[4]) {  // see pack_gate_kernel for the order
    const T* gp = gate_packed + ((int64_t)((j * 4 + wave) * S + t) * 4 * kWave + lane) * 8;
#pragma unroll
    for (int s = 0; s < 4; ++s) g[s] = load16(gp + s * kWave * 8);
  };
  auto frag = [](const vec16& v) {
    union {
      vec16 v;
      typename Mfma16<T>::frag f;
    } u;
    u.v = v;
    return u.f;
  };
  vec16 g[2][4];
  load_gate(0, 0, g[0]);
  // expert block j; jj = j % 2 makes the parity of the running step index (j S + t) a constant expression
  auto expert_block = [&](int j, auto jj) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    static_for<S>([&](auto t) {
      constexpr int par = ((int)jj * S + (int)t) & 1;
      constexpr bool last = (int)t == S - 1;
      if (!last || j + 1 < n_blocks) load_gate(last ? j + 1 : j, last ? 0 : (int)t + 1, g[par ^ 1]);
      // the gate fragment is the first operand: a lane then holds 4 consecutive experts of one row
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = Mfma16<T>::run(frag(g[par][s]), frag(xa[(int)t][s]), acc);
      __builtin_amdgcn_sched_barrier(0);  // keeps the prefetch one step ahead, not S steps
    });
    *reinterpret_cast<f32x4*>(&part[wave][r][16 * j + 4 * q]) = acc;  // experts 16 j + 4 q .. + 3 of row r
  };
  for (int j = 0; j < n_blocks; j += 2) {
    expert_block(j, std::integral_constant<int, 0>{});
    if (j + 1 < n_blocks) expert_block(j + 1, std::integral_constant<int, 1>{});
  }
  __syncthreads();

  // ---- sum the four partial blocks (fixed order), round, store: thread -> row tid / 16, experts 8 (tid % 16) .. + 7
  {
    const int orow = tid >> 4, e0 = (tid & 15) * 8;
    const int64_t grow = row0 + orow;
    if (grow < B && e0 < E) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (part[0][orow][e0 + i] + part[1][orow][e0 + i]) + (part[2][orow][e0 + i] + part[3][orow][e0 + i]);
      T* out = logits + grow * E + e0;
      if (e0 + 8 <= E && (E & 7) == 0) {
        Pack16<T> p;
#pragma unroll
        for (int i = 0; i < 8; ++i) p.e[i] = Elem<T>::down(v[i]);
        store16(out, p.v);
      } else {
        for (int i = 0; i < 8 && e0 + i < E; ++i) out[i] = Elem<T>::down(v[i]);
      }
    }
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_rmsnorm_route(const void* x, const void* norm_weight, const void* gate_weight, float eps, int64_t B,
                                int32_t H, int32_t E, void* y, float* rstd, void* logits, void* x8, float* scale8,
                                void* gate_packed, int32_t dtype, void* stream) {
  const char* name = "ck_rmsnorm_route";
  CK_REQUIRE(B >= 0, "%s: negative row count", name);
  CK_REQUIRE(H >= 512 && H <= 4096 && H % 512 == 0, "%s: H=%d must be a multiple of 512, at most 4096", name, H);
  CK_REQUIRE(E >= 1 && E <= kMaxExperts, "%s: E=%d must be in [1, %d]", name, E, kMaxExperts);
  if (B == 0) return CK_OK;
  CK_REQUIRE(x && gate_weight && y && logits && gate_packed, "%s: x, gate_weight, y, logits and gate_packed are required", name);
  CK_REQUIRE((x8 == nullptr) == (scale8 == nullptr), "%s: x8 and scale8 go together", name);
  CK_REQUIRE(aligned16(x) && aligned16(gate_weight) && aligned16(y) && aligned16(gate_packed) && (norm_weight == nullptr || aligned16(norm_weight)) &&
                 (x8 == nullptr || aligned16(x8)) && ((E & 7) != 0 || aligned16(logits)),
             "%s: pointers must be 16-byte aligned", name);
  const int64_t blocks = ceil_div(B, kRows);
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CK_NR_W(S, W)                                                                                                     \
  hipLaunchKernelGGL((rmsnorm_route_kernel<scalar_t, S, W>), dim3((unsigned)blocks), dim3(kNT), 0, s,                     \
                     static_cast<const scalar_t*>(x), static_cast<const scalar_t*>(norm_weight),                          \
                     static_cast<const scalar_t*>(gate_packed), eps, B, (int)E, static_cast<scalar_t*>(y), rstd,          \
                     static_cast<scalar_t*>(logits), static_cast<uint8_t*>(x8), scale8)
#define CK_NR(S)                           \
  do {                                     \
    if (norm_weight != nullptr) CK_NR_W(S, true); \
    else CK_NR_W(S, false);                \
  } while (0)
  CK_DISPATCH_HALF(dtype, name, {
    const int64_t pieces = ceil_div(E, 16) * 4 * (H / 512) * 4 * kWave;
    hipLaunchKernelGGL((pack_gate_kernel<scalar_t>), dim3((unsigned)ceil_div(pieces, 256)), dim3(256), 0, s,
                       static_cast<const scalar_t*>(gate_weight), (int)E, (int)H, static_cast<scalar_t*>(gate_packed));
    switch (H / 512) {
      case 1: CK_NR(1); break;
      case 2: CK_NR(2); break;
      case 3: CK_NR(3); break;
      case 4: CK_NR(4); break;
      case 5: CK_NR(5); break;
      case 6: CK_NR(6); break;
      case 7: CK_NR(7); break;
      default: CK_NR(8); break;
    }
  });
#undef CK_NR
#undef CK_NR_W
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}
