// Scattered grouped GEMM with fp8 e4m3 operands (OCP e4m3fn on gfx950), fp32 accumulation, bf16 / f16 output.
// Forward (inference) only: Y = (A_e * diag(a_scale)) (W[e] * diag(w_scale[e]))^T, the two scale vectors applied to the
// fp32 accumulators in the epilogue.
//
// Same machinery as the 16-bit kernel (tile-aligned expert segments, 256x256 tile, 8 waves, global -> LDS direct loads,
// four XOR-swizzled 64-byte-row stages, hand-ordered load / fragment-read / MFMA stream, LDS-staged epilogue), with one
// byte per element: a K step is 64 elements = four 16-wide slices of v_mfma_f32_32x32x16_fp8_fp8, fragments are 8 bytes
// per lane, and every byte fetched from L2 carries twice the FLOPs.
#include <stdlib.h>

#include "gemm_common.h"

namespace ck {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WGM = 4, NW = WGM * 2, NT = 64 * NW;  // 8 waves: 4 along M, 2 along N
constexpr int WM = BM / WGM, WN = BN / 2;           // 64 x 128 wave tile
constexpr int MI = WM / 32, NI = WN / 32;
constexpr int BK = 64, KS = BK / 16, NSTAGE = 4;
constexpr int kRowBytes = 64;
constexpr int kStageBytes = (BM + BN) * kRowBytes;
constexpr int A_LD = BM / (16 * NW), B_LD = BN / (16 * NW);
constexpr int kLoadsPerStep = A_LD + B_LD, kReads = MI + NI, kMfma = MI * NI;
constexpr size_t kLdsBytes = (size_t)NSTAGE * kStageBytes;

template <typename TO, int MODE>
__global__ __launch_bounds__(NT) void grouped_gemm_fp8_kernel(const GemmParams prm) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  char* lds_c = reinterpret_cast<char*>(lds_raw);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile (same XCD-aware order as the 16-bit kernel)
  const int live_m = prm.seg_starts[prm.num_experts] / prm.align;
  const int total = live_m * prm.n_tiles;
  int pid = blockIdx.x;
  if (pid >= total) return;
  const int per_xcd = total / kXcds;
  if (pid < per_xcd * kXcds) pid = (pid % kXcds) * per_xcd + pid / kXcds;
  int mt, nt;
  grouped_order(pid, live_m, prm.n_tiles, mt, nt);
  const int expert = prm.tile_expert[mt];
  const int64_t m0 = (int64_t)mt * BM;
  const int64_t valid_end = (int64_t)prm.seg_starts[expert] + prm.counts[expert];

  f32x16 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- global -> LDS addressing: lane l of a wave-load fills slot l (16 bytes) of 64 consecutive slots = 16 rows
  const char* a_base = static_cast<const char*>(prm.a);
  const char* b_base = static_cast<const char*>(prm.w) + (int64_t)expert * prm.w_expert_stride;
  uint32_t a_off[A_LD], b_off[B_LD];
#pragma unroll
  for (int t = 0; t < A_LD; ++t) {
    const int r = (wave * A_LD + t) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ lds_swizzle(r);
    int64_t p = m0 + r;
    if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
    const int64_t row = prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p;
    a_off[t] = (uint32_t)(row * prm.lda + c * 16);
  }
#pragma unroll
  for (int t = 0; t < B_LD; ++t) {
    const int j = (wave * B_LD + t) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ lds_swizzle(j);
    int64_t n;
    if constexpr (MODE == kSwiglu) {
      const int half = (j % WN) / (WN / 2);
      const int within = (j / WN) * (WN / 2) + (j % (WN / 2));
      n = (int64_t)half * prm.I + min((int64_t)nt * (BN / 2) + within, (int64_t)prm.I - 1);
    } else {
      n = min((int64_t)nt * BN + j, (int64_t)prm.N - 1);
    }
    b_off[t] = (uint32_t)(n * prm.ldw + c * 16);
  }
  const int nk = prm.K / BK;

  auto dma16 = [&](const char* src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "m0");
  };
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_c;
  const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * A_LD * 1024);
  const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * kRowBytes + wave * B_LD * 1024);
  auto issue_one = [&](int step, int g) {
    const int64_t kb = (int64_t)min(step, nk - 1) * kRowBytes;  // past the end: re-fetch the last step (never read)
    const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
    if (g < A_LD) dma16(a_base + kb + a_off[g], wave_a + st + g * 1024);
    else dma16(b_base + kb + b_off[g - A_LD], wave_b + st + (g - A_LD) * 1024);
  };
  auto issue = [&](int step) {
#pragma unroll
    for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
  };

  // ---- fragments: slice sl of a row is its 16-byte chunk sl; lanes 0-31 take its first 8 bytes, lanes 32-63 the rest
  const int fsw = lds_swizzle(lane & 31), fh = lane >> 5;
  int slice_off[KS];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) slice_off[sl] = ((sl ^ fsw) * 16) + fh * 8;
  const int fa_row = (wm * WM + (lane & 31)) * kRowBytes;
  const int fb_row = BM * kRowBytes + (wn * WN + (lane & 31)) * kRowBytes;
  long fa[2][MI], fb[2][NI];
  auto read_one = [&](int stage, int sl, int buf, int g) {
    const char* st = lds_c + stage * kStageBytes + slice_off[sl];
    if (g < MI) fa[buf][g] = *reinterpret_cast<const long*>(st + fa_row + g * 32 * kRowBytes);
    else fb[buf][g - MI] = *reinterpret_cast<const long*>(st + fb_row + (g - MI) * 32 * kRowBytes);
  };
  auto read_nth = [&](int stage, int sl, int buf, int n) {  // A0, every B block, then the remaining A blocks
    const int g = n == 0 ? 0 : (n <= NI ? MI + n - 1 : n - NI);
    read_one(stage, sl, buf, g);
  };
  auto mfma_range = [&](int buf, int first, int last) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
        if (i * NI + j >= first && i * NI + j < last)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(fa[buf][i], fb[buf][j], acc[i][j], 0, 0, 0);
  };
  auto mfma_begin = [](int g) { return g * kMfma / kReads; };
  static_assert(kLoadsPerStep <= kReads, "every load of a step has a slot in the last slice");

  if (nk > 0) {
    issue(0);
    issue(1);
    issue(2);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * kLoadsPerStep) : "memory");  // step 0 landed, all waves
#pragma unroll
    for (int g = 0; g < kReads; ++g) read_one(0, 0, 0, g);
    for (int kt = 0; kt < nk; ++kt) {
      const int stage = kt & (NSTAGE - 1);
      // slices 0 .. KS-2: their MFMAs hide the fragment reads of the next slice
#pragma unroll
      for (int sl = 0; sl + 1 < KS; ++sl) {
#pragma unroll
        for (int g = 0; g < kReads; ++g) {
          read_nth(stage, sl + 1, (sl + 1) & 1, g);
          mfma_range(sl & 1, mfma_begin(g), mfma_begin(g + 1));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // step kt + 1 has landed for every wave (only step kt + 2 may be in flight); the barrier also orders the
      // overwrite of stage (kt + 3) % 4, last read in step kt - 1
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLoadsPerStep) : "memory");
      // last slice: hides the loads of step kt + 3 and the slice-0 fragment reads of step kt + 1
#pragma unroll
      for (int g = 0; g < kReads; ++g) {
        if (g < kLoadsPerStep) issue_one(kt + 3, g);
        read_nth((kt + 1) & (NSTAGE - 1), 0, 0, g);
        mfma_range((KS - 1) & 1, mfma_begin(g), mfma_begin(g + 1));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- epilogue through LDS (see the 16-bit kernel): slab S[col][row] of 128 tile columns, 8-byte writes from the
  // accumulator layout, ds_read_b64_tr_b16 back out so that a lane stores 8 consecutive columns of one row
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  constexpr int kSlabCols = 128, kSlabLd = BM + 4;
  TO* slab = reinterpret_cast<TO*>(lds_raw);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  const int col_in_block = lane & 31;
  const int row_quad = (lane >> 5) * 4;
  const TO kZero = Elem<TO>::down(0.f);

  // dequantisation scales of the rows this lane holds
  float rs[MI][4][4];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int64_t p = m0 + wm * WM + i * 32 + 8 * q + row_quad + s;
        float v = 0.f;
        if (p < valid_end) v = prm.a_scale[prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p];
        rs[i][q][s] = v;
      }

  auto stage_blocks = [&](auto&& value) {
    static_for<MI>([&](auto i) {
      static_for<2>([&](auto jj) {
        static_for<4>([&](auto q) {
          const int r = wm * WM + i * 32 + 8 * q + row_quad;
          const int c = wn * 64 + jj * 32 + col_in_block;
          store4(slab + c * kSlabLd + r, value(i, jj, q, std::integral_constant<int, 0>{}),
                 value(i, jj, q, std::integral_constant<int, 1>{}), value(i, jj, q, std::integral_constant<int, 2>{}),
                 value(i, jj, q, std::integral_constant<int, 3>{}));
        });
      });
    });
  };
  auto drain_rows = [&](auto&& out_ptr) {
    const int l16 = tid & 15, grp = tid >> 4;
    const int tq = l16 & 3, tj = l16 >> 2;
    const int oq = l16 >> 2, oe = l16 & 3;
    constexpr int kBlocks = (BM / 4) * (kSlabCols / 32);
#pragma unroll 4
    for (int b = grp; b < kBlocks; b += NT / 16) {
      const int rb = b >> 2, cb = b & 3;
      const TO* src = slab + (cb * 32 + 8 * tq + tj) * kSlabLd + rb * 4;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src + 4 * kSlabLd));
      TO* dst = out_ptr(rb * 4 + oe, cb * 32 + 8 * oq);
      if (dst != nullptr) {
        vec16 v;
        v.w[0] = (uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
        v.w[1] = (uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
        v.w[2] = (uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
        v.w[3] = (uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
        store16(dst, v);
      }
    }
  };
  const float* w_scale = prm.w_scale + (int64_t)expert * prm.N;

  if constexpr (MODE == kGrouped || MODE == kScatter) {
    TO* y = static_cast<TO*>(prm.y);
    static_for<2>([&](auto pass) {
      float cs[2];
      static_for<2>([&](auto jj) {
        const int64_t n = (int64_t)nt * BN + wn * WN + (pass * 2 + jj) * 32 + col_in_block;
        cs[jj] = n < prm.N ? w_scale[n] : 0.f;
      });
      stage_blocks([&](auto i, auto jj, auto q, auto s) {
        return Elem<TO>::down(acc[i][pass * 2 + jj][4 * q + s] * rs[i][q][s] * cs[jj]);
      });
      __syncthreads();
      drain_rows([&](int r, int sc) -> TO* {
        const int64_t p = m0 + r, n = (int64_t)nt * BN + (sc >> 6) * WN + pass * 64 + (sc & 63);
        if (p >= valid_end || n >= prm.N) return nullptr;
        const int64_t row = (MODE == kScatter) ? (int64_t)prm.row_slot[p] : p;
        return y + row * prm.N + n;
      });
      __syncthreads();
    });
  } else {  // kSwiglu: blocks 0, 1 = up, blocks 2, 3 = gate of the same activation columns; only the activation is kept
    TO* act = static_cast<TO*>(prm.aux);
    float cs_up[2], cs_gate[2];
    static_for<2>([&](auto jj) {
      const int64_t col = (int64_t)nt * (BN / 2) + wn * (WN / 2) + jj * 32 + col_in_block;
      cs_up[jj] = col < prm.I ? w_scale[col] : 0.f;
      cs_gate[jj] = col < prm.I ? w_scale[prm.I + col] : 0.f;
    });
    stage_blocks([&](auto i, auto jj, auto q, auto s) {
      // rounded to the output type first, like a pre-activation tensor would be
      const TO up = Elem<TO>::down(acc[i][jj][4 * q + s] * rs[i][q][s] * cs_up[jj]);
      const TO gate = Elem<TO>::down(acc[i][jj + 2][4 * q + s] * rs[i][q][s] * cs_gate[jj]);
      const float gf = Elem<TO>::up(gate);
      return Elem<TO>::down(Elem<TO>::up(up) * gf * sigmoid_fast(gf));
    });
    __syncthreads();
    drain_rows([&](int r, int sc) -> TO* {
      const int64_t p = m0 + r, col = (int64_t)nt * (BN / 2) + (sc >> 6) * (WN / 2) + (sc & 63);
      if (p >= valid_end || col >= prm.I) return nullptr;
      return act + p * prm.I + col;
    });
  }
  (void)kZero;
}

template <typename TO, int MODE>
int launch_fp8(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  auto kernel = grouped_gemm_fp8_kernel<TO, MODE>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kLdsBytes);
    if (e != hipSuccess) {
      set_error("%s: cannot reserve %zu bytes of LDS: %s", name, kLdsBytes, hipGetErrorString(e));
      return CK_ERR_LAUNCH;
    }
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(NT), kLdsBytes, s, prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

// ---- per-row quantisation to e4m3 ------------------------------------------------------------------------------
constexpr int kQuantBlock = 256;
constexpr float kE4M3Max = 448.0f;

// scale[r] = amax(x[r, :]) / 448 (1 for an all-zero row); q[r, c] = e4m3(x[r, c] * (448 / amax)), round to nearest even
template <typename T>
__global__ __launch_bounds__(kQuantBlock) void quant_rows_e4m3_kernel(const T* __restrict__ x, int64_t rows, int cols,
                                                                       uint8_t* __restrict__ q, float* __restrict__ scales) {
  __shared__ float red[kQuantBlock / kWave];
  const int chunks = cols / 16;  // 16 elements: 32 bytes in, 16 bytes out
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* xr = x + row * cols;
    float amax = 0.f;
    for (int ch = threadIdx.x; ch < chunks; ch += kQuantBlock) {
      Pack16<T> a, b;
      a.v = load16(xr + ch * 16);
      b.v = load16(xr + ch * 16 + 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fmaxf(fabsf(Elem<T>::up(a.e[i])), fabsf(Elem<T>::up(b.e[i]))));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = amax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kQuantBlock / kWave; ++w) amax = fmaxf(amax, red[w]);
    const float inv = amax > 0.f ? kE4M3Max / amax : 1.0f;
    if (threadIdx.x == 0) scales[row] = amax > 0.f ? amax / kE4M3Max : 1.0f;
    for (int ch = threadIdx.x; ch < chunks; ch += kQuantBlock) {
      Pack16<T> a, b;
      a.v = load16(xr + ch * 16);  // second read is served by L1 / L2
      b.v = load16(xr + ch * 16 + 8);
      vec16 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const T* src = i < 2 ? a.e : b.e;
        const int k = (i & 1) * 4;
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(src[k]) * inv, Elem<T>::up(src[k + 1]) * inv, w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(Elem<T>::up(src[k + 2]) * inv, Elem<T>::up(src[k + 3]) * inv, w, true);
        o.w[i] = (uint32_t)w;
      }
      store16(q + row * cols + ch * 16, o);
    }
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

extern "C" int ck_quant_rows_e4m3(const void* x, int64_t rows, int32_t cols, void* q, float* scales, int32_t dtype,
                                  void* stream) {
  CK_REQUIRE(rows >= 0 && cols >= 16 && cols % 16 == 0, "ck_quant_rows_e4m3: cols=%d must be a positive multiple of 16", cols);
  if (rows == 0) return CK_OK;
  CK_REQUIRE(x && q && scales && aligned16(x) && aligned16(q), "ck_quant_rows_e4m3: NULL or misaligned pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned blocks = (unsigned)(rows < 65535 * 8 ? rows : 65535 * 8);
  CK_DISPATCH_HALF(dtype, "ck_quant_rows_e4m3", {
    hipLaunchKernelGGL((quant_rows_e4m3_kernel<scalar_t>), dim3(blocks), dim3(kQuantBlock), 0, s,
                       static_cast<const scalar_t*>(x), rows, (int)cols, static_cast<uint8_t*>(q), scales);
  });
  CK_CHECK_LAUNCH("ck_quant_rows_e4m3");
  return CK_OK;
}

extern "C" int ck_grouped_gemm_fp8(const void* a8, const float* a_scale, int32_t a_gather_div, const void* w8,
                                   const float* w_scale, int32_t N, int32_t K, const ck_segments* seg, int32_t epilogue,
                                   void* y, void* aux, int32_t out_dtype, void* stream) {
  const char* name = "ck_grouped_gemm_fp8";
  if (int rc = check_segments(seg, name)) return rc;
  CK_REQUIRE(seg->align == 256, "%s: fp8 tiles are 256 rows high; sort with align = 256", name);
  CK_REQUIRE(N >= 8 && N % 8 == 0, "%s: N=%d must be a positive multiple of 8", name, N);
  CK_REQUIRE(K >= 64 && K % 64 == 0, "%s: K=%d must be a positive multiple of 64", name, K);
  CK_REQUIRE(a_gather_div >= 0, "%s: a_gather_div=%d is negative", name, a_gather_div);
  CK_REQUIRE(epilogue == CK_EPI_GROUPED || epilogue == CK_EPI_SCATTER || epilogue == CK_EPI_SWIGLU,
             "%s: epilogue %d is not available in fp8 (grouped, scatter, swiglu)", name, epilogue);
  if (seg->max_rows == 0) return CK_OK;
  CK_REQUIRE(a8 && a_scale && w8 && w_scale, "%s: operands and scales are required", name);
  CK_REQUIRE(aligned16(a8) && aligned16(w8), "%s: a8 and w8 must be 16-byte aligned", name);
  CK_REQUIRE((int64_t)N * K < ((int64_t)1 << 32) && (a_gather_div > 0 || seg->max_rows * (int64_t)K < ((int64_t)1 << 32)),
             "%s: operands are addressed with 32-bit byte offsets (4 GiB per expert matrix / grouped input)", name);
  GemmParams prm = {};
  prm.a = a8;
  prm.w = w8;
  prm.lda = K;
  prm.ldw = K;
  prm.w_expert_stride = (int64_t)N * K;
  prm.a_gather_div = a_gather_div;
  prm.N = N;
  prm.K = K;
  prm.align = seg->align;
  prm.num_experts = seg->num_experts;
  prm.seg_starts = seg->seg_starts;
  prm.counts = seg->counts;
  prm.tile_expert = seg->tile_expert;
  prm.row_slot = seg->row_slot;
  prm.y = y;
  prm.aux = aux;
  prm.a_scale = a_scale;
  prm.w_scale = w_scale;
  int out_cols = N;
  if (epilogue == CK_EPI_SWIGLU) {
    CK_REQUIRE(N % 16 == 0 && aux != nullptr, "%s: the SwiGLU epilogue needs N = 2*I with I %% 8 == 0 and aux", name);
    prm.I = N / 2;
    out_cols = N / 2;
  } else {
    CK_REQUIRE(y != nullptr, "%s: y is required", name);
  }
  prm.n_tiles = (int)ceil_div(out_cols, epilogue == CK_EPI_SWIGLU ? BN / 2 : BN);
  const int64_t blocks = (seg->max_rows / seg->align) * prm.n_tiles;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  CK_DISPATCH_HALF(out_dtype, name, {
    switch (epilogue) {
      case CK_EPI_GROUPED: return launch_fp8<scalar_t, kGrouped>(prm, (unsigned)blocks, s, name);
      case CK_EPI_SCATTER: return launch_fp8<scalar_t, kScatter>(prm, (unsigned)blocks, s, name);
      default: return launch_fp8<scalar_t, kSwiglu>(prm, (unsigned)blocks, s, name);
    }
  });
  return CK_OK;
}
