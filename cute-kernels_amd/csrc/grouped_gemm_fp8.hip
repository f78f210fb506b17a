// Scattered grouped GEMM with fp8 e4m3 operands (OCP e4m3fn on gfx950), fp32 accumulation, bf16 / f16 output.
// Forward (inference) only: Y = (A_e * diag(a_scale)) (W[e] * diag(w_scale[e]))^T, the two scale vectors applied to the
// fp32 accumulators in the epilogue.
//
// Same machinery as the 16-bit kernel with 128-byte LDS rows (tile-aligned expert segments, 256x256 tile, 8 waves,
// global -> LDS direct loads of whole cache lines, two XOR-swizzled stages, hand-ordered load / fragment-read / MFMA
// stream, LDS-staged epilogue), with one byte per element: a K step is 128 elements = two v_mfma_f32_32x32x64_f8f6f4 per
// 32 x 32 block (twice the rate of the 16-bit MFMA), fragments are 32 bytes per lane, and every byte fetched from L2
// carries twice the FLOPs.
#include <stdlib.h>

#include "gemm_common.h"

#ifndef CK_ABLATE
#define CK_ABLATE 0  // measurement builds only: 2 no loads in the loop, 4 no fragment reads, 32 no epilogue, 64 no MFMA, 128 no main loop
#endif

namespace ck {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WGM = 4, NW = WGM * 2, NT = 64 * NW;  // 8 waves: 4 along M, 2 along N
constexpr int WM = BM / WGM, WN = BN / 2;           // 64 x 128 wave tile
constexpr int MI = WM / 32, NI = WN / 32;
constexpr int BK = 128, KS = BK / 64, NSTAGE = 2;
constexpr int kRowBytes = BK;  // one cache line per tile row and K step
constexpr int kStageBytes = (BM + BN) * kRowBytes;
constexpr int A_LD = BM * kRowBytes / (1024 * NW), B_LD = BN * kRowBytes / (1024 * NW);
// 16-byte chunk c of row r sits in slot c ^ swz128(r): 16 lanes reading one chunk index of 16 consecutive rows then touch
// all 64 banks once (even rows cover banks 0-31 with 8 distinct slots, odd rows 32-63)
__device__ inline int swz128(int row) { return (row >> 1) & 7; }
constexpr int kLoadsPerStep = A_LD + B_LD;
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
constexpr int kMetaOffset = NSTAGE * kStageBytes;  // after the stages: a_scale of the tile's rows, w_scale of its columns,
constexpr int kMetaBytes = (BM + BN + BM) * 4;      // and the output row of every tile row (scatter epilogue)
constexpr size_t kLdsBytes = (size_t)kMetaOffset + kMetaBytes;
static_assert(NT == BM + BN, "one thread per tile row / tile column fetches the epilogue's scales");

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

#if (CK_ABLATE & 256)
  auto stamp = [&](int i) {
    __builtin_amdgcn_s_waitcnt(0);
    if (prm.y_t != nullptr && tid == 0) static_cast<uint64_t*>(prm.y_t)[(size_t)blockIdx.x * 8 + i] = wall_clock64();
  };
#else
  auto stamp = [&](int) {};
#endif
  stamp(0);
  f32x16 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- global -> LDS addressing: lane l of a wave-load fills slot l (16 bytes) of 64 consecutive slots = 8 rows of 128 B
  const char* a_base = static_cast<const char*>(prm.a);
  const char* b_base = static_cast<const char*>(prm.w) + (int64_t)expert * prm.w_expert_stride;
  uint32_t a_off[A_LD], b_off[B_LD];
#pragma unroll
  for (int t = 0; t < A_LD; ++t) {
    const int r = (wave * A_LD + t) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ swz128(r);
    int64_t p = m0 + r;
    if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
    const int64_t row = prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p;
    a_off[t] = (uint32_t)(row * prm.lda + c * 16);
  }
#pragma unroll
  for (int t = 0; t < B_LD; ++t) {
    const int j = (wave * B_LD + t) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ swz128(j);
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
  const int nk = (CK_ABLATE & 128) ? 0 : prm.K / BK;  // 128: no main loop at all

  // ---- what the epilogue needs from global memory is fetched now and parked in LDS after the main loop: thread t < BM
  // takes tile row t (its de-quantisation scale and, for the scatter epilogue, its output row), thread BM + j column j
  float meta_scale = 0.f;
  int meta_row = -1;
  if (tid < BM) {
    const int64_t p = m0 + tid;
    if (p < valid_end) {
      const int slot = (prm.a_gather_div > 0 || MODE == kScatter) ? prm.row_slot[p] : 0;
      meta_scale = prm.a_scale[prm.a_gather_div > 0 ? (int64_t)(slot / prm.a_gather_div) : p];
      meta_row = (MODE == kScatter) ? slot : tid;
    }
  } else {
    const int j = tid - BM;
    const float* w_scale = prm.w_scale + (int64_t)expert * prm.N;
    if constexpr (MODE == kSwiglu) {  // columns 0 .. 127: up scales of the tile's activation columns; 128 .. 255: gate
      const int64_t col = (int64_t)nt * (BN / 2) + (j & (BN / 2 - 1));
      if (col < prm.I) meta_scale = w_scale[(j < BN / 2 ? 0 : prm.I) + col];
    } else {
      const int64_t n = (int64_t)nt * BN + j;
      if (n < prm.N) meta_scale = w_scale[n];
    }
  }

  auto dma16 = [&](const char* src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "m0");
  };
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_c;
  const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * A_LD * 1024);
  const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * kRowBytes + wave * B_LD * 1024);
  auto issue_one = [&](int step, int g) {
    const int64_t kb = (int64_t)step * kRowBytes;
    const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
    if constexpr ((CK_ABLATE & 2) != 0) {
      if (step >= NSTAGE) return;
    }
    if (g < A_LD) dma16(a_base + kb + a_off[g], wave_a + st + g * 1024);
    else dma16(b_base + kb + b_off[g - A_LD], wave_b + st + (g - A_LD) * 1024);
  };
  auto issue = [&](int step) {
#pragma unroll
    for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
  };

  // ---- fragments for v_mfma_f32_32x32x64_f8f6f4: slice sl (64 of the row's 128 bytes) of row l % 32 -- lane l holds its
  // 16-byte chunks 4 sl + 2 h and 4 sl + 2 h + 1, h = l / 32. Both operands use the same byte -> k assignment, which is
  // all a dot product needs.
  const int fsw = swz128(lane & 31), fh = lane >> 5;
  int chunk_lo[KS], chunk_hi[KS];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) {
    chunk_lo[sl] = ((4 * sl + 2 * fh) ^ fsw) * 16;
    chunk_hi[sl] = ((4 * sl + 2 * fh + 1) ^ fsw) * 16;
  }
  const int fa_row = (wm * WM + (lane & 31)) * kRowBytes;
  const int fb_row = BM * kRowBytes + (wn * WN + (lane & 31)) * kRowBytes;
  i32x8 fa[MI], fb[NI];
  auto read_frag = [&](int stage, int sl, int g) {  // g < MI: A block g; else B block g - MI
    if constexpr ((CK_ABLATE & 4) != 0) {
      if (stage != 0 || sl != 0) return;
    }
    const char* row = lds_c + stage * kStageBytes + (g < MI ? fa_row + g * 32 * kRowBytes : fb_row + (g - MI) * 32 * kRowBytes);
    const i32x4 lo = *reinterpret_cast<const i32x4*>(row + chunk_lo[sl]);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(row + chunk_hi[sl]);
    const i32x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    if (g < MI) fa[g] = v;
    else fb[g - MI] = v;
  };
  auto mfma = [&](int i, int j) {
    if constexpr ((CK_ABLATE & 64) != 0) {
      asm volatile("" ::"v"(fa[i]), "v"(fb[j]));
      return;
    }
    // scale operands 0: the compiler emits the unscaled v_mfma_f32_32x32x64_f8f6f4 (both operands e4m3: cbsz = blgp = 0)
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
  };
  static_assert(MI == 2 && NI == 4 && kLoadsPerStep == 8 && KS == 2, "the hand schedule below is written for this shape");

  if (nk > 0) {
    issue(0);
    if (nk > 1) {
      issue(1);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLoadsPerStep) : "memory");  // step 0 landed, all waves
    } else {
      asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    }
#pragma unroll
    for (int g = 0; g < MI + NI; ++g) read_frag(0, 0, g);
    // One 64-byte slice = one MFMA per 32 x 32 block. Fragments are single-buffered and rotate: as soon as the last MFMA
    // that needs a fragment has issued, the same registers are reloaded for the next slice.
    // Slice 0: the next slice is in the same stage. Slice 1 (last): the next slice is slice 0 of step kt + 1 in the other
    // stage -- phase 0 / 1: wait for that stage (the only loads in flight) and for this wave's own fragment reads, then
    // meet the other waves; the whole current stage has been read by everyone, so in phase 0 the loads of step kt + 2
    // overwrite it under this slice's MFMAs. Phase 1 is step nk - 2 (nothing left to fetch), phase 2 the last step.
    auto slice = [&](int kt, auto sl, auto phase) {
      constexpr bool kLast = decltype(sl)::value == KS - 1;
      constexpr int kPhase = decltype(phase)::value;
      const int ns = kLast ? (kt + 1) & (NSTAGE - 1) : kt & (NSTAGE - 1);
      constexpr int nsl = kLast ? 0 : decltype(sl)::value + 1;
      constexpr bool kReload = !(kLast && kPhase == 2);
      constexpr bool kIssue = kLast && kPhase == 0;
      if constexpr (kLast && kPhase < 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        mfma(0, j);
        if constexpr (kIssue) issue_one(kt + 2, j);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (kReload) read_frag(ns, nsl, 0);
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        mfma(1, j);
        if constexpr (kIssue) issue_one(kt + 2, NI + j);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kReload) read_frag(ns, nsl, MI + j);
      }
      if constexpr (kReload) read_frag(ns, nsl, 1);
      __builtin_amdgcn_sched_barrier(0);
    };
    auto k_step = [&](int kt, auto phase) { static_for<KS>([&](auto sl) { slice(kt, sl, phase); }); };
    int kt = 0;
    for (; kt + 2 < nk; ++kt) k_step(kt, std::integral_constant<int, 0>{});
    if (kt + 2 == nk) k_step(kt++, std::integral_constant<int, 1>{});
    k_step(kt, std::integral_constant<int, 2>{});
  }

  // ---- epilogue through LDS (see the 16-bit kernel): slab S[col][row] of 128 tile columns, 8-byte writes from the
  // accumulator layout, ds_read_b64_tr_b16 back out so that a lane stores 8 consecutive columns of one row
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  constexpr int kSlabCols = 128, kSlabLd = BM + 4;
  TO* slab = reinterpret_cast<TO*>(lds_raw);
  stamp(2);
  float* meta_f = reinterpret_cast<float*>(lds_c + kMetaOffset);    // [0, BM): a scales; [BM, BM + BN): w scales
  int* meta_rows = reinterpret_cast<int*>(lds_c + kMetaOffset) + BM + BN;  // [BM]: output row, -1 for a pad row
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  meta_f[tid] = meta_scale;
  if (tid < BM) meta_rows[tid] = meta_row;
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  stamp(3);
  const int col_in_block = lane & 31;
  const int row_quad = (lane >> 5) * 4;

  // de-quantisation scales of the rows this lane holds (0 for pad rows)
  float rs[MI][4][4];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = *reinterpret_cast<const float4*>(meta_f + wm * WM + i * 32 + 8 * q + row_quad);
      rs[i][q][0] = v.x;
      rs[i][q][1] = v.y;
      rs[i][q][2] = v.z;
      rs[i][q][3] = v.w;
    }

  stamp(4);
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
  // Row-major drain as in the 16-bit kernel: 16 lanes take a 4-row x 32-column block, the four lane groups of a wave two
  // adjacent column blocks of two adjacent row blocks (whole 128-byte lines per store instruction); rows and column pairs
  // are walked in unrolled loops, so every address is a per-lane base plus a compile-time offset. row_ptr(tile row) ->
  // address of the output row at the tile's first column (nullptr: pad row), block_col(cb) -> output column of slab
  // column block cb relative to that, cols_left = valid columns from there on, tile_cols = columns the tile spans.
  auto drain_rows = [&](auto&& row_ptr, auto&& block_col, int64_t cols_left, int tile_cols) {
    const int l16 = tid & 15, csel = (tid >> 4) & 1, rsel = (tid >> 5) & 1;
    const int tq = l16 & 3, tj = l16 >> 2;
    const int oq = l16 >> 2, oe = l16 & 3;
    constexpr int kColPairs = kSlabCols / 64, kRowIters = (BM / 4) / (2 * NT / kWave);
    static_assert(kSlabCols % 64 == 0 && (BM / 4) % (2 * NT / kWave) == 0, "whole column pairs and row iterations");
    const bool cols_full = cols_left >= tile_cols;
    auto body = [&](auto checked) {
      static_for<kRowIters>([&](auto it) {
        const int rb = (it * (NT / kWave) + wave) * 2 + rsel;
        TO* dst_row = row_ptr(rb * 4 + oe);
        if (dst_row != nullptr) dst_row += 8 * oq;
        const TO* src_row = slab + (csel * 32 + 8 * tq + tj) * kSlabLd + rb * 4;
        static_for<kColPairs>([&](auto cp) {
          const TO* src = src_row + cp * 64 * kSlabLd;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src + 4 * kSlabLd));
          const int col = csel ? block_col(std::integral_constant<int, 2 * decltype(cp)::value + 1>{})
                               : block_col(std::integral_constant<int, 2 * decltype(cp)::value>{});
          if (dst_row != nullptr && (!checked || col + 8 * oq < cols_left)) {
            vec16 v;
            v.w[0] = (uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
            v.w[1] = (uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
            v.w[2] = (uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
            v.w[3] = (uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
            store16_nt(dst_row + col, v);
          }
        });
      });
    };
    if (cols_full) body(std::false_type{});
    else body(std::true_type{});
  };
  const float* w_sc = meta_f + BM;

  if constexpr ((CK_ABLATE & 32) != 0) {
    float sum = 0.f;
    static_for<MI>([&](auto i) { static_for<NI>([&](auto j) { static_for<16>([&](auto r) { sum += acc[i][j][(int)r]; }); }); });
    if (sum == 12345.678f) static_cast<TO*>(prm.y ? prm.y : prm.aux)[tid] = Elem<TO>::down(sum + rs[0][0][0]);
  } else if constexpr (MODE == kGrouped || MODE == kScatter) {
    TO* y = static_cast<TO*>(prm.y);
    static_for<2>([&](auto pass) {
      float cs[2];
      static_for<2>([&](auto jj) { cs[jj] = w_sc[wn * WN + (pass * 2 + jj) * 32 + col_in_block]; });
      stage_blocks([&](auto i, auto jj, auto q, auto s) {
        return Elem<TO>::down(acc[i][pass * 2 + jj][4 * q + s] * rs[i][q][s] * cs[jj]);
      });
      __syncthreads();
      if constexpr (pass == 0) stamp(6);
      drain_rows(
          [&](int r) -> TO* {
            const int out_row = meta_rows[r];
            if (out_row < 0) return nullptr;
            const int64_t row = (MODE == kScatter) ? (int64_t)out_row : m0 + r;
            return y + row * prm.N + (int64_t)nt * BN;
          },
          [&](auto cb) { return ((cb * 32) >> 6) * WN + pass * 64 + ((cb * 32) & 63); }, prm.N - (int64_t)nt * BN, BN);
      if constexpr (pass == 0) stamp(7);
      __syncthreads();
    });
  } else {  // kSwiglu: blocks 0, 1 = up, blocks 2, 3 = gate of the same activation columns; only the activation is kept
    TO* act = static_cast<TO*>(prm.aux);
    float cs_up[2], cs_gate[2];
    static_for<2>([&](auto jj) {
      cs_up[jj] = w_sc[wn * (WN / 2) + jj * 32 + col_in_block];
      cs_gate[jj] = w_sc[BN / 2 + wn * (WN / 2) + jj * 32 + col_in_block];
    });
    stage_blocks([&](auto i, auto jj, auto q, auto s) {
      // rounded to the output type first, like a pre-activation tensor would be
      const TO up = Elem<TO>::down(acc[i][jj][4 * q + s] * rs[i][q][s] * cs_up[jj]);
      const TO gate = Elem<TO>::down(acc[i][jj + 2][4 * q + s] * rs[i][q][s] * cs_gate[jj]);
      const float gf = Elem<TO>::up(gate);
      return Elem<TO>::down(Elem<TO>::up(up) * gf * sigmoid_fast(gf));
    });
    __syncthreads();
    drain_rows(
        [&](int r) -> TO* {
          const int64_t p = m0 + r;
          return p < valid_end ? act + p * prm.I + (int64_t)nt * (BN / 2) : nullptr;
        },
        [&](auto cb) { return ((cb * 32) >> 6) * (WN / 2) + ((cb * 32) & 63); }, prm.I - (int64_t)nt * (BN / 2), BN / 2);
  }
  stamp(5);
}

template <typename TO, int MODE>
int launch_fp8(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  auto kernel = grouped_gemm_fp8_kernel<TO, MODE>;
  static bool lds_reserved[kMaxDevices] = {};
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kernel), kLdsBytes, lds_reserved, name)) return rc;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(NT), kLdsBytes, s, prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

// ---- per-row quantisation to e4m3 ------------------------------------------------------------------------------
constexpr int kQuantBlock = 256;
constexpr float kE4M3Max = 448.0f;

// scale[r] = amax(x[r, :]) / 448 (1 for an all-zero row); q[r, c] = e4m3(x[r, c] * (448 / amax)), round to nearest even.
// A row is owned by TPR = 64 lanes (one wave, no block synchronisation) or 256 (the block); a lane keeps its NC chunks of
// 16 elements in registers between the reduction and the conversion, so x is read once (NC == 0: long rows, re-read).
template <typename T, int TPR, int NC>
__global__ __launch_bounds__(kQuantBlock) void quant_rows_e4m3_kernel(const T* __restrict__ x, int64_t rows, int cols,
                                                                       uint8_t* __restrict__ q, float* __restrict__ scales) {
  __shared__ float red[kQuantBlock / kWave];
  constexpr int ROWS = kQuantBlock / TPR;
  const int chunks = cols / 16;  // 16 elements: 32 bytes in, 16 bytes out
  const int lane = threadIdx.x % TPR;
  auto chunk_amax = [&](const Pack16<T>& a, const Pack16<T>& b, float m) {
#pragma unroll
    for (int i = 0; i < 8; ++i) m = fmaxf(m, fmaxf(fabsf(Elem<T>::up(a.e[i])), fabsf(Elem<T>::up(b.e[i]))));
    return m;
  };
  auto convert = [&](const Pack16<T>& a, const Pack16<T>& b, float inv) {
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
    return o;
  };
  // TPR == 256: every thread of the block runs the same trip count (the reduction synchronises the block)
  for (int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR; row < rows; row += (int64_t)gridDim.x * ROWS) {
    const T* xr = x + row * cols;
    uint8_t* qr = q + row * cols;
    float amax = 0.f;
    Pack16<T> a[NC > 0 ? NC : 1], b[NC > 0 ? NC : 1];
    if constexpr (NC > 0) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) {
          a[c].v = load16_nt(xr + ch * 16);
          b[c].v = load16_nt(xr + ch * 16 + 8);
          amax = chunk_amax(a[c], b[c], amax);
        }
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        a[0].v = load16(xr + ch * 16);
        b[0].v = load16(xr + ch * 16 + 8);
        amax = chunk_amax(a[0], b[0], amax);
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    if constexpr (TPR == kQuantBlock) {
      __syncthreads();
      if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = amax;
      __syncthreads();
#pragma unroll
      for (int w = 0; w < kQuantBlock / kWave; ++w) amax = fmaxf(amax, red[w]);
    }
    const float inv = amax > 0.f ? kE4M3Max / amax : 1.0f;
    if (lane == 0) scales[row] = amax > 0.f ? amax / kE4M3Max : 1.0f;
    if constexpr (NC > 0) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ch = c * TPR + lane;
        if (ch < chunks) store16_nt(qr + ch * 16, convert(a[c], b[c], inv));
      }
    } else {
      for (int ch = lane; ch < chunks; ch += TPR) {
        a[0].v = load16(xr + ch * 16);  // second read is served by L1 / L2
        b[0].v = load16(xr + ch * 16 + 8);
        store16_nt(qr + ch * 16, convert(a[0], b[0], inv));
      }
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
  const int chunks = cols / 16;
#define CK_QUANT(TPR, NC)                                                                                          \
  do {                                                                                                             \
    const int64_t want = ceil_div(rows, (int64_t)(kQuantBlock / (TPR)));                                           \
    const unsigned blocks = (unsigned)(want < 65535 * 4 ? want : 65535 * 4);                                       \
    hipLaunchKernelGGL((quant_rows_e4m3_kernel<scalar_t, TPR, NC>), dim3(blocks), dim3(kQuantBlock), 0, s,         \
                       static_cast<const scalar_t*>(x), rows, (int)cols, static_cast<uint8_t*>(q), scales);        \
  } while (0)
  CK_DISPATCH_HALF(dtype, "ck_quant_rows_e4m3", {
    if (chunks <= kWave) CK_QUANT(kWave, 1);
    else if (chunks <= 2 * kWave) CK_QUANT(kWave, 2);
    else if (chunks <= kQuantBlock) CK_QUANT(kQuantBlock, 1);
    else if (chunks <= 2 * kQuantBlock) CK_QUANT(kQuantBlock, 2);
    else if (chunks <= 4 * kQuantBlock) CK_QUANT(kQuantBlock, 4);
    else CK_QUANT(kQuantBlock, 0);
  });
#undef CK_QUANT
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
  CK_REQUIRE(K >= 128 && K % 128 == 0, "%s: K=%d must be a positive multiple of 128", name, K);
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
#if (CK_ABLATE & 256)
  if (const char* t = getenv("CK_TRACE_PTR")) prm.y_t = reinterpret_cast<void*>(strtoull(t, nullptr, 16));
#endif
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
