// Scattered grouped GEMM with fp8 e4m3 operands (OCP e4m3fn on gfx950), fp32 accumulation, bf16 / f16 output.
// Forward (inference) only: Y = (A_e * diag(a_scale)) (W[e] * diag(w_scale[e]))^T, the two scale vectors applied to the
// fp32 accumulators in the epilogue.
//
// Same machinery as the 16-bit kernel with 128-byte LDS rows (grouped_gemm_line.hip): tile-aligned expert segments,
// 256 x 256 tile, four waves (one per SIMD) with 128 x 128 wave tiles and the accumulators pinned to AGPRs, global -> LDS
// direct loads of whole cache lines from a scalar base, two XOR-swizzled stages, and an epilogue straight from the
// accumulators. One byte per element: a K step is 128 elements = one v_mfma_f32_16x16x128_f8f6f4 per 16 x 16 block
// (twice the rate of the 16-bit MFMA; on random e4m3 operands a register-only loop of this shape sustains 4.3 PFLOP/s,
// the 32x32x64 shape 3.9), fragments are 32 bytes per lane, and every byte fetched from L2 carries twice the FLOPs.
// A step is a single slice, so there is one fragment set and it rotates: the registers of A row block i are reloaded
// from the next stage as soon as row block i has been multiplied, those of B block j behind the last row block. The
// barrier therefore sits at the start of a step (the next stage must have landed before the first reload), and the loads
// of step kt + 2 go out in the first half of step kt so that the last of them still has half a step to land.
#include <stdlib.h>

#include "gemm_common.h"

#ifndef CK_ABLATE
#define CK_ABLATE 0  // measurement builds only: 2 no loads in the loop, 4 no fragment reads, 32 no epilogue, 64 no MFMA
#endif

namespace ck {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WGM = 2, NW = WGM * 2, NT = 64 * NW;  // 4 waves: 2 along M, 2 along N
constexpr int WM = BM / WGM, WN = BN / 2;           // 128 x 128 wave tile
constexpr int MI = WM / 16, NI = WN / 16;
constexpr int BK = 128, NSTAGE = 2;
constexpr int kRowBytes = BK;  // one cache line per tile row and K step
constexpr int kStageBytes = (BM + BN) * kRowBytes;
constexpr int A_LD = BM * kRowBytes / (1024 * NW), B_LD = BN * kRowBytes / (1024 * NW);
// 16-byte chunk c of row r sits in slot c ^ swz128(r): 16 lanes reading one chunk index of 16 consecutive rows then touch
// all 64 banks once (even rows cover banks 0-31 with 8 distinct slots, odd rows 32-63)
__device__ inline int swz128(int row) { return (row >> 1) & 7; }
constexpr int kLoadsPerStep = A_LD + B_LD;
constexpr int kLoadGap = 2;  // MFMAs between two loads of the next-but-one K step: all out in the first half of a step
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
constexpr size_t kLdsBytes = (size_t)NSTAGE * kStageBytes;
static_assert(kLoadsPerStep * kLoadGap <= MI * NI && NT == BM, "loads fit a step; one thread per tile row");

__device__ inline void mfma_fp8(const i32x8& a, const i32x8& b, f32x4& c) {
  // cbsz = blgp = 0: both operands e4m3; accumulator pinned to AGPRs and updated in place (see Mfma16::run_acc)
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ inline void mfma_fp8_first(const i32x8& a, const i32x8& b, f32x4& c) {  // c = a * b + 0 (see run_acc_first)
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
}

template <typename TO, int MODE>
__global__ __launch_bounds__(NT) void grouped_gemm_fp8_kernel(const GemmParams prm) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  char* lds_c = reinterpret_cast<char*>(lds_raw);
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
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

  f32x4 acc[MI][NI];  // started by the first K step's MFMAs (constant 0 as their third operand): nothing zeroes them

  // ---- global -> LDS addressing: lane l of a wave-load fills slot l (16 bytes) of 64 consecutive slots = 8 rows of 128 B
  const char* a_base = static_cast<const char*>(prm.a);
  const char* b_base = static_cast<const char*>(prm.w) + (int64_t)expert * prm.w_expert_stride;
  uint32_t a_off[A_LD], b_off[B_LD];
  // gathered input: the row_slot entries of this lane's tile rows are fetched together (one wait, not one per load)
  // into the registers that then take the offsets
  if (prm.a_gather_div > 0) {
#pragma unroll
    for (int t = 0; t < A_LD; ++t) {
      int64_t p = m0 + (wave * A_LD + t) * 8 + (lane >> 3);
      if (p >= valid_end) p = valid_end - 1;
      a_off[t] = (uint32_t)prm.row_slot[p];
    }
  }
#pragma unroll
  for (int t = 0; t < A_LD; ++t) {
    const int r = (wave * A_LD + t) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ swz128(r);
    int64_t p = m0 + r;
    if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
    const int64_t row = prm.a_gather_div > 0 ? (int64_t)((int32_t)a_off[t] / prm.a_gather_div) : p;
    a_off[t] = (uint32_t)(row * prm.lda + c * 16);
  }
#pragma unroll
  for (int t = 0; t < B_LD; ++t) {
    const int j = (wave * B_LD + t) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ swz128(j);
    int64_t n;
    if constexpr (MODE == kSwiglu) {  // a wave's WN tile columns: WN/2 up columns, then the gate columns of the same outputs
      const int half = (j % WN) / (WN / 2);
      const int within = (j / WN) * (WN / 2) + (j % (WN / 2));
      n = (int64_t)half * prm.I + min((int64_t)nt * (BN / 2) + within, (int64_t)prm.I - 1);
    } else {
      n = min((int64_t)nt * BN + j, (int64_t)prm.N - 1);
    }
    b_off[t] = (uint32_t)(n * prm.ldw + c * 16);
  }
  const int nk = prm.K / BK;

  // ---- what the epilogue needs per tile row is fetched now and parked in LDS after the main loop: thread t takes tile
  // row t (its de-quantisation scale and, for the scatter epilogue, its output row)
  float meta_scale = 0.f;
  int meta_row = -1;
  {
    const int64_t p = m0 + tid;
    if (p < valid_end) {
      meta_scale = prm.a_scale[prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p];
      meta_row = (MODE == kScatter) ? prm.row_slot_out[p] : tid;
    }
  }

  // (one wait state between the scalar write of M0 and the load that reads it: the compiler inserts it for its own
  // instructions and cannot see into the asm)
  auto dma16 = [&](const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "m0");
  };
  auto uniform_ptr = [](const char* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
  };
  const char* a_base_u = uniform_ptr(a_base);
  const char* b_base_u = uniform_ptr(b_base);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_c;
  const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * A_LD * 1024);
  const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * kRowBytes + wave * B_LD * 1024);
  auto issue_one = [&](int step, int g) {
    const int64_t kb = (int64_t)step * kRowBytes;
    const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
    if constexpr ((CK_ABLATE & 2) != 0) {
      if (step >= NSTAGE) return;
    }
    if (g < A_LD) dma16(a_base_u + kb, a_off[g], wave_a + st + g * 1024);
    else dma16(b_base_u + kb, b_off[g - A_LD], wave_b + st + (g - A_LD) * 1024);
  };
  auto issue = [&](int step) {
#pragma unroll
    for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
  };

  // ---- fragments for v_mfma_f32_16x16x128_f8f6f4: row l % 16, contraction bytes 32 (l / 16) .. + 31 = the row's 16-byte
  // chunks 2 (l / 16) and 2 (l / 16) + 1. Both operands use the same byte -> k assignment, which is all a dot product needs.
  const int fsw = swz128(lane & 15), fq = lane >> 4;
  const int chunk_lo = ((2 * fq) ^ fsw) * 16, chunk_hi = ((2 * fq + 1) ^ fsw) * 16;
  const int fa_row = (wm * WM + (lane & 15)) * kRowBytes;
  const int fb_row = BM * kRowBytes + (wn * WN + (lane & 15)) * kRowBytes;
  i32x8 fa[MI], fb[NI];
  auto read_frag = [&](int stage, int g) {  // g < MI: A block g; else B block g - MI
    if constexpr ((CK_ABLATE & 4) != 0) {
      if (stage != 0) return;
    }
    const char* row = lds_c + stage * kStageBytes + (g < MI ? fa_row + g * 16 * kRowBytes : fb_row + (g - MI) * 16 * kRowBytes);
    const i32x4 lo = *reinterpret_cast<const i32x4*>(row + chunk_lo);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(row + chunk_hi);
    const i32x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    if (g < MI) fa[g] = v;
    else fb[g - MI] = v;
  };
  auto mfma = [&](int i, int j, auto first) {
    if constexpr ((CK_ABLATE & 64) != 0) {
      asm volatile("" ::"v"(fa[i]), "v"(fb[j]));
      if constexpr (decltype(first)::value) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      return;
    }
    // weight fragment first: a lane gets 4 consecutive output columns of one row
    if constexpr (decltype(first)::value) mfma_fp8_first(fb[j], fa[i], acc[i][j]);
    else mfma_fp8(fb[j], fa[i], acc[i][j]);
  };

  if (nk > 0) {
    issue(0);
    if (nk > 1) {
      issue(1);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLoadsPerStep) : "memory");  // step 0 landed, all waves
    } else {
      asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    }
#pragma unroll
    for (int g = 0; g < MI + NI; ++g) read_frag(0, g);

    // One K step: MI x NI MFMAs, row block by row block, and two barriers. At the start of a step every wave holds the
    // step's fragments in registers (read during the step before), so behind the first barrier the stage is free and, in
    // phase 0, the loads of step kt + 2 overwrite it, one every kLoadGap MFMAs of the first half. The second barrier,
    // behind MFMA kRawAt, publishes step kt + 1 (all loads older than this step's own have landed, for every wave): its
    // loads have had a whole step to arrive instead of half of one (c_proj launch of the 128-expert layer 3.78 -> 3.6 ms).
    // The fragments are reloaded from that stage behind the barrier: fa[i] of the row blocks already done one every
    // second MFMA, the others once their row block is done, fb[j] after the MFMA (MI - 1, j). Phase 1 is step nk - 2
    // (nothing left to fetch, one barrier), phase 2 the last step (nothing to wait for, nothing to reload).
    constexpr int kRawAt = 32;
    static_assert(kRawAt % NI == 0 && kRawAt >= kLoadsPerStep * kLoadGap && kRawAt + kRawAt / NI * 2 <= MI * NI - NI, "reload slots");
    auto k_step = [&](int kt, auto phase, auto idle, auto first) {
      constexpr bool kIdle = decltype(idle)::value;  // this wave's rows are all pad rows: no fragments, no MFMAs
      constexpr int kPhase = decltype(phase)::value;
      const int ns = (kt + 1) & (NSTAGE - 1);
      // every wave holds this step's fragments: the stage they came from is free for the loads of step kt + 2
      if constexpr (kPhase == 0) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
      for (int n = 0; n < MI * NI; ++n) {
        const int i = n / NI, j = n % NI;
        if constexpr (kPhase < 2) {
          // step kt + 1 has landed (every load older than this step's own), for all waves: its fragments may be read
          if (n == kRawAt) {
            if constexpr (kPhase == 0) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLoadsPerStep) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
          }
        }
        if constexpr (!kIdle) mfma(i, j, first);
        if constexpr (kPhase == 0) {
          if (n % kLoadGap == 0 && n / kLoadGap < kLoadsPerStep) issue_one(kt + 2, n / kLoadGap);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kPhase < 2 && !kIdle) {
          // row blocks finished in front of the barrier are reloaded behind it, one every second MFMA
          if (n >= kRawAt && (n - kRawAt) % 2 == 0 && (n - kRawAt) / 2 < kRawAt / NI) read_frag(ns, (n - kRawAt) / 2);
          if (j == NI - 1 && i >= kRawAt / NI) read_frag(ns, i);
          if (i == MI - 1) read_frag(ns, MI + j);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    auto k_loop = [&](auto idle) {  // the first step is peeled: its MFMAs start the accumulators
      constexpr std::integral_constant<int, 0> p0{};
      constexpr std::integral_constant<int, 1> p1{};
      constexpr std::integral_constant<int, 2> p2{};
      constexpr std::true_type first{};
      constexpr std::false_type later{};
      if (nk >= 3) {
        k_step(0, p0, idle, first);
        int kt = 1;
        for (; kt + 2 < nk; ++kt) k_step(kt, p0, idle, later);
        k_step(kt++, p1, idle, later);
        k_step(kt, p2, idle, later);
      } else if (nk == 2) {
        k_step(0, p1, idle, first);
        k_step(1, p2, idle, later);
      } else {
        k_step(0, p2, idle, first);
      }
      // behind the last MFMA, inside this variant of the loop: wait out the MFMA result latency and tie every accumulator
      // to that wait, so that none of the compiler's own accumulator reads can move in front of it (see mfma_fence)
      mfma_drain();
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) mfma_fence(acc[i][j]);
    };
    const bool wave_idle = m0 + wm * WM >= valid_end;
    if (__builtin_amdgcn_readfirstlane(wave_idle)) k_loop(std::true_type{});
    else k_loop(std::false_type{});
  }

  // ---- epilogue, straight from the accumulators (as in the 16-bit kernel): a lane holds, per 16x16 block (i, j), the 4
  // consecutive output columns j * 16 + 4 (lane / 16) + 0..3 of tile row i * 16 + lane % 16; both scales are applied in
  // fp32, pairs are rounded and packed by one conversion, and v_permlane16_swap regroups two column blocks into 8
  // consecutive columns per lane, so that every lane stores 16 bytes.
  float* meta_f = reinterpret_cast<float*>(lds_c);  // [BM] a_scale of the tile's rows, then [BM] output rows (scatter)
  int* meta_rows = reinterpret_cast<int*>(lds_c + BM * 4);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the stages
  meta_f[tid] = meta_scale;
  meta_rows[tid] = meta_row;
  __syncthreads();
  if constexpr ((CK_ABLATE & 32) != 0) {
    float sum = 0.f;
    static_for<MI>([&](auto i) { static_for<NI>([&](auto j) { static_for<4>([&](auto r) { sum += acc[i][j][(int)r]; }); }); });
    if (sum == 12345.678f) static_cast<TO*>(prm.y ? prm.y : prm.aux)[tid] = Elem<TO>::down(sum);
    return;
  }
  const int lrow = lane & 15, lg = lane >> 4;
  const bool odd_group = (lg & 1) != 0;
  auto gather8 = [&](uint32_t p0, uint32_t p1, uint32_t q0, uint32_t q1) {
    const auto s0 = __builtin_amdgcn_permlane16_swap(p0, q0, false, false);  // odd rows of p <-> even rows of q
    const auto s1 = __builtin_amdgcn_permlane16_swap(p1, q1, false, false);
    vec16 v;
    v.w[0] = s0[0];
    v.w[1] = s1[0];
    v.w[2] = s0[1];
    v.w[3] = s1[1];
    return v;
  };
  auto pair_col = [&](int j) { return (j + (odd_group ? 1 : 0)) * 16 + 4 * (lg & ~1); };
  auto store_at = [&](char* base_u, uint32_t off, const vec16& v) {
    const u32x4_t d = {v.w[0], v.w[1], v.w[2], v.w[3]};
    // two wait states: a store of more than 8 bytes followed by a vector write to its data registers needs them, and the
    // compiler cannot see into the asm to insert them
    asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" ::"v"(off), "v"(d), "s"(base_u) : "memory");
  };
  auto uniform_out = [](char* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<char*>(((uint64_t)hi << 32) | lo);
  };
  const float4* w_scale4 = reinterpret_cast<const float4*>(prm.w_scale + (int64_t)expert * prm.N);  // N % 8 == 0: 16-byte pieces
  const int64_t tile_row0 = m0 + wm * WM;
  const int rows_left = (int)min((int64_t)WM, valid_end - tile_row0);  // valid rows of this wave; may be <= 0

  if constexpr (MODE == kGrouped || MODE == kScatter) {
    TO* y = static_cast<TO*>(prm.y);
    const int64_t col0 = (int64_t)nt * BN + wn * WN;
    const int cols_left = (int)min((int64_t)WN, (int64_t)prm.N - col0);
    float4 cs[NI];  // the lane's 4 column scales of every column block
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int c = j * 16 + 4 * lg;
      cs[j] = c < cols_left ? w_scale4[(col0 + c) / 4] : float4{0.f, 0.f, 0.f, 0.f};
    }
    char* base = uniform_out(reinterpret_cast<char*>(y + tile_row0 * prm.N + col0));
    const uint32_t row_pitch = (uint32_t)prm.N * (uint32_t)sizeof(TO);
    uint32_t row_off = (uint32_t)lrow * row_pitch;
    static_for<MI>([&](auto i) {
      const int r = i * 16 + lrow;
      const float rs = meta_f[wm * WM + r];
      char* row_ptr = nullptr;
      if constexpr (MODE == kScatter) {
        const int out_row = meta_rows[wm * WM + r];
        row_ptr = reinterpret_cast<char*>(y + (int64_t)(out_row < 0 ? 0 : out_row) * prm.N + col0);
      }
      static_for<NI / 2>([&](auto jp) {
        const f32x4& p = acc[i][2 * jp];
        const f32x4& q = acc[i][2 * jp + 1];
        const float4 cp = cs[2 * jp], cq = cs[2 * jp + 1];
        const vec16 v = gather8(pack_pair<TO>(p[0] * rs * cp.x, p[1] * rs * cp.y), pack_pair<TO>(p[2] * rs * cp.z, p[3] * rs * cp.w),
                                pack_pair<TO>(q[0] * rs * cq.x, q[1] * rs * cq.y), pack_pair<TO>(q[2] * rs * cq.z, q[3] * rs * cq.w));
        const int c = pair_col(2 * jp);
        if (r < rows_left && c < cols_left) {
          if constexpr (MODE == kScatter) store16(row_ptr + (uint32_t)c * (uint32_t)sizeof(TO), v);
          else store_at(base, row_off + (uint32_t)c * (uint32_t)sizeof(TO), v);
        }
      });
      row_off += 16u * row_pitch;
      __builtin_amdgcn_sched_barrier(0);
    });
  } else {  // kSwiglu: the first half of a wave's column blocks are up, the second half the gate of the same activation
            // columns; only the activation is kept (inference)
    TO* act = static_cast<TO*>(prm.aux);
    const int64_t col0 = (int64_t)nt * (BN / 2) + wn * (WN / 2);  // the wave's first activation column
    const int cols_left = (int)min((int64_t)(WN / 2), (int64_t)prm.I - col0);
    constexpr int NH = NI / 2;
    float4 cs_up[NH], cs_gate[NH];
#pragma unroll
    for (int j = 0; j < NH; ++j) {
      const int c = j * 16 + 4 * lg;
      const bool ok = c < cols_left;
      cs_up[j] = ok ? w_scale4[(col0 + c) / 4] : float4{0.f, 0.f, 0.f, 0.f};
      cs_gate[j] = ok ? w_scale4[(prm.I + col0 + c) / 4] : float4{0.f, 0.f, 0.f, 0.f};
    }
    char* base = uniform_out(reinterpret_cast<char*>(act + tile_row0 * prm.I + col0));
    const uint32_t row_pitch = (uint32_t)prm.I * (uint32_t)sizeof(TO);
    uint32_t row_off = (uint32_t)lrow * row_pitch;
    static_for<MI>([&](auto i) {
      const int r = i * 16 + lrow;
      const float rs = meta_f[wm * WM + r];
      static_for<NH / 2>([&](auto jp) {
        uint32_t pk[2][2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const f32x4& u = acc[i][2 * jp + b];
          const f32x4& g = acc[i][2 * jp + b + NH];
          const float su[4] = {cs_up[2 * jp + b].x, cs_up[2 * jp + b].y, cs_up[2 * jp + b].z, cs_up[2 * jp + b].w};
          const float sg[4] = {cs_gate[2 * jp + b].x, cs_gate[2 * jp + b].y, cs_gate[2 * jp + b].z, cs_gate[2 * jp + b].w};
          float a[4];
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            // rounded to the output type first, like a pre-activation tensor would be
            const float up = Elem<TO>::up(Elem<TO>::down(u[s] * rs * su[s]));
            const float gf = Elem<TO>::up(Elem<TO>::down(g[s] * rs * sg[s]));
            a[s] = up * gf * sigmoid_fast(gf);
          }
          pk[b][0] = pack_pair<TO>(a[0], a[1]);
          pk[b][1] = pack_pair<TO>(a[2], a[3]);
        }
        const vec16 v = gather8(pk[0][0], pk[0][1], pk[1][0], pk[1][1]);
        const int c = pair_col(2 * jp);
        if (r < rows_left && c < cols_left) store_at(base, row_off + (uint32_t)c * (uint32_t)sizeof(TO), v);
      });
      row_off += 16u * row_pitch;
      __builtin_amdgcn_sched_barrier(0);
    });
  }
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
  CK_REQUIRE((reinterpret_cast<uintptr_t>(w_scale) & 15) == 0, "%s: w_scale must be 16-byte aligned", name);
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
  prm.row_slot_out = seg->row_slot_out != nullptr ? seg->row_slot_out : seg->row_slot;
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
