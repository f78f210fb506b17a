// Scattered grouped GEMMs over tile-aligned expert segments, bf16 / f16 inputs, fp32 accumulation on MFMA.
//
// Every expert's rows start at a multiple of the tile height in the padded grouped layout, so a workgroup's M-tile
// belongs to exactly one expert: no tile straddles two experts and no K loop is repeated per expert. All GEMMs are
// "NT": both operands are contraction-contiguous (the backward passes get that from transposed copies written by the
// producing epilogues), so global loads are 128-bit along K and LDS fragments feed v_mfma_f32_32x32x16 directly.
//
// This file holds the general kernel (256 x 256 or 128 x 128 tiles, any K % 8 == 0, every epilogue) and the two C entry
// points. Launches with 256-row alignment and a contraction length that is a multiple of 64 go to the kernel with
// 128-byte LDS rows in grouped_gemm_line.hip instead. Here: workgroup = 8 waves in a 4 x 2 grid (or 4 in 2 x 2), wave
// tiles built from 32x32 MFMA blocks, and two pipelines -- K step 32 straight from global memory into four swizzled LDS
// stages (K % 32 == 0), or K step 64 through registers into two padded LDS stages (any K % 8 == 0).
#include <atomic>

#include "gemm_common.h"

namespace ck {
namespace {

constexpr int kThreads = 256;
constexpr int BK = 64;            // K elements per stage
constexpr int kLdsStride = 72;    // elements per LDS row (64 + 8 pad)
constexpr int kChunksPerRow = 8;  // 16-byte chunks per 64-element row


#ifndef CK_ABLATE
#define CK_ABLATE 0  // measurement builds only: 1 no barrier, 2 no loads in the loop, 4 no fragment reads, 8 no load wait
#endif

// Which of two kernels that compute the same result a launch takes, as set through ck_debug_set_option (tests and
// measurements); the defaults are what the product runs.
inline bool force_register_pipeline() { return debug_options().gemm_register_pipeline.load(std::memory_order_relaxed) != 0; }
inline bool eight_waves() { return debug_options().gemm_four_waves.load(std::memory_order_relaxed) == 0; }
inline bool line_kernel_enabled() { return debug_options().gemm_line_kernel.load(std::memory_order_relaxed) != 0; }


// PIPE 0: K step 64, global -> registers -> padded LDS, two stages (any K % 8 == 0).
// PIPE 1: K step 32, global -> LDS directly (no register staging), four XOR-swizzled stages, loads three steps ahead
//         (needs K % 32 == 0).
// WGM: waves along M (2 or 4), always 2 along N: 4 waves = one per SIMD with 128x128 wave tiles at BM = BN = 256;
//      8 waves = two per SIMD with 64x128 wave tiles, so that one wave's memory instructions issue under the other's
//      MFMAs (PIPE 1 only).
// pipeline stages, then one int per tile row: the output row of the scatter epilogue (-1 for a pad row)
template <int BM, int BN, int PIPE>
constexpr size_t stage_bytes() {
  return PIPE == 0 ? (size_t)2 * (BM + BN) * kLdsStride * 2 : (size_t)4 * (BM + BN) * 32 * 2;
}
template <int BM, int BN, int PIPE>
constexpr size_t lds_bytes() {
  return stage_bytes<BM, BN, PIPE>() + (size_t)BM * 4;
}

template <typename T, int BM, int BN, int MODE, int PIPE, int WGM>
__global__ __launch_bounds__(64 * WGM * 2) void grouped_gemm_kernel(const GemmParams prm) {
  static_assert(PIPE == 1 || WGM == 2, "the register-staged pipeline is written for 4 waves");
  constexpr int NW = WGM * 2;                // waves per workgroup
  constexpr int WM = BM / WGM, WN = BN / 2;  // wave tile
  constexpr int MI = WM / 32, NI = WN / 32;  // 32x32 blocks per wave tile
  constexpr int A_CH = BM / 32, B_CH = BN / 32;  // 16-byte chunks per thread per stage
  constexpr int kStageElems = (BM + BN) * kLdsStride;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile: blocks are dealt round-robin to the 8 XCDs, so give each XCD a contiguous run of tiles
  int mt, nt, expert;
  int64_t k_begin = 0;
  int k_len;
  if constexpr (MODE == kDw) {
    // Experts differ in contraction length (their row counts), so every XCD gets a slice of EVERY expert's tile grid:
    // the grid is cut in 8 along its longer side, and a slice is walked in groups of 8 tiles along that side.
    const int per_expert = prm.m_tiles * prm.n_tiles;
    const bool m_major = prm.m_tiles >= prm.n_tiles;
    const int major = m_major ? prm.m_tiles : prm.n_tiles, minor = m_major ? prm.n_tiles : prm.m_tiles;
    int pid = blockIdx.x, a, b;  // a: index along the major side, b: along the minor side
    if (major % kXcds == 0) {
      const int xcd = pid % kXcds, j = pid / kXcds;
      const int slice = major / kXcds, per_slice = slice * minor;
      expert = j / per_slice;
      grouped_order(j - expert * per_slice, slice, minor, a, b);
      a += xcd * slice;
    } else {
      expert = pid / per_expert;
      grouped_order(pid - expert * per_expert, major, minor, a, b);
    }
    mt = m_major ? a : b;
    nt = m_major ? b : a;
    k_begin = prm.seg_starts[expert];
    k_len = (int)((prm.counts[expert] + BK - 1) / BK * BK);
  } else {
    const int live_m = prm.seg_starts[prm.num_experts] / prm.align;
    const int total = live_m * prm.n_tiles;
    int pid = blockIdx.x;
    if (pid >= total) return;
    const int per_xcd = total / kXcds;
    if (pid < per_xcd * kXcds) pid = (pid % kXcds) * per_xcd + pid / kXcds;  // the ragged end keeps its order
    grouped_order(pid, live_m, prm.n_tiles, mt, nt);
    expert = prm.tile_expert[mt];
    k_len = prm.K;
  }
  const int64_t m0 = (int64_t)mt * BM;

  int64_t valid_end = 0;  // forward modes: first pad row of this expert's segment
  if constexpr (MODE != kDw) valid_end = (int64_t)prm.seg_starts[expert] + prm.counts[expert];
  // scatter epilogue: the output row of tile row `tid`, fetched now and parked in LDS once the main loop is over
  int scatter_row = -1;
  if constexpr (MODE == kScatter) {
    for (int r = threadIdx.x; r < BM; r += 64 * WGM * 2)  // at most one trip per thread: BM <= threads
      if (m0 + r < valid_end) scatter_row = prm.row_slot_out[m0 + r];
  }

#if (CK_ABLATE & 256)
  auto stamp = [&](int i) {  // measurement builds: wall-clock (100 MHz) of phase boundaries, one record per workgroup
    __builtin_amdgcn_s_waitcnt(0);
    if (prm.trace != nullptr && tid == 0) static_cast<uint64_t*>(prm.trace)[(size_t)blockIdx.x * 8 + i] = wall_clock64();
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

  if constexpr (PIPE == 0) {
    // ---- per-thread global chunk addresses, as 32-bit offsets in 16-byte chunks from the operand base
    const int cc = tid & (kChunksPerRow - 1);  // chunk within the 64-element K slab
    const int lr = tid >> 3;                   // row within a group of 32
    // 32-bit byte offsets from a wave-uniform base: the loads use scalar-base + vector-offset addressing, and stepping
    // along K only moves the scalar base
    const char* a_base = static_cast<const char*>(prm.a);
    const char* b_base = static_cast<const char*>(prm.w);
    uint32_t a_chunk[A_CH], b_chunk[B_CH];
    if constexpr (MODE == kDw) {
  #pragma unroll
      for (int i = 0; i < A_CH; ++i) {
        const int64_t row = min(m0 + lr + 32 * i, (int64_t)prm.M - 1);
        a_chunk[i] = (uint32_t)((row * prm.lda + k_begin) * 2 + cc * 16);
      }
  #pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        const int64_t row = min((int64_t)nt * BN + lr + 32 * i, (int64_t)prm.N - 1);
        b_chunk[i] = (uint32_t)((row * prm.ldw + k_begin) * 2 + cc * 16);
      }
    } else {
  #pragma unroll
      for (int i = 0; i < A_CH; ++i) {
        int64_t p = m0 + lr + 32 * i;
        if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
        const int64_t row = prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p;
        a_chunk[i] = (uint32_t)(row * prm.lda * 2 + cc * 16);
      }
      b_base += (int64_t)expert * prm.w_expert_stride * 2;
  #pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        const int j = lr + 32 * i;  // row of the LDS B tile
        int64_t n;
        if constexpr (MODE == kSwiglu) {
          // LDS rows [wave column][up half | gate half]: the same lane ends up holding up and gate of one column
          const int half = (j % WN) / (WN / 2);
          const int within = (j / WN) * (WN / 2) + (j % (WN / 2));
          const int64_t col = min((int64_t)nt * (BN / 2) + within, (int64_t)prm.I - 1);
          n = (int64_t)half * prm.I + col;
        } else {
          n = min((int64_t)nt * BN + j, (int64_t)prm.N - 1);
        }
        b_chunk[i] = (uint32_t)(n * prm.ldw * 2 + cc * 16);
      }
    }

    // ---- main loop
    // Per K step of 64: the global loads of step k+1 are issued first and stay in flight; the 64 MFMAs of step k run
    // with the LDS fragment reads of the next 16-wide slice interleaved between them (double-buffered fragments); the
    // LDS stores of step k+1 are interleaved with the MFMAs of the last slice; one barrier closes the step.
    vec16 ra[A_CH], rb[B_CH];
    auto load_global = [&](int kt, auto full) {
      const char* ak = a_base + (int64_t)kt * (BK * 2);
      const char* bk = b_base + (int64_t)kt * (BK * 2);
      if constexpr (decltype(full)::value) {
  #pragma unroll
        for (int i = 0; i < A_CH; ++i) ra[i] = load16(ak + a_chunk[i]);
  #pragma unroll
        for (int i = 0; i < B_CH; ++i) rb[i] = load16(bk + b_chunk[i]);
      } else {
        const bool ok = kt * BK + cc * 8 < k_len;  // K % 8 == 0, so a chunk is entirely inside or outside
  #pragma unroll
        for (int i = 0; i < A_CH; ++i) ra[i] = ok ? load16(ak + a_chunk[i]) : zero16();
  #pragma unroll
        for (int i = 0; i < B_CH; ++i) rb[i] = ok ? load16(bk + b_chunk[i]) : zero16();
      }
    };
    auto store_lds = [&](int stage) {
      T* sa = lds + stage * kStageElems;
      T* sb = sa + BM * kLdsStride;
  #pragma unroll
      for (int i = 0; i < A_CH; ++i) store16(sa + (lr + 32 * i) * kLdsStride + cc * 8, ra[i]);
  #pragma unroll
      for (int i = 0; i < B_CH; ++i) store16(sb + (lr + 32 * i) * kLdsStride + cc * 8, rb[i]);
    };
    typedef typename Mfma<T>::frag frag_t;
    const int frag_a_off = (wm * WM + (lane & 31)) * kLdsStride + (lane >> 5) * 8;
    const int frag_b_off = BM * kLdsStride + (wn * WN + (lane & 31)) * kLdsStride + (lane >> 5) * 8;
    constexpr int KK = BK / 16;  // 16-wide slices per K step; even, so slice 0 always lands in fragment buffer 0
    frag_t fa[2][MI], fb[2][NI];
    auto read_frags = [&](int stage, int kk, int buf) {
      const T* sa = lds + stage * kStageElems + frag_a_off + kk * 16;
      const T* sb = lds + stage * kStageElems + frag_b_off + kk * 16;
  #pragma unroll
      for (int i = 0; i < MI; ++i) fa[buf][i] = *reinterpret_cast<const frag_t*>(sa + i * 32 * kLdsStride);
  #pragma unroll
      for (int j = 0; j < NI; ++j) fb[buf][j] = *reinterpret_cast<const frag_t*>(sb + j * 32 * kLdsStride);
    };
    // MFMAs [first, last) of one slice, row-major over the wave's MI x NI blocks
    auto mfma_range = [&](int buf, int first, int last) {
  #pragma unroll
      for (int i = 0; i < MI; ++i)
  #pragma unroll
        for (int j = 0; j < NI; ++j)
          if (i * NI + j >= first && i * NI + j < last) acc[i][j] = Mfma<T>::run(fa[buf][i], fb[buf][j], acc[i][j]);
    };
    constexpr int kMfmaPerSlice = MI * NI, kReadsPerSlice = MI + NI, kWritesPerStep = A_CH + B_CH;
    // One K step out of LDS stage `stage`, whose slice-0 fragments are already in buffer 0.
    // HAS_NEXT: also prefetch step kt + 1 from global memory (FULL: all of its 64 columns exist), store it into the other
    // LDS stage and fetch its slice-0 fragments.
    auto k_step = [&](int stage, int kt, auto has_next, auto full) {
      constexpr bool HAS_NEXT = decltype(has_next)::value;
      if constexpr (HAS_NEXT) load_global(kt + 1, full);
  #pragma unroll
      for (int kk = 0; kk + 1 < KK; ++kk) {
        read_frags(stage, kk + 1, (kk + 1) & 1);
        mfma_range(kk & 1, 0, kMfmaPerSlice);
  #pragma unroll
        for (int g = 0; g < kReadsPerSlice; ++g) {  // pin the interleave: 1 global load, 1 LDS read, a share of the MFMAs
          if constexpr (HAS_NEXT) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerSlice / kReadsPerSlice, 0);
        }
      }
      constexpr int last = (KK - 1) & 1;
      if constexpr (HAS_NEXT) {
        // last slice: its first half hides the LDS stores of the next step, the barrier, then its second half hides the
        // first fragment reads of the next step
        store_lds(stage ^ 1);
        mfma_range(last, 0, kMfmaPerSlice / 2);
  #pragma unroll
        for (int g = 0; g < kMfmaPerSlice / 2; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x200, (kWritesPerStep + kMfmaPerSlice / 2 - 1) / (kMfmaPerSlice / 2), 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __syncthreads();
        read_frags(stage ^ 1, 0, 0);
        mfma_range(last, kMfmaPerSlice / 2, kMfmaPerSlice);
  #pragma unroll
        for (int g = 0; g < kMfmaPerSlice / 2; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x100, (kReadsPerSlice + kMfmaPerSlice / 2 - 1) / (kMfmaPerSlice / 2), 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
      } else {
        mfma_range(last, 0, kMfmaPerSlice);
      }
    };

    const int nk = (k_len + BK - 1) / BK;
    const int nk_full = k_len / BK;  // steps whose 64 columns all exist
    if (nk > 0) {
      if (nk_full > 0) load_global(0, std::true_type{});
      else load_global(0, std::false_type{});
      store_lds(0);
      __syncthreads();
      read_frags(0, 0, 0);
      int kt = 0;
      for (; kt + 1 < nk_full; ++kt) k_step(kt & 1, kt, std::true_type{}, std::true_type{});
      for (; kt + 1 < nk; ++kt) k_step(kt & 1, kt, std::true_type{}, std::false_type{});  // ragged last columns
      k_step((nk - 1) & 1, nk - 1, std::false_type{}, std::false_type{});
    }

  } else {
    // ---- PIPE 1: direct-to-LDS pipeline
    constexpr int BK1 = 32, NSTAGE = 4, KS = BK1 / 16;
    constexpr int A_LD = BM / (16 * NW), B_LD = BN / (16 * NW);  // 1 KiB wave-loads per wave per step and operand
    static_assert(A_LD >= 1 && B_LD >= 1, "tile too small for this many waves");
    constexpr int kStageBytes = (BM + BN) * BK1 * 2;
    constexpr int kRowBytes = BK1 * 2;  // 64 B = 4 chunks; chunk c of row r sits in slot c ^ swz(r)
    auto swz = [](int row) { return lds_swizzle(row); };
    char* lds_c = reinterpret_cast<char*>(lds_raw);
    const char* a_base = static_cast<const char*>(prm.a);
    const char* b_base = static_cast<const char*>(prm.w);
    // A wave-load writes 64 consecutive 16-byte slots of LDS (lane l -> slot l): 16 tile rows x 4 slots. The lane
    // fetches the global chunk that belongs in its slot.
    uint32_t a_off[A_LD], b_off[B_LD];
    if constexpr (MODE != kDw) b_base += (int64_t)expert * prm.w_expert_stride * 2;
#pragma unroll
    for (int t = 0; t < A_LD; ++t) {
      const int r = (wave * A_LD + t) * 16 + (lane >> 2);
      const int c = (lane & 3) ^ swz(r);
      int64_t row;
      if constexpr (MODE == kDw) {
        row = min(m0 + r, (int64_t)prm.M - 1);
      } else {
        int64_t p = m0 + r;
        if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
        row = prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p;
      }
      a_off[t] = (uint32_t)((row * prm.lda + k_begin) * 2 + c * 16);
    }
#pragma unroll
    for (int t = 0; t < B_LD; ++t) {
      const int j = (wave * B_LD + t) * 16 + (lane >> 2);  // row of the LDS B tile
      const int c = (lane & 3) ^ swz(j);
      int64_t n;
      if constexpr (MODE == kSwiglu) {
        const int half = (j % WN) / (WN / 2);
        const int within = (j / WN) * (WN / 2) + (j % (WN / 2));
        n = (int64_t)half * prm.I + min((int64_t)nt * (BN / 2) + within, (int64_t)prm.I - 1);
      } else {
        n = min((int64_t)nt * BN + j, (int64_t)prm.N - 1);
      }
      b_off[t] = (uint32_t)((n * prm.ldw + k_begin) * 2 + c * 16);
    }
    const int nk = k_len / BK1;
    // loads of K step `step` into stage step % 4; steps past the end re-fetch the last one (never read) so that the
    // number of loads in flight is the same at every wait
    // One wave-load: global -> LDS, no registers in between. Issued as inline asm so that the compiler's wait-count
    // pass does not serialise the pipeline behind it; the waits for these loads are the explicit ones below.
    auto dma16 = [&](const char* src, uint32_t lds_addr) {
#ifndef CK_LOAD_MOD
#define CK_LOAD_MOD ""
#endif
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" CK_LOAD_MOD ::"s"(lds_addr), "v"(src) : "m0");
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_c;
    const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * A_LD * 1024);
    const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * kRowBytes + wave * B_LD * 1024);
    constexpr int kLoadsPerStep = A_LD + B_LD, kReads = MI + NI, kMfma = MI * NI;
    // load number `g` (0 .. kLoadsPerStep) of K step `step` into stage step % 4; steps past the end re-fetch the last
    // one (never read) so that the number of loads in flight is the same at every wait
    auto issue_one = [&](int step, int g) {
      const int64_t kb = (CK_ABLATE & 16) ? (int64_t)0 : (int64_t)min(step, nk - 1) * kRowBytes;  // 16: always K step 0
      const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
      if (g < A_LD) dma16(a_base + kb + a_off[g], wave_a + st + g * 1024);
      else dma16(b_base + kb + b_off[g - A_LD], wave_b + st + (g - A_LD) * 1024);
    };
    auto issue = [&](int step) {
#pragma unroll
      for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
    };
    typedef typename Mfma<T>::frag frag_t;
    const int fsw = swz(lane & 31), fh = lane >> 5;
    int slice_off[KS];
#pragma unroll
    for (int sl = 0; sl < KS; ++sl) slice_off[sl] = (((2 * sl + fh) ^ fsw) * 16);
    const int fa_row = (wm * WM + (lane & 31)) * kRowBytes;
    const int fb_row = BM * kRowBytes + (wn * WN + (lane & 31)) * kRowBytes;
    frag_t fa[2][MI], fb[2][NI];
    // fragment `g` of a slice: g < MI -> A block g, else B block g - MI
    auto read_one = [&](int stage, int sl, int buf, int g) {
      const char* st = lds_c + stage * kStageBytes + slice_off[sl];
      if (g < MI) fa[buf][g] = *reinterpret_cast<const frag_t*>(st + fa_row + g * 32 * kRowBytes);
      else fb[buf][g - MI] = *reinterpret_cast<const frag_t*>(st + fb_row + (g - MI) * 32 * kRowBytes);
    };
    auto mfma_range = [&](int buf, int first, int last) {
      if constexpr ((CK_ABLATE & 64) != 0) return;  // measurement builds: loads and fragment reads only
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
          if (i * NI + j >= first && i * NI + j < last) acc[i][j] = Mfma<T>::run(fa[buf][i], fb[buf][j], acc[i][j]);
    };
    // wait until at most `pending` of this wave's loads are in flight, then meet the other waves
    auto wait_and_barrier = [&](auto pending) {
      constexpr int kPending = decltype(pending)::value;
      if constexpr (!(CK_ABLATE & 8)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kPending) : "memory");
      if constexpr (!(CK_ABLATE & 1)) asm volatile("s_barrier" ::: "memory");
    };
    // fragment read order: A0, then every B block, then the remaining A blocks -- the order the MFMAs need them in
    auto read_nth = [&](int stage, int sl, int buf, int n) {
      const int g = n == 0 ? 0 : (n <= NI ? MI + n - 1 : n - NI);
      if constexpr (!(CK_ABLATE & 4)) read_one(stage, sl, buf, g);
    };
    // MFMAs [mfma_begin(g), mfma_begin(g + 1)) follow fragment read g
    auto mfma_begin = [](int g) { return g * kMfma / kReads; };
    stamp(1);
    if (nk > 0) {
      issue(0);
      issue(1);
      issue(2);
      wait_and_barrier(std::integral_constant<int, 2 * kLoadsPerStep>{});  // step 0 has landed, for every wave
#pragma unroll
      for (int g = 0; g < kReads; ++g) read_one(0, 0, 0, g);
      // phase 0: steady state (prefetch step kt + 3; steps kt + 1, kt + 2 in flight); phase 1: step nk - 3 (nothing left
      // to prefetch, same wait); phase 2: the last two steps (at most one step in flight: wait for all of it)
      auto k_step = [&](int kt, auto phase) {
        constexpr int kPhase = decltype(phase)::value;
        // first half: MFMAs of slice 0 from fragment buffer 0, the fragment reads of slice 1 between them
#pragma unroll
        for (int g = 0; g < kReads; ++g) {
          read_nth(kt & (NSTAGE - 1), 1, 1, g);
          mfma_range(0, mfma_begin(g), mfma_begin(g + 1));
          __builtin_amdgcn_sched_barrier(0);
        }
        // Step kt + 1 has landed for every wave (only step kt + 2 may still be in flight). The barrier also orders
        // the overwrite below: stage (kt + 3) % 4 was last read as slice 1 of step kt - 1, and every wave consumed
        // those fragments (so its reads completed) before arriving here.
        wait_and_barrier(std::integral_constant<int, kPhase == 2 ? 0 : kLoadsPerStep>{});
        // second half: MFMAs of slice 1 from buffer 1; between them the loads of step kt + 3 and the slice-0 fragment
        // reads of step kt + 1
#pragma unroll
        for (int g = 0; g < kReads; ++g) {
          if constexpr (!(CK_ABLATE & 2) && kPhase == 0)
            if (g < kLoadsPerStep) issue_one(kt + 3, g);
          read_nth((kt + 1) & (NSTAGE - 1), 0, 0, g);
          mfma_range(1, mfma_begin(g), mfma_begin(g + 1));
          __builtin_amdgcn_sched_barrier(0);
        }
        static_assert(kLoadsPerStep <= kReads, "every load of a step has a slot in the second half");
      };
      // a prefetch past the end would only re-fetch the last step and waste L2 bandwidth
      int kt = 0;
      for (; kt + 3 < nk; ++kt) k_step(kt, std::integral_constant<int, 0>{});
      if (kt + 3 == nk) k_step(kt++, std::integral_constant<int, 1>{});
      for (; kt < nk; ++kt) k_step(kt, std::integral_constant<int, 2>{});
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // short contractions: the prologue fetched past the end
    }
  }

  stamp(2);
  // ---- epilogue. Lane holds, per 32x32 block and q in 0..3, rows 8q + 4*(lane/32) + 0..3 of column lane%32.
  // static_for keeps every accumulator index a compile-time constant (the accumulators live in AGPRs).
  const int col_in_block = lane & 31;
  const int row_quad = (lane >> 5) * 4;
  // optional per-expert bias row (aux_in = bias [E, N], grouped / scatter epilogues): added to the fp32 accumulators, so
  // that the output is rounded once, like F.linear with a bias. A lane's accumulators of one column block all belong to
  // one output column.
  if constexpr (MODE == kGrouped || MODE == kScatter) {
    if (prm.aux_in != nullptr) {
      const T* bias = static_cast<const T*>(prm.aux_in) + (int64_t)expert * prm.N;
      static_for<NI>([&](auto j) {
        const int64_t n = (int64_t)nt * BN + wn * WN + j * 32 + col_in_block;
        const float b = n < prm.N ? Elem<T>::up(bias[n]) : 0.f;
        static_for<MI>([&](auto i) {
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] += b;
        });
      });
    }
  }
  if constexpr ((CK_ABLATE & 32) != 0) {  // measurement builds: no epilogue (keep the accumulators alive)
    float keep = 0.f;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) keep += acc[i][j][0];
    if (keep == 123.456f) static_cast<float*>(prm.y)[0] = keep;
    return;
  }
  if constexpr (BM == 256 && BN == 256 && MODE != kSwigluBwd && !(CK_ABLATE & 128)) {
    // ---- staged epilogue (256x256 tiles): the tile leaves through LDS so that global stores are 16 bytes per lane
    // and 64+ contiguous bytes per row. A slab = 128 tile columns (2 of each wave's 4 column blocks), kept transposed,
    // S[col][row]: the accumulator layout (4 consecutive rows of one column per lane) writes it with 8-byte stores,
    // row-major outputs come back out through ds_read_b64_tr_b16 (a lane ends up with 8 consecutive columns of one
    // row), transposed outputs through plain 16-byte reads.
    typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
    constexpr int NT = 64 * NW;
    constexpr int kSlabCols = 128, kSlabLd = BM + 4;  // 520-byte rows: 8-byte aligned and spread over the banks
    T* slab = lds;                                    // the pipeline stages are dead by now
    int* scatter_rows = reinterpret_cast<int*>(lds_raw + stage_bytes<BM, BN, PIPE>());
    if constexpr (MODE == kScatter) {
      if (tid < BM) scatter_rows[tid] = scatter_row;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the stages

    // write this wave's blocks (i, jb..jb+1) of a value source into the slab
    auto stage_blocks = [&](auto&& value /* (i, jj, q, s) -> T */) {
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
    // slab column -> column of the block tile, for pass `pass` (which pair of each wave's column blocks is staged)
    auto tile_col = [&](int sc, int pass) { return (sc >> 6) * WN + pass * 64 + (sc & 63); };
    // row-major readout: out_ptr(row, tile column) must return the address of 8 consecutive output columns or nullptr
    auto drain_rows = [&](auto&& out_ptr) {
      const int l16 = tid & 15, grp = tid >> 4;
      const int tq = l16 & 3, tj = l16 >> 2;  // as a source lane: which slab column this lane points at
      const int oq = l16 >> 2, oe = l16 & 3;  // as a destination lane: 8 columns oq of row oe of the 4 x 32 block
      constexpr int kBlocks = (BM / 4) * (kSlabCols / 32);
#pragma unroll 4
      for (int b = grp; b < kBlocks; b += NT / 16) {
        const int rb = b >> 2, cb = b & 3;
        const T* src = slab + (cb * 32 + 8 * tq + tj) * kSlabLd + rb * 4;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src));
        const s16x4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src + 4 * kSlabLd));
        T* dst = out_ptr(rb * 4 + oe, cb * 32 + 8 * oq);
        if (dst != nullptr) {
          vec16 v;
          v.w[0] = (uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
          v.w[1] = (uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
          v.w[2] = (uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
          v.w[3] = (uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
          store16_nt(dst, v);
        }
      }
    };
    // transposed readout: out_ptr(slab column, row) -> address of 8 consecutive rows of that column, or nullptr
    auto drain_cols = [&](auto&& out_ptr) {
      constexpr int kChunks = kSlabCols * (BM / 8);
#pragma unroll 4
      for (int ch = tid; ch < kChunks; ch += NT) {
        const int c = ch / (BM / 8), r = (ch % (BM / 8)) * 8;
        T* dst = out_ptr(c, r);
        if (dst != nullptr) store16_nt(dst, load16(slab + c * kSlabLd + r));
      }
    };
    auto sync_slab = [&]() { __syncthreads(); };
    const T kZero = Elem<T>::down(0.f);
    // most tiles have no pad rows: then nothing is tested per element (the test is a 64-bit compare and a branch each)
    const bool tile_full = MODE == kDw || m0 + BM <= valid_end;

    if constexpr (MODE == kDw) {
      T* dw = static_cast<T*>(prm.y) + (int64_t)expert * prm.M * prm.N;
      static_for<2>([&](auto pass) {
        stage_blocks([&](auto i, auto jj, auto q, auto sidx) { return Elem<T>::down(acc[i][pass * 2 + jj][4 * q + sidx]); });
        sync_slab();
        drain_rows([&](int r, int sc) -> T* {
          const int64_t m = m0 + r, n = (int64_t)nt * BN + tile_col(sc, pass);
          return (m < prm.M && n < prm.N) ? dw + m * prm.N + n : nullptr;
        });
        sync_slab();
      });
    } else if constexpr (MODE == kGrouped || MODE == kScatter) {
      T* y = static_cast<T*>(prm.y);
      T* y_t = static_cast<T*>(prm.y_t);
      static_for<2>([&](auto pass) {
        // pad rows are staged as zeros: the transposed copy must hold zeros there
        if (tile_full) {
          stage_blocks([&](auto i, auto jj, auto q, auto sidx) { return Elem<T>::down(acc[i][pass * 2 + jj][4 * q + sidx]); });
        } else {
          stage_blocks([&](auto i, auto jj, auto q, auto sidx) {
            const int64_t p = m0 + wm * WM + i * 32 + 8 * q + row_quad + sidx;
            return p < valid_end ? Elem<T>::down(acc[i][pass * 2 + jj][4 * q + sidx]) : kZero;
          });
        }
        sync_slab();
        drain_rows([&](int r, int sc) -> T* {
          const int64_t p = m0 + r, n = (int64_t)nt * BN + tile_col(sc, pass);
          if (p >= valid_end || n >= prm.N) return nullptr;
          const int64_t row = (MODE == kScatter) ? (int64_t)scatter_rows[r] : p;
          return y + row * prm.N + n;
        });
        if (MODE == kGrouped && y_t != nullptr) {
          drain_cols([&](int sc, int r) -> T* {
            const int64_t n = (int64_t)nt * BN + tile_col(sc, pass);
            return n < prm.N ? y_t + n * prm.ld_t + m0 + r : nullptr;
          });
        }
        sync_slab();
        if (MODE == kGrouped && prm.aux != nullptr) {  // CK_ACT_GELU_TANH: the activation of the rounded output, to aux
          T* act = static_cast<T*>(prm.aux);
          stage_blocks([&](auto i, auto jj, auto q, auto sidx) {
            return Elem<T>::down(gelu_tanh_fast(Elem<T>::up(Elem<T>::down(acc[i][pass * 2 + jj][4 * q + sidx]))));
          });
          sync_slab();
          drain_rows([&](int r, int sc) -> T* {
            const int64_t p = m0 + r, n = (int64_t)nt * BN + tile_col(sc, pass);
            return (p < valid_end && n < prm.N) ? act + p * prm.N + n : nullptr;
          });
          sync_slab();
        }
      });
    } else {  // kSwiglu: blocks j = 0, 1 are up, j = 2, 3 are gate of the same activation columns
      T* pre = static_cast<T*>(prm.y);
      T* act = static_cast<T*>(prm.aux);
      T* act_t = static_cast<T*>(prm.y_t);
      const int64_t two_i = 2 * (int64_t)prm.I;
      // activation column of slab column sc (64 per wave column)
      auto act_col = [&](int sc) { return (int64_t)nt * (BN / 2) + (sc >> 6) * (WN / 2) + (sc & 63); };
      static_for<3>([&](auto pass) {  // 0: up half of the pre-activation, 1: gate half, 2: activation
        auto value = [&](auto i, auto jj, auto q, auto sidx, bool valid) {
          const T up = Elem<T>::down(acc[i][jj][4 * q + sidx]);
          const T gate = Elem<T>::down(acc[i][jj + 2][4 * q + sidx]);
          if (pass == 0) return up;
          if (pass == 1) return gate;
          const float gf = Elem<T>::up(gate);  // from the rounded pre-activation, like the unfused path
          const float sg = sigmoid_fast(gf);
          const T a = Elem<T>::down(prm.act_kind == CK_ACT_GLU ? Elem<T>::up(up) * sg : Elem<T>::up(up) * gf * sg);  // same association as swiglu_fwd_kernel
          return valid ? a : kZero;
        };
        if (tile_full) {
          stage_blocks([&](auto i, auto jj, auto q, auto sidx) { return value(i, jj, q, sidx, true); });
        } else {
          stage_blocks([&](auto i, auto jj, auto q, auto sidx) {
            return value(i, jj, q, sidx, m0 + wm * WM + i * 32 + 8 * q + row_quad + sidx < valid_end);
          });
        }
        sync_slab();
        drain_rows([&](int r, int sc) -> T* {
          const int64_t p = m0 + r, col = act_col(sc);
          if (p >= valid_end || col >= prm.I) return nullptr;
          if (pass == 0) return pre + p * two_i + col;
          if (pass == 1) return pre + p * two_i + prm.I + col;
          return act + p * prm.I + col;
        });
        if (pass == 2 && act_t != nullptr) {
          drain_cols([&](int sc, int r) -> T* {
            const int64_t col = act_col(sc);
            return col < prm.I ? act_t + col * prm.ld_t + m0 + r : nullptr;
          });
        }
        sync_slab();
      });
    }
    stamp(3);
    return;
  }
  if constexpr (MODE == kDw) {
    T* dw = static_cast<T*>(prm.y) + (int64_t)expert * prm.M * prm.N;
    static_for<MI>([&](auto i) {
      static_for<NI>([&](auto j) {
        const int64_t n = (int64_t)nt * BN + wn * WN + j * 32 + col_in_block;
        static_for<16>([&](auto r) {
          const int64_t m = m0 + wm * WM + i * 32 + 8 * (r / 4) + row_quad + (r % 4);
          if (m < prm.M && n < prm.N) dw[m * prm.N + n] = Elem<T>::down(acc[i][j][(int)r]);
        });
      });
    });
  } else if constexpr (MODE == kGrouped || MODE == kScatter) {
    T* y = static_cast<T*>(prm.y);
    T* y_t = static_cast<T*>(prm.y_t);
    T* act = MODE == kGrouped ? static_cast<T*>(prm.aux) : nullptr;  // CK_ACT_GELU_TANH: second output
    static_for<MI>([&](auto i) {
      static_for<4>([&](auto q) {
        const int64_t p_base = m0 + wm * WM + i * 32 + 8 * q + row_quad;
        int64_t out_row[4];
        static_for<4>([&](auto s) {
          const int64_t p = p_base + s;
          out_row[s] = -1;
          if (p < valid_end) out_row[s] = (MODE == kScatter) ? (int64_t)prm.row_slot_out[p] : p;
        });
        static_for<NI>([&](auto j) {
          const int64_t n = (int64_t)nt * BN + wn * WN + j * 32 + col_in_block;
          if (n < prm.N) {
            T v[4];
            static_for<4>([&](auto s) {
              v[s] = Elem<T>::down(acc[i][j][4 * q + s]);
              if (out_row[s] >= 0) {
                y[out_row[s] * prm.N + n] = v[s];
                if (act != nullptr) act[out_row[s] * prm.N + n] = Elem<T>::down(gelu_tanh_fast(Elem<T>::up(v[s])));
              } else {
                v[s] = Elem<T>::down(0.f);
              }
            });
            if (MODE == kGrouped && y_t != nullptr) store4(y_t + n * prm.ld_t + p_base, v[0], v[1], v[2], v[3]);
          }
        });
      });
    });
  } else if constexpr (MODE == kSwiglu) {
    // acc[i][j] (j < NI/2) = up, acc[i][j + NI/2] = gate of the same column
    T* pre = static_cast<T*>(prm.y);
    T* act = static_cast<T*>(prm.aux);
    T* act_t = static_cast<T*>(prm.y_t);
    const int64_t two_i = 2 * (int64_t)prm.I;
    static_for<MI>([&](auto i) {
      static_for<4>([&](auto q) {
        const int64_t p_base = m0 + wm * WM + i * 32 + 8 * q + row_quad;
        static_for<NI / 2>([&](auto j) {
          const int64_t col = (int64_t)nt * (BN / 2) + wn * (WN / 2) + j * 32 + col_in_block;
          if (col < prm.I) {
            T v[4];
            static_for<4>([&](auto s) {
              const int64_t p = p_base + s;
              const T up = Elem<T>::down(acc[i][j][4 * q + s]);
              const T gate = Elem<T>::down(acc[i][j + NI / 2][4 * q + s]);
              const float gf = Elem<T>::up(gate);
              const float sg = sigmoid_fast(gf);
              v[s] = Elem<T>::down(prm.act_kind == CK_ACT_GLU ? Elem<T>::up(up) * sg : Elem<T>::up(up) * gf * sg);  // same association as swiglu_fwd_kernel
              if (p < valid_end) {
                pre[p * two_i + col] = up;
                pre[p * two_i + prm.I + col] = gate;
                act[p * prm.I + col] = v[s];
              } else {
                v[s] = Elem<T>::down(0.f);
              }
            });
            if (act_t != nullptr) store4(act_t + col * prm.ld_t + p_base, v[0], v[1], v[2], v[3]);
          }
        });
      });
    });
  } else {  // kSwigluBwd: the GEMM result is d_act
    const T* pre = static_cast<const T*>(prm.aux_in);
    T* d_pre = static_cast<T*>(prm.y);
    T* d_pre_t = static_cast<T*>(prm.y_t);
    const int64_t two_i = 2 * (int64_t)prm.I;
    static_for<MI>([&](auto i) {
      static_for<4>([&](auto q) {
        const int64_t p_base = m0 + wm * WM + i * 32 + 8 * q + row_quad;
        static_for<NI>([&](auto j) {
          const int64_t col = (int64_t)nt * BN + wn * WN + j * 32 + col_in_block;
          if (col < prm.I) {
            T du[4], dg[4];
            static_for<4>([&](auto s) {
              const int64_t p = p_base + s;
              du[s] = Elem<T>::down(0.f);
              dg[s] = Elem<T>::down(0.f);
              if (p < valid_end) {
                const float dy = Elem<T>::up(Elem<T>::down(acc[i][j][4 * q + s]));  // d_act as the unfused path rounds it
                const float uf = Elem<T>::up(pre[p * two_i + col]);
                const float gf = Elem<T>::up(pre[p * two_i + prm.I + col]);
                const float sg = sigmoid_fast(gf);
                const float gsg = gf * sg;
                du[s] = Elem<T>::down(dy * gsg);
                dg[s] = Elem<T>::down(dy * uf * (sg + gsg * (1.0f - sg)));
                d_pre[p * two_i + col] = du[s];
                d_pre[p * two_i + prm.I + col] = dg[s];
              }
            });
            if (d_pre_t != nullptr) {
              store4(d_pre_t + col * prm.ld_t + p_base, du[0], du[1], du[2], du[3]);
              store4(d_pre_t + (prm.I + col) * prm.ld_t + p_base, dg[0], dg[1], dg[2], dg[3]);
            }
          }
        });
      });
    });
  }
}

template <typename T, int BM, int BN, int MODE, int PIPE, int WGM>
int launch_pipe(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  auto kernel = grouped_gemm_kernel<T, BM, BN, MODE, PIPE, WGM>;
  static bool lds_reserved[kMaxDevices] = {};
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kernel), lds_bytes<BM, BN, PIPE>(), lds_reserved, name)) return rc;
  constexpr size_t kLds = lds_bytes<BM, BN, PIPE>();
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(64 * WGM * 2), kLds, s, prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

// the direct-to-LDS pipeline whenever the contraction length allows it
template <typename T, int BM, int BN, int MODE>
int launch(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  const bool dma = (MODE == kDw) || (prm.K % 32 == 0);
  if (dma && !force_register_pipeline()) {
    if (eight_waves()) return launch_pipe<T, BM, BN, MODE, 1, 4>(prm, blocks, s, name);
    return launch_pipe<T, BM, BN, MODE, 1, 2>(prm, blocks, s, name);
  }
  return launch_pipe<T, BM, BN, MODE, 0, 2>(prm, blocks, s, name);
}

template <typename T, int MODE>
int launch_by_tile(const GemmParams& prm, int align, unsigned blocks_256, unsigned blocks_128, hipStream_t s,
                   const char* name) {
  if (align == 256) return launch<T, 256, 256, MODE>(prm, blocks_256, s, name);
  return launch<T, 128, 128, MODE>(prm, blocks_128, s, name);
}

}  // namespace
}  // namespace ck

namespace ck {
uint32_t next_split_epoch() {
  static std::atomic<uint32_t> counter{0};
  uint32_t e;
  do e = counter.fetch_add(1, std::memory_order_relaxed) + 1u; while ((e & 0x0fffffffu) == 0);
  return e & 0x0fffffffu;
}
}  // namespace ck

using namespace ck;

namespace {
inline void fill_segments(GemmParams& prm, const ck_segments* seg) {
  prm.align = seg->align;
  prm.num_experts = seg->num_experts;
  prm.seg_starts = seg->seg_starts;
  prm.counts = seg->counts;
  prm.tile_expert = seg->tile_expert;
  prm.row_slot = seg->row_slot;
  prm.row_slot_out = seg->row_slot_out != nullptr ? seg->row_slot_out : seg->row_slot;
  prm.trace = debug_options().trace_buffer.load(std::memory_order_relaxed);  // NULL unless a measurement build was given one
}
// workspace for the split last round (NULL: never split): kSplitWorkspaceBytes, 16-byte aligned, counters zero
inline float* split_workspace(void* workspace, int64_t workspace_bytes) {
  if (workspace == nullptr || workspace_bytes < kSplitWorkspaceBytes || !aligned16(workspace)) return nullptr;
  return static_cast<float*>(workspace);
}
}  // namespace

static int grouped_gemm_impl(const void* a, int32_t a_gather_div, const void* w, int32_t N, int32_t K,
                             const ck_segments* seg, int32_t epilogue, void* y, void* y_t, int64_t ld_t, void* aux,
                             const void* aux_in, int32_t dtype, void* stream, void* workspace, int64_t workspace_bytes) {
  const char* name = "ck_grouped_gemm";
  if (int rc = check_segments(seg, name)) return rc;
  CK_REQUIRE(N >= 8 && K >= 8 && N % 8 == 0 && K % 8 == 0, "%s: N=%d and K=%d must be positive multiples of 8", name, N, K);
  CK_REQUIRE(a_gather_div >= 0, "%s: a_gather_div=%d is negative", name, a_gather_div);
  int act_kind = CK_ACT_SWIGLU;
  if (epilogue == CK_EPI_GLU) {  // same tiles and outputs as the SwiGLU epilogue, another gate function
    act_kind = CK_ACT_GLU;
    epilogue = CK_EPI_SWIGLU;
  } else if (epilogue == CK_EPI_GELU_TANH) {  // the grouped epilogue with the activation as a second output
    CK_REQUIRE(aux != nullptr && y_t == nullptr, "%s: the GELU epilogue needs aux and takes no y_t", name);
    CK_REQUIRE(aligned16(aux), "%s: aux must be 16-byte aligned", name);
    act_kind = CK_ACT_GELU_TANH;
    epilogue = CK_EPI_GROUPED;
  } else if (epilogue == CK_EPI_GROUPED || epilogue == CK_EPI_SCATTER) {
    aux = nullptr;  // no second output
  }
  CK_REQUIRE(epilogue >= CK_EPI_GROUPED && epilogue <= CK_EPI_SWIGLU_BWD, "%s: unknown epilogue %d", name, epilogue);
  if (seg->max_rows == 0) return CK_OK;
  CK_REQUIRE(a && w && y, "%s: a, w and y are required", name);
  CK_REQUIRE(aligned16(a) && aligned16(w), "%s: a and w must be 16-byte aligned", name);
  CK_REQUIRE(y_t == nullptr || (ld_t >= seg->max_rows && ld_t % 8 == 0 && (reinterpret_cast<uintptr_t>(y_t) & 7) == 0),
             "%s: y_t needs ld_t >= max_rows, ld_t %% 8 == 0 and 8-byte alignment", name);
  CK_REQUIRE(epilogue != CK_EPI_SCATTER || y_t == nullptr, "%s: the scatter epilogue has no transposed output", name);

  // rows are addressed with 32-bit byte offsets: from the operand base for a, from the expert's slice for w
  CK_REQUIRE((int64_t)N * K * 2 < ((int64_t)1 << 32), "%s: one expert's weight matrix must stay below 4 GiB", name);
  const bool line_kernel = seg->align == kLineBM && K % kLineK == 0 && epilogue != CK_EPI_SWIGLU_BWD &&
                           !force_register_pipeline() && line_kernel_enabled();
  // the 128-byte-row kernel addresses a grouped input from each tile's first row; the general kernel from the operand base
  CK_REQUIRE(a_gather_div > 0 || line_kernel || seg->max_rows * (int64_t)K * 2 < ((int64_t)1 << 32),
             "%s: the grouped input must stay below 4 GiB", name);
  GemmParams prm = {};
  prm.a = a;
  prm.w = w;
  prm.lda = K;
  prm.ldw = K;
  prm.w_expert_stride = (int64_t)N * K;
  prm.a_gather_div = a_gather_div;
  prm.act_kind = act_kind;
  prm.N = N;
  prm.K = K;
  fill_segments(prm, seg);
  prm.y = y;
  prm.y_t = y_t;
  prm.ld_t = ld_t;
  prm.aux = aux;
  prm.aux_in = aux_in;
  prm.split_ws = split_workspace(workspace, workspace_bytes);
  int out_cols = N;  // columns that tile along the grid
  if (epilogue == CK_EPI_SWIGLU) {
    CK_REQUIRE(N % 16 == 0 && aux != nullptr, "%s: the SwiGLU epilogue needs N = 2*I with I %% 8 == 0 and aux", name);
    prm.I = N / 2;
    out_cols = N / 2;
  } else if (epilogue == CK_EPI_SWIGLU_BWD) {
    CK_REQUIRE(aux_in != nullptr, "%s: the SwiGLU-backward epilogue needs aux_in", name);
    prm.I = N;
  }
  const int64_t m_tiles = seg->max_rows / seg->align;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // kSwiglu tiles cover BN/2 activation columns each
  auto n_tiles_for = [&](int bn) { return (int)ceil_div(out_cols, epilogue == CK_EPI_SWIGLU ? bn / 2 : bn); };
  CK_REQUIRE(aux_in == nullptr || epilogue != CK_EPI_SWIGLU,
             "%s: the bias operand (aux_in) goes with the grouped / scatter epilogues", name);
  if (line_kernel) {
    const bool swiglu = epilogue == CK_EPI_SWIGLU;
    const int bn = 256;
    prm.n_tiles = (int)ceil_div(out_cols, swiglu ? bn / 2 : bn);
    const int64_t line_blocks = m_tiles * prm.n_tiles;
    CK_REQUIRE(line_blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
    return launch_line(prm, epilogue, bn, false, dtype, (unsigned)line_blocks, s, name);
  }
  const int bn = seg->align;  // square tiles
  prm.n_tiles = n_tiles_for(bn);
  const int64_t blocks = m_tiles * prm.n_tiles;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
#define CK_GEMM_MODE(MODE) \
  launch_by_tile<scalar_t, MODE>(prm, seg->align, (unsigned)blocks, (unsigned)blocks, s, name)
  CK_DISPATCH_HALF(dtype, name, {
    switch (epilogue) {
      case CK_EPI_GROUPED: return CK_GEMM_MODE(kGrouped);
      case CK_EPI_SCATTER: return CK_GEMM_MODE(kScatter);
      case CK_EPI_SWIGLU: return CK_GEMM_MODE(kSwiglu);
      default: return CK_GEMM_MODE(kSwigluBwd);
    }
  });
#undef CK_GEMM_MODE
  return CK_OK;
}

extern "C" int ck_grouped_gemm(const void* a, int32_t a_gather_div, const void* w, int32_t N, int32_t K,
                               const ck_segments* seg, int32_t epilogue, void* y, void* y_t, int64_t ld_t, void* aux,
                               const void* aux_in, int32_t dtype, void* stream) {
  return grouped_gemm_impl(a, a_gather_div, w, N, K, seg, epilogue, y, y_t, ld_t, aux, aux_in, dtype, stream, nullptr, 0);
}

extern "C" int ck_grouped_gemm_ws(const void* a, int32_t a_gather_div, const void* w, int32_t N, int32_t K,
                                  const ck_segments* seg, int32_t epilogue, void* y, void* y_t, int64_t ld_t, void* aux,
                                  const void* aux_in, int32_t dtype, void* stream, void* workspace,
                                  int64_t workspace_bytes) {
  return grouped_gemm_impl(a, a_gather_div, w, N, K, seg, epilogue, y, y_t, ld_t, aux, aux_in, dtype, stream, workspace,
                           workspace_bytes);
}

extern "C" int64_t ck_grouped_gemm_workspace_bytes(void) { return kSplitWorkspaceBytes; }

static int grouped_gemm_nn_impl(const void* a, const void* w, int32_t N, int32_t K, const ck_segments* seg,
                                int32_t epilogue, void* y, int32_t dtype, void* stream, void* workspace,
                                int64_t workspace_bytes) {
  const char* name = "ck_grouped_gemm_nn";
  if (int rc = check_segments(seg, name)) return rc;
  CK_REQUIRE(seg->align == kLineBM, "%s: needs 256-row tiles (sort with align = 256)", name);
  CK_REQUIRE(N >= 8 && N % 8 == 0, "%s: N=%d must be a positive multiple of 8", name, N);
  CK_REQUIRE(K >= kLineK && K % kLineK == 0, "%s: K=%d must be a positive multiple of %d", name, K, kLineK);
  CK_REQUIRE(epilogue == CK_EPI_GROUPED || epilogue == CK_EPI_SCATTER, "%s: epilogue %d is not grouped or scatter", name,
             epilogue);
  if (seg->max_rows == 0) return CK_OK;
  CK_REQUIRE(a && w && y && aligned16(a) && aligned16(w), "%s: NULL or misaligned pointer", name);
  CK_REQUIRE((int64_t)N * K * 2 < ((int64_t)1 << 32), "%s: one expert's weight matrix must stay below 4 GiB", name);
  GemmParams prm = {};
  prm.a = a;
  prm.w = w;
  prm.lda = K;
  prm.ldw = N;  // rows of w are contraction indices, N columns each
  prm.w_expert_stride = (int64_t)N * K;
  prm.N = N;
  prm.K = K;
  fill_segments(prm, seg);
  prm.y = y;
  prm.split_ws = split_workspace(workspace, workspace_bytes);
  prm.n_tiles = (int)ceil_div(N, 256);
  const int64_t blocks = (seg->max_rows / seg->align) * prm.n_tiles;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  return launch_line(prm, epilogue, 256, true, dtype, (unsigned)blocks, static_cast<hipStream_t>(stream), name);
}

extern "C" int ck_grouped_gemm_nn(const void* a, const void* w, int32_t N, int32_t K, const ck_segments* seg,
                                  int32_t epilogue, void* y, int32_t dtype, void* stream) {
  return grouped_gemm_nn_impl(a, w, N, K, seg, epilogue, y, dtype, stream, nullptr, 0);
}

extern "C" int ck_grouped_gemm_nn_ws(const void* a, const void* w, int32_t N, int32_t K, const ck_segments* seg,
                                     int32_t epilogue, void* y, int32_t dtype, void* stream, void* workspace,
                                     int64_t workspace_bytes) {
  return grouped_gemm_nn_impl(a, w, N, K, seg, epilogue, y, dtype, stream, workspace, workspace_bytes);
}

extern "C" int ck_grouped_gemm_dw_rows(const void* a, const void* b, int32_t M, int32_t N, const ck_segments* seg,
                                       void* dw, int32_t dtype, void* stream) {
  const char* name = "ck_grouped_gemm_dw_rows";
  if (int rc = check_segments(seg, name)) return rc;
  CK_REQUIRE(a && b && dw, "%s: NULL argument", name);
  CK_REQUIRE(seg->align % kLineK == 0, "%s: segments must start at multiples of %d rows (align=%d)", name, kLineK, seg->align);
  CK_REQUIRE(M >= kLineBM && N >= 256 && M % 8 == 0 && N % 8 == 0,
             "%s: M=%d N=%d must be multiples of 8 and at least 256", name, M, N);
  CK_REQUIRE(aligned16(a) && aligned16(b), "%s: operands need 16-byte alignment", name);
  GemmParams prm = {};
  prm.a = a;
  prm.w = b;
  prm.lda = M;
  prm.ldw = N;
  prm.M = M;
  prm.N = N;
  fill_segments(prm, seg);
  prm.y = dw;
  prm.m_tiles = (int)ceil_div(M, kLineBM);
  prm.n_tiles = (int)ceil_div(N, 256);
  const int64_t blocks = (int64_t)prm.m_tiles * prm.n_tiles * seg->num_experts;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  return launch_line(prm, kDw, 256, true, dtype, (unsigned)blocks, static_cast<hipStream_t>(stream), name);
}

extern "C" int ck_grouped_gemm_dw(const void* a_t, const void* b_t, int64_t ld_t, int32_t M, int32_t N,
                                  const ck_segments* seg, void* dw, int32_t dtype, void* stream) {
  const char* name = "ck_grouped_gemm_dw";
  if (int rc = check_segments(seg, name)) return rc;
  CK_REQUIRE(M >= 1 && N >= 1, "%s: M=%d N=%d must be positive", name, M, N);
  CK_REQUIRE(a_t && b_t && dw, "%s: NULL argument", name);
  CK_REQUIRE(ld_t >= seg->max_rows && ld_t % 8 == 0 && aligned16(a_t) && aligned16(b_t),
             "%s: operands need ld_t >= max_rows, ld_t %% 8 == 0 and 16-byte alignment", name);
  CK_REQUIRE((int64_t)M * ld_t * 2 < ((int64_t)1 << 32) && (int64_t)N * ld_t * 2 < ((int64_t)1 << 32),
             "%s: each transposed operand must stay below 4 GiB", name);
  GemmParams prm = {};
  prm.a = a_t;
  prm.w = b_t;
  prm.lda = ld_t;
  prm.ldw = ld_t;
  prm.M = M;
  prm.N = N;
  fill_segments(prm, seg);
  prm.y = dw;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // tile size follows the problem, not the segment alignment: small weight matrices get 128x128 tiles
  const bool big = (M >= 1024 && N >= 1024);
  if (big && !force_register_pipeline() && line_kernel_enabled()) {
    const int bn = 256;
    prm.m_tiles = (int)ceil_div(M, kLineBM);
    prm.n_tiles = (int)ceil_div(N, bn);
    const int64_t line_blocks = (int64_t)prm.m_tiles * prm.n_tiles * seg->num_experts;
    CK_REQUIRE(line_blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
    return launch_line(prm, kDw, bn, false, dtype, (unsigned)line_blocks, s, name);
  }
  const int bt = big ? 256 : 128;
  prm.m_tiles = (int)ceil_div(M, bt);
  prm.n_tiles = (int)ceil_div(N, bt);
  const int64_t blocks = (int64_t)prm.m_tiles * prm.n_tiles * seg->num_experts;
  CK_REQUIRE(blocks < (int64_t)0x7fffffff, "%s: grid too large", name);
  CK_DISPATCH_HALF(dtype, name, {
    if (big) return launch<scalar_t, 256, 256, kDw>(prm, (unsigned)blocks, s, name);
    return launch<scalar_t, 128, 128, kDw>(prm, (unsigned)blocks, s, name);
  });
  return CK_OK;
}
