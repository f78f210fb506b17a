// Scattered grouped GEMM with 128-byte LDS rows: 256 x BN block tiles (BN = 256 or 384), bf16 / f16 inputs, fp32
// accumulation.
//
// Why 128-byte rows: the grouped GEMMs are bound by L2 -> LDS load throughput, and that throughput depends on how many
// contiguous bytes a tile row fetches per request: measured chip-wide on L2-resident panels, global_load_lds_dwordx4
// streams 15 TB/s with 64 contiguous bytes per row and 27 TB/s with 128 (a full cache line) or more. So a K step is 64
// elements = one 128-byte line per tile row. A stage is then 64 KiB (BN = 256) or 80 KiB (BN = 384), and two stages fill
// the LDS: step kt multiplies out of one stage while the loads of step kt + 1 fill the other.
//
// Workgroup = 8 waves (two per SIMD) in a 4 x 2 grid, wave tile 64 x BN/2 = 2 x (BN/64) v_mfma_f32_32x32x16 blocks.
// Fragments rotate through the four 16-wide slices of a step. BN = 384 has registers for one fragment set: a register is
// reloaded for the next slice as soon as the last MFMA that reads it has issued. BN = 256 keeps two sets and reads the
// next slice's fragments a whole slice ahead. One barrier per step, in front of the last slice: by then
// every wave has read the whole current stage (its last-slice fragments are in registers) and the next stage has landed,
// so the loads of step kt + 2 go out under the last slice's MFMAs, as do the fragment reads of step kt + 1.
// BN = 384 carries 20 % more FLOPs per loaded byte (153.6 against 128) and is used where the contraction is long.
#include <stdlib.h>

#include "gemm_common.h"

#ifndef CK_ABLATE
#define CK_ABLATE 0  // measurement builds only: 1 no barrier, 2 no loads in the loop, 4 no fragment reads, 8 no wait for the loads, 16 every step loads the first two K steps again (L2 hits), 32 no epilogue, 64 no MFMA, 128 no row-major output stores, 512 single fragment set at BN = 256
#endif

namespace ck {
namespace {

constexpr int BM = 256;
constexpr int WGM = 4;                     // waves along M (always 2 along N)
constexpr int NW = 2 * WGM, NT = 64 * NW;
constexpr int WM = BM / WGM, MI = WM / 32;  // 64-row wave tile: 2 row blocks
constexpr int BK = 64, KS = BK / 16, NSTAGE = 2;
constexpr int kRowBytes = BK * 2;  // 128: one cache line per tile row and K step
constexpr int A_LD = BM * kRowBytes / (1024 * NW);  // 1 KiB wave-loads per wave and K step
static_assert(MI == 2, "the slice schedule below is written for two A row blocks per wave");

// 16-byte chunk c of row r sits in slot c ^ swz128(r): 16 lanes reading one chunk index of 16 consecutive rows (one phase
// of a ds_read_b128) then touch all 64 banks once -- even rows cover banks 0-31 with 8 distinct slots, odd rows 32-63.
__device__ inline int swz128(int row) { return (row >> 1) & 7; }

template <int BN>
struct Tile {
  static constexpr int WN = BN / 2, NI = WN / 32;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int B_LD = BN * kRowBytes / (1024 * NW);
  static constexpr int kLoadsPerStep = A_LD + B_LD;
  static constexpr size_t kLdsBytes = (size_t)NSTAGE * kStageBytes;
  // epilogue: slab of half the tile's columns (half of each wave's column blocks), kept transposed S[col][row]
  static constexpr int kSlabBlocks = NI / 2, kSlabCols = 2 * kSlabBlocks * 32, kSlabLd = BM + 4;
  static constexpr int kMetaOffset = kSlabCols * kSlabLd * 2;  // after the slab: output row of every tile row (scatter)
  static_assert(kLdsBytes <= 160 * 1024, "two stages fit the LDS of a CU");
  static_assert(kMetaOffset % 16 == 0 && kMetaOffset + BM * 4 <= (int)kLdsBytes, "slab and row table fit in the dead stages");
  static_assert(kLoadsPerStep <= 2 * NI, "every load of a step has an MFMA of the last slice to hide behind");
};

// BT ("B as stored by its owner"): the weight operand is [contraction, columns] row-major, i.e. contraction-strided --
// the input-gradient GEMMs read W[e] [out, in] this way instead of a transposed copy. Its stage holds 64 contraction rows
// of BN columns, and fragments come out of LDS through ds_read_b64_tr_b16 (see read_b).
template <typename T, int MODE, int BN, bool BT>
__global__ __launch_bounds__(NT) void grouped_gemm_line_kernel(const GemmParams prm) {
  typedef Tile<BN> TL;
  constexpr int WN = TL::WN, NI = TL::NI, B_LD = TL::B_LD, kLoadsPerStep = TL::kLoadsPerStep, kStageBytes = TL::kStageBytes;
  constexpr int kSlabBlocks = TL::kSlabBlocks, kSlabCols = TL::kSlabCols, kSlabLd = TL::kSlabLd, kMetaOffset = TL::kMetaOffset;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  char* lds_c = reinterpret_cast<char*>(lds_raw);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile (same XCD-aware orders as the 256 x 256 kernel)
  int mt, nt, expert;
  int64_t k_begin = 0;
  int k_len;
  if constexpr (MODE == kDw) {
    const int per_expert = prm.m_tiles * prm.n_tiles;
    const bool m_major = prm.m_tiles >= prm.n_tiles;
    const int major = m_major ? prm.m_tiles : prm.n_tiles, minor = m_major ? prm.n_tiles : prm.m_tiles;
    int pid = blockIdx.x, a, b;
    if (major % kXcds == 0) {  // every XCD gets a slice of every expert's tile grid (experts differ in contraction length)
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
    k_len = (int)((prm.counts[expert] + BK - 1) / BK * BK);  // the transposed operands are zero up to the tile boundary
  } else {
    const int live_m = prm.seg_starts[prm.num_experts] / prm.align;
    const int total = live_m * prm.n_tiles;
    int pid = blockIdx.x;
    if (pid >= total) return;
    const int per_xcd = total / kXcds;
    if (pid < per_xcd * kXcds) pid = (pid % kXcds) * per_xcd + pid / kXcds;
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
    if (tid < BM && m0 + tid < valid_end) scatter_row = prm.row_slot[m0 + tid];
  }
  static_assert(NT >= BM, "one thread per tile row");

  f32x16 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- global -> LDS addressing: lane l of a wave-load fills slot l (16 bytes) of 64 consecutive slots = 8 rows of 128 B;
  // the lane fetches the chunk that belongs in its slot, so the 8 lanes of a row read one whole line of global memory
  // AT (weight gradients from row-major operands): both operands are [grouped rows, columns], i.e. contraction-strided;
  // the A stage then has the layout described for BT below (64 contraction rows of BM columns) and its fragments come out
  // through the same transposing reads. Rows past the expert's count are zeroed in LDS (zero_pad_slots).
  constexpr bool AT = BT && MODE == kDw;
  const char* a_base = static_cast<const char*>(prm.a);
  const char* b_base = static_cast<const char*>(prm.w);
  if constexpr (MODE != kDw) b_base += (int64_t)expert * prm.w_expert_stride * 2;
  if constexpr (AT) {
    a_base += k_begin * prm.lda * 2;
    b_base += k_begin * prm.ldw * 2;
  }
  if constexpr (MODE != kDw) {
    if (prm.a_gather_div <= 0) a_base += m0 * prm.lda * 2;
  }
  constexpr int kAtRowBytes = BM * 2;
  auto swap02 = [](int w) { return (w & ~5) | ((w & 1) << 2) | ((w >> 2) & 1); };
  uint32_t a_off[A_LD], b_off[B_LD];
#pragma unroll
  for (int t = 0; t < A_LD; ++t) {
    if constexpr (AT) {
      const int pos = (wave * A_LD + t) * 1024 + lane * 16;  // byte position of this lane's slot in the A stage
      const int n = pos / kAtRowBytes, slot16 = (pos % kAtRowBytes) / 16;
      const int q = swap02((slot16 >> 1) ^ (n & 3));
      int64_t col = m0 + (2 * q + (slot16 & 1)) * 8;
      if (col >= prm.M) col = m0;  // ragged edge: re-read a valid chunk, never stored
      a_off[t] = (uint32_t)(((int64_t)n * prm.lda + col) * 2);
    } else {
      const int r = (wave * A_LD + t) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ swz128(r);
      int64_t row;
      if constexpr (MODE == kDw) {
        row = min(m0 + r, (int64_t)prm.M - 1);
      } else {
        int64_t p = m0 + r;
        if (p >= valid_end) p = valid_end - 1;  // pad rows re-read a valid row; their results are never stored
        // grouped input: offsets are taken from the tile's first row (a_base is moved there below), so that only a tile,
        // not the whole operand, has to fit 32-bit offsets; gathered input: from the start of the token-order tensor
        row = prm.a_gather_div > 0 ? (int64_t)(prm.row_slot[p] / prm.a_gather_div) : p - m0;
      }
      a_off[t] = (uint32_t)((row * prm.lda + k_begin) * 2 + c * 16);
    }
  }
  // BT: 32-byte window q of contraction row n sits at window position swap02(q) ^ (n & 3) of the row (swap02 exchanges
  // bits 0 and 2 of the window index): the 4 rows x 32 bytes one 16-lane group of a transposing read touches fill one
  // 128-byte block, and the neighbouring group (next 16 columns) falls into the other half of the banks.
  constexpr int kBtRowBytes = BN * 2, kBtWindows = kBtRowBytes / 32;
#pragma unroll
  for (int t = 0; t < B_LD; ++t) {
    if constexpr (BT) {
      const int pos = (wave * B_LD + t) * 1024 + lane * 16;  // byte position of this lane's slot in the B stage
      const int n = pos / kBtRowBytes, slot16 = (pos % kBtRowBytes) / 16;
      const int q = swap02((slot16 >> 1) ^ (n & 3));           // the window that belongs at this position
      int64_t col = (int64_t)nt * BN + (2 * q + (slot16 & 1)) * 8;
      if (col >= prm.N) col = (int64_t)nt * BN;                // ragged edge: re-read a valid chunk, never stored
      b_off[t] = (uint32_t)(((int64_t)n * prm.ldw + col) * 2);
    } else {
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
      b_off[t] = (uint32_t)((n * prm.ldw + k_begin) * 2 + c * 16);
    }
  }
  static_assert(!BT || kBtWindows % 8 == 0 || kBtWindows == 24, "window swizzle works on groups of 8 windows");
  const int nk = k_len / BK;

  auto dma16 = [&](const char* src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "m0");
  };
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_c;
  const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * A_LD * 1024);
  const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * kRowBytes + wave * B_LD * 1024);
  auto issue_one = [&](int step, int g) {
    const int64_t kb = (CK_ABLATE & 16) ? (int64_t)(step & 1) * kRowBytes : (int64_t)step * kRowBytes;
    const int64_t kb_b = BT ? (int64_t)((CK_ABLATE & 16) ? (step & 1) : step) * BK * prm.ldw * 2 : kb;  // BT: 64 contraction rows further down
    const int64_t kb_a = AT ? (int64_t)step * BK * prm.lda * 2 : kb;
    const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
    if (g < A_LD) dma16(a_base + kb_a + a_off[g], wave_a + st + g * 1024);
    else dma16(b_base + kb_b + b_off[g - A_LD], wave_b + st + (g - A_LD) * 1024);
  };
  auto issue = [&](int step) {
#pragma unroll
    for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
  };

  // ---- fragments: slice sl of a row is its 16-byte chunks 2 sl (lanes 0-31) and 2 sl + 1 (lanes 32-63)
  typedef typename Mfma<T>::frag frag_t;
  const int fsw = swz128(lane & 31), fh = lane >> 5;
  int slice_off[KS];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) slice_off[sl] = ((2 * sl + fh) ^ fsw) * 16;
  const int fa_row = (wm * WM + (lane & 31)) * kRowBytes;
  const int fb_row = BM * kRowBytes + (wn * WN + (lane & 31)) * kRowBytes;
  // 256-wide tiles have the registers for two fragment sets: the reads for the next slice then go out a whole slice ahead
  constexpr bool kDouble = BN == 256 && (CK_ABLATE & 512) == 0;  // (measured: 2.5 to 3.5 % faster launches)
  constexpr int kSets = kDouble ? 2 : 1;
  frag_t fa[kSets][MI], fb[kSets][NI];
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short tr16x4;
  int at_off[MI];
  if constexpr (AT) {  // as bt_off below, on the A stage
    const int g = lane >> 4, i = lane & 15, n_low = i >> 2;
#pragma unroll
    for (int b = 0; b < MI; ++b) {
      const int q = (wm * WM + b * 32) / 16 + (g & 1);
      at_off[b] = (8 * (g >> 1) + n_low) * kAtRowBytes + (swap02(q) ^ n_low) * 32 + 8 * (i & 3);
    }
  }
  auto read_a = [&](int stage, int sl, int i) {
    if constexpr (AT) {
      const char* p = lds_c + stage * kStageBytes + at_off[i] + 16 * sl * kAtRowBytes;
      union {
        tr16x4 h[2];
        frag_t f;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p + 4 * kAtRowBytes));
      fa[kDouble ? (sl & 1) : 0][i] = u.f;
    } else {
      fa[kDouble ? (sl & 1) : 0][i] = *reinterpret_cast<const frag_t*>(lds_c + stage * kStageBytes + slice_off[sl] + fa_row + i * 32 * kRowBytes);
    }
  };
  // BT: lane l = 16 g + i of a transposing read points at 4 consecutive columns (4 (i % 4) ..) of contraction row i / 4
  // of a 4-row x 16-column patch and receives the 4 rows of column i; two reads (rows +0..3, +4..7) make the 8 contraction
  // values of column 16 (g % 2) + i for k-half g / 2 -- the MFMA's B layout.
  int bt_off[NI];
  if constexpr (BT) {
    const int g = lane >> 4, i = lane & 15, n_low = i >> 2;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int q = (wn * WN + j * 32) / 16 + (g & 1);
      bt_off[j] = BM * kRowBytes + (8 * (g >> 1) + n_low) * kBtRowBytes + (swap02(q) ^ n_low) * 32 + 8 * (i & 3);
    }
  }
  auto read_b = [&](int stage, int sl, int j) {
    if constexpr (BT) {
      const char* p = lds_c + stage * kStageBytes + bt_off[j] + 16 * sl * kBtRowBytes;
      union {
        tr16x4 h[2];
        frag_t f;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p + 4 * kBtRowBytes));
      fb[kDouble ? (sl & 1) : 0][j] = u.f;
    } else {
      fb[kDouble ? (sl & 1) : 0][j] = *reinterpret_cast<const frag_t*>(lds_c + stage * kStageBytes + slice_off[sl] + fb_row + j * 32 * kRowBytes);
    }
  };
  auto mfma = [&](int set, int i, int j) {
    if constexpr ((CK_ABLATE & 64) != 0) {
      asm volatile("" ::"v"(fa[set][i]), "v"(fb[set][j]));
      return;
    }
    acc[i][j] = Mfma<T>::run(fa[set][i], fb[set][j], acc[i][j]);
  };

  // AT: contraction rows past the expert's count (the ragged end of its last K step) hold whatever the buffers hold.
  // Every lane overwrites, with zeros, the slots of such rows that its own loads filled -- after those loads have
  // landed, before the barrier that publishes the stage; both operands, so no 0 * Inf can arise.
  auto zero_pad_slots = [&](int step) {
    if constexpr (AT) {
      const int rows_here = (int)prm.counts[expert] - step * BK;
      if (rows_here >= BK) return;
      char* stage = lds_c + (step & (NSTAGE - 1)) * kStageBytes;
#pragma unroll
      for (int t = 0; t < A_LD; ++t) {
        const int pos = (wave * A_LD + t) * 1024 + lane * 16;
        if (pos / kAtRowBytes >= rows_here) *reinterpret_cast<vec16*>(stage + pos) = zero16();
      }
#pragma unroll
      for (int t = 0; t < B_LD; ++t) {
        const int pos = (wave * B_LD + t) * 1024 + lane * 16;
        if (pos / kBtRowBytes >= rows_here) *reinterpret_cast<vec16*>(stage + BM * kRowBytes + pos) = zero16();
      }
    }
  };

  if (nk > 0) {
    issue(0);
    if (nk > 1) {
      issue(1);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLoadsPerStep) : "memory");  // step 0 landed, all waves
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      zero_pad_slots(0);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
#pragma unroll
    for (int i = 0; i < MI; ++i) read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < NI; ++j) read_b(0, 0, j);

    // One 16-wide slice: 2 * NI MFMAs, A row block 0 then 1, and the reloads for the slice after it (ns, nsl): fa[0] once
    // row block 0 is done, fb[j] after the MFMA (1, j), fa[1] at the end.
    // Slices 0 .. 2 of a step: the next slice is in the same stage.
    // Slice 3: the next slice is slice 0 of step kt + 1 in the other stage. Phase 0 / 1: wait for that stage
    //   (the only loads in flight) and for this wave's own fragment reads, then meet the other waves -- the whole current
    //   stage has been read by everyone, so in phase 0 the loads of step kt + 2 overwrite it under this slice's MFMAs.
    //   Phase 1 is step nk - 2 (nothing left to fetch), phase 2 the last step (nothing to wait for, nothing to reload).
    auto slice = [&](int kt, auto sl, auto phase, auto idle) {
      constexpr bool kIdle = decltype(idle)::value;  // this wave's 64 rows are all pad rows: no fragments, no MFMAs
      constexpr bool kLast = decltype(sl)::value == KS - 1;
      constexpr int kPhase = decltype(phase)::value;
      const int ns = kLast ? (kt + 1) & (NSTAGE - 1) : kt & (NSTAGE - 1);
      constexpr int nsl = kLast ? 0 : decltype(sl)::value + 1;
      constexpr bool kReload = !(kLast && kPhase == 2) && !(CK_ABLATE & 4) && !kIdle;
      if constexpr (kLast && kPhase < 2) {
        if constexpr ((CK_ABLATE & 1) != 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        else if constexpr ((CK_ABLATE & 8) != 0) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else if constexpr (AT && kPhase == 1) {  // the stage that has just landed is the last K step
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          zero_pad_slots(kt + 1);
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        } else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
      constexpr int cur = kDouble ? (decltype(sl)::value & 1) : 0;
      if constexpr (kDouble) {
        // reads for the next slice in the order it needs them, one after each of the first MI + NI MFMAs
        auto reload = [&](int n) {
          if (n == 0) read_a(ns, nsl, 0);
          else if (n <= NI) read_b(ns, nsl, n - 1);
          else read_a(ns, nsl, 1);
        };
#pragma unroll
        for (int n = 0; n < 2 * NI; ++n) {
          if constexpr (!kIdle) mfma(cur, n / NI, n % NI);
          if constexpr (kLast && kPhase == 0 && !(CK_ABLATE & 2)) {
            if (n < kLoadsPerStep) issue_one(kt + 2, n);
          }
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (kReload) {
            if (n < MI + NI) reload(n);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          if constexpr (!kIdle) mfma(0, 0, j);
          if constexpr (kLast && kPhase == 0 && !(CK_ABLATE & 2)) {
            if (j < kLoadsPerStep) issue_one(kt + 2, j);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (kReload) read_a(ns, nsl, 0);
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          if constexpr (!kIdle) mfma(0, 1, j);
          if constexpr (kLast && kPhase == 0 && !(CK_ABLATE & 2)) {
            if (NI + j < kLoadsPerStep) issue_one(kt + 2, NI + j);
          }
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (kReload) read_b(ns, nsl, j);
        }
        if constexpr (kReload) read_a(ns, nsl, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    auto k_loop = [&](auto idle) {
      auto k_step = [&](int kt, auto phase) { static_for<KS>([&](auto sl) { slice(kt, sl, phase, idle); }); };
      int kt = 0;
      for (; kt + 2 < nk; ++kt) k_step(kt, std::integral_constant<int, 0>{});
      if (kt + 2 == nk) k_step(kt++, std::integral_constant<int, 1>{});
      k_step(kt, std::integral_constant<int, 2>{});
    };
    // A wave whose 64 tile rows all lie past the expert's last row (the tile is the ragged end of a segment) still
    // issues its share of the loads and meets every barrier, but multiplies nothing: the wave it shares a SIMD with
    // then has the matrix pipe to itself. Its accumulators stay zero and its rows are never stored.
    bool wave_idle = false;
    if constexpr (MODE != kDw) wave_idle = m0 + wm * WM >= valid_end;
    if (__builtin_amdgcn_readfirstlane(wave_idle)) k_loop(std::true_type{});
    else k_loop(std::false_type{});
  }

  // ---- epilogue through LDS. Lane holds, per 32x32 block and q in 0..3, rows 8q + 4*(lane/32) + 0..3 of column lane%32:
  // 8-byte writes into the transposed slab; ds_read_b64_tr_b16 brings row-major 16-byte pieces back out (a lane ends up
  // with 8 consecutive columns of one row); transposed outputs leave with plain 16-byte reads.
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  T* slab = reinterpret_cast<T*>(lds_raw);
  int* scatter_rows = reinterpret_cast<int*>(lds_c + kMetaOffset);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the stages
  if constexpr (MODE == kScatter) {
    if (tid < BM) scatter_rows[tid] = scatter_row;  // first read after the first slab barrier below
  }
  const int col_in_block = lane & 31;
  const int row_quad = (lane >> 5) * 4;
  const T kZero = Elem<T>::down(0.f);
  // most tiles have no pad rows: then nothing is tested per element (the test is a 64-bit compare and a branch each)
  const bool tile_full = MODE == kDw || m0 + BM <= valid_end;
  if constexpr ((CK_ABLATE & 32) != 0) {
    float keep = 0.f;
    static_for<MI>([&](auto i) { static_for<NI>([&](auto j) { keep += acc[i][j][0]; }); });
    if (keep == 123.456f) static_cast<float*>(prm.y)[0] = keep;
    return;
  }

  auto stage_blocks = [&](auto&& value /* (i, jj, q, s) -> T */) {
    static_for<MI>([&](auto i) {
      static_for<kSlabBlocks>([&](auto jj) {
        static_for<4>([&](auto q) {
          const int r = wm * WM + i * 32 + 8 * q + row_quad;
          const int c = wn * (kSlabBlocks * 32) + jj * 32 + col_in_block;
          store4(slab + c * kSlabLd + r, value(i, jj, q, std::integral_constant<int, 0>{}),
                 value(i, jj, q, std::integral_constant<int, 1>{}), value(i, jj, q, std::integral_constant<int, 2>{}),
                 value(i, jj, q, std::integral_constant<int, 3>{}));
        });
      });
    });
  };
  // slab column -> column of the block tile, for pass `pass` (which half of each wave's column blocks is staged)
  auto tile_col = [&](int sc, int pass) {
    return (sc / (kSlabBlocks * 32)) * WN + pass * (kSlabBlocks * 32) + sc % (kSlabBlocks * 32);
  };
  // Row-major drain. 16 lanes take a 4-row x 32-column block (what one transposing read pair delivers); the four lane
  // groups of a wave take two adjacent column blocks of two adjacent row blocks, so that a store instruction writes whole
  // 128-byte lines. The stores are non-temporal: outputs are written once and read by a later launch, and as plain
  // stores they displace the operand panels that neighbouring tiles re-read from L2 (measured on 256 x 256 tiles with
  // K = 2048: 7 to 13 % of the launch). Rows and column pairs are walked in unrolled loops: every address is a per-lane base plus a compile-time offset. row_ptr(tile row) -> address of the
  // output row at the tile's first column (nullptr: pad row), block_col(cb) -> output column of slab column block cb
  // relative to that, cols_left = valid columns from there on, tile_cols = columns the tile spans.
  auto drain_rows = [&](auto&& row_ptr, auto&& block_col, int64_t cols_left, int tile_cols) {
    const int l16 = tid & 15, csel = (tid >> 4) & 1, rsel = (tid >> 5) & 1;
    const int tq = l16 & 3, tj = l16 >> 2;  // as a source lane: which slab column this lane points at
    const int oq = l16 >> 2, oe = l16 & 3;  // as a destination lane: 8 columns oq of row oe of the 4 x 32 block
    constexpr int kColPairs = kSlabCols / 64, kRowIters = (BM / 4) / (2 * NT / kWave);
    static_assert(kSlabCols % 64 == 0 && (BM / 4) % (2 * NT / kWave) == 0, "whole column pairs and row iterations");
    const bool cols_full = cols_left >= tile_cols;
    auto body = [&](auto checked) {
      static_for<kRowIters>([&](auto it) {
        const int rb = (it * (NT / kWave) + wave) * 2 + rsel;
        T* dst_row = row_ptr(rb * 4 + oe);
        if (dst_row != nullptr) dst_row += 8 * oq;
        const T* src_row = slab + (csel * 32 + 8 * tq + tj) * kSlabLd + rb * 4;
        static_for<kColPairs>([&](auto cp) {
          const T* src = src_row + cp * 64 * kSlabLd;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(src + 4 * kSlabLd));
          const int col = csel ? block_col(std::integral_constant<int, 2 * decltype(cp)::value + 1>{}) : block_col(std::integral_constant<int, 2 * decltype(cp)::value>{});
          if (dst_row != nullptr && (!checked || col + 8 * oq < cols_left) && (!(CK_ABLATE & 128) || lo[0] == 12345)) {
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
  auto drain_cols = [&](auto&& out_ptr /* (slab column, tile row) -> address of 8 rows of that column, or nullptr */) {
    constexpr int kChunks = kSlabCols * (BM / 8);
#pragma unroll 4
    for (int ch = tid; ch < kChunks; ch += NT) {
      const int c = ch / (BM / 8), r = (ch % (BM / 8)) * 8;
      T* dst = out_ptr(c, r);
      if (dst != nullptr) store16_nt(dst, load16(slab + c * kSlabLd + r));
    }
  };

  if constexpr (MODE == kDw) {
    T* dw = static_cast<T*>(prm.y) + (int64_t)expert * prm.M * prm.N;
    static_for<2>([&](auto pass) {
      stage_blocks([&](auto i, auto jj, auto q, auto s) {
        return Elem<T>::down(acc[i][pass * kSlabBlocks + jj][4 * q + s]);
      });
      __syncthreads();
      drain_rows(
          [&](int r) -> T* {
            const int64_t m = m0 + r;
            return m < prm.M ? dw + m * prm.N + (int64_t)nt * BN : nullptr;
          },
          [&](auto cb) { return tile_col(cb * 32, pass); }, prm.N - (int64_t)nt * BN, BN);
      __syncthreads();
    });
  } else if constexpr (MODE == kGrouped || MODE == kScatter) {
    T* y = static_cast<T*>(prm.y);
    T* y_t = static_cast<T*>(prm.y_t);
    // optional per-expert bias row (aux_in = bias [E, N]): added to the fp32 accumulators, so that the output is rounded
    // once, like F.linear with a bias. A lane's accumulators of one column block all belong to one output column.
    if constexpr (!BT) {
      if (prm.aux_in != nullptr) {
        const T* bias = static_cast<const T*>(prm.aux_in) + (int64_t)expert * prm.N;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          const int64_t n = (int64_t)nt * BN + wn * WN + j * 32 + col_in_block;
          const float b = n < prm.N ? Elem<T>::up(bias[n]) : 0.f;
#pragma unroll
          for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] += b;
        }
      }
    }
    static_for<2>([&](auto pass) {
      // pad rows are staged as zeros: the transposed copy must hold zeros there
      if (tile_full) {
        stage_blocks([&](auto i, auto jj, auto q, auto s) { return Elem<T>::down(acc[i][pass * kSlabBlocks + jj][4 * q + s]); });
      } else {
        stage_blocks([&](auto i, auto jj, auto q, auto s) {
          const int64_t p = m0 + wm * WM + i * 32 + 8 * q + row_quad + s;
          return p < valid_end ? Elem<T>::down(acc[i][pass * kSlabBlocks + jj][4 * q + s]) : kZero;
        });
      }
      __syncthreads();
      drain_rows(
          [&](int r) -> T* {
            const int64_t p = m0 + r;
            if (!tile_full && p >= valid_end) return nullptr;
            const int64_t row = (MODE == kScatter) ? (int64_t)scatter_rows[r] : p;
            return y + row * prm.N + (int64_t)nt * BN;
          },
          [&](auto cb) { return tile_col(cb * 32, pass); }, prm.N - (int64_t)nt * BN, BN);
      if (MODE == kGrouped && y_t != nullptr) {
        drain_cols([&](int sc, int r) -> T* {
          const int64_t n = (int64_t)nt * BN + tile_col(sc, pass);
          return n < prm.N ? y_t + n * prm.ld_t + m0 + r : nullptr;
        });
      }
      __syncthreads();
    });
  } else {  // kSwiglu: column blocks 0 .. 2 of a wave are up, 3 .. 5 the gate of the same activation columns
    T* pre = static_cast<T*>(prm.y);
    T* act = static_cast<T*>(prm.aux);
    T* act_t = static_cast<T*>(prm.y_t);
    const int64_t two_i = 2 * (int64_t)prm.I;
    auto act_col = [&](int sc) {
      return (int64_t)nt * (BN / 2) + (sc / (kSlabBlocks * 32)) * (WN / 2) + sc % (kSlabBlocks * 32);
    };
    static_for<3>([&](auto pass) {  // 0: up half of the pre-activation, 1: gate half, 2: activation
      auto value = [&](auto i, auto jj, auto q, auto s, bool valid) {
        const T up = Elem<T>::down(acc[i][jj][4 * q + s]);
        const T gate = Elem<T>::down(acc[i][jj + kSlabBlocks][4 * q + s]);
        if (pass == 0) return up;
        if (pass == 1) return gate;
        const float gf = Elem<T>::up(gate);  // from the rounded pre-activation, like the unfused path
        const float sg = sigmoid_fast(gf);
        const T a = Elem<T>::down(prm.act_kind == CK_ACT_GLU ? Elem<T>::up(up) * sg : Elem<T>::up(up) * gf * sg);  // same association as swiglu_fwd_kernel
        return valid ? a : kZero;
      };
      if (tile_full) {
        stage_blocks([&](auto i, auto jj, auto q, auto s) { return value(i, jj, q, s, true); });
      } else {
        stage_blocks([&](auto i, auto jj, auto q, auto s) {
          return value(i, jj, q, s, m0 + wm * WM + i * 32 + 8 * q + row_quad + s < valid_end);
        });
      }
      __syncthreads();
      const int64_t col0 = (int64_t)nt * (BN / 2);  // the tile's first activation column
      drain_rows(
          [&](int r) -> T* {
            const int64_t p = m0 + r;
            if (!tile_full && p >= valid_end) return nullptr;
            if (pass == 0) return pre + p * two_i + col0;
            if (pass == 1) return pre + p * two_i + prm.I + col0;
            return act + p * prm.I + col0;
          },
          [&](auto cb) { return (int)(act_col(cb * 32) - col0); }, prm.I - col0, BN / 2);
      if (pass == 2 && act_t != nullptr) {
        drain_cols([&](int sc, int r) -> T* {
          const int64_t col = act_col(sc);
          return col < prm.I ? act_t + col * prm.ld_t + m0 + r : nullptr;
        });
      }
      __syncthreads();
    });
  }
}

template <typename T, int MODE, int BN, bool BT>
int launch_mode(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  auto kernel = grouped_gemm_line_kernel<T, MODE, BN, BT>;
  constexpr size_t kLds = Tile<BN>::kLdsBytes;
  static bool lds_reserved[kMaxDevices] = {};
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kernel), kLds, lds_reserved, name)) return rc;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(NT), kLds, s, prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

template <typename T, int BN>
int launch_bn(const GemmParams& prm, int mode, bool bt, unsigned blocks, hipStream_t stream, const char* name) {
  if (bt) {  // the input-gradient GEMMs: grouped or scatter epilogue, 256-wide tiles (the 384-wide tile has no registers
             // left for the transposing reads' addresses)
    if constexpr (BN == 256) {
      if (mode == kGrouped) return launch_mode<T, kGrouped, BN, true>(prm, blocks, stream, name);
      if (mode == kScatter) return launch_mode<T, kScatter, BN, true>(prm, blocks, stream, name);
      if (mode == kDw) return launch_mode<T, kDw, BN, true>(prm, blocks, stream, name);  // both operands row-major
    }
    set_error("%s: contraction-strided operands go with 256-wide tiles and the grouped / scatter / dW epilogues", name);
    return CK_ERR_ARG;
  }
  switch (mode) {
    case kGrouped: return launch_mode<T, kGrouped, BN, false>(prm, blocks, stream, name);
    case kScatter: return launch_mode<T, kScatter, BN, false>(prm, blocks, stream, name);
    case kSwiglu: return launch_mode<T, kSwiglu, BN, false>(prm, blocks, stream, name);
    case kDw: return launch_mode<T, kDw, BN, false>(prm, blocks, stream, name);
    default: break;
  }
  set_error("%s: the 128-byte-row kernel has no epilogue %d", name, mode);
  return CK_ERR_ARG;
}

}  // namespace

int launch_line(const GemmParams& prm, int mode, int bn, bool bt, int dtype, unsigned blocks, hipStream_t stream,
                const char* name) {
  CK_DISPATCH_HALF(dtype, name, {
    if (bn == 384) return launch_bn<scalar_t, 384>(prm, mode, bt, blocks, stream, name);
    return launch_bn<scalar_t, 256>(prm, mode, bt, blocks, stream, name);
  });
  return CK_ERR_ARG;
}

}  // namespace ck
