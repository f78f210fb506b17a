// Scattered grouped GEMM with 128-byte LDS rows: 256 x BN block tiles (BN = 256 or 384), bf16 / f16 inputs, fp32
// accumulation on v_mfma_f32_16x16x32.
//
// Why 128-byte rows: the grouped GEMMs are bound by L2 -> LDS load throughput, and that throughput depends on how many
// contiguous bytes a tile row fetches per request: measured chip-wide on L2-resident panels, global_load_lds_dwordx4
// streams 15 TB/s with 64 contiguous bytes per row and 27 TB/s with 128 (a full cache line) or more. So a K step is 64
// elements = one 128-byte line per tile row. A stage is then 64 KiB (BN = 256) or 80 KiB (BN = 384), and two stages fill
// the LDS: step kt multiplies out of one stage while the loads of step kt + 1 fill the other.
//
// Why 16x16x32 blocks: the chip's clock is power-managed and the 16x16x32 instruction costs less energy per FLOP on
// random operands than 32x32x16 (register-only loops on N(0,1) data: 2.04 against 1.70 PFLOP/s).
//
// Workgroup = WGM x 2 waves: 4 x 2 (eight waves, two per SIMD, wave tile 64 x BN/2) or 2 x 2 (four waves, one per SIMD,
// wave tile 128 x 128 with the accumulators in AGPRs: a third less LDS fragment traffic per FLOP). A K step is two
// 32-wide slices; a slice is MI x NI MFMAs on MI + NI 16-byte fragments. One barrier per step, in front of the last
// slice: by then every wave has read the whole current stage (its last-slice fragments are in registers) and the next
// stage has landed, so the loads of step kt + 2 go out under the last slice's MFMAs (spread over the slice), as do the
// fragment reads of step kt + 1.
// BN = 384 carries 20 % more FLOPs per loaded byte (153.6 against 128) and is used where the contraction is long.
#include <stdlib.h>

#include "gemm_common.h"

// Measurement builds only (build.py --define NAME=n --output FILE.so; the product library is built without either):
// CK_ABLATE, a bit set: 2 no loads in the loop, 4 no fragment reads in the loop, 16 every K step loads the first two K
//   steps again (L2 hits), 512 / 1024 the same for the A operand / the weight operand alone, 128 no output stores.
// CK_STAMP=1: every wave adds up the cycles it spends waiting for the loads and at the barrier of each K step and writes
//   them, with its prologue, main-loop and epilogue cycles, to the buffer given to ck_debug_set_trace_buffer.
#ifndef CK_ABLATE
#define CK_ABLATE 0
#endif
#ifndef CK_STAMP
#define CK_STAMP 0
#endif

namespace ck {
namespace {

constexpr int BM = 256;
constexpr int BK = 64, KS = BK / 32, NSTAGE = 2;
constexpr int kRowBytes = BK * 2;  // 128: one cache line per tile row and K step
static_assert(KS == 2, "a K step is two 32-wide slices");

// 16-byte chunk c of row r sits in slot c ^ swz128(r): 16 lanes reading one chunk index of 16 consecutive rows (one phase
// of a ds_read_b128) then touch all 64 banks once -- even rows cover banks 0-31 with 8 distinct slots, odd rows 32-63.
__device__ inline int swz128(int row) { return (row >> 1) & 7; }

template <int BN, int WGM>
struct Tile {
  static constexpr int NW = 2 * WGM, NT = 64 * NW;   // waves: WGM along M, 2 along N
  static constexpr int WM = BM / WGM, MI = WM / 16;  // wave tile rows: 64 (4 row blocks) or 128 (8)
  static constexpr int WN = BN / 2, NI = WN / 16;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int A_LD = BM * kRowBytes / (1024 * NW);  // 1 KiB wave-loads per wave and K step
  static constexpr int B_LD = BN * kRowBytes / (1024 * NW);
  static constexpr int kLoadsPerStep = A_LD + B_LD;
  static constexpr size_t kLdsBytes = (size_t)NSTAGE * kStageBytes;
  // two fragment sets (the next slice is read a whole slice ahead) where the registers allow: 512 per lane with one
  // wave per SIMD, 256 with two
  static constexpr bool kDouble = WGM == 2;  // (contraction-strided operands: see the kernel)
  static_assert(kLdsBytes <= 160 * 1024, "the stages fit the LDS of a CU");
  static_assert(kLoadsPerStep <= MI * NI, "every load of a step has an MFMA of the last slice to hide behind");
  static_assert(NI % 4 == 0, "whole column-block pairs in each half of a wave's columns");
  static_assert(NT >= BM, "one thread per tile row");
};

// BT ("B as stored by its owner"): the weight operand is [contraction, columns] row-major, i.e. contraction-strided --
// the input-gradient GEMMs read W[e] [out, in] this way instead of a transposed copy. Its stage holds 64 contraction rows
// of BN columns, and fragments come out of LDS through ds_read_b64_tr_b16 (see read_b).
// EXTRA: the launch has a bias operand or a transposed side output (y_t); the instantiations without them carry none of
// that code (it cost the common launches spills, and every spill reload waits for the output stores in flight).
template <typename T, int MODE, int BN, bool BT, int WGM, bool EXTRA>
__global__ __launch_bounds__(64 * 2 * WGM) void grouped_gemm_line_kernel(const GemmParams prm) {
  typedef Tile<BN, WGM> TL;
  constexpr int NW = TL::NW, NT = TL::NT, WM = TL::WM, MI = TL::MI, A_LD = TL::A_LD;
  constexpr int WN = TL::WN, NI = TL::NI, B_LD = TL::B_LD, kLoadsPerStep = TL::kLoadsPerStep, kStageBytes = TL::kStageBytes;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  char* lds_c = reinterpret_cast<char*>(lds_raw);
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // uniform: everything derived from it stays in scalar registers
  const int wm = wave >> 1, wn = wave & 1;
  [[maybe_unused]] uint64_t st_begin = 0, st_loop = 0, st_end = 0, st_vm = 0, st_bar = 0, st_s0 = 0, st_s1 = 0, st_mark = 0;
  if constexpr (CK_STAMP != 0) st_begin = clock64();

  // ---- which tile (same XCD-aware orders as the 256 x 256 kernel)
  constexpr bool kSplit = WGM == 2 && (MODE == kGrouped || MODE == kScatter);  // see the split below
  int mt, nt, expert;
  int64_t k_begin = 0;
  int k_len;
  [[maybe_unused]] int split_slot = -1, split_part = -1, split_parts = kSplitParts;
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
    // `expert` so far is a position in the launch order. Experts differ in contraction length (their row counts), and
    // the hardware hands tiles out in block order: the longest contractions go first, so that the tiles still running
    // when the grid drains are the short ones (position r takes the expert with the r-th largest count, ties by index).
    // Up to NT experts: one thread ranks one expert against the counts parked in LDS (the stages are not in use yet).
    if (prm.num_experts <= NT) {
      int* sh = reinterpret_cast<int*>(lds_c);
      const int E = prm.num_experts;
      if (tid < E) sh[tid] = (int)prm.counts[tid];
      __syncthreads();
      if (tid < E) {
        const int c = sh[tid];
        int rank = 0;
        for (int i = 0; i < E; ++i) {
          const int ci = sh[i];
          rank += (ci > c || (ci == c && i < tid)) ? 1 : 0;
        }
        if (rank == expert) sh[NT] = tid;
      }
      __syncthreads();
      expert = sh[NT];
      __syncthreads();  // everyone holds its expert before the first loads land in the stages
    }
    k_begin = prm.seg_starts[expert];
    k_len = (int)((prm.counts[expert] + BK - 1) / BK * BK);  // the transposed operands are zero up to the tile boundary
  } else {
    const int live_m = prm.seg_starts[prm.num_experts] / prm.align;
    const int total = live_m * prm.n_tiles;
    int pid = blockIdx.x;
    k_len = prm.K;
    if constexpr (kSplit) {
      // The tiles of the last, partial round (the highest block indices: the hardware hands blocks out in order) would
      // each keep one CU busy for a whole tile time while the rest of the chip idles. When that round is at most half
      // full, every such tile is computed by 2 to 4 workgroups (as many as fill the chip), an equal share of the contraction each: part
      // 0 is the tile's own block, parts 1.. are extra blocks behind the regular grid. All write their fp32 accumulators
      // to the workspace; the last to arrive (ticket) adds the parts up in part order and runs the epilogue.
      const int cus = kXcds * 32;
      const int tail = total % cus;
      const bool active = prm.split_ws != nullptr && tail > 0 && tail <= 2 * kSplitMaxTail && total / cus <= kSplitMaxRounds &&
                          prm.K / BK >= kSplitMinSteps;
      split_parts = active ? min(kSplitParts, cus / tail) : kSplitParts;  // as many parts as fill the chip: 4, 3 or 2
      if (pid >= prm.split_base) {  // an extra block
        const int x = pid - prm.split_base;
        split_slot = x / (split_parts - 1);
        split_part = x % (split_parts - 1) + 1;
        if (!active || split_slot >= tail) return;
        pid = total - tail + split_slot;
      } else if (active && pid >= total - tail && pid < total) {
        split_slot = pid - (total - tail);
        split_part = 0;
      }
      if (split_part >= 0) {
        const int steps = prm.K / BK;
        const int first = (int)((int64_t)steps * split_part / split_parts), last = (int)((int64_t)steps * (split_part + 1) / split_parts);
        k_begin = (int64_t)first * BK;
        k_len = (last - first) * BK;
      }
    }
    if (pid >= total) return;
    const int per_xcd = total / kXcds;
    if (pid < per_xcd * kXcds) pid = (pid % kXcds) * per_xcd + pid / kXcds;
    grouped_order(pid, live_m, prm.n_tiles, mt, nt);
    expert = prm.tile_expert[mt];
  }
  const int64_t m0 = (int64_t)mt * BM;
  int64_t valid_end = 0;  // forward modes: first pad row of this expert's segment
  if constexpr (MODE != kDw) valid_end = (int64_t)prm.seg_starts[expert] + prm.counts[expert];
  // scatter epilogue: the output row of tile row `tid`, fetched now and parked in LDS once the main loop is over
  int scatter_row = -1;
  if constexpr (MODE == kScatter) {
    if (tid < BM && m0 + tid < valid_end) scatter_row = prm.row_slot_out[m0 + tid];
  }

  // One wave per SIMD (WGM == 2): nothing zeroes the accumulators; the first slice of the tile multiplies with the
  // constant 0 as its third operand (run_acc_first). A tile without K steps (an expert without rows, weight gradients)
  // zeroes them where it finds that out.
  f32x4 acc[MI][NI];
  if constexpr (WGM != 2) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  }

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
  } else if constexpr (BT) {
    b_base += k_begin * prm.ldw * 2;  // a part of a split contraction starts further down the contraction rows
  }
  if constexpr (MODE != kDw) {
    if (prm.a_gather_div <= 0) a_base += m0 * prm.lda * 2;
  }
  constexpr int kAtRowBytes = BM * 2;
  auto swap02 = [](int w) { return (w & ~5) | ((w & 1) << 2) | ((w >> 2) & 1); };
  // contraction-strided stages (64 contraction rows of 256 columns): 32-byte window q (16 columns) of row n sits at
  // window position swap02(q) ^ tr_swz(n) of the row
  auto tr_swz = [](int n) { return (n & 3) | (((n >> 3) & 1) << 2); };
  uint32_t a_off[A_LD], b_off[B_LD];
  // gathered input: the row_slot entries of this lane's A_LD tile rows, fetched together (one wait, not one per load)
  // into the registers that then take the offsets
  if constexpr (!AT && MODE != kDw) {
    if (prm.a_gather_div > 0) {
#pragma unroll
      for (int t = 0; t < A_LD; ++t) {
        int64_t p = m0 + (wave * A_LD + t) * 8 + (lane >> 3);
        if (p >= valid_end) p = valid_end - 1;
        a_off[t] = (uint32_t)prm.row_slot[p];
      }
    }
  }
#pragma unroll
  for (int t = 0; t < A_LD; ++t) {
    if constexpr (AT) {
      const int pos = (wave * A_LD + t) * 1024 + lane * 16;  // byte position of this lane's slot in the A stage
      const int n = pos / kAtRowBytes, slot16 = (pos % kAtRowBytes) / 16;
      const int q = swap02((slot16 >> 1) ^ tr_swz(n));
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
        row = prm.a_gather_div > 0 ? (int64_t)((int32_t)a_off[t] / prm.a_gather_div) : p - m0;
      }
      a_off[t] = (uint32_t)((row * prm.lda + k_begin) * 2 + c * 16);
    }
  }
  // BT: 32-byte window q of contraction row n sits at window position swap02(q) ^ tr_swz(n) of the row (swap02 exchanges
  // bits 0 and 2 of the window index, tr_swz(n) = bits 0-1 of n and bit 3 of n moved to bit 2): the 4 rows x 32 bytes one
  // 16-lane group of a transposing read touches fill one 128-byte block, and the neighbouring group (the same columns 8
  // contraction rows further down) falls into the other half of the banks.
  constexpr int kBtRowBytes = BN * 2, kBtWindows = kBtRowBytes / 32;
#pragma unroll
  for (int t = 0; t < B_LD; ++t) {
    if constexpr (BT) {
      const int pos = (wave * B_LD + t) * 1024 + lane * 16;  // byte position of this lane's slot in the B stage
      const int n = pos / kBtRowBytes, slot16 = (pos % kBtRowBytes) / 16;
      const int q = swap02((slot16 >> 1) ^ tr_swz(n));         // the window that belongs at this position
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
  const int nk = __builtin_amdgcn_readfirstlane(k_len / BK);  // the same in every lane; says so to the compiler
  // Stage layout: two stages, each A (BM rows) followed by B (BN rows).
  constexpr int kAStage = BM * kRowBytes;
  auto a_stage_at = [&](int st) { return st * kStageBytes; };
  auto b_stage_at = [&](int st) { return st * kStageBytes + kAStage; };

  // One 1 KiB wave-load: scalar base (the operand at this K step, uniform over the wave) + the lane's 32-bit byte offset,
  // so that a load costs no vector arithmetic (a 64-bit vector add per load delayed the MFMA behind it)
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
  const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + wave * B_LD * 1024);
  // load g of K step `step`: g < A_LD: a wave-load of A, else of the weight operand, into stage step % 2
  auto issue_one = [&](int step, int g) __attribute__((always_inline)) {
    step = __builtin_amdgcn_readfirstlane(step);  // uniform; said to the compiler, which wants it in a scalar register
    const uint32_t st = (uint32_t)((step & (NSTAGE - 1)) * kStageBytes);
    // measurement builds: bit 16 = both operands re-read the first two K steps (L2 hits), 512 / 1024 = only A / only B does
    const int64_t kb = (CK_ABLATE & 16) ? (int64_t)(step & 1) * kRowBytes : (int64_t)step * kRowBytes;
    const int64_t kb_hot = (int64_t)(step & 1) * kRowBytes;
    const int64_t kb_b = BT ? (int64_t)((CK_ABLATE & (16 | 1024)) ? (step & 1) : step) * BK * prm.ldw * 2
                            : ((CK_ABLATE & 1024) ? kb_hot : kb);  // BT: 64 contraction rows further down
    const int64_t kb_a = AT ? (int64_t)step * BK * prm.lda * 2 : ((CK_ABLATE & 512) ? kb_hot : kb);
    if (g < A_LD) dma16(a_base_u + kb_a, a_off[g], wave_a + st + g * 1024);
    else dma16(b_base_u + kb_b, b_off[g - A_LD], wave_b + (uint32_t)kAStage + st + (g - A_LD) * 1024);
  };
  auto issue = [&](int step) {
#pragma unroll
    for (int g = 0; g < kLoadsPerStep; ++g) issue_one(step, g);
  };
  // ---- fragments: slice sl of a row is its 16-byte chunks 4 sl + lane / 16 (the lane's 8 contraction values)
  typedef typename Mfma16<T>::frag frag_t;
  const int fsw = swz128(lane & 15), fq = lane >> 4;
  int slice_off[KS];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) slice_off[sl] = ((4 * sl + fq) ^ fsw) * 16;
  const int fa_row = (wm * WM + (lane & 15)) * kRowBytes;
  const int fb_row = (wn * WN + (lane & 15)) * kRowBytes;  // within the B part of a stage
  constexpr bool kDouble = TL::kDouble;
  constexpr int kSets = kDouble ? 2 : 1;
  frag_t fa[kSets][MI], fb[kSets][NI];
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short tr16x4;
  // Contraction-strided stages. Lane l = 16 g + i of a transposing read points at 4 consecutive columns (4 (i % 4) ..) of
  // contraction row i / 4 of a 4-row x 16-column patch and receives the 4 rows of column i; two reads (rows +0..3,
  // +4..7 of the lane group's 8 rows 8 g ..) make the 8 contraction values 8 g .. 8 g + 7 of column i -- the MFMA's layout.
  // Rows 8 g + (i / 4) (+ 4): tr_swz = (i / 4) ^ 4 (g % 2) for both reads' rows up to the +4, which leaves bits 0-1 and 3.
  int at_off[MI];
  if constexpr (AT) {
    const int g = lane >> 4, i = lane & 15, n_low = i >> 2;
#pragma unroll
    for (int b = 0; b < MI; ++b) {
      const int q = (wm * WM + b * 16) / 16;
      at_off[b] = (8 * g + n_low) * kAtRowBytes + (swap02(q) ^ (n_low | ((g & 1) << 2))) * 32 + 8 * (i & 3);
    }
  }
  auto read_a = [&](int set, int stage, int sl, int i) {
    if constexpr (AT) {
      const char* p = lds_c + a_stage_at(stage) + at_off[i] + 32 * sl * kAtRowBytes;
      union {
        tr16x4 h[2];
        frag_t f;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p + 4 * kAtRowBytes));
      fa[set][i] = u.f;
    } else {
      fa[set][i] = *reinterpret_cast<const frag_t*>(lds_c + a_stage_at(stage) + slice_off[sl] + fa_row + i * 16 * kRowBytes);
    }
  };
  int bt_off[NI];
  if constexpr (BT) {
    const int g = lane >> 4, i = lane & 15, n_low = i >> 2;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int q = (wn * WN + j * 16) / 16;
      bt_off[j] = (8 * g + n_low) * kBtRowBytes + (swap02(q) ^ (n_low | ((g & 1) << 2))) * 32 + 8 * (i & 3);
    }
  }
  auto read_b = [&](int set, int stage, int sl, int j) {
    if constexpr (BT) {
      const char* p = lds_c + b_stage_at(stage) + bt_off[j] + 32 * sl * kBtRowBytes;
      union {
        tr16x4 h[2];
        frag_t f;
      } u;
      u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p));
      u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr16x4 __attribute__((address_space(3)))*)(p + 4 * kBtRowBytes));
      fb[set][j] = u.f;
    } else {
      fb[set][j] = *reinterpret_cast<const frag_t*>(lds_c + b_stage_at(stage) + slice_off[sl] + fb_row + j * 16 * kRowBytes);
    }
  };
  auto mfma = [&](int set, int i, int j, auto first) {
    // weight fragment first: a lane gets 4 consecutive output columns of one row
    if constexpr (WGM == 2 && decltype(first)::value) Mfma16<T>::run_acc_first(fb[set][j], fa[set][i], acc[i][j]);
    else if constexpr (WGM == 2) Mfma16<T>::run_acc(fb[set][j], fa[set][i], acc[i][j]);
    else acc[i][j] = Mfma16<T>::run(fb[set][j], fa[set][i], acc[i][j]);
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

  if constexpr (CK_STAMP != 0) st_loop = clock64();
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
    for (int i = 0; i < MI; ++i) read_a(0, 0, 0, i);
#pragma unroll
    for (int j = 0; j < NI; ++j) read_b(0, 0, 0, j);
    if constexpr ((CK_ABLATE & 4) != 0 && kDouble) {  // no fragment reads in the loop: both sets hold the first slice
#pragma unroll
      for (int i = 0; i < MI; ++i) fa[1][i] = fa[0][i];
#pragma unroll
      for (int j = 0; j < NI; ++j) fb[1][j] = fb[0][j];
    }
    if constexpr (CK_STAMP != 0) st_mark = clock64();

    // One 32-wide slice: MI x NI MFMAs, row block by row block, and the fragment reads for the slice after it (ns, nsl).
    // Two fragment sets: the reads go out one after each of the first MI + NI MFMAs, in the order the next slice needs
    // them. One set: fa[i] is reloaded once row block i is done, fb[j] after the MFMA (MI - 1, j).
    // Slice 0 of a step: the next slice is in the same stage. Phase 0 (and 3, the tile's first slice, whose early loads
    //   test nk themselves): early loads of step kt + 2, see below; phase 2: nothing to fetch.
    // Slice 1: the next slice is slice 0 of step kt + 1 in the other stage. Phase 0 / 1: wait for that stage (every
    //   load older than this step's early ones) and for this wave's own fragment reads, then meet the other waves; in
    //   phase 0 the late loads of step kt + 2 go out under this slice's MFMAs. Phase 1 is step nk - 2 (nothing left to
    //   fetch), phase 2 the last step (nothing to wait for, nothing to reload).
    constexpr int kLoadGap = (MI * NI) / kLoadsPerStep;
    // Two barriers per K step. The stage a step reads is dead as soon as every wave holds its fragments of the step's
    // second slice, i.e. early in the first slice (the reads go out behind its first MI + NI MFMAs): a barrier behind
    // MFMA kWarAt of the first slice says so, and the first kEarly loads of step kt + 2 follow it under the rest of
    // that slice; the others go out under the second slice, behind the barrier that publishes step kt + 1. The last
    // load of a step is then in flight for 0.8 of a K step before it is waited for instead of 0.5 (8 early loads
    // from MFMA 20 on, the late ones 6 MFMAs apart: 5 % faster launches than all 16 under the second slice; 6, 10, 12
    // or 16 early loads, other starting points and denser early loads measured the same or slower).
    constexpr int kEarly = kDouble ? 8 : 0, kWarAt = 20, kEarlyGap = 4, kLateGap = kEarly > 0 ? 6 : kLoadGap;
    static_assert(kEarly == 0 || (kWarAt >= MI + NI && kWarAt + (kEarly - 1) * kEarlyGap < MI * NI && kEarly <= kLoadsPerStep), "early loads");
    static_assert((kLoadsPerStep - kEarly - 1) * kLateGap < MI * NI, "late loads");
    auto slice = [&](int kt, auto sl, auto phase, auto idle, auto first) __attribute__((always_inline)) {
      constexpr bool kIdle = decltype(idle)::value;  // this wave's rows are all pad rows: no fragments, no MFMAs
      constexpr bool kLast = decltype(sl)::value == KS - 1;
      constexpr int kPhase = decltype(phase)::value;
      const int ns = kLast ? (kt + 1) & (NSTAGE - 1) : kt & (NSTAGE - 1);
      constexpr int nsl = kLast ? 0 : decltype(sl)::value + 1;
      constexpr bool kReload = !(kLast && kPhase == 2) && !(CK_ABLATE & 4) && !kIdle;
      if constexpr (kLast && kPhase != 2) {
        if constexpr (AT && kPhase == 1) {  // the stage that has just landed is the last K step
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          zero_pad_slots(kt + 1);
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        } else if constexpr (CK_STAMP != 0) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          const uint64_t t0 = clock64();
          if constexpr (kPhase == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kEarly) : "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          const uint64_t t1 = clock64();
          asm volatile("s_barrier" ::: "memory");
          const uint64_t t2 = clock64();
          st_vm += t1 - t0;
          st_bar += t2 - t1;
          st_s0 += t0 - st_mark;  // slice 0 of this step (the slice in front of the wait)
          st_mark = t2;
        } else if constexpr (kPhase == 0) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kEarly) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
      constexpr int cur = kDouble ? (decltype(sl)::value & 1) : 0;
      constexpr int nxt = kDouble ? (cur ^ 1) : 0;
#pragma unroll
      for (int n = 0; n < MI * NI; ++n) {
        const int i = n / NI, j = n % NI;
        if constexpr (!kIdle) mfma(cur, i, j, first);
        if constexpr (kLast && kPhase == 0 && !(CK_ABLATE & 2)) {
          if (n % kLateGap == 0 && n / kLateGap < kLoadsPerStep - kEarly) issue_one(kt + 2, kEarly + n / kLateGap);
        }
        if constexpr (!kLast && (kPhase == 0 || kPhase == 3) && kEarly > 0 && !(CK_ABLATE & 2)) {
          // every wave holds its fragments of this stage's second slice: once all have said so the stage is dead and the
          // first kEarly loads of step kt + 2 overwrite it under the rest of this slice
          if (n == kWarAt) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          if (n >= kWarAt && (n - kWarAt) % kEarlyGap == 0 && (n - kWarAt) / kEarlyGap < kEarly && (kPhase == 0 || nk > 2))
            issue_one(kt + 2, (n - kWarAt) / kEarlyGap);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kReload) {
          if constexpr (kDouble) {  // behind the first MI + NI MFMAs, in the order the next slice needs them (spreading
                                    // them over the whole slice measured the same)
            if (n < MI) read_a(nxt, ns, nsl, n);
            else if (n < MI + NI) read_b(nxt, ns, nsl, n - MI);
          } else {
            if (j == NI - 1) read_a(0, ns, nsl, i);
            if (i == MI - 1) read_b(0, ns, nsl, j);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (CK_STAMP != 0 && kLast && kPhase != 2) {
        const uint64_t t3 = clock64();
        st_s1 += t3 - st_mark;  // slice 1: from the barrier to the end of the step
        st_mark = t3;
      }
    };
    // The first slice of the tile is peeled (its MFMAs start the accumulators). Every branch on the way has one arm
    // and the loop body none: two variants of a slice meeting behind a two-armed branch make the compiler move the
    // 256 accumulators around (spills between MFMAs whose results it cannot know to be in flight). The lambdas are
    // force-inlined: left to the inliner's budget they become calls and the accumulators go to memory.
    auto k_loop = [&](auto idle) __attribute__((always_inline)) {
      constexpr std::integral_constant<int, 0> s0{}, p0{};
      constexpr std::integral_constant<int, 1> s1{}, p1{};
      constexpr std::integral_constant<int, 2> p2{};
      constexpr std::false_type later{};
      // A step kt with kt + 2 < nk fetches step kt + 2 (phase 0 of both its slices); the first slice of the last two
      // steps is phase 2 (nothing to fetch). The tile's very first slice is phase 3: its early loads sit under a test
      // of nk each, so that one variant serves every tile and the accumulators start in one place.
      constexpr std::integral_constant<int, 3> p3{};
      if constexpr (WGM == 2) slice(0, s0, p3, idle, std::true_type{});
      else slice(0, s0, p3, idle, later);
      int kt = 0;
      if (nk > 2) {
        slice(0, s1, p0, idle, later);
        for (kt = 1; kt + 2 < nk; ++kt) {
          slice(kt, s0, p0, idle, later);
          slice(kt, s1, p0, idle, later);
        }
        slice(kt, s0, p2, idle, later);
      }
      if (kt + 2 == nk) {
        slice(kt, s1, p1, idle, later);
        slice(kt + 1, s0, p2, idle, later);
        ++kt;
      }
      slice(kt, s1, p2, idle, later);
      // Behind the last MFMA, still inside this variant of the loop (in front of the point where the idle and the
      // multiplying variant meet again, where the compiler may move accumulators around): wait out the MFMA result
      // latency and tie every accumulator to that wait (see mfma_fence).
      if constexpr (WGM == 2) {
        mfma_drain();
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) mfma_fence(acc[i][j]);
      }
    };
    // A wave whose tile rows all lie past the expert's last row (the tile is the ragged end of a segment) still issues
    // its share of the loads and meets every barrier, but multiplies nothing: the wave it shares a SIMD with then has
    // the matrix pipe to itself. Its accumulators hold nothing meaningful and its rows are never stored.
    bool wave_idle = false;
    if constexpr (MODE != kDw) wave_idle = m0 + wm * WM >= valid_end;
    if (__builtin_amdgcn_readfirstlane(wave_idle)) k_loop(std::true_type{});
    else k_loop(std::false_type{});
  } else if constexpr (WGM == 2 && MODE == kDw) {  // only a weight-gradient tile can have no K step (the host requires K >= 64)
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- epilogue, straight from the accumulators. The weight fragment is the MFMA's first operand, so a lane holds, per
  // 16x16 block (i, j), the 4 consecutive output columns j * 16 + 4 (lane / 16) + 0..3 of tile row i * 16 + lane % 16:
  // two packed registers. v_permlane16_swap exchanges them between neighbouring 16-lane rows for a pair of column blocks
  // (j, j + 1): an even lane group ends up with 8 consecutive columns of block j, an odd one with 8 of block j + 1, so
  // every lane stores 16 bytes and a store instruction writes 64 contiguous bytes of each of 16 output rows. No LDS
  // round trip and no barrier (a slab in LDS took 16 k of the 196 k cycles of a K = 4096 tile on one wave per SIMD; this
  // form 9 k, of which 5 k are the register reads, conversions and swaps and 4 k the stores).
  // Plain (cached) stores: L2 merges the two 64-byte halves of an output line before it leaves for memory (measured
  // against non-temporal stores: 3 % faster launches at K = 4096).

  if constexpr (kSplit) {
    if (split_part >= 0) {
      // every part leaves its accumulators in the workspace, in its own register layout (16 bytes per lane)
      float* slot_ws = prm.split_ws + (int64_t)split_slot * split_parts * kSplitPartFloats;
      float* mine = slot_ws + (int64_t)split_part * kSplitPartFloats + ((int64_t)wave * MI * NI * kWave + lane) * 4;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) *reinterpret_cast<f32x4*>(mine + (i * NI + j) * kWave * 4) = acc[i][j];
      uint32_t* arrivals = reinterpret_cast<uint32_t*>(prm.split_ws + (int64_t)kSplitMaxTail * kSplitParts * kSplitPartFloats);
      uint32_t* flag = reinterpret_cast<uint32_t*>(lds_c);  // the stages are dead
      __threadfence();  // the partial tile is visible device-wide before the ticket is taken
      __syncthreads();
      if (tid == 0) {
        // ticket = arrivals of THIS launch so far: a word left by another launch (any epoch but ours) counts as zero
        uint32_t cur = __hip_atomic_load(&arrivals[split_slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), nxt;
        for (;;) {  // bounded: another part of this tile (at most three) changed the word in between
          nxt = (cur >> 4) == prm.split_epoch ? cur + 1u : ((prm.split_epoch << 4) | 1u);
          const uint32_t seen = atomicCAS(&arrivals[split_slot], cur, nxt);
          if (seen == cur) break;
          cur = seen;
        }
        *flag = nxt & 15u;
      }
      __syncthreads();
      const bool last = *flag == (uint32_t)split_parts;
      __syncthreads();  // everyone has read the flag before the epilogue reuses LDS
      if (!last) return;
      __threadfence();  // the other parts' tiles are read from memory, not from a stale cache line
      const float* theirs = slot_ws + ((int64_t)wave * MI * NI * kWave + lane) * 4;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) {  // a fixed order of additions whichever part arrived last
          const float* q = theirs + (i * NI + j) * kWave * 4;
          f32x4 sum = *reinterpret_cast<const f32x4*>(q) + *reinterpret_cast<const f32x4*>(q + kSplitPartFloats);
          if (split_parts > 2) sum += *reinterpret_cast<const f32x4*>(q + 2 * kSplitPartFloats);
          if (split_parts > 3) sum += *reinterpret_cast<const f32x4*>(q + 3 * kSplitPartFloats);
          acc[i][j] = sum;
        }
    }
  }
  if constexpr (CK_STAMP != 0) st_end = clock64();
  auto store_out = [](void* p, const vec16& v) { store16(p, v); };
  const int lrow = lane & 15, lg = lane >> 4;
  const bool odd_group = (lg & 1) != 0;
  const T kZero = Elem<T>::down(0.f);
  // 8 consecutive columns for this lane out of the column blocks j (packed pairs p0, p1) and j + 1 (q0, q1) of one row block
  auto gather8 = [&](uint32_t p0, uint32_t p1, uint32_t q0, uint32_t q1) {
    const auto s0 = __builtin_amdgcn_permlane16_swap(p0, q0, false, false);  // odd rows of p <-> even rows of q
    const auto s1 = __builtin_amdgcn_permlane16_swap(p1, q1, false, false);
    vec16 v;  // even group: own p, then the p of the group above; odd group: the q of the group below, then own q
    v.w[0] = s0[0];
    v.w[1] = s1[0];
    v.w[2] = s0[1];
    v.w[3] = s1[1];
    return v;
  };
  auto gather8_acc = [&](const f32x4& p, const f32x4& q) {
    return gather8(pack_pair<T>(p[0], p[1]), pack_pair<T>(p[2], p[3]), pack_pair<T>(q[0], q[1]), pack_pair<T>(q[2], q[3]));
  };
  // column (relative to the wave's first column) of the 8 values gather8 leaves in this lane for the block pair (j, j + 1)
  auto pair_col = [&](int j) { return (j + (odd_group ? 1 : 0)) * 16 + 4 * (lg & ~1); };
  // store_lines(v1, v2, j, ptr_of_row, row_ok, col_ok): the block quad j .. j + 3 of one row block, two 16-byte pieces per
  // lane (v1: blocks j, j + 1; v2: blocks j + 2, j + 3); ptr_of_row(r) -> address of the wave's first column in row r
  // (0 .. 15) of the row block; row_ok(r), col_ok(c) -> inside the matrix. (Regrouping the pieces so that every store
  // writes whole 128-byte lines -- a rotation by 8 inside the 16-lane rows -- measured the same and is not done.)
  auto store_lines = [&](const vec16& v1, const vec16& v2, int j, auto&& ptr_of_row, auto&& row_ok, auto&& col_ok) {
    const int c1 = pair_col(j), c2 = pair_col(j + 2);
    if (row_ok(lrow) && col_ok(c1) && (!(CK_ABLATE & 128) || prm.K == -12345)) store_out(ptr_of_row(lrow) + (uint32_t)c1 * 2u, v1);
    if (row_ok(lrow) && col_ok(c2) && (!(CK_ABLATE & 128) || prm.K == -12345)) store_out(ptr_of_row(lrow) + (uint32_t)c2 * 2u, v2);
  };
  // The same for outputs whose rows are `pitch` bytes apart from a uniform base (every epilogue but the scatter one): the
  // store takes the base in scalar registers and the lane's 32-bit byte offset (row_off: lane row * pitch, advanced by
  // 16 rows per row block, + column bytes), so that it costs one or two 32-bit vector instructions and no 64-bit vector
  // arithmetic; `inside`: the wave's whole tile lies inside the matrix and nothing is tested per store.
  auto store_at = [&](char* base_u, uint32_t off, const vec16& v) {
    const u32x4_t d = {v.w[0], v.w[1], v.w[2], v.w[3]};
    // The two wait states behind the store are the hardware's rule for a store of more than 8 bytes whose data registers
    // the next vector instruction overwrites; the compiler inserts them for its own stores and cannot see into this one.
    asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" ::"v"(off), "v"(d), "s"(base_u) : "memory");
  };
  auto store_lines_at = [&](const vec16& v1, const vec16& v2, int j, char* base_u, uint32_t row_off, bool inside, bool row_in,
                            int cols_left) {
    const uint32_t o1 = row_off + (uint32_t)pair_col(j) * 2u, o2 = row_off + (uint32_t)pair_col(j + 2) * 2u;
    if ((CK_ABLATE & 128) && prm.K != -12345) return;
    if (inside) {
      store_at(base_u, o1, v1);
      store_at(base_u, o2, v2);
    } else {
      if (row_in && pair_col(j) < cols_left) store_at(base_u, o1, v1);
      if (row_in && pair_col(j + 2) < cols_left) store_at(base_u, o2, v2);
    }
  };
  auto uniform_out = [](char* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<char*>(((uint64_t)hi << 32) | lo);
  };
  const int64_t tile_row0 = m0 + wm * WM;  // first row of this wave's tile rows (padded row / dW row)

  if constexpr (MODE == kScatter) {  // output row of every tile row, through LDS (the stages are dead)
    int* scatter_rows = reinterpret_cast<int*>(lds_c);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the stages
    if (tid < BM) scatter_rows[tid] = scatter_row;
    __syncthreads();
  }

  // Addresses: a uniform 64-bit base (the wave's first output element) plus 32-bit byte offsets per lane, so that a store
  // costs one 32-bit add at most (rows of one tile are less than 4 GiB apart; scattered rows get their own 64-bit base).
  auto convert4 = [&](const f32x4& v, T (&o)[4]) {
#pragma unroll
    for (int s = 0; s < 4; ++s) o[s] = Elem<T>::down(v[s]);
  };
  if constexpr (MODE == kDw) {
    const int64_t col0 = (int64_t)nt * BN + wn * WN;
    char* base = uniform_out(reinterpret_cast<char*>(static_cast<T*>(prm.y) + (int64_t)expert * prm.M * prm.N + tile_row0 * prm.N + col0));
    const uint32_t row_pitch = (uint32_t)prm.N * 2u;
    const int rows_left = (int)min((int64_t)WM, (int64_t)prm.M - tile_row0);   // rows of this wave that exist
    const int cols_left = (int)min((int64_t)WN, (int64_t)prm.N - col0);        // columns of this wave that exist
    const bool inside = rows_left >= WM && cols_left >= WN;
    uint32_t row_off = (uint32_t)lrow * row_pitch;
    static_for<MI>([&](auto i) {
      static_for<NI / 4>([&](auto jq) {
        const vec16 v1 = gather8_acc(acc[i][4 * jq], acc[i][4 * jq + 1]), v2 = gather8_acc(acc[i][4 * jq + 2], acc[i][4 * jq + 3]);
        store_lines_at(v1, v2, 4 * jq, base, row_off, inside, i * 16 + lrow < rows_left, cols_left);
      });
      row_off += 16u * row_pitch;
      __builtin_amdgcn_sched_barrier(0);  // row block by row block: the stores of one drain under the conversions of the next
    });
  } else if constexpr (MODE == kGrouped || MODE == kScatter) {
    T* y = static_cast<T*>(prm.y);
    T* y_t = static_cast<T*>(prm.y_t);
    const int64_t col0 = (int64_t)nt * BN + wn * WN;
    const int cols_left = (int)min((int64_t)WN, (int64_t)prm.N - col0);
    const int rows_left = (int)min((int64_t)WM, valid_end - tile_row0);  // valid (non-pad) rows of this wave; may be <= 0
    // optional per-expert bias row (aux_in = bias [E, N]): added to the fp32 accumulators, so that the output is rounded
    // once, like F.linear with a bias
    if constexpr (!BT && EXTRA) {
      if (prm.aux_in != nullptr) {
        const T* bias = static_cast<const T*>(prm.aux_in) + (int64_t)expert * prm.N;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const int64_t n = col0 + j * 16 + 4 * lg + s;
            const float b = n < prm.N ? Elem<T>::up(bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < MI; ++i) acc[i][j][s] += b;
          }
        }
      }
    }
    if constexpr (MODE == kGrouped && EXTRA) if (y_t != nullptr) {
      // transposed copy [N, ld_t] with zeros in pad rows: a side output for the transposed-operand weight-gradient form
      // (matrices narrower than 256); 2-byte stores, off the benchmark shapes' path
      static_for<MI>([&](auto i) {
        const int r = i * 16 + lrow;
        const int64_t prow = tile_row0 + r;
        static_for<NI>([&](auto j) {
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const int64_t n = col0 + j * 16 + 4 * lg + s;
            if (n < prm.N) y_t[n * prm.ld_t + prow] = r < rows_left ? Elem<T>::down(acc[i][j][s]) : kZero;
          }
        });
      });
    }
    char* base = uniform_out(reinterpret_cast<char*>(y + tile_row0 * prm.N + col0));
    // second output of the grouped epilogue (aux, same shape as y): the tanh-approximated GELU of the 8 rounded outputs
    char* act_base = nullptr;
    if constexpr (MODE == kGrouped && EXTRA && !BT) {
      if (prm.aux != nullptr) act_base = uniform_out(reinterpret_cast<char*>(static_cast<T*>(prm.aux) + tile_row0 * prm.N + col0));
    }
    auto gelu8 = [&](const vec16& v) {
      Pack16<T> in;
      in.v = v;
      vec16 o;
#pragma unroll
      for (int w = 0; w < 4; ++w)
        o.w[w] = pack_pair<T>(gelu_tanh_fast(Elem<T>::up(in.e[2 * w])), gelu_tanh_fast(Elem<T>::up(in.e[2 * w + 1])));
      return o;
    };
    const uint32_t row_pitch = (uint32_t)prm.N * 2u;
    const bool inside = rows_left >= WM && cols_left >= WN;
    uint32_t row_off = (uint32_t)lrow * row_pitch;
    static_for<MI>([&](auto i) {
      char* row_a = nullptr;  // scatter: the output row this lane writes in this row block
      if constexpr (MODE == kScatter) {
        const int* rows = reinterpret_cast<const int*>(lds_c) + wm * WM + i * 16;
        row_a = reinterpret_cast<char*>(y + (int64_t)rows[lrow] * prm.N + col0);
      }
      static_for<NI / 4>([&](auto jq) {
        const vec16 v1 = gather8_acc(acc[i][4 * jq], acc[i][4 * jq + 1]), v2 = gather8_acc(acc[i][4 * jq + 2], acc[i][4 * jq + 3]);
        if constexpr (MODE == kScatter) {
          store_lines(v1, v2, 4 * jq, [&](int) { return row_a; }, [&](int r) { return i * 16 + r < rows_left; },
                      [&](int c) { return c < cols_left; });
        } else {
          store_lines_at(v1, v2, 4 * jq, base, row_off, inside, i * 16 + lrow < rows_left, cols_left);
          if constexpr (EXTRA && !BT) if (act_base != nullptr) {  // CK_ACT_GELU_TANH: the activation of the rounded output
            store_lines_at(gelu8(v1), gelu8(v2), 4 * jq, act_base, row_off, inside, i * 16 + lrow < rows_left, cols_left);
          }
        }
      });
      row_off += 16u * row_pitch;
      __builtin_amdgcn_sched_barrier(0);
    });
  } else {  // kSwiglu: the first half of a wave's column blocks are up, the second half the gate of the same activation columns
    T* pre = static_cast<T*>(prm.y);
    T* act = static_cast<T*>(prm.aux);
    T* act_t = static_cast<T*>(prm.y_t);
    const int64_t two_i = 2 * (int64_t)prm.I;
    const int64_t col0 = (int64_t)nt * (BN / 2) + wn * (WN / 2);  // the wave's first activation column
    const int cols_left = (int)min((int64_t)(WN / 2), (int64_t)prm.I - col0);
    const int rows_left = (int)min((int64_t)WM, valid_end - tile_row0);
    constexpr int NH = NI / 2;  // column blocks per half
    static_assert(NH % 2 == 0, "whole block pairs in each half");
    char* pre_base = uniform_out(reinterpret_cast<char*>(pre + tile_row0 * two_i + col0));
    char* act_base = uniform_out(reinterpret_cast<char*>(act + tile_row0 * prm.I + col0));
    const uint32_t pre_pitch = (uint32_t)two_i * 2u, act_pitch = (uint32_t)prm.I * 2u, gate_off = (uint32_t)prm.I * 2u;
    const bool inside = rows_left >= WM && cols_left >= WN / 2;
    uint32_t pre_off = (uint32_t)lrow * pre_pitch, act_off = (uint32_t)lrow * act_pitch;
    static_for<MI>([&](auto i) {
      const int r = i * 16 + lrow;
      const bool valid = r < rows_left;
      static_assert(NH == 4, "one quad of column blocks per half");
      vec16 vu_[2], vg_[2], va_[2];
      static_for<NH / 2>([&](auto jp) {
        T up[2][4], gate[2][4], a[2][4];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          convert4(acc[i][2 * jp + b], up[b]);
          convert4(acc[i][2 * jp + b + NH], gate[b]);
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const float gf = Elem<T>::up(gate[b][s]);  // from the rounded pre-activation, like the unfused path
            const float sg = sigmoid_fast(gf);
            a[b][s] = Elem<T>::down(prm.act_kind == CK_ACT_GLU ? Elem<T>::up(up[b][s]) * sg : Elem<T>::up(up[b][s]) * gf * sg);  // same association as swiglu_fwd_kernel
          }
        }
        if constexpr (EXTRA) if (act_t != nullptr) {  // transposed activation [I, ld_t], zeros in pad rows (side output, 2-byte stores)
#pragma unroll
          for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              const int64_t n = col0 + (2 * jp + b) * 16 + 4 * lg + s;
              if (n < prm.I) act_t[n * prm.ld_t + tile_row0 + r] = valid ? a[b][s] : kZero;
            }
          }
        }
        auto pk = [&](const T (&v)[4], int h) { return (uint32_t)bits16(v[2 * h]) | ((uint32_t)bits16(v[2 * h + 1]) << 16); };
        const vec16 vu = gather8(pk(up[0], 0), pk(up[0], 1), pk(up[1], 0), pk(up[1], 1));
        const vec16 vg = gather8(pk(gate[0], 0), pk(gate[0], 1), pk(gate[1], 0), pk(gate[1], 1));
        const vec16 va = gather8(pk(a[0], 0), pk(a[0], 1), pk(a[1], 0), pk(a[1], 1));
        vu_[jp] = vu;
        vg_[jp] = vg;
        va_[jp] = va;
      });
      store_lines_at(vu_[0], vu_[1], 0, pre_base, pre_off, inside, valid, cols_left);
      store_lines_at(vg_[0], vg_[1], 0, pre_base, pre_off + gate_off, inside, valid, cols_left);
      store_lines_at(va_[0], va_[1], 0, act_base, act_off, inside, valid, cols_left);
      pre_off += 16u * pre_pitch;
      act_off += 16u * act_pitch;
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  if constexpr (CK_STAMP != 0) {  // per wave: prologue, main loop, of which load wait and barrier wait, epilogue (cycles)
    if (prm.trace != nullptr && lane == 0) {
      uint64_t* t = static_cast<uint64_t*>(prm.trace) + ((size_t)blockIdx.x * NW + wave) * 8;
      t[0] = st_loop - st_begin;
      t[1] = st_end - st_loop;
      t[2] = st_vm;
      t[3] = st_bar;
      t[4] = clock64() - st_end;
      t[5] = (uint64_t)nk;
      t[6] = st_s0;
      t[7] = st_s1;
    }
  }
}

template <typename T, int MODE, int BN, bool BT, int WGM, bool EXTRA>
int launch_extra(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  auto kernel = grouped_gemm_line_kernel<T, MODE, BN, BT, WGM, EXTRA>;
  constexpr size_t kLds = Tile<BN, WGM>::kLdsBytes;
  static bool lds_reserved[kMaxDevices] = {};
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kernel), kLds, lds_reserved, name)) return rc;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(Tile<BN, WGM>::NT), kLds, s, prm);
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

template <typename T, int MODE, int BN, bool BT, int WGM>
int launch_mode(const GemmParams& prm, unsigned blocks, hipStream_t s, const char* name) {
  if constexpr (!BT && MODE != kDw) {
    if (prm.aux_in != nullptr || prm.y_t != nullptr || (MODE == kGrouped && prm.aux != nullptr))
      return launch_extra<T, MODE, BN, BT, WGM, true>(prm, blocks, s, name);
  }
  return launch_extra<T, MODE, BN, BT, WGM, false>(prm, blocks, s, name);
}

template <typename T, int BN, int WGM>
int launch_bn(const GemmParams& prm, int mode, bool bt, unsigned blocks, hipStream_t stream, const char* name) {
  if (bt) {  // the input-gradient GEMMs: grouped or scatter epilogue, 256-wide tiles
    if constexpr (BN == 256) {
      if (mode == kGrouped) return launch_mode<T, kGrouped, BN, true, WGM>(prm, blocks, stream, name);
      if (mode == kScatter) return launch_mode<T, kScatter, BN, true, WGM>(prm, blocks, stream, name);
      if (mode == kDw) return launch_mode<T, kDw, BN, true, WGM>(prm, blocks, stream, name);  // both operands row-major
    }
    set_error("%s: contraction-strided operands go with 256-wide tiles and the grouped / scatter / dW epilogues", name);
    return CK_ERR_ARG;
  }
  switch (mode) {
    case kGrouped: return launch_mode<T, kGrouped, BN, false, WGM>(prm, blocks, stream, name);
    case kScatter: return launch_mode<T, kScatter, BN, false, WGM>(prm, blocks, stream, name);
    case kSwiglu: return launch_mode<T, kSwiglu, BN, false, WGM>(prm, blocks, stream, name);
    case kDw: return launch_mode<T, kDw, BN, false, WGM>(prm, blocks, stream, name);
    default: break;
  }
  set_error("%s: the 128-byte-row kernel has no epilogue %d", name, mode);
  return CK_ERR_ARG;
}

}  // namespace

int launch_line(const GemmParams& prm_in, int mode, int bn, bool bt, int dtype, unsigned blocks, hipStream_t stream,
                const char* name) {
  GemmParams prm = prm_in;
  if (prm.split_ws != nullptr && (mode == kGrouped || mode == kScatter)) {
    prm.split_base = (int)blocks;  // the extra workgroups of a split last round sit behind the regular grid
    prm.split_epoch = next_split_epoch();
    blocks += kSplitMaxTail * (kSplitParts - 1);
  } else {
    prm.split_ws = nullptr;
    prm.split_base = 0x7fffffff;
  }
  CK_DISPATCH_HALF(dtype, name, { return launch_bn<scalar_t, 256, 2>(prm, mode, bt, blocks, stream, name); });
  return CK_ERR_ARG;
}

}  // namespace ck
