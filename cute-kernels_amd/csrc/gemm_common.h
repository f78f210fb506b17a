// Pieces shared by the grouped GEMM kernels (bf16 / f16 in grouped_gemm.hip, fp8 e4m3 in grouped_gemm_fp8.hip).
#pragma once

#include <type_traits>

#include "ck_common.h"

namespace ck {

constexpr int kXcds = 8;

enum Mode { kGrouped = CK_EPI_GROUPED, kScatter = CK_EPI_SCATTER, kSwiglu = CK_EPI_SWIGLU, kSwigluBwd = CK_EPI_SWIGLU_BWD, kDw = 4 };

struct GemmParams {
  const void* a;      // forward modes: [*, K]; dW: a_t [M, ld_t]
  const void* w;      // forward modes: [E, N, K]; dW: b_t [N, ld_t]
  int64_t lda;        // row stride of a (elements)
  int64_t ldw;        // row stride of w (elements)
  int64_t w_expert_stride;
  int a_gather_div;   // > 0: A row p comes from a[row_slot[p] / div]
  int M;              // dW only: rows of a_t
  int N;              // output columns of the GEMM (2I for kSwiglu)
  int K;              // contraction length (forward modes)
  int I;              // kSwiglu / kSwigluBwd: intermediate size
  int n_tiles;        // tiles along N
  int m_tiles;        // dW only: tiles along M
  int align;          // rows per M tile (== BM) in the padded layout
  int num_experts;
  const int32_t* seg_starts;
  const uint32_t* counts;
  const int32_t* tile_expert;
  const int32_t* row_slot;      // padded row -> index of the A row it reads (gathered input)
  const int32_t* row_slot_out;  // padded row -> output row of the scatter epilogue (ck_segments::row_slot_out, else row_slot)
  void* y;
  void* y_t;
  int64_t ld_t;
  void* aux;
  const void* aux_in;
  const float* a_scale;  // fp8 only: per-row dequantisation scale of a (indexed like the rows of a)
  const float* w_scale;  // fp8 only: per-output-channel scale of w, [E, N]
  int act_kind;          // kSwiglu epilogue: CK_ACT_SWIGLU (up * gate * sigmoid(gate)) or CK_ACT_GLU (up * sigmoid(gate));
                         // kGrouped epilogue with aux: CK_ACT_GELU_TANH (aux = gelu(y), second output)
  void* trace;           // measurement builds only (CK_STAMP): per-wave cycle counts, 8 x uint64 each, else NULL
  // Split contraction for the last, partial round of tiles (128-byte-row kernel, grouped / scatter epilogues):
  // split_ws = [tiles][parts][4 waves][64 blocks][64 lanes] f32x4 partial accumulators (at most kSplitMaxTail tiles in
  // kSplitParts parts or twice as many in half as many parts), followed by 2 * kSplitMaxTail arrival words; NULL = never
  // split. split_base = the launch's grid without the extra workgroups (they are blockIdx split_base ..).
  // An arrival word holds (launch epoch << 4) | parts arrived. A part that finds another epoch in the word starts the
  // count afresh, so the words need no initial value and nothing resets them: whatever an earlier launch (or one that
  // was cut short) left behind reads as "nobody has arrived yet". split_epoch: 1 .. 2^28 - 1, unique per launch.
  float* split_ws;
  int split_base;
  uint32_t split_epoch;
};
uint32_t next_split_epoch();  // process-wide launch counter (grouped_gemm.hip)
constexpr int kSplitParts = 4, kSplitMaxTail = 64, kSplitMaxRounds = 64, kSplitMinSteps = 16;
constexpr int64_t kSplitPartFloats = 4 * 64 * 64 * 4;  // one workgroup's 256 x 256 fp32 tile
constexpr int64_t kSplitWorkspaceBytes = kSplitMaxTail * kSplitParts * kSplitPartFloats * 4 + 2 * kSplitMaxTail * 4;

// The 16-bit kernel with 128-byte LDS rows (grouped_gemm_line.hip): 256 x bn tiles, bn = 256 or 384, contraction length a
// multiple of 64, modes kGrouped, kScatter, kSwiglu, kDw. The caller fills `prm` for these tile dimensions (n_tiles,
// m_tiles) and sizes the grid accordingly.
constexpr int kLineBM = 256, kLineK = 64;
// bt: the weight operand is [E, contraction, columns] (contraction-strided) instead of [E, columns, contraction];
// grouped and scatter epilogues only, prm.ldw = its row length.
int launch_line(const GemmParams& prm, int mode, int bn, bool bt, int dtype, unsigned blocks, hipStream_t stream,
                const char* name);

namespace {

// The dynamic-LDS limit of a kernel is a per-device attribute: set it once per (instantiation, device). `done` is the
// instantiation's own table; the call is idempotent, so a race between host threads only repeats it.
constexpr int kMaxDevices = 64;
inline int reserve_lds(const void* kernel, size_t bytes, bool (&done)[kMaxDevices], const char* name) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = -1;
  if (dev >= 0 && done[dev]) return CK_OK;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) {
    set_error("%s: cannot reserve %zu bytes of LDS: %s", name, bytes, hipGetErrorString(e));
    return CK_ERR_LAUNCH;
  }
  if (dev >= 0) done[dev] = true;
  return CK_OK;
}

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
  typedef bf16x8 frag;
  __device__ static inline f32x16 run(const frag& a, const frag& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma<f16_t> {
  typedef f16x8 frag;
  __device__ static inline f32x16 run(const frag& a, const frag& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// v_mfma_f32_16x16x32: A lane l holds row l % 16, contraction values 8 (l / 16) .. + 7; B likewise for column l % 16; the
// result register s of lane l is row 4 (l / 16) + s, column l % 16. On N(0,1) operands a register-only loop of this
// shape sustains about 2.0 PFLOP/s where the 32x32x16 shape sustains 1.7 (the clock is power-managed), hence its use in
// the 128-byte-row kernel.
template <typename T>
struct Mfma16;
// run_acc: the same instruction with the accumulator pinned to the accumulation registers (AGPRs) and updated in place.
// With one wave per SIMD a kernel has 256 of them next to its 256 vector registers; left to choose, the register
// allocator spreads 256 accumulator values over both files and shuffles them at every loop boundary. The instruction is
// opaque to the compiler's hazard checks: a caller that reads the accumulators with vector instructions afterwards
// waits out the MFMA write latency itself (mfma_drain).
template <>
struct Mfma16<bf16_t> {
  typedef bf16x8 frag;
  __device__ static inline f32x4 run(const frag& a, const frag& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static inline void run_acc(const frag& a, const frag& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  // the first product of a tile: c = a * b + 0 (the constant as the third operand), so that nothing has to zero the
  // accumulators first -- 256 v_accvgpr_write per wave, which the compiler also re-materialised in front of the loop
  __device__ static inline void run_acc_first(const frag& a, const frag& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
  }
};
template <>
struct Mfma16<f16_t> {
  typedef f16x8 frag;
  __device__ static inline f32x4 run(const frag& a, const frag& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ static inline void run_acc(const frag& a, const frag& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  __device__ static inline void run_acc_first(const frag& a, const frag& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
  }
};
// After the last run_acc, before anything else reads the accumulators: longer than any MFMA's result latency. The wait
// alone is not enough: nothing ties the compiler's own reads of the accumulators (v_accvgpr_read, spills) to it, and the
// scheduler is free to hoist them above the wait, right behind the MFMA that writes them (it did: a few stale values
// per tile). mfma_fence(c) makes c a result of an empty asm statement placed behind the wait; volatile asm statements
// keep their order, so every later read of c stays behind the wait. Call it for every accumulator.
__device__ inline void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
__device__ inline void mfma_fence(f32x4& c) { asm volatile("" : "+a"(c)); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <int N, typename F>
__device__ inline void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

template <typename T>
__device__ inline uint16_t bits16(T v) {
  union {
    T t;
    uint16_t u;
  } c;
  c.t = v;
  return c.u;
}

// two fp32 values rounded (to nearest even) and packed into one register: one v_cvt_pk instruction
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
template <typename T>
__device__ inline uint32_t pack_pair(float a, float b);
template <>
__device__ inline uint32_t pack_pair<bf16_t>(float a, float b) {
  const f32x2_t v = {a, b};
  union {
    bf16x2_t h;
    uint32_t u;
  } c;
  c.h = __builtin_convertvector(v, bf16x2_t);
  return c.u;
}
template <>
__device__ inline uint32_t pack_pair<f16_t>(float a, float b) {
  const f32x2_t v = {a, b};
  union {
    f16x2_t h;
    uint32_t u;
  } c;
  c.h = __builtin_convertvector(v, f16x2_t);
  return c.u;
}

// 4 consecutive 16-bit values as one 8-byte store
template <typename T>
__device__ inline void store4(T* p, T v0, T v1, T v2, T v3) {
  uint2 u;
  u.x = (uint32_t)bits16(v0) | ((uint32_t)bits16(v1) << 16);
  u.y = (uint32_t)bits16(v2) | ((uint32_t)bits16(v3) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// Tile order inside a run of tiles: groups of 8 along `a` (the side with a_count tiles), then `b`, with `a` fastest
// inside a group -- 32 consecutive tiles form an 8 x 4 block that shares 8 + 4 operand panels.
// (measured at 4 / 8 / 16 / 32 tiles per group on the Mixtral-shape and fine-grained layers: 8 is fastest on both)
__device__ inline void grouped_order(int r, int a_count, int b_count, int& a, int& b) {
  constexpr int GROUP = 8;
  const int group_sz = GROUP * b_count;
  const int g = r / group_sz;
  const int first = g * GROUP;
  const int in_group = min(GROUP, a_count - first);
  const int q = r - g * group_sz;
  b = q / in_group;
  a = first + (q - b * in_group);
}


// XOR swizzle of the 64-byte LDS rows of the direct-to-LDS pipeline: 16-byte chunk c of row r sits in slot
// c ^ lds_swizzle(r). Found by exhaustive search: fragment reads (32 consecutive rows, same chunk) are free of bank
// conflicts both for 8 lanes over 32 banks and for 16 lanes over 64 banks.
__device__ inline int lds_swizzle(int row) { return ((row >> 2) & 1) | ((((row >> 1) ^ (row >> 3)) & 1) << 1); }

inline int check_segments(const ck_segments* seg, const char* name) {
  CK_REQUIRE(seg != nullptr, "%s: seg is NULL", name);
  CK_REQUIRE(seg->seg_starts && seg->counts && seg->tile_expert && seg->row_slot, "%s: NULL table in seg", name);
  CK_REQUIRE(seg->align == 128 || seg->align == 256, "%s: align=%d must be 128 or 256", name, seg->align);
  CK_REQUIRE(seg->num_experts >= 1, "%s: num_experts=%d", name, seg->num_experts);
  CK_REQUIRE(seg->max_rows >= 0 && seg->max_rows % seg->align == 0, "%s: max_rows=%lld is not a multiple of align", name,
             (long long)seg->max_rows);
  return CK_OK;
}

}  // namespace
}  // namespace ck
