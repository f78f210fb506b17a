// Expert histogram, offset scans and the stable token->expert counting sort.
//
// count:  one launch. Waves privatise the histogram (ballot/popcount counters in registers for <= 16 bins, per-wave LDS
//         copies up to 1024 bins, one LDS copy beyond), blocks merge into a zero-initialised global accumulator, and the
//         last block to finish (ticket counter) scans the bins, writes counts / inclusive ends / exclusive starts and
//         puts the accumulator back to zero.
// sort:   two launches. (1) every wave histograms its contiguous segment of the ids into a bin-major table
//         [bin][segment]; the last block scans that flattened table, which is exactly the destination of the first id of
//         every (bin, segment) pair in a stable sort, and derives counts / offsets / tile-aligned segment starts /
//         tile->expert table. (2) every wave re-reads its segment in order and ranks ids 64 at a time with bit-ballots.
#include <stdlib.h>

#include "ck_common.h"

namespace ck {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxCountBins = 16384;
constexpr int kMaxSortBins = 4096;
constexpr int kSortTableWords = 16384;  // bins * segments held in LDS by the scanning block

// Exclusive scan, in place, of data[0..n) (LDS) by a block of kBlock threads. Returns the total. tmp: kWavesPerBlock words.
__device__ uint32_t block_exclusive_scan(uint32_t* data, int n, uint32_t* tmp) {
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  const int per = (n + kBlock - 1) / kBlock;
  const int b = min(n, t * per), e = min(n, b + per);
  uint32_t s = 0;
  for (int i = b; i < e; ++i) s += data[i];
  uint32_t incl = s;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t v = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += v;
  }
  __syncthreads();
  if (lane == kWave - 1) tmp[wave] = incl;
  __syncthreads();
  uint32_t wave_off = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    const uint32_t v = tmp[w];
    if (w < wave) wave_off += v;
    total += v;
  }
  uint32_t run = wave_off + incl - s;
  for (int i = b; i < e; ++i) {
    const uint32_t v = data[i];
    data[i] = run;
    run += v;
  }
  __syncthreads();
  return total;
}

// Returns true in every thread of exactly one block: the last one to arrive. Blocks must have made their global
// writes before calling; the caller may read other blocks' writes after a true return.
// FENCE = false is for blocks that publish their data only through device-scope atomics: those are coherent across the
// XCDs by themselves and are complete once the barrier below has drained the wave's memory counters, so the L2
// write-back + invalidate of a full fence (about 0.2 us per block, serialised) is not needed.
template <bool FENCE>
__device__ bool last_block_ticket(uint32_t* ticket, uint32_t* lds_flag) {
  if constexpr (FENCE) __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t prev = atomicAdd(ticket, 1u);
    *lds_flag = (prev == gridDim.x - 1) ? 1u : 0u;
  }
  __syncthreads();
  const bool last = (*lds_flag != 0u);
  if (FENCE && last) __threadfence();
  return last;
}

template <typename id_t>
__device__ inline int load_id(const id_t* p) {
  const id_t v = *p;
  // ids outside int32 are out of range by definition; map them to -1
  if constexpr (sizeof(id_t) == 8) return (v >= 0 && v < (id_t)0x7fffffff) ? (int)v : -1;
  return (int)v;
}

// ------------------------------------------------------------------------------------------------------------
// count
// ------------------------------------------------------------------------------------------------------------
template <int REG_BINS>
struct RegCounters {
  uint32_t c[REG_BINS];
  __device__ RegCounters() {
#pragma unroll
    for (int i = 0; i < REG_BINS; ++i) c[i] = 0;
  }
  __device__ inline void add(int id) {
#pragma unroll
    for (int e = 0; e < REG_BINS; ++e) c[e] += (uint32_t)__popcll(__ballot(id == e));
  }
};

// REG_BINS > 0: wave-uniform register counters via ballot (num_bins <= REG_BINS): a handful of bins would make every
//               lane of an LDS atomic hit the same few addresses.
// REG_BINS == 0: LDS atomics on per-wave copies of the histogram.
template <typename id_t, int REG_BINS>
__global__ __launch_bounds__(kBlock) void count_kernel(const id_t* __restrict__ ids, int64_t n, int num_bins,
                                                        int lds_copies, int replicas, uint32_t* __restrict__ counts,
                                                        uint32_t* __restrict__ ends, uint32_t* __restrict__ starts,
                                                        uint32_t* __restrict__ ws) {
  extern __shared__ uint32_t lds[];  // [lds_copies][num_bins] then kWavesPerBlock + 1 words of scan scratch
  uint32_t* hist = lds;
  uint32_t* tmp = lds + (size_t)lds_copies * num_bins;
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;

  for (int i = t; i < lds_copies * num_bins; i += kBlock) hist[i] = 0;
  __syncthreads();
  uint32_t* my_hist = hist + (size_t)(lds_copies > 1 ? wave : 0) * num_bins;

  constexpr int VEC = 16 / sizeof(id_t);
  // scalar head up to the first 16-byte boundary, vector body, scalar tail
  const uintptr_t addr = reinterpret_cast<uintptr_t>(ids);
  int64_t head = ((16 - (addr & 15)) & 15) / sizeof(id_t);
  if (head > n) head = n;
  const int64_t nvec = (n - head) / VEC;
  const int64_t tail_begin = head + nvec * VEC;

  RegCounters<(REG_BINS > 0 ? REG_BINS : 1)> rc;
  auto tally = [&](int id) {
    if constexpr (REG_BINS > 0) {
      rc.add(id);
    } else {
      if ((unsigned)id < (unsigned)num_bins) atomicAdd(&my_hist[id], 1u);
    }
  };

  const id_t* body = ids + head;
  const int64_t gthreads = (int64_t)gridDim.x * kBlock;
  const int64_t gtid = (int64_t)blockIdx.x * kBlock + t;
  constexpr int UNROLL = 4;
  // every wave runs the same number of iterations so that ballots see whole waves
  const int64_t iters = (nvec + gthreads * UNROLL - 1) / (gthreads * UNROLL);
  for (int64_t it = 0; it < iters; ++it) {
    vec16 v[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t vi = (it * UNROLL + u) * gthreads + gtid;
      ok[u] = vi < nvec;
      v[u] = ok[u] ? load16_nt(body + vi * VEC) : zero16();  // ids are read once
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if constexpr (sizeof(id_t) == 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) tally(ok[u] ? (int)v[u].w[j] : -1);
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int64_t x = (int64_t)(((uint64_t)v[u].w[2 * j + 1] << 32) | v[u].w[2 * j]);
          tally((ok[u] && x >= 0 && x < 0x7fffffff) ? (int)x : -1);
        }
      }
    }
  }
  if (blockIdx.x == 0) {  // ragged ends, at most VEC-1 ids each; whole waves participate (ballot)
    const int64_t ragged = head + (n - tail_begin);
    for (int64_t base = 0; base < ragged; base += kBlock) {
      const int64_t r = base + t;
      int id = -1;
      if (r < ragged) id = load_id(ids + (r < head ? r : tail_begin + (r - head)));
      tally(id);
    }
  }

  if constexpr (REG_BINS > 0) {
    if (lane == 0) {
#pragma unroll
      for (int e = 0; e < REG_BINS; ++e)
        if (e < num_bins && rc.c[e]) atomicAdd(&hist[e], rc.c[e]);
    }
  }
  __syncthreads();
  if (lds_copies > 1) {
    for (int e = t; e < num_bins; e += kBlock) {
      uint32_t s = 0;
      for (int c = 0; c < lds_copies; ++c) s += hist[(size_t)c * num_bins + e];
      hist[e] = s;  // copy 0 row becomes the block total; other rows are not read again
    }
    __syncthreads();
  }

  // Blocks merge into one of `replicas` global accumulators (thousands of atomics on one cache line would serialise in a
  // single L2 channel); the last block adds the replicas up and puts them back to zero.
  uint32_t* acc = ws + 1;
  if (gridDim.x > 1) {
    uint32_t* my_acc = acc + (size_t)(blockIdx.x % replicas) * num_bins;
    for (int e = t; e < num_bins; e += kBlock)
      if (hist[e]) atomicAdd(&my_acc[e], hist[e]);
    if (!last_block_ticket<false>(ws, tmp + kWavesPerBlock)) return;
    // Sum the replicas that were used and put them back to zero. Device-scope atomic loads read the values where the
    // other blocks' atomics left them; the loads of one thread are independent, so their latencies overlap.
    const int used = min(replicas, (int)gridDim.x);
    for (int e = t; e < num_bins; e += kBlock) hist[e] = 0;
    __syncthreads();
    for (int idx = t; idx < used * num_bins; idx += kBlock) {  // (replica, bin) pairs spread over the whole block
      const uint32_t v = __hip_atomic_load(&acc[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      acc[idx] = 0u;  // visible to the next launch at the kernel boundary; nobody reads it before
      if (v) atomicAdd(&hist[idx % num_bins], v);
    }
    if (t == 0) ws[0] = 0u;
    __syncthreads();
  }
  // hist[0..num_bins) now holds the global counts
  for (int e = t; e < num_bins; e += kBlock) counts[e] = hist[e];
  if (ends != nullptr || starts != nullptr) {
    __syncthreads();
    block_exclusive_scan(hist, num_bins, tmp);
    for (int e = t; e < num_bins; e += kBlock) {
      const uint32_t s = hist[e];
      if (starts) starts[e] = s;
      if (ends) ends[e] = s + counts[e];  // counts[e] was written by this same thread above
    }
  }
}

// ------------------------------------------------------------------------------------------------------------
// sort
// ------------------------------------------------------------------------------------------------------------
constexpr int kSortUnroll = 8;  // ids a lane fetches before it consumes them

struct SortPlan {
  int segments;    // multiple of kWavesPerBlock
  int64_t seg_len; // multiple of kWave
};

// ids per wave segment (measured at 256 .. 4096: more, shorter segments lengthen the last block's scan; 1024 is fastest)
constexpr int64_t kSortIdsPerSegment = 1024;

SortPlan make_sort_plan(int64_t R, int E) {
  int64_t cap = kSortTableWords / (E > 0 ? E : 1);
  cap = (cap / kWavesPerBlock) * kWavesPerBlock;
  if (cap < kWavesPerBlock) cap = kWavesPerBlock;
  int64_t want = ceil_div(R > 0 ? R : 1, kSortIdsPerSegment);
  want = round_up(want, kWavesPerBlock);
  SortPlan p;
  p.segments = (int)(want < cap ? want : cap);
  p.seg_len = round_up(ceil_div(R > 0 ? R : 1, p.segments), kWave);
  return p;
}

// ws layout (uint32 words): [0] ticket, [1 .. 1 + E*S) bin-major table, scanned in place by the last block.
template <typename id_t>
__global__ __launch_bounds__(kBlock) void sort_hist_kernel(const id_t* __restrict__ ids, int64_t R, int E, int S,
                                                            int64_t seg_len, int align, int64_t max_tiles,
                                                            uint32_t* __restrict__ counts, uint32_t* __restrict__ ends,
                                                            uint32_t* __restrict__ starts, int32_t* __restrict__ seg_starts,
                                                            int32_t* __restrict__ tile_expert, uint32_t* __restrict__ ws) {
  extern __shared__ uint32_t lds[];  // max(4*E, E*S + E + 1) words + scan scratch (placed at the end)
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  uint32_t* my_hist = lds + (size_t)wave * E;
  for (int i = t; i < kWavesPerBlock * E; i += kBlock) lds[i] = 0;
  __syncthreads();

  const int seg = blockIdx.x * kWavesPerBlock + wave;
  const int64_t begin = (int64_t)seg * seg_len;
  const int64_t end = min(R, begin + seg_len);
  // kSortUnroll loads in flight per lane: a segment is a handful of dependent-latency round trips otherwise
  for (int64_t base = begin + lane; base < end; base += kSortUnroll * kWave) {
    int id[kSortUnroll];
#pragma unroll
    for (int u = 0; u < kSortUnroll; ++u) {
      const int64_t i = base + u * kWave;
      id[u] = i < end ? load_id(ids + i) : -1;
    }
#pragma unroll
    for (int u = 0; u < kSortUnroll; ++u)
      if ((unsigned)id[u] < (unsigned)E) atomicAdd(&my_hist[id[u]], 1u);
  }
  __syncthreads();
  uint32_t* table = ws + 1;
  for (int e = lane; e < E; e += kWave) table[(size_t)e * S + seg] = my_hist[e];

  const int table_words = E * S;
  uint32_t* tmp = lds + max(kWavesPerBlock * E, table_words + E + 1);
  if (!last_block_ticket<true>(ws, tmp + kWavesPerBlock)) return;

  // ---- last block: scan the flattened bin-major table in LDS
  uint32_t* tab = lds;
  for (int i = t; i < table_words; i += kBlock) tab[i] = table[i];
  __syncthreads();
  const uint32_t total = block_exclusive_scan(tab, table_words, tmp);
  for (int i = t; i < table_words; i += kBlock) table[i] = tab[i];
  uint32_t* padded = tab + table_words;  // [E + 1]
  for (int e = t; e < E; e += kBlock) {
    const uint32_t s = tab[(size_t)e * S];
    const uint32_t nxt = (e + 1 < E) ? tab[(size_t)(e + 1) * S] : total;
    const uint32_t c = nxt - s;
    counts[e] = c;
    starts[e] = s;
    ends[e] = nxt;
    padded[e] = (c + (uint32_t)align - 1) / (uint32_t)align * (uint32_t)align;
  }
  __syncthreads();
  const uint32_t padded_total = block_exclusive_scan(padded, E, tmp);
  if (t == 0) padded[E] = padded_total;
  __syncthreads();
  for (int e = t; e <= E; e += kBlock) seg_starts[e] = (int32_t)padded[e];
  for (int64_t tile = t; tile < max_tiles; tile += kBlock) {
    const uint32_t row = (uint32_t)(tile * align);
    int32_t owner = -1;
    if (row < padded_total) {
      // last e with padded[e] <= row; empty experts share a start with their successor and are skipped by "last"
      int lo = 0, hi = E - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (padded[mid] <= row) lo = mid; else hi = mid - 1;
      }
      owner = lo;
    }
    tile_expert[tile] = owner;
  }
  if (t == 0) ws[0] = 0u;
}

template <typename id_t>
__global__ __launch_bounds__(kBlock) void sort_scatter_kernel(const id_t* __restrict__ ids, int64_t R, int E, int S,
                                                               int64_t seg_len, int id_bits,
                                                               const uint32_t* __restrict__ starts,
                                                               const int32_t* __restrict__ seg_starts,
                                                               int32_t* __restrict__ sorted_expert_idxs,
                                                               int32_t* __restrict__ sorted_scattered_idxs,
                                                               int32_t* __restrict__ row_slot,
                                                               const uint32_t* __restrict__ ws) {
  extern __shared__ uint32_t lds[];  // [kWavesPerBlock][E] running destination of the next id of each bin
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  uint32_t* next = lds + (size_t)wave * E;
  const int seg = blockIdx.x * kWavesPerBlock + wave;
  const uint32_t* table = ws + 1;
  for (int e = lane; e < E; e += kWave) next[e] = table[(size_t)e * S + seg];
  // LDS traffic below is wave-private and a wave's LDS operations complete in program order: no barrier needed.
  const int64_t begin = (int64_t)seg * seg_len;
  const int64_t end = min(R, begin + seg_len);
  const uint64_t lanes_below = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));
  for (int64_t chunk = begin; chunk < end; chunk += kSortUnroll * kWave) {
    int ids_ahead[kSortUnroll];  // the ids of the next kSortUnroll rounds, fetched together
#pragma unroll
    for (int u = 0; u < kSortUnroll; ++u) {
      const int64_t i = chunk + u * kWave + lane;
      ids_ahead[u] = i < end ? load_id(ids + i) : -1;
    }
#pragma unroll
    for (int u = 0; u < kSortUnroll; ++u) {
    const int64_t base = chunk + u * kWave;
    if (base >= end) break;
    const int64_t i = base + lane;
    const int id = ids_ahead[u];
    const bool valid = (unsigned)id < (unsigned)E;
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < id_bits; ++b) {
      const bool bit = (id >> b) & 1;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    if (valid) {
      const uint32_t rank = (uint32_t)__popcll(peers & lanes_below);
      const uint32_t group = (uint32_t)__popcll(peers);
      const uint32_t pos = next[id] + rank;
      if (rank == group - 1) next[id] = pos + 1;  // highest lane of the group advances the bin
      sorted_expert_idxs[pos] = id;
      sorted_scattered_idxs[pos] = (int32_t)i;
      row_slot[(uint32_t)seg_starts[id] + (pos - starts[id])] = (int32_t)i;
    }
    }
  }
}

}  // namespace
}  // namespace ck

using namespace ck;

// global accumulator replicas: as many as fit in 16384 words, at most 32
static int count_replicas(int num_bins) {
  int r = kMaxCountBins / (num_bins > 0 ? num_bins : 1);
  return r < 1 ? 1 : (r > 32 ? 32 : r);
}

extern "C" int64_t ck_count_workspace_words(int32_t num_bins) {
  return 1 + (int64_t)(num_bins > 0 ? num_bins : 0) * count_replicas(num_bins);
}

namespace ck {
namespace {

// Validates the arguments and launches count_kernel on `workspace` (zero on entry, zero again on exit).
int launch_count(const char* name, const void* ids, int32_t ids_are_i64, int64_t n, int32_t num_bins, uint32_t* counts,
                 uint32_t* ends, uint32_t* starts, uint32_t* workspace, hipStream_t s) {
  CK_REQUIRE(num_bins >= 1 && num_bins <= kMaxCountBins, "%s: num_bins=%d outside [1, %d]", name, num_bins, kMaxCountBins);
  CK_REQUIRE(n >= 0, "%s: n=%lld is negative", name, (long long)n);
  CK_REQUIRE(counts != nullptr && workspace != nullptr, "%s: counts and workspace are required", name);
  CK_REQUIRE(n == 0 || ids != nullptr, "%s: ids is NULL", name);
  const size_t esz = ids_are_i64 ? 8 : 4;
  CK_REQUIRE((reinterpret_cast<uintptr_t>(ids) & (esz - 1)) == 0, "%s: ids is not element-aligned", name);

  const int64_t vec = 16 / (int64_t)esz;
  // 4 vectors per thread per trip; one block for small inputs. Large inputs: 2 blocks per CU stream fastest with the LDS
  // path (6.5 TB/s at 512 blocks, 6.1 at 1024, 3.7 at 256); the ballot path is VALU-heavier and wants 4 per CU.
  int64_t blocks = ceil_div(n, (int64_t)kBlock * vec * 4 * 4);
  if (blocks < 1) blocks = 1;
  const int64_t max_blocks = num_bins <= 8 ? 1024 : 512;
  if (blocks > max_blocks) blocks = max_blocks;
  // up to 8 bins: ballot counters in registers (5.8 TB/s; LDS atomics on so few addresses serialise: 2.1-5.1 TB/s);
  // more bins: LDS atomics (6.3-6.5 TB/s; 16 register counters measured 3.3 TB/s)
  const int reg_bins = num_bins <= 8 ? 8 : 0;  // 16 register counters measured slower (3.3 TB/s) than LDS atomics (5.6)
  const int copies = reg_bins > 0 ? 1 : (num_bins <= 1024 ? kWavesPerBlock : 1);
  const size_t lds_bytes = ((size_t)copies * num_bins + kWavesPerBlock + 2) * sizeof(uint32_t);
#define CK_LAUNCH_COUNT(ID_T, RB)                                                                              \
  hipLaunchKernelGGL((count_kernel<ID_T, RB>), dim3((unsigned)blocks), dim3(kBlock), lds_bytes, s,            \
                     static_cast<const ID_T*>(ids), n, (int)num_bins, copies, count_replicas(num_bins), counts, ends,   \
                     starts, workspace)
  if (ids_are_i64) {
    if (reg_bins == 8) CK_LAUNCH_COUNT(int64_t, 8);
    else CK_LAUNCH_COUNT(int64_t, 0);
  } else {
    if (reg_bins == 8) CK_LAUNCH_COUNT(int32_t, 8);
    else CK_LAUNCH_COUNT(int32_t, 0);
  }
#undef CK_LAUNCH_COUNT
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------------
// The count kernel's workspace (ticket + replicated global accumulators: at most 1 + 16384 words) lives in this
// file-scope device array instead of a caller's buffer. Every GPU holds its own copy at its own address until the
// process ends. In host code the array's name is only a handle for hipGetSymbolAddress: the address a kernel may use is
// looked up once per device, with that device current, and kept in g_scratch_ptr.
constexpr int kScratchWords = 1 + kMaxCountBins;
static __device__ __align__(256) uint32_t scratch[kScratchWords];

constexpr int kMaxScratchDevices = 64;
uint32_t* g_scratch_ptr[kMaxScratchDevices] = {};

int scratch_for_current_device(const char* name, uint32_t** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxScratchDevices) {
    set_error("%s: cannot tell the current device (%s, device %d)", name, hipGetErrorString(e), dev);
    return CK_ERR_LAUNCH;
  }
  uint32_t* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p == nullptr) {  // first call on this device; a race between host threads only repeats the same lookup
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || sym == nullptr) {
      set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", name, dev, hipGetErrorString(e));
      return CK_ERR_LAUNCH;
    }
    p = static_cast<uint32_t*>(sym);
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);
  }
  *out = p;
  return CK_OK;
}

__global__ __launch_bounds__(kBlock) void zero_words_kernel(uint32_t* __restrict__ p, int words) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < words) p[i] = 0u;
}

}  // namespace
}  // namespace ck

extern "C" int ck_count_offsets(const void* ids, int32_t ids_are_i64, int64_t n, int32_t num_bins, uint32_t* counts,
                                uint32_t* ends, uint32_t* starts, uint32_t* workspace, void* stream) {
  return launch_count("ck_count_offsets", ids, ids_are_i64, n, num_bins, counts, ends, starts, workspace,
                      static_cast<hipStream_t>(stream));
}

extern "C" int ck_count_offsets_static(const void* ids, int32_t ids_are_i64, int64_t n, int32_t num_bins, uint32_t* counts,
                                       uint32_t* ends, uint32_t* starts, void* stream) {
  const char* name = "ck_count_offsets_static";
  CK_REQUIRE(num_bins >= 1 && num_bins <= kMaxCountBins,
             "%s: num_bins=%d outside [1, %d] (the built-in workspace holds %d words)", name, num_bins, kMaxCountBins,
             kScratchWords);
  const int64_t words = ck_count_workspace_words(num_bins);
  CK_REQUIRE(words <= kScratchWords, "%s: num_bins=%d needs %lld workspace words, the built-in workspace holds %d", name,
             num_bins, (long long)words, kScratchWords);
  uint32_t* ws = nullptr;
  if (int rc = scratch_for_current_device(name, &ws)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The array keeps whatever the last call on this GPU left (zeros after a completed call, anything after one that was
  // cut short): the words this call uses are cleared first, by a kernel, so that the sequence can be captured in a graph.
  hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)ceil_div(words, kBlock)), dim3(kBlock), 0, s, ws, (int)words);
  CK_CHECK_LAUNCH(name);
  return launch_count(name, ids, ids_are_i64, n, num_bins, counts, ends, starts, ws, s);
}

// The padded grouped layout from a sort somebody else did (torch.sort + bincount + cumsum in the reference's own layer):
// every block derives the tile-aligned segment starts from the inclusive offsets (E is small), block 0 writes the tables,
// and every sorted position p of expert e goes to padded row seg_starts[e] + (p - starts[e]).
template <typename id_t, typename off_t>
__global__ __launch_bounds__(kBlock) void segments_from_sorted_kernel(
    const id_t* __restrict__ sorted_expert_idxs, const id_t* __restrict__ sorted_scattered_idxs,
    const off_t* __restrict__ ends, int64_t R, int E, int align, int64_t max_tiles, uint32_t* __restrict__ counts,
    int32_t* __restrict__ seg_starts, int32_t* __restrict__ row_slot, int32_t* __restrict__ row_pos,
    int32_t* __restrict__ tile_expert) {
  extern __shared__ uint32_t lds[];  // padded[E + 1], starts[E], count[E], scan scratch
  uint32_t* padded = lds;
  uint32_t* first = lds + E + 1;
  uint32_t* count = first + E;
  uint32_t* tmp = count + E;
  const int t = threadIdx.x;
  for (int e = t; e < E; e += kBlock) {
    const uint32_t end = (uint32_t)ends[e], begin = e > 0 ? (uint32_t)ends[e - 1] : 0u;
    const uint32_t c = end >= begin ? end - begin : 0u;
    first[e] = begin;
    count[e] = c;
    padded[e] = (c + (uint32_t)align - 1) / (uint32_t)align * (uint32_t)align;
  }
  __syncthreads();
  const uint32_t padded_total = block_exclusive_scan(padded, E, tmp);
  if (t == 0) padded[E] = padded_total;
  __syncthreads();
  if (blockIdx.x == 0) {
    for (int e = t; e < E; e += kBlock) counts[e] = count[e];
    for (int e = t; e <= E; e += kBlock) seg_starts[e] = (int32_t)padded[e];
    for (int64_t tile = t; tile < max_tiles; tile += kBlock) {
      const uint32_t row = (uint32_t)(tile * align);
      int32_t owner = -1;
      if (row < padded_total) {  // last e with padded[e] <= row (empty experts share a start with their successor)
        int lo = 0, hi = E - 1;
        while (lo < hi) {
          const int mid = (lo + hi + 1) >> 1;
          if (padded[mid] <= row) lo = mid; else hi = mid - 1;
        }
        owner = lo;
      }
      tile_expert[tile] = owner;
    }
  }
  for (int64_t p = (int64_t)blockIdx.x * kBlock + t; p < R; p += (int64_t)gridDim.x * kBlock) {
    const int e = load_id(sorted_expert_idxs + p);
    if ((unsigned)e >= (unsigned)E) continue;
    const int64_t j = p - (int64_t)first[e];
    if (j < 0 || j >= (int64_t)count[e]) continue;  // offsets that do not describe these ids: the row stays unowned
    const int64_t dst = (int64_t)padded[e] + j;
    row_slot[dst] = load_id(sorted_scattered_idxs + p);
    row_pos[dst] = (int32_t)p;
  }
}

extern "C" int ck_segments_from_sorted(const void* sorted_expert_idxs, const void* sorted_scattered_idxs,
                                       int32_t idxs_are_i64, const void* expert_offsets, int32_t offsets_are_i64,
                                       int64_t R, int32_t E, int32_t align, uint32_t* counts, int32_t* seg_starts,
                                       int32_t* row_slot, int32_t* row_pos, int32_t* tile_expert, void* stream) {
  const char* name = "ck_segments_from_sorted";
  CK_REQUIRE(E >= 1 && E <= kMaxSortBins, "%s: E=%d outside [1, %d]", name, E, kMaxSortBins);
  CK_REQUIRE(align >= 1, "%s: align=%d must be positive", name, align);
  CK_REQUIRE(R >= 0 && R < (int64_t)0x7fffffff - (int64_t)E * align, "%s: R=%lld out of range", name, (long long)R);
  CK_REQUIRE(expert_offsets && counts && seg_starts && row_slot && row_pos && tile_expert, "%s: NULL argument", name);
  CK_REQUIRE(R == 0 || (sorted_expert_idxs && sorted_scattered_idxs), "%s: NULL index tensor", name);
  const int64_t max_tiles = ck_sort_max_rows(R, E, align) / align;
  int64_t blocks = ceil_div(R > 0 ? R : 1, (int64_t)kBlock * 4);
  if (blocks > 1024) blocks = 1024;
  const size_t lds_bytes = ((size_t)3 * E + 1 + kWavesPerBlock) * sizeof(uint32_t);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CK_LAUNCH_SEGMENTS(ID_T, OFF_T)                                                                               \
  hipLaunchKernelGGL((segments_from_sorted_kernel<ID_T, OFF_T>), dim3((unsigned)blocks), dim3(kBlock), lds_bytes, s, \
                     static_cast<const ID_T*>(sorted_expert_idxs), static_cast<const ID_T*>(sorted_scattered_idxs),   \
                     static_cast<const OFF_T*>(expert_offsets), R, (int)E, (int)align, max_tiles, counts, seg_starts, \
                     row_slot, row_pos, tile_expert)
  if (idxs_are_i64) {
    if (offsets_are_i64) CK_LAUNCH_SEGMENTS(int64_t, int64_t);
    else CK_LAUNCH_SEGMENTS(int64_t, int32_t);
  } else {
    if (offsets_are_i64) CK_LAUNCH_SEGMENTS(int32_t, int64_t);
    else CK_LAUNCH_SEGMENTS(int32_t, int32_t);
  }
#undef CK_LAUNCH_SEGMENTS
  CK_CHECK_LAUNCH(name);
  return CK_OK;
}

extern "C" int64_t ck_sort_max_rows(int64_t R, int32_t E, int32_t align) {
  if (R < 0 || E < 1 || align < 1) return 0;
  // sum_e round_up(c_e, align) <= R + E * (align - 1); round to whole tiles
  return round_up(R + (int64_t)E * (align - 1), align);
}

extern "C" int64_t ck_sort_workspace_words(int64_t R, int32_t E) {
  if (E < 1) return 1;
  const SortPlan p = make_sort_plan(R, E);
  return 1 + (int64_t)E * p.segments;
}

extern "C" int ck_sort_by_expert(const void* expert_ids, int32_t ids_are_i64, int64_t R, int32_t E, int32_t align,
                                 int32_t* sorted_expert_idxs, int32_t* sorted_scattered_idxs, uint32_t* counts,
                                 uint32_t* ends, uint32_t* starts, int32_t* seg_starts, int32_t* row_slot,
                                 int32_t* tile_expert, uint32_t* workspace, void* stream) {
  CK_REQUIRE(E >= 1 && E <= kMaxSortBins, "ck_sort_by_expert: E=%d outside [1, %d]", E, kMaxSortBins);
  CK_REQUIRE(R >= 0 && R < (int64_t)0x7fffffff - (int64_t)E * align, "ck_sort_by_expert: R=%lld out of range",
             (long long)R);
  CK_REQUIRE(align >= 1, "ck_sort_by_expert: align=%d must be positive", align);
  CK_REQUIRE(R == 0 || expert_ids != nullptr, "ck_sort_by_expert: expert_ids is NULL");
  CK_REQUIRE(sorted_expert_idxs && sorted_scattered_idxs && counts && ends && starts && seg_starts && row_slot &&
                 tile_expert && workspace,
             "ck_sort_by_expert: every output and the workspace are required");
  const SortPlan p = make_sort_plan(R, E);
  const int blocks = p.segments / kWavesPerBlock;
  const int64_t max_tiles = ck_sort_max_rows(R, E, align) / align;
  int id_bits = 0;
  while ((1 << id_bits) < E) ++id_bits;
  const size_t table_words = (size_t)E * p.segments;
  size_t lds_words = (size_t)kWavesPerBlock * E;
  if (table_words + E + 1 > lds_words) lds_words = table_words + E + 1;
  const size_t lds_hist = (lds_words + kWavesPerBlock + 2) * sizeof(uint32_t);
  const size_t lds_scatter = (size_t)kWavesPerBlock * E * sizeof(uint32_t);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ids_are_i64) {
    const int64_t* ids = static_cast<const int64_t*>(expert_ids);
    hipLaunchKernelGGL((sort_hist_kernel<int64_t>), dim3(blocks), dim3(kBlock), lds_hist, s, ids, R, (int)E,
                       p.segments, p.seg_len, (int)align, max_tiles, counts, ends, starts, seg_starts, tile_expert,
                       workspace);
    hipLaunchKernelGGL((sort_scatter_kernel<int64_t>), dim3(blocks), dim3(kBlock), lds_scatter, s, ids, R, (int)E,
                       p.segments, p.seg_len, id_bits, starts, seg_starts, sorted_expert_idxs, sorted_scattered_idxs,
                       row_slot, workspace);
  } else {
    const int32_t* ids = static_cast<const int32_t*>(expert_ids);
    hipLaunchKernelGGL((sort_hist_kernel<int32_t>), dim3(blocks), dim3(kBlock), lds_hist, s, ids, R, (int)E,
                       p.segments, p.seg_len, (int)align, max_tiles, counts, ends, starts, seg_starts, tile_expert,
                       workspace);
    hipLaunchKernelGGL((sort_scatter_kernel<int32_t>), dim3(blocks), dim3(kBlock), lds_scatter, s, ids, R, (int)E,
                       p.segments, p.seg_len, id_bits, starts, seg_starts, sorted_expert_idxs, sorted_scattered_idxs,
                       row_slot, workspace);
  }
  CK_CHECK_LAUNCH("ck_sort_by_expert");
  return CK_OK;
}
