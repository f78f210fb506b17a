/*
 * ck_oracle.c -- CPU restatement of the integer stages of the cute-kernels MoE path, in plain C.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker, never the product: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may build, load or call it. The shipped path is the HIP library; it never falls back here.
 *
 * Every function cites the reference lines it restates (paths relative to the reference root) and is pinned in
 * tests/test_oracle.py against library routines (numpy / torch bincount, cumsum, stable sort), brute force on tiny
 * inputs and invariants -- not against itself.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Histogram of ids in [0, num_bins); ids outside the range are not counted.
 * Reference: continuous_count_torch = x.bincount(minlength=size).to(uint32),
 * cute_kernels/kernels/continuous_count/torch_implementation.py:8-10; "values outside this range are ignored",
 * cute_kernels/kernels/continuous_count/__init__.py:15-17. */
void oracle_count(const int64_t* ids, int64_t n, int32_t num_bins, uint32_t* counts) {
  memset(counts, 0, sizeof(uint32_t) * (size_t)num_bins);
  for (int64_t i = 0; i < n; ++i)
    if (ids[i] >= 0 && ids[i] < num_bins) counts[ids[i]] += 1u;
}

/* Inclusive ("ends") and exclusive ("starts") prefix sums of the counts.
 * Reference: expert_offsets = bincount(...).cumsum(-1), scattermoe/triton_implementation/__init__.py:83; consumed as
 * inclusive ends at scattermoe/triton_implementation/kernels.py:174-179. */
void oracle_offsets(const uint32_t* counts, int32_t num_bins, uint32_t* ends, uint32_t* starts) {
  uint32_t run = 0;
  for (int32_t e = 0; e < num_bins; ++e) {
    starts[e] = run;
    run += counts[e];
    ends[e] = run;
  }
}

/* Stable sort of the flat (token, slot) expert ids.
 * Reference: sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort(),
 * scattermoe/triton_implementation/__init__.py:82; index_sorted_experts = selected_experts.argsort(),
 * scattermoe/torch_implementation.py:182. Ties keep input order (stable), which makes the permutation unique. */
void oracle_sort_by_expert(const int64_t* ids, int64_t n, int32_t num_experts, int32_t* sorted_expert_idxs,
                           int32_t* sorted_scattered_idxs) {
  int64_t* next = (int64_t*)calloc((size_t)num_experts + 1, sizeof(int64_t));
  for (int64_t i = 0; i < n; ++i) next[ids[i] + 1] += 1;
  for (int32_t e = 0; e < num_experts; ++e) next[e + 1] += next[e];
  for (int64_t i = 0; i < n; ++i) {
    const int64_t pos = next[ids[i]]++;
    sorted_expert_idxs[pos] = (int32_t)ids[i];
    sorted_scattered_idxs[pos] = (int32_t)i;
  }
  free(next);
}

/* Tile-aligned expert segments of the padded grouped layout (this build's own layout; no reference counterpart):
 * seg_starts[e] = sum_{e' < e} round_up(counts[e'], align); row_slot[seg_starts[e] + j] = j-th sorted slot of e
 * (-1 in pad rows); tile_expert[t] = owner of rows [t*align, (t+1)*align), -1 past the end. */
void oracle_segments(const uint32_t* counts, const int32_t* sorted_scattered_idxs, int32_t num_experts, int32_t align,
                     int64_t max_rows, int32_t* seg_starts, int32_t* row_slot, int32_t* tile_expert) {
  int64_t run = 0, src = 0;
  for (int64_t p = 0; p < max_rows; ++p) row_slot[p] = -1;
  for (int64_t t = 0; t < max_rows / align; ++t) tile_expert[t] = -1;
  for (int32_t e = 0; e < num_experts; ++e) {
    seg_starts[e] = (int32_t)run;
    for (uint32_t j = 0; j < counts[e]; ++j) row_slot[run + j] = sorted_scattered_idxs[src + j];
    src += counts[e];
    const int64_t padded = ((int64_t)counts[e] + align - 1) / align * align;
    for (int64_t t = run / align; t < (run + padded) / align; ++t) tile_expert[t] = e;
    run += padded;
  }
  seg_starts[num_experts] = (int32_t)run;
}

/* Top-k over one row of logits and softmax over the k selected logits.
 * Reference: MoE_Torch._get_topk (x.topk(k), values sorted descending) and
 * F.softmax(router_weights.float(), dim=-1), scattermoe/torch_implementation.py:127-133,195-201.
 * torch.topk leaves the order of equal logits unspecified; this build fixes it: lowest expert index first.
 * -0.0 and +0.0 compare equal; NaN ranks above every number (torch's ordering). */
static int ranks_before(float a, int32_t ia, float b, int32_t ib) {
  const int a_nan = isnan(a), b_nan = isnan(b);
  if (a_nan || b_nan) {
    if (a_nan && b_nan) return ia < ib;
    return a_nan;
  }
  if (a != b) return a > b;
  return ia < ib;
}

void oracle_topk_softmax(const float* logits, int64_t T, int32_t E, int32_t k, int32_t* selected, float* gates,
                         float* values) {
  uint8_t* taken = (uint8_t*)malloc((size_t)E);
  for (int64_t t = 0; t < T; ++t) {
    const float* row = logits + t * E;
    memset(taken, 0, (size_t)E);
    for (int32_t j = 0; j < k; ++j) {
      int32_t best = -1;
      for (int32_t e = 0; e < E; ++e) {
        if (taken[e]) continue;
        if (best < 0 || ranks_before(row[e], e, row[best], best)) best = e;
      }
      taken[best] = 1;
      selected[t * k + j] = best;
      values[t * k + j] = row[best];
    }
    /* softmax in fp32 with the usual max subtraction; the first selected value is the max */
    const float m = values[t * k];
    float denom = 0.f;
    for (int32_t j = 0; j < k; ++j) {
      gates[t * k + j] = expf(values[t * k + j] - m);
      denom += gates[t * k + j];
    }
    for (int32_t j = 0; j < k; ++j) gates[t * k + j] /= denom;
  }
  free(taken);
}
