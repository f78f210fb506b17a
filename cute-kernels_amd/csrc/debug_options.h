// ck_debug_set_option: process-wide choices between kernels that compute the same result (tests and measurements).
// The defaults are what the product runs.
#pragma once

#include <atomic>

namespace ck {

struct DebugOptions {
  std::atomic<int> gemm_line_kernel{1};        // 0: every 16-bit grouped GEMM runs on the general kernel
  std::atomic<int> gemm_register_pipeline{0};  // 1: the general kernel stages through registers (its K % 8 pipeline)
  std::atomic<int> gemm_four_waves{0};         // 1: the general kernel's direct-to-LDS pipeline with 4 waves instead of 8
  std::atomic<void*> trace_buffer{nullptr};    // CK_STAMP measurement builds write their cycle counts here
};
DebugOptions& debug_options();

}  // namespace ck
