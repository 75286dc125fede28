// Host-only part of the library: status text, per-thread error message, and the
// integer helpers of the C ABI.

#include <stdarg.h>
#include <stdio.h>

#include <mutex>
#include <utility>
#include <vector>

#include "elementwise.hpp"
#include "softmax.hpp"

namespace oslo {
namespace {
thread_local char g_error[256] = "";
}

int fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return status;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return OSLO_OK;
  return fail(OSLO_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

int raise_lds_limit(const void *kernel, unsigned bytes, const char *what) {
  static std::mutex mutex;
  static std::vector<std::pair<const void *, int>> done; // (kernel, device)
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(OSLO_E_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(mutex);
  for (const auto &entry : done)
    if (entry.first == kernel && entry.second == dev) return OSLO_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess)
    return fail(OSLO_E_LAUNCH, "%s: %u bytes of dynamic LDS refused: %s", what, bytes, hipGetErrorString(e));
  done.emplace_back(kernel, dev);
  return OSLO_OK;
}

} // namespace oslo

extern "C" int oslo_abi_version(void) { return 1; }

extern "C" int oslo_softmax_max_cols(void) { return oslo::kSoftmaxMaxCols; }

extern "C" const char *oslo_status_string(int status) {
  switch (status) {
  case OSLO_OK: return "ok";
  case OSLO_E_BAD_ARG: return "bad argument";
  case OSLO_E_UNSUPPORTED: return "unsupported shape";
  case OSLO_E_LAUNCH: return "kernel launch failed";
  default: return "unknown status";
  }
}

extern "C" const char *oslo_last_error(void) { return oslo::g_error; }

// The reference's arithmetic (oslo/fused_kernels/includes/fused_softmax.h
// :328-340) with its constants: 32-lane warps, 128 threads per block, two rows
// per warp up to 128 keys.
extern "C" int oslo_get_batch_per_block(int sq, int sk, int batches, int heads) {
  (void)sq;
  (void)batches;
  (void)heads;
  int log2_elements = 0;
  while ((1 << log2_elements) < sk) ++log2_elements;
  const int next_pow2 = 1 << log2_elements;
  const int warp_size = next_pow2 < 32 ? next_pow2 : 32;
  const int rows_per_warp = next_pow2 <= 128 ? 2 : 1;
  return rows_per_warp * (128 / warp_size);
}

extern "C" size_t oslo_colsum_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  // One fp32 partial row per block of rows; no backward kernel covers fewer
  // than kBwdMinRowsPerBlock rows per block, whatever the dtype and alignment.
  const int64_t parts =
      (rows + oslo::kBwdMinRowsPerBlock - 1) / oslo::kBwdMinRowsPerBlock;
  return (size_t)parts * (size_t)cols * sizeof(float);
}
