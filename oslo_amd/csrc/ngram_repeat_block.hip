// Repeated n-gram blocking for beam search, for gfx950: for every hypothesis
// (row) the tokens that would complete an n-gram already present in the row get
// log-probability -inf. Behaviour follows banRepeatedTokens
// (oslo/fused_kernels/fused_ngram_repeat_block.cu:18-49) and its launcher
// (:54-75).
//
// The reference launches one thread per earlier n-gram (so at most 1024 tokens
// per hypothesis) and stages the row in shared memory. Here a block of 256
// threads strides over the positions, so any length works, and the tokens are
// read in place: a row is a few KiB that all threads of the block share through
// the cache, and the kernel is launch-latency bound either way. It runs on the
// caller's stream (the reference uses the default stream,
// oslo/fused_kernels/fused_ngram_repeat_block.cu:72-73).

#include "common.hpp"

namespace oslo {
namespace {

__global__ __launch_bounds__(kBlockThreads) void ngram_repeat_block_kernel(
    float *__restrict__ lprobs, const int64_t *__restrict__ tokens,
    int64_t max_len, int64_t step, int64_t vocab, int n) {
  const int64_t row = blockIdx.x;
  const int64_t *t = tokens + row * max_len;
  float *lp = lprobs + row * vocab;
  // the last n-1 tokens start here; earlier n-grams start at 0 .. last_start-1
  const int64_t last_start = step - n + 2;
  for (int64_t i = threadIdx.x; i < last_start; i += kBlockThreads) {
    bool same = true;
    for (int k = 0; k < n - 1; ++k) {
      if (t[i + k] != t[last_start + k]) {
        same = false;
        break;
      }
    }
    if (same) {
      const int64_t banned = t[i + n - 1];
      if (banned >= 0 && banned < vocab) lp[banned] = -INFINITY;
    }
  }
}

} // namespace
} // namespace oslo

extern "C" int oslo_ngram_repeat_block(float *lprobs, const int64_t *tokens,
                                       int64_t rows, int64_t max_len,
                                       int64_t step, int64_t vocab, int n,
                                       oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || max_len < 0 || step < 0 || vocab < 0 || n <= 0)
    return fail(OSLO_E_BAD_ARG, "ngram_repeat_block: negative size or n <= 0");
  if (step + 1 > max_len)
    return fail(OSLO_E_BAD_ARG,
                "ngram_repeat_block: step %lld needs %lld tokens per row, rows hold %lld",
                (long long)step, (long long)(step + 1), (long long)max_len);
  if (rows > INT32_MAX)
    return fail(OSLO_E_UNSUPPORTED, "ngram_repeat_block: too many rows for one launch");
  if (rows == 0 || vocab == 0 || step - n + 2 <= 0) return OSLO_OK; // nothing can repeat yet
  if (!lprobs || !tokens)
    return fail(OSLO_E_BAD_ARG, "ngram_repeat_block: null tensor");
  ngram_repeat_block_kernel<<<dim3((unsigned)rows), dim3(kBlockThreads), 0,
                              static_cast<hipStream_t>(stream)>>>(
      lprobs, tokens, max_len, step, vocab, n);
  return check_launch("ngram_repeat_block");
}
