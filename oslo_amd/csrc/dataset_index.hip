// Index builders of the data pipeline, host code: they run once when a dataset
// is opened, on arrays that live in host memory (numpy memory maps), and are
// sequential by nature, so they stay on the CPU, as in the reference
// (oslo/fused_kernels/bindings/pybind_datasets.cpp:35-160). Unlike the
// reference they check every index they follow and report a status instead of
// reading past the end of an array.

#include <vector>

#include "common.hpp"

extern "C" int64_t oslo_sample_idx_rows(int32_t seq_length, int32_t num_epochs,
                                        int64_t tokens_per_epoch) {
  if (seq_length <= 1 || num_epochs <= 0 || tokens_per_epoch <= 1) return -1;
  return ((int64_t)num_epochs * tokens_per_epoch - 1) / seq_length + 1;
}

// Walks the documents in doc_idx order as one token stream. Sample k covers
// seq_length + 1 tokens starting where sample k-1 ended minus one (neighbouring
// samples share a token: the last label of one is the first input of the next);
// row k of the result is (position in doc_idx, offset in that document) of its
// first token, row `rows-1` the end of the last sample.
extern "C" int oslo_build_sample_idx(int32_t *sample_idx, int64_t rows,
                                     const int32_t *sizes, int64_t num_docs,
                                     const int32_t *doc_idx, int64_t doc_idx_len,
                                     int32_t seq_length, int32_t num_epochs,
                                     int64_t tokens_per_epoch) {
  using namespace oslo;
  const char *name = "build_sample_idx";
  const int64_t want = oslo_sample_idx_rows(seq_length, num_epochs, tokens_per_epoch);
  if (want < 0)
    return fail(OSLO_E_BAD_ARG, "%s: needs seq_length > 1, num_epochs > 0, tokens_per_epoch > 1", name);
  if (rows != want)
    return fail(OSLO_E_BAD_ARG, "%s: sample_idx has %lld rows, %lld are needed", name,
                (long long)rows, (long long)want);
  if (!sample_idx || !sizes || !doc_idx || num_docs <= 0 || doc_idx_len <= 0)
    return fail(OSLO_E_BAD_ARG, "%s: null or empty array", name);

  int64_t at = 0;     // position in doc_idx
  int32_t offset = 0; // offset in that document
  sample_idx[0] = 0;
  sample_idx[1] = 0;
  for (int64_t k = 1; k < rows; ++k) {
    int64_t remaining = (int64_t)seq_length + 1;
    while (remaining != 0) {
      if (at >= doc_idx_len)
        return fail(OSLO_E_BAD_ARG, "%s: doc_idx holds too few tokens for sample %lld", name,
                    (long long)k);
      const int32_t doc = doc_idx[at];
      if (doc < 0 || doc >= num_docs)
        return fail(OSLO_E_BAD_ARG, "%s: doc_idx[%lld] = %d is outside [0, %lld)", name,
                    (long long)at, doc, (long long)num_docs);
      const int64_t left_in_doc = (int64_t)sizes[doc] - offset;
      remaining -= left_in_doc;
      if (remaining <= 0) { // the sample ends inside this document
        offset += (int32_t)(remaining + left_in_doc - 1);
        remaining = 0;
      } else {
        ++at;
        offset = 0;
      }
    }
    if (at > INT32_MAX)
      return fail(OSLO_E_UNSUPPORTED, "%s: more than 2^31 documents", name);
    sample_idx[2 * k] = (int32_t)at;
    sample_idx[2 * k + 1] = offset;
  }
  return OSLO_OK;
}

// Greedy blending: sample i goes to the dataset whose share so far lags its
// weight most, error_d = weights[d] * max(i, 1) - drawn_d, lowest d on ties;
// dataset_sample_index is the running count within that dataset. The full
// dataset number is stored (the reference narrows it to 8 bits first,
// pybind_datasets.cpp:73, which only matters beyond 256 datasets).
extern "C" int oslo_build_blending_indices(int32_t *dataset_index,
                                           int64_t *dataset_sample_index,
                                           const double *weights, int32_t num_datasets,
                                           int64_t size) {
  using namespace oslo;
  const char *name = "build_blending_indices";
  if (num_datasets <= 0 || size < 0)
    return fail(OSLO_E_BAD_ARG, "%s: needs num_datasets > 0 and size >= 0", name);
  if (size == 0) return OSLO_OK;
  if (!dataset_index || !dataset_sample_index || !weights)
    return fail(OSLO_E_BAD_ARG, "%s: null array", name);
  // counts kept as doubles (exact far beyond any dataset size): the error
  // term needs them as doubles in every step
  if (size >= ((int64_t)1 << 52))
    return fail(OSLO_E_UNSUPPORTED, "%s: size too large", name);
  std::vector<double> drawn((size_t)num_datasets, 0.0);
  const double *w = weights;
  double *n = drawn.data();
  for (int64_t i = 0; i < size; ++i) {
    const double at = i > 1 ? (double)i : 1.0;
    int32_t best = 0;
    double best_error = w[0] * at - n[0];
    for (int32_t d = 1; d < num_datasets; ++d) {
      const double error = w[d] * at - n[d];
      if (error > best_error) {
        best_error = error;
        best = d;
      }
    }
    dataset_index[i] = best;
    dataset_sample_index[i] = (int64_t)n[best];
    n[best] += 1.0;
  }
  return OSLO_OK;
}
