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

// ---------------------------------------------------------------------------
// Sentence-span builders (BERT-style and block datasets): every document, a run
// of sentences docs[d] .. docs[d+1]-1 with sizes[] tokens each, is cut into
// samples of consecutive sentences whose length reaches a target; the samples
// of all epochs are then shuffled. Replaces build_mapping and
// build_blocks_mapping (oslo/fused_kernels/bindings/pybind_datasets.cpp
// :178-372 and :374-574). The reference walks the corpus twice inside one call
// (count, allocate, fill); here the caller asks for the row count first and
// then hands over the array, and one walker serves both builders and both
// passes.
// ---------------------------------------------------------------------------

#include <random>

namespace {

constexpr int32_t kLongSentence = 512; // a document with a longer sentence is skipped

struct Corpus {
  const int64_t *docs;
  int64_t num_docs; // docs has num_docs + 1 entries
  const int32_t *sizes;
  int64_t num_sentences;
};

struct CutRules {
  int32_t num_epochs;
  uint64_t max_samples;  // checked at the start of an epoch only, as in the reference
  int64_t min_in_sample; // sentences a document needs, and a sample needs before it may end early
  int64_t min_behind;    // sentences that must remain after a sample that ends early
  int64_t long_check_from; // documents with at least this many sentences are scanned for a long one
};

// Calls target(doc) for the length the next sample of `doc` aims at and
// emit(index, first, last_plus_1, doc, serial_in_epoch, target) for every
// sample; returns the number of samples, or -1 if docs / sizes do not describe
// each other.
template <typename Target, typename Emit>
int64_t cut_documents(const Corpus &c, const CutRules &r, Target &&target, Emit &&emit) {
  uint64_t count = 0;
  for (int32_t epoch = 0; epoch < r.num_epochs; ++epoch) {
    if (count >= r.max_samples) break;
    int64_t serial = 0;
    for (int64_t doc = 0; doc < c.num_docs; ++doc) {
      const int64_t first = c.docs[doc], last = c.docs[doc + 1];
      if (first < 0 || last < first || last > c.num_sentences) return -1;
      int64_t left = last - first;
      if (left < r.min_in_sample) continue;
      bool has_long = false;
      if (left >= r.long_check_from)
        for (int64_t s = first; s < last && !has_long; ++s) has_long = c.sizes[s] > kLongSentence;
      if (has_long) continue;
      int64_t start = first, in_sample = 0;
      int32_t length = 0;
      int32_t aim = target(doc);
      for (int64_t s = first; s < last; ++s) {
        length += c.sizes[s];
        ++in_sample;
        --left;
        const bool early = length >= aim && left >= r.min_behind && in_sample >= r.min_in_sample;
        if (early || left == 0) {
          emit(count, start, s + 1, doc, serial, aim);
          ++count;
          ++serial;
          start = s + 1;
          aim = target(doc);
          length = 0;
          in_sample = 0;
        }
      }
    }
  }
  return (int64_t)count;
}

// The reference's shuffle: from the last row down, swap with a row drawn by
// mt19937_64(seed + 1) modulo the rows not yet fixed.
template <typename Index, int W>
void shuffle_rows(Index *rows, int64_t n, int32_t seed) {
  std::mt19937_64 gen((uint64_t)((int64_t)seed + 1));
  for (int64_t i = n - 1; i > 0; --i) {
    const int64_t j = (int64_t)(gen() % (uint64_t)(i + 1));
    for (int w = 0; w < W; ++w) std::swap(rows[W * i + w], rows[W * j + w]);
  }
}

int check_corpus(const char *name, const int64_t *docs, int64_t docs_len, const int32_t *sizes,
                 int64_t sizes_len, int32_t num_epochs, int32_t max_seq_length, int32_t seed,
                 int index_bytes) {
  using namespace oslo;
  if (!docs || docs_len < 1 || (!sizes && sizes_len > 0) || sizes_len < 0)
    return fail(OSLO_E_BAD_ARG, "%s: docs needs at least one entry, sizes one per sentence", name);
  if (num_epochs <= 0 || max_seq_length <= 1 || seed <= 0)
    return fail(OSLO_E_BAD_ARG, "%s: needs num_epochs > 0, max_seq_length > 1, seed > 0", name);
  if (index_bytes != 4 && index_bytes != 8)
    return fail(OSLO_E_BAD_ARG, "%s: rows are uint32 or uint64 (index_bytes 4 or 8)", name);
  if (index_bytes == 4 && sizes_len > (int64_t)UINT32_MAX)
    return fail(OSLO_E_UNSUPPORTED, "%s: more than 2^32 sentences need 64-bit rows", name);
  return OSLO_OK;
}

} // namespace

extern "C" int64_t oslo_build_mapping(void *maps, int64_t rows, int index_bytes,
                                      const int64_t *docs, int64_t docs_len,
                                      const int32_t *sizes, int64_t sizes_len,
                                      int32_t num_epochs, uint64_t max_num_samples,
                                      int32_t max_seq_length, double short_seq_prob,
                                      int32_t seed, int32_t min_num_sent) {
  using namespace oslo;
  const char *name = "build_mapping";
  const int s = check_corpus(name, docs, docs_len, sizes, sizes_len, num_epochs, max_seq_length, seed,
                             index_bytes);
  if (s != OSLO_OK) return s;
  if (!(short_seq_prob >= 0.0 && short_seq_prob <= 1.0))
    return fail(OSLO_E_BAD_ARG, "%s: short_seq_prob outside [0, 1]", name);
  // one sample in `ratio` is short; the draw that decides it also gives its length
  const int32_t ratio = short_seq_prob > 0 ? (int32_t)round(1.0 / short_seq_prob) : 0;
  std::mt19937 gen((uint32_t)seed);
  auto target = [&](int64_t) -> int32_t {
    if (ratio == 0) return max_seq_length;
    const uint32_t draw = gen();
    return draw % (uint32_t)ratio == 0 ? (int32_t)(2 + draw % (uint32_t)(max_seq_length - 1)) : max_seq_length;
  };
  const Corpus corpus{docs, docs_len - 1, sizes, sizes_len};
  // a sample may end early only if more than one sentence stays behind; only
  // documents of two sentences or more are scanned for a long sentence
  const CutRules rules{num_epochs, max_num_samples, (int64_t)min_num_sent, 2, 2};
  int64_t n;
  if (maps == nullptr) {
    n = cut_documents(corpus, rules, target, [](uint64_t, int64_t, int64_t, int64_t, int64_t, int32_t) {});
  } else if (index_bytes == 4) {
    uint32_t *out = static_cast<uint32_t *>(maps);
    n = cut_documents(corpus, rules, target, [&](uint64_t i, int64_t a, int64_t b, int64_t, int64_t, int32_t aim) {
      if ((int64_t)i < rows) out[3 * i] = (uint32_t)a, out[3 * i + 1] = (uint32_t)b, out[3 * i + 2] = (uint32_t)aim;
    });
  } else {
    uint64_t *out = static_cast<uint64_t *>(maps);
    n = cut_documents(corpus, rules, target, [&](uint64_t i, int64_t a, int64_t b, int64_t, int64_t, int32_t aim) {
      if ((int64_t)i < rows) out[3 * i] = (uint64_t)a, out[3 * i + 1] = (uint64_t)b, out[3 * i + 2] = (uint64_t)aim;
    });
  }
  if (n < 0) return fail(OSLO_E_BAD_ARG, "%s: docs is not an ascending index into sizes", name);
  if (maps == nullptr) return n;
  if (n != rows)
    return fail(OSLO_E_BAD_ARG, "%s: maps has %lld rows, %lld are needed", name, (long long)rows, (long long)n);
  if (index_bytes == 4) shuffle_rows<uint32_t, 3>(static_cast<uint32_t *>(maps), n, seed);
  else shuffle_rows<uint64_t, 3>(static_cast<uint64_t *>(maps), n, seed);
  return n;
}

extern "C" int64_t oslo_build_blocks_mapping(void *maps, int64_t rows, int index_bytes,
                                             const int64_t *docs, int64_t docs_len,
                                             const int32_t *sizes, int64_t sizes_len,
                                             const int32_t *titles_sizes,
                                             int32_t num_epochs, uint64_t max_num_samples,
                                             int32_t max_seq_length, int32_t seed,
                                             int use_one_sent_blocks) {
  using namespace oslo;
  const char *name = "build_blocks_mapping";
  const int s = check_corpus(name, docs, docs_len, sizes, sizes_len, num_epochs, max_seq_length, seed,
                             index_bytes);
  if (s != OSLO_OK) return s;
  if (!titles_sizes && docs_len > 1) return fail(OSLO_E_BAD_ARG, "%s: null titles_sizes", name);
  // a block leaves room for its document's title
  auto target = [&](int64_t doc) -> int32_t { return max_seq_length - titles_sizes[doc]; };
  const Corpus corpus{docs, docs_len - 1, sizes, sizes_len};
  const int64_t least = use_one_sent_blocks ? 1 : 2;
  const CutRules rules{num_epochs, max_num_samples, least, least, least};
  int64_t n;
  if (maps == nullptr) {
    n = cut_documents(corpus, rules, target, [](uint64_t, int64_t, int64_t, int64_t, int64_t, int32_t) {});
  } else if (index_bytes == 4) {
    uint32_t *out = static_cast<uint32_t *>(maps);
    n = cut_documents(corpus, rules, target, [&](uint64_t i, int64_t a, int64_t b, int64_t doc, int64_t serial, int32_t) {
      if ((int64_t)i < rows)
        out[4 * i] = (uint32_t)a, out[4 * i + 1] = (uint32_t)b, out[4 * i + 2] = (uint32_t)doc, out[4 * i + 3] = (uint32_t)serial;
    });
  } else {
    uint64_t *out = static_cast<uint64_t *>(maps);
    n = cut_documents(corpus, rules, target, [&](uint64_t i, int64_t a, int64_t b, int64_t doc, int64_t serial, int32_t) {
      if ((int64_t)i < rows)
        out[4 * i] = (uint64_t)a, out[4 * i + 1] = (uint64_t)b, out[4 * i + 2] = (uint64_t)doc, out[4 * i + 3] = (uint64_t)serial;
    });
  }
  if (n < 0) return fail(OSLO_E_BAD_ARG, "%s: docs is not an ascending index into sizes", name);
  if (maps == nullptr) return n;
  if (n != rows)
    return fail(OSLO_E_BAD_ARG, "%s: maps has %lld rows, %lld are needed", name, (long long)rows, (long long)n);
  if (index_bytes == 4) shuffle_rows<uint32_t, 4>(static_cast<uint32_t *>(maps), n, seed);
  else shuffle_rows<uint64_t, 4>(static_cast<uint64_t *>(maps), n, seed);
  return n;
}
