// Host-side check of the block -> tile numberings of the kernels: every tile
// (epilogues) and every row (softmax) is visited by exactly one workgroup, and
// a softmax workgroup's XCD (block % 8) matches the 4 KiB address class of the
// rows it takes. Runs on the CPU.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <utility>
#include <vector>

#include "elementwise.hpp"
#include "softmax.hpp"

using namespace oslo;

static int failures = 0;
#define CHECK(cond, ...)                                                      \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::printf("FAIL %s:%d: ", __FILE__, __LINE__);                        \
      std::printf(__VA_ARGS__);                                               \
      std::printf("\n");                                                      \
      ++failures;                                                             \
    }                                                                         \
  } while (0)

static void check_elementwise(int64_t rows, int64_t cols, int vec, int max_tx, int unroll) {
  const EwPlan p = plan_elementwise(rows, cols / vec, max_tx, unroll);
  CHECK(p.ok, "plan not ok");
  CHECK((int64_t)p.grid.x == p.row_blocks * p.col_tiles, "grid size");
  CHECK(p.row_blocks * p.rows_per_block >= rows && (int64_t)p.col_tiles * p.block.x * vec >= cols,
        "tiles do not cover the tensor");
  CHECK(p.block.x * p.block.y == (unsigned)kBlockThreads, "block shape");
  std::set<std::pair<int64_t, int64_t>> seen;
  for (int64_t b = 0; b < (int64_t)p.grid.x; ++b) {
    const EwTile t = ew_tile(p.col_tiles, b);
    CHECK(t.col_tile >= 0 && t.col_tile < p.col_tiles && t.row_block >= 0 &&
              t.row_block < p.row_blocks, "tile out of range");
    CHECK(seen.insert({t.row_block, t.col_tile}).second, "tile visited twice");
  }
  CHECK((int64_t)seen.size() == p.row_blocks * p.col_tiles, "tile missed");
  // the dbias workspace bound: one partial row per row block, at most ceil(rows/32)
  if (max_tx == kBwdMaxTx && unroll >= kBwdMinUnroll && rows >= 1)
    CHECK(p.row_blocks <= (rows + kBwdMinRowsPerBlock - 1) / kBwdMinRowsPerBlock,
          "more partial rows than the workspace holds");
}

static void check_rows(int64_t total_rows, int rows_per_block, int64_t row_bytes, bool paired) {
  const RowMap m = make_row_map(total_rows, rows_per_block, row_bytes, paired);
  std::vector<int> seen((size_t)total_rows, 0);
  const int64_t blocks = m.blocks_per_xcd * kXcds;
  for (int64_t b = 0; b < blocks; ++b)
    for (int w = 0; w < rows_per_block; ++w) {
      const int64_t r = mapped_row_of(m, rows_per_block, b, w);
      CHECK(r >= 0, "negative row");
      if (r >= total_rows) continue;
      ++seen[(size_t)r];
      // a unit of one 4 KiB chunk lies in the class of its XCD; a longer row
      // starts in class (XCD * chunks per row) % 8
      if ((int64_t)m.unit_rows * row_bytes == 4096)
        CHECK(((r * row_bytes) / 4096) % 8 == b % 8, "row %lld on XCD %lld", (long long)r,
              (long long)(b % 8));
      else if (row_bytes % 4096 == 0)
        CHECK(((r * row_bytes) / 4096) % 8 == (b % 8) * (row_bytes / 4096) % 8,
              "row %lld on XCD %lld", (long long)r, (long long)(b % 8));
    }
  for (int64_t r = 0; r < total_rows; ++r)
    if (seen[(size_t)r] != 1) {
      CHECK(false, "rows %lld x %lld B: row %lld visited %d times", (long long)total_rows,
            (long long)row_bytes, (long long)r, seen[(size_t)r]);
      break;
    }
}

int main() {
  // epilogue tiles: forward (64 threads wide, 2 rows per thread) and backward
  // (32 wide, 4 or 8 rows per thread)
  for (int k = 0; k < 3; ++k) {
    const int max_tx = k == 0 ? kFwdMaxTx : kBwdMaxTx;
    const int unroll = k == 0 ? kFwdUnroll : (k == 1 ? 4 : 8);
    check_elementwise(2048, 16384, 8, max_tx, unroll);
    check_elementwise(2048, 4096, 4, max_tx, unroll);
    check_elementwise(1000, 4096, 8, max_tx, unroll);
    check_elementwise(77, 768, 8, max_tx, unroll);
    check_elementwise(5, 24, 4, max_tx, unroll);
    check_elementwise(1, 8, 8, max_tx, unroll);
    check_elementwise(33, 1001, 1, max_tx, unroll); // element-wise path
  }
  // softmax rows: 16-bit and fp32 rows of several lengths, odd row counts
  for (int paired = 0; paired < 2; ++paired) {
    check_rows(8 * 2048, 4, 4096, paired);
    check_rows(3 * 2048 + 5, 4, 4096, paired);
    check_rows(2 * 1024, 4, 2048, paired);
    check_rows(1000, 4, 1024, paired);
    check_rows(7 * 64, 4, 128, paired);
    check_rows(4096, 2, 8192, paired);
    check_rows(555, 1, 16384, paired);
    check_rows(9, 4, 10, paired);
    check_rows(1, 4, 2, paired);
  }
  // a few hundred pseudo-random shapes on top of the hand-picked ones
  uint64_t state = 0x9E3779B97F4A7C15ull;
  auto next = [&](uint64_t n) {
    state = state * 6364136223846793005ull + 1442695040888963407ull;
    return (state >> 33) % n;
  };
  for (int i = 0; i < 300; ++i) {
    const int64_t rows = 1 + (int64_t)next(5000);
    const int vec = next(2) ? 8 : 4;
    const int64_t cols = vec * (1 + (int64_t)next(700));
    const int k = (int)next(3);
    check_elementwise(rows, cols, vec, k == 0 ? kFwdMaxTx : kBwdMaxTx,
                      k == 0 ? kFwdUnroll : (k == 1 ? 4 : 8));
    const int rpb = 1 << next(3);                        // 1, 2 or 4 rows per block
    const int64_t row_bytes = 16 * (1 + (int64_t)next(1024)); // up to 16 KiB
    check_rows(1 + (int64_t)next(20000), rpb, row_bytes, next(2) != 0);
  }
  if (failures == 0) std::printf("tile maps ok\n");
  return failures == 0 ? 0 : 1;
}
