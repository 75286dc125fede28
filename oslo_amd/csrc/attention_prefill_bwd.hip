// Backward of the one-kernel causal prompt attention (attention_prefill.hip):
// dQ, dK and dV from Q, K, V, dO, the forward's output O and the log-sum-exp
// of every row, without the [S, S] matrices in memory (or, for the entry
// point with a tile store, with their tiles below the diagonal in a workspace
// between two passes of one call). With
//   P  = exp2(scale*log2e * Q K^T + pad*log2e - lse)      (the probabilities)
//   dP = dO V^T,   delta[q] = sum_d dO[q,d] * O[q,d]
//   dS = scale * P o (dP - delta)
// the gradients are dV = P^T dO, dQ = dS K, dK = dS^T Q. It replaces, for
// training, the backward of the three launches of the reference's fused
// attention (oslo/models/gptj/modeling_gptj.py:936-951: matmul, softmax
// kernel, matmul, differentiated by autograd), which keeps the probabilities
// and their gradient as [B, H, S, S] tensors.
//
// One kernel template serves every gradient. A block owns 128 positions (32
// per wave, one per lane of each half) and walks over the positions of the
// other kind in tiles: for dQ it owns queries and walks the keys up to the
// diagonal, for dK and dV it owns keys and walks the queries from the
// diagonal on. Both score-like products put the own position in the lane:
//   T1[other, own] = Other1 (A operand, LDS, rows = other) x Own1^T (B, fixed)
//   T2[other, own] = Other2 (A operand, LDS)               x Own2^T (B, fixed)
// (dQ: T1 = K Q^T = S^T, T2 = V dO^T = dP^T; dK/dV: T1 = Q K^T = S, T2 = dO V^T
// = dP), so P and dS come out in the accumulator layout of
// v_mfma_f32_32x32x16, which is also the B-operand layout of the accumulating
// products
//   Acc^T[d, own] += OtherT (A operand, LDS, rows = features) x X[other, own]
// (dQ^T += K^T dS^T; dK^T += Q^T dS; dV^T += dO^T P) once the contraction
// order is permuted the way the forward does it for V^T. Quantities indexed by
// the own position are per-lane scalars, those indexed by the other position
// are read per tile from LDS. Each block sums in a fixed order and no two
// blocks write the same element: the gradients are deterministic. The price is
// that scores are computed once per owner kind: dQ takes three matrix products
// per visible (query, key) tile and dK and dV together four (7 instead of 5)
// where one pass can hold both accumulators (heads of 64 and 128 features);
// at 256 features dK takes three and dV two in passes of their own (8).
//
// The kernel is built the way the forward is: tiles of 32 positions of the
// other kind loaded straight into LDS (four buffers per tensor), stored as they
// are in memory, read as A operands of the score-like products 16 bytes per
// lane and as A operands of the accumulating product through the transposing
// read (no transposed copy, no staging through registers); a tile's code is
// ordered by hand: the products of T1, those of T2, then the accumulating
// products of the previous tile with this tile's probabilities and score
// gradients worked out between them. One permutation of a row's 16-byte chunks
// serves both reads (f(row) below).

#include <algorithm>

#include "attention.hpp"

namespace oslo {
namespace {

// Largest head size whose dK and dV share a pass (a build switch for
// measurements: 256 compiles the combined pass there too, where it spills).
#ifndef OSLO_BWD_COMBINED_MAX_DIM
#define OSLO_BWD_COMBINED_MAX_DIM 128
#endif
// Waves of a block of the pass that reads the tile store (32 keys each), heads
// of 128 and 256 features (a build switch for measurements: 4 or 8).
#ifndef OSLO_STORED_WAVES
#define OSLO_STORED_WAVES 8
#endif

constexpr int kOwnPerBlock = 128;
constexpr float kLog2eB = 1.4426950408889634f;

// kRoleDKV: dK and dV in one pass (both own keys and walk queries: the scores
// and the probabilities are computed once for the two, 4 products per tile
// where the two passes have 5; it needs both accumulators in registers).
enum Role { kRoleDQ = 0, kRoleDK = 1, kRoleDV = 2, kRoleDKV = 3 };

// Blocks per CU the kernel is compiled for (a wave per SIMD each).
constexpr int bwd_blocks_per_cu(int D, int role) {
  if (role == kRoleDKV) return D == 256 ? 1 : D == 128 ? 1 : 2;
  return D == 256 ? 1 : D == 128 ? 2 : 3;
}

struct Strides3 {
  int64_t b, h, s; // element strides: batch, head, position
};

struct BwdArgs {
  const void *q, *k, *v, *dout;
  void *dq, *dk, *dv;
  const float *lse;   // [batch * heads, S], log2 units, from the forward
  const float *delta; // [batch * heads, S]
  const float *pad;   // [batch, S] additive, or null
  Strides3 sq, sk, sv, sdo, sdq, sdk, sdv;
  float scale, scale_log2e;
  int S, heads, batch_heads, head_groups, own_blocks, window;
  DropArgs drop; // attention dropout of the forward (the DROP variants)
  // The passes that exchange the probabilities through memory (below): the
  // tile store, the first head of the launch (a launch covers the heads
  // [bh0, bh0 + 8 * head_groups) below batch_heads; tiles of head bh0 come
  // first in the store), and the number of tiles a head has there.
  unsigned char *tiles;
  int bh0;
  int64_t head_tiles;
};

// The tile store. P (after dropout) and dS / scale of the 32 queries x 32 keys of
// query tile Qb and key tile Kb <= Qb of a head are 2 KiB each, one behind the
// other at tile index Qb (Qb + 1) / 2 + Kb, each as the pass that computes
// them holds it: [operand u][lane][8 values], the B operand u = 0, 1 of that
// pass's own accumulating product of lane (query, half h), whose value i is
// key 16 u + 8 (i / 4) + 4 h + i % 4: a store instruction of a wave writes 1 KiB
// in a row. The pass that consumes them gathers a tile into LDS as rows of
// [query][slot], slot 16 u + 8 h + i, and reads it through the transposing LDS
// read, key slot in the lane.
constexpr int kStoredTileBytes = 2048;                      // one of the two
constexpr int kStoredPairBytes = 2 * kStoredTileBytes;      // P, then dS
__host__ __device__ constexpr int64_t stored_head_tiles(int64_t own_blocks) {
  const int64_t n = own_blocks * (kOwnPerBlock / 32);
  return n * (n + 1) / 2;
}

constexpr int kSchedTile = 32;
constexpr int kSchedBuffers = 4;

template <typename T, int D, int ROLE>
constexpr unsigned sched_lds_bytes() {
  return 2u * kSchedBuffers * kSchedTile * D * sizeof(T) + kSchedBuffers * 2u * 256u * sizeof(float) +
         kWavesPerBlock * 32u * sizeof(uint32_t);
}

template <typename T, int D, int ROLE, bool HAS_PAD, bool HAS_WINDOW, bool DROP, bool STORE = false>
__global__ __launch_bounds__(kBlockThreads, bwd_blocks_per_cu(D, ROLE)) void attention_bwd_kernel(
    const BwdArgs a) {
  static_assert(ROLE >= kRoleDQ && ROLE <= kRoleDKV, "unknown pass");
  static_assert(!STORE || ROLE == kRoleDQ, "the pass that owns queries writes the tile store");
  using Op = MatrixOp<T>;
  using Frag = typename Op::Frag;
  constexpr bool kKeysOwn = ROLE != kRoleDQ;
  constexpr bool kNeedT2 = ROLE != kRoleDV;
  constexpr bool kTwoAcc = ROLE == kRoleDKV; // acc = dK^T, acc2 = dV^T
  constexpr bool kKeepP = kTwoAcc || STORE;  // the probabilities are wanted beside dS
  constexpr int kChunks = D / 8;   // 16-byte chunks of a position
  constexpr int kSteps = D / 16;   // contraction steps over the features
  constexpr int kBlocksD = D / 32; // 32-row blocks of the accumulator
  constexpr int kLoadsN = kSchedTile * kChunks / kBlockThreads; // loads per thread and tile of a tensor
  constexpr int kTile = kSchedTile * D; // elements
  constexpr int kRowBytes = D * (int)sizeof(T);
  constexpr int kSwizzle = kChunks >= 16 ? 15 : 7;
  constexpr int kRowSlots = 256; // floats of a tile's per-position values: the first 32 count

  extern __shared__ __align__(1024) unsigned char lds_raw[];
  T *const o1_lds = reinterpret_cast<T *>(lds_raw);            // [4][position][chunk ^ f(position)][8]
  T *const o2_lds = o1_lds + kSchedBuffers * kTile;            // the same for the second tensor
  // per-position values of a tile: queries: log-sum-exp and delta; keys: the padding mask's value
  float *const rows_lds = reinterpret_cast<float *>(o2_lds + kSchedBuffers * kTile); // [4][2][256]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;
  uint32_t *const keep_lds =
      reinterpret_cast<uint32_t *>(rows_lds + kSchedBuffers * 2 * kRowSlots) + 32 * wave; // a wave's keep bits of a tile

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int bh = a.bh0 + xcd + 8 * (slot % a.head_groups);
  const int idx = slot / a.head_groups;
  const int own_block = kKeysOwn ? idx : a.own_blocks - 1 - idx;
  if (bh >= a.batch_heads) return; // the whole block
  const int b = bh / a.heads;
  const int hd = bh - b * a.heads;
  const int S = a.S;
  const int own0 = own_block * kOwnPerBlock;
  const int wave_own0 = own0 + 32 * wave;
  const int own = wave_own0 + col;

  auto slice = [&](const void *p, const Strides3 &st) __attribute__((always_inline)) {
    return static_cast<const T *>(p) + b * st.b + hd * st.h;
  };
  auto slice_bytes = [&](const Strides3 &st) __attribute__((always_inline)) {
    return (uint32_t)(((int64_t)(S - 1) * st.s + D) * sizeof(T));
  };
  const Strides3 &st_own1 = kKeysOwn ? a.sk : a.sq;
  const Strides3 &st_own2 = kKeysOwn ? a.sv : a.sdo;
  const Strides3 &st_o1 = kKeysOwn ? a.sq : a.sk;
  const Strides3 &st_o2 = kKeysOwn ? a.sdo : a.sv;
  const T *own1_p = slice(kKeysOwn ? a.k : a.q, st_own1);
  const T *own2_p = slice(kKeysOwn ? a.v : a.dout, st_own2);
  const T *o1_p = slice(kKeysOwn ? a.q : a.k, st_o1);
  const T *o2_p = slice(kKeysOwn ? a.dout : a.v, st_o2);
  const uint32_t o1_row = (uint32_t)st_o1.s * sizeof(T);
  const uint32_t o2_row = (uint32_t)st_o2.s * sizeof(T);

  // B operands of the own positions, in registers for the whole kernel
  Frag own1[kSteps], own2[kNeedT2 ? kSteps : 1];
  {
    const BufRsrc rs1 = make_rsrc(own1_p, slice_bytes(st_own1));
    const uint32_t row1 = (uint32_t)st_own1.s * sizeof(T);
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
      own1[s] = __builtin_bit_cast(Frag, __builtin_amdgcn_raw_buffer_load_b128(
                                             rs1, (uint32_t)own * row1 + (uint32_t)(16 * s + 8 * half) * sizeof(T), 0, 0));
    if constexpr (kNeedT2) {
      const BufRsrc rs2 = make_rsrc(own2_p, slice_bytes(st_own2));
      const uint32_t row2 = (uint32_t)st_own2.s * sizeof(T);
#pragma unroll
      for (int s = 0; s < kSteps; ++s)
        own2[s] = __builtin_bit_cast(Frag, __builtin_amdgcn_raw_buffer_load_b128(
                                               rs2, (uint32_t)own * row2 + (uint32_t)(16 * s + 8 * half) * sizeof(T), 0, 0));
    }
  }
  const int64_t stat_row = (int64_t)bh * S;
  float own_lse = 0.f, own_delta = 0.f, own_pad = 0.f; // (the padding value, floored)
  if constexpr (!kKeysOwn) {
    if (own < S) {
      own_lse = a.lse[stat_row + own];
      own_delta = a.delta[stat_row + own];
    }
  } else if constexpr (HAS_PAD) {
    if (own < S) own_pad = fmaxf(a.pad[(int64_t)b * S + own], kMaskFloor);
  }

  // Tiles [first_tile, tiles) of the other kind this block walks. Those before
  // masked_until and those from plain_until on may hold pairs that are not
  // visible; the tiles between them are visible in full to every own position.
  // Own queries: the causal boundary crosses the last four tiles, the edges of
  // the queries' windows the first ones. Own keys: the boundary crosses the
  // first four; a window ends the walk at the last query that sees the block's
  // last key, and its edge crosses the tiles from the first query that no
  // longer sees the block's first key on.
  const int window = HAS_WINDOW ? a.window : 0;
  int first_tile, tiles, masked_until, plain_until;
  if constexpr (!kKeysOwn) {
    const int last_key = (own0 + kOwnPerBlock < S ? own0 + kOwnPerBlock : S) - 1;
    tiles = last_key / kSchedTile + 1;
    first_tile = HAS_WINDOW && own0 - window + 1 > 0 ? (own0 - window + 1) / kSchedTile : 0;
    masked_until = HAS_WINDOW && own0 + kOwnPerBlock - window > 0
                       ? (own0 + kOwnPerBlock - window + kSchedTile - 1) / kSchedTile
                       : 0;
    plain_until = own0 / kSchedTile;
  } else {
    first_tile = own0 / kSchedTile;
    int last_query = S - 1;
    if (HAS_WINDOW && own0 + kOwnPerBlock - 1 + window - 1 < last_query) last_query = own0 + kOwnPerBlock - 1 + window - 1;
    tiles = last_query / kSchedTile + 1;
    masked_until = first_tile + kOwnPerBlock / kSchedTile;
    plain_until = HAS_WINDOW ? (own0 + window) / kSchedTile : tiles;
  }
  if (masked_until > tiles) masked_until = tiles;
  if (plain_until > tiles) plain_until = tiles;

  // The permutation of a row's chunks: chunk c of row r lies at c ^ f(r). The
  // 16 lanes that read 16 consecutive rows at one chunk (natural operands) must
  // get 16 values of f, the 16 lanes of a transposing read (rows 4c .. 4c + 3,
  // two chunks, both halves of each) four values that differ above bit 0: f
  // puts the row's two low bits at bits 1 and 2, bit 2 at bit 0, bit 3 stays.
  // (At 256 features, where the registers for eight lane offsets are there, f is
  // 4 (r % 4) + r / 4 % 4 instead: the four rows of a transposing read then use four
  // different quarters of the banks for both 16-feature halves at once; with the
  // f above two of the four share theirs, two more cycles for every such read.)
  constexpr bool kQuads = D == 256;
  auto f_of = [](int r) __attribute__((always_inline)) {
    if (kQuads) return ((r & 3) << 2) | ((r >> 2) & 3);
    return (((r & 3) << 1) | ((r >> 2) & 1) | (r & 8)) & kSwizzle;
  };
  uint32_t o1_off[kLoadsN], o2_off[kLoadsN];
#pragma unroll
  for (int j = 0; j < kLoadsN; ++j) {
    const int sigma = (4 * j + wave) * kWave + lane;
    const int row = sigma / kChunks, at = sigma % kChunks;
    o1_off[j] = (uint32_t)row * o1_row + (uint32_t)(at ^ f_of(row)) * 16u;
    o2_off[j] = (uint32_t)row * o2_row + (uint32_t)(at ^ f_of(row)) * 16u;
  }
  const uint32_t row_off = tid < kSchedTile ? (uint32_t)tid * 4u : 0x80000000u;
  TileStream o1_src, o2_src, lse_src, delta_src; // the next tile to load (tile t + 2 while tile t is computed)
  o1_src.start(o1_p, slice_bytes(st_o1), o1_row, kSchedTile, first_tile, tiles);
  o2_src.start(o2_p, slice_bytes(st_o2), o2_row, kSchedTile, first_tile, tiles);
  if constexpr (kKeysOwn) {
    lse_src.start(a.lse + stat_row, (uint32_t)S * 4u, 4u, kSchedTile, first_tile, tiles);
    if constexpr (kNeedT2) delta_src.start(a.delta + stat_row, (uint32_t)S * 4u, 4u, kSchedTile, first_tile, tiles);
  } else if constexpr (HAS_PAD) { // the keys' mask values take the first of the two rows
    lse_src.start(a.pad + (int64_t)b * S, (uint32_t)S * 4u, 4u, kSchedTile, first_tile, tiles);
  }
  constexpr int kRowItems = kKeysOwn ? (kNeedT2 ? 2 : 1) : HAS_PAD ? 1 : 0; // (the dV pass needs no delta)
  constexpr int kItems = 2 * kLoadsN + kRowItems;
  constexpr int kLoadsPerTile = kItems;
  int t = first_tile;
  // buffer of tile t + d
  auto buffer_of = [&](int d) __attribute__((always_inline)) { return (t + d) & (kSchedBuffers - 1); };
  // item `it` of the staging of tile t: the loads of tile t + 2
  auto stage_item = [&](int it) __attribute__((always_inline)) {
    const int buf = buffer_of(2);
    if (it < kLoadsN) {
      lds_load_b128(o1_src.descriptor(), o1_lds + buf * kTile + (4 * it + wave) * (kWave * 8), o1_off[it]);
      if (it == kLoadsN - 1) o1_src.advance();
      return;
    }
    it -= kLoadsN;
    if (it < kLoadsN) {
      lds_load_b128(o2_src.descriptor(), o2_lds + buf * kTile + (4 * it + wave) * (kWave * 8), o2_off[it]);
      if (it == kLoadsN - 1) o2_src.advance();
      return;
    }
    it -= kLoadsN;
    if constexpr (kRowItems > 0) {
      // every wave loads 64 values into a quarter of its own; the first 32 of the first wave's count
      float *dst = rows_lds + (buf * 2 + it) * kRowSlots + wave * kWave;
      if (it == 0) {
        lds_load_b32(lse_src.descriptor(), dst, row_off);
        lse_src.advance();
      } else {
        lds_load_b32(delta_src.descriptor(), dst, row_off);
        delta_src.advance();
      }
    }
  };

  // natural operand s of the tile in `base`: lane (row, half) takes chunk 2 s + half of its row
  const uint32_t nat_lane = (uint32_t)col * kRowBytes + (uint32_t)((half ^ f_of(col)) << 4);
  auto read_natural = [&](const T *base, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const Frag *>(reinterpret_cast<const char *>(base) + (nat_lane ^ (uint32_t)(s << 5)));
  };
  // Transposed operand n (16 positions u into block i of 32 features): of 16
  // lanes, lane j points at 8 bytes (4 features) of position j / 4; lane i gets
  // back feature i of the four positions. Two reads make an operand: slots 0..3
  // are positions 16u + 4h + 0..3, slots 4..7 positions 16u + 8 + 4h + 0..3 (h
  // the lane's half of the wave): the rows the accumulator layout gives a lane.
  typedef short Short4 __attribute__((ext_vector_type(4)));
  uint32_t tr_lane[kQuads ? 8 : 2]; // for even and odd blocks of 32 features (kQuads: per block % 4 and read of the two)
  {
    const int j = lane & 15, group = lane >> 4;
    const int kq = j >> 2, fb = j & 3, hh = group >> 1, fg = group & 1;
    if constexpr (kQuads) {
      // row 16 u + 8 jj + 4 hh + kq, chunk 4 i + w of it, w = 2 fg + fb / 2: f is 4 kq + 2 jj + hh, so the chunk lies
      // at 16 (i / 4) + 4 (i % 4 ^ kq) + (w ^ hh ^ 2 jj): the lane's part, with the read's i % 4 and jj folded in
      const uint32_t own_part = (uint32_t)(4 * hh + kq) * kRowBytes + 64u * (uint32_t)kq +
                                16u * (uint32_t)((2 * fg + (fb >> 1)) ^ hh) + 8u * (uint32_t)(fb & 1);
#pragma unroll
      for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) tr_lane[2 * v + jj] = own_part ^ (uint32_t)(64 * v + 32 * jj);
    } else {
      // f of the lane's rows 16u + 8jj + 4hh + kq is 2 kq | hh | 8 jj; the part below bit 3:
      const int flow = ((kq << 1) | hh) & kSwizzle;
      const int x = (2 * fg + (fb >> 1)) ^ (flow & 3);
      const int flip = flow >> 2; // its bit 2 swaps neighbouring blocks of four chunks
      const uint32_t base = (uint32_t)(4 * hh + kq) * kRowBytes + (uint32_t)x * 16u + (uint32_t)(fb & 1) * 8u;
      tr_lane[0] = base + 64u * (uint32_t)flip;
      tr_lane[1] = base + 64u * (uint32_t)(1 ^ flip);
    }
  }
  auto read_transposed = [&](const T *base, int n) __attribute__((always_inline)) {
    const int u = n / kBlocksD, i = n % kBlocksD;
    Short4 part[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const char *at;
      if constexpr (kQuads) {
        at = reinterpret_cast<const char *>(base) + tr_lane[2 * (i & 3) + jj] + 256 * (i >> 2) + (16 * u + 8 * jj) * kRowBytes;
      } else {
        // rows with bit 3 set (jj = 1) have bit 3 of f set: blocks two apart swap (head sizes of 16 chunks and more)
        const int ii = kSwizzle >= 8 ? i ^ (2 * jj) : i;
        at = reinterpret_cast<const char *>(base) + tr_lane[ii & 1] + 64 * (ii & ~1) + (16 * u + 8 * jj) * kRowBytes;
      }
      part[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) Short4 *)(at));
    }
    return __builtin_bit_cast(Frag, __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7));
  };

  f32x16 acc[kBlocksD], acc2[kTwoAcc ? kBlocksD : 1];
#pragma unroll
  for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  if constexpr (kTwoAcc) {
#pragma unroll
    for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[i][r] = 0.f;
  }
  // what the accumulating products take of the last tile computed: xf = P (dV
  // pass) or P o (dP - delta); in the combined pass xp = P as well
  Frag xf[2], xp[2];

  // which tensor the accumulating product reads transposed: K (dQ), Q (dK), dO (dV)
  auto transposed_tile = [&](int d) __attribute__((always_inline)) {
    return (ROLE == kRoleDV ? o2_lds : o1_lds) + buffer_of(d) * kTile;
  };
  auto transposed_tile2 = [&](int d) __attribute__((always_inline)) { return o2_lds + buffer_of(d) * kTile; }; // dO (combined pass)
  // slice `n` of `slices` of a tile's elementwise work: P = exp2(scale*log2e *
  // T1 + pad*log2e - lse), X = P (dV) or P (T2 - delta) (the scale goes onto
  // the result). With attention dropout the forward multiplied V with
  // keep * P / (1-p): the P product takes the kept probabilities (1/(1-p) goes
  // onto dV at the end), and the gradient of the dropped-out probabilities is
  // keep * dP / (1-p). The keep bits of the tile are drawn in the first slice.
  u32x4 keep_words[4];
  uint32_t keep_bits = 0;
  // The tile's per-position values of register r (row 8 (r / 4) + 4 half + r % 4
  // of the tile) are read kAhead registers before they are used: read where
  // they are used, every slice of the elementwise work would wait for the LDS.
  // (Not at head_dim 64, where the registers for it are not there.)
  constexpr bool kRowValues = kKeysOwn || HAS_PAD;
  constexpr int kAhead = D >= 128 ? 4 : 0;
  float row_a[16], row_b[16];
  auto read_row_values = [&](int r) __attribute__((always_inline)) {
    if constexpr (kRowValues) {
      const float *rows = rows_lds + buffer_of(0) * 2 * kRowSlots + 8 * (r >> 2) + 4 * half + (r & 3);
      row_a[r] = rows[0];
      if constexpr (kKeysOwn && kNeedT2) row_b[r] = rows[kRowSlots];
    }
  };
  auto elementwise = [&]<bool MASKED>(f32x16 &t1, f32x16 &t2, int n, int slices, Frag (&x)[2], Frag (&x2)[2])
                         __attribute__((always_inline)) {
    if constexpr (DROP) {
      if (n == 0) {
        const int other0 = t * kSchedTile;
        stage_keep_bits(keep_lds, a.drop, bh, S, kKeysOwn ? other0 : wave_own0, kKeysOwn ? wave_own0 : other0, lane);
        if constexpr (kKeysOwn) {
#pragma unroll
          for (int j = 0; j < 4; ++j) keep_words[j] = keep_words_key_lane(keep_lds, j, half);
        } else {
          keep_bits = keep_word_query_lane(keep_lds, col) >> (4 * half);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (r * slices / 16 != n) continue;
      const int rr = 8 * (r >> 2) + 4 * half + (r & 3); // the register's row of the tile
      if (r + kAhead < 16) read_row_values(r + kAhead);
      float shift, delta_r = own_delta;
      if constexpr (kKeysOwn) {
        // (the same fused multiply-add as in the pass that owns queries: every pass sees the same P, bit for bit)
        shift = HAS_PAD ? __builtin_fmaf(own_pad, kLog2eB, -row_a[r]) : -row_a[r];
        if constexpr (kNeedT2) delta_r = row_b[r];
      } else if constexpr (HAS_PAD) {
        shift = __builtin_fmaf(fmaxf(row_a[r], kMaskFloor), kLog2eB, -own_lse);
      } else {
        shift = -own_lse;
      }
      float p = __builtin_amdgcn_exp2f(__builtin_fmaf(t1[r], a.scale_log2e, shift));
      if constexpr (MASKED) {
        const int other = t * kSchedTile + rr;
        const bool visible = kKeysOwn ? own <= other && (!HAS_WINDOW || other - window < own)
                                      : other <= own && (!HAS_WINDOW || other > own - window);
        p = visible ? p : 0.f;
      }
      float grad = t2[r];
      float kept = p; // the probability the values met (the combined pass keeps it beside dS)
      if constexpr (DROP) {
        const bool keep = kKeysOwn ? ((keep_words[r >> 2][r & 3] >> col) & 1u) != 0
                                   : ((keep_bits >> (8 * (r >> 2) + (r & 3))) & 1u) != 0;
        grad = keep ? grad * a.drop.keep_scale : 0.f;
        if constexpr (!kNeedT2) p = keep ? p : 0.f;
        if constexpr (kKeepP) kept = keep ? p : 0.f;
      }
      if constexpr (kNeedT2) p *= grad - delta_r;
      t1[r] = p;
      asm volatile("" : "+v"(t1[r])); // (keeps the computation in its slice)
      if constexpr (kKeepP) {
        t2[r] = kept;
        asm volatile("" : "+v"(t2[r]));
      }
    }
    if (n == slices - 1) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 8; ++i) x[u][i] = static_cast<T>(t1[8 * u + i]);
      if constexpr (kKeepP) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 8; ++i) x2[u][i] = static_cast<T>(t2[8 * u + i]);
      }
    }
  };
  // The wave's tiles of the store: query tile own0 / 32 + wave, key tile t. A
  // tile that lies wholly above the diagonal has no place there (and holds zeros).
  unsigned char *tile_row = nullptr;
  const int own_tile = own0 / 32 + wave;
  if constexpr (STORE)
    tile_row = a.tiles + ((int64_t)(bh - a.bh0) * a.head_tiles + (int64_t)own_tile * (own_tile + 1) / 2) * kStoredPairBytes +
               lane * 16;
  auto store_tiles = [&](const Frag (&ds)[2], const Frag (&pk)[2]) __attribute__((always_inline)) {
    if constexpr (STORE) {
      if (t <= own_tile) {
        unsigned char *at = tile_row + (int64_t)t * kStoredPairBytes;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          // (written once and read once by the next pass: non-temporal, so that K and V stay in the caches)
          __builtin_nontemporal_store(pk[u], reinterpret_cast<Frag *>(at + 1024 * u));
          __builtin_nontemporal_store(ds[u], reinterpret_cast<Frag *>(at + kStoredTileBytes + 1024 * u));
        }
      }
    }
  };
  constexpr int kStoresPerTile = STORE ? 4 : 0;

  // prologue: the first two tiles on their way
#pragma unroll
  for (int rep = 0; rep < 2; ++rep) {
    t = first_tile - 2 + rep; // (an item loads tile t + 2)
#pragma unroll
    for (int it = 0; it < kItems; ++it) stage_item(it);
  }
  t = first_tile;

  // the block's first tile: nothing to accumulate yet; plain order
  {
    wait_vm<kLoadsPerTile>();
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kItems; ++it) stage_item(it);
    f32x16 t1, t2;
#pragma unroll
    for (int r = 0; r < 16; ++r) t1[r] = t2[r] = 0.f;
    const T *b1 = o1_lds + buffer_of(0) * kTile, *b2 = o2_lds + buffer_of(0) * kTile;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) t1 = Op::run(read_natural(b1, s), own1[s], t1);
    if constexpr (kNeedT2) {
#pragma unroll
      for (int s = 0; s < kSteps; ++s) t2 = Op::run(read_natural(b2, s), own2[s], t2);
    }
#pragma unroll
    for (int r = 0; r < kAhead; ++r) read_row_values(r);
    elementwise.template operator()<true>(t1, t2, 0, 1, xf, xp);
    store_tiles(xf, xp);
    ++t;
  }

  // A tile as one straight run of code between fences: the products of T1 with
  // the next tiles' loads between them, those of T2, then the accumulating
  // products of the previous tile with this tile's elementwise work between
  // them. Operands are read from LDS kRing products ahead.
  auto scheduled_tile = [&]<bool MASKED>() __attribute__((always_inline)) {
    constexpr int kRing = 4;
    constexpr int kProducts = 2 * kBlocksD;
    // the combined pass: the products of dV^T (dO^T x P) first, then those of dK^T (Q^T x dS)
    constexpr int kAccProducts = (kTwoAcc ? 2 : 1) * kProducts;
    constexpr int kOperands = kSteps + (kNeedT2 ? kSteps : 0) + kAccProducts;
    constexpr int kPerStep = (kItems + kSteps - 1) / kSteps;
    const T *b1 = o1_lds + buffer_of(0) * kTile, *b2 = o2_lds + buffer_of(0) * kTile;
    const T *bt = transposed_tile(-1);
    const T *bt2 = transposed_tile2(-1);
    Frag ring[kRing];
    auto read_operand = [&](int p) __attribute__((always_inline)) {
      if (p < kSteps) ring[p % kRing] = read_natural(b1, p);
      else if (kNeedT2 && p < 2 * kSteps) ring[p % kRing] = read_natural(b2, p - kSteps);
      else {
        const int q = p - (kNeedT2 ? 2 : 1) * kSteps;
        if (kTwoAcc && q < kProducts) ring[p % kRing] = read_transposed(bt2, q);
        else ring[p % kRing] = read_transposed(bt, q - (kTwoAcc ? kProducts : 0));
      }
    };
#pragma unroll
    for (int p = 0; p < kRing; ++p) read_operand(p);
    __builtin_amdgcn_sched_barrier(0);
    f32x16 t1, t2;
#pragma unroll
    for (int r = 0; r < 16; ++r) t1[r] = t2[r] = 0.f;
    int p = 0;
#pragma unroll
    for (int s = 0; s < kSteps; ++s, ++p) {
      t1 = Op::run(ring[p % kRing], own1[s], t1);
      if (p + kRing < kOperands) read_operand(p + kRing);
#pragma unroll
      for (int it = s * kPerStep; it < (s + 1) * kPerStep && it < kItems; ++it) stage_item(it);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (kNeedT2) {
#pragma unroll
      for (int s = 0; s < kSteps; ++s, ++p) {
        t2 = Op::run(ring[p % kRing], own2[s], t2);
        if (p + kRing < kOperands) read_operand(p + kRing);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    Frag xn[2], xpn[2];
#pragma unroll
    for (int r = 0; r < kAhead; ++r) read_row_values(r);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kAccProducts; ++n, ++p) {
      if (kTwoAcc && n < kProducts) {
        acc2[n % kBlocksD] = Op::run(ring[p % kRing], xp[n / kBlocksD], acc2[n % kBlocksD]);
      } else {
        const int m = n - (kTwoAcc ? kProducts : 0);
        acc[m % kBlocksD] = Op::run(ring[p % kRing], xf[m / kBlocksD], acc[m % kBlocksD]);
      }
      if (p + kRing < kOperands) read_operand(p + kRing);
      elementwise.template operator()<MASKED>(t1, t2, n, kAccProducts, xn, xpn);
      __builtin_amdgcn_sched_barrier(0);
    }
    xf[0] = xn[0], xf[1] = xn[1];
    if constexpr (kKeepP) xp[0] = xpn[0], xp[1] = xpn[1];
    store_tiles(xf, xp);
  };
  // each kind of tile in a loop of its own
  auto run_tiles = [&]<bool MASKED>(int end) __attribute__((always_inline)) {
    for (; t < end; ++t) {
      // (Vector-memory operations are counted in order. Behind the loads of tile t
      // come the stores of tile t - 2, the loads of tile t + 1 and the stores of
      // tile t - 1: none of them is waited for here. A store into the tile store
      // takes long to be acknowledged; waited for a tile after it was issued, the
      // stores cost this pass 100 us of 600.)
      if (!STORE) wait_vm<kLoadsPerTile>();
      else if (t - 1 > own_tile) wait_vm<kLoadsPerTile>(); // (a wave past its diagonal stored nothing)
      else if (t - 2 < first_tile) wait_vm<kLoadsPerTile + kStoresPerTile>(); // (the block's second tile)
      else wait_vm<kLoadsPerTile + 2 * kStoresPerTile>();
      __syncthreads(); // tile t is in LDS; the buffer written next (tile t - 2's) has been read
      scheduled_tile.template operator()<MASKED>();
    }
  };
  if constexpr (kKeysOwn || HAS_WINDOW) run_tiles.template operator()<true>(masked_until);
  run_tiles.template operator()<false>(plain_until);
  if constexpr (!kKeysOwn || HAS_WINDOW) run_tiles.template operator()<true>(tiles);
  // the last tile's accumulating products
  wait_vm<0>(); // (nothing may still be on its way into LDS when the block ends)
  __syncthreads();
  {
    const T *bt = transposed_tile(-1);
    if constexpr (kTwoAcc) {
      const T *bt2 = transposed_tile2(-1);
#pragma unroll
      for (int n = 0; n < 2 * kBlocksD; ++n)
        acc2[n % kBlocksD] = Op::run(read_transposed(bt2, n), xp[n / kBlocksD], acc2[n % kBlocksD]);
    }
#pragma unroll
    for (int n = 0; n < 2 * kBlocksD; ++n)
      acc[n % kBlocksD] = Op::run(read_transposed(bt, n), xf[n / kBlocksD], acc[n % kBlocksD]);
  }

  if (own >= S) return;
  typedef T Out4 __attribute__((ext_vector_type(4)));
  auto store = [&](const f32x16 (&sums)[kBlocksD], void *out_base, const Strides3 &st_out, float factor)
                   __attribute__((always_inline)) {
    T *op = static_cast<T *>(out_base) + b * st_out.b + hd * st_out.h + (int64_t)own * st_out.s;
#pragma unroll
    for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Out4 w;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) w[tt] = static_cast<T>(sums[i][4 * j + tt] * factor);
        *reinterpret_cast<Out4 *>(op + 32 * i + 8 * j + 4 * half) = w;
      }
  };
  const float p_factor = DROP ? a.drop.keep_scale : 1.0f; // the 1/(1-p) of the kept probabilities
  if constexpr (ROLE == kRoleDQ) store(acc, a.dq, a.sdq, a.scale);
  else if constexpr (ROLE == kRoleDK) store(acc, a.dk, a.sdk, a.scale);
  else if constexpr (ROLE == kRoleDV) store(acc, a.dv, a.sdv, p_factor);
  else {
    store(acc, a.dk, a.sdk, a.scale);
    store(acc2, a.dv, a.sdv, p_factor);
  }
}

template <typename T, int D, int ROLE, bool STORE = false>
int launch_role(const BwdArgs &a, hipStream_t stream) {
  const dim3 grid((unsigned)(8 * a.head_groups * a.own_blocks));
  constexpr unsigned kLds = sched_lds_bytes<T, D, ROLE>();
  auto go = [&]<bool HAS_PAD, bool DROP>() -> int {
    auto *kernel = a.window > 0 ? attention_bwd_kernel<T, D, ROLE, HAS_PAD, true, DROP, STORE>
                                : attention_bwd_kernel<T, D, ROLE, HAS_PAD, false, DROP, STORE>;
    if (kLds > 64u * 1024u) {
      const int s = raise_lds_limit(reinterpret_cast<const void *>(kernel), kLds, "oslo_attention_prefill_bwd");
      if (s != OSLO_OK) return s;
    }
    kernel<<<grid, dim3(kBlockThreads), kLds, stream>>>(a);
    return check_launch("attention_prefill_bwd");
  };
  if (a.pad != nullptr) {
    if (a.drop.drop) return go.template operator()<true, true>();
    return go.template operator()<true, false>();
  }
  if (a.drop.drop) return go.template operator()<false, true>();
  return go.template operator()<false, false>();
}

// dK and dV from the tile store: dK^T += Q^T dS and dV^T += dO^T P over the query
// tiles from the diagonal on, nothing else: no scores, no exponentials, no
// mask, no dropout (all of it is in the stored tiles). A block owns 32 keys per
// wave (256 with eight waves) and one of the two gradients (even blocks dK, odd
// blocks dV); a pair of waves has 64 keys and each wave of the pair half of the
// features, so a wave holds one accumulator of 64 keys x D / 2 features (D / 2
// registers), no fixed operands, and uses every transposed operand of Q (or
// dO) it reads from LDS for two products. The tiles of Q (or dO) go through LDS
// as in the other passes (three buffers: tile t is read while t + 1 and t + 2
// are on their way), shared by the block; every wave loads one 2 KiB tile of dS
// (or P) beside them, which it and its partner read back transposed, key slot
// in the lane: lane c holds the key at slot c of the store's rows, key c with
// bits 2 and 3 swapped. What this pass waits for is its loads (with none of
// them issued it takes 0.22 ms instead of 0.40 at [8,16,2048,256], without its
// products still 0.39): the more keys share a tile of Q, the fewer bytes per
// product, hence eight waves.
// Tiles of a tensor in LDS: the one that is read and those on their way. (The
// pass is bound by its loads, but not by their latency: with four or five
// buffers at 256 features, 128 and 160 KiB, it takes the same time as with three.
// Nor does it help to issue the loads of half of the waves one operand later
// than those of the others: 430 against 390 us.)
#ifndef OSLO_STORED_BUFFERS
#define OSLO_STORED_BUFFERS 3
#endif
constexpr int stored_buffers(int D) { return D == 256 ? OSLO_STORED_BUFFERS : 3; }
// waves of a block (32 keys each), by head size
constexpr int stored_waves(int D) { return D == 64 ? 4 : OSLO_STORED_WAVES; }

template <typename T, int D>
constexpr unsigned stored_lds_bytes() {
  return (unsigned)stored_buffers(D) * (kSchedTile * D * sizeof(T) + stored_waves(D) * kStoredTileBytes);
}

// blocks that share a CU: what the 160 KiB of LDS hold, four at most
template <typename T, int D>
constexpr int stored_blocks_per_cu() {
  const unsigned fit = 160u * 1024u / stored_lds_bytes<T, D>();
  return fit > 4u ? 4 : (int)fit;
}

template <typename T, int D, bool HAS_WINDOW>
__global__ __launch_bounds__(stored_waves(D) * kWave, (stored_blocks_per_cu<T, D>())) void attention_bwd_stored_kernel(
    const BwdArgs a) {
  constexpr int kStoredWaves = stored_waves(D);
  constexpr int kStoredKeys = 32 * kStoredWaves; // keys of a block
  constexpr int kStoredBuffers = stored_buffers(D);
  using Op = MatrixOp<T>;
  using Frag = typename Op::Frag;
  constexpr int kChunks = D / 8;
  constexpr int kBlocksD = D / 32;
  constexpr int kTile = kSchedTile * D;
  constexpr int kRowBytes = D * (int)sizeof(T);
  constexpr int kSwizzle = kChunks >= 16 ? 15 : 7;
  constexpr int kLoadsN = kSchedTile * kChunks / (kStoredWaves * kWave); // loads per thread and tile of Q (or dO)
  static_assert(kLoadsN >= 1, "a tile of fewer entries than the block has threads");
  constexpr int kItems = kLoadsN + 2;  // and the wave's own tile of the store
  constexpr int kHalfBlocks = kBlocksD / 2; // 32-feature blocks of a wave's half of the features
  constexpr int kOperands = 2 * kHalfBlocks; // transposed operands of Q or dO per tile, each used for both key tiles

  extern __shared__ __align__(1024) unsigned char lds_raw[];
  T *const t_lds = reinterpret_cast<T *>(lds_raw); // [3][query][chunk ^ f(query)][8]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;
  // two pairs of waves, 64 keys each; of a pair, a wave per half of the features
  const int feature_half = wave & 1;
  unsigned char *const x_lds = reinterpret_cast<unsigned char *>(t_lds + kStoredBuffers * kTile) +
                               wave * (kStoredBuffers * kStoredTileBytes); // [3][query][slot]
  // the two stored tiles the wave multiplies with: its own and its partner's
  const unsigned char *const x_pair = reinterpret_cast<unsigned char *>(t_lds + kStoredBuffers * kTile) +
                                      (wave & ~1) * (kStoredBuffers * kStoredTileBytes);

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 4;
  const bool for_dv = ((blockIdx.x >> 3) & 1) != 0;
  // The blocks of a head follow one another on one XCD, the longest walk
  // first: the two or three heads an XCD works on at a time keep their Q and dO
  // (2 x S x D values each) in its L2 while every block of the head reads them.
  const int S = a.S;
  const int key_blocks = (S + kStoredKeys - 1) / kStoredKeys;
  const int bh = a.bh0 + xcd + 8 * (slot / key_blocks);
  const int own_block = slot % key_blocks;
  if (bh >= a.batch_heads) return; // the whole block
  const int b = bh / a.heads;
  const int hd = bh - b * a.heads;
  const int own0 = own_block * kStoredKeys;
  const int key_tile = own0 / 32 + wave; // the key tile whose stored tiles this wave loads
  const int window = HAS_WINDOW ? a.window : 0;

  const int first_tile = own0 / kSchedTile;
  int last_query = S - 1;
  if (HAS_WINDOW && own0 + kStoredKeys - 1 + window - 1 < last_query) last_query = own0 + kStoredKeys - 1 + window - 1;
  const int tiles = last_query / kSchedTile + 1;

  const Strides3 &st_in = for_dv ? a.sdo : a.sq;
  const T *in_p = static_cast<const T *>(for_dv ? a.dout : a.q) + b * st_in.b + hd * st_in.h;
  const uint32_t in_row = (uint32_t)st_in.s * sizeof(T);
  // The permutation of a row's 16-byte chunks in LDS: chunk c of row r lies at
  // c ^ f(r). A transposing read takes, per half of the wave, 4 chunks (64 bytes)
  // of 4 consecutive rows, and rows lie a multiple of 256 bytes apart: with the
  // rows' low two bits in bits 2 and 3 of f the four rows use four different
  // quarters of the banks. (The permutation of the other passes, which leaves two
  // rows on the same banks, costs every such read two cycles.)
  constexpr bool kQuads = kChunks >= 16;
  auto f_of = [](int r) __attribute__((always_inline)) {
    if (kQuads) return ((r & 3) << 2) | ((r >> 2) & 3);
    return (((r & 3) << 1) | ((r >> 2) & 1) | (r & 8)) & kSwizzle;
  };
  // load j of a thread: entry (kStoredWaves j + wave) * 64 + lane of the tile
  uint32_t src_off[kLoadsN];
#pragma unroll
  for (int j = 0; j < kLoadsN; ++j) {
    const int entry = (kStoredWaves * j + wave) * kWave + lane;
    const int row = entry / kChunks, at = entry % kChunks;
    src_off[j] = (uint32_t)row * in_row + (uint32_t)(at ^ f_of(row)) * 16u;
  }
  TileStream src; // the next tile to load
  src.start(in_p, (uint32_t)(((int64_t)(S - 1) * st_in.s + D) * sizeof(T)), in_row, kSchedTile, first_tile, tiles);
  // The wave's tile of the store for query tile qt: nothing (zeros, without a
  // memory access) where the pass that writes the store left none: above the
  // diagonal, past the last query tile, and before the first key tile that the
  // block owning qt walks under a window.
  uint64_t store_at = reinterpret_cast<uint64_t>(a.tiles) +
                      (uint64_t)(((int64_t)(bh - a.bh0) * a.head_tiles + (int64_t)first_tile * (first_tile + 1) / 2 + key_tile) *
                                     kStoredPairBytes +
                                 (for_dv ? 0 : kStoredTileBytes));
  int store_tile = first_tile; // the query tile store_at belongs to
  auto store_descriptor = [&]() __attribute__((always_inline)) {
    bool there = store_tile >= key_tile && store_tile < tiles;
    if constexpr (HAS_WINDOW) {
      const int walk0 = (store_tile / 4) * kOwnPerBlock - window + 1;
      there = there && key_tile >= (walk0 > 0 ? walk0 / kSchedTile : 0);
    }
    u32x4 d;
    d[0] = __builtin_amdgcn_readfirstlane((uint32_t)store_at);
    d[1] = __builtin_amdgcn_readfirstlane((uint32_t)(store_at >> 32) & 0xffffu);
    d[2] = __builtin_amdgcn_readfirstlane(there ? (uint32_t)kStoredTileBytes : 0u);
    d[3] = 0x00020000u;
    return d;
  };
  int t = first_tile;
  int buf_now = 0, buf_load = 0; // buffers of tile t and of the tile being loaded (t + kStoredBuffers - 1 in the loop)
  auto next_buffer = [](int b) __attribute__((always_inline)) { return b == kStoredBuffers - 1 ? 0 : b + 1; };
  // item `it` of the loads of the next tile to load
  auto stage_item = [&](int it) __attribute__((always_inline)) {
    if (it < kLoadsN) {
      lds_load_b128(src.descriptor(), t_lds + buf_load * kTile + (kStoredWaves * it + wave) * (kWave * 8), src_off[it]);
      if (it == kLoadsN - 1) src.advance();
      return;
    }
    it -= kLoadsN;
    // (read once: past the caches' usual replacement, so that the tiles of Q and dO stay)
    // LDS gets rows of [query][slot] (lane L of load `it`: query 16 it + L / 4, 16-byte chunk L % 4 of its row);
    // in memory that chunk, operand u = (L % 4) / 2 of half h = L % 2 of the wave that wrote it, lies at
    // 1024 u + 16 (query + 32 h)
    lds_load_b128_once(store_descriptor(), x_lds + buf_load * kStoredTileBytes + it * 1024,
                       (uint32_t)(1024 * ((lane >> 1) & 1) + 16 * (16 * it + (lane >> 2) + 32 * (lane & 1))));
    if (it == 1) {
      store_at += (uint64_t)(store_tile + 1) * kStoredPairBytes;
      ++store_tile;
      buf_load = next_buffer(buf_load);
    }
  };

  // transposed operands of the tiles of Q and dO (the passes above read them the same way)
  typedef short Short4 __attribute__((ext_vector_type(4)));
  // Transposed operand (u, ib): 16 queries u of block feature_half * kHalfBlocks + ib of 32 features; two reads
  // (jj) each. tr_lane[ib][jj]: the lane's byte offset in the tile, the row of the read apart.
  uint32_t tr_lane[kHalfBlocks][2], x_lane;
  {
    const int j = lane & 15, group = lane >> 4;
    const int kq = j >> 2, fb = j & 3, hh = group >> 1, fg = group & 1;
#pragma unroll
    for (int ib = 0; ib < kHalfBlocks; ++ib) {
      const int i = feature_half * kHalfBlocks + ib;
      if constexpr (kQuads) {
        // row 16 u + 8 jj + 4 hh + kq, chunk 4 i + w of it, w = 2 fg + fb / 2: f is 4 kq + 2 jj + hh, so the chunk
        // lies at 16 (i / 4) + 4 (i % 4 ^ kq) + (w ^ hh ^ 2 jj)
        const uint32_t own = (uint32_t)(4 * hh + kq) * kRowBytes + 64u * (uint32_t)kq +
                             16u * (uint32_t)((2 * fg + (fb >> 1)) ^ hh) + 8u * (uint32_t)(fb & 1);
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
          tr_lane[ib][jj] = (own ^ (uint32_t)(64 * (i & 3) + 32 * jj)) + 256u * (uint32_t)(i >> 2);
      } else {
        const int flow = ((kq << 1) | hh) & kSwizzle;
        const int x = (2 * fg + (fb >> 1)) ^ (flow & 3);
        const int flip = flow >> 2;
        const uint32_t base = (uint32_t)(4 * hh + kq) * kRowBytes + (uint32_t)x * 16u + (uint32_t)(fb & 1) * 8u;
        tr_lane[ib][0] = tr_lane[ib][1] = base + 64u * (uint32_t)(flip ^ (i & 1)) + 64u * (uint32_t)(i & ~1);
      }
    }
    // the same read of a stored tile: rows of 64 bytes, no permutation of chunks
    x_lane = (uint32_t)(4 * hh + kq) * 64u + (uint32_t)fg * 32u + (uint32_t)fb * 8u;
  }
  auto read_transposed = [&](const T *base, int n) __attribute__((always_inline)) {
    const int u = n / kHalfBlocks, ib = n % kHalfBlocks;
    Short4 part[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const char *at = reinterpret_cast<const char *>(base) + tr_lane[ib][jj] + (16 * u + 8 * jj) * kRowBytes;
      part[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) Short4 *)(at));
    }
    return __builtin_bit_cast(Frag, __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_stored = [&](const unsigned char *base, int u) __attribute__((always_inline)) {
    Short4 part[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
      part[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) Short4 *)(base + x_lane + (16 * u + 8 * jj) * 64));
    return __builtin_bit_cast(Frag, __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7));
  };

  f32x16 acc[2][kHalfBlocks]; // [key tile of the pair][block of features]
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int i = 0; i < kHalfBlocks; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[g][i][r] = 0.f;

  constexpr int kRing = kOperands < 4 ? kOperands : 4;
  constexpr int kPerOperand = (kItems + kOperands - 1) / kOperands;
  // A tile as one straight run of code: operands are read from LDS kRing
  // operands ahead, a later tile's loads go between the products.
  auto one_tile = [&]() __attribute__((always_inline)) {
    const T *bt = t_lds + buf_now * kTile;
    const unsigned char *bx = x_pair + buf_now * kStoredTileBytes;
    Frag x[2][2], ring[kRing];
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int u = 0; u < 2; ++u) x[g][u] = read_stored(bx + g * (kStoredBuffers * kStoredTileBytes), u);
#pragma unroll
    for (int p = 0; p < kRing; ++p) ring[p] = read_transposed(bt, p);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kOperands; ++n) {
      const int u = n / kHalfBlocks, ib = n % kHalfBlocks;
      acc[0][ib] = Op::run(ring[n % kRing], x[0][u], acc[0][ib]);
      acc[1][ib] = Op::run(ring[n % kRing], x[1][u], acc[1][ib]);
      if (n + kRing < kOperands) ring[n % kRing] = read_transposed(bt, n + kRing);
#pragma unroll
      for (int it = n * kPerOperand; it < (n + 1) * kPerOperand && it < kItems; ++it) stage_item(it);
      __builtin_amdgcn_sched_barrier(0);
    }
    buf_now = next_buffer(buf_now);
  };
  // the first tiles on their way
#pragma unroll
  for (int rep = 0; rep < kStoredBuffers - 1; ++rep)
#pragma unroll
    for (int it = 0; it < kItems; ++it) stage_item(it);
  // (Two tiles between barriers, with four buffers, measured slower: 413-445 against 352-391 us.)
  for (; t < tiles; ++t) {
    wait_vm<(kStoredBuffers - 2) * kItems>(); // (the tiles after t may still be on their way)
    __syncthreads(); // tile t is in LDS; the buffers written next (tile t - 1's) have been read
    one_tile();
  }
  wait_vm<0>(); // (nothing may still be on its way into LDS when the block ends)

  typedef T Out4 __attribute__((ext_vector_type(4)));
  const Strides3 &st_out = for_dv ? a.sdv : a.sdk;
  const float factor = for_dv ? (a.drop.drop ? a.drop.keep_scale : 1.0f) : a.scale;
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    // lane c holds the key at slot c of the store's rows: c with bits 2 and 3 swapped
    const int own = own0 + 32 * ((wave & ~1) + g) + ((col & 0x13) | ((col & 4) << 1) | ((col & 8) >> 1));
    if (own >= S) continue;
    T *op = static_cast<T *>(for_dv ? a.dv : a.dk) + b * st_out.b + hd * st_out.h + (int64_t)own * st_out.s +
            32 * kHalfBlocks * feature_half;
#pragma unroll
    for (int i = 0; i < kHalfBlocks; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Out4 w;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) w[tt] = static_cast<T>(acc[g][i][4 * j + tt] * factor);
        *reinterpret_cast<Out4 *>(op + 32 * i + 8 * j + 4 * half) = w;
      }
  }
}

// delta[bh, q] = sum_d dO[q, d] * O[q, d], fp32. D / 8 lanes share a row.
template <typename T, int D>
__global__ __launch_bounds__(kBlockThreads) void attention_delta_kernel(
    float *delta, const T *out, const T *dout, Strides3 so, Strides3 sdo, int S,
    int heads, int64_t rows) {
  constexpr int kLanes = D / 8;
  constexpr int kRows = kBlockThreads / kLanes;
  int64_t row = (int64_t)blockIdx.x * kRows + threadIdx.x / kLanes;
  const bool live = row < rows;
  if (!live) row = rows - 1; // the lanes of a group stay together for the reduction
  const int part = threadIdx.x % kLanes;
  const int64_t bh = row / S;
  const int q = (int)(row - bh * S);
  const int64_t b = bh / heads, hd = bh - b * heads;
  typedef T Vec8 __attribute__((ext_vector_type(8)));
  const Vec8 o = *reinterpret_cast<const Vec8 *>(out + b * so.b + hd * so.h + (int64_t)q * so.s + 8 * part);
  const Vec8 g = *reinterpret_cast<const Vec8 *>(dout + b * sdo.b + hd * sdo.h + (int64_t)q * sdo.s + 8 * part);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s = __builtin_fmaf(static_cast<float>(o[i]), static_cast<float>(g[i]), s);
  s = sum_over_lanes<kLanes>(s);
  if (live && part == 0) delta[row] = s;
}

// dK and dV of the heads [a.bh0, a.bh0 + 8 * a.head_groups) from the tile store
template <typename T, int D>
int launch_stored(const BwdArgs &a, hipStream_t stream) {
  const int key_blocks = (a.S + 32 * stored_waves(D) - 1) / (32 * stored_waves(D));
  const dim3 grid((unsigned)(2 * 8 * a.head_groups * key_blocks)); // a block per gradient
  constexpr unsigned kLds = stored_lds_bytes<T, D>();
  auto *kernel = a.window > 0 ? attention_bwd_stored_kernel<T, D, true> : attention_bwd_stored_kernel<T, D, false>;
  if (kLds > 64u * 1024u) {
    const int s = raise_lds_limit(reinterpret_cast<const void *>(kernel), kLds, "oslo_attention_prefill_bwd_stored");
    if (s != OSLO_OK) return s;
  }
  kernel<<<grid, dim3(stored_waves(D) * kWave), kLds, stream>>>(a);
  return check_launch("attention_prefill_bwd_stored");
}

template <typename T, int D>
int launch_bwd_dim(const BwdArgs &a, float *delta, const void *out, const Strides3 &so,
                   hipStream_t stream, size_t store_bytes) {
  const int64_t rows = (int64_t)a.batch_heads * a.S;
  constexpr int kRows = kBlockThreads / (D / 8);
  attention_delta_kernel<T, D><<<dim3((unsigned)((rows + kRows - 1) / kRows)), dim3(kBlockThreads), 0, stream>>>(
      delta, static_cast<const T *>(out), static_cast<const T *>(a.dout), so, a.sdo, a.S, a.heads, rows);
  int s = check_launch("attention_prefill_bwd(delta)");
  if (s != OSLO_OK) return s;
  if (a.tiles != nullptr) {
    // The probabilities through memory: the dQ pass writes P and dS of every tile
    // on or below the diagonal, a second pass accumulates dK and dV from them (5
    // matrix products per tile, the number the mathematics has). Groups of 8
    // heads, as many at a time as the store holds, in launches of equal size.
    const int64_t per_group = 8 * a.head_tiles * kStoredPairBytes;
    const int fit = (int)std::min<int64_t>((int64_t)(store_bytes / (size_t)per_group), a.head_groups);
    const int launches = (a.head_groups + fit - 1) / fit;
    const int each = (a.head_groups + launches - 1) / launches;
    for (int g = 0; g < a.head_groups; g += each) {
      BwdArgs part = a;
      part.bh0 = 8 * g;
      part.head_groups = std::min(each, a.head_groups - g);
      s = launch_role<T, D, kRoleDQ, true>(part, stream);
      if (s != OSLO_OK) return s;
      s = launch_stored<T, D>(part, stream);
      if (s != OSLO_OK) return s;
    }
    return OSLO_OK;
  }
  s = launch_role<T, D, kRoleDQ>(a, stream);
  if (s != OSLO_OK) return s;
  // dK and dV: one combined pass where both accumulators fit a lane's registers
  // (heads of 64 and 128 features: 2 x 32 and 2 x 64 accumulator registers; timed
  // at [8,32,2048,64] 692 against 816 us for the whole backward, at [8,16,2048,128]
  // 635 against 648, with dropout 778 against 873). At 256 features they are 2 x
  // 128 beside 128 registers of fixed operands: the compiler spills 47 to 178
  // registers per lane, 39 scratch accesses in every tile, and the backward takes
  // 2917 us instead of 1382; there each gradient keeps a pass of its own.
  if constexpr (D <= OSLO_BWD_COMBINED_MAX_DIM) {
    return launch_role<T, D, kRoleDKV>(a, stream);
  } else {
    s = launch_role<T, D, kRoleDK>(a, stream);
    if (s != OSLO_OK) return s;
    return launch_role<T, D, kRoleDV>(a, stream);
  }
}

template <typename T>
int launch_bwd(const BwdArgs &a, float *delta, const void *out, const Strides3 &so, int head_dim,
               hipStream_t stream, size_t store_bytes) {
  switch (head_dim) {
    case 64: return launch_bwd_dim<T, 64>(a, delta, out, so, stream, store_bytes);
    case 128: return launch_bwd_dim<T, 128>(a, delta, out, so, stream, store_bytes);
    default: return launch_bwd_dim<T, 256>(a, delta, out, so, stream, store_bytes);
  }
}


} // namespace
} // namespace oslo

extern "C" size_t oslo_attention_prefill_bwd_workspace_bytes(int64_t batch, int64_t heads, int64_t S) {
  if (batch <= 0 || heads <= 0 || S <= 0) return 0;
  return (size_t)batch * (size_t)heads * (size_t)S * sizeof(float);
}

namespace oslo {

// Both entry points: `store` null = every pass computes the scores it needs.
static int prefill_bwd(const char *name, void *dq, void *dk, void *dv, const void *dout, const void *q, const void *k,
                const void *v, const void *out, const float *lse, float *workspace, void *store,
                size_t store_bytes, const float *pad, float scale, float p, uint64_t philox_seed,
                uint64_t philox_offset, int64_t batch, int64_t heads, int64_t S, int64_t head_dim,
                int64_t window, const int64_t *strides, int dtype, oslo_stream_t stream) {
  if (batch < 0 || heads < 0 || S < 0 || head_dim < 0 || window < 0)
    return fail(OSLO_E_BAD_ARG, "%s: negative size", name);
  if (dtype != OSLO_F16 && dtype != OSLO_BF16) {
    if (dtype == OSLO_F32) return fail(OSLO_E_UNSUPPORTED, "%s: fp16 and bf16 are taken, not fp32", name);
    return fail(OSLO_E_BAD_ARG, "unknown dtype %d", dtype);
  }
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(OSLO_E_UNSUPPORTED, "%s: heads of %lld features (64, 128 or 256 are taken)", name,
                (long long)head_dim);
  if (!(scale > 0.0f)) return fail(OSLO_E_BAD_ARG, "%s: the scale must be positive", name);
  DropArgs drop;
  const int ds = make_drop_args(name, p, philox_seed, philox_offset, &drop);
  if (ds != OSLO_OK) return ds;
  if (batch == 0 || heads == 0 || S == 0) return OSLO_OK;
  if (drop.drop && S % 8 != 0)
    return fail(OSLO_E_UNSUPPORTED, "%s: with attention dropout S must be a multiple of 8", name);
  if (!dq || !dk || !dv || !dout || !q || !k || !v || !out || !lse || !workspace || !strides)
    return fail(OSLO_E_BAD_ARG, "%s: null pointer", name);
  if (batch * heads > (int64_t)0x7fffffff / 8 || batch * heads * S > (int64_t)0x7fffffff)
    return fail(OSLO_E_UNSUPPORTED, "%s: too many rows for one launch", name);
  // strides: q, k, v, out, dout, dq, dk, dv (batch, head, position each)
  const void *ptrs[8] = {q, k, v, out, dout, dq, dk, dv};
  for (int i = 0; i < 8; ++i) {
    if (!aligned16(ptrs[i])) return fail(OSLO_E_UNSUPPORTED, "%s: tensors must be 16-byte aligned", name);
    const int64_t sb = strides[3 * i], sh = strides[3 * i + 1], ss = strides[3 * i + 2];
    if (sb < 0 || sh < 0 || ss < head_dim || sb % 8 || sh % 8 || ss % 8)
      return fail(OSLO_E_UNSUPPORTED,
                  "%s: strides must be multiples of 8 elements, the position stride at least head_dim", name);
    if ((S + kOwnPerBlock) * ss * 2 > (int64_t)0x7fffffff)
      return fail(OSLO_E_UNSUPPORTED, "%s: a head's slice exceeds 2 GiB", name);
  }
  if (pad != nullptr && (S % 4 != 0 || !aligned16(pad)))
    return fail(OSLO_E_UNSUPPORTED,
                "%s: with a padding mask S must be a multiple of 4 and the mask 16-byte aligned", name);
  if (!aligned16(lse) || !aligned16(workspace) || !aligned16(store))
    return fail(OSLO_E_UNSUPPORTED, "%s: lse and the workspaces must be 16-byte aligned", name);
  auto st = [&](int i) { return Strides3{strides[3 * i], strides[3 * i + 1], strides[3 * i + 2]}; };
  BwdArgs a;
  a.q = q, a.k = k, a.v = v, a.dout = dout, a.dq = dq, a.dk = dk, a.dv = dv;
  a.lse = lse, a.delta = workspace, a.pad = pad, a.drop = drop;
  a.sq = st(0), a.sk = st(1), a.sv = st(2), a.sdo = st(4), a.sdq = st(5), a.sdk = st(6), a.sdv = st(7);
  a.scale = scale;
  a.scale_log2e = scale * kLog2eB;
  a.S = (int)S;
  a.heads = (int)heads;
  a.batch_heads = (int)(batch * heads);
  a.head_groups = (a.batch_heads + 7) / 8;
  a.own_blocks = (int)((S + kOwnPerBlock - 1) / kOwnPerBlock);
  a.window = window >= S ? 0 : (int)window;
  a.tiles = static_cast<unsigned char *>(store);
  a.bh0 = 0;
  a.head_tiles = stored_head_tiles(a.own_blocks);

  if (store != nullptr && store_bytes < (size_t)(8 * a.head_tiles * kStoredPairBytes))
    return fail(OSLO_E_BAD_ARG, "%s: a store of %zu bytes; 8 heads of %lld positions need %lld", name, store_bytes,
                (long long)S, (long long)(8 * a.head_tiles * kStoredPairBytes));
  if ((int64_t)16 * a.head_groups * a.own_blocks > (int64_t)0x7fffffff)
    return fail(OSLO_E_UNSUPPORTED, "%s: too many blocks for one launch", name);
  hipStream_t stm = static_cast<hipStream_t>(stream);
  if (dtype == OSLO_F16) return launch_bwd<f16>(a, workspace, out, st(3), (int)head_dim, stm, store_bytes);
  return launch_bwd<bf16>(a, workspace, out, st(3), (int)head_dim, stm, store_bytes);
}

} // namespace oslo

extern "C" size_t oslo_attention_prefill_bwd_store_bytes(int64_t batch, int64_t heads, int64_t S) {
  if (batch <= 0 || heads <= 0 || S <= 0) return 0;
  const int64_t groups = (batch * heads + 7) / 8;
  const int64_t own_blocks = (S + oslo::kOwnPerBlock - 1) / oslo::kOwnPerBlock;
  return (size_t)(8 * groups) * (size_t)oslo::stored_head_tiles(own_blocks) * (size_t)oslo::kStoredPairBytes;
}

extern "C" int oslo_attention_prefill_bwd(void *dq, void *dk, void *dv, const void *dout,
                                          const void *q, const void *k, const void *v,
                                          const void *out, const float *lse,
                                          float *workspace, const float *pad, float scale,
                                          float p, uint64_t philox_seed,
                                          uint64_t philox_offset,
                                          int64_t batch, int64_t heads, int64_t S,
                                          int64_t head_dim, int64_t window,
                                          const int64_t *strides, int dtype,
                                          oslo_stream_t stream) {
  return oslo::prefill_bwd("oslo_attention_prefill_bwd", dq, dk, dv, dout, q, k, v, out, lse, workspace, nullptr, 0,
                           pad, scale, p, philox_seed, philox_offset, batch, heads, S, head_dim, window, strides,
                           dtype, stream);
}

extern "C" int oslo_attention_prefill_bwd_stored(void *dq, void *dk, void *dv, const void *dout,
                                                 const void *q, const void *k, const void *v,
                                                 const void *out, const float *lse,
                                                 float *workspace, void *store, size_t store_bytes,
                                                 const float *pad, float scale,
                                                 float p, uint64_t philox_seed,
                                                 uint64_t philox_offset,
                                                 int64_t batch, int64_t heads, int64_t S,
                                                 int64_t head_dim, int64_t window,
                                                 const int64_t *strides, int dtype,
                                                 oslo_stream_t stream) {
  if (store == nullptr)
    return oslo::fail(OSLO_E_BAD_ARG, "oslo_attention_prefill_bwd_stored: null store");
  return oslo::prefill_bwd("oslo_attention_prefill_bwd_stored", dq, dk, dv, dout, q, k, v, out, lse, workspace, store,
                           store_bytes, pad, scale, p, philox_seed, philox_offset, batch, heads, S, head_dim, window,
                           strides, dtype, stream);
}

