// Causal attention over a whole prompt in one kernel (no [S, S] matrix in
// memory):
//   out[q, :] = sum_{k <= q} softmax_k(scale * Q[q, :] . K[k, :] + pad[k]) * V[k, :]
// for every (batch, head), 16-bit inputs, fp32 accumulation. It replaces the
// three launches of the fused attention -- batched matmul
// Q K^T, the fused scale + mask + softmax, batched matmul P V
// (oslo/models/gptj/modeling_gptj.py:936-951,
// oslo/models/gpt_neo/modeling_gpt_neo.py:993-1008,
// oslo/models/gpt2/modeling_gpt2.py:1435-1459) -- which write the scores,
// read and write them again in the softmax and read them a fourth time. This
// is the one kernel of the library that is bound by the matrix cores, not by
// HBM: 4 * S^2/2 * head_dim flops per head against 4 * S * head_dim elements.
//
// One block of four waves takes 128 queries of one head, 32 per wave, and walks
// the keys in tiles of 32. Everything is computed transposed, so that a query
// is a lane and not a register index:
//   S^T[key, q] = K_tile (A operand, rows = keys, from LDS) x Q^T (B operand,
//                 held in registers for the whole kernel),
//   O^T[d, q]  += V_tile^T (A operand, rows = features, from LDS) x P^T (B).
// In the accumulator layout of v_mfma_f32_32x32x16 a lane holds one column
// (lane % 32 = the query) and 16 rows, so the reference maximum, the sum and
// the rescaling of O are per-lane scalars: the softmax needs no LDS. The 16
// rows of a lane are keys 8j + 4h + t (j, t = 0..3; h = lane / 32), and a B
// operand wants, per half, 8 consecutive contraction slots: the probabilities
// are used where they are, and the contraction order of V^T is permuted to
// match.
// K and V tiles go from global memory straight into LDS (three buffers each),
// stored as they are in memory; the transposition of V happens in the LDS
// read (ds_read_b64_tr_b16). What limits the kernel is not the matrix core
// alone but what a wave can issue: with one wave per SIMD (head_dim 256: O^T
// and Q^T take 192 of a lane's registers) a matrix product keeps the wave from
// issuing for most of its 32 cycles, and every other instruction costs four
// more. So a tile is one straight run of code, ordered by hand: the products
// of S^T with the next tiles' loads between them, then the products of
// O^T of the previous tile with the softmax of this one between them.

#include "attention.hpp"

namespace oslo {
namespace {

constexpr int kQueriesPerBlock = 128;
constexpr int kKeysPerTile = 32;
constexpr float kLog2e = 1.4426950408889634f;
// See the kernel: how far a score may exceed the reference maximum (log2
// units). A general tile raises the maximum of a query when a score exceeds it
// by more than kRaise; the scheduled tiles do not look at the scores but at a
// lane's sum of 16 exponentials: none of them exceeds the sum, and a sum above
// 2^kSlack means a score more than kSlack - 4 = kRaise above the maximum, so
// that doing such a tile again in plain order (redo_tile) does raise it.
constexpr float kRaise = 4.0f;
constexpr float kSumLimit = 256.0f; // 2^kSlack, kSlack = 8
// The reference of a query that has not seen a key yet (sliding windows): any
// finite score lies more than kRaise above it, and 2^(score - floor) is +inf.
constexpr float kReferenceFloor = -3.0e38f;

struct PrefillArgs {
  void *out;
  const void *q, *k, *v;
  const float *pad; // [batch, S] additive, or null
  float *lse;       // [batch * heads, S] or null: log2 of the row's sum of exponentials
  int64_t q_b, q_h, q_s; // element strides: batch, head, position
  int64_t k_b, k_h, k_s;
  int64_t v_b, v_h, v_s;
  int64_t o_b, o_h, o_s;
  float scale, scale_log2e;
  int S;
  int heads;
  int batch_heads;
  int head_groups; // ceil(batch_heads / 8)
  int query_blocks;
  int window; // 0: every key up to the query; else the last `window` of them
  DropArgs drop; // attention dropout (the DROP variants of the kernel)
};

// Tiles of K and of V go from global memory straight into LDS (buffer loads
// with the LDS as destination: a wave's instruction puts its 64 x 16 bytes at
// consecutive addresses), three buffers each: the one being read, the one that
// has landed and the one in flight. Both are stored as they are in memory,
// [key][feature], 16-byte chunks permuted within a key's row so that the lanes
// the LDS serves together hit different banks: K is read 16 bytes per lane by
// 16 lanes with consecutive keys (chunk ^ key), V through the transposing read,
// 8 bytes per lane by 4 keys x 4 chunk halves (chunk ^ 2 (key % 4)). The
// permutation is applied on the global side: a lane fetches the chunk that
// belongs at its LDS slot.
constexpr int kBuffers = 3;
constexpr int kPadSlots = kBlockThreads; // mask values of a tile: the first 32 count, every wave loads 64
template <typename T, int D>
constexpr unsigned prefill_lds_bytes() {
  return 2u * kBuffers * kKeysPerTile * D * sizeof(T) + kBuffers * kPadSlots * sizeof(float) +
         kWavesPerBlock * 32u * sizeof(uint32_t);
}

template <typename T, int D, bool HAS_PAD, bool HAS_WINDOW, bool DROP>
__global__ __launch_bounds__(kBlockThreads, D == 256 ? 1 : D == 128 ? 2 : 3) void attention_prefill_kernel(
    const PrefillArgs a) {
  using Op = MatrixOp<T>;
  using Frag = typename Op::Frag;
  constexpr int kChunks = D / 8;   // 16-byte chunks of a key
  constexpr int kSteps = D / 16;   // contraction steps of Q K^T
  constexpr int kBlocksD = D / 32; // 32-row blocks of O^T
  constexpr int kLoadsK = kKeysPerTile * kChunks / kBlockThreads; // per thread and tile
  constexpr int kTile = kKeysPerTile * D;      // elements of a K or V buffer
  constexpr int kRowBytes = D * (int)sizeof(T);
  constexpr int kKeyShift = D == 64 ? 1 : 0;   // rows of 128 bytes: two keys share a set of banks
  constexpr int kSwizzleK = kChunks >= 16 ? 15 : 7;
  extern __shared__ __align__(1024) unsigned char lds_raw[];
  T *const k_lds = reinterpret_cast<T *>(lds_raw); // [3][key][chunk ^ swizzle(key)][8]
  T *const vt_lds = k_lds + kBuffers * kTile;      // [3][key][chunk ^ 2 (key % 4)][8]
  float *const pad_lds = reinterpret_cast<float *>(vt_lds + kBuffers * kTile); // [3][key], as loaded

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;
  uint32_t *const keep_lds = reinterpret_cast<uint32_t *>(pad_lds + kBuffers * kPadSlots) + 32 * wave;

  // All query blocks of a head run on one XCD (blocks go round-robin over
  // the 8 XCDs), so its keys and values are read from HBM into one L2; the
  // blocks with the most keys start first.
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int bh = xcd + 8 * (slot % a.head_groups);
  const int qb = a.query_blocks - 1 - slot / a.head_groups;
  if (bh >= a.batch_heads) return; // the whole block
  const int b = bh / a.heads;
  const int hd = bh - b * a.heads;
  const int S = a.S;
  const int q0 = qb * kQueriesPerBlock;

  const T *qp = static_cast<const T *>(a.q) + b * a.q_b + hd * a.q_h;
  const T *kp = static_cast<const T *>(a.k) + b * a.k_b + hd * a.k_h;
  const T *vp = static_cast<const T *>(a.v) + b * a.v_b + hd * a.v_h;
  // (rows at or past S fall outside the descriptors and read as zeros)
  const uint32_t q_row = (uint32_t)a.q_s * sizeof(T);
  const uint32_t k_row = (uint32_t)a.k_s * sizeof(T);
  const uint32_t v_row = (uint32_t)a.v_s * sizeof(T);

  // Q^T as B operands, in registers for the whole kernel: lane (query, half)
  // holds features 16 s + 8 half .. + 7 (loaded in the prologue, by way of LDS)
  const int wave_q0 = q0 + 32 * wave;
  const int qrow = wave_q0 + col;
  Frag qf[kSteps];

  const float *padr = HAS_PAD ? a.pad + (int64_t)b * S : nullptr;
  const int window = HAS_WINDOW ? a.window : 0;
  const int behind = HAS_WINDOW ? qrow - window : -1; // the last key behind the query's window

  const int last_key = (q0 + kQueriesPerBlock < S ? q0 + kQueriesPerBlock : S) - 1;
  const int tiles = last_key / kKeysPerTile + 1;
  // with a sliding window the block starts at the tile of its first query's
  // first visible key
  const int first_tile = HAS_WINDOW && q0 - window + 1 > 0 ? (q0 - window + 1) / kKeysPerTile : 0;
  // Tiles [plain_begin, plain_end) are visible in full to every query of the
  // block: no comparison, no wave sits one out. The block's first tile is not
  // among them (its queries have no reference maximum yet).
  const int plain_end = q0 / kKeysPerTile;
  int plain_begin = !HAS_WINDOW ? 0
                    : q0 + kQueriesPerBlock - window > 0
                        ? (q0 + kQueriesPerBlock - window + kKeysPerTile - 1) / kKeysPerTile
                        : 0;
  if (plain_begin < first_tile + 1) plain_begin = first_tile + 1;

  // A tile travels global -> LDS without passing through registers. While tile
  // t is computed (S^T of tile t, then O^T += V^T P^T of tile t - 1 under the
  // softmax of tile t) the loads of K of tile t + 2 and of V of tile t + 1 are
  // issued, into the buffers that tile t - 1 (K) and tile t - 2 (V) have left;
  // they are waited for a whole tile later, before the barrier that opens tile
  // t + 2. The staging is cut into items (one load each), so that a tile's
  // straight-line code can place them one by one.
  // Load j of wave w fills the 64 slots of 16 bytes from (4 j + w) * 64 on: slot
  // sigma is (row = sigma / kChunks, chunk position = sigma % kChunks) and holds
  // the chunk whose index is the position with the row's permutation undone.
  uint32_t k_off[kLoadsK], v_off[kLoadsK];
#pragma unroll
  for (int j = 0; j < kLoadsK; ++j) {
    const int sigma = (4 * j + wave) * kWave + lane;
    const int row = sigma / kChunks, at = sigma % kChunks;
    k_off[j] = (uint32_t)row * k_row + (uint32_t)(at ^ ((row >> kKeyShift) & kSwizzleK)) * 16u;
    v_off[j] = (uint32_t)row * v_row + (uint32_t)(at ^ (2 * (row & 3))) * 16u;
  }
  // The padding mask of a tile travels with its keys, the same way: every
  // wave loads 64 values into a quarter of its own of the tile's slots; the
  // first 32 of the first wave's are the tile's (lanes past them, and the
  // other waves, read outside the descriptor: zeros, and no branch).
  // A tile is loaded through a descriptor of its own (base = the tile's first
  // key, size = what is left of the head's slice from there, nothing for tiles
  // past the block's last one: rows at or past S and whole tiles that are not
  // needed read as zeros without a memory access). The descriptors of the next
  // tiles to load are kept as scalars and stepped from tile to tile; the vector
  // offsets of a thread's loads are the same for every tile.
  struct TileSource {
    uint64_t base;  // the tile's first key
    uint32_t left;  // bytes from there to the end of the head's slice
    uint32_t step;  // bytes from a tile to the next
    int tile;       // its index
    __device__ __forceinline__ void start(const void *p, uint32_t bytes, uint32_t row_bytes, int t) {
      step = kKeysPerTile * row_bytes;
      tile = t;
      const uint32_t skip = (uint32_t)(t < 0 ? 0 : t) * step;
      base = reinterpret_cast<uint64_t>(p) + skip;
      left = skip < bytes ? bytes - skip : 0u;
    }
    __device__ __forceinline__ void advance() {
      base += step;
      left = left > step ? left - step : 0u;
      ++tile;
    }
    // raw 32-bit buffer descriptor (word 3 = 0x00020000, as make_rsrc builds it)
    __device__ __forceinline__ u32x4 descriptor(int tiles) const {
      u32x4 d; // (read as scalars: the hand-written load takes the descriptor in scalar registers)
      d[0] = __builtin_amdgcn_readfirstlane((uint32_t)base);
      d[1] = __builtin_amdgcn_readfirstlane((uint32_t)(base >> 32) & 0xffffu);
      d[2] = __builtin_amdgcn_readfirstlane(tile >= 0 && tile < tiles ? left : 0u);
      d[3] = 0x00020000u;
      return d;
    }
  };
  TileSource k_src, v_src, pad_src; // the next tiles to load: K of tile t + 2, V of tile t + 1, mask of tile t + 2
  k_src.start(kp, (uint32_t)(((int64_t)(S - 1) * a.k_s + D) * sizeof(T)), k_row, first_tile);
  v_src.start(vp, (uint32_t)(((int64_t)(S - 1) * a.v_s + D) * sizeof(T)), v_row, first_tile);
  if constexpr (HAS_PAD) pad_src.start(padr, (uint32_t)S * (uint32_t)sizeof(float), (uint32_t)sizeof(float), first_tile);
  // (lanes past the tile's 32 mask values read outside every descriptor)
  const uint32_t pad_off = tid < kKeysPerTile ? (uint32_t)tid * (uint32_t)sizeof(float) : 0x80000000u;
  int pad_at[3] = {0, kPadSlots, 2 * kPadSlots}; // the mask slots of tiles t, t + 1, t + 2
  constexpr int kItems = 2 * kLoadsK + (HAS_PAD ? 1 : 0);
  constexpr int kLoadsPerTile = 2 * kLoadsK + (HAS_PAD ? 1 : 0); // what a tile leaves in flight
  // The load itself is written out: the compiler, told of a load into LDS,
  // waits for every such load before the next LDS read of any buffer; these
  // are waited for by count, a tile later (wait_loads).
  auto load_to_lds = [&](const u32x4 &desc, const T *dst, uint32_t offset) __attribute__((always_inline)) {
    const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)reinterpret_cast<uintptr_t>(dst)); // LDS addresses are the low 32 bits
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(at), "v"(offset), "s"(desc) : "m0");
  };
  // the three buffers of K and of V, as element offsets, in the order (tile t,
  // t + 1, t + 2) and (t - 1, t, t + 1); rotated from tile to tile
  int k_at[3] = {0, kTile, 2 * kTile}, v_at[3] = {2 * kTile, 0, kTile};
  int t = first_tile;
  auto next_tile = [&]() __attribute__((always_inline)) {
    ++t;
    const int k0 = k_at[0], v0 = v_at[0];
    k_at[0] = k_at[1], k_at[1] = k_at[2], k_at[2] = k0;
    v_at[0] = v_at[1], v_at[1] = v_at[2], v_at[2] = v0;
    if constexpr (HAS_PAD) {
      const int p0 = pad_at[0];
      pad_at[0] = pad_at[1], pad_at[1] = pad_at[2], pad_at[2] = p0;
    }
  };
  auto k_buffer = [&](int d) __attribute__((always_inline)) { return k_lds + k_at[d]; };      // of tile t + d, d = 0 .. 2
  auto v_buffer = [&](int d) __attribute__((always_inline)) { return vt_lds + v_at[d + 1]; }; // of tile t + d, d = -1 .. 1
  // item `it` of the staging of a tile: the loads of K of tile t + 2 into kw,
  // then those of V of tile t + 1 into vw, then the mask values
  auto stage_item = [&](int it, T *kw, T *vw) __attribute__((always_inline)) {
    if (it < kLoadsK) {
      load_to_lds(k_src.descriptor(tiles), kw + (4 * it + wave) * (kWave * 8), k_off[it]);
      if (it == kLoadsK - 1) k_src.advance();
      return;
    }
    it -= kLoadsK;
    if (it < kLoadsK) {
      load_to_lds(v_src.descriptor(tiles), vw + (4 * it + wave) * (kWave * 8), v_off[it]);
      if (it == kLoadsK - 1) v_src.advance();
      return;
    }
    it -= kLoadsK;
    if constexpr (HAS_PAD) {
      const uint32_t at = __builtin_amdgcn_readfirstlane(
          (uint32_t)reinterpret_cast<uintptr_t>(pad_lds + pad_at[2] + wave * kWave));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(at), "v"(pad_off), "s"(pad_src.descriptor(tiles)) : "m0");
      pad_src.advance();
    }
  };
  // what the loads issued before the current tile's have to be waited for with
  // (the tile's own stay in flight): vmcnt <= N, nothing else
  auto wait_loads = []<int N>() __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
  };

  f32x16 o[kBlocksD];
#pragma unroll
  for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m = 0.f; // reference maximum of the query's scores, log2 units (the block's first tile sets it)
  float l = 0.f;       // this lane's share of the running sum
  Frag pf[2];          // P^T of the last tile computed, not yet multiplied with V

  // K operand s of the tile at kb: lane (key, half) takes chunk 2 s + half of
  // its key's row, wherever the permutation has put it
  const uint32_t k_lane = (uint32_t)col * kRowBytes + (uint32_t)((half ^ ((col >> kKeyShift) & kSwizzleK)) << 4);
  auto read_k = [&](const T *kb, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const Frag *>(reinterpret_cast<const char *>(kb) + (k_lane ^ (uint32_t)(s << 5)));
  };
  // Operand n of O^T += V^T P^T (the first 16 keys into every block of O^T,
  // then the other 16), through the transposing LDS read: of 16 lanes, lane j
  // points at 8 bytes (4 features) of one key; lane i gets back, of the four
  // words that lanes i/4 + 4k point at, element i % 4 each. With lane j at key
  // j / 4 and feature block j % 4, lane i holds feature i of the four keys:
  // what a lane of the product's A operand needs (its own feature, contraction
  // in its registers). Two reads make an operand: slots 0..3 are keys 16u + 4h +
  // 0..3, slots 4..7 keys 16u + 8 + 4h + 0..3, h the lane's half of the wave:
  // where the accumulator layout leaves the probabilities (rows 8j' + 4h + t of
  // S^T), so that P^T is used where it is.
  typedef short Short4 __attribute__((ext_vector_type(4)));
  uint32_t v_lane[2]; // for even and odd blocks of 32 features
  {
    const int j = lane & 15, group = lane >> 4; // group: bit 0 = second 16 features of the block, bit 1 = half
    const int key = 4 * (group >> 1) + (j >> 2);
    const int x = (2 * (group & 1) + ((j & 3) >> 1)) ^ (2 * (j >> 2) & 3); // chunk within the block of four chunks
    const int flip = (j >> 2) >> 1; // the permutation's bit 2 swaps neighbouring blocks
    const uint32_t base = (uint32_t)key * kRowBytes + (uint32_t)x * 16u + (uint32_t)(j & 1) * 8u;
    v_lane[0] = base + 64u * (uint32_t)flip;
    v_lane[1] = base + 64u * (uint32_t)(1 ^ flip);
  }
  auto read_v = [&](const T *vb, int n) __attribute__((always_inline)) {
    const int u = n / kBlocksD, i = n % kBlocksD;
    const char *at = reinterpret_cast<const char *>(vb) + v_lane[i & 1] + 64 * (i & ~1) + 16 * u * kRowBytes;
    const Short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) Short4 *)(at));
    const Short4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) Short4 *)(at + 8 * kRowBytes));
    return __builtin_bit_cast(Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  // scale and padding mask (without a mask the scores stay raw: the scale,
  // positive, commutes with the maximum and goes into the exponent's
  // multiply-add)
  auto add_pad = [&](f32x16 &sc) __attribute__((always_inline)) {
    if constexpr (HAS_PAD) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 p4 = *reinterpret_cast<const float4 *>(&pad_lds[pad_at[0] + 8 * j + 4 * half]);
        sc[4 * j + 0] = __builtin_fmaf(sc[4 * j + 0], a.scale, fmaxf(p4.x, kMaskFloor));
        sc[4 * j + 1] = __builtin_fmaf(sc[4 * j + 1], a.scale, fmaxf(p4.y, kMaskFloor));
        sc[4 * j + 2] = __builtin_fmaf(sc[4 * j + 2], a.scale, fmaxf(p4.z, kMaskFloor));
        sc[4 * j + 3] = __builtin_fmaf(sc[4 * j + 3], a.scale, fmaxf(p4.w, kMaskFloor));
      }
    }
  };
  // what turns a score as add_pad leaves it into log2 units
  const float to_log2 = HAS_PAD ? kLog2e : a.scale_log2e;
  auto tile_max = [&](const f32x16 &sc) __attribute__((always_inline)) -> float {
    float mt = sc[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mt = fmaxf(mt, sc[r]);
    mt *= to_log2;
    return halves_max(mt);
  };
  auto exponential = [&](float x, float shift) __attribute__((always_inline)) {
    return __builtin_amdgcn_exp2f(__builtin_fmaf(x, to_log2, -shift));
  };
  // attention dropout: the sum keeps every probability, the product with V
  // only the kept ones (their 1/(1-p) goes into the final normalisation);
  // then P^T in the storage type, like the unfused path's cast
  auto finish_probabilities = [&](f32x16 &sc, int keyb, Frag (&p)[2]) __attribute__((always_inline)) {
    if constexpr (DROP) {
      stage_keep_bits(keep_lds, a.drop, bh, S, wave_q0, keyb, lane);
      const uint32_t bits = keep_word_query_lane(keep_lds, col) >> (4 * half);
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = (bits >> (8 * (r >> 2) + (r & 3))) & 1u ? sc[r] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) p[u][i] = static_cast<T>(sc[8 * u + i]);
  };

  // The reference maximum m only follows the scores when they exceed it by
  // more than kSlack (log2 units): exponentials up to 2^kSlack are as exact
  // as those up to 1 in fp32, fp16 and bf16, and the softmax does not depend
  // on the shift. Rescaling O costs as much as the softmax of a tile, and with
  // an exact running maximum some query of a wave raises it in most tiles;
  // with the slack it happens in the first tiles only.

  // A tile in plain order, with the rescaling of O that the scheduled tiles
  // leave out: a scheduled tile whose sum shows that some reference maximum
  // has to rise is done again here (its staging and the products of the tile
  // before it are done). It is kept out of the loops of the scheduled tiles:
  // with the multiplications of O in code that every tile runs through, the
  // compiler copies all of O's accumulators to vector registers in every tile
  // (it places the copies that the rare multiplication needs ahead of the
  // branch).
  auto redo_tile = [&](int t) __attribute__((always_inline)) {
    const int keyb = t * kKeysPerTile;
    f32x16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    {
      const T *kb = k_buffer(0);
#pragma unroll
      for (int s = 0; s < kSteps; ++s) sc = Op::run(read_k(kb, s), qf[s], sc);
    }
    add_pad(sc);
    if (keyb + 31 > wave_q0 || (HAS_WINDOW && keyb <= wave_q0 + 31 - window)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kr = keyb + 8 * (r >> 2) + 4 * half + (r & 3);
        sc[r] = kr <= qrow && (!HAS_WINDOW || kr > behind) ? sc[r] : -INFINITY;
      }
    }
    const float mt = tile_max(sc);
    // (m is finite from the block's first tile on: with a window, the floor
    // that tile leaves for a query that has seen no key yet)
    const bool raise = mt > m + kRaise;
    const float m_new = raise ? mt : m;
    const float alpha = raise ? __builtin_amdgcn_exp2f(m - m_new) : 1.0f; // 0 above the floor (nothing accumulated)
    l *= alpha;
#pragma unroll
    for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = exponential(sc[r], m);
      sum += sc[r];
    }
    l += sum;
    finish_probabilities(sc, keyb, pf);
  };
  // prologue: K of the first two tiles and V of the first on their way, all
  // issued before any is waited for (the sources then stand at tile t + 2 and
  // t + 1, where a tile's staging expects them)
  // The block's queries come first. A lane's operands of Q^T are 16 bytes from
  // each chunk pair of its own row: loaded straight from memory, every lane of
  // a load touches a cache line of its own. The 128 rows go into LDS the way
  // four tiles of K do, whole rows at a time (into the third buffer of K and
  // the three of V, which lie one behind the other and are not in use yet),
  // and each wave reads its tile from there like a tile of K. V of the first
  // tile is loaded once every wave has its operands.
  {
    TileStream q_src;
    q_src.start(qp, (uint32_t)(((int64_t)(S - 1) * a.q_s + D) * sizeof(T)), q_row, kQueriesPerBlock, qb, a.query_blocks);
    const u32x4 qd = q_src.descriptor();
#pragma unroll
    for (int j = 0; j < kQueriesPerBlock / kKeysPerTile; ++j)
#pragma unroll
      for (int it = 0; it < kLoadsK; ++it) {
        const int sigma = (4 * it + wave) * kWave + lane;
        const int row = sigma / kChunks, at = sigma % kChunks;
        load_to_lds(qd, k_lds + (2 + j) * kTile + (4 * it + wave) * (kWave * 8),
                    (uint32_t)(kKeysPerTile * j + row) * q_row + (uint32_t)(at ^ ((row >> kKeyShift) & kSwizzleK)) * 16u);
      }
#pragma unroll
    for (int it = 0; it < kLoadsK; ++it) stage_item(it, k_buffer(0), nullptr);
    if constexpr (HAS_PAD) { // the mask values of the first tile, then (as the staging of a tile expects) of the second
      const int p2 = pad_at[2];
      pad_at[2] = pad_at[0];
      stage_item(kItems - 1, nullptr, nullptr);
      pad_at[2] = pad_at[1];
      stage_item(kItems - 1, nullptr, nullptr);
      pad_at[2] = p2;
    }
#pragma unroll
    for (int it = 0; it < kLoadsK; ++it) stage_item(it, k_buffer(1), nullptr);
    wait_loads.template operator()<0>();
    __syncthreads();
#pragma unroll
    for (int s = 0; s < kSteps; ++s) qf[s] = read_k(k_lds + (2 + wave) * kTile, s);
    __syncthreads(); // (also: K of the first tile is in LDS)
#pragma unroll
    for (int it = kLoadsK; it < 2 * kLoadsK; ++it) stage_item(it, nullptr, v_buffer(0));
  }

  // A tile as one straight run of code, its order fixed by hand (the fences
  // keep the compiler's scheduler from moving anything across them). First the
  // matrix products of S^T (tile t), whose K operands are read from LDS kRing
  // products ahead, with a share of the staging in each product's shadow; then
  // those of O^T (tile t - 1), with a slice of the softmax of tile t in each
  // one's shadow. A wave issues in order, so whatever it issues between two
  // products beyond the seven vector-ALU slots one product lasts leaves the
  // matrix core idle. The run assumes that no reference maximum rises; the
  // caller looks at the tile's maximum `mt` afterwards and, if one has to,
  // throws the tile's probabilities away and does the tile again the general
  // way. MASKED: the causal boundary crosses the tile. FIRST: the block's first
  // tile: nothing is pending, and the tile's maximum becomes the reference.
  auto scheduled_tile = [&]<bool MASKED, bool FIRST>(int t, float &mt, float &sum, Frag (&pn)[2])
                            __attribute__((always_inline)) {
    with_distinct_buffers(k_buffer(0), k_buffer(2), v_buffer(-1), v_buffer(1),
                          [&](const T *kr, T *kw, const T *vr, T *vw) __attribute__((always_inline)) {
      constexpr int kRing = 4;
      constexpr int kProducts = 2 * kBlocksD;
      constexpr int kPerStep = (kItems + kSteps - 1) / kSteps;
      Frag ring[kRing];
#pragma unroll
      for (int s = 0; s < kRing; ++s) ring[s] = read_k(kr, s);
      __builtin_amdgcn_sched_barrier(0);
      f32x16 sc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        sc = Op::run(ring[s % kRing], qf[s], sc);
        const int next = s + kRing;
        if (next < kSteps)
          ring[s % kRing] = read_k(kr, next);
        else if (!FIRST && next - kSteps < kProducts)
          ring[s % kRing] = read_v(vr, next - kSteps);
#pragma unroll
        for (int it = s * kPerStep; it < (s + 1) * kPerStep && it < kItems; ++it) stage_item(it, kw, vw);
        __builtin_amdgcn_sched_barrier(0);
      }
      // softmax slices, spread over the products: the exponentials (an
      // exponential is added to the sum one slice later: the adder would wait
      // for it), the conversion last. Only the first tile takes the maximum;
      // elsewhere the caller looks at the sum (an exponential above 2^kSlack
      // shows there) to see whether a reference maximum has to rise.
      sum = 0.f;
      auto slice_of = [](int r) __attribute__((always_inline)) { return FIRST ? 1 + r * (kProducts - 1) / 16 : r * kProducts / 16; };
#pragma unroll
      for (int n = 0; n < kProducts; ++n) {
        if constexpr (!FIRST) {
          const int at = (kSteps + n) % kRing;
          o[n % kBlocksD] = Op::run(ring[at], pf[n / kBlocksD], o[n % kBlocksD]);
          if (n + kRing < kProducts) ring[at] = read_v(vr, n + kRing);
        }
        if (n == 0) {
          add_pad(sc);
          if constexpr (MASKED) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int kr_ = t * kKeysPerTile + 8 * (r >> 2) + 4 * half + (r & 3);
              sc[r] = kr_ <= qrow && (!HAS_WINDOW || kr_ > behind) ? sc[r] : -INFINITY;
            }
          }
          if constexpr (FIRST) {
            mt = tile_max(sc);
            // With a window a query may see nothing in the first tiles of its
            // wave: its reference then is a floor so far down that the first
            // visible score overflows the tile's sum, which has the tile done
            // again in plain order, where the reference rises to that score.
            m = HAS_WINDOW ? fmaxf(mt, kReferenceFloor) : mt;
          }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (slice_of(r) == n) {
            sc[r] = exponential(sc[r], m);
            // (an empty statement that "changes" a value keeps its computation
            // in this slice: the results are only used behind the branch that
            // follows the tile)
            asm volatile("" : "+v"(sc[r]));
          }
          if (slice_of(r) == n - 1) sum += sc[r];
        }
        if (n == kProducts - 1) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (slice_of(r) == n) sum += sc[r];
          finish_probabilities(sc, t * kKeysPerTile, pn);
          u32x4 p0 = __builtin_bit_cast(u32x4, pn[0]), p1 = __builtin_bit_cast(u32x4, pn[1]);
          asm volatile("" : "+v"(p0), "+v"(p1), "+v"(sum));
          pn[0] = __builtin_bit_cast(Frag, p0), pn[1] = __builtin_bit_cast(Frag, p1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };

  { // the block's first tile (the causal boundary, or the window's edge, may cross it)
    float mt, sum;
    scheduled_tile.template operator()<true, true>(t, mt, sum, pf);
    l = sum;
    next_tile();
  }

  // The tiles the edge of some query's window crosses, those every query of the
  // block sees in full, then those the causal boundary crosses, each kind in a
  // loop of its own (one loop with
  // a branch per kind has the compiler shuffle the accumulators where the
  // branches meet, in every tile). A wave whose queries all lie before a tile
  // still computes it, every score masked: it adds zeros, and it would wait at
  // the tile's barrier anyway.
  auto scheduled_range = [&]<bool MASKED>(int end) __attribute__((always_inline)) {
    while (t < end) {
      bool rescale = false;
      for (; t < end; next_tile()) {
        wait_loads.template operator()<kLoadsPerTile>();
        __syncthreads(); // tile t's K (and tile t - 1's V) are in LDS; the buffers written next have been read
        float mt, sum;
        Frag pn[2];
        scheduled_tile.template operator()<MASKED, false>(t, mt, sum, pn);
        if (__any(!(sum <= kSumLimit))) {
          rescale = true;
          break;
        }
        l += sum;
        pf[0] = pn[0], pf[1] = pn[1];
      }
      if (!rescale) break;
      redo_tile(t);
      next_tile();
    }
  };
  if constexpr (HAS_WINDOW) scheduled_range.template operator()<true>(plain_begin < tiles ? plain_begin : tiles);
  scheduled_range.template operator()<false>(plain_end);
  scheduled_range.template operator()<true>(tiles);

  wait_loads.template operator()<0>(); // (nothing may still be on its way into LDS when the block ends)
  __syncthreads(); // V of the last tile is in LDS
  {
    const T *vb = v_buffer(-1);
#pragma unroll
    for (int n = 0; n < 2 * kBlocksD; ++n) o[n % kBlocksD] = Op::run(read_v(vb, n), pf[n / kBlocksD], o[n % kBlocksD]);
  }

  l = halves_sum(l);
  const float inv = DROP ? a.drop.keep_scale / l : 1.0f / l;
  if (a.lse != nullptr && half == 0 && qrow < S)
    a.lse[(int64_t)bh * S + qrow] = m + __builtin_amdgcn_logf(l); // v_log_f32 is log2
  // O^T leaves through LDS: a lane holds 4 features of its query at a time, and
  // the queries' rows lie far apart in memory; the wave puts its 32 x D tile
  // into LDS (once every wave is done with K and V), rows padded by 16 bytes,
  // and stores whole rows, 16 bytes a lane.
  __syncthreads();
  constexpr int kOutRow = kRowBytes + 16;
  char *const stage = reinterpret_cast<char *>(k_lds) + wave * (32 * kOutRow);
  typedef T Out4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      Out4 w;
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) w[tt] = static_cast<T>(o[i][4 * j + tt] * inv);
      *reinterpret_cast<Out4 *>(stage + col * kOutRow + (32 * i + 8 * j + 4 * half) * (int)sizeof(T)) = w;
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  T *const out_head = static_cast<T *>(a.out) + b * a.o_b + hd * a.o_h;
  constexpr int kRowsPerStore = kWave / kChunks;
#pragma unroll
  for (int k = 0; k < 32 / kRowsPerStore; ++k) {
    const int row = kRowsPerStore * k + lane / kChunks, piece = lane % kChunks;
    const u32x4 w = *reinterpret_cast<const u32x4 *>(stage + row * kOutRow + piece * 16);
    if (wave_q0 + row < S)
      *reinterpret_cast<u32x4 *>(out_head + (int64_t)(wave_q0 + row) * a.o_s + 8 * piece) = w;
  }
}

template <typename T, int D>
int launch_prefill_dim(const PrefillArgs &a, hipStream_t stream) {
  const dim3 grid((unsigned)(8 * a.head_groups * a.query_blocks));
  // All LDS of the kernel is dynamic. At head_dim 256 it exceeds the 64 KiB a
  // kernel gets unasked, so the limit is raised for the kernel (on the current
  // device; a host-side setting, not a stream operation), once.
  constexpr unsigned kDynamic = prefill_lds_bytes<T, D>();
  auto go = [&]<bool HAS_PAD, bool HAS_WINDOW>() -> int {
    auto *kernel = a.drop.drop ? attention_prefill_kernel<T, D, HAS_PAD, HAS_WINDOW, true>
                               : attention_prefill_kernel<T, D, HAS_PAD, HAS_WINDOW, false>;
    if (kDynamic > 64u * 1024u) {
      const int s = raise_lds_limit(reinterpret_cast<const void *>(kernel), kDynamic, "oslo_attention_prefill_fwd");
      if (s != OSLO_OK) return s;
    }
    kernel<<<grid, dim3(kBlockThreads), kDynamic, stream>>>(a);
    return check_launch("attention_prefill_fwd");
  };
  if (a.window > 0) {
    if (a.pad != nullptr) return go.template operator()<true, true>();
    return go.template operator()<false, true>();
  }
  if (a.pad != nullptr) return go.template operator()<true, false>();
  return go.template operator()<false, false>();
}

template <typename T>
int launch_prefill(const PrefillArgs &a, int head_dim, hipStream_t stream) {
  switch (head_dim) {
    case 64: return launch_prefill_dim<T, 64>(a, stream);
    case 128: return launch_prefill_dim<T, 128>(a, stream);
    default: return launch_prefill_dim<T, 256>(a, stream);
  }
}

} // namespace
} // namespace oslo

namespace {
int prefill_entry(void *out, float *lse, const oslo::DropArgs &drop, const void *q,
                  const void *k, const void *v,
                  const float *pad, float scale, int64_t batch, int64_t heads,
                  int64_t S, int64_t head_dim, int64_t window,
                  const int64_t *strides, int dtype, oslo_stream_t stream) {
  using namespace oslo;
  if (batch < 0 || heads < 0 || S < 0 || head_dim < 0 || window < 0)
    return fail(OSLO_E_BAD_ARG, "oslo_attention_prefill_fwd: negative size");
  if (dtype != OSLO_F16 && dtype != OSLO_BF16) {
    if (dtype == OSLO_F32)
      return fail(OSLO_E_UNSUPPORTED, "oslo_attention_prefill_fwd: fp16 and bf16 are taken, not fp32");
    return fail(OSLO_E_BAD_ARG, "unknown dtype %d", dtype);
  }
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_attention_prefill_fwd: heads of %lld features (64, 128 or 256 are taken)",
                (long long)head_dim);
  if (!(scale > 0.0f))
    return fail(OSLO_E_BAD_ARG, "oslo_attention_prefill_fwd: the scale must be positive");
  if (batch == 0 || heads == 0 || S == 0) return OSLO_OK;
  if (!out || !q || !k || !v || !strides)
    return fail(OSLO_E_BAD_ARG, "oslo_attention_prefill_fwd: null pointer");
  if (batch * heads > (int64_t)0x7fffffff / 8)
    return fail(OSLO_E_UNSUPPORTED, "oslo_attention_prefill_fwd: too many heads for one launch");
  const void *ptrs[4] = {q, k, v, out};
  for (int i = 0; i < 4; ++i) {
    if (!aligned16(ptrs[i]))
      return fail(OSLO_E_UNSUPPORTED, "oslo_attention_prefill_fwd: tensors must be 16-byte aligned");
    const int64_t sb = strides[3 * i], sh = strides[3 * i + 1], ss = strides[3 * i + 2];
    if (sb < 0 || sh < 0 || ss < head_dim || sb % 8 || sh % 8 || ss % 8)
      return fail(OSLO_E_UNSUPPORTED,
                  "oslo_attention_prefill_fwd: strides must be multiples of 8 elements, "
                  "the position stride at least head_dim");
    // byte offsets inside one (batch, head) slice are 32-bit
    if ((S + kQueriesPerBlock) * ss * 2 > (int64_t)0x7fffffff)
      return fail(OSLO_E_UNSUPPORTED, "oslo_attention_prefill_fwd: a head's slice exceeds 2 GiB");
  }
  if (pad != nullptr && (S % 4 != 0 || !aligned16(pad)))
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_attention_prefill_fwd: with a padding mask S must be a multiple of 4 and the mask 16-byte aligned");
  PrefillArgs a;
  if (drop.drop && S % 8 != 0)
    return fail(OSLO_E_UNSUPPORTED,
                "oslo_attention_prefill_fwd_lse: with attention dropout S must be a multiple of 8");
  a.out = out, a.q = q, a.k = k, a.v = v, a.pad = pad, a.lse = lse, a.drop = drop;
  a.q_b = strides[0], a.q_h = strides[1], a.q_s = strides[2];
  a.k_b = strides[3], a.k_h = strides[4], a.k_s = strides[5];
  a.v_b = strides[6], a.v_h = strides[7], a.v_s = strides[8];
  a.o_b = strides[9], a.o_h = strides[10], a.o_s = strides[11];
  a.scale = scale;
  a.scale_log2e = scale * kLog2e;
  a.S = (int)S;
  a.heads = (int)heads;
  a.batch_heads = (int)(batch * heads);
  a.head_groups = (a.batch_heads + 7) / 8;
  a.query_blocks = (int)((S + kQueriesPerBlock - 1) / kQueriesPerBlock);
  a.window = window >= S ? 0 : (int)window;
  if ((int64_t)8 * a.head_groups * a.query_blocks > (int64_t)0x7fffffff)
    return fail(OSLO_E_UNSUPPORTED, "oslo_attention_prefill_fwd: too many blocks for one launch");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == OSLO_F16) return launch_prefill<f16>(a, (int)head_dim, st);
  return launch_prefill<bf16>(a, (int)head_dim, st);
}
} // namespace

extern "C" int oslo_attention_prefill_fwd(void *out, const void *q, const void *k,
                                          const void *v, const float *pad,
                                          float scale, int64_t batch, int64_t heads,
                                          int64_t S, int64_t head_dim,
                                          int64_t window,
                                          const int64_t *strides, int dtype,
                                          oslo_stream_t stream) {
  oslo::DropArgs none{};
  return prefill_entry(out, nullptr, none, q, k, v, pad, scale, batch, heads, S, head_dim,
                       window, strides, dtype, stream);
}

extern "C" int oslo_attention_prefill_fwd_lse(void *out, float *lse, const void *q,
                                              const void *k, const void *v,
                                              const float *pad, float scale, float p,
                                              uint64_t philox_seed,
                                              uint64_t philox_offset, int64_t batch,
                                              int64_t heads, int64_t S,
                                              int64_t head_dim, int64_t window,
                                              const int64_t *strides, int dtype,
                                              oslo_stream_t stream) {
  oslo::DropArgs drop;
  const int s = oslo::make_drop_args("oslo_attention_prefill_fwd_lse", p, philox_seed,
                                     philox_offset, &drop);
  if (s != OSLO_OK) return s;
  if (lse == nullptr && batch > 0 && heads > 0 && S > 0)
    return oslo::fail(OSLO_E_BAD_ARG, "oslo_attention_prefill_fwd_lse: null lse");
  return prefill_entry(out, lse, drop, q, k, v, pad, scale, batch, heads, S, head_dim,
                       window, strides, dtype, stream);
}
