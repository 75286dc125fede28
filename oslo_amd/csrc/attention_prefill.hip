// Causal attention over a whole prompt in one kernel (no [S, S] matrix in
// memory):
//   out[q, :] = sum_{k <= q} softmax_k(scale * Q[q, :] . K[k, :] + pad[k]) * V[k, :]
// for every (batch, head), 16-bit inputs, fp32 accumulation. It replaces, for
// inference, the three launches of the fused attention -- batched matmul
// Q K^T, the fused scale + mask + softmax, batched matmul P V
// (oslo/models/gptj/modeling_gptj.py:936-951,
// oslo/models/gpt_neo/modeling_gpt_neo.py:993-1008,
// oslo/models/gpt2/modeling_gpt2.py:1435-1459) -- which write the scores,
// read and write them again in the softmax and read them a fourth time. This
// is the one kernel of the library that is bound by the matrix cores, not by
// HBM: 4 * S^2/2 * head_dim flops per head against 4 * S * head_dim elements.
//
// One block of four waves takes 128 queries of one head, 32 per wave, and walks
// the keys in tiles of 64. Everything is computed transposed, so that a query
// is a lane and not a register index:
//   S^T[key, q] = K_tile (A operand, rows = keys, from LDS) x Q^T (B operand,
//                 held in registers for the whole kernel),
//   O^T[d, q]  += V_tile^T (A operand, rows = features, from LDS) x P^T (B).
// In the accumulator layout of v_mfma_f32_32x32x16 a lane holds one column
// (lane % 32 = the query) and 16 rows, so the running maximum, the sum and
// the rescaling of O are per-lane scalars: the softmax needs one exchange
// between the two halves of the wave per step and no LDS. The 16 rows of a
// lane are keys 8j + 4h + t (j, t = 0..3; h = lane / 32), and a B operand
// wants, per half, 8 consecutive contraction slots: the probabilities are used
// where they are, and the contraction order is permuted instead -- V^T is
// written to LDS with key 8j + 4h + t of each group of 16 (j = 0, 1 there) at
// slot 8h + 4j + t.
// V arrives as [key][feature]; each thread transposes an 8 x 8 block in
// registers and writes 128-bit rows of V^T. Both LDS tiles are swizzled by
// 16-byte chunk so that the 128-bit reads of a wave (the LDS serves 16 lanes
// at a time: 16 rows at one chunk) and the writes spread over the banks. A
// tile of keys is taken in two steps of 32, each a step of the running
// softmax, and the next tile's global loads are in flight meanwhile.

#include "attention.hpp"

namespace oslo {
namespace {

constexpr int kQueriesPerBlock = 128;
constexpr int kKeysPerTile = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kSlack = 8.0f; // see the kernel: how far a score may exceed the reference maximum

struct PrefillArgs {
  void *out;
  const void *q, *k, *v;
  const float *pad; // [batch, S] additive, or null
  float *lse;       // [batch * heads, S] or null: log2 of the row's sum of exponentials
  int64_t q_b, q_h, q_s; // element strides: batch, head, position
  int64_t k_b, k_h, k_s;
  int64_t v_b, v_h, v_s;
  int64_t o_b, o_h, o_s;
  float scale_log2e;
  int S;
  int heads;
  int batch_heads;
  int head_groups; // ceil(batch_heads / 8)
  int query_blocks;
  int window; // 0: every key up to the query; else the last `window` of them
  DropArgs drop; // attention dropout (the DROP variants of the kernel)
};

template <typename T, int D, bool HAS_PAD, bool HAS_WINDOW, bool DROP>
__global__ __launch_bounds__(kBlockThreads, D == 256 ? 1 : 2) void attention_prefill_kernel(
    const PrefillArgs a) {
  using Op = MatrixOp<T>;
  using Frag = typename Op::Frag;
  constexpr int kChunks = D / 8;   // 16-byte chunks of a key
  constexpr int kSteps = D / 16;   // contraction steps of Q K^T
  constexpr int kBlocksD = D / 32; // 32-row blocks of O^T
  constexpr int kLoadsK = kKeysPerTile * kChunks / kBlockThreads; // per thread and tile
  constexpr int kSwizzleK = kChunks >= 16 ? 15 : 7;                // rows over which K's chunks rotate
  // At head_dim 256 the 64 registers of Q^T are what pushes a wave past its
  // 256 vector registers: the compiler then parks half of Q^T in the
  // accumulator file, moves it back before every product and has one buffer
  // left for the K operand, so that every product waits for its own LDS read.
  // There Q^T lives in (dynamic) LDS instead, in operand order, each wave its
  // own 16 KiB, and both operands of S^T = K Q^T are read from LDS.
  constexpr bool kQInLds = D == 256;
  constexpr bool kTwoLoops = D == 256; // see `step` below
  extern __shared__ __align__(16) unsigned char dynamic_lds[];
  __shared__ __align__(16) T k_lds[kKeysPerTile * D];  // [key][chunk ^ (key & kSwizzleK)][8]
  __shared__ __align__(16) T vt_lds[D * kKeysPerTile]; // [d][(slot + d + d/8) & 7][8]
  __shared__ __align__(16) float pad_lds[HAS_PAD ? kKeysPerTile : 4]; // the tile's mask values, log2 units
  __shared__ __align__(16) uint32_t keep_lds[DROP ? kWavesPerBlock : 1][32]; // a wave's keep bits of a step

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;

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
  // rows at or past S fall outside the descriptors and read as zeros
  const BufRsrc qrs = make_rsrc(qp, (uint32_t)(((int64_t)(S - 1) * a.q_s + D) * sizeof(T)));
  const BufRsrc krs = make_rsrc(kp, (uint32_t)(((int64_t)(S - 1) * a.k_s + D) * sizeof(T)));
  const BufRsrc vrs = make_rsrc(vp, (uint32_t)(((int64_t)(S - 1) * a.v_s + D) * sizeof(T)));
  const uint32_t q_row = (uint32_t)a.q_s * sizeof(T);
  const uint32_t k_row = (uint32_t)a.k_s * sizeof(T);
  const uint32_t v_row = (uint32_t)a.v_s * sizeof(T);

  // Q^T as B operands: lane (query, half) holds features 16 s + 8 half .. + 7
  const int wave_q0 = q0 + 32 * wave;
  const int qrow = wave_q0 + col;
  Frag qf[kQInLds ? 1 : kSteps];
  u32x4 *q_lds = reinterpret_cast<u32x4 *>(dynamic_lds) + wave * kSteps * kWave + lane;
  if constexpr (kQInLds) {
    u32x4 tmp[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
      tmp[s] = __builtin_amdgcn_raw_buffer_load_b128(
          qrs, (uint32_t)qrow * q_row + (uint32_t)(16 * s + 8 * half) * sizeof(T), 0, 0);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) q_lds[s * kWave] = tmp[s];
  } else {
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
      qf[s] = __builtin_bit_cast(
          Frag, __builtin_amdgcn_raw_buffer_load_b128(
                    qrs, (uint32_t)qrow * q_row + (uint32_t)(16 * s + 8 * half) * sizeof(T), 0, 0));
  }

  const float *padr = HAS_PAD ? a.pad + (int64_t)b * S : nullptr;
  const int behind = HAS_WINDOW ? qrow - a.window : -1; // the last key behind the query's window

  // A tile travels global -> registers -> LDS; the loads of the next tile are
  // in flight while this one is computed.
  // K: thread takes chunk tid % kChunks of rows tid / kChunks + j * (256 / kChunks).
  // V: a task is 8 keys (one contraction chunk 2u + h of the tile) x 8 features.
  const int k_ch = tid % kChunks, k_r0 = tid / kChunks;
  const bool v_task = tid < D;
  const int v_g = tid % kChunks, v_kg = tid / kChunks;
  u32x4 kreg[kLoadsK], vreg[8];
  // the padding mask of a tile travels with it: 16 lanes take four keys each
  // (keys at or past S read as 0; they only meet queries they are masked for)
  const BufRsrc prs = make_rsrc(padr, HAS_PAD ? (uint32_t)S * (uint32_t)sizeof(float) : 0u);
  float4 padreg = make_float4(0.f, 0.f, 0.f, 0.f);
  auto issue_loads = [&](int key0) {
    if constexpr (HAS_PAD) {
      if (tid < kKeysPerTile / 4)
        padreg = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(
                                                prs, (uint32_t)(key0 + 4 * tid) * (uint32_t)sizeof(float), 0, 0));
    }
#pragma unroll
    for (int j = 0; j < kLoadsK; ++j)
      kreg[j] = __builtin_amdgcn_raw_buffer_load_b128(
          krs, (uint32_t)(key0 + k_r0 + j * (kBlockThreads / kChunks)) * k_row + (uint32_t)k_ch * 16u, 0, 0);
    if (v_task) {
      const int kbase = key0 + 16 * (v_kg >> 1) + 4 * (v_kg & 1);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        vreg[i] = __builtin_amdgcn_raw_buffer_load_b128(
            vrs, (uint32_t)(kbase + 8 * (i >> 2) + (i & 3)) * v_row + (uint32_t)v_g * 16u, 0, 0);
    }
  };
  auto store_tile = [&]() {
    if constexpr (HAS_PAD) {
      if (tid < kKeysPerTile / 4)
        *reinterpret_cast<float4 *>(&pad_lds[4 * tid]) = make_float4(
            fmaxf(padreg.x * kLog2e, kMaskFloorLog2), fmaxf(padreg.y * kLog2e, kMaskFloorLog2),
            fmaxf(padreg.z * kLog2e, kMaskFloorLog2), fmaxf(padreg.w * kLog2e, kMaskFloorLog2));
    }
#pragma unroll
    for (int j = 0; j < kLoadsK; ++j) {
      const int row = k_r0 + j * (kBlockThreads / kChunks);
      *reinterpret_cast<u32x4 *>(&k_lds[(row * kChunks + (k_ch ^ (row & kSwizzleK))) * 8]) = kreg[j];
    }
    if (v_task) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { // 8 x 8 transposition of 16-bit values
        u32x4 tr;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t lo = vreg[2 * w][e >> 1], hi = vreg[2 * w + 1][e >> 1];
          tr[w] = (e & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
        }
        const int d = 8 * v_g + e;
        *reinterpret_cast<u32x4 *>(&vt_lds[(d * 8 + ((v_kg + e + v_g) & 7)) * 8]) = tr;
      }
    }
  };

  f32x16 o[kBlocksD];
#pragma unroll
  for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m = -INFINITY; // running maximum of the query's scores, log2 units
  float l = 0.f;       // this lane's share of the running sum

  const int last_key = (q0 + kQueriesPerBlock < S ? q0 + kQueriesPerBlock : S) - 1;
  const int tiles = last_key / kKeysPerTile + 1;
  // with a sliding window the block starts at the tile of its first query's
  // first visible key
  const int window = HAS_WINDOW ? a.window : 0;
  const int first_tile = HAS_WINDOW && q0 - window + 1 > 0 ? (q0 - window + 1) / kKeysPerTile : 0;
  // One step of 32 keys of the tile in LDS. RESCALE: O may be rescaled to a
  // higher reference maximum. The loop over the tiles runs the variant without
  // it and falls back, for a single step, when a query that has already
  // accumulated something needs a higher reference: with the multiplications
  // of O in the same loop, the compiler copies all of O's accumulators to
  // vector registers in every tile (it places the copies that the rare
  // multiplication needs ahead of the branch), 128 moves and 128 registers at
  // head_dim 256. Returns false if nothing was done for that reason.
  auto step = [&]<bool RESCALE>(int key0, int kb) -> bool {
    const int keyb = key0 + 32 * kb;
    if (keyb > wave_q0 + 31) return true; // every key is ahead of the wave's queries
    if (HAS_WINDOW && keyb + 31 <= wave_q0 - window) return true; // or behind their windows

    // S^T = K Q^T
    f32x16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    const int key = 32 * kb + col;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const Frag kf = *reinterpret_cast<const Frag *>(
          &k_lds[(key * kChunks + ((2 * s + half) ^ (key & kSwizzleK))) * 8]);
      if constexpr (kQInLds)
        sc = Op::run(kf, __builtin_bit_cast(Frag, q_lds[s * kWave]), sc);
      else
        sc = Op::run(kf, qf[s], sc);
    }
    // The LDS reads run kAhead steps ahead of the products that use them (left
    // alone, the scheduler keeps one operand buffer and every product waits
    // out its own read). 0x100: LDS reads, 0x008: matrix products.
    {
      constexpr int kReads = kQInLds ? 2 : 1; // per step
      constexpr int kAhead = kSteps < 3 ? kSteps : 3;
      __builtin_amdgcn_sched_group_barrier(0x100, kReads * kAhead, 0);
#pragma unroll
      for (int s = 0; s < kSteps - kAhead; ++s) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    }

    // Causal and padding mask, maximum. Without a padding mask the scores
    // stay raw: the scale (positive) commutes with the maximum and goes
    // into the exponent's multiply-add.
    const bool diagonal = keyb + 31 > wave_q0 || (HAS_WINDOW && keyb <= wave_q0 + 31 - window);
    float mt = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float pv[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (HAS_PAD) {
        const float4 p4 = *reinterpret_cast<const float4 *>(&pad_lds[32 * kb + 8 * j + 4 * half]);
        pv[0] = p4.x, pv[1] = p4.y, pv[2] = p4.z, pv[3] = p4.w;
      }
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        float x = sc[4 * j + tt];
        if constexpr (HAS_PAD) x = __builtin_fmaf(x, a.scale_log2e, pv[tt]);
        sc[4 * j + tt] = x;
      }
    }
    if (diagonal) {
      // a branch of its own (the empty asm keeps it one): the comparisons
      // run in the last tiles of a block only
      asm volatile("");
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kr = keyb + 8 * (r >> 2) + 4 * half + (r & 3);
        sc[r] = kr <= qrow && (!HAS_WINDOW || kr > behind) ? sc[r] : -INFINITY;
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) mt = fmaxf(mt, sc[r]);
    if constexpr (!HAS_PAD) mt *= a.scale_log2e;
    mt = fmaxf(mt, other_half(mt));
    // The reference maximum m only follows the scores when they exceed it by
    // more than kSlack (log2 units): exponentials up to 2^kSlack are as exact
    // as those up to 1 in fp32, fp16 and bf16, and the softmax does not
    // depend on the shift. Rescaling O costs as much as the softmax of a
    // step, and with an exact running maximum some query of a wave raises it
    // in most steps; with the slack it happens in the first steps only.
    // Without a window key 0 is visible to every query and m is finite
    // after the first step; with one, a query may see nothing in the first
    // steps of its wave: m stays -inf, nothing is rescaled, and the
    // exponentials (of -inf) are taken against 0.
    const bool raise = mt > m + kSlack; // true at the first visible key (m = -inf)
    if constexpr (RESCALE) {
      if (__any(raise)) { // wave-uniform
        const float m_new = raise ? mt : m;
        const float alpha = !HAS_WINDOW || raise ? __builtin_amdgcn_exp2f(m - m_new) : 1.0f;
        m = m_new;
        l *= alpha;
#pragma unroll
        for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
      }
    } else {
      // a query that has accumulated nothing yet (m = -inf) takes its
      // reference maximum without rescaling anything; any other raise is
      // left to the caller's slow path, before this step has changed anything
      if (__any(raise && m != -INFINITY)) return false;
      m = raise ? mt : m;
    }
    float sum = 0.f;
    const float shift = HAS_WINDOW && m == -INFINITY ? 0.f : m;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if constexpr (HAS_PAD)
        sc[r] = __builtin_amdgcn_exp2f(sc[r] - shift);
      else
        sc[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[r], a.scale_log2e, -shift));
      sum += sc[r];
    }
    l += sum;
    if constexpr (DROP) {
      // attention dropout: the sum keeps every probability, the product with V
      // only the kept ones (their 1/(1-p) goes into the final normalisation)
      stage_keep_bits(keep_lds[wave], a.drop, bh, S, wave_q0, keyb, lane);
      const uint32_t bits = keep_word_query_lane(keep_lds[wave], col) >> (4 * half);
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = (bits >> (8 * (r >> 2) + (r & 3))) & 1u ? sc[r] : 0.f;
    }

    // P^T as B operands, in the storage type like the unfused path's cast
    Frag pf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[u][i] = static_cast<T>(sc[8 * u + i]);

    // O^T += V^T P^T, the first 16 keys into every block of O^T, then the
    // other 16: the products of the first half only need the first half of
    // the exponentials
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int i = 0; i < kBlocksD; ++i) {
        const int d = 32 * i + col;
        const Frag vf = *reinterpret_cast<const Frag *>(
            &vt_lds[(d * 8 + ((4 * kb + 2 * u + half + d + (d >> 3)) & 7)) * 8]);
        o[i] = Op::run(vf, pf[u], o[i]);
      }
    }
    {
      constexpr int kProducts = 2 * kBlocksD;
      constexpr int kAhead = kProducts < 3 ? kProducts : 3;
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 1);
#pragma unroll
      for (int n = 0; n < kProducts - kAhead; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 1);
    }
    return true;
  };

  issue_loads(first_tile * kKeysPerTile);
  int t = first_tile;
  if constexpr (!kTwoLoops) {
    for (; t < tiles; ++t) {
      const int key0 = t * kKeysPerTile;
      __syncthreads(); // the reads of the previous tile are done
      store_tile();
      __syncthreads();
      if (t + 1 < tiles) issue_loads(key0 + kKeysPerTile);
      step.template operator()<true>(key0, 0);
      step.template operator()<true>(key0, 1);
    }
  }
  while (kTwoLoops && t < tiles) {
    int redo = -1; // the step of tile t that needs the rescaling variant
    for (; t < tiles; ++t) {
      const int key0 = t * kKeysPerTile;
      __syncthreads(); // the reads of the previous tile are done
      store_tile();
      __syncthreads();
      if (t + 1 < tiles) issue_loads(key0 + kKeysPerTile);
      if (!step.template operator()<false>(key0, 0)) {
        redo = 0;
        break;
      }
      if (!step.template operator()<false>(key0, 1)) {
        redo = 1;
        break;
      }
    }
    if (redo < 0) break;
#pragma unroll 1
    for (int kb = redo; kb < 2; ++kb) step.template operator()<true>(t * kKeysPerTile, kb);
    ++t;
  }

  l += other_half(l);
  const float inv = DROP ? a.drop.keep_scale / l : 1.0f / l;
  if (qrow >= S) return;
  if (a.lse != nullptr && half == 0)
    a.lse[(int64_t)bh * S + qrow] = m + __builtin_amdgcn_logf(l); // v_log_f32 is log2
  T *op = static_cast<T *>(a.out) + b * a.o_b + hd * a.o_h + (int64_t)qrow * a.o_s;
  typedef T Out4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int i = 0; i < kBlocksD; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      Out4 w;
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) w[tt] = static_cast<T>(o[i][4 * j + tt] * inv);
      *reinterpret_cast<Out4 *>(op + 32 * i + 8 * j + 4 * half) = w;
    }
}

template <typename T, int D>
int launch_prefill_dim(const PrefillArgs &a, hipStream_t stream) {
  const dim3 grid((unsigned)(8 * a.head_groups * a.query_blocks));
  // head_dim 256 keeps Q^T in dynamic LDS: 128 queries x 256 features. Static
  // and dynamic LDS together exceed the 64 KiB a kernel gets unasked, so the
  // limit is raised for the kernel (on the current device; a host-side
  // setting, not a stream operation) before every launch.
  constexpr unsigned kDynamic = D == 256 ? kQueriesPerBlock * D * sizeof(T) : 0;
  auto go = [&]<bool HAS_PAD, bool HAS_WINDOW>() -> int {
    auto *kernel = a.drop.drop ? attention_prefill_kernel<T, D, HAS_PAD, HAS_WINDOW, true>
                               : attention_prefill_kernel<T, D, HAS_PAD, HAS_WINDOW, false>;
    if (kDynamic > 0) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynamic);
      if (e != hipSuccess)
        return fail(OSLO_E_LAUNCH, "oslo_attention_prefill_fwd: %u bytes of dynamic LDS refused: %s",
                    kDynamic, hipGetErrorString(e));
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
