// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
// SC'11) as a pure function of (key, counter). Usable from host and device
// code; the dropout kernels and the host-side checks share this one text.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define OSLO_HD __host__ __device__ __forceinline__
#else
#define OSLO_HD inline
#endif

namespace oslo {

struct Philox4 {
  uint32_t w[4];
};

// key = (seed low, seed high); counter = (c0, c1, c2, c3).
OSLO_HD Philox4 philox4x32_10(uint32_t k0, uint32_t k1, uint32_t c0,
                              uint32_t c1, uint32_t c2, uint32_t c3) {
  constexpr uint32_t kM0 = 0xD2511F53u, kM1 = 0xCD9E8D57u;
  constexpr uint32_t kW0 = 0x9E3779B9u, kW1 = 0xBB67AE85u;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)kM0 * c0;
    const uint64_t p1 = (uint64_t)kM1 * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += kW0;
    k1 += kW1;
  }
  return Philox4{{c0, c1, c2, c3}};
}

// Dropout draw for a group of eight consecutive elements: key = seed,
// counter = (offset/4 as 64 bits, group index as 64 bits). The generator
// offset counts 32-bit words, a counter step yields four of them. The four
// words equal the first four outputs of
// at::Philox4_32(seed, /*subsequence=*/group, /*offset=*/offset/4) from
// ATen/core/PhiloxRNGEngine.h. Element e (0..7) of the group owns 16 of the
// 128 bits: the low half of word e/2 when e is even, the high half when odd.
// Ten Philox rounds cost about as much issue time as the memory traffic of
// eight 16-bit elements, so a draw is shared by eight elements, not four.
OSLO_HD Philox4 dropout_draw(uint64_t seed, uint64_t offset, uint64_t group) {
  const uint64_t block = offset >> 2;
  return philox4x32_10((uint32_t)seed, (uint32_t)(seed >> 32), (uint32_t)block,
                       (uint32_t)(block >> 32), (uint32_t)group,
                       (uint32_t)(group >> 32));
}

OSLO_HD uint32_t dropout_bits(const Philox4 &d, int e) {
  return (d.w[e >> 1] >> ((e & 1) * 16)) & 0xFFFFu;
}

// keep = bits >= threshold, threshold = floor(p * 2^16): P(drop) = threshold/2^16
// (p is quantised to a multiple of 2^-16).
OSLO_HD uint32_t dropout_threshold(float p) {
  const double t = (double)p * 65536.0;
  return t >= 65535.0 ? 0xFFFFu : (uint32_t)t;
}

} // namespace oslo
