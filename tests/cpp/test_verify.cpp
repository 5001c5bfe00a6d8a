// CPU-only test of the host-side checks in vrank/allreduce.hpp (verifyAllReduce,
// verifyAllgather, verifyTransmit <- allreduce.cpp:519-585, 832-838) and of the
// element arithmetic they rest on.  The oracle is linked as the checker.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "vr_oracle.h"
#include "vrank/allreduce.hpp"

static int failures = 0;
#define EXPECT(c)                                                    \
  do {                                                               \
    if (!(c)) {                                                      \
      ++failures;                                                    \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);     \
    }                                                                \
  } while (0)

typedef unsigned short half_bits;

int main() {
  using namespace vrank;
  // 1. every binary16 pattern survives half -> float -> half, and agrees with the oracle's conversion
  size_t bad = 0;
  for (unsigned h = 0; h < 65536; ++h) {
    const float f = detail::half_bits_to_float((uint16_t)h);
    const float g = vro_f16_to_f32((uint16_t)h);
    if (f != g && !(f != f && g != g)) ++bad;
    const uint16_t back = detail::float_to_half_bits(f);
    if (back != h && !((h & 0x7c00) == 0x7c00 && (h & 0x3ff))) ++bad;
  }
  EXPECT(bad == 0);
  // 2. the element add against the oracle's integer-only add: every pair over a
  //    stratified operand set (all exponents and signs, edge significands), plus
  //    16M seeded random pairs
  std::vector<uint16_t> ops;
  for (unsigned s = 0; s < 2; ++s)
    for (unsigned e = 0; e < 32; ++e)
      for (unsigned m : {0u, 1u, 2u, 3u, 0x1ffu, 0x200u, 0x201u, 0x2aau, 0x3feu, 0x3ffu})
        ops.push_back((uint16_t)((s << 15) | (e << 10) | m));
  bad = 0;
  for (uint16_t a : ops)
    for (uint16_t b : ops)
      if (!vro_f16_same(detail::elem_add(VR_DTYPE_F16, a, b), vro_f16_add_soft(a, b))) ++bad;
  EXPECT(bad == 0);
  uint64_t z = 0x1234567;
  bad = 0;
  for (int i = 0; i < (1 << 24); ++i) {
    z = z * 6364136223846793005ull + 1442695040888963407ull;
    const uint16_t a = (uint16_t)(z >> 20), b = (uint16_t)(z >> 40);
    if (!vro_f16_same(detail::elem_add(VR_DTYPE_F16, a, b), vro_f16_add_soft(a, b))) ++bad;
    const uint16_t x = detail::elem_add(VR_DTYPE_BF16, a, b), y = vro_bf16_add(a, b);
    const bool xnan = (x & 0x7f80) == 0x7f80 && (x & 0x7f), ynan = (y & 0x7f80) == 0x7f80 && (y & 0x7f);
    if (x != y && !(xnan && ynan)) ++bad;
  }
  EXPECT(bad == 0);
  // hand cases: ties to even, overflow
  EXPECT(detail::elem_add(VR_DTYPE_F16, 0x6800 /*2048*/, 0x3c00 /*1*/) == 0x6800);
  EXPECT(detail::elem_add(VR_DTYPE_F16, 0x6800 /*2048*/, 0x4200 /*3*/) == 0x6802 /*2052*/);
  EXPECT(detail::elem_add(VR_DTYPE_F16, 0x7bff /*65504*/, 0x4b80 /*15*/) == 0x7bff);
  EXPECT(detail::elem_add(VR_DTYPE_F16, 0x7bff /*65504*/, 0x4c00 /*16*/) == 0x7c00);

  // 3. verifyAllReduce / verifyTransmit: the closed form (i % 32) * N (N + 1) / 2 passes; a
  //    flipped element is counted and printed; the return value is 0 either way
  for (int world : {2, 4, 8}) {
    const size_t n = 1920;
    std::vector<half_bits> good(n);
    for (size_t i = 0; i < n; ++i) good[i] = vro_f32_to_f16((float)((i % 32) * world * (world + 1) / 2));
    size_t miss = 99;
    EXPECT(verifyAllReduce<half_bits>(good.data(), 0, world, n, &miss) == 0 && miss == 0);
    EXPECT(verifyTransmit<half_bits>(nullptr, good.data(), 1, 0, world, 16, n, &miss) == 0 && miss == 0);
    good[77] ^= 1;
    good[1000] ^= 0x8000;
    EXPECT(verifyAllReduce<half_bits>(good.data(), 3, world, n, &miss) == 0 && miss == (world == 2 ? 2u : 2u));
    // all-gather: the concatenated patterns
    std::vector<half_bits> cat(n * world);
    for (int r = 0; r < world; ++r) vro_fill_pattern(cat.data() + (size_t)r * n, r, n);
    EXPECT(verifyAllgather<half_bits>(cat.data(), 1, world, n, &miss) == 0 && miss == 0);
    cat[n * world - 1] ^= 4;
    EXPECT(verifyAllgather<half_bits>(cat.data(), 1, world, n, &miss) == 0 && miss == 1);
  }
  // bfloat16: the reference's host sum is a rank-order chain in the element type; the
  // oracle's rank-order mode must agree with it on fill_pattern for 8 ranks (where
  // partial sums no longer fit 8 bits and the order matters)
  {
    const int world = 8;
    const size_t n = 512;
    std::vector<std::vector<uint16_t>> in(world, std::vector<uint16_t>(n));
    const uint16_t *ptrs[8];
    for (int r = 0; r < world; ++r) {
      vro_fill_pattern_dt(1, in[r].data(), r, n);
      ptrs[r] = in[r].data();
    }
    std::vector<uint16_t> want(n);
    EXPECT(vro_allreduce_order_dt(1, 0 /* rank order */, want.data(), ptrs, world, n) == 0);
    std::vector<bfloat16> host(n);
    for (size_t i = 0; i < n; ++i) host[i].bits = want[i];
    size_t miss = 99;
    EXPECT(verifyAllReduce<bfloat16>(host.data(), 0, world, n, &miss) == 0 && miss == 0);
  }
  std::printf("%s (%d failures)\n", failures ? "verify FAILED" : "verify ok", failures);
  return failures ? 1 : 0;
}
