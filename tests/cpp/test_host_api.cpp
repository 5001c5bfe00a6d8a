// Exercises the C++ host API (vrank/allreduce.hpp) the way a program written
// against the reference's AllReduce / bisectPAllReduce / AllGather templates
// would, and checks every result bit for bit against the CPU oracle.
#include <stdio.h>
#include <string.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "vr_oracle.h"
#include "vrank/allreduce.hpp"

using namespace vrank;
typedef uint16_t half_bits;   // T: any 2-byte type

static int failures = 0;
#define EXPECT(cond)                                                    \
  do {                                                                  \
    if (!(cond)) {                                                      \
      printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);            \
      ++failures;                                                       \
    }                                                                   \
  } while (0)

struct Ranks {
  int n;
  size_t nelems;
  std::vector<std::vector<half_bits>> host;
  std::vector<half_bits *> dev;
  Ranks(int n, size_t nelems, uint64_t seed, size_t out_mult = 1) : n(n), nelems(nelems), host(n), dev(n) {
    for (int r = 0; r < n; ++r) {
      host[r].resize(nelems);
      vro_generate(host[r].data(), nelems, seed + r, VRO_DIST_NORMAL, 0.0, 1.0);
      void *p;
      check(vr_malloc(0, nelems * 2 * out_mult, &p));
      dev[r] = (half_bits *)p;
      check(vr_copy_to_device(p, host[r].data(), nelems * 2));
    }
  }
  ~Ranks() { for (auto p : dev) vr_free(p); }
  std::vector<const uint16_t *> host_ptrs() const {
    std::vector<const uint16_t *> v;
    for (auto &h : host) v.push_back(h.data());
    return v;
  }
  size_t mismatches(const std::vector<uint16_t> &want) const {
    size_t bad = 0;
    std::vector<uint16_t> got(want.size());
    for (int r = 0; r < n; ++r) {
      check(vr_copy_to_host(got.data(), dev[r], want.size() * 2));
      bad += vro_count_mismatch(got.data(), want.data(), want.size());
    }
    return bad;
  }
};

template <typename F>
static std::string thrown(F &&f) {
  try { f(); } catch (const std::logic_error &e) { return e.what(); } catch (const std::exception &e) { return std::string("other: ") + e.what(); }
  return "";
}

static int run_all() {
  // --- AllReduce<T, 8, Rt64_128, ParallelTransmit>: construct, then call ----------------------
  {
    VirtualRanks ranks(8);
    Ranks b(8, 8 * 4096 + 8 * 4 * 3, 11);
    std::vector<uint16_t> want(b.nelems);
    auto hp = b.host_ptrs();
    vro_allreduce_rotated(want.data(), hp.data(), 8, b.nelems);
    AllReduce<half_bits, 8, Rt64_128, ParallelTransmit> ar(ranks, b.dev.data(), b.nelems, 7);
    uint32_t step = 7;
    LaunchParam lp = ar.getLaunchParam(step);
    EXPECT(lp.subgroups == 64 && lp.simd == 16 && step > 7);
    ar();
    ranks.wait();
    EXPECT(b.mismatches(want) == 0);
    EXPECT(ar.workSize() == b.nelems * 2 / 8);
  }
  // --- static launch with a running step counter (allreduce.hpp:64-74) ---------------------------
  {
    VirtualRanks ranks(4);
    Ranks b(4, 4 * 1000, 21);
    std::vector<uint16_t> want(b.nelems);
    auto hp = b.host_ptrs();
    vro_allreduce_rotated(want.data(), hp.data(), 4, b.nelems);
    uint32_t step = 100;
    AllReduce<half_bits, 4, Rt64, ParallelTransmit>::launch(ranks, b.dev.data(), b.nelems, step);
    ranks.wait();
    EXPECT(step > 100);
    EXPECT(b.mismatches(want) == 0);
  }
  // --- ring and sequential transmits share the rotated order --------------------------------------
  {
    VirtualRanks ranks(8);
    Ranks b(8, 8 * 8 * 777, 31), c(8, 8 * 8 * 777, 31);
    std::vector<uint16_t> want(b.nelems);
    auto hp = b.host_ptrs();
    vro_allreduce_rotated(want.data(), hp.data(), 8, b.nelems);
    uint32_t step = 1;
    AllReduce<half_bits, 8, Rt64_128_PCIE, RingTransmit>::launch(ranks, b.dev.data(), b.nelems, step);
    AllReduce<half_bits, 8, Rt64_PCIE, SequentialTransmit>::launch(ranks, c.dev.data(), c.nelems, step);
    ranks.wait();
    EXPECT(b.mismatches(want) == 0);
    EXPECT(c.mismatches(want) == 0);
  }
  // --- bisectPAllReduce<T, 8> --------------------------------------------------------------------
  {
    VirtualRanks ranks(8);
    Ranks b(8, 8 * 4 * 12345, 41);
    std::vector<uint16_t> want(b.nelems), rot(b.nelems);
    auto hp = b.host_ptrs();
    vro_allreduce_bisect(want.data(), hp.data(), 8, b.nelems);
    vro_allreduce_rotated(rot.data(), hp.data(), 8, b.nelems);
    EXPECT(vro_count_mismatch(want.data(), rot.data(), b.nelems) > 0);
    bisectPAllReduce<half_bits, 8> ar(ranks, b.dev.data(), b.nelems, 3);
    ar();
    ranks.wait();
    EXPECT(b.mismatches(want) == 0);
  }
  // --- AllGather<T, 4, Rt64_128_PCIE, RingTransmit>, out of place ------------------------------------
  {
    VirtualRanks ranks(4);
    Ranks in(4, 8 * 999, 51), out(4, 8 * 999, 52, 4);
    std::vector<uint16_t> want(4 * in.nelems);
    auto hp = in.host_ptrs();
    vro_allgather(want.data(), hp.data(), 4, in.nelems);
    uint32_t step = 9;
    AllGather<half_bits, 4, Rt64_128_PCIE, RingTransmit>::launch(ranks, in.dev.data(), out.dev.data(),
                                                                 in.nelems, step);
    ranks.wait();
    EXPECT(out.mismatches(want) == 0);
  }
  // --- string dispatch with a user grid, like main.cpp + testTransmit ---------------------------------
  {
    VirtualRanks ranks(8);
    for (const char *algo : {"small", "simple", "bisect", "small_ring", "simple_pcie"}) {
      Ranks b(8, 14336, 61);
      std::vector<uint16_t> want(b.nelems);
      auto hp = b.host_ptrs();
      if (std::string(algo) == "bisect") vro_allreduce_bisect(want.data(), hp.data(), 8, b.nelems);
      else vro_allreduce_rotated(want.data(), hp.data(), 8, b.nelems);
      testTransmit<half_bits>(algo, {13, 8, 16}, ranks, b.dev.data(), b.nelems, 0xe00f100f);
      ranks.wait();
      EXPECT(b.mismatches(want) == 0);
    }
  }
  // --- testAllgather with a user grid, both transports, then the reference's host checks --------------
  {
    VirtualRanks ranks(4);
    ranks.reserveWire();
    for (int transport : {VR_TRANSPORT_DIRECT, VR_TRANSPORT_WIRE}) {
      ranks.setTransport(transport);
      uint32_t step = 0xe00f100f;
      for (const char *algo : {"allgather_small", "allgather_simple"}) {
        for (LaunchParam grid : {LaunchParam{1, 4, 16}, LaunchParam{7, 8, 16}, LaunchParam{19, 32, 32}}) {
          Ranks in(4, 8 * 1237, 53), out(4, 8 * 1237, 54, 4);
          std::vector<uint16_t> want(4 * in.nelems);
          auto hp = in.host_ptrs();
          vro_allgather(want.data(), hp.data(), 4, in.nelems);
          testAllgather<half_bits>(algo, grid, ranks, in.dev.data(), out.dev.data(), in.nelems, step);
          ranks.wait();
          step += 100;
          EXPECT(out.mismatches(want) == 0);
        }
      }
    }
    ranks.setTransport(VR_TRANSPORT_DEFAULT);
    EXPECT(thrown([&] { Ranks in(4, 64, 1), out(4, 64, 2, 4);
                        testAllgather<half_bits>("small", {1, 4, 16}, ranks, in.dev.data(), out.dev.data(), in.nelems, 1); }) ==
           "Transmit type not support");
    EXPECT(thrown([&] { Ranks in(4, 64, 1), out(4, 64, 2, 4);
                        testAllgather<half_bits>("allgather_small", {1, 2, 16}, ranks, in.dev.data(), out.dev.data(), in.nelems, 1); }) ==
           "Subgroup numbers must be multiple of 4");
  }
  // --- verifyTransmit / verifyAllgather on what the device produced from fill_pattern (main.cpp -v) ----
  {
    const int W = 8;
    const size_t n = 14336;
    VirtualRanks ranks(W);
    std::vector<half_bits *> dev(W), gathered(W);
    std::vector<uint16_t> host(n);
    for (int r = 0; r < W; ++r) {
      void *p;
      check(vr_malloc(0, n * 2, &p));
      dev[r] = (half_bits *)p;
      check(vr_malloc(0, n * 2 * W, &p));
      gathered[r] = (half_bits *)p;
      check(vr_memset(p, 1, n * 2 * W));
      vr_fill_pattern(host.data(), r, n);
      check(vr_copy_to_device(dev[r], host.data(), n * 2));
    }
    testAllgather<half_bits>("allgather_simple", {7, 8, 16}, ranks, dev.data(), gathered.data(), n, 5);
    ranks.wait();
    testTransmit<half_bits>("bisect", {13, 8, 16}, ranks, dev.data(), n, 0xe00f100f);
    ranks.wait();
    std::vector<half_bits> got(n), cat(n * W);
    for (int r = 0; r < W; ++r) {
      size_t bad = 99;
      check(vr_copy_to_host(got.data(), dev[r], n * 2));
      EXPECT(verifyTransmit<half_bits>(nullptr, got.data(), 0xe00f100f, r, W, 16, n, &bad) == 0 && bad == 0);
      check(vr_copy_to_host(cat.data(), gathered[r], n * 2 * W));
      EXPECT(verifyAllgather<half_bits>(cat.data(), r, W, n, &bad) == 0 && bad == 0);
      vr_free(dev[r]);
      vr_free(gathered[r]);
    }
  }
  // --- bfloat16 through the same templates -----------------------------------------------------------
  {
    VirtualRanks ranks(8);
    const size_t n = 8 * 4 * 777;
    std::vector<std::vector<uint16_t>> host(8, std::vector<uint16_t>(n));
    std::vector<bfloat16 *> dev(8);
    std::vector<const uint16_t *> hp;
    for (int r = 0; r < 8; ++r) {
      vro_generate_dt(VRO_BF16, host[r].data(), n, 91 + r, VRO_DIST_NORMAL, 0.0, 1.0);
      void *p;
      check(vr_malloc(0, n * 2, &p));
      dev[r] = (bfloat16 *)p;
      check(vr_copy_to_device(p, host[r].data(), n * 2));
      hp.push_back(host[r].data());
    }
    std::vector<uint16_t> want(n), got(n);
    vro_allreduce_order_dt(VRO_BF16, 2, want.data(), hp.data(), 8, n);
    uint32_t step = 5;
    bisectPAllReduce<bfloat16, 8>::launch(ranks, dev.data(), n, step);
    ranks.wait();
    for (int r = 0; r < 8; ++r) {
      check(vr_copy_to_host(got.data(), dev[r], n * 2));
      EXPECT(memcmp(got.data(), want.data(), n * 2) == 0);
      vr_free(dev[r]);
    }
    ranks.setDtype(VR_DTYPE_F16);
  }
  // --- one rank per object: the reference's own constructor / launch / testTransmit lists -------------
  // (allreduce.hpp:18-28, 64-74, 337-343; allgather.hpp:19-29): N launches on N streams of
  // this process against scratch the caller owns (main.cpp:241-269).
  {
    const int W = 4;
    void *streams[W] = {nullptr, nullptr, nullptr, nullptr};
    for (int r = 1; r < W; ++r) check(vr_stream_create(0, &streams[r]));
    const size_t sink = scratchBytes(W) / 2;
    half_bits *ipcbuf0[W], *ipcbuf1[W];            // peerbuf0[i], peerbuf1[i] of main.cpp:260-269
    for (int r = 0; r < W; ++r) {
      void *p;
      check(vr_malloc(0, 2 * sink, &p));
      ipcbuf0[r] = (half_bits *)p;
      ipcbuf1[r] = (half_bits *)((char *)p + sink);
    }
    auto zero = [&] { for (int r = 0; r < W; ++r) check(vr_memset(ipcbuf0[r], 0, 2 * sink)); };
    auto wait_all = [&] { for (int r = 0; r < W; ++r) AllReduce<half_bits, W, Rt64_128, ParallelTransmit>::wait(streams[r]); };
    uint32_t step = 0xe00f100f;
    {  // AllReduce<...>::launch per rank
      zero();
      Ranks b(W, W * 4 * 5001, 81);
      std::vector<uint16_t> want(b.nelems);
      auto hp = b.host_ptrs();
      vro_allreduce_rotated(want.data(), hp.data(), W, b.nelems);
      uint32_t next = step;
      for (int r = 0; r < W; ++r) {
        next = step;
        AllReduce<half_bits, W, Rt64_128, ParallelTransmit>::launch(b.dev[r], ipcbuf0[r], ipcbuf1[r], ipcbuf0,
                                                                    ipcbuf1, b.nelems, r, next, streams[r]);
      }
      wait_all();
      EXPECT(next > step);
      step = next;
      EXPECT(b.mismatches(want) == 0);
    }
    {  // bisectPAllReduce constructed per rank, then called
      zero();
      Ranks b(W, W * 4 * 3333, 82);
      std::vector<uint16_t> want(b.nelems);
      auto hp = b.host_ptrs();
      vro_allreduce_bisect(want.data(), hp.data(), W, b.nelems);
      for (int r = 0; r < W; ++r) {
        bisectPAllReduce<half_bits, W> ar(b.dev[r], b.nelems, r, step, ipcbuf0[r], ipcbuf1[r], ipcbuf0, ipcbuf1);
        EXPECT(ar.workSize() == b.nelems * 2 / W);
        ar(streams[r]);
      }
      wait_all();
      step += 1000;
      EXPECT(b.mismatches(want) == 0);
    }
    {  // testTransmit<T>(algo, nd_range, input, ipcbuf0, ipcbuf1, peerbuf0, peerbuf1, nelems, rank, world, step, simd, queue)
      for (const char *algo : {"small", "simple_ring"}) {
        zero();
        Ranks b(W, 14336, 83);
        std::vector<uint16_t> want(b.nelems);
        auto hp = b.host_ptrs();
        vro_allreduce_rotated(want.data(), hp.data(), W, b.nelems);
        for (int r = 0; r < W; ++r)
          testTransmit<half_bits>(algo, {7, 8, 16}, b.dev[r], ipcbuf0[r], ipcbuf1[r], ipcbuf0, ipcbuf1, b.nelems,
                                  r, W, step, 16, streams[r]);
        wait_all();
        step += 1000;
        EXPECT(b.mismatches(want) == 0);
      }
    }
    {  // AllGather per rank
      zero();
      Ranks in(W, 8 * 999, 84), out(W, 8 * 999, 85, W);
      std::vector<uint16_t> want(W * in.nelems);
      auto hp = in.host_ptrs();
      vro_allgather(want.data(), hp.data(), W, in.nelems);
      for (int r = 0; r < W; ++r) {
        uint32_t s2 = step;
        AllGather<half_bits, W, Rt64_128_PCIE, RingTransmit>::launch(in.dev[r], out.dev[r], ipcbuf0[r], ipcbuf1[r],
                                                                     ipcbuf0, ipcbuf1, in.nelems, r, s2, streams[r]);
      }
      wait_all();
      EXPECT(out.mismatches(want) == 0);
    }
    {  // testAllgather<T>(algo, nd_range, input, output, ipcbuf0, ipcbuf1, peerbuf0, peerbuf1, nelems, rank, world, step, subgroup, queue)
      for (const char *algo : {"allgather_small", "allgather_simple"}) {
        for (LaunchParam grid : {LaunchParam{1, 4, 16}, LaunchParam{13, 8, 16}}) {
          zero();
          Ranks in(W, 8 * 2049, 87), out(W, 8 * 2049, 88, W);
          std::vector<uint16_t> want(W * in.nelems);
          auto hp = in.host_ptrs();
          vro_allgather(want.data(), hp.data(), W, in.nelems);
          for (int r = 0; r < W; ++r)
            testAllgather<half_bits>(algo, grid, in.dev[r], out.dev[r], ipcbuf0[r], ipcbuf1[r], ipcbuf0, ipcbuf1,
                                     in.nelems, r, W, step, 16, streams[r]);
          wait_all();
          step += 1000;
          EXPECT(out.mismatches(want) == 0);
        }
      }
      Ranks in(W, 64, 1), out(W, 64, 2, W);
      EXPECT(thrown([&] { testAllgather<half_bits>("simple", {1, 4, 16}, in.dev[0], out.dev[0], ipcbuf0[0], ipcbuf1[0], ipcbuf0, ipcbuf1, in.nelems, 0, W, 1, 16); }) ==
             "Transmit type not support");
    }
    {  // the constructor's exceptions, per rank
      Ranks b(W, W * 64, 86);
      EXPECT(thrown([&] { AllReduce<half_bits, W, Rt64, ParallelTransmit> a((half_bits *)((char *)b.dev[0] + 4), b.nelems, 0, 1, ipcbuf0[0], ipcbuf1[0], ipcbuf0, ipcbuf1); }) ==
             "We only support aligned pointer for now");
      EXPECT(thrown([&] { AllReduce<half_bits, W, Rt64, ParallelTransmit> a(b.dev[0], W * 4 + 4, 0, 1, ipcbuf0[0], ipcbuf1[0], ipcbuf0, ipcbuf1); }) ==
             "We don't support non-even divide yet");
      EXPECT(thrown([&] { testTransmit<half_bits>("tree", {1, 4, 16}, b.dev[0], ipcbuf0[0], ipcbuf1[0], ipcbuf0, ipcbuf1, b.nelems, 0, W, 1, 16); }) ==
             "Transmit type not support");
    }
    for (int r = 0; r < W; ++r) vr_free(ipcbuf0[r]);
    for (int r = 1; r < W; ++r) vr_stream_destroy(streams[r]);
  }
  // --- the reference's exceptions -------------------------------------------------------------------------
  {
    VirtualRanks ranks(8), two(2);
    Ranks b(8, 8 * 64, 71);
    EXPECT(thrown([&] { testTransmit<half_bits>("tree", {1, 4, 16}, ranks, b.dev.data(), b.nelems, 1); }) ==
           "Transmit type not support");
    EXPECT(thrown([&] { testTransmit<half_bits>("small", {1, 2, 16}, ranks, b.dev.data(), b.nelems, 1); }) ==
           "Subgroup numbers must be multiple of 4");
    EXPECT(thrown([&] { testTransmit<half_bits>("small", {1, 4, 8}, ranks, b.dev.data(), b.nelems, 1); }) ==
           "Unsupported Sub-group size");
    EXPECT(thrown([&] { AllReduce<half_bits, 8, Rt64, ParallelTransmit> a(ranks, b.dev.data(), 8 * 4 + 4, 1); }) ==
           "We don't support non-even divide yet");
    std::vector<half_bits *> odd(b.dev);
    odd[3] = (half_bits *)((char *)odd[3] + 4);
    EXPECT(thrown([&] { AllReduce<half_bits, 8, Rt64, ParallelTransmit> a(ranks, odd.data(), b.nelems, 1); }) ==
           "We only support aligned pointer for now");
    EXPECT(thrown([&] { AllReduce<half_bits, 8, Rt64, ParallelTransmit> a(two, b.dev.data(), b.nelems, 1); }) ==
           "Unsupported communication topology");
    EXPECT(thrown([&] { VirtualRanks three(3); }) == "Unsupported communication topology");
  }
  return failures;
}

int main() {
  try {
    if (run_all()) {
      printf("%d check(s) failed\n", failures);
      return 1;
    }
  } catch (const std::exception &e) {
    printf("unexpected exception: %s\n", e.what());
    return 2;
  }
  printf("host API ok\n");
  return 0;
}
