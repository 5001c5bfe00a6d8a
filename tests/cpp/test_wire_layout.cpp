// CPU bounds check of the wire transport's sinks: walks every (rank, wave, peer,
// slot) combination the kernels of each flow form, with the slot functions the
// kernels themselves use (vr_wire_layout.h), and proves that every message slot
// and every flag word lies inside a sink sized by the host code's layout_for().
// No GPU, no library: plain g++.
#include <stdio.h>

#include <initializer_list>

#include "vr_wire_layout.h"

using namespace vr::wl;

static int failures = 0;
#define EXPECT(cond)                                                         \
  do {                                                                       \
    if (!(cond)) {                                                           \
      if (failures < 20) printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      ++failures;                                                            \
    }                                                                        \
  } while (0)

struct Probe {
  const Layout &l;
  size_t need;      // slots_needed() of the flow under test
  size_t max_slot = 0;
  void touch(uint32_t slot) {
    if (slot > max_slot) max_slot = slot;
    EXPECT(slot < need);
    EXPECT(slot < l.slots);
    // payload of the largest format, then the slot's flag word, both inside the sink
    EXPECT(((size_t)slot + 1) * kSlotBytesMax <= l.flag_off);
    EXPECT(l.flag_off + ((size_t)slot + 1) * sizeof(uint32_t) <= l.sink_bytes);
  }
};

static void walk(int flow, int N, uint32_t wpr, const Layout &l) {
  Probe p{l, slots_needed(flow, N, wpr)};
  const int B = N / 2;
  for (int r = 0; r < N; ++r)
    for (uint32_t wid = 0; wid < wpr; ++wid) {
      switch (flow) {
        case PARALLEL: {
          const uint32_t x_id = wid / N * N;
          for (uint32_t s = 0; s < (uint32_t)kSlotsFlat; ++s)
            for (int q = 0; q < N; ++q) p.touch(parallel_slot(x_id, q, s));   // senders and owners, all peers
          break;
        }
        case SEQUENTIAL:
        case RING:
        case ALLGATHER:
          for (uint32_t s = 0; s < (uint32_t)kSlotsRing; ++s)
            for (int peer = 0; peer < N; ++peer) p.touch(ring_slot(wpr, peer, wid, s));
          break;
        case BISECT: {
          const uint32_t wg = wid / B * B;
          for (uint32_t s = 0; s < (uint32_t)kSlotsFlat; ++s) {
            for (int l2 = 0; l2 < B; ++l2) p.touch(bisect_close_slot(wg, l2, s));
            p.touch(bisect_far_slot(wpr, B, wid, s));
          }
          break;
        }
        case SIMPLE:
          // ring position of message t * wpr + wid; a power-of-two wpr keeps each
          // position with one wave
          for (uint32_t t = 0; t < 3 * kSimplePerSection / wpr + 3; ++t) {
            const uint32_t pos = (t * wpr + wid) % kSimplePerSection;
            EXPECT(pos % wpr == wid);
            for (int section = 0; section < N; ++section) p.touch(simple_slot(section, pos));
          }
          break;
      }
    }
  // the bound is tight enough to mean something: the walk reaches its last slot
  EXPECT(p.max_slot + 1 == p.need);
}

int main() {
  const int ranks[] = {2, 4, 8, 16};
  int cases = 0;
  for (int N : ranks)
    for (uint32_t wpr_max = 4; wpr_max <= 2048; wpr_max *= 2)
      for (int with_simple = 0; with_simple < 2; ++with_simple) {
        const Layout l = layout_for(N, wpr_max, with_simple != 0);
        EXPECT(l.sink_bytes % 256 == 0);
        EXPECT(l.rank_bytes == 2 * l.sink_bytes);
        for (int flow = 0; flow < FLOW_COUNT; ++flow) {
          if (flow == BISECT && N < 4) continue;
          if (flow == SIMPLE && !with_simple) continue;
          const uint32_t psg = flow == PARALLEL ? N : flow == BISECT ? N / 2 : 1;
          // every wire count the host may launch: multiples of psg up to wpr_max
          // (SimpleTransmit: powers of two up to half a section)
          for (uint32_t wpr = psg; wpr <= wpr_max; wpr += psg) {
            if (flow == SIMPLE && ((wpr & (wpr - 1)) || wpr > kSimplePerSection / 2)) continue;
            if (wpr > 64 && wpr != wpr_max / psg * psg && wpr % 37) continue;   // thin out the big ones
            walk(flow, N, wpr, l);
            ++cases;
          }
        }
      }
  // wires_fitting is the inverse of slots_needed: the largest wire count whose slots fit,
  // and a walk at exactly that count stays inside the sink
  for (int N : ranks)
    for (size_t slots : {64u, 1000u, 1024u, 4096u, 12288u, 100000u}) {
      Layout l = layout_for(N, 4, false);
      l.slots = slots;
      l.flag_off = slots * kSlotBytesMax;
      l.sink_bytes = (l.flag_off + slots * sizeof(uint32_t) + 255) / 256 * 256;
      for (int flow : {PARALLEL, SEQUENTIAL, RING, BISECT, ALLGATHER}) {
        if (flow == BISECT && N < 4) continue;
        const uint32_t fit = wires_fitting(flow, N, slots);
        EXPECT(fit == 0 || slots_needed(flow, N, fit) <= slots);
        EXPECT(slots_needed(flow, N, fit + 1) > slots);
        const uint32_t psg = flow == PARALLEL ? N : flow == BISECT ? N / 2 : 1;
        const uint32_t wpr = fit / psg * psg;
        if (wpr >= psg && wpr <= 4096) {
          walk(flow, N, wpr, l);
          ++cases;
        }
      }
    }
  // the fixed region of the allocation-free entry point: 8 ranks x 32 wires, no SimpleTransmit
  const Layout fixed = layout_for(8, 32, false);
  EXPECT(8 * fixed.rank_bytes + 256 <= (34u << 20));
  printf("%d layout cases, %d failures\n", cases, failures);
  return failures ? 1 : 0;
}
