// Sink geometry of the wire transport: which message slot of a rank's scatter or
// gather sink a wave touches, for every flow.  The kernels (vr_wire.hip), the host
// code that sizes the scratch (vr_wire_host.cpp) and a CPU bounds test all use these
// same functions, so a sink can be proven large enough without a GPU.
//
// A sink is `slots` message slots of kSlotBytesMax bytes followed by `slots`
// 32-bit flag words (used only by the fenced flag-word format).  A rank's scratch
// is its scatter sink followed by its gather sink, the shape of the reference's
// one allocation ipcbuf0 | ipcbuf1 (main.cpp:241-243).
#pragma once

#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define VR_HD __host__ __device__ constexpr
#else
#define VR_HD constexpr
#endif

namespace vr {
namespace wl {

constexpr uint32_t kSlotBytesMax = 2048;        // largest message any format stores per wave and step
constexpr uint32_t kSimplePerSection = 1024;    // messages per sender section of SimpleTransmit
                                                // (2 MiB of 2 KiB messages, simple_transmit.hpp:11)
constexpr int kSlotsFlat = 8;                   // nSlot of ParallelTransmit / BisectPTransmit
constexpr int kSlotsRing = 4;                   // nSlot of SequentialTransmit / RingTransmit

enum Flow : int { PARALLEL, SEQUENTIAL, RING, BISECT, ALLGATHER, SIMPLE, FLOW_COUNT };

// ---- slot index of a message ------------------------------------------------------------
// ParallelTransmit: sink entry (x_id + sender), ring of 8 slots per entry
// (parallel_transmit.hpp:47-58, 93).
VR_HD uint32_t parallel_slot(uint32_t x_id, int sender, uint32_t s) {
  return (x_id + (uint32_t)sender) * kSlotsFlat + s;
}
// SequentialTransmit / RingTransmit / ring all-gather: entry [peer][wire], 4 slots
// (sequential_transmit.hpp:69-77, 273-277).
VR_HD uint32_t ring_slot(uint32_t wpr, int peer, uint32_t wid, uint32_t s) {
  return ((uint32_t)peer * wpr + wid) * kSlotsRing + s;
}
// BisectPTransmit: close entries (wg + l) first, the far entries behind them
// (bisect_transmit.hpp:445-481).
VR_HD uint32_t bisect_close_slot(uint32_t wg, int l, uint32_t s) {
  return (wg + (uint32_t)l) * kSlotsFlat + s;
}
VR_HD uint32_t bisect_far_slot(uint32_t wpr, int half_ranks, uint32_t wid, uint32_t s) {
  return (wpr + (uint32_t)half_ranks + wid) * kSlotsFlat + s;
}
// SimpleTransmit: one section of kSimplePerSection messages per sender.
VR_HD uint32_t simple_slot(int section, uint32_t pos) {
  return (uint32_t)section * kSimplePerSection + pos;
}

// ---- slots a sink must hold ---------------------------------------------------------------
// `wpr` = wires (waves) per rank.  Exclusive upper bound of every slot index the
// flow's kernel forms for `nranks` ranks.
VR_HD size_t slots_needed(int flow, int nranks, uint32_t wpr) {
  switch (flow) {
    case PARALLEL: return (size_t)kSlotsFlat * wpr;
    case BISECT: return (size_t)kSlotsFlat * (2u * (size_t)wpr + (size_t)nranks / 2);
    case SIMPLE: return (size_t)nranks * kSimplePerSection;
    default: return (size_t)kSlotsRing * (size_t)nranks * wpr;
  }
}

// Largest number of wires per rank whose slot range still fits `slots` slots (the
// inverse of slots_needed; SimpleTransmit's range does not depend on the wire
// count).
VR_HD uint32_t wires_fitting(int flow, int nranks, size_t slots) {
  switch (flow) {
    case PARALLEL: return (uint32_t)(slots / kSlotsFlat);
    case BISECT: {
      const size_t entries = slots / kSlotsFlat, half = (size_t)nranks / 2;
      return entries > half ? (uint32_t)((entries - half) / 2) : 0u;
    }
    case SIMPLE: return slots >= (size_t)nranks * kSimplePerSection ? kSimplePerSection / 2 : 0u;
    default: return (uint32_t)(slots / ((size_t)kSlotsRing * (size_t)nranks));
  }
}

struct Layout {
  size_t slots;        // message slots per sink
  size_t flag_off;     // byte offset of the flag words inside a sink
  size_t sink_bytes;   // payload slots + flag words, a multiple of 256
  size_t rank_bytes;   // scatter sink + gather sink of one rank
};

// Scratch sized for every flow at up to `wpr_max` wires per rank; `with_simple`
// adds room for SimpleTransmit's sender sections.
VR_HD Layout layout_for(int nranks, uint32_t wpr_max, bool with_simple) {
  size_t slots = 0;
  for (int f = 0; f < FLOW_COUNT; ++f) {
    if (f == SIMPLE && !with_simple) continue;
    const size_t n = slots_needed(f, nranks, wpr_max);
    if (n > slots) slots = n;
  }
  const size_t flag_off = slots * kSlotBytesMax;
  const size_t sink_bytes = (flag_off + slots * sizeof(uint32_t) + 255) / 256 * 256;
  return Layout{slots, flag_off, sink_bytes, 2 * sink_bytes};
}

}  // namespace wl
}  // namespace vr
