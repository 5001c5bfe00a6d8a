// Host-side internals shared by the library's translation units: error
// reporting, the algorithm table, the context, and the entry into the wire
// transport's host code (vr_wire_host.cpp).
#pragma once

#include <string>

#include "vr_internal.h"

namespace vr {

// ---- errors: record the thread's detail text, return the status -----------------------
int fail(int status, const std::string &detail);
int fail_hip(hipError_t e, const char *what);

#define HIP_TRY(expr)                                     \
  do {                                                    \
    hipError_t e__ = (expr);                              \
    if (e__ != hipSuccess) return ::vr::fail_hip(e__, #expr); \
  } while (0)

static inline size_t div_up(size_t x, size_t m) { return (x + m - 1) / m; }

// ---- algorithm table --------------------------------------------------------------------
enum TransmitKind { T_PARALLEL, T_BISECT, T_RING, T_SEQUENTIAL, T_SIMPLE };

struct AlgoInfo {
  const char *name;
  TransmitKind transmit;
  int msg_bytes;       // sizeof(message_t) at sub-group size 16
  int wire_capacity;   // payload bytes per wire at sub-group size 16
  bool allgather;
  Order order;
  bool latency_tuned;  // "small" family: one-shot grid, cached accesses
  WireFlow wire_flow() const {
    if (allgather) return WIRE_ALLGATHER;
    switch (transmit) {
      case T_BISECT: return WIRE_BISECT;
      case T_RING: return WIRE_RING;
      case T_SEQUENTIAL: return WIRE_SEQUENTIAL;
      case T_SIMPLE: return WIRE_SIMPLE;
      default: return WIRE_PARALLEL;
    }
  }
  // Rt64 -> self-validating 8-byte messages; Rt64_PCIE -> 16-byte messages with
  // the flag twice; Rt64_128 -> 128-byte messages, Rt64_128_PCIE -> 256-byte
  // messages, both with a flag in every 64 bytes.
  WireFormat wire_format() const {
    if (latency_tuned) return msg_bytes == 16 ? WIRE_FMT_LL16 : WIRE_FMT_LL;
    return msg_bytes == 16 ? WIRE_FMT_RT256 : WIRE_FMT_RT128;
  }
};

extern const AlgoInfo kAlgos[VR_ALGO_COUNT_];
const AlgoInfo *algo_info(int algo);

// ---- context ------------------------------------------------------------------------------
// User overrides of the launch heuristics; -1 = let the library decide.
struct TuningOverrides {
  int block = -1, waves_per_cu = -1, unroll = -1, nt_load = -1, nt_store = -1, oneshot = -1;
  int segment_kib = -1, f16_wide = -1, wgs_per_cu = -1, deal = -1, run = -1;
  int wire_fenced = -1, wire_cooperative = -1, wire_blocks_per_cu = -1, wire_ahead = -1, wire_msg16 = -1;
  int wire_stream_io = -1;
};

// Where the messages of a wire-transport launch go: every rank's scatter and
// gather sink (the reference's peerBuf0[] / peerBuf1[], main.cpp:260-269) and what
// they were sized for.
struct WireSinks {
  void *scatter[VR_MAX_RANKS] = {}, *gather[VR_MAX_RANKS] = {};
  wl::Layout layout = {};
  uint32_t wpr_max = 0;        // wires per rank the sinks hold
  bool simple_ok = false;      // room for SimpleTransmit's sender sections
  void *region = nullptr;      // library-owned sinks lie back to back in one region of
  size_t region_bytes = 0;     // this many bytes (cleared with one launch)
};

// What earlier launches left in a set of sinks.
struct WireHistory {
  bool used = false;           // a launch has written flags since the last clear
  uint32_t next_min_seq = 0;   // smallest flag value the next launch may start at
  int last_flow = -1, last_fmt = -1;
};

// Scratch of the wire transport owned by a context: ONE allocation holding, per
// virtual rank, a scatter sink followed by a gather sink (the reference's
// ipcbuf0 | ipcbuf1, main.cpp:241-251), made and zeroed by vr_ctx_reserve_wire.
struct WireState {
  bool ready = false;
  void *base = nullptr;
  size_t bytes = 0;
  WireSinks sinks;
  WireHistory hist;
};

constexpr uint32_t kWireBlockThreads = 256;   // 4 wires per work-group

}  // namespace vr

// The opaque handle of the C ABI.
struct vr_ctx {
  int nranks = 0;
  vr::DeviceInfo dev;
  vr::TuningOverrides tune;
  uint32_t seq_no = 1;
  uint64_t spin_limit = 0;
  vr::DType dtype = vr::DT_F16;
  uint32_t *status = nullptr;     // time-out word of this context's wire launches (256 B)
  vr::WireState wire;
};

namespace vr {

// Every launch path starts here: kernels go to the context's device whatever the
// calling thread's current device is.
int use_device(const vr_ctx *ctx);
bool ranges_partially_overlap(const void *a, const void *b, size_t bytes);

// A validated all-reduce call.
struct Prepared {
  const AlgoInfo *a;
  PtrTable in, out;
  size_t chunk_elems;
  int vec_halves;
  vr_geometry geom;
  bool in_place;
  size_t bytes_all_ranks;   // nranks * nelems * 2
};
int prepare_allreduce(vr_ctx *ctx, int algo, void *const bufs[], void *const outs[], size_t nelems,
                      Prepared *p);

// ---- wire transport, host side (vr_wire_host.cpp) ------------------------------------------
void wire_free(vr_ctx *c);
// Launch on the context's own scratch; see wire_launch for the arguments.
int wire_launch_ctx(vr_ctx *c, hipStream_t s, const AlgoInfo *a, const PtrTable &in, const PtrTable &out,
                    size_t chunk_bytes, int vec_halves, uint32_t *seq_io, uint32_t user_wires,
                    uint32_t *flags_used);

}  // namespace vr
