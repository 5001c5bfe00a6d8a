// Host side of the wire transport: scratch ownership (context, caller, the
// library's fixed region), launch sizing and sequence-number bookkeeping, the
// one-rank entry points and the time-out check.  Kernels: vr_wire.hip.

#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <string>
#include <unordered_map>

#include "vr_host.h"

using namespace vr;

static const uint32_t kDefaultSpinLimit = 1u << 22;
static const int kWireBlocksPerCu = 3;
static const uint32_t kWireAhead = 4;

namespace vr {
void wire_free(vr_ctx *c) {
  WireState &w = c->wire;
  if (w.base) (void)hipFree(w.base);
  w = WireState();
}
}  // namespace vr

// Wires per rank the context's launches may use: a few 256-lane work-groups per
// CU (default three, what every flow's kernel fits) keep every wire of every
// rank co-resident.
static uint32_t wire_wpr_max(const vr_ctx *c) {
  const int per_cu = c->tune.wire_blocks_per_cu > 0 ? c->tune.wire_blocks_per_cu : kWireBlocksPerCu;
  uint32_t blocks = (uint32_t)(c->dev.cus * per_cu / c->nranks);
  if (blocks == 0) blocks = 1;
  return blocks * (kWireBlockThreads / 64);
}

static void sinks_at(WireSinks *k, int nranks, char *base, const wl::Layout &l, uint32_t wpr_max,
                     bool simple_ok) {
  *k = WireSinks();
  for (int r = 0; r < nranks; ++r) {
    k->scatter[r] = base + (size_t)r * l.rank_bytes;
    k->gather[r] = base + (size_t)r * l.rank_bytes + l.sink_bytes;
  }
  k->layout = l;
  k->wpr_max = wpr_max;
  k->simple_ok = simple_ok;
  k->region = base;
  k->region_bytes = (size_t)nranks * l.rank_bytes;
}

extern "C" int vr_ctx_reserve_wire(vr_ctx *c) {
  if (!c) return fail(VR_ERR_INVALID, "null ctx");
  WireState &w = c->wire;
  if (w.ready) return VR_OK;
  HIP_TRY(hipSetDevice(c->dev.device));
  const uint32_t wpr_max = wire_wpr_max(c);
  const wl::Layout l = wl::layout_for(c->nranks, wpr_max, true);
  w.bytes = (size_t)c->nranks * l.rank_bytes;
  hipError_t e = hipMalloc(&w.base, w.bytes);
  if (e == hipSuccess) e = hipMemset(w.base, 0, w.bytes);      // zeroed once, main.cpp:251
  if (e == hipSuccess) e = hipDeviceSynchronize();
  if (e != hipSuccess) {
    wire_free(c);
    return fail_hip(e, "reserving the wire-transport scratch");
  }
  sinks_at(&w.sinks, c->nranks, static_cast<char *>(w.base), l, wpr_max, true);
  w.ready = true;
  return VR_OK;
}

extern "C" int vr_rank_scratch_bytes(const vr_ctx *c, size_t *sink_bytes) {
  if (!c || !sink_bytes) return fail(VR_ERR_INVALID, "null argument");
  *sink_bytes = wl::layout_for(c->nranks, wire_wpr_max(c), true).sink_bytes;
  return VR_OK;
}

// Forget every flag ever written (asynchronous, ordered on `s`).
static int wire_clear(const WireSinks &k, int nranks, hipStream_t s) {
  if (k.region) {
    const hipError_t e = launch_wire_clear(s, k.region, k.region_bytes);
    return e == hipSuccess ? VR_OK : fail_hip(e, "launch_wire_clear");
  }
  for (int r = 0; r < nranks; ++r) {
    hipError_t e = launch_wire_clear(s, k.scatter[r], k.layout.sink_bytes);
    if (e == hipSuccess) e = launch_wire_clear(s, k.gather[r], k.layout.sink_bytes);
    if (e != hipSuccess) return fail_hip(e, "launch_wire_clear");
  }
  return VR_OK;
}

struct WireLaunch {
  const WireSinks *sinks;
  WireHistory *hist;      // null: the caller owns the sinks and the sequence numbers (rank-group launches)
  uint32_t *status;
  int first, count;       // the launch holds the wires of ranks [first, first + count)
  bool always_clear;      // clear the sinks before every launch (fixed scratch shared by contexts)
  bool io_narrow = false; // inputs / outputs of this launch are only 8-byte aligned
};

// How the Rt64_128 families synchronise (the "wire_fenced" setting).  Left to the
// library, the all-to-all flows (ParallelTransmit, BisectPTransmit, SimpleTransmit)
// take flag words with agent-scope accesses ordered by store completion: as fast as
// or faster than the reference's embedded-flag messages at every size measured, and
// resting on nothing but the scope semantics of the accesses.  The neighbour-ring and
// sequential flows keep the reference's messages, which are up to 15 % faster there.
static int flag_word_mode(const vr_ctx *c, const AlgoInfo *a) {
  if (c->tune.wire_fenced >= 0) return c->tune.wire_fenced;
  if (a->allgather) return 0;
  return (a->transmit == T_PARALLEL || a->transmit == T_BISECT || a->transmit == T_SIMPLE) ? 4 : 0;
}

// Wire format of an algo under the context's settings.  `vec_halves` = 8 says that
// every pointer and the chunk allow 16-byte accesses.
static WireFormat format_for(const vr_ctx *c, const AlgoInfo *a, size_t chunk_bytes, int vec_halves) {
  WireFormat fmt = a->wire_format();
  const bool big = fmt == WIRE_FMT_RT128 || fmt == WIRE_FMT_RT256;
  const int fenced = flag_word_mode(c, a);
  if (big && fenced == 1) fmt = WIRE_FMT_FLAG;
  // Self-validating 8-byte messages for the Rt64_128 families too: nothing beyond
  // 8-byte store atomicity is assumed, at half the payload per message.
  if (big && fenced == 2) fmt = WIRE_FMT_LL;
  if (big && fenced == 3) fmt = WIRE_FMT_FLAG_WT;
  if (big && fenced == 4) fmt = WIRE_FMT_FLAG_SCOPED;
  if (fmt == WIRE_FMT_LL16 && c->tune.wire_msg16 == 0) fmt = WIRE_FMT_LL;
  // `parallel` names the transmit, not a wire format: it takes the reference's
  // 256-byte messages (16 bytes per lane) when every pointer and the chunk allow
  // 16-byte accesses, its 128-byte messages otherwise.
  if (fmt == WIRE_FMT_RT128 && a == &kAlgos[VR_ALGO_PARALLEL] && vec_halves == 8 && chunk_bytes % 16 == 0)
    fmt = WIRE_FMT_RT256;
  return fmt;
}

// Does the algo's wire format, as the context is set, carry 16 bytes per lane when
// the chunk is a multiple of 16 bytes?  (Then every rank must decide so from the
// element count alone; a rank whose buffers are only 8-byte aligned moves each
// lane's 16 bytes as two 8-byte accesses.)  The 8-byte-message formats (Rt64,
// Rt64_128) and the 16-byte-message formats (whose calcWorkSize already demands
// 16-byte alignment) do not depend on it.
static bool format_widens_with_alignment(const vr_ctx *c, const AlgoInfo *a) {
  if (a == &kAlgos[VR_ALGO_PARALLEL]) return true;
  const WireFormat fmt = a->wire_format();
  const bool big = fmt == WIRE_FMT_RT128 || fmt == WIRE_FMT_RT256;
  const int fenced = flag_word_mode(c, a);
  return big && (fenced == 1 || fenced == 3 || fenced == 4);
}

// Shape of one wire-transport launch: which kernel, how many wires per rank, how
// many loop steps and how many consecutive flag values it consumes.
struct WirePlan {
  WireFlow flow;
  WireFormat fmt;
  uint32_t wpr = 0;              // wires (waves) per rank; 0 = nothing to move
  uint32_t blocks_per_rank = 0;
  size_t steps = 0;
  uint32_t flags_used = 0;
};

// `user_wires` (0 = automatic) is the number of sub-groups per rank a caller asked
// for with -g/-w; `k` the sinks the launch will use.
static int plan_wire(const vr_ctx *c, const AlgoInfo *a, size_t chunk_bytes, int vec_halves,
                     uint32_t user_wires, const WireSinks &k, WirePlan *plan) {
  const int N = c->nranks;
  const WireFlow flow = a->wire_flow();
  const WireFormat fmt = format_for(c, a, chunk_bytes, vec_halves);
  *plan = WirePlan();
  plan->flow = flow;
  plan->fmt = fmt;
  if (flow == WIRE_SIMPLE && !k.simple_ok)
    return fail(VR_ERR_INVALID, "these sinks have no room for SimpleTransmit's 2 MiB sender sections");
  const uint32_t psg = flow == WIRE_PARALLEL ? (uint32_t)N : flow == WIRE_BISECT ? (uint32_t)N / 2 : 1u;
  const uint32_t waves_per_block = kWireBlockThreads / 64;
  // Every wave may wait for any other: keep the grid (for rank-group launches: the
  // groups' grids together) within what the device holds at once.
  int per_cu = 0;
  if (hipError_t e = wire_blocks_per_cu(flow, fmt, vec_halves, N, kWireBlockThreads, c->dtype, &per_cu))
    return fail_hip(e, "occupancy query");
  const uint32_t resident_wpr = (uint32_t)((size_t)c->dev.cus * (size_t)per_cu / (size_t)N) * waves_per_block;
  // and within what the sinks hold for this flow (the all-to-all flows index fewer
  // slots per wire than the ring flows the sinks are sized for)
  const uint32_t fit = wl::wires_fitting((int)flow, N, k.layout.slots);
  const uint32_t wpr_cap = fit < resident_wpr ? fit : resident_wpr;
  const uint32_t wpr_limit = wpr_cap / psg * psg;
  if (wpr_limit < psg) return fail(VR_ERR_INVALID, "sinks or device too small for this rank count");
  const uint32_t wire_bytes = wire_bytes_per_step(fmt, vec_halves);
  const size_t wires_per_chunk = div_up(chunk_bytes, wire_bytes);
  if (wires_per_chunk == 0) return VR_OK;
  size_t want = user_wires ? (size_t)user_wires / psg * psg : wires_per_chunk * psg;
  if (want < psg) want = psg;
  if (want > wpr_limit) want = wpr_limit;
  if (flow == WIRE_SIMPLE) {
    // A sender runs at most one step ahead of its receivers, so two steps must fit
    // a section; and only a power of two divides the section, which keeps every
    // ring position with the wave that used it before.
    if (want > wl::kSimplePerSection / 2) want = wl::kSimplePerSection / 2;
    size_t pow2 = 1;
    while (pow2 * 2 <= want) pow2 *= 2;
    want = pow2;
  }
  const uint32_t wpr = (uint32_t)want;
  if (wl::slots_needed((int)flow, N, wpr) > k.layout.slots)
    return fail(VR_ERR_INVALID, "internal: sink smaller than the flow's slot range");
  plan->wpr = wpr;
  plan->blocks_per_rank = (uint32_t)div_up(wpr, waves_per_block);
  plan->steps = div_up(wires_per_chunk, wpr / psg);
  const uint32_t nslot_min = 4;
  plan->flags_used = flow == WIRE_SIMPLE ? (uint32_t)(plan->steps * wpr / wl::kSimplePerSection + 1)
                                         : (uint32_t)((plan->steps - 1) / nslot_min + 1);
  return VR_OK;
}

// Launches one wire-transport collective.  *seq_io is the first flag value the
// caller proposes; it is replaced by the one actually used (it restarts from 1
// when the 32-bit counter would wrap through 0).  Returns through *flags_used how
// many consecutive flag values the launch consumes.
static int wire_launch(vr_ctx *c, hipStream_t s, const AlgoInfo *a, const PtrTable &in,
                       const PtrTable &out, size_t chunk_bytes, int vec_halves, uint32_t *seq_io,
                       uint32_t user_wires, uint32_t *flags_used, const WireLaunch &wlch) {
  uint32_t seq = *seq_io;
  if (seq == 0)
    return fail(VR_ERR_INVALID, "sequence number 0 cannot be told from freshly zeroed scratch");
  const WireSinks &k = *wlch.sinks;
  const int N = c->nranks;
  // The flag values of a launch are kernel arguments, and whether the sinks must
  // be cleared first is decided here on the host: a captured launch would replay
  // with stale flags.  (With always_clear every replay starts from clean sinks.)
  if (!wlch.always_clear) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(VR_ERR_INVALID, "the wire transport cannot be captured into a graph: its flag values "
                                  "are per-launch kernel arguments (capture the direct transport)");
    (void)hipGetLastError();
  }
  WirePlan plan;
  if (int rc = plan_wire(c, a, chunk_bytes, vec_halves, user_wires, k, &plan)) return rc;
  *flags_used = plan.flags_used;
  if (plan.wpr == 0) return VR_OK;
  const WireFlow flow = plan.flow;
  const WireFormat fmt = plan.fmt;
  const uint32_t wpr = plan.wpr, blocks_per_rank = plan.blocks_per_rank;

  // Flags must strictly increase on every slot and never be 0 (the value of
  // cleared scratch); a different flow or format re-interprets the sinks.  In all
  // those cases start from a clean slate.
  const bool wraps = (uint32_t)(seq + *flags_used) < seq;
  if (wraps && !wlch.hist && !wlch.always_clear)
    return fail(VR_ERR_INVALID, "the sequence number would wrap through 0: zero every rank's scratch "
                                "and restart from 1");
  if (wraps) seq = 1;
  if (wlch.always_clear) {
    // only what this launch will look at: the message slots of its slot range where
    // the flag travels inside the message, the flag words of those slots where it
    // does not (a flag-word payload is never read before its flag has been seen)
    PtrTable sc, ga;
    memset(&sc, 0, sizeof sc);
    memset(&ga, 0, sizeof ga);
    for (int r = 0; r < N; ++r) {
      sc.p[r] = k.scatter[r];
      ga.p[r] = k.gather[r];
    }
    const size_t slots = wl::slots_needed((int)flow, N, wpr);
    const bool flag_words = wire_fmt_is_flag(fmt);
    const hipError_t e = launch_wire_clear_sinks(s, sc, ga, N, flag_words ? 0 : slots * wire_slot_bytes(fmt, vec_halves),
                                                 k.layout.flag_off, flag_words ? slots * 4 : 0);
    if (e != hipSuccess) return fail_hip(e, "launch_wire_clear_sinks");
  } else if (wlch.hist) {
    WireHistory &h = *wlch.hist;
    const bool moved_back = h.used && (int32_t)(seq - h.next_min_seq) < 0;
    if (wraps || moved_back || (h.used && (h.last_flow != (int)flow || h.last_fmt != (int)fmt))) {
      if (int rc = wire_clear(k, N, s)) return rc;
      h.used = false;
    }
  }
  *seq_io = seq;

  WireArgs args;
  memset(&args, 0, sizeof args);
  args.in = in;
  args.out = out;
  for (int r = 0; r < N; ++r) {
    args.scatter.p[r] = k.scatter[r];
    args.gather.p[r] = k.gather[r];
  }
  args.flag_off = k.layout.flag_off;
  args.chunk_bytes = chunk_bytes;
  args.waves_per_rank = wpr;
  args.seq = seq;
  const uint64_t limit = c->spin_limit ? c->spin_limit : kDefaultSpinLimit;
  args.spin_limit = limit > 0xffffffffull ? 0xffffffffu : (uint32_t)limit;
  args.status = wlch.status;
  args.ahead = c->tune.wire_ahead > 0 ? (uint32_t)c->tune.wire_ahead : kWireAhead;
  args.io_narrow = wlch.io_narrow ? 1u : 0u;
  args.rank_first = wlch.first;
  args.rank_count = wlch.count;
  // Inputs and outputs that cannot stay in the 256 MiB memory-side cache anyway are
  // streamed past it, which leaves that cache to the sinks (measured: faster from
  // 256 MiB of inputs + outputs on, slower below).
  const size_t io_bytes = a->allgather ? (size_t)N * chunk_bytes * (1 + (size_t)N)    // N slices in, N x N out
                                       : 2 * (size_t)N * chunk_bytes * (size_t)N;     // N chunks per rank, in + out
  args.stream_io = c->tune.wire_stream_io >= 0 ? (uint32_t)c->tune.wire_stream_io
                                               : (io_bytes >= (256ull << 20) ? 1u : 0u);
  // The grid is co-resident by construction; a cooperative launch (on request)
  // lets the runtime check that once more.  A launch that holds some of the ranks
  // cannot vouch for the other ranks' work-groups: always plain.
  const bool cooperative = wlch.count == N && c->tune.wire_cooperative == 1;
  const uint32_t blocks = blocks_per_rank * (uint32_t)wlch.count;
  hipError_t e = launch_wire(s, flow, fmt, vec_halves, N, blocks, kWireBlockThreads, args,
                             cooperative, c->dtype);
  if (e != hipSuccess) return fail_hip(e, "launch_wire");
  if (wlch.hist) {
    wlch.hist->used = true;
    wlch.hist->next_min_seq = seq + *flags_used;
    wlch.hist->last_flow = (int)flow;
    wlch.hist->last_fmt = (int)fmt;
  }
  return VR_OK;
}

// Launch on the context's own scratch.
namespace vr {
int wire_launch_ctx(vr_ctx *c, hipStream_t s, const AlgoInfo *a, const PtrTable &in,
                           const PtrTable &out, size_t chunk_bytes, int vec_halves, uint32_t *seq_io,
                           uint32_t user_wires, uint32_t *flags_used) {
  if (!c->wire.ready)
    return fail(VR_ERR_INVALID, "the wire transport's scratch is not reserved: call "
                                "vr_ctx_reserve_wire(ctx) once before the first wire-transport launch");
  const WireLaunch wlch = {&c->wire.sinks, &c->wire.hist, c->status, 0, c->nranks, false};
  return wire_launch(c, s, a, in, out, chunk_bytes, vec_halves, seq_io, user_wires, flags_used, wlch);
}
}  // namespace vr


// The library's fixed scratch region on the context's device, laid out as sinks
// for the context's rank count.
static int static_sinks(const vr_ctx *ctx, WireSinks *k) {
  void *fixed = nullptr;
  size_t bytes = 0;
  hipError_t e = wire_static_scratch(ctx->dev.device, &fixed, &bytes);
  if (e != hipSuccess) return fail_hip(e, "hipGetSymbolAddress(scratch)");
  const wl::Layout l = wl::layout_for(ctx->nranks, kStaticWiresPerRank, false);
  if ((size_t)ctx->nranks * l.rank_bytes > bytes)
    return fail(VR_ERR_INVALID, "the fixed scratch region holds at most " +
                                    std::to_string(kStaticMaxRanks) + " ranks");
  sinks_at(k, ctx->nranks, static_cast<char *>(fixed), l, kStaticWiresPerRank, false);
  return VR_OK;
}

// Largest input the allocation-free entry point accepts: the sweep's largest
// point, 256 MiB per rank.
static const size_t kStaticMaxBytesPerRank = 256ull << 20;

extern "C" int vr_allreduce_static(vr_ctx *ctx, void *stream, int algo, void *const bufs[],
                                   void *const outs[], size_t nelems) {
  Prepared p;
  if (int rc = prepare_allreduce(ctx, algo, bufs, outs, nelems, &p)) return rc;
  if (ctx->nranks > kStaticMaxRanks)
    return fail(VR_ERR_INVALID, "vr_allreduce_static serves at most " + std::to_string(kStaticMaxRanks) +
                                    " ranks, this context has " + std::to_string(ctx->nranks));
  if (nelems * 2 > kStaticMaxBytesPerRank)
    return fail(VR_ERR_INVALID, "vr_allreduce_static serves at most " +
                                    std::to_string(kStaticMaxBytesPerRank) + " bytes per rank, got " +
                                    std::to_string(nelems * 2));
  if (p.a->wire_flow() == WIRE_SIMPLE)
    return fail(VR_ERR_INVALID, "vr_allreduce_static has no room for SimpleTransmit's 2 MiB sender sections");
  WireSinks k;
  if (int rc = static_sinks(ctx, &k)) return rc;
  // The region is shared by every context on the device and keeps the last
  // call's messages: every call first clears the slots it is about to use (a
  // fill kernel on the stream), so the flags can start from 1 each time.  The
  // time-out word is the context's own, like that of its other wire launches.
  const WireLaunch wlch = {&k, nullptr, ctx->status, 0, ctx->nranks, true};
  uint32_t seq = 1, used = 0;
  return wire_launch(ctx, (hipStream_t)stream, p.a, p.in, p.out, p.chunk_elems * 2, p.vec_halves, &seq,
                     0, &used, wlch);
}

// Caller-owned sinks of a rank-group launch: every rank's scatter and gather sink,
// the launch's own ranks included.
static int group_sinks(const vr_ctx *ctx, void *const peer_buf0[], void *const peer_buf1[],
                       size_t sink_bytes, WireSinks *k) {
  const int N = ctx->nranks;
  if (!peer_buf0 || !peer_buf1) return fail(VR_ERR_INVALID, "null scratch pointer");
  const uint32_t wpr_max = wire_wpr_max(ctx);
  const wl::Layout l = wl::layout_for(N, wpr_max, true);
  if (sink_bytes < l.sink_bytes)
    return fail(VR_ERR_INVALID, "sinks hold " + std::to_string(sink_bytes) + " bytes, this context needs " +
                                    std::to_string(l.sink_bytes) + " (vr_rank_scratch_bytes)");
  *k = WireSinks();
  k->layout = l;
  k->wpr_max = wpr_max;
  k->simple_ok = true;
  for (int r = 0; r < N; ++r) {
    k->scatter[r] = peer_buf0[r];
    k->gather[r] = peer_buf1[r];
    if (!k->scatter[r] || !k->gather[r]) return fail(VR_ERR_INVALID, "null sink for rank " + std::to_string(r));
    if ((uintptr_t)k->scatter[r] % 16 || (uintptr_t)k->gather[r] % 16)
      return fail(VR_ERR_UNALIGNED, "sinks must be 16-byte aligned");
  }
  return VR_OK;
}

// The launches that form one collective against caller-owned sinks wait for each
// other, so their kernels must run at the same time.  Inside one process that
// takes one hardware queue per launch: two launches on one stream run one after
// the other, and a process has only a few hardware queues (GPU_MAX_HW_QUEUES, 4
// unless the environment says otherwise) which further streams share.  Both would
// end in a poll time-out; they are refused here instead, with the remedy.  A
// collective is recognised by its sinks (rank 0's scatter sink) and its sequence
// number, which every one of its launches must pass alike.
namespace {
struct GroupLaunches {
  uint32_t seq = 0;
  int nranks = 0;
  void *stream_of[VR_MAX_RANKS] = {};
  bool launched[VR_MAX_RANKS] = {};
};
std::mutex g_groups_lock;
std::unordered_map<const void *, GroupLaunches> g_groups;

int hardware_queues() {
  const char *env = getenv("GPU_MAX_HW_QUEUES");
  const int v = env ? atoi(env) : 0;
  return v > 0 ? v : 4;
}
}  // namespace

static int admit_group_launch(const vr_ctx *ctx, const void *family, void *stream, int first, int count,
                              uint32_t seq) {
  const int N = ctx->nranks;
  if (count == N) return VR_OK;
  std::lock_guard<std::mutex> hold(g_groups_lock);
  GroupLaunches &g = g_groups[family];
  if (g.seq != seq || g.nranks != N) {
    g = GroupLaunches();
    g.seq = seq;
    g.nranks = N;
  }
  int streams = 0;
  void *seen[VR_MAX_RANKS];
  for (int r = 0; r < N; ++r) {
    if (!g.launched[r] || (r >= first && r < first + count)) continue;
    if (g.stream_of[r] == stream)
      return fail(VR_ERR_INVALID, "ranks " + std::to_string(first) + ".." + std::to_string(first + count - 1) +
                                      " and rank " + std::to_string(r) + " of one collective were launched on the "
                                      "same stream: their kernels wait for each other and must run at the same "
                                      "time (one stream per launch, or one vr_allreduce_ranks launch for both)");
    bool known = false;
    for (int i = 0; i < streams; ++i) known = known || seen[i] == g.stream_of[r];
    if (!known) seen[streams++] = g.stream_of[r];
  }
  const int limit = hardware_queues();
  if (streams + 1 > limit)
    return fail(VR_ERR_INVALID, "this collective would need " + std::to_string(streams + 1) +
                                    " concurrent launches from one process, which has " + std::to_string(limit) +
                                    " hardware queues (GPU_MAX_HW_QUEUES): hold several ranks per launch with "
                                    "vr_allreduce_ranks, or run the ranks in separate processes");
  for (int r = first; r < first + count; ++r) {
    g.launched[r] = true;
    g.stream_of[r] = stream;
  }
  return VR_OK;
}

// Ranks [first, first + count) of an all-reduce, the form the reference constructs
// once per process for one rank (allreduce.hpp:18-28, parallel_transmit.hpp:36-60,
// bisect_transmit.hpp:427-482).
static int allreduce_ranks(vr_ctx *ctx, void *stream, int algo, int first, int count,
                           void *const inputs[], void *const outputs[], void *const peer_buf0[],
                           void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no,
                           uint32_t user_wires) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || a->allgather) return fail(VR_ERR_ALGO, "not an all-reduce algo");
  const int N = ctx->nranks;
  if (first < 0 || count < 1 || first + count > N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!inputs) return fail(VR_ERR_INVALID, "null input table");
  if (!seq_no) return fail(VR_ERR_INVALID, "a rank-group launch needs the caller's sequence number");
  // Every rank must pick the same message shape, so the access width may depend on
  // nothing but the algo, the context's settings and the element count.  Formats
  // that move 16 bytes per lane when the chunk is a multiple of 16 bytes then need
  // 16-byte aligned buffers on every rank; the others accept what calcWorkSize
  // accepts (allreduce.hpp:108-122).
  const bool widens = format_widens_with_alignment(ctx, a);
  PtrTable in, out;
  memset(&in, 0, sizeof in);
  memset(&out, 0, sizeof out);
  size_t work = 0;
  int vec_halves = a->msg_bytes == 16 ? 8 : 4;
  bool narrow = false;
  for (int i = 0; i < count; ++i) {
    void *input = inputs[i], *output = outputs && outputs[i] ? outputs[i] : inputs[i];
    // calcWorkSize sees one rank's pointers at a time
    const void *table[VR_MAX_RANKS];
    for (int r = 0; r < N; ++r) table[r] = input;
    if (int rc = vr_check_allreduce(algo, N, table, nelems, &work)) return rc;
    for (int r = 0; r < N; ++r) table[r] = output;
    if (int rc = vr_check_allreduce(algo, N, table, nelems, &work)) return rc;
    if (ranges_partially_overlap(output, input, nelems * 2))
      return fail(VR_ERR_OVERLAP, "output partially overlaps input");
    if (widens && (work / 2) % 8 == 0) vec_halves = 8;
    if ((uintptr_t)input % 16 || (uintptr_t)output % 16) narrow = true;
    in.p[first + i] = input;
    out.p[first + i] = output;
  }
  WireSinks k;
  if (int rc = group_sinks(ctx, peer_buf0, peer_buf1, sink_bytes, &k)) return rc;
  vr_geometry geom;
  if (int rc = vr_launch_geometry(algo, N, nelems, &geom)) return rc;
  if (int rc = admit_group_launch(ctx, k.scatter[0], stream, first, count, *seq_no)) return rc;
  const WireLaunch wlch = {&k, nullptr, ctx->status, first, count, false, narrow};
  uint32_t seq = *seq_no, used = 0;
  if (int rc = wire_launch(ctx, (hipStream_t)stream, a, in, out, work, vec_halves, &seq, user_wires, &used,
                           wlch))
    return rc;
  *seq_no = seq + (used > geom.steps ? used : geom.steps);
  if (*seq_no == 0) *seq_no = 1;
  return VR_OK;
}

// The reference's one-rank parameter list: the rank's own sinks beside the peers'.
static int one_rank_tables(const vr_ctx *ctx, int rank, void *scatter_buf, void *gather_buf,
                           void *const peer_buf0[], void *const peer_buf1[], void *p0[], void *p1[]) {
  const int N = ctx ? ctx->nranks : 0;
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  if (rank < 0 || rank >= N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!scatter_buf || !gather_buf || !peer_buf0 || !peer_buf1)
    return fail(VR_ERR_INVALID, "null scratch pointer");
  for (int r = 0; r < N; ++r) {
    p0[r] = r == rank ? scatter_buf : peer_buf0[r];
    p1[r] = r == rank ? gather_buf : peer_buf1[r];
  }
  return VR_OK;
}

static int check_grid(uint32_t groups, uint32_t subgroups, uint32_t simd, uint32_t *wires) {
  // main.cpp:289-291, then allreduce.cpp:852/917.
  if (subgroups % 4 != 0) return fail(VR_ERR_GEOMETRY, "subgroups = " + std::to_string(subgroups));
  if (simd != 16 && simd != 32) return fail(VR_ERR_SUBGROUP, "simd = " + std::to_string(simd));
  if (groups == 0 || subgroups == 0) return fail(VR_ERR_INVALID, "empty grid");
  const uint64_t w = (uint64_t)groups * subgroups;
  *wires = w > 0xffffffffull ? 0xffffffffu : (uint32_t)w;
  return VR_OK;
}

// How many consecutive flag values one rank-group launch of this shape consumes,
// so that a caller who hands out sequence numbers by value (testTransmit's `step`)
// knows how far apart they must lie.
extern "C" int vr_rank_flags_used(vr_ctx *ctx, int algo, size_t nelems, uint32_t groups,
                                  uint32_t subgroups, uint32_t *flags_used) {
  if (!ctx || !flags_used) return fail(VR_ERR_INVALID, "null argument");
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a) return fail(VR_ERR_ALGO, "unknown algo");
  const int N = ctx->nranks;
  const void *table[VR_MAX_RANKS];
  for (int r = 0; r < N; ++r) table[r] = nullptr;          // address 0: aligned to everything
  size_t work = 0;
  if (a->allgather) {
    work = nelems * 2;
    if (work % (size_t)a->msg_bytes) return fail(VR_ERR_UNEVEN, "nelems " + std::to_string(nelems));
  } else if (nelems == 0) {
    *flags_used = 0;
    return VR_OK;
  } else {
    const size_t msgs = nelems * 2 / (size_t)a->msg_bytes;
    if (msgs * (size_t)a->msg_bytes != nelems * 2 || msgs % (size_t)N) return fail(VR_ERR_UNEVEN, "nelems " + std::to_string(nelems));
    work = nelems * 2 / (size_t)N;
  }
  const int vec_halves = a->msg_bytes == 16 || (format_widens_with_alignment(ctx, a) && (work / 2) % 8 == 0) ? 8 : 4;
  WireSinks k;
  const uint32_t wpr_max = wire_wpr_max(ctx);
  k.layout = wl::layout_for(N, wpr_max, true);
  k.wpr_max = wpr_max;
  k.simple_ok = true;
  const uint64_t wires = (uint64_t)groups * subgroups;
  WirePlan plan;
  if (int rc = plan_wire(ctx, a, work, vec_halves, wires > 0xffffffffull ? 0xffffffffu : (uint32_t)wires, k, &plan))
    return rc;
  *flags_used = plan.flags_used;
  return VR_OK;
}

extern "C" int vr_allreduce_rank(vr_ctx *ctx, void *stream, int algo, int rank, void *input,
                                 void *output, void *scatter_buf, void *gather_buf,
                                 void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes,
                                 size_t nelems, uint32_t *seq_no) {
  void *p0[VR_MAX_RANKS] = {}, *p1[VR_MAX_RANKS] = {};
  if (int rc = one_rank_tables(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, p0, p1)) return rc;
  return allreduce_ranks(ctx, stream, algo, rank, 1, &input, &output, p0, p1, sink_bytes, nelems, seq_no, 0);
}

// testTransmit's per-rank form with a user grid (main.cpp:67-71, 289-294): every
// rank launches groups x subgroups sub-groups of `simd` lanes.
extern "C" int vr_allreduce_rank_grid(vr_ctx *ctx, void *stream, int algo, int rank, void *input,
                                      void *output, void *scatter_buf, void *gather_buf,
                                      void *const peer_buf0[], void *const peer_buf1[],
                                      size_t sink_bytes, size_t nelems, uint32_t seq_no,
                                      uint32_t groups, uint32_t subgroups, uint32_t simd) {
  uint32_t wires = 0;
  if (int rc = check_grid(groups, subgroups, simd, &wires)) return rc;
  void *p0[VR_MAX_RANKS] = {}, *p1[VR_MAX_RANKS] = {};
  if (int rc = one_rank_tables(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, p0, p1)) return rc;
  uint32_t seq = seq_no;
  return allreduce_ranks(ctx, stream, algo, rank, 1, &input, &output, p0, p1, sink_bytes, nelems, &seq, wires);
}

extern "C" int vr_allreduce_ranks(vr_ctx *ctx, void *stream, int algo, int first_rank, int nranks_here,
                                  void *const inputs[], void *const outputs[], void *const peer_buf0[],
                                  void *const peer_buf1[], size_t sink_bytes, size_t nelems,
                                  uint32_t *seq_no) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  return allreduce_ranks(ctx, stream, algo, first_rank, nranks_here, inputs, outputs, peer_buf0, peer_buf1,
                         sink_bytes, nelems, seq_no, 0);
}

// Ranks [first, first + count) of the ring all-gather (AllGather(input, output, nelems,
// rank, seqNo, scatterBuf, gatherBuf, peerBuf0, peerBuf1), allgather.hpp:19-29, 58-70).
static int allgather_ranks(vr_ctx *ctx, void *stream, int algo, int first, int count,
                           const void *const inputs[], void *const outputs[], void *const peer_buf0[],
                           void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no,
                           uint32_t user_wires) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || !a->allgather) return fail(VR_ERR_ALGO, "not an all-gather algo");
  const int N = ctx->nranks;
  if (first < 0 || count < 1 || first + count > N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!inputs || !outputs) return fail(VR_ERR_INVALID, "null buffer table");
  if (!seq_no) return fail(VR_ERR_INVALID, "a rank-group launch needs the caller's sequence number");
  const size_t bytes = nelems * 2;
  PtrTable in, out;
  memset(&in, 0, sizeof in);
  memset(&out, 0, sizeof out);
  for (int i = 0; i < count; ++i) {
    const int rank = first + i;
    // allgather.hpp:104-117 for one rank's pointers at a time
    const void *ins[VR_MAX_RANKS];
    void *outs[VR_MAX_RANKS];
    for (int r = 0; r < N; ++r) {
      ins[r] = inputs[i];
      outs[r] = outputs[i];
    }
    if (int rc = vr_check_allgather(algo, N, ins, outs, nelems, nullptr)) return rc;
    const char *own_slot = static_cast<const char *>(outputs[i]) + (size_t)rank * bytes;
    const uintptr_t x = (uintptr_t)inputs[i], y = (uintptr_t)outputs[i];
    if (x < y + bytes * N && y < x + bytes && (const void *)own_slot != inputs[i])
      return fail(VR_ERR_OVERLAP, "input overlaps output other than as its own slot");
    in.p[rank] = const_cast<void *>(inputs[i]);
    out.p[rank] = outputs[i];
  }
  WireSinks k;
  if (int rc = group_sinks(ctx, peer_buf0, peer_buf1, sink_bytes, &k)) return rc;
  vr_geometry geom;
  if (int rc = vr_launch_geometry(algo, N, nelems, &geom)) return rc;
  if (int rc = admit_group_launch(ctx, k.scatter[0], stream, first, count, *seq_no)) return rc;
  const WireLaunch wlch = {&k, nullptr, ctx->status, first, count, false};
  uint32_t seq = *seq_no, used = 0;
  // messages are 16 bytes, so every pointer and the slice allow 16-byte accesses
  if (int rc = wire_launch(ctx, (hipStream_t)stream, a, in, out, bytes, 8, &seq, user_wires, &used, wlch))
    return rc;
  *seq_no = seq + (used > geom.steps ? used : geom.steps);
  if (*seq_no == 0) *seq_no = 1;
  return VR_OK;
}

extern "C" int vr_allgather_rank(vr_ctx *ctx, void *stream, int algo, int rank, const void *input,
                                 void *output, void *scatter_buf, void *gather_buf,
                                 void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes,
                                 size_t nelems, uint32_t *seq_no) {
  void *p0[VR_MAX_RANKS] = {}, *p1[VR_MAX_RANKS] = {};
  if (int rc = one_rank_tables(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, p0, p1)) return rc;
  return allgather_ranks(ctx, stream, algo, rank, 1, &input, &output, p0, p1, sink_bytes, nelems, seq_no, 0);
}

// testAllgather's per-rank form with a user grid (allreduce.cpp:1191-1213, main.cpp:110-166).
extern "C" int vr_allgather_rank_grid(vr_ctx *ctx, void *stream, int algo, int rank, const void *input,
                                      void *output, void *scatter_buf, void *gather_buf,
                                      void *const peer_buf0[], void *const peer_buf1[],
                                      size_t sink_bytes, size_t nelems, uint32_t seq_no,
                                      uint32_t groups, uint32_t subgroups, uint32_t simd) {
  uint32_t wires = 0;
  if (int rc = check_grid(groups, subgroups, simd, &wires)) return rc;
  void *p0[VR_MAX_RANKS] = {}, *p1[VR_MAX_RANKS] = {};
  if (int rc = one_rank_tables(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, p0, p1)) return rc;
  uint32_t seq = seq_no;
  return allgather_ranks(ctx, stream, algo, rank, 1, &input, &output, p0, p1, sink_bytes, nelems, &seq, wires);
}

extern "C" int vr_allgather_ranks(vr_ctx *ctx, void *stream, int algo, int first_rank, int nranks_here,
                                  const void *const inputs[], void *const outputs[],
                                  void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes,
                                  size_t nelems, uint32_t *seq_no) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  return allgather_ranks(ctx, stream, algo, first_rank, nranks_here, inputs, outputs, peer_buf0, peer_buf1,
                         sink_bytes, nelems, seq_no, 0);
}

// Reads one time-out word; if set, resets it and reports the time-out.
static int check_status_word(uint32_t *word, bool *timed_out) {
  uint32_t status = 0;
  HIP_TRY(hipMemcpy(&status, word, sizeof status, hipMemcpyDeviceToHost));
  if (status != 0) {
    HIP_TRY(hipMemset(word, 0, sizeof status));
    HIP_TRY(hipStreamSynchronize(nullptr));
    *timed_out = true;
  }
  return VR_OK;
}

extern "C" int vr_ctx_check(vr_ctx *ctx, void *stream) {
  if (int rc = use_device(ctx)) return rc;
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  bool timed_out = false;
  if (int rc = check_status_word(ctx->status, &timed_out)) return rc;
  if (!timed_out) return VR_OK;
  // A poll gave up: results of that launch are undefined and half-delivered
  // messages may still sit in the sinks.  Scratch the context owns starts over
  // from zeros; vr_allreduce_static clears what it uses in every call anyway; sinks
  // a caller handed to vr_allreduce_rank* / vr_allreduce_ranks are the caller's to
  // zero again.
  if (ctx->wire.ready) {
    if (int rc = wire_clear(ctx->wire.sinks, ctx->nranks, (hipStream_t)stream)) return rc;
    ctx->wire.hist.used = false;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  }
  return fail(VR_ERR_TIMEOUT, std::string("a wire-transport poll exceeded the spin limit; ") +
                                  (ctx->wire.ready ? "the context's own scratch was reset; " : "") +
                                  "caller-owned sinks of rank-group launches must be zeroed again by their owner");
}
