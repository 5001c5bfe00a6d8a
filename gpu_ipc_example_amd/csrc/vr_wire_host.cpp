// Host side of the wire transport: scratch ownership (context, caller, the
// library's fixed region), launch sizing and sequence-number bookkeeping, the
// one-rank entry points and the time-out check.  Kernels: vr_wire.hip.

#include <string.h>

#include <string>

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
  WireHistory *hist;      // null: the caller owns the sinks and the sequence numbers (one-rank launches)
  uint32_t *status;
  int solo_rank;          // >= 0: launch this rank's wires only
  bool always_clear;      // clear the sinks before every launch (fixed scratch shared by contexts)
};

// Launches one wire-transport collective.  `user_wires` (0 = automatic) is the
// number of sub-groups per rank a caller asked for with -g/-w.  *seq_io is the
// first flag value the caller proposes; it is replaced by the one actually used
// (it restarts from 1 when the 32-bit counter would wrap through 0).  Returns
// through *flags_used how many consecutive flag values the launch consumes.
static int wire_launch(vr_ctx *c, hipStream_t s, const AlgoInfo *a, const PtrTable &in,
                       const PtrTable &out, size_t chunk_bytes, int vec_halves, uint32_t *seq_io,
                       uint32_t user_wires, uint32_t *flags_used, const WireLaunch &wlch) {
  uint32_t seq = *seq_io;
  if (seq == 0)
    return fail(VR_ERR_INVALID, "sequence number 0 cannot be told from freshly zeroed scratch");
  const WireSinks &k = *wlch.sinks;
  const int N = c->nranks;
  const WireFlow flow = a->wire_flow();
  WireFormat fmt = a->wire_format();
  const bool big = fmt == WIRE_FMT_RT128 || fmt == WIRE_FMT_RT256;
  if (big && c->tune.wire_fenced == 1) fmt = WIRE_FMT_FLAG;
  // Self-validating 8-byte messages for the Rt64_128 families too: nothing beyond
  // 8-byte store atomicity is assumed, at half the payload per message.
  if (big && c->tune.wire_fenced == 2) fmt = WIRE_FMT_LL;
  if (fmt == WIRE_FMT_LL16 && c->tune.wire_msg16 == 0) fmt = WIRE_FMT_LL;
  if (flow == WIRE_SIMPLE && !k.simple_ok)
    return fail(VR_ERR_INVALID, "these sinks have no room for SimpleTransmit's 2 MiB sender sections");
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
  // `parallel` names the transmit, not a wire format: it takes the reference's
  // 256-byte messages (16 bytes per lane) when every pointer and the chunk allow
  // 16-byte accesses, its 128-byte messages otherwise.
  if (fmt == WIRE_FMT_RT128 && a == &kAlgos[VR_ALGO_PARALLEL] && vec_halves == 8 && chunk_bytes % 16 == 0)
    fmt = WIRE_FMT_RT256;
  const uint32_t psg = flow == WIRE_PARALLEL ? (uint32_t)N : flow == WIRE_BISECT ? (uint32_t)N / 2 : 1u;
  const uint32_t waves_per_block = kWireBlockThreads / 64;
  // Every wave may wait for any other: keep the grid (for one-rank launches: the N
  // grids together) within what the device holds at once.
  int per_cu = 0;
  if (hipError_t e = wire_blocks_per_cu(flow, fmt, vec_halves, N, kWireBlockThreads, c->dtype, &per_cu))
    return fail_hip(e, "occupancy query");
  const uint32_t resident_wpr = (uint32_t)((size_t)c->dev.cus * (size_t)per_cu / (size_t)N) * waves_per_block;
  const uint32_t wpr_cap = k.wpr_max < resident_wpr ? k.wpr_max : resident_wpr;
  const uint32_t wpr_limit = wpr_cap / psg * psg;
  if (wpr_limit < psg) return fail(VR_ERR_INVALID, "sinks or device too small for this rank count");
  const uint32_t wire_bytes = wire_bytes_per_step(fmt, vec_halves);
  const size_t wires_per_chunk = div_up(chunk_bytes, wire_bytes);
  if (wires_per_chunk == 0) { *flags_used = 0; return VR_OK; }
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
  const uint32_t blocks_per_rank = (uint32_t)div_up(wpr, waves_per_block);
  const size_t steps = div_up(wires_per_chunk, wpr / psg);
  const uint32_t nslot_min = 4;
  *flags_used = flow == WIRE_SIMPLE ? (uint32_t)(steps * wpr / wl::kSimplePerSection + 1)
                                    : (uint32_t)((steps - 1) / nslot_min + 1);

  // Flags must strictly increase on every slot and never be 0 (the value of
  // cleared scratch); a different flow or format re-interprets the sinks.  In all
  // those cases start from a clean slate.
  const bool wraps = (uint32_t)(seq + *flags_used) < seq;
  if (wraps && !wlch.hist && !wlch.always_clear)
    return fail(VR_ERR_INVALID, "the sequence number would wrap through 0: zero every rank's scratch "
                                "and restart from 1");
  if (wraps) seq = 1;
  if (wlch.always_clear) {
    if (int rc = wire_clear(k, N, s)) return rc;
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
  args.solo_rank = wlch.solo_rank;
  // Inputs and outputs that cannot stay in the 256 MiB memory-side cache anyway are
  // streamed past it, which leaves that cache to the sinks (measured: faster from
  // 256 MiB of inputs + outputs on, slower below).
  const size_t io_bytes = a->allgather ? (size_t)N * chunk_bytes * (1 + (size_t)N)    // N slices in, N x N out
                                       : 2 * (size_t)N * chunk_bytes * (size_t)N;     // N chunks per rank, in + out
  args.stream_io = c->tune.wire_stream_io >= 0 ? (uint32_t)c->tune.wire_stream_io
                                               : (io_bytes >= (256ull << 20) ? 1u : 0u);
  const bool solo = wlch.solo_rank >= 0;
  // The grid is co-resident by construction; a cooperative launch (on request)
  // lets the runtime check that once more.  One rank's launch cannot vouch for
  // the other ranks' work-groups: always plain.
  const bool cooperative = !solo && c->tune.wire_cooperative == 1;
  const uint32_t blocks = solo ? blocks_per_rank : blocks_per_rank * (uint32_t)N;
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
  const WireLaunch wlch = {&c->wire.sinks, &c->wire.hist, c->status, -1, false};
  return wire_launch(c, s, a, in, out, chunk_bytes, vec_halves, seq_io, user_wires, flags_used, wlch);
}
}  // namespace vr


// The library's fixed scratch region on the context's device: its sinks (for the
// context's rank count) and its status word.
static int static_sinks(const vr_ctx *ctx, WireSinks *k, uint32_t **status) {
  void *fixed = nullptr;
  size_t bytes = 0;
  hipError_t e = wire_static_scratch(ctx->dev.device, &fixed, &bytes);
  if (e != hipSuccess) return fail_hip(e, "hipGetSymbolAddress(scratch)");
  const wl::Layout l = wl::layout_for(ctx->nranks, kStaticWiresPerRank, false);
  if ((size_t)ctx->nranks * l.rank_bytes + 256 > bytes)
    return fail(VR_ERR_INVALID, "the fixed scratch region holds at most " +
                                    std::to_string(kStaticMaxRanks) + " ranks");
  sinks_at(k, ctx->nranks, static_cast<char *>(fixed), l, kStaticWiresPerRank, false);
  *status = reinterpret_cast<uint32_t *>(static_cast<char *>(fixed) + bytes - 256);
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
  uint32_t *status = nullptr;
  if (int rc = static_sinks(ctx, &k, &status)) return rc;
  // The region is shared by every context on the device and keeps the last
  // call's messages: every call clears the sinks first (a fill kernel on the
  // stream), so the flags can start from 1 each time.
  const WireLaunch wlch = {&k, nullptr, status, -1, true};
  uint32_t seq = 1, used = 0;
  ctx->static_used = true;
  return wire_launch(ctx, (hipStream_t)stream, p.a, p.in, p.out, p.chunk_elems * 2, p.vec_halves, &seq,
                     0, &used, wlch);
}

// Caller-owned sinks of a one-rank launch: the rank's own pair and its peers'.
static int rank_sinks(const vr_ctx *ctx, int rank, void *scatter_buf, void *gather_buf,
                      void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes, WireSinks *k) {
  const int N = ctx->nranks;
  if (rank < 0 || rank >= N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!scatter_buf || !gather_buf || !peer_buf0 || !peer_buf1)
    return fail(VR_ERR_INVALID, "null scratch pointer");
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
    k->scatter[r] = r == rank ? scatter_buf : peer_buf0[r];
    k->gather[r] = r == rank ? gather_buf : peer_buf1[r];
    if (!k->scatter[r] || !k->gather[r]) return fail(VR_ERR_INVALID, "null peer sink for rank " + std::to_string(r));
    if ((uintptr_t)k->scatter[r] % 16 || (uintptr_t)k->gather[r] % 16)
      return fail(VR_ERR_UNALIGNED, "sinks must be 16-byte aligned");
  }
  return VR_OK;
}

// One rank of an all-reduce, the form the reference constructs per process
// (allreduce.hpp:18-28, parallel_transmit.hpp:36-60, bisect_transmit.hpp:427-482).
static int allreduce_rank(vr_ctx *ctx, void *stream, int algo, int rank, void *input, void *output,
                          void *scatter_buf, void *gather_buf, void *const peer_buf0[],
                          void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no,
                          uint32_t user_wires) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || a->allgather) return fail(VR_ERR_ALGO, "not an all-reduce algo");
  const int N = ctx->nranks;
  if (rank < 0 || rank >= N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!seq_no) return fail(VR_ERR_INVALID, "a one-rank launch needs the caller's sequence number");
  if (!output) output = input;
  // calcWorkSize sees this rank's pointers only (allreduce.hpp:108-122).
  const void *table[VR_MAX_RANKS];
  for (int r = 0; r < N; ++r) table[r] = input;
  size_t work = 0;
  if (int rc = vr_check_allreduce(algo, N, table, nelems, &work)) return rc;
  for (int r = 0; r < N; ++r) table[r] = output;
  if (int rc = vr_check_allreduce(algo, N, table, nelems, &work)) return rc;
  if (ranges_partially_overlap(output, input, nelems * 2))
    return fail(VR_ERR_OVERLAP, "output partially overlaps input");
  WireSinks k;
  if (int rc = rank_sinks(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, sink_bytes, &k)) return rc;
  PtrTable in, out;
  memset(&in, 0, sizeof in);
  memset(&out, 0, sizeof out);
  in.p[rank] = input;
  out.p[rank] = output;
  const size_t chunk_elems = work / 2;
  // Every rank must pick the same message shape, so the access width may depend on
  // nothing but the element count: 16-byte accesses whenever the chunk is a
  // multiple of 16 bytes, and then this rank's buffers must allow them.
  const int vec_halves = chunk_elems % 8 == 0 ? 8 : 4;
  if (vec_halves == 8 && ((uintptr_t)input % 16 || (uintptr_t)output % 16))
    return fail(VR_ERR_UNALIGNED, "one-rank launches move a chunk that is a multiple of 16 bytes with 16-byte "
                                  "accesses on every rank: input and output must be 16-byte aligned");
  vr_geometry geom;
  if (int rc = vr_launch_geometry(algo, N, nelems, &geom)) return rc;
  const WireLaunch wlch = {&k, nullptr, ctx->status, rank, false};
  uint32_t seq = *seq_no, used = 0;
  if (int rc = wire_launch(ctx, (hipStream_t)stream, a, in, out, chunk_elems * 2, vec_halves, &seq,
                           user_wires, &used, wlch))
    return rc;
  *seq_no = seq + (used > geom.steps ? used : geom.steps);
  if (*seq_no == 0) *seq_no = 1;
  return VR_OK;
}

extern "C" int vr_allreduce_rank(vr_ctx *ctx, void *stream, int algo, int rank, void *input,
                                 void *output, void *scatter_buf, void *gather_buf,
                                 void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes,
                                 size_t nelems, uint32_t *seq_no) {
  return allreduce_rank(ctx, stream, algo, rank, input, output, scatter_buf, gather_buf, peer_buf0,
                        peer_buf1, sink_bytes, nelems, seq_no, 0);
}

// testTransmit's per-rank form with a user grid (main.cpp:67-71, 289-294): every
// rank launches groups x subgroups sub-groups of `simd` lanes.
extern "C" int vr_allreduce_rank_grid(vr_ctx *ctx, void *stream, int algo, int rank, void *input,
                                      void *output, void *scatter_buf, void *gather_buf,
                                      void *const peer_buf0[], void *const peer_buf1[],
                                      size_t sink_bytes, size_t nelems, uint32_t seq_no,
                                      uint32_t groups, uint32_t subgroups, uint32_t simd) {
  if (subgroups % 4 != 0) return fail(VR_ERR_GEOMETRY, "subgroups = " + std::to_string(subgroups));
  if (simd != 16 && simd != 32) return fail(VR_ERR_SUBGROUP, "simd = " + std::to_string(simd));
  if (groups == 0 || subgroups == 0) return fail(VR_ERR_INVALID, "empty grid");
  const uint64_t wires = (uint64_t)groups * subgroups;
  uint32_t seq = seq_no;
  return allreduce_rank(ctx, stream, algo, rank, input, output, scatter_buf, gather_buf, peer_buf0,
                        peer_buf1, sink_bytes, nelems, &seq,
                        wires > 0xffffffffull ? 0xffffffffu : (uint32_t)wires);
}

// One rank of the ring all-gather (AllGather(input, output, nelems, rank, seqNo, scatterBuf,
// gatherBuf, peerBuf0, peerBuf1), allgather.hpp:19-29, 58-70).
extern "C" int vr_allgather_rank(vr_ctx *ctx, void *stream, int algo, int rank, const void *input,
                                 void *output, void *scatter_buf, void *gather_buf,
                                 void *const peer_buf0[], void *const peer_buf1[], size_t sink_bytes,
                                 size_t nelems, uint32_t *seq_no) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || !a->allgather) return fail(VR_ERR_ALGO, "not an all-gather algo");
  const int N = ctx->nranks;
  if (rank < 0 || rank >= N) return fail(VR_ERR_INVALID, "rank out of range");
  if (!seq_no) return fail(VR_ERR_INVALID, "a one-rank launch needs the caller's sequence number");
  // allgather.hpp:104-117 for this rank's pointers
  const void *ins[VR_MAX_RANKS];
  void *outs[VR_MAX_RANKS];
  for (int r = 0; r < N; ++r) {
    ins[r] = input;
    outs[r] = output;
  }
  if (int rc = vr_check_allgather(algo, N, ins, outs, nelems, nullptr)) return rc;
  const size_t bytes = nelems * 2;
  const char *own_slot = static_cast<const char *>(output) + (size_t)rank * bytes;
  const uintptr_t x = (uintptr_t)input, y = (uintptr_t)output;
  if (x < y + bytes * N && y < x + bytes && (const void *)own_slot != input)
    return fail(VR_ERR_OVERLAP, "input overlaps output other than as its own slot");
  WireSinks k;
  if (int rc = rank_sinks(ctx, rank, scatter_buf, gather_buf, peer_buf0, peer_buf1, sink_bytes, &k)) return rc;
  PtrTable in, out;
  memset(&in, 0, sizeof in);
  memset(&out, 0, sizeof out);
  in.p[rank] = const_cast<void *>(input);
  out.p[rank] = output;
  vr_geometry geom;
  if (int rc = vr_launch_geometry(algo, N, nelems, &geom)) return rc;
  const WireLaunch wlch = {&k, nullptr, ctx->status, rank, false};
  uint32_t seq = *seq_no, used = 0;
  // messages are 16 bytes, so every pointer and the slice allow 16-byte accesses
  if (int rc = wire_launch(ctx, (hipStream_t)stream, a, in, out, bytes, 8, &seq, 0, &used, wlch)) return rc;
  *seq_no = seq + (used > geom.steps ? used : geom.steps);
  if (*seq_no == 0) *seq_no = 1;
  return VR_OK;
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
  if (timed_out && ctx->wire.ready) {
    // A poll gave up: results of that launch are undefined and half-delivered
    // messages may still sit in the sinks.  Start over from clean scratch.
    if (int rc = wire_clear(ctx->wire.sinks, ctx->nranks, (hipStream_t)stream)) return rc;
    ctx->wire.hist.used = false;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  }
  if (ctx->static_used) {
    WireSinks k;
    uint32_t *word = nullptr;
    if (int rc = static_sinks(ctx, &k, &word)) return rc;
    if (int rc = check_status_word(word, &timed_out)) return rc;   // its sinks are cleared by every call
  }
  if (timed_out)
    return fail(VR_ERR_TIMEOUT, "a wire-transport poll exceeded the spin limit; scratch was reset");
  return VR_OK;
}
