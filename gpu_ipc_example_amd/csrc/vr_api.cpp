// C ABI of the virtual-rank all-reduce library: validation, dispatch, timing and
// small host utilities.  Device work lives in vr_direct.hip / vr_wire.hip.

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <string>
#include <thread>
#include <vector>

#include "vr_host.h"

using namespace vr;

// ---------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------

static thread_local std::string g_detail;

namespace vr {
int fail(int status, const std::string &detail) {
  g_detail = detail;
  return status;
}

int fail_hip(hipError_t e, const char *what) {
  return fail(VR_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace vr

extern "C" const char *vr_strerror(int status) {
  switch (status) {
    case VR_OK: return "ok";
    case VR_ERR_UNALIGNED: return "We only support aligned pointer for now";
    case VR_ERR_UNEVEN: return "We don't support non-even divide yet";
    case VR_ERR_ALGO: return "Transmit type not support";
    case VR_ERR_TOPOLOGY: return "Unsupported communication topology";
    case VR_ERR_SUBGROUP: return "Unsupported Sub-group size";
    case VR_ERR_GEOMETRY: return "Subgroup numbers must be multiple of 4";
    case VR_ERR_INVALID: return "invalid argument";
    case VR_ERR_HIP: return "HIP runtime error";
    case VR_ERR_NO_DEVICE: return "no gfx950 device";
    case VR_ERR_TIMEOUT: return "flag poll exceeded its spin limit";
    case VR_ERR_OVERLAP: return "output partially overlaps an input";
    default: return "unknown status";
  }
}

extern "C" const char *vr_last_error_detail(void) { return g_detail.c_str(); }
extern "C" const char *vr_version(void) { return "vrank_allreduce 0.1 (gfx950)"; }

// ---------------------------------------------------------------------------------
// algorithm table
// ---------------------------------------------------------------------------------

// message_t / wireCapacity: rt64.hpp:335-340 (8 B, 64 B), rt64_128.hpp:539-551 (8 B, 120 B),
// rt64.hpp:3-20 (16 B, 128 B), rt64_128.hpp:3-30 (16 B, 240 B), bisect_transmit.hpp:17-25.
namespace vr {
const AlgoInfo kAlgos[VR_ALGO_COUNT_] = {
    {"small", T_PARALLEL, 8, 64, false, ORDER_ROTATED, true},
    {"simple", T_PARALLEL, 8, 120, false, ORDER_ROTATED, false},
    {"bisect", T_BISECT, 8, 120, false, ORDER_BISECT, false},
    {"parallel", T_PARALLEL, 8, 120, false, ORDER_ROTATED, false},
    {"small_pcie_p", T_PARALLEL, 16, 128, false, ORDER_ROTATED, true},
    {"simple_pcie_p", T_PARALLEL, 16, 240, false, ORDER_ROTATED, false},
    {"small_ring", T_RING, 16, 128, false, ORDER_ROTATED, true},
    {"simple_ring", T_RING, 16, 240, false, ORDER_ROTATED, false},
    {"small_pcie", T_SEQUENTIAL, 16, 128, false, ORDER_ROTATED, true},
    {"simple_pcie", T_SEQUENTIAL, 16, 240, false, ORDER_ROTATED, false},
    {"allgather_small", T_RING, 16, 128, true, ORDER_ROTATED, true},
    {"allgather_simple", T_RING, 16, 240, true, ORDER_ROTATED, false},
    {"simple_transmit", T_SIMPLE, 8, 120, false, ORDER_ROTATED, false},
};

const AlgoInfo *algo_info(int algo) {
  return (algo >= 0 && algo < VR_ALGO_COUNT_) ? &kAlgos[algo] : nullptr;
}
}  // namespace vr

extern "C" int vr_algo_from_string(const char *name, int *algo_out) {
  if (!name) return fail(VR_ERR_INVALID, "null algo name");
  for (int i = 0; i < VR_ALGO_COUNT_; ++i)
    if (strcmp(name, kAlgos[i].name) == 0) {
      if (algo_out) *algo_out = i;
      return VR_OK;
    }
  return fail(VR_ERR_ALGO, std::string("unknown algo '") + name + "'");
}

extern "C" const char *vr_algo_name(int algo) {
  const AlgoInfo *a = algo_info(algo);
  return a ? a->name : "?";
}

extern "C" int vr_algo_is_allgather(int algo) {
  const AlgoInfo *a = algo_info(algo);
  return a ? (a->allgather ? 1 : 0) : 0;
}

extern "C" size_t vr_algo_message_bytes(int algo) {
  const AlgoInfo *a = algo_info(algo);
  return a ? (size_t)a->msg_bytes : 0;
}

// World sizes each dispatcher switches over (allreduce.cpp:854-881, 1003-1030).
static int check_topology(const AlgoInfo *a, int nranks) {
  const bool ok = (a->transmit == T_BISECT) ? (nranks == 4 || nranks == 8 || nranks == 16)
                                            : (nranks == 2 || nranks == 4 || nranks == 8);
  if (!ok) return fail(VR_ERR_TOPOLOGY, std::string(a->name) + " does not run on " + std::to_string(nranks) + " ranks");
  return VR_OK;
}


// Largest element count per rank: keeps nranks * nelems * 2 bytes (and the
// all-gather's nranks times that) far inside size_t.
static const size_t kMaxElems = (size_t)1 << 40;

// calcWorkSize (allreduce.hpp:108-122): alignment is tested before divisibility.
static int calc_work_size(uintptr_t addr, size_t bytes, size_t nchunks, size_t msg, size_t *work) {
  if (addr % msg != 0) return VR_ERR_UNALIGNED;
  const size_t msgs = div_up(bytes, msg);
  const size_t chunk = div_up(msgs, nchunks);
  if (msgs * msg != bytes || chunk * msg * nchunks > bytes) return VR_ERR_UNEVEN;
  *work = chunk * msg;
  return VR_OK;
}

extern "C" int vr_check_allreduce(int algo, int nranks, const void *const bufs[], size_t nelems,
                                  size_t *work_bytes) {
  const AlgoInfo *a = algo_info(algo);
  if (!a || a->allgather) return fail(VR_ERR_ALGO, "not an all-reduce algo");
  if (!bufs) return fail(VR_ERR_INVALID, "null buffer table");
  if (nelems > kMaxElems) return fail(VR_ERR_INVALID, "nelems too large");
  if (int rc = check_topology(a, nranks)) return rc;
  size_t work = 0;
  for (int r = 0; r < nranks; ++r) {
    if (!bufs[r] && nelems) return fail(VR_ERR_INVALID, "null buffer for rank " + std::to_string(r));
    int rc = calc_work_size((uintptr_t)bufs[r], nelems * 2, (size_t)nranks, (size_t)a->msg_bytes, &work);
    if (rc) return fail(rc, "rank " + std::to_string(r) + ", nelems " + std::to_string(nelems));
  }
  if (work_bytes) *work_bytes = work;
  return VR_OK;
}

extern "C" int vr_check_allgather(int algo, int nranks, const void *const inputs[],
                                  void *const outputs[], size_t nelems, size_t *work_bytes) {
  const AlgoInfo *a = algo_info(algo);
  if (!a || !a->allgather) return fail(VR_ERR_ALGO, "not an all-gather algo");
  if (!inputs || !outputs) return fail(VR_ERR_INVALID, "null buffer table");
  if (nelems > kMaxElems) return fail(VR_ERR_INVALID, "nelems too large");
  if (int rc = check_topology(a, nranks)) return rc;
  size_t work = 0;
  for (int r = 0; r < nranks; ++r) {
    if ((!inputs[r] || !outputs[r]) && nelems) return fail(VR_ERR_INVALID, "null buffer for rank " + std::to_string(r));
    // allgather.hpp:104-117: input and output alignment, then whole messages.
    if ((uintptr_t)inputs[r] % a->msg_bytes || (uintptr_t)outputs[r] % a->msg_bytes)
      return fail(VR_ERR_UNALIGNED, "rank " + std::to_string(r));
    int rc = calc_work_size(0, nelems * 2, 1, (size_t)a->msg_bytes, &work);
    if (rc) return fail(rc, "nelems " + std::to_string(nelems));
  }
  if (work_bytes) *work_bytes = work;
  return VR_OK;
}

extern "C" int vr_launch_geometry(int algo, int nranks, size_t nelems, vr_geometry *out) {
  const AlgoInfo *a = algo_info(algo);
  if (!a || !out) return fail(VR_ERR_INVALID, "bad algo or null output");
  if (int rc = check_topology(a, nranks)) return rc;
  // getLaunchParam (allreduce.hpp:37-62, 237-258; allgather.hpp:32-56), PVC constants.
  const size_t n_threads = 64, max_ss = 64;
  const size_t w = (a->transmit == T_PARALLEL || a->transmit == T_BISECT) ? (size_t)nranks : 1;
  const size_t work = a->allgather ? nelems * 2 : nelems * 2 / (size_t)nranks;
  const size_t wire_per_ss = n_threads / w;
  const size_t n_wire = div_up(work, (size_t)a->wire_capacity);
  const size_t n_ss = div_up(n_wire, wire_per_ss);
  const size_t actual_ss = n_ss < max_ss ? n_ss : max_ss;
  out->steps = actual_ss ? (uint32_t)div_up(n_wire, actual_ss * wire_per_ss) : 0;
  out->subgroups = (uint32_t)(wire_per_ss * w);
  out->groups = (uint32_t)actual_ss;
  return VR_OK;
}

// ---------------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------------

extern "C" int vr_ctx_create(int device, int nranks, vr_ctx **out) {
  if (!out) return fail(VR_ERR_INVALID, "null out");
  *out = nullptr;
  if (!(nranks == 2 || nranks == 4 || nranks == 8 || nranks == 16))
    return fail(VR_ERR_TOPOLOGY, "nranks must be 2, 4, 8 or 16");
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
    (void)hipGetLastError();
    return fail(VR_ERR_NO_DEVICE, "no HIP device visible");
  }
  if (device < 0 || device >= count) return fail(VR_ERR_INVALID, "device index out of range");
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(VR_ERR_NO_DEVICE, std::string("device is ") + prop.gcnArchName + ", kernels are built for gfx950");
  HIP_TRY(hipSetDevice(device));
  // Set-up work that must not happen in a hot call: the context's time-out word,
  // and the device address of the library's fixed scratch region on this device.
  uint32_t *status = nullptr;
  HIP_TRY(hipMalloc((void **)&status, 256));
  hipError_t e = hipMemset(status, 0, 256);
  if (e == hipSuccess) e = hipStreamSynchronize(nullptr);   // the fill has run before any stream may read the word
  void *fixed = nullptr;
  size_t fixed_bytes = 0;
  if (e == hipSuccess) e = wire_static_scratch(device, &fixed, &fixed_bytes);
  if (e != hipSuccess) {
    (void)hipFree(status);
    return fail_hip(e, "vr_ctx_create set-up");
  }
  vr_ctx *c = new vr_ctx;
  c->nranks = nranks;
  c->dev.device = device;
  c->dev.cus = prop.multiProcessorCount;
  c->dev.lds_per_cu = prop.maxSharedMemoryPerMultiProcessor;
  snprintf(c->dev.arch, sizeof c->dev.arch, "%s", prop.gcnArchName);
  c->status = status;
  *out = c;
  return VR_OK;
}

extern "C" int vr_ctx_destroy(vr_ctx *ctx) {
  if (!ctx) return VR_OK;
  wire_free(ctx);
  if (ctx->status) (void)hipFree(ctx->status);
  delete ctx;
  return VR_OK;
}

extern "C" int vr_ctx_nranks(const vr_ctx *ctx) { return ctx ? ctx->nranks : 0; }

extern "C" int vr_ctx_set_dtype(vr_ctx *ctx, int dtype) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  if (dtype != VR_DTYPE_F16 && dtype != VR_DTYPE_BF16) return fail(VR_ERR_INVALID, "unknown element type");
  ctx->dtype = dtype == VR_DTYPE_BF16 ? DT_BF16 : DT_F16;
  return VR_OK;
}

extern "C" int vr_ctx_get_dtype(const vr_ctx *ctx) { return ctx ? (int)ctx->dtype : -1; }

extern "C" int vr_ctx_set_spin_limit(vr_ctx *ctx, uint64_t polls) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  ctx->spin_limit = polls;
  return VR_OK;
}

static int *tuning_field(vr_ctx *ctx, const char *key) {
  if (!ctx || !key) return nullptr;
  if (!strcmp(key, "block")) return &ctx->tune.block;
  if (!strcmp(key, "waves_per_cu")) return &ctx->tune.waves_per_cu;
  if (!strcmp(key, "unroll")) return &ctx->tune.unroll;
  if (!strcmp(key, "nt_load")) return &ctx->tune.nt_load;
  if (!strcmp(key, "nt_store")) return &ctx->tune.nt_store;
  if (!strcmp(key, "oneshot")) return &ctx->tune.oneshot;
  if (!strcmp(key, "segment_kib")) return &ctx->tune.segment_kib;
  if (!strcmp(key, "f16_wide")) return &ctx->tune.f16_wide;
  if (!strcmp(key, "wgs_per_cu")) return &ctx->tune.wgs_per_cu;
  if (!strcmp(key, "deal")) return &ctx->tune.deal;
  if (!strcmp(key, "run")) return &ctx->tune.run;
  if (!strcmp(key, "wire_fenced")) return &ctx->tune.wire_fenced;
  if (!strcmp(key, "wire_cooperative")) return &ctx->tune.wire_cooperative;
  if (!strcmp(key, "wire_blocks_per_cu")) return &ctx->tune.wire_blocks_per_cu;
  if (!strcmp(key, "wire_ahead")) return &ctx->tune.wire_ahead;
  if (!strcmp(key, "wire_msg16")) return &ctx->tune.wire_msg16;
  if (!strcmp(key, "wire_stream_io")) return &ctx->tune.wire_stream_io;
  return nullptr;
}

extern "C" int vr_ctx_set_tuning(vr_ctx *ctx, const char *key, int value) {
  int *f = tuning_field(ctx, key);
  if (!f) return fail(VR_ERR_INVALID, std::string("unknown tuning key ") + (key ? key : "(null)"));
  if (value != -1) {
    if (!strcmp(key, "block") && (value < 64 || value > 1024 || value % 64))
      return fail(VR_ERR_INVALID, "block must be a multiple of 64 in [64,1024]");
    if (!strcmp(key, "waves_per_cu") && (value < 1 || value > 64))
      return fail(VR_ERR_INVALID, "waves_per_cu must be in [1,64]");
    if (!strcmp(key, "unroll") && !(value == 1 || value == 2 || value == 4))
      return fail(VR_ERR_INVALID, "unroll must be 1, 2 or 4");
    if ((!strcmp(key, "nt_load") || !strcmp(key, "oneshot") || !strcmp(key, "wire_msg16") || !strcmp(key, "f16_wide") || !strcmp(key, "wire_stream_io") ||
         !strcmp(key, "wire_cooperative")) &&
        !(value == 0 || value == 1))
      return fail(VR_ERR_INVALID, "flag must be 0, 1 or -1 (automatic)");
    if (!strcmp(key, "wire_fenced") && (value < 0 || value > 4))
      return fail(VR_ERR_INVALID, "wire_fenced must be 0 (embedded flags), 1 (flag words with fences), 2 (8-byte messages), "
                                  "3 (flag words with fences, payload written through), 4 (flag words, agent-scope "
                                  "accesses ordered by store completion) or -1");
    if (!strcmp(key, "nt_store") && (value < 0 || value > 2))
      return fail(VR_ERR_INVALID, "nt_store must be 0 (cached), 1 (streaming), 2 (streaming, written through at agent scope) or -1 (automatic)");
    if (!strcmp(key, "segment_kib") && (value < 1 || value > (1 << 20)))
      return fail(VR_ERR_INVALID, "segment_kib must be in [1, 1048576]");
    if (!strcmp(key, "wgs_per_cu") && (value < 0 || value > 12))
      return fail(VR_ERR_INVALID, "wgs_per_cu must be in [0,12] (0 = no cap)");
    if (!strcmp(key, "deal") && (value < 0 || value > ctx->nranks || (value && ctx->nranks % value)))
      return fail(VR_ERR_INVALID, "deal must be 0 or a divisor of the rank count");
    if (!strcmp(key, "run") && (value < 0 || value > 256 || (value & (value - 1))))
      return fail(VR_ERR_INVALID, "run must be 0 or a power of two up to 256");
    if (!strcmp(key, "wire_ahead") && (value < 1 || value > kWireMaxSlots - 2))
      return fail(VR_ERR_INVALID, "wire_ahead must be in [1,6]");
    if (!strcmp(key, "wire_blocks_per_cu")) {
      if (value < 1 || value > 4) return fail(VR_ERR_INVALID, "wire_blocks_per_cu must be in [1,4]");
      if (ctx->wire.ready) return fail(VR_ERR_INVALID, "wire_blocks_per_cu must be set before vr_ctx_reserve_wire");
    }
  }
  *f = value;
  return VR_OK;
}

extern "C" int vr_ctx_get_tuning(vr_ctx *ctx, const char *key, int *value) {
  int *f = tuning_field(ctx, key);
  if (!f || !value) return fail(VR_ERR_INVALID, "unknown tuning key");
  *value = *f;
  return VR_OK;
}

// ---------------------------------------------------------------------------------
// hot path
// ---------------------------------------------------------------------------------

// Every launch path starts here: kernels go to the context's device whatever the
// calling thread's current device is.
namespace vr {
int use_device(const vr_ctx *ctx) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  HIP_TRY(hipSetDevice(ctx->dev.device));
  return VR_OK;
}

bool ranges_partially_overlap(const void *a, const void *b, size_t bytes) {
  if (a == b) return false;
  const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
  return x < y + bytes && y < x + bytes;
}
}  // namespace vr

// Launch heuristics of the direct kernels.  `read_bytes` / `write_bytes` are the
// distinct bytes a launch reads and writes; what matters is how they compare with
// the 256 MiB memory-side cache (Infinity Cache) in front of HBM.  Store policy 2
// (streaming, written through at agent scope) is the fastest way to HBM but takes
// the results out of the L2 a following in-place launch would read them from.
static Tuning default_tuning(int nranks, const AlgoInfo *a, size_t read_bytes, size_t write_bytes,
                             bool in_place) {
  const size_t kMall = 256ull << 20;
  Tuning t;
  t.block = 256;
  t.unroll = 1;
  t.oneshot = 0;
  if (a->allgather) {
    // One load per lane: the CU's full 32 waves cover the latency.  Each input
    // byte is read once (cached loads measured faster than streaming ones), each
    // output byte is written once and not read back here.
    t.waves_per_cu = 32;
    t.nt_load = 0;
    t.nt_store = 2;
    // From 32 MiB of output on (below, launches are latency-bound and the two grids
    // measure alike; at 32 and 48 MiB the capped one-trip launch is 3 to 17 % faster, on
    // cache-resident and on cold inputs): a one-trip grid (one tile per work-group).  The
    // hardware starts work-groups in index order, so the launch sweeps every stream
    // front to back with all CUs close together, where the work-groups of a
    // persistent grid drift apart: 9 to 20 % faster on inputs no cache holds, as fast
    // or faster when the inputs are cache-resident, slower only for launch-bound sizes.
    // With 48 / N waves per CU or a few more (the stores in flight per CU are what
    // counts: a wave issues N of them per load) and the sources worked on one at a
    // time, another 2 to 12 %.  Cold sets, HIP events, persistent grid -> uncapped
    // one-trip grid -> capped:
    //   4 x 8 MiB 33.4 -> 30.5 -> 29.4 us    4 x 32 MiB 126 -> 108 -> 102.9 us
    //   8 x 4 MiB 62.1 -> 52.7 -> 50.5 us    8 x 16 MiB 233 -> 192.5 -> 189.1 us
    //   2 x 16 MiB 20.2 -> 19.2 -> 18.4 us   2 x 64 MiB 73.2 -> 66.3 -> 64.2 us
    if (write_bytes >= ((size_t)32 << 20)) {
      t.oneshot = 1;
      t.deal = 1;
      const size_t slice = read_bytes / (size_t)nranks;
      switch (nranks) {
        case 2:
          t.block = 512, t.wgs_per_cu = 3;
          break;
        case 4:
          t.block = 256, t.wgs_per_cu = 4;
          break;
        default:  // 8
          if (write_bytes < ((size_t)512 << 20)) t.block = 256, t.wgs_per_cu = 3;
          else t.block = 128, t.wgs_per_cu = 6;
          break;
      }
      // Up to 32 MiB of inputs in all: every XCD takes one contiguous eighth of a slice
      // (runs of tiles / 8 consecutive tiles) instead of every eighth tile.  Alternating
      // runs on one box, without -> with: 4 x 8 MiB 29.8 -> 28.4 us, 4 x 4 MiB 17.2 -> 15.8,
      // 8 x 4 MiB 55.5 -> 50.6, 8 x 2 MiB 30.1 -> 27.0, 8 x 3 MiB 42.1 -> 40.5.  Longer slices gain
      // nothing from runs (4 x 32 MiB) or lose (8 x 8 MiB +5 %, 8 x 16 MiB +9 %).
      if (nranks >= 4 && read_bytes <= ((size_t)32 << 20)) {
        const size_t tiles = slice / ((size_t)t.block * 16);
        int run = 1;
        while ((size_t)run * 2 * 8 <= tiles && run < 256) run *= 2;
        t.run = run;
      }
    }
  } else if (a->latency_tuned && (in_place ? read_bytes : read_bytes + write_bytes) < kMall) {
    // "small" family at the sizes it is meant for: every lane makes one trip;
    // results stay cacheable for the kernel that consumes them next.  (Beyond the
    // cache it streams like the other protocols.)
    t.waves_per_cu = 8;
    t.oneshot = 1;
    t.nt_load = 0;
    t.nt_store = 0;
  } else {
    const size_t footprint = in_place ? read_bytes : read_bytes + write_bytes;
    // Cache-resident shapes: 8 waves per CU, except with eight ranks, where 4 measured
    // equal or up to 5 % faster at every size from 2 to 32 MiB per rank, in place and
    // out of place, and 3 % faster when an in-place 256 MiB set turns out not to be
    // resident after all.
    const int cached_waves = nranks == 8 ? 4 : 8;
    // (A footprint of exactly the cache's size counts as streaming: nothing else may have
    // touched memory for it to be resident, and the streaming launch takes 82 us on eight
    // 32 MiB buffers in place whether they are resident or not, where the cached policy
    // takes 77 us if they are and 93-104 us if they are not.)
    if (footprint < kMall) {             // everything can live in the memory-side cache
      t.waves_per_cu = cached_waves;
      t.nt_load = 0;
      t.nt_store = 1;
      // Out of place with inputs about the size of the L2s together (8 x 4 MiB): results
      // that allocate there push out inputs still to be read; written through, they leave
      // them alone (32 MiB of inputs: 10.1 -> 8.7 us at 8 ranks, 10.3 -> 8.6 at 4, 11.4 -> 9.1
      // at 2; 40 MiB: 1-7 % faster).  Not below: those launches are latency-bound and
      // written-through stores end them 0.3-0.5 us later; no difference beyond.
      const size_t MiB = (size_t)1 << 20;
      if (!in_place && read_bytes > 24 * MiB && read_bytes <= 40 * MiB) t.nt_store = 2;
      // Four ranks, in place, from 96 MiB on: the one-trip grid of the streaming sizes
      // with the cacheable policy.  A little faster than the persistent grid when the data
      // is resident and 4 to 11 % faster when it turns out not to be (96 / 160 / 248 MiB in
      // all, resident: 30.7 -> 30.1, 49.3 -> 48.1, 82.3 -> 79.6 us; not resident: 40.9 -> 39.2,
      // 68.4 -> 61.1, 99.4 -> 89.2 us).  Below 80 MiB the persistent grid leads (48 MiB: 13.8
      // against 19.4 us), at eight ranks it leads throughout, at two the two are even.
      if (in_place && nranks == 4 && footprint >= 96 * MiB)
        t.oneshot = 1, t.block = 64, t.wgs_per_cu = 8, t.deal = 1;
    } else if (read_bytes <= kMall / 2) {  // inputs may still be resident; stream the results past them
      t.waves_per_cu = cached_waves;
      t.nt_load = 0;
      t.nt_store = 2;
    } else {
      // Pure streaming.  DRAM runs best with about 32 loads per CU in flight:
      // N loads per lane times 4 waves (8 waves for two ranks).
      t.waves_per_cu = nranks >= 4 ? 4 : 8;
      t.nt_load = 1;
      t.nt_store = 2;
      // Same sums, computed through binary32: the longer ALU section between a
      // trip's loads and its stores shortens the launch by 2.5 % at 8 ranks (0.5 %
      // at 4; it costs 1-2 % at 2 and 16 ranks and 8 % when the data is cache-resident).
      t.f16_wide = nranks == 4 || nranks == 8;
      // One-trip grids: every work-group handles one tile and ends; the hardware starts
      // work-groups in index order, so the launch sweeps the buffers front to back with
      // all CUs close together, where the work-groups of a persistent grid drift apart.
      // Small work-groups (one wave) with a residency cap of 4 to 8 per CU keep 32 to
      // 64 KiB of loads per CU in flight.  `deal` says how many chunks are worked on at a
      // time, i.e. how many XCDs share a chunk (with eight ranks: deal 8 = every XCD its
      // own chunk, deal 1 = all CUs sweep one chunk after the other, which is what lets
      // the write side of HBM run: eight write streams that all XCDs fill together take
      // 40.6 us for 256 MiB, the same streams filled one XCD per chunk 43-46 us).
      // Measured on cold sets against the persistent grid it replaces (fractions of the
      // HBM peak, HIP events):
      //   2 ranks  0.78 -> 0.82-0.85 (128, 256 MiB per rank)
      //   4 ranks  0.74-0.78 -> 0.82 (64 MiB), 0.75-0.79 -> 0.84 (128 MiB), 0.71 -> 0.84 (256 MiB)
      //   8 ranks  0.72-0.75 -> 0.805 (32 MiB), 0.71 -> 0.79 (40, 48 MiB), 0.73 -> 0.82 (64 MiB),
      //            0.69 -> 0.81 (96 MiB), 0.72-0.74 -> 0.82 (128 MiB), 0.68-0.75 -> 0.81 (256 MiB),
      //            0.69 -> 0.78 (512 MiB)
      //   16 ranks 0.68-0.70 -> 0.75 (16 MiB), 0.72 -> 0.78 (32 MiB), 0.71 -> 0.79 (64 MiB)
      const size_t chunk = read_bytes / ((size_t)nranks * nranks);
      const size_t MiB = (size_t)1 << 20;
      t.oneshot = 1;
      t.unroll = 1;
      switch (nranks) {
        case 2:
          t.block = 512, t.wgs_per_cu = 2;
          break;
        case 4:
          t.block = 64, t.wgs_per_cu = 8, t.deal = 1;
          break;
        case 8:
          t.block = 64, t.deal = 1;
          t.wgs_per_cu = (chunk >= 16 * MiB && chunk <= 32 * MiB) ? 6 : 5;
          break;
        default:   // 16
          t.block = 64, t.wgs_per_cu = 4, t.deal = chunk < 2 * MiB ? 2 : 1;
          break;
      }
    }
  }
  return t;
}

// The same with the context's overrides (vr_ctx_set_tuning) applied.
static Tuning tuning_for(const vr_ctx *ctx, const AlgoInfo *a, size_t read_bytes, size_t write_bytes,
                         bool in_place) {
  Tuning t = default_tuning(ctx->nranks, a, read_bytes, write_bytes, in_place);
  const TuningOverrides &o = ctx->tune;
  if (o.block != -1) t.block = o.block;
  if (o.waves_per_cu != -1) t.waves_per_cu = o.waves_per_cu;
  if (o.unroll != -1) t.unroll = o.unroll;
  if (o.nt_load != -1) t.nt_load = o.nt_load;
  if (o.nt_store != -1) t.nt_store = o.nt_store;
  if (o.oneshot != -1) t.oneshot = o.oneshot;
  if (o.segment_kib != -1) t.segment_bytes = (size_t)o.segment_kib << 10;
  if (o.f16_wide != -1) t.f16_wide = o.f16_wide;
  if (o.wgs_per_cu != -1) t.wgs_per_cu = o.wgs_per_cu;
  if (o.deal != -1) t.deal = o.deal;
  if (o.run != -1) t.run = o.run;
  return t;
}


extern "C" int vr_direct_launch_plan(int algo, int nranks, size_t nelems, int in_place, vr_launch_plan *out) {
  const AlgoInfo *a = algo_info(algo);
  if (!a) return fail(VR_ERR_ALGO, "unknown algo");
  if (!out) return fail(VR_ERR_INVALID, "null plan");
  if (nranks != 2 && nranks != 4 && nranks != 8 && nranks != 16) return fail(VR_ERR_TOPOLOGY, "nranks");
  if (nelems > kMaxElems) return fail(VR_ERR_INVALID, "nelems too large");
  const size_t in_bytes = (size_t)nranks * nelems * 2;
  const Tuning t = a->allgather ? default_tuning(nranks, a, in_bytes, in_bytes * nranks, false)
                                : default_tuning(nranks, a, in_bytes, in_bytes, in_place != 0);
  out->one_trip = t.oneshot;
  out->block = t.block;
  out->unroll = t.unroll;
  out->waves_per_cu = t.oneshot ? 0 : t.waves_per_cu;
  out->wgs_per_cu = t.wgs_per_cu;
  out->deal = t.deal > 0 ? t.deal : nranks;
  out->run = t.run > 1 ? t.run : 1;
  out->nt_load = t.nt_load;
  out->nt_store = t.nt_store;
  out->f16_wide = t.f16_wide;
  return VR_OK;
}

namespace vr {
int prepare_allreduce(vr_ctx *ctx, int algo, void *const bufs[], void *const outs[],
                             size_t nelems, Prepared *p) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || a->allgather) return fail(VR_ERR_ALGO, "not an all-reduce algo");
  const int N = ctx->nranks;
  size_t work = 0;
  if (int rc = vr_check_allreduce(algo, N, (const void *const *)bufs, nelems, &work)) return rc;
  if (outs) {
    if (int rc = vr_check_allreduce(algo, N, (const void *const *)outs, nelems, &work)) return rc;
    for (int r = 0; r < N; ++r)
      for (int q = 0; q < N; ++q) {
        if (ranges_partially_overlap(outs[r], bufs[q], nelems * 2))
          return fail(VR_ERR_OVERLAP, "outs[" + std::to_string(r) + "] vs bufs[" + std::to_string(q) + "]");
        if (r != q && ranges_partially_overlap(outs[r], outs[q], nelems * 2))
          return fail(VR_ERR_OVERLAP, "outs[" + std::to_string(r) + "] vs outs[" + std::to_string(q) + "]");
      }
  }
  p->a = a;
  memset(&p->in, 0, sizeof p->in);
  memset(&p->out, 0, sizeof p->out);
  bool align16 = true;
  for (int r = 0; r < N; ++r) {
    p->in.p[r] = bufs[r];
    p->out.p[r] = outs ? outs[r] : bufs[r];
    align16 = align16 && ((uintptr_t)p->in.p[r] % 16 == 0) && ((uintptr_t)p->out.p[r] % 16 == 0);
  }
  p->chunk_elems = work / 2;
  p->vec_halves = (align16 && p->chunk_elems % 8 == 0) ? 8 : 4;
  p->in_place = true;
  for (int r = 0; r < N; ++r) p->in_place = p->in_place && (p->in.p[r] == p->out.p[r]);
  p->bytes_all_ranks = (size_t)N * nelems * 2;
  return vr_launch_geometry(algo, N, nelems, &p->geom);
}
}  // namespace vr

static int resolve_transport(const AlgoInfo *a, int transport, int *out) {
  if (transport == VR_TRANSPORT_DEFAULT)
    transport = (a == &kAlgos[VR_ALGO_PARALLEL]) ? VR_TRANSPORT_WIRE : VR_TRANSPORT_DIRECT;
  if (transport != VR_TRANSPORT_DIRECT && transport != VR_TRANSPORT_WIRE)
    return fail(VR_ERR_INVALID, "bad transport");
  *out = transport;
  return VR_OK;
}

// Runs one all-reduce starting at sequence number `seq_no`; *next_seq receives
// the sequence number the following launch should start at.
static int run_allreduce(vr_ctx *ctx, hipStream_t s, const Prepared &p, int transport,
                         const Tuning &t, uint32_t seq_no, uint32_t user_wires, uint32_t *next_seq) {
  uint32_t advance = p.geom.steps;  // getLaunchParam: updateSeqNo += nSteps
  *next_seq = seq_no + advance;
  if (*next_seq == 0) *next_seq = 1;   // 0 is the value of cleared scratch: never hand it out
  if (transport == VR_TRANSPORT_WIRE) {
    uint32_t used = 0;
    if (int rc = wire_launch_ctx(ctx, s, p.a, p.in, p.out, p.chunk_elems * 2, p.vec_halves, &seq_no,
                                 user_wires, &used))
      return rc;
    if (used > advance) advance = used;
    *next_seq = seq_no + advance;
    if (*next_seq == 0) *next_seq = 1;
    return VR_OK;
  }
  hipError_t e = launch_direct_allreduce(s, ctx->dev, t, ctx->nranks, p.a->order, ctx->dtype, p.in,
                                         p.out, p.chunk_elems, p.vec_halves);
  if (e != hipSuccess) return fail_hip(e, "launch_direct_allreduce");
  return VR_OK;
}

extern "C" int vr_allreduce(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                            void *const outs[], size_t nelems, uint32_t *seq_no) {
  Prepared p;
  if (int rc = prepare_allreduce(ctx, algo, bufs, outs, nelems, &p)) return rc;
  int tr;
  if (int rc = resolve_transport(p.a, transport, &tr)) return rc;
  uint32_t *seq = seq_no ? seq_no : &ctx->seq_no;
  uint32_t next = *seq;
  if (int rc = run_allreduce(ctx, (hipStream_t)stream, p, tr,
                             tuning_for(ctx, p.a, p.bytes_all_ranks, p.bytes_all_ranks, p.in_place),
                             *seq, 0, &next))
    return rc;
  *seq = next;
  return VR_OK;
}

// The test harness's grid (main.cpp:289-294): rejections in the reference's order
// (main.cpp:289-291, then allreduce.cpp:852/917), then its mapping onto this
// device.  Direct transport: a block holds the same number of lanes (rounded to
// whole waves, at most 1024) and the launch holds ceil(groups / nranks) blocks for
// every virtual rank.  Wire transport: groups x subgroups is the number of
// sub-groups (wires) per rank.
static int apply_user_grid(const vr_ctx *ctx, uint32_t groups, uint32_t subgroups, uint32_t simd,
                           Tuning *t, uint32_t *wires) {
  if (subgroups % 4 != 0) return fail(VR_ERR_GEOMETRY, "subgroups = " + std::to_string(subgroups));
  if (simd != 16 && simd != 32) return fail(VR_ERR_SUBGROUP, "simd = " + std::to_string(simd));
  if (groups == 0 || subgroups == 0) return fail(VR_ERR_INVALID, "empty grid");
  size_t lanes = (size_t)subgroups * simd;
  lanes = ((lanes + 63) / 64) * 64;
  if (lanes > 1024) lanes = 1024;
  t->block = (int)lanes;
  t->unroll = 1;
  t->oneshot = 0;
  t->wgs_per_cu = 0;
  t->deal = 0;
  t->run = 0;
  t->force_blocks_per_rank = (uint32_t)div_up(groups, (size_t)ctx->nranks);
  const uint64_t w = (uint64_t)groups * subgroups;
  *wires = w > 0xffffffffull ? 0xffffffffu : (uint32_t)w;
  return VR_OK;
}

extern "C" int vr_allreduce_grid(vr_ctx *ctx, void *stream, int algo, int transport,
                                 void *const bufs[], void *const outs[], size_t nelems,
                                 uint32_t seq_no, uint32_t groups, uint32_t subgroups,
                                 uint32_t simd) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  Tuning grid;
  uint32_t wires = 0;
  if (int rc = apply_user_grid(ctx, groups, subgroups, simd, &grid, &wires)) return rc;
  Prepared p;
  if (int rc = prepare_allreduce(ctx, algo, bufs, outs, nelems, &p)) return rc;
  int tr;
  if (int rc = resolve_transport(p.a, transport, &tr)) return rc;
  Tuning t = tuning_for(ctx, p.a, p.bytes_all_ranks, p.bytes_all_ranks, p.in_place);
  (void)apply_user_grid(ctx, groups, subgroups, simd, &t, &wires);
  uint32_t next = 0;
  return run_allreduce(ctx, (hipStream_t)stream, p, tr, t, seq_no, wires, &next);
}

struct PreparedGather {
  const AlgoInfo *a;
  PtrTable in, out;
  int vec_halves;
  vr_geometry geom;
};

static int prepare_allgather(vr_ctx *ctx, int algo, const void *const inputs[],
                             void *const outputs[], size_t nelems, PreparedGather *p) {
  if (int rc = use_device(ctx)) return rc;
  const AlgoInfo *a = algo_info(algo);
  if (!a || !a->allgather) return fail(VR_ERR_ALGO, "not an all-gather algo");
  const int N = ctx->nranks;
  if (int rc = vr_check_allgather(algo, N, inputs, outputs, nelems, nullptr)) return rc;
  const size_t bytes = nelems * 2;
  for (int r = 0; r < N; ++r)
    for (int q = 0; q < N; ++q) {
      // input q may be exactly slot q of output r == q; anything else must be disjoint
      const char *slot_q = (const char *)outputs[r] + (size_t)q * bytes;
      const bool same = (const void *)slot_q == inputs[q];
      const uintptr_t x = (uintptr_t)inputs[q], y = (uintptr_t)outputs[r];
      const bool overlap = x < y + bytes * N && y < x + bytes;
      if (overlap && !same) return fail(VR_ERR_OVERLAP, "outputs[" + std::to_string(r) + "] vs inputs[" + std::to_string(q) + "]");
      if (r != q) {
        const uintptr_t z = (uintptr_t)outputs[q];
        if (z < y + bytes * N && y < z + bytes * N) return fail(VR_ERR_OVERLAP, "outputs overlap");
      }
    }
  p->a = a;
  memset(&p->in, 0, sizeof p->in);
  memset(&p->out, 0, sizeof p->out);
  bool align16 = true;
  for (int r = 0; r < N; ++r) {
    p->in.p[r] = const_cast<void *>(inputs[r]);
    p->out.p[r] = outputs[r];
    align16 = align16 && ((uintptr_t)inputs[r] % 16 == 0) && ((uintptr_t)outputs[r] % 16 == 0);
  }
  p->vec_halves = (align16 && nelems % 8 == 0) ? 8 : 4;
  // An 8-byte-granular tail cannot occur: the all-gather messages are 16 bytes.
  return vr_launch_geometry(algo, N, nelems, &p->geom);
}

// Runs one all-gather starting at sequence number `seq_no`; *next_seq receives
// the sequence number the following launch should start at.
static int run_allgather(vr_ctx *ctx, hipStream_t s, const PreparedGather &p, int transport,
                         const Tuning &t, size_t nelems, uint32_t seq_no, uint32_t user_wires,
                         uint32_t *next_seq) {
  if (transport == VR_TRANSPORT_WIRE) {
    uint32_t used = 0, start = seq_no;
    if (int rc = wire_launch_ctx(ctx, s, p.a, p.in, p.out, nelems * 2, p.vec_halves, &start, user_wires, &used))
      return rc;
    *next_seq = start + (used > p.geom.steps ? used : p.geom.steps);
    if (*next_seq == 0) *next_seq = 1;
    return VR_OK;
  }
  if (transport != VR_TRANSPORT_DEFAULT && transport != VR_TRANSPORT_DIRECT) return fail(VR_ERR_INVALID, "bad transport");
  hipError_t e = launch_direct_allgather(s, ctx->dev, t, ctx->nranks, p.in, p.out, nelems, p.vec_halves);
  if (e != hipSuccess) return fail_hip(e, "launch_direct_allgather");
  *next_seq = seq_no + p.geom.steps;
  if (*next_seq == 0) *next_seq = 1;
  return VR_OK;
}

static Tuning allgather_tuning(const vr_ctx *ctx, const AlgoInfo *a, size_t nelems) {
  const size_t in_bytes = (size_t)ctx->nranks * nelems * 2;
  return tuning_for(ctx, a, in_bytes, in_bytes * ctx->nranks, false);
}

extern "C" int vr_allgather(vr_ctx *ctx, void *stream, int algo, int transport,
                            const void *const inputs[], void *const outputs[], size_t nelems,
                            uint32_t *seq_no) {
  PreparedGather p;
  if (int rc = prepare_allgather(ctx, algo, inputs, outputs, nelems, &p)) return rc;
  uint32_t *seq = seq_no ? seq_no : &ctx->seq_no;
  uint32_t next = *seq;
  if (int rc = run_allgather(ctx, (hipStream_t)stream, p, transport, allgather_tuning(ctx, p.a, nelems), nelems,
                             *seq, 0, &next))
    return rc;
  *seq = next;
  return VR_OK;
}

extern "C" int vr_allgather_grid(vr_ctx *ctx, void *stream, int algo, int transport,
                                 const void *const inputs[], void *const outputs[], size_t nelems,
                                 uint32_t seq_no, uint32_t groups, uint32_t subgroups, uint32_t simd) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  Tuning grid;
  uint32_t wires = 0;
  if (int rc = apply_user_grid(ctx, groups, subgroups, simd, &grid, &wires)) return rc;
  PreparedGather p;
  if (int rc = prepare_allgather(ctx, algo, inputs, outputs, nelems, &p)) return rc;
  Tuning t = allgather_tuning(ctx, p.a, nelems);
  (void)apply_user_grid(ctx, groups, subgroups, simd, &t, &wires);
  uint32_t next = 0;
  return run_allgather(ctx, (hipStream_t)stream, p, transport, t, nelems, seq_no, wires, &next);
}

// ---------------------------------------------------------------------------------
// timing
// ---------------------------------------------------------------------------------

template <typename F>
static int time_launches(hipStream_t s, int iters, float *ms_out, F &&launch) {
  if (iters <= 0 || !ms_out) return fail(VR_ERR_INVALID, "iters <= 0 or null ms_out");
  const int kBatch = 128;   // events in flight before the host waits
  std::vector<hipEvent_t> ev(2 * (size_t)kBatch, nullptr);
  int rc = VR_OK;
  for (auto &e : ev) {
    hipError_t err = hipEventCreate(&e);
    if (err != hipSuccess) {
      rc = fail_hip(err, "hipEventCreate");
      break;
    }
  }
  for (int done = 0; done < iters && rc == VR_OK; done += kBatch) {
    const int n = (iters - done < kBatch) ? iters - done : kBatch;
    for (int i = 0; i < n && rc == VR_OK; ++i) {
      if (hipEventRecord(ev[2 * i], s) != hipSuccess) rc = fail(VR_ERR_HIP, "hipEventRecord");
      if (rc == VR_OK) rc = launch();
      if (rc == VR_OK && hipEventRecord(ev[2 * i + 1], s) != hipSuccess) rc = fail(VR_ERR_HIP, "hipEventRecord");
    }
    if (rc != VR_OK) break;
    hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) { rc = fail_hip(e, "hipStreamSynchronize"); break; }
    for (int i = 0; i < n; ++i) {
      float ms = 0.f;
      e = hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]);
      if (e != hipSuccess) { rc = fail_hip(e, "hipEventElapsedTime"); break; }
      ms_out[done + i] = ms;
    }
  }
  for (auto &e : ev)
    if (e) (void)hipEventDestroy(e);
  return rc;
}

extern "C" int vr_time_allreduce(vr_ctx *ctx, void *stream, int algo, int transport,
                                 void *const bufs[], void *const outs[], size_t nelems, int iters,
                                 float *ms_out) {
  Prepared p;
  if (int rc = prepare_allreduce(ctx, algo, bufs, outs, nelems, &p)) return rc;
  int tr;
  if (int rc = resolve_transport(p.a, transport, &tr)) return rc;
  const Tuning t = tuning_for(ctx, p.a, p.bytes_all_ranks, p.bytes_all_ranks, p.in_place);
  hipStream_t s = (hipStream_t)stream;
  return time_launches(s, iters, ms_out, [&]() -> int {
    uint32_t next = ctx->seq_no;
    int rc = run_allreduce(ctx, s, p, tr, t, ctx->seq_no, 0, &next);
    ctx->seq_no = next;
    return rc;
  });
}

extern "C" int vr_time_allgather(vr_ctx *ctx, void *stream, int algo, int transport,
                                 const void *const inputs[], void *const outputs[], size_t nelems,
                                 int iters, float *ms_out) {
  PreparedGather p;
  if (int rc = prepare_allgather(ctx, algo, inputs, outputs, nelems, &p)) return rc;
  const Tuning t = allgather_tuning(ctx, p.a, nelems);
  hipStream_t s = (hipStream_t)stream;
  return time_launches(s, iters, ms_out, [&]() -> int {
    uint32_t next = ctx->seq_no;
    int rc = run_allgather(ctx, s, p, transport, t, nelems, ctx->seq_no, 0, &next);
    ctx->seq_no = next;
    return rc;
  });
}

// Per-launch kernel execution times from events attached to the dispatches
// themselves: what a kernel trace shows, measured in the running program.
template <typename F>
static int time_kernels_attached(hipStream_t s, int iters, float *ms_out, F &&launch) {
  if (iters <= 0 || !ms_out) return fail(VR_ERR_INVALID, "iters <= 0 or null ms_out");
  const int kBatch = 128;
  std::vector<hipEvent_t> ev(2 * (size_t)kBatch, nullptr);
  int rc = VR_OK;
  for (auto &e : ev)
    if (hipError_t err = hipEventCreate(&e); err != hipSuccess) { rc = fail_hip(err, "hipEventCreate"); break; }
  for (int done = 0; done < iters && rc == VR_OK; done += kBatch) {
    const int n = (iters - done < kBatch) ? iters - done : kBatch;
    for (int i = 0; i < n && rc == VR_OK; ++i) {
      tl_kernel_events.start = ev[2 * i];
      tl_kernel_events.stop = ev[2 * i + 1];
      rc = launch();
      tl_kernel_events = KernelEvents();
    }
    if (rc != VR_OK) break;
    if (hipError_t e = hipStreamSynchronize(s); e != hipSuccess) { rc = fail_hip(e, "hipStreamSynchronize"); break; }
    for (int i = 0; i < n; ++i) {
      float ms = 0.f;
      if (hipError_t e = hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]); e != hipSuccess) {
        rc = fail_hip(e, "hipEventElapsedTime (kernel-attached events)");
        break;
      }
      ms_out[done + i] = ms;
    }
  }
  tl_kernel_events = KernelEvents();
  for (auto &e : ev)
    if (e) (void)hipEventDestroy(e);
  return rc;
}

extern "C" int vr_time_allreduce_kernel(vr_ctx *ctx, void *stream, int algo, int transport,
                                        void *const bufs[], void *const outs[], size_t nelems,
                                        int iters, float *ms_out) {
  Prepared p;
  if (int rc = prepare_allreduce(ctx, algo, bufs, outs, nelems, &p)) return rc;
  int tr;
  if (int rc = resolve_transport(p.a, transport, &tr)) return rc;
  const Tuning t = tuning_for(ctx, p.a, p.bytes_all_ranks, p.bytes_all_ranks, p.in_place);
  hipStream_t s = (hipStream_t)stream;
  return time_kernels_attached(s, iters, ms_out, [&]() -> int {
    uint32_t next = ctx->seq_no;
    int rc = run_allreduce(ctx, s, p, tr, t, ctx->seq_no, 0, &next);
    ctx->seq_no = next;
    return rc;
  });
}

extern "C" int vr_time_allgather_kernel(vr_ctx *ctx, void *stream, int algo, int transport,
                                        const void *const inputs[], void *const outputs[],
                                        size_t nelems, int iters, float *ms_out) {
  PreparedGather p;
  if (int rc = prepare_allgather(ctx, algo, inputs, outputs, nelems, &p)) return rc;
  const Tuning t = allgather_tuning(ctx, p.a, nelems);
  hipStream_t s = (hipStream_t)stream;
  return time_kernels_attached(s, iters, ms_out, [&]() -> int {
    uint32_t next = ctx->seq_no;
    int rc = run_allgather(ctx, s, p, transport, t, nelems, ctx->seq_no, 0, &next);
    ctx->seq_no = next;
    return rc;
  });
}

// `groups` event pairs, each around `per_group` back-to-back vr_allreduce calls made
// exactly as a caller makes them (validation, launch heuristics and launch in every
// call).  ms_out[g] = device time of group g divided by per_group; *host_call_us
// (optional) = host wall time one vr_allreduce call took to return, averaged over
// all of them.
extern "C" int vr_time_allreduce_grouped(vr_ctx *ctx, void *stream, int algo, int transport,
                                         void *const bufs[], void *const outs[], size_t nelems,
                                         int groups, int per_group, float *ms_out,
                                         double *host_call_us) {
  if (!ctx) return fail(VR_ERR_INVALID, "null ctx");
  if (groups <= 0 || per_group <= 0 || !ms_out) return fail(VR_ERR_INVALID, "groups, per_group > 0 and ms_out");
  if (groups > 4096) return fail(VR_ERR_INVALID, "at most 4096 groups");
  if (int rc = use_device(ctx)) return rc;
  hipStream_t s = (hipStream_t)stream;
  std::vector<hipEvent_t> ev(2 * (size_t)groups, nullptr);
  int rc = VR_OK;
  for (auto &e : ev)
    if (hipError_t err = hipEventCreate(&e); err != hipSuccess) { rc = fail_hip(err, "hipEventCreate"); break; }
  double host_s = 0.0;
  for (int g = 0; g < groups && rc == VR_OK; ++g) {
    if (hipEventRecord(ev[2 * g], s) != hipSuccess) rc = fail(VR_ERR_HIP, "hipEventRecord");
    timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int i = 0; i < per_group && rc == VR_OK; ++i)
      rc = vr_allreduce(ctx, stream, algo, transport, bufs, outs, nelems, nullptr);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    host_s += (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    if (rc == VR_OK && hipEventRecord(ev[2 * g + 1], s) != hipSuccess) rc = fail(VR_ERR_HIP, "hipEventRecord");
    // keep the queue short: a group is waited for before the one after next is issued
    if (rc == VR_OK && g >= 1)
      if (hipError_t err = hipEventSynchronize(ev[2 * (g - 1) + 1]); err != hipSuccess) rc = fail_hip(err, "hipEventSynchronize");
  }
  if (rc == VR_OK)
    if (hipError_t err = hipStreamSynchronize(s); err != hipSuccess) rc = fail_hip(err, "hipStreamSynchronize");
  for (int g = 0; g < groups && rc == VR_OK; ++g) {
    float ms = 0.f;
    if (hipError_t err = hipEventElapsedTime(&ms, ev[2 * g], ev[2 * g + 1]); err != hipSuccess) {
      rc = fail_hip(err, "hipEventElapsedTime");
      break;
    }
    ms_out[g] = ms / (float)per_group;
  }
  for (auto &e : ev)
    if (e) (void)hipEventDestroy(e);
  if (rc == VR_OK && host_call_us) *host_call_us = host_s * 1e6 / ((double)groups * per_group);
  return rc;
}

// The probes are pure streaming: streaming loads, streaming agent-scope stores, as
// one-trip grids (one tile per work-group, started in index order, so the launch
// sweeps the buffer front to back) with the residency that measured best for each:
// a 1:1 copy with six 256-lane work-groups per CU (6.87 TB/s against 6.3 for the
// best persistent grid), reads with two 256-lane work-groups of four vectors per
// lane (7.3 against 6.9), writes with eight 128-lane work-groups (7.4 against 6.6).
static int copy_tuning(vr_ctx *ctx, void *dst, const void *src, size_t bytes, int mode, Tuning *t) {
  if (!ctx || !dst || !src) return fail(VR_ERR_INVALID, "null argument");
  if (int rc = use_device(ctx)) return rc;
  if (bytes % 16 || (uintptr_t)dst % 16 || (uintptr_t)src % 16)
    return fail(VR_ERR_UNALIGNED, "copy wants 16-byte granules");
  Tuning d;
  d.block = mode == 2 ? 128 : 256;
  d.waves_per_cu = mode == 0 ? 4 : 16;     // (persistent grids only: "oneshot" = 0)
  d.unroll = mode == 1 ? 4 : 1;
  d.nt_load = 1;
  d.nt_store = 2;
  d.oneshot = 1;
  d.wgs_per_cu = mode == 0 ? 6 : mode == 1 ? 2 : 8;
  const TuningOverrides &o = ctx->tune;
  if (o.block != -1) d.block = o.block;
  if (o.waves_per_cu != -1) d.waves_per_cu = o.waves_per_cu;
  if (o.unroll != -1) d.unroll = o.unroll;
  if (o.nt_load != -1) d.nt_load = o.nt_load;
  if (o.nt_store != -1) d.nt_store = o.nt_store;
  if (o.segment_kib != -1) d.segment_bytes = (size_t)o.segment_kib << 10;
  if (o.oneshot != -1) d.oneshot = o.oneshot;
  if (o.wgs_per_cu != -1) d.wgs_per_cu = o.wgs_per_cu;
  *t = d;
  return VR_OK;
}

extern "C" int vr_stream_probe(vr_ctx *ctx, void *stream, int mode, void *dst, const void *src,
                               size_t bytes) {
  Tuning t;
  if (mode < 0 || mode > 2) return fail(VR_ERR_INVALID, "bad probe mode");
  if (int rc = copy_tuning(ctx, dst, src, bytes, mode, &t)) return rc;
  hipError_t e = launch_copy((hipStream_t)stream, ctx->dev, t, dst, src, bytes, mode);
  return e == hipSuccess ? VR_OK : fail_hip(e, "launch_copy");
}

extern "C" int vr_stream_probe_multi(vr_ctx *ctx, void *stream, void *const dsts[],
                                     const void *const srcs[], size_t bytes_each) {
  if (int rc = use_device(ctx)) return rc;
  if (!dsts || !srcs) return fail(VR_ERR_INVALID, "null table");
  const int N = ctx->nranks;
  if (bytes_each % (16 * (size_t)N)) return fail(VR_ERR_UNEVEN, "bytes per stream must be a multiple of 16 * nranks");
  PtrTable in, out;
  memset(&in, 0, sizeof in);
  memset(&out, 0, sizeof out);
  for (int r = 0; r < N; ++r) {
    if (!dsts[r] || !srcs[r]) return fail(VR_ERR_INVALID, "null stream pointer");
    if ((uintptr_t)dsts[r] % 16 || (uintptr_t)srcs[r] % 16) return fail(VR_ERR_UNALIGNED, "16-byte alignment");
    in.p[r] = const_cast<void *>(srcs[r]);
    out.p[r] = dsts[r];
  }
  // Exactly the launch an out-of-place all-reduce of this size would get.
  const size_t all = (size_t)N * bytes_each;
  const Tuning t = tuning_for(ctx, &kAlgos[VR_ALGO_BISECT], all, all, false);
  hipError_t e = launch_direct_allreduce((hipStream_t)stream, ctx->dev, t, N, ORDER_COPY, DT_F16, in, out,
                                         bytes_each / 2 / (size_t)N, 8);
  return e == hipSuccess ? VR_OK : fail_hip(e, "launch_direct_allreduce (copy yardstick)");
}

extern "C" int vr_probe_xcc_ids(vr_ctx *ctx, uint32_t blocks, uint32_t *ids_host) {
  if (!ids_host || blocks == 0 || blocks > 65536) return fail(VR_ERR_INVALID, "bad argument");
  if (int rc = use_device(ctx)) return rc;
  uint32_t *d = nullptr;
  HIP_TRY(hipMalloc((void **)&d, (size_t)blocks * 4));
  hipError_t e = launch_xcc_probe(nullptr, blocks, d);
  if (e == hipSuccess) e = hipMemcpy(ids_host, d, (size_t)blocks * 4, hipMemcpyDeviceToHost);
  (void)hipFree(d);
  return e == hipSuccess ? VR_OK : fail_hip(e, "xcc probe");
}

extern "C" int vr_time_copy(vr_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes,
                            int iters, float *ms_out) {
  Tuning t;
  if (int rc = copy_tuning(ctx, dst, src, bytes, 0, &t)) return rc;
  hipStream_t s = (hipStream_t)stream;
  return time_launches(s, iters, ms_out, [&]() -> int {
    hipError_t e = launch_copy(s, ctx->dev, t, dst, src, bytes);
    return e == hipSuccess ? VR_OK : fail_hip(e, "launch_copy");
  });
}

// ---------------------------------------------------------------------------------
// host helpers
// ---------------------------------------------------------------------------------

// double -> binary16, one rounding (round-to-nearest-even), overflow to infinity.
static uint16_t f64_to_f16(double d) {
  if (d != d) return 0x7e00;
  const uint16_t sign = signbit(d) ? 0x8000 : 0;
  const double a = fabs(d);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00);
  if (a == 0.0) return sign;
  int ex;
  (void)frexp(a, &ex);
  int e = ex - 1;
  if (e < -14) e = -14;
  const uint32_t q = (uint32_t)nearbyint(ldexp(a, 10 - e));
  uint32_t bits = (e == -14 && q < 1024) ? q : (((uint32_t)(e + 15) << 10) + q - 1024);
  if (bits >= 0x7c00) bits = 0x7c00;
  return (uint16_t)(sign | bits);
}

// double -> bfloat16, one rounding (round-to-nearest-even), overflow to infinity.
static uint16_t f64_to_bf16(double d) {
  if (d != d) return 0x7fc0;
  const uint16_t sign = signbit(d) ? 0x8000 : 0;
  const double a = fabs(d);
  if (a == 0.0) return sign;
  if (a >= 0x1.ffp127) return (uint16_t)(sign | 0x7f80);
  int ex;
  (void)frexp(a, &ex);
  int e = ex - 1;
  if (e < -126) e = -126;
  const uint32_t q = (uint32_t)nearbyint(ldexp(a, 7 - e));
  uint32_t bits = (e == -126 && q < 128) ? q : (((uint32_t)(e + 127) << 7) + q - 128);
  if (bits >= 0x7f80) bits = 0x7f80;
  return (uint16_t)(sign | bits);
}

static inline uint16_t f64_to_elem(int dtype, double d) {
  return dtype == VR_DTYPE_BF16 ? f64_to_bf16(d) : f64_to_f16(d);
}

extern "C" void vr_fill_pattern_dt(int dtype, uint16_t *host_buf, int rank, size_t n) {
  for (size_t i = 0; i < n; ++i) host_buf[i] = f64_to_elem(dtype, (double)((int)(i % 32) * (rank + 1)));
}

extern "C" void vr_fill_pattern(uint16_t *host_buf, int rank, size_t n) {
  vr_fill_pattern_dt(VR_DTYPE_F16, host_buf, rank, n);
}

static inline uint64_t splitmix64_at(uint64_t seed, uint64_t k) {
  uint64_t z = seed + (k + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

extern "C" void vr_generate(uint16_t *host_buf, size_t n, uint64_t seed, int dist, double p0,
                            double p1) {
  vr_generate_dt(VR_DTYPE_F16, host_buf, n, seed, dist, p0, p1);
}

static void generate_range(int dtype, uint16_t *host_buf, size_t begin, size_t end, uint64_t seed, int dist,
                           double p0, double p1) {
  for (size_t i = begin; i < end; ++i) {
    const uint64_t z0 = splitmix64_at(seed, 2 * (uint64_t)i);
    const uint64_t z1 = splitmix64_at(seed, 2 * (uint64_t)i + 1);
    double x;
    if (dist == 0) {
      x = p0 + (p1 - p0) * ((double)(z0 >> 11) * 0x1.0p-53);
    } else {
      const double u1 = (double)((z0 >> 11) + 1) * 0x1.0p-53;
      const double u2 = (double)(z1 >> 11) * 0x1.0p-53;
      x = p0 + p1 * (sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2));
    }
    host_buf[i] = f64_to_elem(dtype, x);
  }
}

// Element i depends on (seed, i) only, so large buffers are filled by several
// host threads, each on a contiguous range; the result does not depend on how
// many there are.
extern "C" void vr_generate_dt(int dtype, uint16_t *host_buf, size_t n, uint64_t seed, int dist,
                               double p0, double p1) {
  size_t threads = n >> 20;                           // at least 1 Mi elements per thread
  const size_t hw = std::thread::hardware_concurrency();
  if (threads > hw) threads = hw;
  if (threads > 16) threads = 16;
  if (threads <= 1) {
    generate_range(dtype, host_buf, 0, n, seed, dist, p0, p1);
    return;
  }
  std::vector<std::thread> pool;
  const size_t per = (n + threads - 1) / threads;
  for (size_t t = 0; t < threads; ++t) {
    const size_t b = t * per, e = b + per < n ? b + per : n;
    if (b < e) pool.emplace_back(generate_range, dtype, host_buf, b, e, seed, dist, p0, p1);
  }
  for (auto &th : pool) th.join();
}

extern "C" int vr_parse_nelems(const char *text, size_t *out) {
  if (!text || !out) return fail(VR_ERR_INVALID, "null argument");
  // main.cpp:17-34: the last K / M / G anywhere in the string picks the base,
  // the leading digits are the count ("8MB" -> 8 * 1024 * 1024).
  size_t base = 1;
  if (strrchr(text, 'K')) base = 1024ull;
  else if (strrchr(text, 'M')) base = 1024ull * 1024;
  else if (strrchr(text, 'G')) base = 1024ull * 1024 * 1024;
  char *end = nullptr;
  const unsigned long long v = strtoull(text, &end, 10);
  if (end == text) return fail(VR_ERR_INVALID, std::string("no digits in '") + text + "'");
  *out = (size_t)v * base;
  return VR_OK;
}

extern "C" int vr_device_count(int *count) {
  if (!count) return fail(VR_ERR_INVALID, "null argument");
  if (hipGetDeviceCount(count) != hipSuccess) {
    (void)hipGetLastError();
    *count = 0;
  }
  return VR_OK;
}

extern "C" int vr_device_name(int device, char *buf, size_t buflen) {
  if (!buf || !buflen) return fail(VR_ERR_INVALID, "null argument");
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  snprintf(buf, buflen, "%s (%s, %d CUs, %zu KiB LDS per CU)", prop.name, prop.gcnArchName, prop.multiProcessorCount,
           (size_t)prop.maxSharedMemoryPerMultiProcessor >> 10);
  return VR_OK;
}

extern "C" int vr_malloc(int device, size_t bytes, void **out) {
  if (!out) return fail(VR_ERR_INVALID, "null argument");
  HIP_TRY(hipSetDevice(device));
  HIP_TRY(hipMalloc(out, bytes ? bytes : 16));
  return VR_OK;
}

extern "C" int vr_free(void *ptr) {
  if (ptr) HIP_TRY(hipFree(ptr));
  return VR_OK;
}

extern "C" int vr_memset(void *ptr, int value, size_t bytes) {
  HIP_TRY(hipMemset(ptr, value, bytes));
  // hipMemset of device memory may return before the fill has run; callers zero
  // scratch that kernels on other streams, or other processes, write into next.
  HIP_TRY(hipStreamSynchronize(nullptr));
  return VR_OK;
}

extern "C" int vr_copy_to_device(void *dst, const void *src_host, size_t bytes) {
  HIP_TRY(hipMemcpy(dst, src_host, bytes, hipMemcpyHostToDevice));
  return VR_OK;
}

extern "C" int vr_copy_to_host(void *dst_host, const void *src, size_t bytes) {
  HIP_TRY(hipMemcpy(dst_host, src, bytes, hipMemcpyDeviceToHost));
  return VR_OK;
}

extern "C" int vr_stream_create(int device, void **stream_out) {
  if (!stream_out) return fail(VR_ERR_INVALID, "null argument");
  HIP_TRY(hipSetDevice(device));
  hipStream_t s;
  HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream_out = s;
  return VR_OK;
}

extern "C" int vr_stream_destroy(void *stream) {
  if (stream) HIP_TRY(hipStreamDestroy((hipStream_t)stream));
  return VR_OK;
}

extern "C" int vr_stream_sync(void *stream) {
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return VR_OK;
}

extern "C" int vr_event_create(void **event_out) {
  if (!event_out) return fail(VR_ERR_INVALID, "null argument");
  hipEvent_t e;
  HIP_TRY(hipEventCreate(&e));
  *event_out = e;
  return VR_OK;
}

extern "C" int vr_event_record(void *event, void *stream) {
  HIP_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return VR_OK;
}

extern "C" int vr_event_elapsed_ms(void *start, void *stop, float *ms_out) {
  if (!ms_out) return fail(VR_ERR_INVALID, "null argument");
  HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
  HIP_TRY(hipEventElapsedTime(ms_out, (hipEvent_t)start, (hipEvent_t)stop));
  return VR_OK;
}

extern "C" int vr_event_destroy(void *event) {
  if (event) HIP_TRY(hipEventDestroy((hipEvent_t)event));
  return VR_OK;
}
