// Internal interface between the C ABI (vr_api.cpp, vr_wire_host.cpp) and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "vrank_allreduce.h"
#include "vr_wire_layout.h"

namespace vr {

// Device pointers of all virtual ranks, passed to kernels by value (like the
// reference functor's by-value pointer tables, parallel_transmit.hpp:134-145).
struct PtrTable {
  void *p[VR_MAX_RANKS];
};

enum DType : int {
  DT_F16 = 0,   // IEEE binary16, added with v_pk_add_f16
  DT_BF16 = 1,  // bfloat16, added as binary32 and rounded to nearest even (v_cvt_pk_bf16_f32)
  // binary16 added as binary32 and rounded back after every add.  Bit-identical to
  // DT_F16: a binary32 sum of two binary16 values is exact or correctly rounded
  // with 24 >= 2 * 11 + 2 significand bits, so the second rounding is innocuous.
  // The longer ALU section paces the streaming loop better (measured).
  DT_F16_WIDE = 2,
};

enum Order : int {
  ORDER_ROTATED = 0,  // chain from the chunk owner: parallel/sequential/ring/simple transmit
  ORDER_BISECT = 1,   // pair sums, then chain over pairs: BisectPTransmit
  ORDER_COPY = 2,     // yardstick: no adds, output k receives input k (same launch shape and traffic)
};

struct Tuning {
  int block = 512;        // threads per work-group
  int waves_per_cu = 32;  // resident waves per CU the persistent grid asks for
  int unroll = 2;         // 16-byte vectors in flight per lane and rank
  int nt_load = 1;         // 1: streaming loads (nt)
  int nt_store = 1;        // 1: streaming stores (nt); 2: streaming and written through at agent scope (nt sc1)
  size_t segment_bytes = 1ull << 30;  // bytes of a chunk one launch addresses (32-bit offsets); multiple of 16
  int oneshot = 0;        // 1: grid covers the whole buffer, no grid-stride loop
  int f16_wide = 0;       // 1: binary16 adds through binary32 (same bits, longer ALU section)
  uint32_t force_blocks_per_rank = 0;  // non-zero: use exactly this many blocks per rank
  int deal = 0;           // chunks the work-groups of an all-reduce work on at a time (a divisor of the rank
                          // count; 0 = all of them: work-group b serves owner b % N throughout)
  int run = 0;            // all-gather, one source at a time: each XCD takes runs of this many consecutive
                          // tiles (a power of two) instead of every eighth tile; 0 or 1 = no permutation
  int wgs_per_cu = 0;     // non-zero: at most this many work-groups of the launch share a CU (the launch
                          // asks for dynamic LDS it never touches, so that no more fit); for one-trip grids,
                          // whose residency the grid size does not bound
};

struct DeviceInfo {
  int device = 0;
  int cus = 0;
  size_t lds_per_cu = 0;   // bytes of LDS a compute unit has
  char arch[64] = {0};
};

// Events to attach to the next collective's kernel dispatches on this host thread
// (hipExtLaunchKernel): `start` is stamped when the first kernel of the collective
// begins to execute, `stop` when its last kernel ends, from the dispatches' own
// timestamps, the counterpart of the reference's SYCL event profiling
// (main.cpp:36-43).  Both null (the default): plain launches.
struct KernelEvents {
  hipEvent_t start = nullptr, stop = nullptr;
};
extern thread_local KernelEvents tl_kernel_events;

// Direct transport -----------------------------------------------------------
// in/out hold nranks pointers; chunk_elems = nelems / nranks; vec_halves is 8
// (16-byte accesses) or 4 (8-byte accesses, for chunks or pointers that are only
// 8-byte aligned).
hipError_t launch_direct_allreduce(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   Order order, DType dtype, const PtrTable &in, const PtrTable &out,
                                   size_t chunk_elems, int vec_halves);
hipError_t launch_direct_allgather(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   const PtrTable &in, const PtrTable &out, size_t nelems,
                                   int vec_halves);
// mode: 0 copy, 1 read only, 2 write only
hipError_t launch_copy(hipStream_t s, const DeviceInfo &dev, const Tuning &t, void *dst,
                       const void *src, size_t bytes, int mode = 0);


hipError_t launch_xcc_probe(hipStream_t s, uint32_t blocks, uint32_t *out_device);

// Wire transport ------------------------------------------------------------------
enum WireFlow : int { WIRE_PARALLEL, WIRE_SEQUENTIAL, WIRE_RING, WIRE_BISECT, WIRE_ALLGATHER, WIRE_SIMPLE };
enum WireFormat : int {
  WIRE_FMT_LL = 0,    // 4 B payload + 4 B flag per 8-byte store (Rt64 family)
  WIRE_FMT_RT128 = 1, // the reference's 128-byte message: 120 B payload, a flag per 64-byte half (Rt64_128)
  WIRE_FMT_FLAG = 2,  // 16 B payload lines + one fenced flag word per message
  WIRE_FMT_LL16 = 3,  // 8 B payload + the flag twice per 16-byte store (Rt64_PCIE family)
  WIRE_FMT_RT256 = 4, // the reference's 256-byte message: 240 B payload, a flag per 64 bytes (Rt64_128_PCIE)
  WIRE_FMT_FLAG_WT = 5,      // WIRE_FMT_FLAG with the payload stored written through at agent scope
  WIRE_FMT_FLAG_SCOPED = 6,  // flag words, every access at agent scope, ordered by store completion: no fences
};
static inline bool wire_fmt_is_flag(int fmt) {
  return fmt == WIRE_FMT_FLAG || fmt == WIRE_FMT_FLAG_WT || fmt == WIRE_FMT_FLAG_SCOPED;
}
constexpr int kWireMaxSlots = 8;     // deepest slot ring any flow uses

struct WireArgs {
  PtrTable in, out;          // per-rank input / output (only the entries of the ranks the launch holds)
  PtrTable scatter, gather;  // per-rank sinks (the reference's peerBuf0[] / peerBuf1[])
  size_t flag_off;           // byte offset of the flag words inside a sink (WIRE_FMT_FLAG)
  size_t chunk_bytes;        // bytes per rank-chunk (all-gather: bytes of one slice)
  uint32_t waves_per_rank;   // wires each virtual rank runs (multiple of the flow's waves per column)
  uint32_t seq;              // first flag value of this launch
  uint32_t spin_limit;
  uint32_t ahead;            // steps the scatters of the parallel flow run ahead of its gathers
  int rank_first, rank_count; // the grid holds the wires of ranks [rank_first, rank_first + rank_count):
                             // block b is rank rank_first + b % rank_count (all ranks: 0, N)
  uint32_t stream_io;        // 1: inputs are loaded and outputs stored with streaming cache policies
  uint32_t io_narrow;        // 1: this launch's inputs / outputs are only 8-byte aligned: a lane's 16 bytes
                             //    travel as two 8-byte accesses (the messages are the same)
  uint32_t *status;          // non-zero once any poll gave up
};

uint32_t wire_bytes_per_step(WireFormat fmt, int vec_halves);
// Work-groups of the flow's kernel one compute unit holds at once (occupancy query).
hipError_t wire_blocks_per_cu(WireFlow flow, WireFormat fmt, int vec_halves, int nranks,
                              uint32_t block_threads, DType dtype, int *per_cu);
// cooperative: hipLaunchCooperativeKernel instead of a plain launch.
hipError_t launch_wire(hipStream_t s, WireFlow flow, WireFormat fmt, int vec_halves, int nranks,
                       uint32_t blocks, uint32_t block_threads, WireArgs &args, bool cooperative,
                       DType dtype);
hipError_t launch_wire_clear(hipStream_t s, void *p, size_t bytes);
// Bytes of a message slot in the sinks for a format.
uint32_t wire_slot_bytes(WireFormat fmt, int vec_halves);
// Clears, in every rank's scatter and gather sink, the first `slot_bytes` bytes
// and `flag_bytes` bytes of flag words at `flag_off`.
hipError_t launch_wire_clear_sinks(hipStream_t s, const PtrTable &scatter, const PtrTable &gather, int nranks,
                                   size_t slot_bytes, size_t flag_off, size_t flag_bytes);
// The library's own fixed scratch region in device memory (one per GPU, held
// until the process ends): its device address on the current device and its size.
constexpr uint32_t kStaticWiresPerRank = 32;
constexpr int kStaticMaxRanks = 8;
hipError_t wire_static_scratch(int device, void **ptr, size_t *bytes);


#ifdef __HIPCC__
// Element-wise sum of two registers holding 16-bit elements of type DT.  The
// registers are typed as _Float16 vectors for the memory instructions; bfloat16
// reinterprets them for the add.
template <int DT, typename V>
__device__ __forceinline__ V vadd(V a, V b) {
  if constexpr (DT == DT_F16) {
    return a + b;
  } else if constexpr (DT == DT_F16_WIDE) {
    constexpr int E = sizeof(V) / 2;
    typedef float F __attribute__((ext_vector_type(E)));
    F sum = __builtin_convertvector(a, F) + __builtin_convertvector(b, F);
    // Keep the compiler from narrowing this back into a binary16 add.
#pragma unroll
    for (int e = 0; e < E; ++e) {
      float t = sum[e];
      asm volatile("" : "+v"(t));
      sum[e] = t;
    }
    return __builtin_convertvector(sum, V);
  } else {
    typedef __bf16 B __attribute__((ext_vector_type(sizeof(V) / 2)));
    return __builtin_bit_cast(V, __builtin_bit_cast(B, a) + __builtin_bit_cast(B, b));
  }
}
#endif

}  // namespace vr
