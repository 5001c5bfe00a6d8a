// Internal interface between the C ABI (vr_api.cpp) and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "vrank_allreduce.h"

namespace vr {

// Device pointers of all virtual ranks, passed to kernels by value (like the
// reference functor's by-value pointer tables, parallel_transmit.hpp:134-145).
struct PtrTable {
  void *p[VR_MAX_RANKS];
};

enum Order : int {
  ORDER_ROTATED = 0,  // chain from the chunk owner: parallel/sequential/ring/simple transmit
  ORDER_BISECT = 1,   // pair sums, then chain over pairs: BisectPTransmit
};

struct Tuning {
  int block = 512;        // threads per work-group
  int waves_per_cu = 32;  // resident waves per CU the persistent grid asks for
  int unroll = 2;         // 16-byte vectors in flight per lane and rank
  int nt_load = 1;
  int nt_store = 1;
  int oneshot = 0;        // 1: grid covers the whole buffer, no grid-stride loop
  uint32_t force_blocks_per_rank = 0;  // non-zero: use exactly this many blocks per rank
};

struct DeviceInfo {
  int device = 0;
  int cus = 0;
  char arch[64] = {0};
};

// Direct transport -----------------------------------------------------------
// in/out hold nranks pointers; chunk_elems = nelems / nranks; vec_halves is 8
// (16-byte accesses) or 4 (8-byte accesses, for chunks or pointers that are only
// 8-byte aligned).
hipError_t launch_direct_allreduce(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   Order order, const PtrTable &in, const PtrTable &out,
                                   size_t chunk_elems, int vec_halves);
hipError_t launch_direct_allgather(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   const PtrTable &in, const PtrTable &out, size_t nelems,
                                   int vec_halves);
// mode: 0 copy, 1 read only, 2 write only
hipError_t launch_copy(hipStream_t s, const DeviceInfo &dev, const Tuning &t, void *dst,
                       const void *src, size_t bytes, int mode = 0);

}  // namespace vr
