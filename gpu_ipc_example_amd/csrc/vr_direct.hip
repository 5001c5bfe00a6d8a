// Direct transport: one pass over HBM.
//
// The work-groups of a launch are partitioned between the virtual ranks.  The
// groups of rank R handle the chunk R owns in the reference (chunk R for the
// flat transmits, parallel_transmit.hpp:104; chunk (R&1)*N/2 + R/2 for bisect,
// bisect_transmit.hpp:439-444,462-469): they read that chunk from every rank's
// input (the "scatter", pulled instead of pushed), add in the reference's order,
// and write the result into every rank's output (the "gather").
//
// Two grids.  Cache-resident data: a persistent grid with a grid-stride loop, block b
// serving rank b % N; HIP hands consecutive blocks to consecutive XCDs, so an 8-rank
// launch gives each XCD exactly one rank's chunk and no two L2s touch the same line.
// Data streamed from HBM: a one-trip grid, one tile per work-group; the hardware
// starts work-groups in index order, so the launch sweeps the buffers front to back,
// its residency capped through dynamic LDS that is never touched, and the chunks dealt
// to the work-groups one (or a few) at a time, so that all XCDs fill the same region
// of every output together, which is how HBM's write side runs best.
//
// Per 16-byte column a lane issues N independent dwordx4 loads, N-1 packed
// binary16 adds per half2, and N dwordx4 stores; nothing is staged in LDS
// because no datum is used twice.
//
// Memory is addressed through buffer resources (one per rank and direction,
// built in scalar registers from the chunk's base pointer and byte length): a
// lane supplies a 32-bit byte offset, the hardware drops every access at or
// beyond the length, so the last tile of a chunk needs no predicate (the
// reference predicates its tail wire per lane, rt64_128.hpp:570-582), and the
// cache-policy bits of each access are chosen per launch.

#include <hip/hip_ext.h>

#include <mutex>
#include <set>
#include <utility>

#include "vr_internal.h"

namespace vr {

thread_local KernelEvents tl_kernel_events;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Cache-policy operand of the buffer instructions (gfx940 encoding): bit 0 = sc0,
// bit 1 = nt, bit 4 = sc1.
constexpr int kAuxCached = 0;
constexpr int kAuxStream = 2;            // nt: streaming, do not keep in L2
constexpr int kAuxStreamAgent = 2 | 16;  // nt sc1: streaming store written through at agent scope

constexpr int load_aux(int nt) { return nt ? kAuxStream : kAuxCached; }
constexpr int store_aux(int nt) { return nt == 2 ? kAuxStreamAgent : nt == 1 ? kAuxStream : kAuxCached; }

// Raw buffer over [p, p + bytes): stride 0, 32-bit data format word for gfx9.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

template <typename V, int AUX>
__device__ __forceinline__ V ld(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  if constexpr (sizeof(V) == 16)
    return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, AUX));
  else
    return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, AUX));
}

template <typename V, int AUX>
__device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, uint32_t off, V v) {
  if constexpr (sizeof(V) == 16)
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, off, 0, AUX);
  else
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), r, off, 0, AUX);
}

// The chunk a protocol owner reduces.
template <int N, int ORDER>
__device__ __forceinline__ int chunk_of_owner(int owner) {
  // (The no-add yardstick stands beside the bisect all-reduce, so it deals the
  // chunks to the work-groups, and thereby to the XCDs, the same way.)
  if constexpr (ORDER == ORDER_BISECT || ORDER == ORDER_COPY)
    return (owner & 1) * (N / 2) + (owner >> 1);
  else
    return owner;
}

// t[k] = t[(k + a) % M] for 0 <= a < M, M a power of two: log2(M) rounds of scalar
// selects, no memory access.
template <int M, typename T>
__device__ __forceinline__ void rotate_left(T (&t)[M], int a) {
#pragma unroll
  for (int s = 1; s < M; s <<= 1) {
    const bool bit = (a & s) != 0;
    T u[M];
#pragma unroll
    for (int k = 0; k < M; ++k) u[k] = bit ? t[(k + s) % M] : t[k];
#pragma unroll
    for (int k = 0; k < M; ++k) t[k] = u[k];
  }
}

// op[k] = the input that is the k-th operand of the chain for the chunk owned by
// `owner`.  All N pointers are fetched with static indices (one scalar load of the
// whole table) and permuted in registers: a table lookup per operand would be N
// dependent scalar loads at the head of every work-group.
template <int N, int ORDER>
__device__ __forceinline__ void select_operands(const PtrTable &in, int owner, const char *(&op)[N]) {
  if constexpr (ORDER == ORDER_COPY) {
#pragma unroll
    for (int k = 0; k < N; ++k) op[k] = static_cast<const char *>(in.p[k]);
  } else if constexpr (ORDER == ORDER_ROTATED) {
    // own chunk first, then rank+1, rank+2, ...
#pragma unroll
    for (int k = 0; k < N; ++k) op[k] = static_cast<const char *>(in.p[k]);
    rotate_left<N>(op, owner);
  } else {
    // pair sums in the order l, l+1, ... (mod N/2); inside a pair the rank of the
    // owner's parity supplies its own data (even k) and its partner the message (odd k)
    constexpr int B = N / 2;
    const int h = owner & 1, l = owner >> 1;
    const char *ev[B], *od[B];
#pragma unroll
    for (int j = 0; j < B; ++j) {
      ev[j] = static_cast<const char *>(in.p[2 * j]);
      od[j] = static_cast<const char *>(in.p[2 * j + 1]);
    }
    rotate_left<B>(ev, l);
    rotate_left<B>(od, l);
#pragma unroll
    for (int j = 0; j < B; ++j) {
      op[2 * j] = h ? od[j] : ev[j];      // k even: the same-parity rank that formed pair sum j
      op[2 * j + 1] = h ? ev[j] : od[j];  // k odd: its pair's message
    }
  }
}

// The protocol owner served by the work-groups whose index is x modulo N.
// Consecutive work-groups run on consecutive XCDs.  With 8 ranks of 32 MiB,
// letting XCDs 0-3 and XCDs 4-7 each work on both halves of every buffer measured
// 0.5 to 3 % faster than XCD x -> chunk x (at other sizes either may lead by a few
// per cent, depending on where the buffers lie); the bisect order's
// chunk_of_owner spreads the chunks that way by itself, and the rotated orders
// are dealt alike.
template <int N, int ORDER>
__device__ __forceinline__ int owner_of_group(int x) {
  if constexpr (N == 8 && ORDER == ORDER_ROTATED)
    return (x & 1) * (N / 2) + (x >> 1);
  else
    return x;
}

// Sum of the N operands in the protocol's association.  The received message is
// always the left operand of the add (rt64_128.hpp:951-956).
template <int N, int ORDER, int DT, typename V>
__device__ __forceinline__ V reduce_operands(const V (&x)[N]) {
  if constexpr (ORDER == ORDER_ROTATED) {
    V acc = x[0];
#pragma unroll
    for (int k = 1; k < N; ++k) acc = vadd<DT>(x[k], acc);
    return acc;
  } else {
    V acc = vadd<DT>(x[1], x[0]);
#pragma unroll
    for (int k = 2; k < N; k += 2) {
      const V pair = vadd<DT>(x[k + 1], x[k]);
      acc = vadd<DT>(pair, acc);
    }
    return acc;
  }
}

// One launch covers bytes [seg_off, seg_off + seg_bytes) of every chunk;
// chunk_pitch is the full chunk length (the distance between chunk starts).
template <int N, int ORDER, int DT, typename V, int UNROLL, int LD_AUX, int ST_AUX>
__global__ __launch_bounds__(1024) void k_direct_allreduce(PtrTable in, PtrTable out,
                                                           size_t chunk_pitch, size_t seg_off,
                                                           uint32_t seg_bytes,
                                                           uint32_t blocks_per_rank, uint32_t deal_log2,
                                                           uint32_t row) {
  // 2^deal_log2 chunks ("deal") are worked on at a time: row y of the grid, deal *
  // blocks_per_rank work-groups, belongs to owners y * deal ... y * deal + deal - 1,
  // round robin (rows are dispatched one after the other).  deal = N: work-group b
  // serves owner b % N throughout (with 8 ranks every XCD its own chunk); deal = 1: all
  // work-groups, and with them all XCDs, sweep one chunk after the other.
  const uint32_t deal = 1u << deal_log2;
  const int owner = owner_of_group<N, ORDER>((int)(blockIdx.y * deal + (blockIdx.x & (deal - 1))));
  const uint32_t jblock = blockIdx.x >> deal_log2;
  const size_t base = (size_t)chunk_of_owner<N, ORDER>(owner) * chunk_pitch + seg_off;

  const char *op[N];
  select_operands<N, ORDER>(in, owner, op);
  __amdgpu_buffer_rsrc_t src[N], dst[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    src[k] = make_rsrc(op[k] + base, seg_bytes);
    dst[k] = make_rsrc(static_cast<char *>(out.p[k]) + base, seg_bytes);
  }
  const uint32_t lane = threadIdx.x * (uint32_t)sizeof(V);
  // `row` = bytes one unroll step spans, blockDim.x * sizeof(V): an argument, so that it
  // arrives with the others instead of through a separate load of the launch's dimensions
  const uint32_t tile = row * UNROLL;
  const uint32_t stride = tile * blocks_per_rank;
  // Every work-group has a first tile (the host launches at most one work-group per tile),
  // so the loop tests at its end and nothing separates the kernel's argument loads.
  uint32_t t = jblock * tile;
  do {
    V x[UNROLL][N];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < N; ++k) x[u][k] = ld<V, LD_AUX>(src[k], t + u * row + lane);
    // Every load of the trip is issued before the first add waits for one: left to
    // itself the scheduler may hold a load back behind the adds of earlier operands,
    // which puts a whole memory latency into the trip (measured: +4 us on 83).  (Not
    // where a trip's loads alone fill 64 registers or more: pinned there, they spill.)
    if constexpr (UNROLL * N * sizeof(V) <= 256) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if constexpr (ORDER == ORDER_COPY) {
        // the all-reduce's N read streams and N write streams with the adds removed
#pragma unroll
        for (int k = 0; k < N; ++k) st<V, ST_AUX>(dst[k], t + u * row + lane, x[u][k]);
      } else {
        const V acc = reduce_operands<N, ORDER, DT, V>(x[u]);
#pragma unroll
        for (int k = 0; k < N; ++k) st<V, ST_AUX>(dst[k], t + u * row + lane, acc);
      }
    }
    t += stride;
  } while (t < seg_bytes);
}

// All-gather: the groups of rank p read p's slice once and store it into slot p
// of every rank's output (allgather.hpp:79-100 collapsed to one hop).
template <int N, typename V, int UNROLL, int LD_AUX, int ST_AUX>
__global__ __launch_bounds__(1024) void k_direct_allgather(PtrTable in, PtrTable out,
                                                           size_t slice_pitch, size_t seg_off,
                                                           uint32_t seg_bytes,
                                                           uint32_t blocks_per_rank, uint32_t deal_log2,
                                                           uint32_t row) {
  // 2^deal_log2 source slices are worked on at a time (see k_direct_allreduce): deal = N
  // gives work-group b to source b % N throughout, deal = 1 lets all work-groups sweep
  // one source's slice after the other.
  const uint32_t run_log2 = deal_log2 >> 8;   // second byte: tiles per XCD run (see below)
  deal_log2 &= 0xff;
  const uint32_t deal = 1u << deal_log2;
  const int p = (int)(blockIdx.y * deal + (blockIdx.x & (deal - 1)));
  uint32_t jblock = blockIdx.x >> deal_log2;
  // Consecutive work-groups run on consecutive XCDs, so XCD k gets every eighth tile.  With
  // runs, the work-groups of each group of 8 * run are permuted so that XCD k gets `run`
  // consecutive tiles (the ragged last group of a slice stays as it is).
  if (run_log2) {
    const uint32_t group = 8u << run_log2, first = jblock & ~(group - 1), r = jblock & (group - 1);
    if (first + group <= blocks_per_rank) jblock = first + ((r & 7u) << run_log2) + (r >> 3);
  }
  // the source pointer picked from the whole table with scalar selects: a look-up
  // by p would be a second, dependent scalar load at the head of every work-group
  uintptr_t picked = 0;
#pragma unroll
  for (int k = 0; k < N; ++k) picked |= p == k ? reinterpret_cast<uintptr_t>(in.p[k]) : (uintptr_t)0;
  const char *src_ptr = reinterpret_cast<const char *>(picked) + seg_off;
  const __amdgpu_buffer_rsrc_t src = make_rsrc(src_ptr, seg_bytes);
  __amdgpu_buffer_rsrc_t dst[N];
#pragma unroll
  for (int r = 0; r < N; ++r) {
    char *d = static_cast<char *>(out.p[r]) + (size_t)p * slice_pitch + seg_off;
    // The reference skips the store when a rank's input already is its own
    // output slot (sequential_transmit.hpp:496-497).  Here such a destination gets
    // a resource of length zero, so the hardware drops its stores: no branch sits
    // between the N stores of a trip (with branches there, launches with few waves
    // per CU ran up to 20 % slower).
    dst[r] = make_rsrc(d, d == src_ptr ? 0u : seg_bytes);
  }
  const uint32_t lane = threadIdx.x * (uint32_t)sizeof(V);
  const uint32_t tile = row * UNROLL;
  const uint32_t stride = tile * blocks_per_rank;
  uint32_t t = jblock * tile;   // every work-group has a first tile, as in k_direct_allreduce
  do {
    V x[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) x[u] = ld<V, LD_AUX>(src, t + u * row + lane);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int r = 0; r < N; ++r) st<V, ST_AUX>(dst[r], t + u * row + lane, x[u]);
    t += stride;
  } while (t < seg_bytes);
}

// Streaming yardsticks over one segment: MODE 0 copies, 1 only reads (the sum is
// kept alive by a store that never executes for finite data), 2 only writes.
template <int MODE, int UNROLL, int LD_AUX, int ST_AUX>
__global__ __launch_bounds__(1024) void k_probe(char *dst_ptr, const char *src_ptr, uint32_t seg_bytes) {
  const __amdgpu_buffer_rsrc_t src = make_rsrc(src_ptr, seg_bytes);
  const __amdgpu_buffer_rsrc_t dst = make_rsrc(dst_ptr, seg_bytes);
  const uint32_t lane = threadIdx.x * 16u, row = blockDim.x * 16u;
  const uint32_t tile = row * UNROLL, stride = tile * gridDim.x;
  h8 acc = {0, 0, 0, 0, 0, 0, 0, 0};
  for (uint32_t t = blockIdx.x * tile; t < seg_bytes; t += stride) {
    h8 x[UNROLL];
    if constexpr (MODE != 2) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) x[u] = ld<h8, LD_AUX>(src, t + u * row + lane);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if constexpr (MODE == 0) st<h8, ST_AUX>(dst, t + u * row + lane, x[u]);
      if constexpr (MODE == 1) acc = acc + x[u];
      if constexpr (MODE == 2) st<h8, ST_AUX>(dst, t + u * row + lane, acc);
    }
  }
  if constexpr (MODE == 1) {
    if (acc[0] == (_Float16)12345.0f && acc[7] == (_Float16)-321.0f) st<h8, kAuxCached>(dst, 0, acc);
  }
}

// Records which XCD (accelerator complex die) each work-group of a launch ran on:
// the rank-to-XCD affinity of the kernels above rests on consecutive work-groups
// being dealt to consecutive XCDs.
__global__ void k_xcc_ids(uint32_t *out) {
  if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20);  // XCC_ID[3:0]
}

hipError_t launch_xcc_probe(hipStream_t s, uint32_t blocks, uint32_t *out_device) {
  hipLaunchKernelGGL(k_xcc_ids, dim3(blocks), dim3(256), 0, s, out_device);
  return hipGetLastError();
}

// ---- host-side launch plumbing -------------------------------------------------

// Residency cap of a one-trip grid.  The hardware places as many work-groups on a
// CU as registers and LDS allow; a launch that wants at most `wgs` there asks for
// so much dynamic LDS (never touched) that one more would not fit.  0 = no cap.
static uint32_t lds_cap_bytes(const DeviceInfo &dev, int wgs) {
  if (wgs <= 0 || dev.lds_per_cu == 0) return 0;
  if (wgs > 12) wgs = 12;
  // 15/16 of an equal share: `wgs` shares fit with room for allocation granules,
  // wgs + 1 exceed the CU's LDS for every wgs <= 12.
  size_t b = dev.lds_per_cu / (size_t)wgs / 16 * 15;
  b -= b % 1024;
  return (uint32_t)b;
}

// A kernel may ask for more than 48 KiB of dynamic LDS only after its limit has been
// raised, once per kernel and device.
static hipError_t allow_dynamic_lds(const void *kernel, const DeviceInfo &dev, uint32_t bytes) {
  const int device = dev.device;
  if (bytes <= 48u * 1024u) return hipSuccess;
  static std::mutex lock;
  static std::set<std::pair<const void *, int>> done;
  std::lock_guard<std::mutex> hold(lock);
  if (done.count({kernel, device})) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dev.lds_per_cu);
  if (e == hipSuccess) done.insert({kernel, device});
  return e;
}

// A launch addresses each chunk with 32-bit byte offsets, so longer chunks are
// covered by several launches of at most Tuning::segment_bytes per chunk.
static size_t segment_of(const Tuning &t) {
  size_t seg = t.segment_bytes - t.segment_bytes % 16;
  if (seg == 0) seg = 16;
  return seg > (1ull << 30) ? (1ull << 30) : seg;
}

static uint32_t blocks_per_rank_for(const DeviceInfo &dev, const Tuning &t, int nranks,
                                    size_t bytes_per_rank, size_t tile_bytes) {
  size_t tiles = (bytes_per_rank + tile_bytes - 1) / tile_bytes;
  if (tiles == 0) tiles = 1;
  size_t need = tiles;
  if (t.force_blocks_per_rank) {
    need = t.force_blocks_per_rank;
  } else if (!t.oneshot) {
    const int waves_per_block = t.block / 64;
    size_t resident = (size_t)dev.cus * t.waves_per_cu / waves_per_block;  // whole launch
    size_t cap = resident / nranks;
    if (cap == 0) cap = 1;
    if (need > cap) need = cap;
  }
  if (need > tiles) need = tiles;   // a block without a tile has nothing to do
  return (uint32_t)need;
}

// Calls f(std::integral_constant<int, load aux>, std::integral_constant<int, store aux>)
// for the launch's cache policies.
template <int V>
struct IntC {
  static constexpr int value = V;
};

template <typename F>
static hipError_t with_policy(const Tuning &t, F &&f) {
  const int ld_nt = t.nt_load ? 1 : 0;
  const int st_nt = t.nt_store < 0 ? 0 : (t.nt_store > 2 ? 2 : t.nt_store);
#define VR_POLICY(L, S) \
  if (ld_nt == L && st_nt == S) return f(IntC<load_aux(L)>(), IntC<store_aux(S)>());
  VR_POLICY(0, 0) VR_POLICY(0, 1) VR_POLICY(0, 2) VR_POLICY(1, 0) VR_POLICY(1, 1) VR_POLICY(1, 2)
#undef VR_POLICY
  return hipErrorInvalidValue;
}

template <int N, int ORDER, int DT, typename V, int UNROLL>
static hipError_t launch_ar_segments(hipStream_t s, const DeviceInfo &dev, const Tuning &t,
                                     const PtrTable &in, const PtrTable &out, size_t chunk_bytes) {
  const uint32_t row = (uint32_t)(t.block * sizeof(V));   // bytes one unroll step of a work-group spans
  const size_t tile = (size_t)row * UNROLL;
  const size_t seg_max = segment_of(t);
  const uint32_t lds = lds_cap_bytes(dev, t.wgs_per_cu);
  // chunks dealt at a time: a divisor of N, N itself unless the launch says otherwise
  const uint32_t deal = (t.deal > 0 && t.deal <= N && N % t.deal == 0) ? (uint32_t)t.deal : (uint32_t)N;
  const uint32_t deal_log2 = (uint32_t)__builtin_ctz(deal);   // N is a power of two, so are its divisors
  for (size_t off = 0; off < chunk_bytes; off += seg_max) {
    const size_t seg = chunk_bytes - off < seg_max ? chunk_bytes - off : seg_max;
    const uint32_t bpr = blocks_per_rank_for(dev, t, N, seg, tile);
    const dim3 grid(bpr * deal, N / deal), block(t.block);
    // kernel-attached profiling events: start on the first segment, stop on the last
    hipEvent_t ev0 = off == 0 ? tl_kernel_events.start : nullptr;
    hipEvent_t ev1 = off + seg >= chunk_bytes ? tl_kernel_events.stop : nullptr;
    hipError_t e = with_policy(t, [&](auto ld_aux, auto st_aux) {
      auto kernel = k_direct_allreduce<N, ORDER, DT, V, UNROLL, decltype(ld_aux)::value, decltype(st_aux)::value>;
      if (hipError_t a = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), dev, lds); a != hipSuccess) return a;
      if (ev0 || ev1)
        hipExtLaunchKernelGGL(kernel, grid, block, lds, s, ev0, ev1, 0, in, out, chunk_bytes, off, (uint32_t)seg, bpr, deal_log2, row);
      else
        hipLaunchKernelGGL(kernel, grid, block, lds, s, in, out, chunk_bytes, off, (uint32_t)seg, bpr, deal_log2, row);
      return hipGetLastError();
    });
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int N, int ORDER, int DT, typename V>
static hipError_t launch_ar_unroll(hipStream_t s, const DeviceInfo &dev, const Tuning &t,
                                   const PtrTable &in, const PtrTable &out, size_t chunk_bytes) {
  // 16 ranks already keep 16 loads per lane in flight; the bfloat16 add needs
  // binary32 temporaries, which leaves no room for four vectors per rank.
  const int unroll = (N >= 16) ? 1 : (t.unroll >= 4 ? 4 : (t.unroll >= 2 ? 2 : 1));
  if constexpr (N <= 8) {
    // (the no-add yardstick at eight ranks would hold 128 registers of loaded data: two vectors at most)
    if constexpr (DT == DT_F16 && !(ORDER == ORDER_COPY && N == 8))
      if (unroll == 4) return launch_ar_segments<N, ORDER, DT, V, 4>(s, dev, t, in, out, chunk_bytes);
    if (unroll >= 2) return launch_ar_segments<N, ORDER, DT, V, 2>(s, dev, t, in, out, chunk_bytes);
  }
  return launch_ar_segments<N, ORDER, DT, V, 1>(s, dev, t, in, out, chunk_bytes);
}
template <int N, int ORDER>
static hipError_t launch_ar_vec(hipStream_t s, const DeviceInfo &dev, const Tuning &t, DType dtype,
                                const PtrTable &in, const PtrTable &out, size_t chunk_elems,
                                int vec_halves) {
  const size_t bytes = chunk_elems * 2;
  if (dtype == DT_BF16) {
    if (vec_halves == 8) return launch_ar_unroll<N, ORDER, DT_BF16, h8>(s, dev, t, in, out, bytes);
    return launch_ar_unroll<N, ORDER, DT_BF16, h4>(s, dev, t, in, out, bytes);
  }
  if (vec_halves == 8) {
    if (t.f16_wide) return launch_ar_unroll<N, ORDER, DT_F16_WIDE, h8>(s, dev, t, in, out, bytes);
    return launch_ar_unroll<N, ORDER, DT_F16, h8>(s, dev, t, in, out, bytes);
  }
  return launch_ar_unroll<N, ORDER, DT_F16, h4>(s, dev, t, in, out, bytes);
}

hipError_t launch_direct_allreduce(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   Order order, DType dtype, const PtrTable &in, const PtrTable &out,
                                   size_t chunk_elems, int vec_halves) {
  if (chunk_elems == 0) return hipSuccess;
  if (t.block < 64 || t.block > 1024 || t.block % 64) return hipErrorInvalidValue;
#define VR_CASE(NN)                                                                              \
  case NN:                                                                                       \
    if (order == ORDER_COPY) {                                                                   \
      if (vec_halves != 8) return hipErrorInvalidValue;                                          \
      return launch_ar_unroll<NN, ORDER_COPY, DT_F16, h8>(s, dev, t, in, out, chunk_elems * 2);  \
    }                                                                                            \
    if (order == ORDER_BISECT) {                                                                 \
      if constexpr (NN >= 4)                                                                     \
        return launch_ar_vec<NN, ORDER_BISECT>(s, dev, t, dtype, in, out, chunk_elems, vec_halves);     \
      return hipErrorInvalidValue;                                                               \
    }                                                                                            \
    return launch_ar_vec<NN, ORDER_ROTATED>(s, dev, t, dtype, in, out, chunk_elems, vec_halves);
  switch (nranks) {
    VR_CASE(2)
    VR_CASE(4)
    VR_CASE(8)
    VR_CASE(16)
    default:
      return hipErrorInvalidValue;
  }
#undef VR_CASE
}

template <int N, typename V, int UNROLL>
static hipError_t launch_ag_segments(hipStream_t s, const DeviceInfo &dev, const Tuning &t,
                                     const PtrTable &in, const PtrTable &out, size_t slice_bytes) {
  const uint32_t row = (uint32_t)(t.block * sizeof(V));   // bytes one unroll step of a work-group spans
  const size_t tile = (size_t)row * UNROLL;
  const size_t seg_max = segment_of(t);
  const uint32_t lds = lds_cap_bytes(dev, t.wgs_per_cu);
  const uint32_t deal = (t.deal > 0 && t.deal <= N && N % t.deal == 0) ? (uint32_t)t.deal : (uint32_t)N;
  uint32_t deal_log2 = (uint32_t)__builtin_ctz(deal);
  // tiles per XCD run: only where a row of the grid is one source's slice and a one-trip launch
  if (t.run > 1 && deal == 1 && t.oneshot) deal_log2 |= (uint32_t)__builtin_ctz((unsigned)t.run) << 8;
  for (size_t off = 0; off < slice_bytes; off += seg_max) {
    const size_t seg = slice_bytes - off < seg_max ? slice_bytes - off : seg_max;
    const uint32_t bpr = blocks_per_rank_for(dev, t, N, seg, tile);
    const dim3 grid(bpr * deal, N / deal), block(t.block);
    hipEvent_t ev0 = off == 0 ? tl_kernel_events.start : nullptr;
    hipEvent_t ev1 = off + seg >= slice_bytes ? tl_kernel_events.stop : nullptr;
    hipError_t e = with_policy(t, [&](auto ld_aux, auto st_aux) {
      auto kernel = k_direct_allgather<N, V, UNROLL, decltype(ld_aux)::value, decltype(st_aux)::value>;
      if (hipError_t a = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), dev, lds); a != hipSuccess) return a;
      if (ev0 || ev1)
        hipExtLaunchKernelGGL(kernel, grid, block, lds, s, ev0, ev1, 0, in, out, slice_bytes, off, (uint32_t)seg, bpr, deal_log2, row);
      else
        hipLaunchKernelGGL(kernel, grid, block, lds, s, in, out, slice_bytes, off, (uint32_t)seg, bpr, deal_log2, row);
      return hipGetLastError();
    });
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int N, typename V>
static hipError_t launch_ag(hipStream_t s, const DeviceInfo &dev, const Tuning &t, const PtrTable &in,
                            const PtrTable &out, size_t slice_bytes) {
  if (t.unroll >= 2) return launch_ag_segments<N, V, 2>(s, dev, t, in, out, slice_bytes);
  return launch_ag_segments<N, V, 1>(s, dev, t, in, out, slice_bytes);
}

hipError_t launch_direct_allgather(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   const PtrTable &in, const PtrTable &out, size_t nelems,
                                   int vec_halves) {
  if (nelems == 0) return hipSuccess;
  if (t.block < 64 || t.block > 1024 || t.block % 64) return hipErrorInvalidValue;
#define VR_CASE(NN)                                                              \
  case NN:                                                                       \
    if (vec_halves == 8) return launch_ag<NN, h8>(s, dev, t, in, out, nelems * 2); \
    return launch_ag<NN, h4>(s, dev, t, in, out, nelems * 2);
  switch (nranks) {
    VR_CASE(2)
    VR_CASE(4)
    VR_CASE(8)
    VR_CASE(16)
    default:
      return hipErrorInvalidValue;
  }
#undef VR_CASE
}

template <int MODE, int UNROLL>
static hipError_t launch_probe_segments(hipStream_t s, const DeviceInfo &dev, const Tuning &t,
                                        char *dst, const char *src, size_t bytes) {
  const size_t tile = (size_t)t.block * 16 * UNROLL;
  const size_t seg_max = segment_of(t);
  const uint32_t lds = lds_cap_bytes(dev, t.wgs_per_cu);
  for (size_t off = 0; off < bytes; off += seg_max) {
    const size_t seg = bytes - off < seg_max ? bytes - off : seg_max;
    size_t blocks = (seg + tile - 1) / tile;
    const size_t resident = (size_t)dev.cus * t.waves_per_cu / (t.block / 64);
    if (!t.oneshot && blocks > resident) blocks = resident;
    if (blocks == 0) blocks = 1;
    const dim3 grid((uint32_t)blocks), block(t.block);
    hipError_t e = with_policy(t, [&](auto ld_aux, auto st_aux) {
      auto kernel = k_probe<MODE, UNROLL, decltype(ld_aux)::value, decltype(st_aux)::value>;
      if (hipError_t a = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), dev, lds); a != hipSuccess) return a;
      hipLaunchKernelGGL(kernel, grid, block, lds, s, dst + off, src + off, (uint32_t)seg);
      return hipGetLastError();
    });
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_copy(hipStream_t s, const DeviceInfo &dev, const Tuning &t, void *dst,
                       const void *src, size_t bytes, int mode) {
  bytes -= bytes % 16;
  if (bytes == 0) return hipSuccess;
  if (t.block < 64 || t.block > 1024 || t.block % 64) return hipErrorInvalidValue;
  char *d = static_cast<char *>(dst);
  const char *sp = static_cast<const char *>(src);
  const bool u4 = t.unroll >= 4;
  switch (mode) {
    case 1:
      return u4 ? launch_probe_segments<1, 4>(s, dev, t, d, sp, bytes) : launch_probe_segments<1, 1>(s, dev, t, d, sp, bytes);
    case 2:
      return u4 ? launch_probe_segments<2, 4>(s, dev, t, d, sp, bytes) : launch_probe_segments<2, 1>(s, dev, t, d, sp, bytes);
    default:
      return u4 ? launch_probe_segments<0, 4>(s, dev, t, d, sp, bytes) : launch_probe_segments<0, 1>(s, dev, t, d, sp, bytes);
  }
}

}  // namespace vr
