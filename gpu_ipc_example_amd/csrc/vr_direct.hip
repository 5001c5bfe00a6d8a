// Direct transport: one pass over HBM.
//
// The work-groups of a launch are partitioned between the virtual ranks.  The
// groups of rank R handle the chunk R owns in the reference (chunk R for the
// flat transmits, parallel_transmit.hpp:104; chunk (R&1)*N/2 + R/2 for bisect,
// bisect_transmit.hpp:439-444,462-469): they read that chunk from every rank's
// input (the "scatter", pulled instead of pushed), add in the reference's order,
// and write the result into every rank's output (the "gather").  With block b
// serving rank b % N and HIP handing consecutive blocks to consecutive XCDs, an
// 8-rank launch gives each XCD exactly one rank's chunk: no two L2s ever touch
// the same line.
//
// Per 16-byte column a lane issues N independent dwordx4 loads, N-1 packed
// binary16 adds per half2, and N dwordx4 stores; nothing is staged in LDS
// because no datum is used twice.

#include "vr_internal.h"

namespace vr {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));

template <typename V, bool NT>
__device__ __forceinline__ V ld(const V *p) {
  if constexpr (NT)
    return __builtin_nontemporal_load(p);
  else
    return *p;
}

template <typename V, bool NT>
__device__ __forceinline__ void st(V *p, V v) {
  if constexpr (NT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// Rank whose input is the k-th operand of the chain for the chunk owned by
// `owner`, and the chunk index itself.
template <int N, int ORDER>
__device__ __forceinline__ int chunk_of_owner(int owner) {
  if constexpr (ORDER == ORDER_ROTATED)
    return owner;
  else
    return (owner & 1) * (N / 2) + (owner >> 1);
}

template <int N, int ORDER>
__device__ __forceinline__ int operand_rank(int owner, int k) {
  if constexpr (ORDER == ORDER_ROTATED) {
    return (owner + k) % N;                       // own chunk first, then rank+1, rank+2, ...
  } else {
    constexpr int B = N / 2;
    const int h = owner & 1, l = owner >> 1;
    const int j = (l + (k >> 1)) % B;             // pair index walks l, l+1, ...
    const int self = 2 * j + h;                   // the same-parity rank that formed pair sum j
    return (k & 1) ? (self ^ 1) : self;           // k even: its own data; k odd: its pair's message
  }
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

template <int N, int ORDER, int DT, typename V, int UNROLL, bool NT_LD, bool NT_ST>
__global__ __launch_bounds__(1024) void k_direct_allreduce(PtrTable in, PtrTable out,
                                                           size_t chunk_vecs,
                                                           uint32_t blocks_per_rank) {
  const int owner = blockIdx.x % N;
  const uint32_t jblock = blockIdx.x / N;
  const int chunk = chunk_of_owner<N, ORDER>(owner);
  const size_t chunk_base = (size_t)chunk * chunk_vecs;

  // Uniform (scalar) byte pointers to this chunk in every rank's buffer; a lane
  // adds only its own 32-bit byte offset, so every access is
  // "global_load/store_dwordx4 v, v_lane, s[base]" and no 64-bit vector address
  // arithmetic is needed.
  const char *src[N];
  char *dst[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    src[k] = static_cast<const char *>(in.p[operand_rank<N, ORDER>(owner, k)]) + chunk_base * sizeof(V);
    dst[k] = static_cast<char *>(out.p[k]) + chunk_base * sizeof(V);
  }
  const uint32_t lane = threadIdx.x * (uint32_t)sizeof(V);
  const uint32_t row = blockDim.x * (uint32_t)sizeof(V);       // bytes one unroll step spans

  const size_t tile = (size_t)blockDim.x * UNROLL;
  const size_t stride = tile * blocks_per_rank;
  for (size_t base = (size_t)jblock * tile; base < chunk_vecs; base += stride) {
    V x[UNROLL][N];
    const size_t base_bytes = base * sizeof(V);
    if (base + tile <= chunk_vecs) {
      // Whole tile in range: UNROLL*N loads in flight with no predication.
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < N; ++k)
          x[u][k] = ld<V, NT_LD>(reinterpret_cast<const V *>(src[k] + base_bytes + u * row + lane));
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const V acc = reduce_operands<N, ORDER, DT, V>(x[u]);
#pragma unroll
        for (int k = 0; k < N; ++k)
          st<V, NT_ST>(reinterpret_cast<V *>(dst[k] + base_bytes + u * row + lane), acc);
      }
    } else {
      // Tail tile of the chunk: per-lane predicate, like the reference's tail wire.
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (base + (size_t)u * blockDim.x + threadIdx.x < chunk_vecs) {
#pragma unroll
          for (int k = 0; k < N; ++k)
            x[0][k] = ld<V, NT_LD>(reinterpret_cast<const V *>(src[k] + base_bytes + u * row + lane));
          const V acc = reduce_operands<N, ORDER, DT, V>(x[0]);
#pragma unroll
          for (int k = 0; k < N; ++k)
            st<V, NT_ST>(reinterpret_cast<V *>(dst[k] + base_bytes + u * row + lane), acc);
        }
      }
    }
  }
}

// All-gather: the groups of rank p read p's slice once and store it into slot p
// of every rank's output (allgather.hpp:79-100 collapsed to one hop).
template <int N, typename V, int UNROLL, bool NT_LD, bool NT_ST>
__global__ __launch_bounds__(1024) void k_direct_allgather(PtrTable in, PtrTable out,
                                                           size_t slice_vecs,
                                                           uint32_t blocks_per_rank) {
  const int p = blockIdx.x % N;
  const uint32_t jblock = blockIdx.x / N;
  const V *src = reinterpret_cast<const V *>(in.p[p]);
  V *dst[N];
#pragma unroll
  for (int r = 0; r < N; ++r) dst[r] = reinterpret_cast<V *>(out.p[r]) + (size_t)p * slice_vecs;

  const size_t tile = (size_t)blockDim.x * UNROLL;
  const size_t stride = tile * blocks_per_rank;
  for (size_t base = (size_t)jblock * tile; base < slice_vecs; base += stride) {
    V x[UNROLL];
    size_t idx[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      idx[u] = base + (size_t)u * blockDim.x + threadIdx.x;
      if (idx[u] < slice_vecs) x[u] = ld<V, NT_LD>(src + idx[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (idx[u] < slice_vecs) {
#pragma unroll
        for (int r = 0; r < N; ++r) {
          // The reference skips the store when a rank's input already is its
          // own output slot (sequential_transmit.hpp:496-497).
          if (reinterpret_cast<const V *>(dst[r]) != src) st<V, NT_ST>(dst[r] + idx[u], x[u]);
        }
      }
    }
  }
}

// Streaming yardsticks: MODE 0 copies, 1 only reads (the sum is kept alive by a
// store that never executes for finite data), 2 only writes.
template <int MODE, int UNROLL, bool NT>
__global__ __launch_bounds__(1024) void k_probe(h8 *dst, const h8 *src, size_t vecs) {
  const size_t tile = (size_t)blockDim.x * UNROLL;
  const size_t stride = tile * gridDim.x;
  h8 acc = {0, 0, 0, 0, 0, 0, 0, 0};
  for (size_t base = (size_t)blockIdx.x * tile; base < vecs; base += stride) {
    const size_t first = base + threadIdx.x;
    if (base + tile <= vecs) {
      h8 x[UNROLL];
      if constexpr (MODE != 2) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) x[u] = ld<h8, NT>(src + first + (size_t)u * blockDim.x);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if constexpr (MODE == 0) st<h8, NT>(dst + first + (size_t)u * blockDim.x, x[u]);
        if constexpr (MODE == 1) acc = acc + x[u];
        if constexpr (MODE == 2) st<h8, NT>(dst + first + (size_t)u * blockDim.x, acc);
      }
    } else {
      for (int u = 0; u < UNROLL; ++u) {
        const size_t i = first + (size_t)u * blockDim.x;
        if (i < vecs) {
          if constexpr (MODE == 0) st<h8, NT>(dst + i, ld<h8, NT>(src + i));
          if constexpr (MODE == 1) acc = acc + ld<h8, NT>(src + i);
          if constexpr (MODE == 2) st<h8, NT>(dst + i, acc);
        }
      }
    }
  }
  if constexpr (MODE == 1) {
    if (acc[0] == (_Float16)12345.0f && acc[7] == (_Float16)-321.0f) dst[0] = acc;
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

static uint32_t blocks_per_rank_for(const DeviceInfo &dev, const Tuning &t, int nranks,
                                    size_t vecs_per_rank, int unroll) {
  const size_t tile = (size_t)t.block * unroll;
  size_t need = (vecs_per_rank + tile - 1) / tile;
  if (need == 0) need = 1;
  if (t.force_blocks_per_rank) {
    need = t.force_blocks_per_rank;
  } else if (!t.oneshot) {
    const int waves_per_block = t.block / 64;
    size_t resident = (size_t)dev.cus * t.waves_per_cu / waves_per_block;  // whole launch
    size_t cap = resident / nranks;
    if (cap == 0) cap = 1;
    if (need > cap) need = cap;
  }
  if (need > 0x7fffffffu / (size_t)nranks) need = 0x7fffffffu / (size_t)nranks;
  return (uint32_t)need;
}

template <int N, int ORDER, int DT, typename V, int UNROLL>
static hipError_t launch_ar_nt(hipStream_t s, dim3 grid, dim3 block, const Tuning &t,
                               const PtrTable &in, const PtrTable &out, size_t chunk_vecs,
                               uint32_t bpr) {
  if (t.nt_load && t.nt_store)
    hipLaunchKernelGGL((k_direct_allreduce<N, ORDER, DT, V, UNROLL, true, true>), grid, block, 0, s, in,
                       out, chunk_vecs, bpr);
  else if (t.nt_load)
    hipLaunchKernelGGL((k_direct_allreduce<N, ORDER, DT, V, UNROLL, true, false>), grid, block, 0, s,
                       in, out, chunk_vecs, bpr);
  else if (t.nt_store)
    hipLaunchKernelGGL((k_direct_allreduce<N, ORDER, DT, V, UNROLL, false, true>), grid, block, 0, s,
                       in, out, chunk_vecs, bpr);
  else
    hipLaunchKernelGGL((k_direct_allreduce<N, ORDER, DT, V, UNROLL, false, false>), grid, block, 0, s,
                       in, out, chunk_vecs, bpr);
  return hipGetLastError();
}

template <int N, int ORDER, int DT, typename V>
static hipError_t launch_ar_unroll(hipStream_t s, const DeviceInfo &dev, const Tuning &t,
                                   const PtrTable &in, const PtrTable &out, size_t chunk_vecs) {
  const int unroll = (N >= 16) ? 1 : (t.unroll >= 4 && N <= 8 ? 4 : (t.unroll >= 2 ? 2 : 1));
  const uint32_t bpr = blocks_per_rank_for(dev, t, N, chunk_vecs, unroll);
  const dim3 grid(bpr * N), block(t.block);
  switch (unroll) {
    case 4:
      if constexpr (N <= 8) return launch_ar_nt<N, ORDER, DT, V, 4>(s, grid, block, t, in, out, chunk_vecs, bpr);
      [[fallthrough]];
    case 2:
      if constexpr (N <= 8) return launch_ar_nt<N, ORDER, DT, V, 2>(s, grid, block, t, in, out, chunk_vecs, bpr);
      [[fallthrough]];
    default:
      return launch_ar_nt<N, ORDER, DT, V, 1>(s, grid, block, t, in, out, chunk_vecs, bpr);
  }
}

template <int N, int ORDER>
static hipError_t launch_ar_vec(hipStream_t s, const DeviceInfo &dev, const Tuning &t, DType dtype,
                                const PtrTable &in, const PtrTable &out, size_t chunk_elems,
                                int vec_halves) {
  if (dtype == DT_BF16) {
    if (vec_halves == 8) return launch_ar_unroll<N, ORDER, DT_BF16, h8>(s, dev, t, in, out, chunk_elems / 8);
    return launch_ar_unroll<N, ORDER, DT_BF16, h4>(s, dev, t, in, out, chunk_elems / 4);
  }
  if (vec_halves == 8) return launch_ar_unroll<N, ORDER, DT_F16, h8>(s, dev, t, in, out, chunk_elems / 8);
  return launch_ar_unroll<N, ORDER, DT_F16, h4>(s, dev, t, in, out, chunk_elems / 4);
}

hipError_t launch_direct_allreduce(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   Order order, DType dtype, const PtrTable &in, const PtrTable &out,
                                   size_t chunk_elems, int vec_halves) {
  if (chunk_elems == 0) return hipSuccess;
#define VR_CASE(NN)                                                                              \
  case NN:                                                                                       \
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

template <int N, typename V>
static hipError_t launch_ag(hipStream_t s, const DeviceInfo &dev, const Tuning &t, const PtrTable &in,
                            const PtrTable &out, size_t slice_vecs) {
  const int unroll = t.unroll >= 2 ? 2 : 1;
  const uint32_t bpr = blocks_per_rank_for(dev, t, N, slice_vecs, unroll);
  const dim3 grid(bpr * N), block(t.block);
  if (unroll == 2) {
    if (t.nt_store)
      hipLaunchKernelGGL((k_direct_allgather<N, V, 2, true, true>), grid, block, 0, s, in, out, slice_vecs, bpr);
    else
      hipLaunchKernelGGL((k_direct_allgather<N, V, 2, false, false>), grid, block, 0, s, in, out, slice_vecs, bpr);
  } else {
    if (t.nt_store)
      hipLaunchKernelGGL((k_direct_allgather<N, V, 1, true, true>), grid, block, 0, s, in, out, slice_vecs, bpr);
    else
      hipLaunchKernelGGL((k_direct_allgather<N, V, 1, false, false>), grid, block, 0, s, in, out, slice_vecs, bpr);
  }
  return hipGetLastError();
}

hipError_t launch_direct_allgather(hipStream_t s, const DeviceInfo &dev, const Tuning &t, int nranks,
                                   const PtrTable &in, const PtrTable &out, size_t nelems,
                                   int vec_halves) {
  if (nelems == 0) return hipSuccess;
#define VR_CASE(NN)                                                              \
  case NN:                                                                       \
    if (vec_halves == 8) return launch_ag<NN, h8>(s, dev, t, in, out, nelems / 8); \
    return launch_ag<NN, h4>(s, dev, t, in, out, nelems / 4);
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

hipError_t launch_copy(hipStream_t s, const DeviceInfo &dev, const Tuning &t, void *dst,
                       const void *src, size_t bytes, int mode) {
  const size_t vecs = bytes / 16;
  if (vecs == 0) return hipSuccess;
  const int unroll = t.unroll >= 4 ? 4 : 1;
  const size_t tile = (size_t)t.block * unroll;
  size_t blocks = (vecs + tile - 1) / tile;
  const size_t resident = (size_t)dev.cus * t.waves_per_cu / (t.block / 64);
  if (!t.oneshot && blocks > resident) blocks = resident;
  const dim3 grid((uint32_t)blocks), block(t.block);
  h8 *d = static_cast<h8 *>(dst);
  const h8 *sp = static_cast<const h8 *>(src);
#define VR_PROBE(M, U)                                                                    \
  if (t.nt_load || t.nt_store)                                                            \
    hipLaunchKernelGGL((k_probe<M, U, true>), grid, block, 0, s, d, sp, vecs);             \
  else                                                                                    \
    hipLaunchKernelGGL((k_probe<M, U, false>), grid, block, 0, s, d, sp, vecs);
#define VR_PROBE_U(M)  \
  if (unroll == 4) {   \
    VR_PROBE(M, 4)     \
  } else {             \
    VR_PROBE(M, 1)     \
  }
  if (mode == 1) {
    VR_PROBE_U(1)
  } else if (mode == 2) {
    VR_PROBE_U(2)
  } else {
    VR_PROBE_U(0)
  }
#undef VR_PROBE_U
#undef VR_PROBE
  return hipGetLastError();
}

}  // namespace vr
