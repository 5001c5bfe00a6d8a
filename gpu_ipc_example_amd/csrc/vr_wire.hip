// Wire transport: the reference's message-passing stage structure on one GPU.
//
// One persistent kernel holds the work-groups of ALL virtual ranks (block b
// belongs to rank b % N), or of a group of consecutive ranks (WireArgs::rank_first,
// rank_count): one rank per launch is how one process per GPU would run it, k
// ranks per launch is k ranks per process.  A wavefront plays the part of
// a reference sub-group ("wire"): it loads its rank's input, pushes messages
// into peers' scatter/gather sinks in device scratch, polls its own sinks, adds
// in the reference's order and stores.  Sink indexing, slot rotation and flag
// values follow parallel_transmit.hpp:47-58,75,93-122, sequential_transmit.hpp:
// 57-81,112-206 (Sequential), 262-278,333-516 (Ring), simple_transmit.hpp:16-179
// and bisect_transmit.hpp:286-424,432-481, re-tiled for 64-lane wavefronts.
//
// Five wire formats:
//   WireLL    (Rt64, rt64.hpp:334-341): every 8-byte store carries 4 bytes
//             of payload and the 4-byte flag, so a message validates itself; the
//             receiver re-polls until a wave-wide vote says every lane's flag is
//             the expected one (the sub-group vote of parallel_transmit.hpp:95-101).
//             Needs nothing but 8-byte store atomicity.
//   WireLL16  (Rt64_PCIE, rt64.hpp:3-20): 16-byte stores of 8 bytes of payload and
//             the flag twice.
//   WireRt128 (Rt64_128, rt64_128.hpp:538-553): the reference's 128-byte message,
//             30 payload dwords and a flag in each 64-byte half, byte for byte.
//   WireRt256 (Rt64_128_PCIE, rt64_128.hpp:3-30): the reference's 256-byte message,
//             60 payload dwords and a flag in each 64-byte quarter, byte for byte.
//   WireFlag  (assumption-free alternative for the Rt64_128 families): payload lines
//             plus a separate flag word, ordered by agent-scope release/acquire
//             fences.
//
// Every poll is bounded: after `spin_limit` unsuccessful polls (or as soon as
// another wave has given up) a wave records a time-out in the status word and
// runs to completion without waiting again, so the grid always drains.

#include <hip/hip_ext.h>

#include <mutex>
#include <unordered_map>

#include "vr_internal.h"

namespace vr {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));

#define VR_AGENT __HIP_MEMORY_SCOPE_AGENT

// Cache-policy operand of the buffer instructions: bit 1 = nt, bit 4 = sc1.
constexpr int kIoCached = 0;
constexpr int kIoStreamLoad = 2;        // nt
constexpr int kIoStreamStore = 2 | 16;  // nt sc1: streaming, written through at agent scope

// Inputs and outputs are addressed through a buffer resource over the bytes that
// remain of the chunk at the wire's offset: the hardware returns zero for loads
// and drops stores at or beyond that length, which is the per-lane predicate of
// the reference's tail wire (rt64_128.hpp:570-582).  The wire's address and
// length depend on the wave's index only; saying so keeps the resource in scalar
// registers.
static __device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(const void *p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  // (the builtin returns int: go through uint32_t, or a low half with bit 31 set
  // would sign-extend into the high half)
  const uint64_t u = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                     ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32);
  const int n = __builtin_amdgcn_readfirstlane((int)bytes);
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char *>(u), 0, n, 0x00020000);
}

typedef unsigned int io_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int io_u32x4 __attribute__((ext_vector_type(4)));

// `io`: bit 0 = streaming cache policy (nt loads, nt sc1 stores) instead of cached
// accesses; bit 1 = the launch's inputs / outputs are only 8-byte aligned, so a
// lane's 16 bytes travel as two 8-byte accesses (same registers, same messages).
constexpr uint32_t kIoStream = 1u, kIoNarrow = 2u;

static __device__ __forceinline__ uint32_t io_ld32(__amdgpu_buffer_rsrc_t rs, uint32_t off, uint32_t io) {
  return (io & kIoStream) ? __builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, kIoStreamLoad)
                          : __builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, kIoCached);
}
static __device__ __forceinline__ io_u32x2 io_ld64(__amdgpu_buffer_rsrc_t rs, uint32_t off, uint32_t io) {
  return (io & kIoStream) ? __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, kIoStreamLoad)
                          : __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, kIoCached);
}
static __device__ __forceinline__ io_u32x4 io_ld128(__amdgpu_buffer_rsrc_t rs, uint32_t off, uint32_t io) {
  if (io & kIoNarrow) {
    const io_u32x2 lo = io_ld64(rs, off, io), hi = io_ld64(rs, off + 8u, io);
    return io_u32x4{lo.x, lo.y, hi.x, hi.y};
  }
  return (io & kIoStream) ? __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, kIoStreamLoad)
                          : __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, kIoCached);
}
static __device__ __forceinline__ void io_st32(__amdgpu_buffer_rsrc_t rs, uint32_t off, uint32_t v, uint32_t io) {
  if (io & kIoStream) __builtin_amdgcn_raw_buffer_store_b32(v, rs, off, 0, kIoStreamStore);
  else __builtin_amdgcn_raw_buffer_store_b32(v, rs, off, 0, kIoCached);
}
static __device__ __forceinline__ void io_st64(__amdgpu_buffer_rsrc_t rs, uint32_t off, io_u32x2 v, uint32_t io) {
  if (io & kIoStream) __builtin_amdgcn_raw_buffer_store_b64(v, rs, off, 0, kIoStreamStore);
  else __builtin_amdgcn_raw_buffer_store_b64(v, rs, off, 0, kIoCached);
}
static __device__ __forceinline__ void io_st128(__amdgpu_buffer_rsrc_t rs, uint32_t off, io_u32x4 v, uint32_t io) {
  if (io & kIoNarrow) {
    io_st64(rs, off, io_u32x2{v.x, v.y}, io);
    io_st64(rs, off + 8u, io_u32x2{v.z, v.w}, io);
    return;
  }
  if (io & kIoStream) __builtin_amdgcn_raw_buffer_store_b128(v, rs, off, 0, kIoStreamStore);
  else __builtin_amdgcn_raw_buffer_store_b128(v, rs, off, 0, kIoCached);
}

struct Spin {
  uint32_t limit;
  uint32_t *status;
  uint32_t lane;
  bool dead;
  // Called after an unsuccessful poll (wave-uniform).  True = stop waiting.
  __device__ __forceinline__ bool give_up(uint32_t &polls) {
    ++polls;
    if (polls >= limit ||
        ((polls & 63u) == 0 && __hip_atomic_load(status, __ATOMIC_RELAXED, VR_AGENT) != 0)) {
      dead = true;
      if (lane == 0) __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, VR_AGENT);
      return true;
    }
    __builtin_amdgcn_s_sleep(1);
    return false;
  }
};

// ---- wire formats ---------------------------------------------------------------

// Every embedded-flag format ends a slot with a flag word (the last lane's last
// dword).  A wave first reads the whole messages (one round trip when they are
// already there).  If some flag is still old it stops re-reading payload and
// watches just that last word of each message: lane i < M loads the last dword
// of slot i, so an unsuccessful look costs one 4-byte access per message.  The
// full read that follows again checks every flag of every message.
template <int M>
static __device__ __forceinline__ bool await_last_flags(const char *const (&slot)[M], uint32_t slot_bytes,
                                                        uint32_t flag, uint32_t lane, Spin &spin) {
  static_assert(M <= 64, "one lane per message");
  if (spin.dead) return false;
  const char *mine = slot[0];
#pragma unroll
  for (int i = 1; i < M; ++i) mine = lane == (uint32_t)i ? slot[i] : mine;
  const uint32_t *word = reinterpret_cast<const uint32_t *>(mine + slot_bytes - 4);
  uint32_t polls = 0;
  for (;;) {
    const bool ok = lane >= (uint32_t)M || __hip_atomic_load(word, __ATOMIC_RELAXED, VR_AGENT) == flag;
    if (__all(ok)) return true;
    if (spin.give_up(polls)) return false;
  }
}

// Row-wise lane moves inside each group of 16 lanes (a DPP row): lane i receives
// the value of lane i - N (shift right) or i + N (shift left); lanes without a
// source keep `old`.
template <int N>
static __device__ __forceinline__ uint32_t row_shr(uint32_t old, uint32_t src) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, 0x110 + N, 0xf, 0xf, false);
}
template <int N>
static __device__ __forceinline__ uint32_t row_shl(uint32_t old, uint32_t src) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, 0x100 + N, 0xf, 0xf, false);
}

constexpr uint32_t kOffNowhere = 0x7ffffff0u;   // beyond any buffer: loads give 0, stores are dropped


template <int U, int DT>
struct WireLL {
  static constexpr uint32_t kWireBytes = 64u * 4u * U;   // payload one wave moves per step
  static constexpr uint32_t kSlotBytes = 64u * 8u * U;   // message bytes in the sink
  static constexpr bool kBatchSends = false;   // the flag travels inside every message
  struct Reg {
    uint32_t d[U];
  };

  static __device__ __forceinline__ Reg load(const char *p, uint32_t left, uint32_t lane, uint32_t nt) {
    Reg r;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) r.d[u] = io_ld32(rs, (u * 64u + lane) * 4u, nt);
    return r;
  }
  static __device__ __forceinline__ void store(char *p, uint32_t left, uint32_t lane, const Reg &r,
                                               uint32_t nt) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) io_st32(rs, (u * 64u + lane) * 4u, r.d[u], nt);
  }
  // v = m + v, element-wise binary16, message on the left (rt64.hpp:452-463).
  static __device__ __forceinline__ void add(Reg &v, const Reg &m) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const h2 s = vadd<DT>(__builtin_bit_cast(h2, m.d[u]), __builtin_bit_cast(h2, v.d[u]));
      v.d[u] = __builtin_bit_cast(uint32_t, s);
    }
  }
  static __device__ __forceinline__ void send(char *slot, uint32_t *, const Reg &v, uint32_t flag,
                                              uint32_t lane) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t msg = (uint64_t)v.d[u] | ((uint64_t)flag << 32);
      __hip_atomic_store(reinterpret_cast<uint64_t *>(slot) + u * 64 + lane, msg, __ATOMIC_RELAXED,
                         VR_AGENT);
    }
  }
  // The same payload to M sinks (the owner's gather), and M payloads to M sinks
  // (a scatter): the flag travels inside every message, nothing to batch.
  template <int M>
  static __device__ __forceinline__ void send_many(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg &v, uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v, flag, lane);
  }
  template <int M>
  static __device__ __forceinline__ void send_each(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg (&v)[M], uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v[i], flag, lane);
  }
  // watch_first: the message is expected to be still on its way, so start by
  // watching its last flag word instead of reading the whole message in vain.
  static __device__ __forceinline__ bool recv(const char *slot, const uint32_t *, Reg &v,
                                              uint32_t flag, uint32_t lane, Spin &spin,
                                              bool watch_first = false) {
    if (spin.dead) return false;
    const char *const one[1] = {slot};
    if (watch_first && !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    uint32_t polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t msg = __hip_atomic_load(reinterpret_cast<const uint64_t *>(slot) + u * 64 + lane,
                                               __ATOMIC_RELAXED, VR_AGENT);
        v.d[u] = (uint32_t)msg;
        ok = ok & ((uint32_t)(msg >> 32) == flag);
      }
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    }
  }
  // M messages at once: all loads are in flight together, so the wait costs one
  // memory round trip instead of M.  Re-polls everything until all have arrived.
  template <int M>
  static __device__ __forceinline__ bool recv_many(const char *const (&slot)[M],
                                                   const uint32_t *const (&)[M], Reg (&v)[M],
                                                   uint32_t flag, uint32_t lane, Spin &spin) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint64_t msg = __hip_atomic_load(
              reinterpret_cast<const uint64_t *>(slot[i]) + u * 64 + lane, __ATOMIC_RELAXED, VR_AGENT);
          v[i].d[u] = (uint32_t)msg;
          ok = ok & ((uint32_t)(msg >> 32) == flag);
        }
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<M>(slot, kSlotBytes, flag, lane, spin)) return false;
    }
  }
};

// Rt64_PCIE (rt64.hpp:3-20, 100-134, 290-315): a lane's message is one 16-byte
// store [d0, d1, flag, flag]: 8 bytes of payload, the flag twice.  The receiver
// accepts a message once both flag words carry the expected value.  Only the
// upper 8 bytes validate themselves, so like the reference's format this rests on
// a lane's 16-byte store becoming visible as a whole (it lies inside one 64-byte
// segment; the 64-byte format below rests on the stronger form of the same
// property).  Moved with buffer instructions: 128-bit accesses with an
// agent-scope policy, which the 64-bit atomic builtins cannot express.
template <int U, int DT>
struct WireLL16 {
  static constexpr uint32_t kWireBytes = 64u * 8u * U;    // payload one wave moves per step
  static constexpr uint32_t kSlotBytes = 64u * 16u * U;   // message bytes in the sink
  static constexpr bool kBatchSends = false;   // the flag travels inside every message
  static constexpr int kAuxAgent = 16;                             // sc1
  static constexpr int kAuxAgentVolatile = (int)0x80000010u;       // sc1, never hoisted or merged
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  struct Reg {
    uint32_t d[U][2];
  };
  // A slot address is the same in every lane of a wave.
  static __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const char *slot) {
    return wave_rsrc(slot, kSlotBytes);
  }
  static __device__ __forceinline__ Reg load(const char *p, uint32_t left, uint32_t lane, uint32_t nt) {
    Reg r;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x2 z = io_ld64(rs, (u * 64u + lane) * 8u, nt);
      r.d[u][0] = z.x;
      r.d[u][1] = z.y;
    }
    return r;
  }
  static __device__ __forceinline__ void store(char *p, uint32_t left, uint32_t lane, const Reg &r,
                                               uint32_t nt) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x2 z = {r.d[u][0], r.d[u][1]};
      io_st64(rs, (u * 64u + lane) * 8u, z, nt);
    }
  }
  static __device__ __forceinline__ void add(Reg &v, const Reg &m) {   // rt64.hpp:126-134
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const h2 s = vadd<DT>(__builtin_bit_cast(h2, m.d[u][k]), __builtin_bit_cast(h2, v.d[u][k]));
        v.d[u][k] = __builtin_bit_cast(uint32_t, s);
      }
  }
  static __device__ __forceinline__ void send(char *slot, uint32_t *, const Reg &v, uint32_t flag,
                                              uint32_t lane) {
    const __amdgpu_buffer_rsrc_t rs = rsrc(slot);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4 msg = {v.d[u][0], v.d[u][1], flag, flag};
      __builtin_amdgcn_raw_buffer_store_b128(msg, rs, (u * 64u + lane) * 16u, 0, kAuxAgent);
    }
  }
  // The same payload to M sinks (the owner's gather), and M payloads to M sinks
  // (a scatter): the flag travels inside every message, nothing to batch.
  template <int M>
  static __device__ __forceinline__ void send_many(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg &v, uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v, flag, lane);
  }
  template <int M>
  static __device__ __forceinline__ void send_each(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg (&v)[M], uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v[i], flag, lane);
  }
  // watch_first: the message is expected to be still on its way, so start by
  // watching its last flag word instead of reading the whole message in vain.
  static __device__ __forceinline__ bool recv(const char *slot, const uint32_t *, Reg &v,
                                              uint32_t flag, uint32_t lane, Spin &spin,
                                              bool watch_first = false) {
    if (spin.dead) return false;
    const char *const one[1] = {slot};
    if (watch_first && !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    const __amdgpu_buffer_rsrc_t rs = rsrc(slot);
    uint32_t polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const u32x4 msg = __builtin_amdgcn_raw_buffer_load_b128(rs, (u * 64u + lane) * 16u, 0, kAuxAgentVolatile);
        v.d[u][0] = msg.x;
        v.d[u][1] = msg.y;
        ok = ok & (msg.z == flag) & (msg.w == flag);
      }
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    }
  }
  template <int M>
  static __device__ __forceinline__ bool recv_many(const char *const (&slot)[M],
                                                   const uint32_t *const (&)[M], Reg (&v)[M],
                                                   uint32_t flag, uint32_t lane, Spin &spin) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < M; ++i) {
        const __amdgpu_buffer_rsrc_t rs = rsrc(slot[i]);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const u32x4 msg = __builtin_amdgcn_raw_buffer_load_b128(rs, (u * 64u + lane) * 16u, 0, kAuxAgentVolatile);
          v[i].d[u][0] = msg.x;
          v[i].d[u][1] = msg.y;
          ok = ok & (msg.z == flag) & (msg.w == flag);
        }
      }
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<M>(slot, kSlotBytes, flag, lane, spin)) return false;
    }
  }
};

// Rt64_128 at sub-group size 16 (rt64_128.hpp:538-553, 635-685, 724-802), byte for
// byte: a 128-byte message is sixteen 8-byte lanes; lanes 0..14 load 120
// contiguous payload bytes; shuffleData parks payload dword 15 (lane 7's second
// dword) in dword 30 (lane 15's first dword); insertFlags writes the flag to
// dwords 15 and 31, one per 64-byte half "because a 128-byte transaction is not
// atomic across HBM channels".  A 64-lane wave carries four such messages side by
// side per instruction (rows of 16 lanes), so a slot is U x 4 reference messages
// over U x 480 consecutive payload bytes.  A receiver accepts a message once
// every flag lane has seen the expected flag (wave vote).  Like the reference's
// format this rests on a 64-byte half written by one store instruction becoming
// visible as a whole.
template <int U, int DT>
struct WireRt128 {
  static constexpr uint32_t kWireBytes = 480u * U;
  static constexpr uint32_t kSlotBytes = 512u * U;
  static constexpr bool kBatchSends = false;   // the flag travels inside every message
  struct Reg {
    uint32_t d[U][2];
  };
  // Byte offset of the lane's 8 payload bytes inside the wire (lane 15 of a row: none).
  static __device__ __forceinline__ uint32_t io_off(int u, uint32_t lane) {
    return (lane & 15u) == 15u ? kOffNowhere : (uint32_t)u * 480u + (lane >> 4) * 120u + (lane & 15u) * 8u;
  }
  static __device__ __forceinline__ Reg load(const char *p, uint32_t left, uint32_t lane, uint32_t nt) {
    Reg r;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x2 z = io_ld64(rs, io_off(u, lane), nt);
      r.d[u][0] = z.x;
      r.d[u][1] = z.y;
    }
    return r;
  }
  static __device__ __forceinline__ void store(char *p, uint32_t left, uint32_t lane, const Reg &r,
                                               uint32_t nt) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x2 z = {r.d[u][0], r.d[u][1]};
      io_st64(rs, io_off(u, lane), z, nt);
    }
  }
  static __device__ __forceinline__ void add(Reg &v, const Reg &m) {   // rt64_128.hpp:947-957
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < 2; ++k) {   // lane 15 adds leftovers; send() rewrites both of its dwords
        const h2 s = vadd<DT>(__builtin_bit_cast(h2, m.d[u][k]), __builtin_bit_cast(h2, v.d[u][k]));
        v.d[u][k] = __builtin_bit_cast(uint32_t, s);
      }
  }
  static __device__ __forceinline__ void send(char *slot, uint32_t *, const Reg &v, uint32_t flag,
                                              uint32_t lane) {
    const uint32_t l = lane & 15u;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t parked = row_shr<8>(0u, v.d[u][1]);                 // lane 15 <- lane 7's second dword
      const uint32_t x = l == 15u ? parked : v.d[u][0];                  // shuffleData
      const uint32_t y = (l == 7u || l == 15u) ? flag : v.d[u][1];       // insertFlags
      __hip_atomic_store(reinterpret_cast<uint64_t *>(slot) + u * 64 + lane, (uint64_t)x | ((uint64_t)y << 32),
                         __ATOMIC_RELAXED, VR_AGENT);
    }
  }
  // The same payload to M sinks (the owner's gather), and M payloads to M sinks
  // (a scatter): the flag travels inside every message, nothing to batch.
  template <int M>
  static __device__ __forceinline__ void send_many(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg &v, uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v, flag, lane);
  }
  template <int M>
  static __device__ __forceinline__ void send_each(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg (&v)[M], uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v[i], flag, lane);
  }
  // All loads of a poll are issued before any of them is looked at, so that a
  // poll costs one memory round trip however many messages it covers.
  static __device__ __forceinline__ uint64_t fetch(const char *slot, int u, uint32_t lane) {
    return __hip_atomic_load(reinterpret_cast<const uint64_t *>(slot) + u * 64 + lane, __ATOMIC_RELAXED,
                             VR_AGENT);
  }
  // Unpacks message u into v, undoing the shuffle; false if a flag lane saw another flag.
  static __device__ __forceinline__ bool decode(uint64_t msg, int u, Reg &v, uint32_t flag, uint32_t lane) {
    const uint32_t l = lane & 15u;
    const uint32_t x = (uint32_t)msg, y = (uint32_t)(msg >> 32);
    const uint32_t back = row_shl<8>(0u, x);                             // lane 7 <- lane 15's first dword
    v.d[u][0] = x;
    v.d[u][1] = l == 7u ? back : y;                                      // restoreData
    return ((l & 7u) != 7u) | (y == flag);
  }
  // watch_first: the message is expected to be still on its way, so start by
  // watching its last flag word instead of reading the whole message in vain.
  static __device__ __forceinline__ bool recv(const char *slot, const uint32_t *, Reg &v,
                                              uint32_t flag, uint32_t lane, Spin &spin,
                                              bool watch_first = false) {
    if (spin.dead) return false;
    const char *const one[1] = {slot};
    if (watch_first && !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    uint32_t polls = 0;
    for (;;) {
      uint64_t raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) raw[u] = fetch(slot, u, lane);
      bool ok = true;
#pragma unroll
      for (int u = 0; u < U; ++u) ok = ok & decode(raw[u], u, v, flag, lane);
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    }
  }
  template <int M>
  static __device__ __forceinline__ bool recv_many(const char *const (&slot)[M],
                                                   const uint32_t *const (&)[M], Reg (&v)[M],
                                                   uint32_t flag, uint32_t lane, Spin &spin) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    for (;;) {
      uint64_t raw[M][U];
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) raw[i][u] = fetch(slot[i], u, lane);
      bool ok = true;
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) ok = ok & decode(raw[i][u], u, v[i], flag, lane);
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<M>(slot, kSlotBytes, flag, lane, spin)) return false;
    }
  }
};

// Rt64_128_PCIE at sub-group size 16 (rt64_128.hpp:3-30, 101-233), byte for byte:
// a 256-byte message is sixteen 16-byte lanes; lanes 0..14 load 240 contiguous
// payload bytes; insertFlags writes the flag to the last dword of lanes 3, 7, 11
// and 15 (dwords 15, 31, 47, 63: one per 64 bytes); shuffleData parks the payload
// dwords displaced from 15, 31 and 47 in lane 15's first three dwords (60, 61,
// 62).  A wave carries four messages per instruction.  Moved with 128-bit buffer
// instructions at agent scope.
template <int U, int DT>
struct WireRt256 {
  static constexpr uint32_t kWireBytes = 960u * U;
  static constexpr uint32_t kSlotBytes = 1024u * U;
  static constexpr bool kBatchSends = false;   // the flag travels inside every message
  static constexpr int kAuxAgent = 16;                             // sc1
  static constexpr int kAuxAgentVolatile = (int)0x80000010u;       // sc1, never hoisted or merged
  struct Reg {
    uint32_t d[U][4];
  };
  static __device__ __forceinline__ uint32_t io_off(int u, uint32_t lane) {
    return (lane & 15u) == 15u ? kOffNowhere : (uint32_t)u * 960u + (lane >> 4) * 240u + (lane & 15u) * 16u;
  }
  static __device__ __forceinline__ Reg load(const char *p, uint32_t left, uint32_t lane, uint32_t nt) {
    Reg r;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x4 z = io_ld128(rs, io_off(u, lane), nt);
      r.d[u][0] = z.x;
      r.d[u][1] = z.y;
      r.d[u][2] = z.z;
      r.d[u][3] = z.w;
    }
    return r;
  }
  static __device__ __forceinline__ void store(char *p, uint32_t left, uint32_t lane, const Reg &r,
                                               uint32_t nt) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const io_u32x4 z = {r.d[u][0], r.d[u][1], r.d[u][2], r.d[u][3]};
      io_st128(rs, io_off(u, lane), z, nt);
    }
  }
  static __device__ __forceinline__ void add(Reg &v, const Reg &m) {   // rt64_128.hpp:516-524
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const h2 s = vadd<DT>(__builtin_bit_cast(h2, m.d[u][k]), __builtin_bit_cast(h2, v.d[u][k]));
        v.d[u][k] = __builtin_bit_cast(uint32_t, s);
      }
  }
  static __device__ __forceinline__ void send(char *slot, uint32_t *, const Reg &v, uint32_t flag,
                                              uint32_t lane) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(slot, kSlotBytes);
    const uint32_t l = lane & 15u;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // shuffleData: lane 15 collects the last dwords of lanes 3, 7 and 11
      const uint32_t p3 = row_shr<12>(0u, v.d[u][3]), p7 = row_shr<8>(0u, v.d[u][3]),
                     p11 = row_shr<4>(0u, v.d[u][3]);
      const bool last = l == 15u;
      const io_u32x4 msg = {last ? p3 : v.d[u][0], last ? p7 : v.d[u][1], last ? p11 : v.d[u][2],
                            (l & 3u) == 3u ? flag : v.d[u][3]};            // insertFlags
      __builtin_amdgcn_raw_buffer_store_b128(msg, rs, (u * 64u + lane) * 16u, 0, kAuxAgent);
    }
  }
  static __device__ __forceinline__ io_u32x4 fetch(__amdgpu_buffer_rsrc_t rs, int u, uint32_t lane) {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, (u * 64u + lane) * 16u, 0, kAuxAgentVolatile);
  }
  static __device__ __forceinline__ bool decode(io_u32x4 msg, int u, Reg &v, uint32_t flag, uint32_t lane) {
    const uint32_t l = lane & 15u;
    // restoreData: lanes 3, 7 and 11 take their last dword back from lane 15
    const uint32_t b3 = row_shl<12>(0u, msg.x), b7 = row_shl<8>(0u, msg.y), b11 = row_shl<4>(0u, msg.z);
    v.d[u][0] = msg.x;
    v.d[u][1] = msg.y;
    v.d[u][2] = msg.z;
    v.d[u][3] = l == 3u ? b3 : l == 7u ? b7 : l == 11u ? b11 : msg.w;
    return ((l & 3u) != 3u) | (msg.w == flag);
  }
  // The same payload to M sinks (the owner's gather), and M payloads to M sinks
  // (a scatter): the flag travels inside every message, nothing to batch.
  template <int M>
  static __device__ __forceinline__ void send_many(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg &v, uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v, flag, lane);
  }
  template <int M>
  static __device__ __forceinline__ void send_each(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg (&v)[M], uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) send(slot[i], fw[i], v[i], flag, lane);
  }
  // watch_first: the message is expected to be still on its way, so start by
  // watching its last flag word instead of reading the whole message in vain.
  static __device__ __forceinline__ bool recv(const char *slot, const uint32_t *, Reg &v,
                                              uint32_t flag, uint32_t lane, Spin &spin,
                                              bool watch_first = false) {
    if (spin.dead) return false;
    const char *const one[1] = {slot};
    if (watch_first && !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(slot, kSlotBytes);
    uint32_t polls = 0;
    for (;;) {
      io_u32x4 raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) raw[u] = fetch(rs, u, lane);
      bool ok = true;
#pragma unroll
      for (int u = 0; u < U; ++u) ok = ok & decode(raw[u], u, v, flag, lane);
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<1>(one, kSlotBytes, flag, lane, spin)) return false;
    }
  }
  template <int M>
  static __device__ __forceinline__ bool recv_many(const char *const (&slot)[M],
                                                   const uint32_t *const (&)[M], Reg (&v)[M],
                                                   uint32_t flag, uint32_t lane, Spin &spin) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    for (;;) {
      io_u32x4 raw[M][U];
#pragma unroll
      for (int i = 0; i < M; ++i) {
        const __amdgpu_buffer_rsrc_t rs = wave_rsrc(slot[i], kSlotBytes);
#pragma unroll
        for (int u = 0; u < U; ++u) raw[i][u] = fetch(rs, u, lane);
      }
      bool ok = true;
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) ok = ok & decode(raw[i][u], u, v[i], flag, lane);
      if (__all(ok)) return true;
      if (spin.give_up(polls) || !await_last_flags<M>(slot, kSlotBytes, flag, lane, spin)) return false;
    }
  }
};

// Flag-word format: full 16-byte-per-lane payload lines plus ONE flag word per
// message in a separate array.  Three ways to order payload and flag:
//   FLAG_FENCE        the sender stores the payload, executes an agent-scope release
//                     fence (buffer_wbl2: L2 write-back), then stores the flag; the
//                     receiver polls the flag word and executes an acquire fence
//                     (buffer_inv: cache invalidate) before it loads the payload.
//                     Assumes nothing beyond the HIP memory model and pays two
//                     cache-maintenance operations per synchronisation for it.
//   FLAG_FENCE_WT     the same fences, payload stored written through at agent scope
//                     (sc1), so the release finds nothing dirty to write back.
//   FLAG_SCOPED       every access at agent scope and no cache maintenance: payload
//                     stores are written through (sc1), the sender waits until they
//                     have completed (s_waitcnt vmcnt(0)) before it stores the flag;
//                     the receiver polls the flag and then loads the payload with
//                     agent-scope loads (sc1), which never hit a stale line.
// A wave that owes several messages at once stores all payloads, synchronises
// ONCE, then stores all flags (send_many / send_each); a wave that waits for
// several polls all flag words and synchronises once (recv_many).
enum FlagSync : int { FLAG_FENCE = 0, FLAG_FENCE_WT = 1, FLAG_SCOPED = 2 };

template <int U, typename V, int DT, int SYNC>
struct WireFlag {
  static constexpr uint32_t kWireBytes = 64u * (uint32_t)sizeof(V) * U;
  static constexpr uint32_t kSlotBytes = kWireBytes;
  static constexpr bool kBatchSends = true;
  static constexpr int kAuxAgent = 16;                             // sc1
  static constexpr int kAuxAgentVolatile = (int)0x80000010u;       // sc1, never hoisted or merged
  struct Reg {
    V d[U];
  };

  static __device__ __forceinline__ Reg load(const char *p, uint32_t left, uint32_t lane, uint32_t nt) {
    Reg r;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t off = (u * 64u + lane) * (uint32_t)sizeof(V);
      if constexpr (sizeof(V) == 16) r.d[u] = __builtin_bit_cast(V, io_ld128(rs, off, nt));
      else r.d[u] = __builtin_bit_cast(V, io_ld64(rs, off, nt));
    }
    return r;
  }
  static __device__ __forceinline__ void store(char *p, uint32_t left, uint32_t lane, const Reg &r,
                                               uint32_t nt) {
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p, left);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t off = (u * 64u + lane) * (uint32_t)sizeof(V);
      if constexpr (sizeof(V) == 16) io_st128(rs, off, __builtin_bit_cast(io_u32x4, r.d[u]), nt);
      else io_st64(rs, off, __builtin_bit_cast(io_u32x2, r.d[u]), nt);
    }
  }
  static __device__ __forceinline__ void add(Reg &v, const Reg &m) {
#pragma unroll
    for (int u = 0; u < U; ++u) v.d[u] = vadd<DT>(m.d[u], v.d[u]);
  }

  // Payload of one message into its slot; not yet announced.
  static __device__ __forceinline__ void put(char *slot, const Reg &v, uint32_t lane) {
    if constexpr (SYNC == FLAG_FENCE) {
#pragma unroll
      for (int u = 0; u < U; ++u) reinterpret_cast<V *>(slot)[u * 64 + lane] = v.d[u];
    } else {
      const __amdgpu_buffer_rsrc_t rs = wave_rsrc(slot, kSlotBytes);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t off = (u * 64u + lane) * (uint32_t)sizeof(V);
        if constexpr (sizeof(V) == 16)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(io_u32x4, v.d[u]), rs, off, 0, kAuxAgent);
        else
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(io_u32x2, v.d[u]), rs, off, 0, kAuxAgent);
      }
    }
  }
  // Everything put so far is visible at agent scope once this returns.
  static __device__ __forceinline__ void publish() {
    if constexpr (SYNC == FLAG_SCOPED) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  }
  // After the flags have been seen: what the senders published may be loaded.
  static __device__ __forceinline__ void subscribe() {
    if constexpr (SYNC == FLAG_SCOPED) asm volatile("" ::: "memory");
    else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  static __device__ __forceinline__ void get(const char *slot, Reg &v, uint32_t lane) {
    if constexpr (SYNC == FLAG_SCOPED) {
      const __amdgpu_buffer_rsrc_t rs = wave_rsrc(slot, kSlotBytes);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t off = (u * 64u + lane) * (uint32_t)sizeof(V);
        if constexpr (sizeof(V) == 16)
          v.d[u] = __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, kAuxAgentVolatile));
        else
          v.d[u] = __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, kAuxAgentVolatile));
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) v.d[u] = reinterpret_cast<const V *>(slot)[u * 64 + lane];
    }
  }
  // Lane i < M stores the flag of message i.
  template <int M>
  static __device__ __forceinline__ void raise(uint32_t *const (&fw)[M], uint32_t flag, uint32_t lane) {
    static_assert(M <= 64, "one lane per flag word");
    uint32_t *mine = fw[0];
#pragma unroll
    for (int i = 1; i < M; ++i) mine = lane == (uint32_t)i ? fw[i] : mine;
    if (lane < (uint32_t)M) __hip_atomic_store(mine, flag, __ATOMIC_RELAXED, VR_AGENT);
  }

  static __device__ __forceinline__ void send(char *slot, uint32_t *flagword, const Reg &v,
                                              uint32_t flag, uint32_t lane) {
    put(slot, v, lane);
    publish();
    if (lane == 0) __hip_atomic_store(flagword, flag, __ATOMIC_RELAXED, VR_AGENT);
  }
  template <int M>
  static __device__ __forceinline__ void send_many(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg &v, uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) put(slot[i], v, lane);
    publish();
    raise<M>(fw, flag, lane);
  }
  template <int M>
  static __device__ __forceinline__ void send_each(char *const (&slot)[M], uint32_t *const (&fw)[M],
                                                   const Reg (&v)[M], uint32_t flag, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < M; ++i) put(slot[i], v[i], lane);
    publish();
    raise<M>(fw, flag, lane);
  }
  static __device__ __forceinline__ bool recv(const char *slot, const uint32_t *flagword, Reg &v,
                                              uint32_t flag, uint32_t lane, Spin &spin,
                                              bool /*watch_first*/ = false) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    // All lanes read the same word, so the loop condition is wave-uniform.
    while (__hip_atomic_load(flagword, __ATOMIC_RELAXED, VR_AGENT) != flag) {
      if (spin.give_up(polls)) return false;
    }
    subscribe();
    get(slot, v, lane);
    return true;
  }
  // M messages: wait for every flag word, synchronise ONCE, then all payloads.
  template <int M>
  static __device__ __forceinline__ bool recv_many(const char *const (&slot)[M],
                                                   const uint32_t *const (&flagword)[M], Reg (&v)[M],
                                                   uint32_t flag, uint32_t lane, Spin &spin) {
    if (spin.dead) return false;
    uint32_t polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < M; ++i)
        ok = ok & (__hip_atomic_load(flagword[i], __ATOMIC_RELAXED, VR_AGENT) == flag);
      if (ok) break;                       // same words in every lane: wave-uniform
      if (spin.give_up(polls)) return false;
    }
    subscribe();
#pragma unroll
    for (int i = 0; i < M; ++i) get(slot[i], v[i], lane);
    return true;
  }
};

// ---- sinks --------------------------------------------------------------------------
// A rank's scatter / gather sink: message slots of W::kSlotBytes, then (at
// flag_off) one flag word per slot.  Slot indices come from vr_wire_layout.h.
template <typename W>
struct Sinks {
  const WireArgs &a;
  __device__ __forceinline__ char *scat(int rank, uint32_t slot) const {
    return static_cast<char *>(a.scatter.p[rank]) + (size_t)slot * W::kSlotBytes;
  }
  __device__ __forceinline__ char *gath(int rank, uint32_t slot) const {
    return static_cast<char *>(a.gather.p[rank]) + (size_t)slot * W::kSlotBytes;
  }
  __device__ __forceinline__ uint32_t *sflag(int rank, uint32_t slot) const {
    return reinterpret_cast<uint32_t *>(static_cast<char *>(a.scatter.p[rank]) + a.flag_off) + slot;
  }
  __device__ __forceinline__ uint32_t *gflag(int rank, uint32_t slot) const {
    return reinterpret_cast<uint32_t *>(static_cast<char *>(a.gather.p[rank]) + a.flag_off) + slot;
  }
};

// Rank and wire of this wave.  A launch holds the work-groups of the ranks
// [rank_first, rank_first + rank_count): all N of them (block b belongs to rank
// b % N), one rank only, or any group in between; block b belongs to rank
// rank_first + b % rank_count.
#define VR_WAVE_PROLOGUE                                                             \
  const uint32_t held = (uint32_t)a.rank_count;                                      \
  const int r = a.rank_first + (int)(blockIdx.x % held);                             \
  const uint32_t lane = threadIdx.x & 63u;                                           \
  const uint32_t wid = (blockIdx.x / held) * (blockDim.x >> 6) + (threadIdx.x >> 6); \
  if (wid >= a.waves_per_rank) return;                                               \
  Spin spin{a.spin_limit, a.status, lane, false};                                    \
  const uint32_t nt = (a.stream_io ? kIoStream : 0u) | (a.io_narrow ? kIoNarrow : 0u);  \
  const size_t chunk = a.chunk_bytes

static __device__ __forceinline__ uint32_t bytes_left(size_t chunk, size_t off, uint32_t wire) {
  const size_t left = chunk - off;
  return left < wire ? (uint32_t)left : wire;
}

// ---- ParallelTransmit::run (parallel_transmit.hpp:63-131) -----------------------------
// N waves per wire column; wave y serves chunk y.  The wave with y == rank owns
// the column's reduction for its rank's chunk.
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_parallel(WireArgs a) {
  constexpr uint32_t NSLOT = wl::kSlotsFlat;
  const uint32_t kAhead = a.ahead;   // 1 ... NSLOT - 2, checked by the host
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t y = wid % N, x_id = wid / N * N;
  const size_t columns = a.waves_per_rank / N;
  const char *src = static_cast<const char *>(a.in.p[r]) + y * chunk;
  char *dst = static_cast<char *>(a.out.p[r]) + y * chunk;
  const size_t first = (size_t)(wid / N) * W::kWireBytes, stride = columns * W::kWireBytes;
  if ((int)y != r) {
    // Scatter, then wait for the gather.  The scatters run kAhead steps ahead of
    // the gathers waited for (kAhead + 1 of the ring's 8 slots in use; the
    // reference's sub-groups stay within one step of each other,
    // parallel_transmit.hpp:88-122), so the owner always finds its next messages
    // waiting and the column runs at the owner's pace.
    auto scatter = [&](size_t off, uint32_t step) {
      const typename W::Reg p = W::load(src + off, bytes_left(chunk, off, W::kWireBytes), lane, nt);
      const uint32_t slot = wl::parallel_slot(x_id, r, step % NSLOT);
      W::send(sk.scat(y, slot), sk.sflag(y, slot), p, a.seq + step / NSLOT, lane);
    };
    for (uint32_t k = 0; k < kAhead; ++k)
      if (first + k * stride < chunk) scatter(first + k * stride, k);
    uint32_t t = 0;
    for (size_t off = first; off < chunk; off += stride, ++t) {
      const uint32_t flag = a.seq + t / NSLOT, s = t % NSLOT;
      const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
      if (off + kAhead * stride < chunk) scatter(off + kAhead * stride, t + kAhead);
      typename W::Reg v;
      const uint32_t slot = wl::parallel_slot(x_id, y, s);
      W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin, true);   // the owner is still reducing
      W::store(dst + off, left, lane, v, nt);
    }
  } else {
    // Wait, reduce, broadcast.
    uint32_t t = 0;
    for (size_t off = first; off < chunk; off += stride, ++t) {
      const uint32_t flag = a.seq + t / NSLOT, s = t % NSLOT;
      const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
      typename W::Reg v = W::load(src + off, left, lane, nt);
      const char *ms[N - 1];
      const uint32_t *mf[N - 1];
      typename W::Reg m[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        const uint32_t slot = wl::parallel_slot(x_id, next, s);
        ms[i] = sk.scat(r, slot);
        mf[i] = sk.sflag(r, slot);
      }
      W::template recv_many<N - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
      for (int i = 0; i < N - 1; ++i) W::add(v, m[i]);    // peers in order rank+1, rank+2, ...
      const uint32_t mine = wl::parallel_slot(x_id, r, s);
      char *gs[N - 1];
      uint32_t *gf[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        gs[i] = sk.gath(next, mine);
        gf[i] = sk.gflag(next, mine);
      }
      W::template send_many<N - 1>(gs, gf, v, flag, lane);
      W::store(dst + off, left, lane, v, nt);
    }
  }
}

// ---- SequentialTransmit::run (sequential_transmit.hpp:83-207) -----------------------------
// One wave does everything its rank owes a wire column, peer after peer.
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_sequential(WireArgs a) {
  constexpr uint32_t NSLOT = wl::kSlotsRing;
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t wpr = a.waves_per_rank;
  const char *src = static_cast<const char *>(a.in.p[r]);
  char *dst = static_cast<char *>(a.out.p[r]);
  uint32_t t = 0;
  for (size_t off = (size_t)wid * W::kWireBytes; off < chunk; off += (size_t)wpr * W::kWireBytes, ++t) {
    const uint32_t flag = a.seq + t / NSLOT, s = t % NSLOT;
    const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
    const uint32_t mine = wl::ring_slot(wpr, r, wid, s);
    if constexpr (W::kBatchSends) {
      // all N - 1 scatters behind one synchronisation
      char *ss[N - 1];
      uint32_t *sf[N - 1];
      typename W::Reg p[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        p[i] = W::load(src + next * chunk + off, left, lane, nt);
        ss[i] = sk.scat(next, mine);
        sf[i] = sk.sflag(next, mine);
      }
      W::template send_each<N - 1>(ss, sf, p, flag, lane);
    } else {
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        const typename W::Reg p = W::load(src + next * chunk + off, left, lane, nt);
        W::send(sk.scat(next, mine), sk.sflag(next, mine), p, flag, lane);
      }
    }
    typename W::Reg v = W::load(src + r * chunk + off, left, lane, nt);
    const char *ms[N - 1];
    const uint32_t *mf[N - 1];
    typename W::Reg m[N - 1];
#pragma unroll
    for (int i = 0; i < N - 1; ++i) {
      const uint32_t slot = wl::ring_slot(wpr, (r + i + 1) % N, wid, s);
      ms[i] = sk.scat(r, slot);
      mf[i] = sk.sflag(r, slot);
    }
    W::template recv_many<N - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
    for (int i = 0; i < N - 1; ++i) W::add(v, m[i]);      // peers in order rank+1, rank+2, ...
    {
      char *gs[N - 1];
      uint32_t *gf[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        gs[i] = sk.gath(next, mine);
        gf[i] = sk.gflag(next, mine);
      }
      W::template send_many<N - 1>(gs, gf, v, flag, lane);
    }
    W::store(dst + r * chunk + off, left, lane, v, nt);
#pragma unroll
    for (int i = 0; i < N - 1; ++i) {
      const uint32_t slot = wl::ring_slot(wpr, (r + i + 1) % N, wid, s);
      ms[i] = sk.gath(r, slot);
      mf[i] = sk.gflag(r, slot);
    }
    W::template recv_many<N - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
    for (int i = 0; i < N - 1; ++i)
      W::store(dst + ((r + i + 1) % N) * chunk + off, left, lane, m[i], nt);
  }
}

// ---- SimpleTransmit (simple_transmit.hpp:16-179) ---------------------------------------------
// The older three-phase form: scatter / pollRecvReduceBcast / pollGatherOutputs.
// Same data flow as the sequential transmit, but the sinks are linear rings: each
// sender owns one section of every peer's sink, a message lands at ringOffset =
// messages sent so far % section, and the flag counts how often the ring has
// wrapped (seqNo + messages / section).  The host launches a power-of-two
// number of wires per rank, so a ring position is only ever reused by the wave
// that used it before.
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_simple(WireArgs a) {
  constexpr uint32_t kPerSection = wl::kSimplePerSection;
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t wpr = a.waves_per_rank;
  const char *src = static_cast<const char *>(a.in.p[r]);
  char *dst = static_cast<char *>(a.out.p[r]);
  size_t t = 0;
  for (size_t off = (size_t)wid * W::kWireBytes; off < chunk; off += (size_t)wpr * W::kWireBytes, ++t) {
    const size_t message = t * wpr + wid;                         // sinkOffset / wireTransSize
    const uint32_t pos = (uint32_t)(message % kPerSection);       // ringOffset
    const uint32_t flag = a.seq + (uint32_t)(message / kPerSection);   // seqNo + seqDelta
    const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
    const uint32_t mine = wl::simple_slot(r, pos);
    if constexpr (W::kBatchSends) {                               // scatter, one synchronisation
      char *ss[N - 1];
      uint32_t *sf[N - 1];
      typename W::Reg p[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        p[i] = W::load(src + next * chunk + off, left, lane, nt);
        ss[i] = sk.scat(next, mine);
        sf[i] = sk.sflag(next, mine);
      }
      W::template send_each<N - 1>(ss, sf, p, flag, lane);
    } else {
      for (int i = 0; i < N - 1; ++i) {                           // scatter
        const int next = (r + i + 1) % N;
        const typename W::Reg p = W::load(src + next * chunk + off, left, lane, nt);
        W::send(sk.scat(next, mine), sk.sflag(next, mine), p, flag, lane);
      }
    }
    typename W::Reg v = W::load(src + r * chunk + off, left, lane, nt);    // pollRecvReduceBcast
    const char *ms[N - 1];
    const uint32_t *mf[N - 1];
    typename W::Reg m[N - 1];
#pragma unroll
    for (int i = 0; i < N - 1; ++i) {
      const uint32_t slot = wl::simple_slot((r + i + 1) % N, pos);
      ms[i] = sk.scat(r, slot);
      mf[i] = sk.sflag(r, slot);
    }
    W::template recv_many<N - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
    for (int i = 0; i < N - 1; ++i) W::add(v, m[i]);
    W::store(dst + r * chunk + off, left, lane, v, nt);           // write back locally first
    {
      char *gs[N - 1];
      uint32_t *gf[N - 1];
#pragma unroll
      for (int i = 0; i < N - 1; ++i) {
        const int next = (r + i + 1) % N;
        gs[i] = sk.gath(next, mine);
        gf[i] = sk.gflag(next, mine);
      }
      W::template send_many<N - 1>(gs, gf, v, flag, lane);
    }
#pragma unroll
    for (int i = 0; i < N - 1; ++i) {                             // pollGatherOutputs
      const uint32_t slot = wl::simple_slot((r + i + 1) % N, pos);
      ms[i] = sk.gath(r, slot);
      mf[i] = sk.gflag(r, slot);
    }
    W::template recv_many<N - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
    for (int i = 0; i < N - 1; ++i)
      W::store(dst + ((r + i + 1) % N) * chunk + off, left, lane, m[i], nt);
  }
}

// ---- RingTransmit::runAllreduce (sequential_transmit.hpp:429-472) ----------------------------
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_ring(WireArgs a) {
  constexpr uint32_t NSLOT = wl::kSlotsRing;
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t wpr = a.waves_per_rank;
  const int next = (r + 1) % N;
  const char *src = static_cast<const char *>(a.in.p[r]);
  char *dst = static_cast<char *>(a.out.p[r]);
  uint32_t t = 0;
  for (size_t off = (size_t)wid * W::kWireBytes; off < chunk; off += (size_t)wpr * W::kWireBytes, ++t) {
    const uint32_t flag = a.seq + t / NSLOT, s = (a.seq + t) % NSLOT;
    const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
    int peer = r;
    uint32_t slot = wl::ring_slot(wpr, peer, wid, s);
    typename W::Reg v = W::load(src + peer * chunk + off, left, lane, nt);       // step 0: send
    W::send(sk.scat(next, slot), sk.sflag(next, slot), v, flag, lane);
    for (int i = 1; i < N - 1; ++i) {                                            // reduce and forward
      peer = (r + N - i) % N;
      slot = wl::ring_slot(wpr, peer, wid, s);
      v = W::load(src + peer * chunk + off, left, lane, nt);
      typename W::Reg m;
      W::recv(sk.scat(r, slot), sk.sflag(r, slot), m, flag, lane, spin);
      W::add(v, m);
      W::send(sk.scat(next, slot), sk.sflag(next, slot), v, flag, lane);
    }
    peer = (r + 1) % N;                                                          // last add, start the gather ring
    slot = wl::ring_slot(wpr, peer, wid, s);
    v = W::load(src + peer * chunk + off, left, lane, nt);
    {
      typename W::Reg m;
      W::recv(sk.scat(r, slot), sk.sflag(r, slot), m, flag, lane, spin);
      W::add(v, m);
    }
    W::send(sk.gath(next, slot), sk.gflag(next, slot), v, flag, lane);
    W::store(dst + peer * chunk + off, left, lane, v, nt);
    for (int i = 1; i < N - 1; ++i) {                                            // forward and write back
      peer = (r + 1 + N - i) % N;
      slot = wl::ring_slot(wpr, peer, wid, s);
      W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin);
      W::send(sk.gath(next, slot), sk.gflag(next, slot), v, flag, lane);
      W::store(dst + peer * chunk + off, left, lane, v, nt);
    }
    peer = (r + 2) % N;                                                          // last hop: write back only
    slot = wl::ring_slot(wpr, peer, wid, s);
    W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin);
    W::store(dst + peer * chunk + off, left, lane, v, nt);
  }
}

// ---- RingTransmit::runAllgather (sequential_transmit.hpp:474-516) ----------------------------
// chunk = bytes of one rank's slice; out[r] holds N slices.
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_allgather(WireArgs a) {
  constexpr uint32_t NSLOT = wl::kSlotsRing;
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t wpr = a.waves_per_rank;
  const int next = (r + 1) % N;
  const char *src = static_cast<const char *>(a.in.p[r]);
  char *dst = static_cast<char *>(a.out.p[r]);
  uint32_t t = 0;
  for (size_t off = (size_t)wid * W::kWireBytes; off < chunk; off += (size_t)wpr * W::kWireBytes, ++t) {
    const uint32_t flag = a.seq + t / NSLOT, s = (a.seq + t) % NSLOT;
    const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
    int peer = r;
    uint32_t slot = wl::ring_slot(wpr, peer, wid, s);
    typename W::Reg v = W::load(src + off, left, lane, nt);
    if (src != dst + (size_t)peer * chunk) W::store(dst + (size_t)peer * chunk + off, left, lane, v, nt);
    W::send(sk.gath(next, slot), sk.gflag(next, slot), v, flag, lane);
    for (int i = 1; i < N - 1; ++i) {
      peer = (r + N - i) % N;
      slot = wl::ring_slot(wpr, peer, wid, s);
      W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin);
      W::send(sk.gath(next, slot), sk.gflag(next, slot), v, flag, lane);
      W::store(dst + (size_t)peer * chunk + off, left, lane, v, nt);
    }
    peer = (r + 1) % N;
    slot = wl::ring_slot(wpr, peer, wid, s);
    W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin);
    W::store(dst + (size_t)peer * chunk + off, left, lane, v, nt);
  }
}

// ---- bisectPAllReduce::operator() (allreduce.hpp:275-296, bisect_transmit.hpp:286-424) -------------
// N/2 waves per wire column; even ranks own the first half of the buffer, odd
// ranks the second; pair exchange first, then the flat exchange among the ranks
// of the same parity.
template <int N, typename W>
__global__ __launch_bounds__(256) void k_wire_bisect(WireArgs a) {
  constexpr uint32_t NSLOT = wl::kSlotsFlat;
  constexpr int B = N / 2;
  VR_WAVE_PROLOGUE;
  const Sinks<W> sk{a};
  const uint32_t y = wid % B, wg = wid / B * B;
  const uint32_t wpr = a.waves_per_rank;
  const size_t columns = wpr / B;
  const int h = r & 1, l = r >> 1, pair = r ^ 1;
  const size_t close_off = (h ? (size_t)B * chunk : 0) + y * chunk;
  const size_t far_off = (h ? 0 : (size_t)B * chunk) + y * chunk;
  const char *src = static_cast<const char *>(a.in.p[r]);
  char *dst = static_cast<char *>(a.out.p[r]);
  const size_t first = (size_t)(wid / B) * W::kWireBytes, stride = columns * W::kWireBytes;
  // The stages that only feed other waves run ahead of the ones that wait (the
  // reference keeps every sub-group inside one step, bisect_transmit.hpp:347-424,
  // and so uses one of its eight slots): scatterFar two steps ahead, the pair sum
  // and the close scatter one step ahead.  Same messages, slots and flag values.
  auto scatter_far = [&](size_t off, uint32_t step) {
    const typename W::Reg f = W::load(src + far_off + off, bytes_left(chunk, off, W::kWireBytes), lane, nt);
    const uint32_t slot = wl::bisect_far_slot(wpr, B, wid, step % NSLOT);
    W::send(sk.scat(pair, slot), sk.sflag(pair, slot), f, a.seq + step / NSLOT, lane);
  };
  // Pair sum of a step, sent on to the chunk's owner unless this wave is the owner.
  auto pair_sum = [&](size_t off, uint32_t step) {
    const uint32_t s = step % NSLOT, flag = a.seq + step / NSLOT;
    typename W::Reg v = W::load(src + close_off + off, bytes_left(chunk, off, W::kWireBytes), lane, nt);
    typename W::Reg m;
    const uint32_t far = wl::bisect_far_slot(wpr, B, wid, s);
    W::recv(sk.scat(r, far), sk.sflag(r, far), m, flag, lane, spin);
    W::add(v, m);
    if ((int)y != l) {
      const int owner = 2 * (int)y + h;
      const uint32_t slot = wl::bisect_close_slot(wg, l, s);
      W::send(sk.scat(owner, slot), sk.sflag(owner, slot), v, flag, lane);
    }
    return v;
  };
  if (first >= chunk) return;
  scatter_far(first, 0);
  if (first + stride < chunk) scatter_far(first + stride, 1);
  typename W::Reg cur = pair_sum(first, 0);
  uint32_t t = 0;
  for (size_t off = first; off < chunk; off += stride, ++t) {
    const uint32_t flag = a.seq + t / NSLOT, s = t % NSLOT;
    const uint32_t left = bytes_left(chunk, off, W::kWireBytes);
    if (off + 2 * stride < chunk) scatter_far(off + 2 * stride, t + 2);
    typename W::Reg nxt = cur;
    if (off + stride < chunk) nxt = pair_sum(off + stride, t + 1);
    typename W::Reg v = cur;
    if ((int)y != l) {
      const uint32_t slot = wl::bisect_close_slot(wg, y, s);
      W::recv(sk.gath(r, slot), sk.gflag(r, slot), v, flag, lane, spin, true);   // the owner is still reducing
    } else {
      const char *ms[B - 1];
      const uint32_t *mf[B - 1];
      typename W::Reg m[B - 1];
#pragma unroll
      for (int i = 0; i < B - 1; ++i) {
        const uint32_t slot = wl::bisect_close_slot(wg, (l + i + 1) % B, s);
        ms[i] = sk.scat(r, slot);
        mf[i] = sk.sflag(r, slot);
      }
      W::template recv_many<B - 1>(ms, mf, m, flag, lane, spin);
#pragma unroll
      for (int i = 0; i < B - 1; ++i) W::add(v, m[i]);    // pair sums in order l+1, l+2, ...
      // gather to the same-parity ranks and forward to the pair (bisect_transmit.hpp:411-417)
      const uint32_t mine = wl::bisect_close_slot(wg, l, s);
      const uint32_t far_out = wl::bisect_far_slot(wpr, B, wid, s);
      char *gs[B];
      uint32_t *gf[B];
#pragma unroll
      for (int i = 0; i < B - 1; ++i) {
        const int nx = (r + i * 2 + 2) % N;
        gs[i] = sk.gath(nx, mine);
        gf[i] = sk.gflag(nx, mine);
      }
      gs[B - 1] = sk.gath(pair, far_out);
      gf[B - 1] = sk.gflag(pair, far_out);
      W::template send_many<B>(gs, gf, v, flag, lane);
    }
    const uint32_t far = wl::bisect_far_slot(wpr, B, wid, s);
    if ((int)y != l) W::send(sk.gath(pair, far), sk.gflag(pair, far), v, flag, lane);
    W::store(dst + close_off + off, left, lane, v, nt);
    {                                                 // pollFarGatherOutput
      typename W::Reg m;
      W::recv(sk.gath(r, far), sk.gflag(r, far), m, flag, lane, spin, true);      // the pair forwards last
      W::store(dst + far_off + off, left, lane, m, nt);
    }
    cur = nxt;
  }
}

// Clears the sinks' flag state on the stream (a fill kernel rather than a memset
// node, so that callers may capture the launch sequence in a graph).
__global__ void k_wire_clear(uint64_t *p, size_t n64) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n64;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = 0;
}

// Clears the first `slot_bytes` bytes (message slots) and the first `flag_bytes`
// bytes at `flag_off` (flag words) of every rank's scatter and gather sink: what
// one launch is about to use.  blockIdx.y picks the sink; all sizes are multiples
// of 16.
__global__ void k_wire_clear_sinks(PtrTable scatter, PtrTable gather, int nranks, size_t slot_bytes,
                                   size_t flag_off, size_t flag_bytes) {
  const int which = (int)blockIdx.y;
  char *sink = static_cast<char *>(which < nranks ? scatter.p[which] : gather.p[which - nranks]);
  const size_t n_slots = slot_bytes / 16, n_flags = flag_bytes / 16;
  const io_u32x4 zero = {0u, 0u, 0u, 0u};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_slots + n_flags;
       i += (size_t)gridDim.x * blockDim.x) {
    io_u32x4 *p = reinterpret_cast<io_u32x4 *>(i < n_slots ? sink + i * 16 : sink + flag_off + (i - n_slots) * 16);
    __builtin_nontemporal_store(zero, p);   // streamed: nothing is left dirty in L2 for the kernel's end to write back
  }
}

// Messages per lane and step for each format; every slot stays within 2 KiB.
constexpr int kUnrollLL = 4;     // 1 KiB payload in a 2 KiB message
constexpr int kUnrollLL16 = 2;   // 1 KiB payload in a 2 KiB message
constexpr int kUnrollRt128 = 4;  // 1920 B payload in a 2 KiB slot (sixteen 128-byte messages)
constexpr int kUnrollRt256 = 2;  // 1920 B payload in a 2 KiB slot (eight 256-byte messages)
constexpr int kUnrollFlag = 2;   // 2 KiB payload (16-byte lanes), flag word elsewhere

static_assert(WireLL<kUnrollLL, DT_F16>::kSlotBytes <= wl::kSlotBytesMax, "slot too large");
static_assert(WireLL16<kUnrollLL16, DT_F16>::kSlotBytes <= wl::kSlotBytesMax, "slot too large");
static_assert(WireRt128<kUnrollRt128, DT_F16>::kSlotBytes <= wl::kSlotBytesMax, "slot too large");
static_assert(WireRt256<kUnrollRt256, DT_F16>::kSlotBytes <= wl::kSlotBytesMax, "slot too large");
static_assert(WireFlag<kUnrollFlag, h8, DT_F16, FLAG_FENCE>::kSlotBytes <= wl::kSlotBytesMax, "slot too large");

// ---- the library's own scratch -----------------------------------------------------------
// Fixed region for the entry point that must not allocate: every rank's scatter
// and gather sink for up to kStaticMaxRanks ranks of kStaticWiresPerRank wires
// (no SimpleTransmit sections), padded by 256 bytes.  In host code the array's
// name is only a handle: its device address is looked up once per device with
// hipGetSymbolAddress.
constexpr size_t kStaticScratchBytes =
    (size_t)kStaticMaxRanks * wl::layout_for(kStaticMaxRanks, kStaticWiresPerRank, false).rank_bytes + 256;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_static_ptr[kMaxDevices];

hipError_t wire_static_scratch(int device, void **ptr, size_t *bytes) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  static std::mutex lock;   // contexts may be created from several threads
  std::lock_guard<std::mutex> hold(lock);
  if (!g_static_ptr[device]) {
    // The caller has made `device` current: each GPU holds its own copy of the
    // array at its own address.
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_static_ptr[device] = p;
  }
  *ptr = g_static_ptr[device];
  *bytes = kStaticScratchBytes;
  return hipSuccess;
}

// ---- host side --------------------------------------------------------------------------

// The kernel of a flow for a wire format W.
template <typename W>
static const void *flow_kernel(WireFlow flow, int nranks) {
  const void *fn = nullptr;
  // World sizes the reference's dispatchers instantiate: 2, 4, 8 for the flat and
  // ring transmits (allreduce.cpp:854-881), 4, 8, 16 for bisect (l.1003-1030).
#define VR_PICK(NN)                                                                         \
  case NN:                                                                                  \
    if constexpr (NN <= 8) {                                                                \
      switch (flow) {                                                                       \
        case WIRE_PARALLEL: fn = reinterpret_cast<const void *>(&k_wire_parallel<NN, W>); break;   \
        case WIRE_SEQUENTIAL: fn = reinterpret_cast<const void *>(&k_wire_sequential<NN, W>); break; \
        case WIRE_SIMPLE: fn = reinterpret_cast<const void *>(&k_wire_simple<NN, W>); break;         \
        case WIRE_RING: fn = reinterpret_cast<const void *>(&k_wire_ring<NN, W>); break;           \
        case WIRE_ALLGATHER: fn = reinterpret_cast<const void *>(&k_wire_allgather<NN, W>); break;  \
        default: break;                                                                     \
      }                                                                                     \
    }                                                                                       \
    if constexpr (NN >= 4) {                                                                \
      if (flow == WIRE_BISECT) fn = reinterpret_cast<const void *>(&k_wire_bisect<NN, W>);  \
    }                                                                                       \
    break;
  switch (nranks) {
    VR_PICK(2)
    VR_PICK(4)
    VR_PICK(8)
    VR_PICK(16)
    default: break;
  }
#undef VR_PICK
  return fn;
}

template <int DT>
static const void *wire_kernel_dt(WireFlow flow, WireFormat fmt, int vec_halves, int nranks) {
  switch (fmt) {
    case WIRE_FMT_LL: return flow_kernel<WireLL<kUnrollLL, DT>>(flow, nranks);
    case WIRE_FMT_RT128: return flow_kernel<WireRt128<kUnrollRt128, DT>>(flow, nranks);
    case WIRE_FMT_RT256: return flow_kernel<WireRt256<kUnrollRt256, DT>>(flow, nranks);
    case WIRE_FMT_LL16: return flow_kernel<WireLL16<kUnrollLL16, DT>>(flow, nranks);
    case WIRE_FMT_FLAG_WT:
      return vec_halves == 8 ? flow_kernel<WireFlag<kUnrollFlag, h8, DT, FLAG_FENCE_WT>>(flow, nranks)
                             : flow_kernel<WireFlag<kUnrollFlag, h4, DT, FLAG_FENCE_WT>>(flow, nranks);
    case WIRE_FMT_FLAG_SCOPED:
      return vec_halves == 8 ? flow_kernel<WireFlag<kUnrollFlag, h8, DT, FLAG_SCOPED>>(flow, nranks)
                             : flow_kernel<WireFlag<kUnrollFlag, h4, DT, FLAG_SCOPED>>(flow, nranks);
    default:
      return vec_halves == 8 ? flow_kernel<WireFlag<kUnrollFlag, h8, DT, FLAG_FENCE>>(flow, nranks)
                             : flow_kernel<WireFlag<kUnrollFlag, h4, DT, FLAG_FENCE>>(flow, nranks);
  }
}

static const void *wire_kernel(WireFlow flow, WireFormat fmt, int vec_halves, int nranks, DType dtype) {
  return dtype == DT_BF16 ? wire_kernel_dt<DT_BF16>(flow, fmt, vec_halves, nranks)
                          : wire_kernel_dt<DT_F16>(flow, fmt, vec_halves, nranks);
}

uint32_t wire_bytes_per_step(WireFormat fmt, int vec_halves) {
  switch (fmt) {
    case WIRE_FMT_LL: return WireLL<kUnrollLL, DT_F16>::kWireBytes;
    case WIRE_FMT_RT128: return WireRt128<kUnrollRt128, DT_F16>::kWireBytes;
    case WIRE_FMT_RT256: return WireRt256<kUnrollRt256, DT_F16>::kWireBytes;
    case WIRE_FMT_LL16: return WireLL16<kUnrollLL16, DT_F16>::kWireBytes;
    default:   // the three flag-word variants move the same wires
      return vec_halves == 8 ? WireFlag<kUnrollFlag, h8, DT_F16, FLAG_FENCE>::kWireBytes
                             : WireFlag<kUnrollFlag, h4, DT_F16, FLAG_FENCE>::kWireBytes;
  }
}

uint32_t wire_slot_bytes(WireFormat fmt, int vec_halves) {
  switch (fmt) {
    case WIRE_FMT_LL: return WireLL<kUnrollLL, DT_F16>::kSlotBytes;
    case WIRE_FMT_RT128: return WireRt128<kUnrollRt128, DT_F16>::kSlotBytes;
    case WIRE_FMT_RT256: return WireRt256<kUnrollRt256, DT_F16>::kSlotBytes;
    case WIRE_FMT_LL16: return WireLL16<kUnrollLL16, DT_F16>::kSlotBytes;
    default:
      return vec_halves == 8 ? WireFlag<kUnrollFlag, h8, DT_F16, FLAG_FENCE>::kSlotBytes
                             : WireFlag<kUnrollFlag, h4, DT_F16, FLAG_FENCE>::kSlotBytes;
  }
}

// Waves spin on other work-groups' progress, which is only safe when all of them
// are resident at once.  The occupancy query says how many work-groups of the
// flow's kernel one compute unit holds; the host keeps every grid within that
// bound, so it is co-resident on a device that runs nothing else.
hipError_t wire_blocks_per_cu(WireFlow flow, WireFormat fmt, int vec_halves, int nranks,
                              uint32_t block_threads, DType dtype, int *per_cu) {
  const void *fn = wire_kernel(flow, fmt, vec_halves, nranks, dtype);
  if (!fn) return hipErrorInvalidValue;
  // The answer is a property of the kernel (every launch uses the same block size
  // and no dynamic LDS): ask the runtime once per kernel, not once per launch.
  static std::mutex lock;
  static std::unordered_map<const void *, int> known;
  {
    std::lock_guard<std::mutex> hold(lock);
    const auto it = known.find(fn);
    if (it != known.end()) {
      *per_cu = it->second;
      return hipSuccess;
    }
  }
  const hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, fn, (int)block_threads, 0);
  if (e == hipSuccess) {
    std::lock_guard<std::mutex> hold(lock);
    known[fn] = *per_cu;
  }
  return e;
}

// cooperative: a cooperative launch makes the runtime check co-residency once
// more; the plain launch path is about 16 us shorter.
hipError_t launch_wire(hipStream_t s, WireFlow flow, WireFormat fmt, int vec_halves, int nranks,
                       uint32_t blocks, uint32_t block_threads, WireArgs &args, bool cooperative,
                       DType dtype) {
  const void *fn = wire_kernel(flow, fmt, vec_halves, nranks, dtype);
  if (!fn) return hipErrorInvalidValue;
  void *kargs[] = {&args};
  const dim3 grid(blocks), block(block_threads);
  if (cooperative) return hipLaunchCooperativeKernel(fn, grid, block, kargs, 0, s);
  if (tl_kernel_events.start || tl_kernel_events.stop)
    return hipExtLaunchKernel(fn, grid, block, kargs, 0, s, tl_kernel_events.start, tl_kernel_events.stop, 0);
  return hipLaunchKernel(fn, grid, block, kargs, 0, s);
}

hipError_t launch_wire_clear_sinks(hipStream_t s, const PtrTable &scatter, const PtrTable &gather, int nranks,
                                   size_t slot_bytes, size_t flag_off, size_t flag_bytes) {
  slot_bytes = (slot_bytes + 15) / 16 * 16;
  flag_bytes = (flag_bytes + 15) / 16 * 16;
  if (flag_off % 16) return hipErrorInvalidValue;
  const size_t per_sink = (slot_bytes + flag_bytes) / 16;
  if (per_sink == 0) return hipSuccess;
  size_t bx = (per_sink + 255) / 256;
  if (bx > 256) bx = 256;
  hipLaunchKernelGGL(k_wire_clear_sinks, dim3((uint32_t)bx, 2u * (uint32_t)nranks), dim3(256), 0, s, scatter,
                     gather, nranks, slot_bytes, flag_off, flag_bytes);
  return hipGetLastError();
}

hipError_t launch_wire_clear(hipStream_t s, void *p, size_t bytes) {
  if (bytes == 0) return hipSuccess;
  hipLaunchKernelGGL(k_wire_clear, dim3(1024), dim3(256), 0, s, static_cast<uint64_t *>(p), bytes / 8);
  return hipGetLastError();
}

}  // namespace vr
