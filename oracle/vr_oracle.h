/*
 * vr_oracle.h — CPU restatement of the reference's single-shot all-reduce /
 * all-gather arithmetic.  TEST INFRASTRUCTURE ONLY: nothing that ships (the
 * HIP library, its C++ host wrapper, the CLI) may link or call this; only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * All half-precision buffers are passed as raw IEEE binary16 bit patterns
 * (uint16_t) so that no compiler's notion of "half" leaks into the contract.
 *
 * Parity status of each function (what pins it) is listed next to its
 * declaration; a function with no independent pin would say "parity unpinned".
 */
#ifndef VR_ORACLE_H
#define VR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- binary16 arithmetic ------------------------------------------------ */

/* IEEE-754 binary16 add, round-to-nearest-even, subnormals kept, written with
 * integer operations only.  Restates the `sycl::vec<half,k>::operator+` used by
 * rt64.hpp:452-463, rt64_128.hpp:947-957, bisect_transmit.hpp:273-284.
 * Pinned by: exhaustive agreement with vro_f16_add (float path, all 2^32
 * pairs), numpy.float16 on stratified samples, and the textbook special cases
 * (ties-to-even 2048+1, 2048+3; overflow 65504+15 / +16; subnormal sums). */
uint16_t vro_f16_add_soft(uint16_t a, uint16_t b);

/* Same add computed as half(float(a)+float(b)) — how the reference's host
 * oracle evaluates `sum += x` on sycl::half (allreduce.cpp:18-27).  Exact
 * because 24 >= 2*11+2 makes the double rounding innocuous.  Uses F16C when the
 * CPU has it, otherwise integer conversions. */
uint16_t vro_f16_add(uint16_t a, uint16_t b);

float    vro_f16_to_f32(uint16_t h);
uint16_t vro_f32_to_f16(float f);          /* RNE, overflow -> inf */

/* 1 if both are NaN or the bit patterns are equal. */
int vro_f16_same(uint16_t a, uint16_t b);

/* ---- fixtures and generators --------------------------------------------- */

/* utils.hpp:15-19: input[i] = (T)((i % 32) * (rank + 1)). */
void vro_fill_pattern(uint16_t *buf, int rank, size_t n);

enum { VRO_DIST_UNIFORM = 0, VRO_DIST_NORMAL = 1 };

/* Seeded synthetic data: splitmix64 stream keyed by `seed`; element i uses
 * draws 2i and 2i+1 so that any sub-range can be generated independently.
 *   UNIFORM: lo + (hi-lo)*u,          p0 = lo,   p1 = hi
 *   NORMAL : mean + sd*BoxMuller(u,v), p0 = mean, p1 = sd
 * computed in double, rounded once to binary16 (RNE). */
void vro_generate(uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1);

/* ---- chunking (allreduce.hpp:108-122, allgather.hpp:104-117) --------------- */

enum {
  VRO_OK = 0,
  VRO_ERR_UNALIGNED = 1,  /* "We only support aligned pointer for now"   */
  VRO_ERR_UNEVEN = 2,     /* "We don't support non-even divide yet"      */
};

/* Returns the status; on VRO_OK *work_bytes = bytes each rank-chunk holds.
 * msg_bytes = sizeof(message_t) of the protocol (8 or 16). nchunks = NRanks for
 * all-reduce, 1 for all-gather. */
int vro_calc_work_size(uintptr_t input_addr, size_t bytes, int nchunks, size_t msg_bytes,
                       size_t *work_bytes);

/* ---- summation orders ------------------------------------------------------- *
 * Each returns 0, or -2 when the shape is outside what the reference accepts
 * (n not a multiple of nranks; bisect with an odd or < 4 rank count). */

/* Reference host oracle (allreduce.cpp:18-27): sum = 0; for r in 0..N-1: sum += x_r[i].
 * Pinned by fill_pattern closed form (i%32)*N(N+1)/2 and brute force on tiny inputs. */
int vro_allreduce_rank_order(uint16_t *out, const uint16_t *const in[], int nranks, size_t n);

/* Device order of ParallelTransmit / SequentialTransmit / RingTransmit / SimpleTransmit
 * (parallel_transmit.hpp:51-55,82-116; sequential_transmit.hpp:135-171,429-472;
 * simple_transmit.hpp:27-29,122-131): element i lies in chunk c = i / (n/N); the
 * chain starts at the chunk owner c and walks ranks c+1, c+2, ... mod N, no zero
 * initial value.  n must be a multiple of N.
 * Pinned by the N=4 and N=8 hand KATs (2048,1,1,0 / 2048,0,1,0,1,0,0,0), by
 * agreement with the message-level emulators below, and by fill_pattern. */
int vro_allreduce_rotated(uint16_t *out, const uint16_t *const in[], int nranks, size_t n);

/* Device order of BisectPTransmit (bisect_transmit.hpp:347-424,432-481): pair sums
 * p_j = x_{2j} + x_{2j+1}; chunk c = h*(N/2)+l is owned by rank 2l+h and equals
 * ((p_l + p_{l+1}) + p_{l+2}) + ... with pair indices mod N/2.  N even, n % N == 0.
 * Pinned by the N=4 / N=8 three-way KATs, the emulator, and fill_pattern. */
int vro_allreduce_bisect(uint16_t *out, const uint16_t *const in[], int nranks, size_t n);

/* allreduce.cpp:30-35: out[r*n + i] = in_r[i].  Pinned by the copy invariant. */
void vro_allgather(uint16_t *out, const uint16_t *const in[], int nranks, size_t n);

/* Number of positions where a and b differ (NaN == NaN). */
size_t vro_count_mismatch(const uint16_t *a, const uint16_t *b, size_t n);

/* ---- message-level emulation of the reference kernels ------------------------ *
 * A second, independent restatement: it moves wires through scatter / gather
 * sinks exactly as the device code indexes them, one virtual rank after the
 * other, instead of using the closed-form orders above.  `io[r]` is rank r's
 * in-place buffer of n halves.  groups/subgroups give the launch geometry of
 * main.cpp (-g, -w; total sub-groups = groups*subgroups).  Returns 0, or a
 * negative value when a poll would never be satisfied (protocol violation). */

enum {
  VRO_WIRE_RT64 = 0,      /* rt64.hpp:334-341      64 B payload / 128 B message (SG16) */
  VRO_WIRE_RT64_128 = 1,  /* rt64_128.hpp:538-553 120 B payload / 128 B message        */
  VRO_WIRE_RT64_PCIE = 2,      /* rt64.hpp:3-9       128 B payload / 256 B message (ring, sequential, all-gather) */
  VRO_WIRE_RT64_128_PCIE = 3,  /* rt64_128.hpp:3-21  240 B payload / 256 B message (ring, sequential, all-gather) */
};

/* One message of a wire format, byte for byte as the reference's device code lays it
 * out at sub-group size 16: `payload` holds vro_wire_payload_dwords(wire) dwords,
 * `msg` vro_wire_message_dwords(wire) dwords (32 or 64).  Unpack returns -1 when a
 * flag position does not carry `flag`.  Pinned by hand-derived positions
 * (rt64.hpp:3-20, 335-341; rt64_128.hpp:7-13, 101-117, 194-203, 544-553, 635-685,
 * 724-762) and the reference's dead stage verifier (allreduce.cpp:71, 131-133). */
int vro_wire_payload_dwords(int wire);
int vro_wire_message_dwords(int wire);
int vro_pack_message(int wire, uint32_t *msg, const uint32_t *payload, uint32_t flag);
int vro_unpack_message(int wire, const uint32_t *msg, uint32_t *payload, uint32_t flag);

/* AllReduce<T,N,Proto,ParallelTransmit,16>::operator() for every rank
 * (allreduce.hpp:83-104 + parallel_transmit.hpp:63-131). */
int vro_emulate_parallel(uint16_t *const io[], int nranks, size_t n, int wire,
                         int groups, int subgroups, uint32_t seq_no);

/* AllReduce<T,N,Proto,RingTransmit,16> (sequential_transmit.hpp:429-472); the
 * messages travel packed in the wire format's byte layout. */
int vro_emulate_ring(uint16_t *const io[], int nranks, size_t n, int wire,
                     int groups, int subgroups, uint32_t seq_no);

/* AllReduce<T,N,Proto,SequentialTransmit,16> (sequential_transmit.hpp:57-81, 83-207). */
int vro_emulate_sequential(uint16_t *const io[], int nranks, size_t n, int wire,
                           int groups, int subgroups, uint32_t seq_no);

/* AllGather<T,N,Proto,RingTransmit,16> (allgather.hpp:79-100 + sequential_transmit.hpp:
 * 474-516).  out[r] holds nranks * n halves; out[r] + r * n may alias in[r]. */
int vro_emulate_allgather_ring(uint16_t *const out[], const uint16_t *const in[], int nranks, size_t n,
                               int wire, int groups, int subgroups, uint32_t seq_no);

/* bisectPAllReduce<T,N,BisectPTransmit,16> (allreduce.hpp:275-296 +
 * bisect_transmit.hpp:286-424). */
int vro_emulate_bisect(uint16_t *const io[], int nranks, size_t n,
                       int groups, int subgroups, uint32_t seq_no);

/* ---- bfloat16 (the reference's other instantiated type, allreduce.cpp:1229-1294) ------- *
 * sycl::ext::oneapi::bfloat16 adds as float and rounds the sum to nearest even;
 * `dtype` below is VRO_F16 or VRO_BF16 and selects the element arithmetic of the
 * same order / emulator code.  Pinned by torch.bfloat16 CPU arithmetic on random
 * and boundary operands, hand cases (256+1, 256+3, overflow to inf) and the
 * emulator-vs-closed-form agreement. */
enum { VRO_F16 = 0, VRO_BF16 = 1 };
uint16_t vro_bf16_add(uint16_t a, uint16_t b);
uint16_t vro_f64_to_bf16(double d);
void vro_fill_pattern_dt(int dtype, uint16_t *buf, int rank, size_t n);
void vro_generate_dt(int dtype, uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1);
/* mode: 0 rank order, 1 rotated, 2 bisect. */
int vro_allreduce_order_dt(int dtype, int mode, uint16_t *out, const uint16_t *const in[], int nranks,
                           size_t n);
int vro_emulate_parallel_dt(int dtype, uint16_t *const io[], int nranks, size_t n, int wire, int groups,
                            int subgroups, uint32_t seq_no);
int vro_emulate_bisect_dt(int dtype, uint16_t *const io[], int nranks, size_t n, int groups,
                          int subgroups, uint32_t seq_no);

/* ---- host threading for the timed baseline ---------------------------------- */
/* The order functions are OpenMP-parallel over elements like the reference's
 * host loop; this sets the thread count (0 = leave the runtime's default) and
 * returns the count that will be used. */
int vro_set_threads(int nthreads);

#ifdef __cplusplus
}
#endif
#endif /* VR_ORACLE_H */
