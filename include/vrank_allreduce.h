/*
 * vrank_allreduce.h — C ABI of the MI355X single-shot all-reduce / all-gather
 * data path over "virtual ranks" (NRanks separate device allocations in one
 * GPU's HBM).
 *
 * This is the boundary a host program binds instead of the reference's SYCL
 * functors.  Plain pointers and sizes only; every function returns a vr_status
 * (0 = success) and never throws.  The C++ header vrank/allreduce.hpp turns the
 * codes back into the reference's std::logic_error texts.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   vr_allreduce      <- AllReduce<T,N,Proto,Transmit>::launch       allreduce.hpp:64-74
 *                        bisectPAllReduce<T,N>::launch               allreduce.hpp:260-270
 *                        testTransmit<T>(std::string algo, ...)      allreduce.cpp:1118-1189
 *   vr_allgather      <- AllGather<T,N,Proto,Transmit>::launch       allgather.hpp:58-70
 *                        testAllgather<T>(std::string algo, ...)     allreduce.cpp:1191-1213
 *   vr_check_allreduce<- AllReduce::calcWorkSize                     allreduce.hpp:108-122
 *   vr_check_allgather<- AllGather::calcWorkSize                     allgather.hpp:104-117
 *   vr_launch_geometry<- AllReduce::getLaunchParam                   allreduce.hpp:37-62, 237-258
 *   vr_algo_from_string<- the -a string switch                       allreduce.cpp:1128-1188, 1198-1212
 *   vr_fill_pattern   <- fill_pattern                                utils.hpp:15-19
 *   vr_parse_nelems   <- parse_nelems                                main.cpp:17-34
 *   vr_ctx_create     <- per-process set-up                          main.cpp:212-227
 *   vr_ctx_reserve_wire<- scratch allocation + zeroing + peer tables  main.cpp:241-283
 *   vr_allreduce_rank <- AllReduce(input, nelems, rank, seqNo, scatterBuf, gatherBuf,
 *                        peerBuf0[], peerBuf1[]) + queue.submit      allreduce.hpp:18-28, 64-74
 *                        ParallelTransmit / BisectPTransmit ctors    parallel_transmit.hpp:36-60,
 *                                                                    bisect_transmit.hpp:427-482
 *   vr_allgather_rank <- AllGather(input, output, nelems, rank, seqNo, ...)  allgather.hpp:19-29, 58-70
 *   vr_allgather_grid, vr_allgather_rank_grid
 *                     <- testAllgather<T>(algo, nd_range, input, output, ipcbuf0, ipcbuf1, peerbuf0,
 *                        peerbuf1, nelems, rank, world, step, subgroup, queue)  allreduce.cpp:1191-1213,
 *                        called by benchAllgather with the -g/-w/-s grid    main.cpp:110-166, 296-314
 *   vr_allreduce_ranks, vr_allgather_ranks
 *                     <- the same constructors for a process that holds k of the N ranks
 *                        (the reference always holds one: main.cpp:212-227)
 *   vr_rank_scratch_bytes <- interm_size = world * 8 MiB             main.cpp:241
 *   vr_ipc_open_all   <- open_all_ipc_mems                           ipc_exchange.cpp:277-311
 *                        (un_allgather over AF_UNIX sockets,         ipc_exchange.cpp:173-265)
 *   vr_ipc_barrier    <- MPI_Barrier                                 main.cpp:101, 287
 */
#ifndef VRANK_ALLREDUCE_H
#define VRANK_ALLREDUCE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VR_MAX_RANKS 16

typedef enum vr_status {
  VR_OK = 0,
  VR_ERR_UNALIGNED = 1,   /* "We only support aligned pointer for now"      allreduce.hpp:111 */
  VR_ERR_UNEVEN = 2,      /* "We don't support non-even divide yet"         allreduce.hpp:118 */
  VR_ERR_ALGO = 3,        /* "Transmit type not support"                    allreduce.cpp:1187 */
  VR_ERR_TOPOLOGY = 4,    /* "Unsupported communication topology"           allreduce.cpp:880  */
  VR_ERR_SUBGROUP = 5,    /* "Unsupported Sub-group size"                   allreduce.cpp:917  */
  VR_ERR_GEOMETRY = 6,    /* "Subgroup numbers must be multiple of 4"       main.cpp:289-291   */
  VR_ERR_INVALID = 7,     /* null pointer / bad enum / size beyond what the context was built for */
  VR_ERR_HIP = 8,         /* a HIP runtime call failed; see vr_last_error_detail()             */
  VR_ERR_NO_DEVICE = 9,   /* no gfx950 device visible                                          */
  VR_ERR_TIMEOUT = 10,    /* a flag poll in the wire transport exceeded its spin limit         */
  VR_ERR_OVERLAP = 11,    /* out-of-place buffers alias in a way the kernel cannot honour      */
} vr_status;

/* The -a strings of the reference (README.md:18, allreduce.cpp:1128-1212) plus
 * "parallel" (ParallelTransmit named directly). */
typedef enum vr_algo {
  VR_ALGO_SMALL = 0,            /* Rt64          + ParallelTransmit   */
  VR_ALGO_SIMPLE = 1,           /* Rt64_128      + ParallelTransmit   */
  VR_ALGO_BISECT = 2,           /* BisectPTransmit                    */
  VR_ALGO_PARALLEL = 3,         /* ParallelTransmit, message-passing form (see vr_transport) */
  VR_ALGO_SMALL_PCIE_P = 4,     /* Rt64_PCIE     + ParallelTransmit   */
  VR_ALGO_SIMPLE_PCIE_P = 5,    /* Rt64_128_PCIE + ParallelTransmit   */
  VR_ALGO_SMALL_RING = 6,       /* Rt64_PCIE     + RingTransmit       */
  VR_ALGO_SIMPLE_RING = 7,      /* Rt64_128_PCIE + RingTransmit       */
  VR_ALGO_SMALL_PCIE = 8,       /* Rt64_PCIE     + SequentialTransmit */
  VR_ALGO_SIMPLE_PCIE = 9,      /* Rt64_128_PCIE + SequentialTransmit */
  VR_ALGO_ALLGATHER_SMALL = 10, /* Rt64_PCIE     + RingTransmit::runAllgather */
  VR_ALGO_ALLGATHER_SIMPLE = 11,/* Rt64_128_PCIE + RingTransmit::runAllgather */
  VR_ALGO_SIMPLE_TRANSMIT = 12, /* Rt64_128 + SimpleTransmit (simple_transmit.hpp; has no -a string
                                   in the reference, whose include of it is disabled) */
  VR_ALGO_COUNT_
} vr_algo;

/* How data travels between virtual ranks.
 *  DIRECT: the workgroups of the rank that owns a chunk read every rank's input
 *          in place, add in the protocol's order, and write every rank's output.
 *          One pass over HBM; no scratch, no flags.  Default for every algo
 *          except VR_ALGO_PARALLEL.
 *  WIRE  : the reference's stage structure — scatter into the owner's sink,
 *          reduce, gather into every peer's sink — through the context's scratch,
 *          one persistent kernel whose workgroups are partitioned between the
 *          virtual ranks.  Receivers learn of a message from a flag: the reference's
 *          flag inside every message (Rt64, Rt64_PCIE, and on request Rt64_128 /
 *          Rt64_128_PCIE byte for byte), or one flag word per message beside full
 *          payload lines, every access at agent scope (what the Rt64_128 families of
 *          the all-to-all flows take when left alone; see "wire_fenced").  This is
 *          the form that carries over to several GPUs.  Default for
 *          VR_ALGO_PARALLEL. */
typedef enum vr_transport {
  VR_TRANSPORT_DEFAULT = 0,
  VR_TRANSPORT_DIRECT = 1,
  VR_TRANSPORT_WIRE = 2,
} vr_transport;

/* Element types the reference instantiates (allreduce.cpp:1215-1294: sycl::half and
 * sycl::ext::oneapi::bfloat16; main.cpp:45 runs bfloat16).  Both are 2 bytes, so
 * sizes, alignment rules and data movement are identical; only the add differs:
 * binary16 adds natively, bfloat16 adds as binary32 and rounds the sum to nearest
 * even.  A context starts as VR_DTYPE_F16. */
typedef enum vr_dtype {
  VR_DTYPE_F16 = 0,
  VR_DTYPE_BF16 = 1,
} vr_dtype;

typedef struct vr_ctx vr_ctx;

/* ---- lifetime --------------------------------------------------------------- */

/* Creates a context for `nranks` virtual ranks on HIP device `device`.  nranks
 * must be 2, 4, 8 or 16.  The direct transport needs no scratch. */
int vr_ctx_create(int device, int nranks, vr_ctx **out);
int vr_ctx_destroy(vr_ctx *ctx);
/* Allocates and zeroes, once, the wire transport's scratch: one device allocation
 * holding a scatter and a gather sink per rank (ipcbuf0 | ipcbuf1 and the peer
 * tables of main.cpp:241-283).  This is the only place the wire transport
 * allocates or synchronises: a wire-transport launch on a context whose scratch
 * is not reserved returns VR_ERR_INVALID.  Idempotent. */
int vr_ctx_reserve_wire(vr_ctx *ctx);
int vr_ctx_nranks(const vr_ctx *ctx);
int vr_ctx_set_dtype(vr_ctx *ctx, int dtype);   /* element type of the following collectives */
int vr_ctx_get_dtype(const vr_ctx *ctx);

/* ---- validation (host only, no GPU needed) ------------------------------------ */

int vr_algo_from_string(const char *name, int *algo_out);        /* VR_ERR_ALGO if unknown */
const char *vr_algo_name(int algo);
int vr_algo_is_allgather(int algo);
size_t vr_algo_message_bytes(int algo);                          /* sizeof(message_t): 8 or 16 */

/* calcWorkSize: pointer alignment and even divisibility for an all-reduce of
 * `nelems` halves per rank.  *work_bytes (optional) = bytes per rank-chunk. */
int vr_check_allreduce(int algo, int nranks, const void *const bufs[], size_t nelems,
                       size_t *work_bytes);
int vr_check_allgather(int algo, int nranks, const void *const inputs[], void *const outputs[],
                       size_t nelems, size_t *work_bytes);

/* getLaunchParam: the grid the reference would pick for this size, and how far
 * it advances the sequence number. */
typedef struct vr_geometry {
  uint32_t groups;        /* work-groups                              */
  uint32_t subgroups;     /* sub-groups (16 lanes) per work-group     */
  uint32_t steps;         /* loop steps each wire makes = seqNo bump  */
} vr_geometry;
int vr_launch_geometry(int algo, int nranks, size_t nelems, vr_geometry *out);

/* ---- the hot path ------------------------------------------------------------ */

/* All-reduce of `nelems` binary16 values per rank across ctx's virtual ranks.
 *   bufs[r]  : rank r's input (device memory, message-aligned).
 *   outs     : NULL for the reference's in-place semantics (bufs[r] receives the
 *              sum), or N output pointers (outs[r] may equal bufs[r]).
 *   seq_no   : in/out sequence number, advanced like getLaunchParam does; only the
 *              wire transport consumes it.  May be NULL (context keeps its own).
 * Asynchronous on `stream` (a hipStream_t; NULL = the null stream).  The sum is
 * bit-identical to the reference kernels' order for `algo`: rotated chain from
 * the chunk owner (all but bisect), pair tree (bisect). */
int vr_allreduce(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                 void *const outs[], size_t nelems, uint32_t *seq_no);

/* All-gather: outputs[r][p*nelems + i] = inputs[p][i] for every rank r.
 * outputs[r] + r*nelems may alias inputs[r] (sequential_transmit.hpp:496-497). */
int vr_allgather(vr_ctx *ctx, void *stream, int algo, int transport, const void *const inputs[],
                 void *const outputs[], size_t nelems, uint32_t *seq_no);

/* One rank of a wire-transport all-reduce against caller-owned scratch: the form
 * the reference constructs in every process.  The launch holds `rank`'s wires
 * only; the other ranks' launches (other streams of this process, or other
 * processes that mapped the same sinks) must run at the same time, since every
 * wave waits, with a bounded spin, for its peers' messages.
 *   input / output : this rank's buffer (output NULL = in place).
 *   scatter_buf, gather_buf : this rank's own sinks; peer_buf0[q] / peer_buf1[q]
 *              the scatter / gather sink of rank q (entry `rank` is ignored).
 *              Each sink holds `sink_bytes` >= vr_rank_scratch_bytes() bytes, is
 *              16-byte aligned, and was zeroed once before the first launch.
 *   seq_no   : in/out; must be the same on every rank and only ever grow; a
 *              change of algo needs freshly zeroed sinks.
 * Same validation and error codes as vr_allreduce for this rank's pointers
 * (calcWorkSize: alignment to the protocol's message_t, 8 or 16 bytes) and
 * nothing stricter: where a format carries 16 bytes per lane, a rank whose
 * buffers are only 8-byte aligned moves them as two 8-byte accesses.
 * The library neither allocates nor clears anything here.  vr_ctx_check(ctx,
 * stream) reports a time-out of this context's launches; after one, the caller
 * zeroes its sinks again.
 * Concurrency inside one process: every launch of a collective needs a stream of
 * its own and a hardware queue of its own.  A process has GPU_MAX_HW_QUEUES of
 * them (4 unless the environment says otherwise), so at most that many one-rank
 * launches can form a collective in one process; a launch that would exceed it,
 * or that shares a stream with another rank of the same collective (same sinks,
 * same seq_no), is refused with VR_ERR_INVALID before anything is enqueued.
 * Hold several ranks per launch (vr_allreduce_ranks) or run the ranks in
 * separate processes instead. */
int vr_allreduce_rank(vr_ctx *ctx, void *stream, int algo, int rank, void *input, void *output,
                      void *scatter_buf, void *gather_buf, void *const peer_buf0[],
                      void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no);
/* The same with the test harness's user grid (testTransmit<T>(algo, nd_range, input,
 * ipcbuf0, ipcbuf1, peerbuf0, peerbuf1, nelems, rank, world, step, simd, queue),
 * allreduce.hpp:337-343, main.cpp:67-71): `groups` x `subgroups` sub-groups per
 * rank; every rank must pass the same grid.  Rejections as vr_allreduce_grid. */
int vr_allreduce_rank_grid(vr_ctx *ctx, void *stream, int algo, int rank, void *input, void *output,
                           void *scatter_buf, void *gather_buf, void *const peer_buf0[],
                           void *const peer_buf1[], size_t sink_bytes, size_t nelems,
                           uint32_t seq_no, uint32_t groups, uint32_t subgroups, uint32_t simd);
/* One rank of the ring all-gather, same contract (AllGather(input, output, nelems,
 * rank, seqNo, scatterBuf, gatherBuf, peerBuf0, peerBuf1), allgather.hpp:19-29):
 * output holds nranks * nelems elements; output + rank * nelems may be input. */
int vr_allgather_rank(vr_ctx *ctx, void *stream, int algo, int rank, const void *input, void *output,
                      void *scatter_buf, void *gather_buf, void *const peer_buf0[],
                      void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no);
/* The same with the test harness's user grid: testAllgather<T>(algo, nd_range, input,
 * output, ipcbuf0, ipcbuf1, peerbuf0, peerbuf1, nelems, rank, world, step, subgroup,
 * queue) (allreduce.cpp:1191-1213; benchAllgather, main.cpp:110-166).  Rejections as
 * vr_allreduce_grid. */
int vr_allgather_rank_grid(vr_ctx *ctx, void *stream, int algo, int rank, const void *input,
                           void *output, void *scatter_buf, void *gather_buf, void *const peer_buf0[],
                           void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t seq_no,
                           uint32_t groups, uint32_t subgroups, uint32_t simd);
/* Ranks [first_rank, first_rank + nranks_here) of a collective in ONE launch: what a
 * process that owns k of the N ranks enqueues (the reference's processes own one
 * each, allreduce.hpp:18-28).  inputs[i] / outputs[i] belong to rank first_rank + i
 * (outputs NULL, or an entry NULL = in place); peer_buf0[] / peer_buf1[] hold every
 * rank's scatter / gather sink, the launch's own ranks included.  Otherwise the
 * contract of vr_allreduce_rank / vr_allgather_rank.  N ranks on a process's 4
 * hardware queues: N / 4 ranks per launch on 4 streams. */
int vr_allreduce_ranks(vr_ctx *ctx, void *stream, int algo, int first_rank, int nranks_here,
                       void *const inputs[], void *const outputs[], void *const peer_buf0[],
                       void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no);
int vr_allgather_ranks(vr_ctx *ctx, void *stream, int algo, int first_rank, int nranks_here,
                       const void *const inputs[], void *const outputs[], void *const peer_buf0[],
                       void *const peer_buf1[], size_t sink_bytes, size_t nelems, uint32_t *seq_no);
/* Consecutive flag values one rank-group launch of this shape consumes (groups = 0:
 * the library's own grid).  Sequence numbers of successive launches on the same
 * sinks must lie at least this far apart; main.cpp's fixed offsets (flag, +100,
 * +150, +200; l.67-106) allow 50. */
int vr_rank_flags_used(vr_ctx *ctx, int algo, size_t nelems, uint32_t groups, uint32_t subgroups,
                       uint32_t *flags_used);
/* Bytes a scatter sink (and equally a gather sink) must hold for this context's
 * rank count, device and "wire_blocks_per_cu" setting. */
int vr_rank_scratch_bytes(const vr_ctx *ctx, size_t *sink_bytes);

/* ---- ranks in separate processes ------------------------------------------------ */

/* open_all_ipc_mems: every one of `world` processes (one rank each, all on the
 * same GPU or on GPUs with peer access) calls this with a pointer into a device
 * allocation of its own (under 2 GiB).  The processes exchange IPC handles over
 * AF_UNIX sockets named after `instance` and the rank (in $TMPDIR, else /tmp) and
 * map each other's allocation: on return rank i's memory is at
 * (char *)peer_bases[i] + offsets[i]; entry `rank` is `ptr` itself with offset 0.
 * A peer that does not show up within 30 s (environment VRANK_IPC_TIMEOUT_MS
 * overrides) ends the call with VR_ERR_TIMEOUT. */
int vr_ipc_open_all(void *ptr, int rank, int world, void *peer_bases[], size_t offsets[],
                    const char *instance);
/* Unmaps what vr_ipc_open_all mapped (not the own entry). */
int vr_ipc_close_all(int rank, int world, void *const peer_bases[]);
/* Returns once all `world` processes of `instance` have called it with the same
 * `generation` (a different number for every barrier of a run). */
int vr_ipc_barrier(int rank, int world, const char *instance, int generation);

/* No counterpart in the reference.  For callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  A wire-transport vr_allreduce whose sinks live in a fixed
 * region of device memory that is part of the library's code object (about
 * 32 MiB per GPU, held until the process ends) instead of scratch reserved by the
 * context.  Calls no hipMalloc / hipFree and does not synchronise.
 * Limits: at most 8 ranks, at most 256 MiB (134217728 elements) per rank, every
 * all-reduce algo except simple_transmit; 32 to 128 wires per rank.  Beyond them:
 * VR_ERR_INVALID.  Every context on a GPU shares that GPU's region and each call
 * first clears the message slots it is about to use (a fill kernel on `stream`),
 * so calls that overlap in time on one GPU race: keep them on one stream or
 * otherwise ordered.  A time-out is recorded in the calling context's own status
 * word and reported by vr_ctx_check like those of vr_allreduce. */
int vr_allreduce_static(vr_ctx *ctx, void *stream, int algo, void *const bufs[], void *const outs[],
                        size_t nelems);

/* Reference test-harness flavour (testTransmit with a user grid, main.cpp:289-314):
 * `groups` x `subgroups` sub-groups of `simd` lanes.  Results never depend on the
 * grid; unusable grids are rejected the way the reference's host code rejects
 * them (VR_ERR_GEOMETRY / VR_ERR_SUBGROUP). */
int vr_allreduce_grid(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                      void *const outs[], size_t nelems, uint32_t seq_no, uint32_t groups,
                      uint32_t subgroups, uint32_t simd);

/* testAllgather with a user grid for all ranks at once (allreduce.cpp:1191-1213,
 * main.cpp:110-166, 293-307): `groups` x `subgroups` sub-groups of `simd` lanes per
 * rank; same rejections as vr_allreduce_grid. */
int vr_allgather_grid(vr_ctx *ctx, void *stream, int algo, int transport, const void *const inputs[],
                      void *const outputs[], size_t nelems, uint32_t seq_no, uint32_t groups,
                      uint32_t subgroups, uint32_t simd);

/* After a wire-transport launch has completed: VR_OK, or VR_ERR_TIMEOUT if any
 * poll gave up.  (Synchronises `stream`.)  After a time-out the context's own
 * scratch has been zeroed again; sinks a caller handed to the rank-group launches
 * are the caller's to zero. */
int vr_ctx_check(vr_ctx *ctx, void *stream);
/* Poll budget of the wire transport's bounded spin (0 = library default). */
int vr_ctx_set_spin_limit(vr_ctx *ctx, uint64_t polls);

/* Tuning knobs for the direct kernels (benchmark sweeps).  Unknown keys are
 * VR_ERR_INVALID.  Keys: "block" (threads per work-group), "waves_per_cu"
 * (persistent grid size = CUs * this / waves per block), "unroll" (16-byte
 * vectors in flight per lane and rank), "nt_load" (0 cached, 1 streaming loads),
 * "nt_store" (0 cached, 1 streaming stores, 2 streaming stores written through
 * at agent scope), "oneshot" (1 = one-trip grid: one tile per work-group, no
 * grid-stride loop; the hardware starts work-groups in index order, so the launch
 * sweeps the buffers front to back), "wgs_per_cu" (0..12: at most this many
 * work-groups of a one-trip grid share a compute unit, 0 = as many as fit),
 * "deal" (chunks the work-groups of an all-reduce work on at a time: a divisor
 * of the rank count, 0 = all of them, i.e. work-group b serves owner b % N
 * throughout; 1 = all compute units sweep one chunk after the other),
 * "run" (all-gather, one-trip grid, one source at a time: every XCD takes runs of
 * this many consecutive tiles, a power of two up to 256, instead of every eighth
 * tile; 0 = no permutation),
 * "f16_wide" (1 = binary16 adds computed through
 * binary32 and rounded back after every add: the same bits, a longer ALU section),
 * "segment_kib" (KiB of a chunk one launch
 * covers; chunks longer than this, at most 1 GiB, take several launches);
 * for the wire transport "wire_fenced" (how the Rt64_128 families, i.e. simple,
 * bisect, parallel, simple_pcie_p, simple_ring, simple_pcie, simple_transmit,
 * tell a receiver that a message is there: 0 = the reference's 128 / 256-byte
 * messages with a flag in every 64 bytes; 1 = full payload lines and a separate
 * flag word, ordered by agent-scope release / acquire fences; 2 = self-validating
 * 8-byte messages; 3 = as 1 with the payload stored written through; 4 = flag
 * words with every payload and flag access at agent scope (stores written
 * through, loads never served from a stale line), the flag stored once the
 * payload stores have completed: no cache maintenance.  Left alone (-1): 4 for
 * the all-to-all flows ParallelTransmit / BisectPTransmit / SimpleTransmit, 0 for
 * the ring and sequential flows) and
 * "wire_cooperative" (1 = cooperative launch; by default a plain launch: the
 * library sizes every grid within the occupancy query's bound, so it is
 * co-resident on an otherwise idle device),
 * "wire_stream_io" (1 = inputs loaded and outputs stored with streaming cache
 * policies, 0 = cached; by default streaming from 256 MiB of inputs + outputs on),
 * "wire_ahead" (1..6 steps the parallel flow's scatters run ahead of its gathers),
 * "wire_msg16" (0 = the Rt64_PCIE family sends self-validating 8-byte messages
 * instead of 16-byte stores that carry the flag twice) and
 * "wire_blocks_per_cu" (1..4 resident work-groups per CU; set it before
 * vr_ctx_reserve_wire, it sizes the scratch).
 * -1 restores the library's own choice. */
/* The launch the direct transport gives a collective of this shape when nothing
 * is overridden: pure host arithmetic, no device needed (nelems per rank; in_place
 * is ignored for an all-gather).  No counterpart in the reference, whose launch
 * shape is the user's -g / -w / -s (main.cpp:181-198). */
typedef struct vr_launch_plan {
  int one_trip;      /* 1: one tile per work-group, started in index order; 0: persistent grid-stride grid */
  int block;         /* threads per work-group */
  int unroll;        /* vectors in flight per lane and rank */
  int waves_per_cu;  /* persistent grid: waves per compute unit; 0 for a one-trip grid */
  int wgs_per_cu;    /* one-trip grid: residency cap in work-groups per compute unit, 0 = none */
  int deal;          /* chunks (all-gather: sources) worked on at a time */
  int run;           /* all-gather: consecutive tiles per XCD (1 = every eighth tile) */
  int nt_load;       /* 0 cached, 1 streaming loads */
  int nt_store;      /* 0 cached, 1 streaming, 2 streaming and written through at agent scope */
  int f16_wide;      /* 1: binary16 adds computed through binary32 (same bits) */
} vr_launch_plan;
int vr_direct_launch_plan(int algo, int nranks, size_t nelems, int in_place, vr_launch_plan *out);

int vr_ctx_set_tuning(vr_ctx *ctx, const char *key, int value);
int vr_ctx_get_tuning(vr_ctx *ctx, const char *key, int *value);

/* ---- timing ------------------------------------------------------------------- */

/* Launches the all-reduce `iters` times on `stream`, each bracketed by its own
 * pair of HIP events recorded on that stream, and returns the per-launch kernel
 * times in milliseconds (ms_out[iters]).  Out-of-place when outs != NULL. */
int vr_time_allreduce(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                      void *const outs[], size_t nelems, int iters, float *ms_out);
/* Per-launch kernel EXECUTION times in milliseconds, from events attached to the
 * kernel dispatches themselves (their own begin / end timestamps, what a kernel
 * trace shows and what the reference prints from its SYCL event, main.cpp:36-43);
 * no host or event-command overhead is included.  A collective that takes several
 * kernels (chunks above 1 GiB) is timed from the first one's begin to the last
 * one's end. */
int vr_time_allreduce_kernel(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                             void *const outs[], size_t nelems, int iters, float *ms_out);
int vr_time_allgather_kernel(vr_ctx *ctx, void *stream, int algo, int transport,
                             const void *const inputs[], void *const outputs[], size_t nelems,
                             int iters, float *ms_out);
/* `groups` event pairs, each around `per_group` back-to-back vr_allreduce calls made
 * exactly as a caller makes them.  ms_out[g] = device time of group g / per_group;
 * *host_call_us (optional) = host wall time one vr_allreduce call takes to return
 * (validation, launch heuristics, kernel enqueue), averaged over all calls. */
int vr_time_allreduce_grouped(vr_ctx *ctx, void *stream, int algo, int transport, void *const bufs[],
                              void *const outs[], size_t nelems, int groups, int per_group,
                              float *ms_out, double *host_call_us);
int vr_time_allgather(vr_ctx *ctx, void *stream, int algo, int transport,
                      const void *const inputs[], void *const outputs[], size_t nelems, int iters,
                      float *ms_out);
/* Plain device copy of `bytes` (dwordx4 loads, nontemporal stores) timed the
 * same way: the practical HBM ceiling next to which the all-reduce is read. */
int vr_time_copy(vr_ctx *ctx, void *stream, void *dst, const void *src, size_t bytes, int iters,
                 float *ms_out);
/* One asynchronous launch of a plain streaming kernel over `bytes` (16-byte
 * granules): the yardsticks an all-reduce figure is read against.
 *   VR_PROBE_COPY  dst[i] = src[i]         (bytes read + bytes written)
 *   VR_PROBE_READ  reads src, writes nothing
 *   VR_PROBE_WRITE writes dst, reads nothing */
enum { VR_PROBE_COPY = 0, VR_PROBE_READ = 1, VR_PROBE_WRITE = 2 };
int vr_stream_probe(vr_ctx *ctx, void *stream, int mode, void *dst, const void *src, size_t bytes);

/* The all-reduce's own access shape as a yardstick: one launch of the direct
 * all-reduce kernel with the adds removed, so that dsts[k] receives srcs[k]
 * (`bytes_each` bytes, a multiple of 16 * nranks) for each of the context's
 * nranks streams: the same grid, chunk walk, buffer addressing and cache policies
 * as an out-of-place vr_allreduce of that size, N read streams and N write
 * streams.  What this shape of traffic can reach without any arithmetic. */
int vr_stream_probe_multi(vr_ctx *ctx, void *stream, void *const dsts[], const void *const srcs[],
                          size_t bytes_each);

/* Diagnostic: launches `blocks` work-groups and reports the XCD each one ran on
 * (ids_host[b]).  The direct kernels give work-group b to virtual rank b % N and
 * count on the hardware dealing consecutive work-groups to consecutive XCDs
 * (XCD (b + s) % 8, s = wherever the previous launch stopped), so that within a
 * launch of 8 ranks every XCD serves exactly one rank's chunk.  Synchronous. */
int vr_probe_xcc_ids(vr_ctx *ctx, uint32_t blocks, uint32_t *ids_host);

/* ---- host helpers -------------------------------------------------------------- */

void vr_fill_pattern(uint16_t *host_buf, int rank, size_t n);     /* utils.hpp:15-19 */
/* Seeded data: dist 0 = uniform [p0,p1), 1 = normal(mean p0, sd p1); splitmix64
 * keyed by seed, element i from draws 2i, 2i+1; rounded once to binary16. */
void vr_generate(uint16_t *host_buf, size_t n, uint64_t seed, int dist, double p0, double p1);
/* The same two for either element type. */
void vr_fill_pattern_dt(int dtype, uint16_t *host_buf, int rank, size_t n);
void vr_generate_dt(int dtype, uint16_t *host_buf, size_t n, uint64_t seed, int dist, double p0,
                    double p1);
/* "8MB" -> 8*1024*1024, "64K", "2G", plain digits (main.cpp:17-34). */
int vr_parse_nelems(const char *text, size_t *out);

/* Thin device-memory plumbing so that C, Python (ctypes) and the CLI need no
 * other GPU runtime binding. */
int vr_device_count(int *count);
int vr_device_name(int device, char *buf, size_t buflen);
int vr_malloc(int device, size_t bytes, void **out);
int vr_free(void *ptr);
int vr_memset(void *ptr, int value, size_t bytes);                 /* complete on return */
int vr_copy_to_device(void *dst, const void *src_host, size_t bytes);
int vr_copy_to_host(void *dst_host, const void *src, size_t bytes);
int vr_stream_create(int device, void **stream_out);
int vr_stream_destroy(void *stream);
int vr_stream_sync(void *stream);
/* HIP events recorded on `stream`, for callers that time their own launch sequences. */
int vr_event_create(void **event_out);
int vr_event_record(void *event, void *stream);
int vr_event_elapsed_ms(void *start, void *stop, float *ms_out);   /* waits for `stop` */
int vr_event_destroy(void *event);

/* ---- errors ---------------------------------------------------------------------- */

const char *vr_strerror(int status);          /* the reference's exception text where one exists */
const char *vr_last_error_detail(void);       /* thread-local detail of the last non-zero status */
const char *vr_version(void);

#ifdef __cplusplus
}
#endif
#endif /* VRANK_ALLREDUCE_H */
