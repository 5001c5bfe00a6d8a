"""GPU parity tests of the wire transport (message passing through scratch with
flags, one persistent kernel holding every virtual rank's work-groups).  Same
oracle, same bit-exact bar as the direct transport."""
import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from tests import vr_helpers as H
from tests.oracle_lib import DIST_NORMAL, DIST_UNIFORM

pytestmark = pytest.mark.gpu
WIRE = vr.TRANSPORT_WIRE


@pytest.fixture(scope="module")
def ctxs():
    made = {n: vr.VirtualRanks(n) for n in (2, 4, 8, 16)}
    yield made
    for c in made.values():
        c.close()


def h(x):
    return int(np.array([x], np.float16).view(np.uint16)[0])


def per_chunk(out, nranks):
    chunk = len(out) // nranks
    return [float(out[c * chunk:(c + 1) * chunk].view(np.float16)[0]) for c in range(nranks)]


@pytest.mark.parametrize("algo", ["small", "simple", "parallel", "bisect", "small_ring", "simple_ring",
                                  "small_pcie", "simple_pcie", "simple_transmit"])
def test_kat_n8(ctxs, algo):
    ins = [np.full(1024, h(v), np.uint16) for v in (2048, 0, 1, 0, 1, 0, 0, 0)]
    got, _ = H.run_allreduce(ctxs[8], algo, ins, transport=WIRE)
    want = ([2048, 2050, 2048, 2048, 2048, 2050, 2048, 2048] if algo == "bisect"
            else [2048, 2050, 2050, 2048, 2048, 2048, 2048, 2048])
    for g in got:
        assert per_chunk(g, 8) == want
        assert (g.reshape(8, -1) == g.reshape(8, -1)[:, :1]).all()


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("algo", H.ROTATED_ALGOS + ("parallel", "bisect"))
def test_random_all_algos(ctxs, oracle, nranks, algo):
    if algo == "bisect" and nranks < 4:
        pytest.skip("bisect needs >= 4 ranks")
    msg = 16 if ("pcie" in algo or "ring" in algo) else 8
    unit = (msg // 2) * nranks
    for k, n in enumerate((unit, unit * 3, unit * 129, unit * 1000 + unit, 1 << 20)):
        n = (n // unit) * unit
        ins = H.make_inputs(oracle, nranks, n, 3000 * nranks + 10 * k)
        want = H.expected(oracle, algo, ins)
        got, _ = H.run_allreduce(ctxs[nranks], algo, ins, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, want, "%s N=%d n=%d in-place" % (algo, nranks, n))
        got, kept = H.run_allreduce(ctxs[nranks], algo, ins, inplace=False, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, want, "%s N=%d n=%d out-of-place" % (algo, nranks, n))
        for a, b in zip(kept, ins):
            assert (a == b).all()


def test_bisect_16_ranks(ctxs, oracle):
    for n in (64, 64 * 77, 1 << 18):
        ins = H.make_inputs(oracle, 16, n, 78)
        got, _ = H.run_allreduce(ctxs[16], "bisect", ins, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, oracle.bisect(ins))


@pytest.mark.parametrize("algo", ["simple", "bisect", "small"])
def test_eight_byte_granularity(ctxs, oracle, algo):
    for n in (32 * 1, 32 * 3, 32 * 1001):
        ins = H.make_inputs(oracle, 8, n, 41 + n)
        got, _ = H.run_allreduce(ctxs[8], algo, ins, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), "n=%d" % n)
    ins = H.make_inputs(oracle, 8, 1 << 16, 9)
    got, _ = H.run_allreduce(ctxs[8], algo, ins, offset_bytes=8, transport=WIRE)
    H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), "offset 8")


@pytest.mark.parametrize("groups", [1, 2, 4, 8, 16, 32, 64, 7, 13, 15, 17, 19])
def test_result_independent_of_grid(ctxs, oracle, groups):
    n = 14336
    ins = H.make_inputs(oracle, 8, n, 501)
    for algo in ("small", "simple", "bisect", "simple_ring"):
        want = H.expected(oracle, algo, ins)
        for subgroups in (4, 8, 32, 64):
            got, _ = H.run_allreduce(ctxs[8], algo, ins, grid=(groups, subgroups, 16), transport=WIRE)
            H.assert_all_ranks_equal(oracle, got, want, "%s g=%d w=%d" % (algo, groups, subgroups))


def test_many_launches_reuse_slots_and_flags(ctxs, oracle):
    """Back-to-back launches without host synchronisation: slot rings wrap, the
    sequence number keeps the flags apart."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    ctx = ctxs[8]
    n = 8 * 4096 * 6            # several steps per launch at the automatic grid
    for algo in ("small", "simple", "bisect", "small_ring", "simple_pcie", "simple_transmit"):
        base = H.make_inputs(oracle, 8, n, 900)
        cur = [a.copy() for a in base]
        bufs = [DeviceBuffer(n * 2) for _ in range(8)]
        for b, a in zip(bufs, cur):
            b.upload(a)
        rounds = 5
        for _ in range(rounds):
            ctx.allreduce(algo, [b.ptr for b in bufs], n, transport=WIRE)     # in place, async
        ctx.check()
        for _ in range(rounds):
            s = H.expected(oracle, algo, cur)
            cur = [s.copy() for _ in range(8)]
        for b in bufs:
            assert oracle.count_mismatch(b.download(np.uint16, n), cur[0]) == 0, algo
            b.free()


def test_sequence_number_moving_backwards_is_safe(ctxs, oracle):
    ctx = ctxs[8]
    ins = H.make_inputs(oracle, 8, 8 * 4096, 77)
    want = oracle.rotated(ins)
    for seq in (0xE00F100F, 0xE00F100F, 5, 5, 1):          # repeats and regressions
        got, _ = H.run_allreduce(ctx, "simple", ins, grid=(16, 8, 16), transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, want)
        src = H.RankBuffers(8, len(ins[0]))
        src.upload(ins)
        ctx.allreduce_grid("simple", src.ptrs, len(ins[0]), 16, 8, 16, transport=WIRE, seq_no=seq)
        ctx.check()
        H.assert_all_ranks_equal(oracle, src.download(), want, "seq %#x" % seq)
        src.free()
    with pytest.raises(vr.VRError) as e:
        src = H.RankBuffers(8, len(ins[0]))
        ctx.allreduce_grid("simple", src.ptrs, len(ins[0]), 16, 8, 16, transport=WIRE, seq_no=0)
    assert e.value.code == "INVALID"


def test_sequence_number_wrap_never_uses_flag_zero(ctxs, oracle):
    """A 32-bit counter that would run through 0 restarts from 1 on clean scratch."""
    import ctypes as C
    ctx = ctxs[8]
    n = 8 * 4096 * 8
    ins = H.make_inputs(oracle, 8, n, 88)
    want = oracle.rotated(ins)
    ctx.seq_no = C.c_uint32(0xFFFFFFFF)
    for _ in range(3):
        got, _ = H.run_allreduce(ctx, "simple", ins, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, want)
        assert ctx.seq_no.value != 0
    assert ctx.seq_no.value < 1000
    src = H.RankBuffers(8, n)
    src.upload(ins)
    ctx.allreduce_grid("small", src.ptrs, n, 8, 8, 16, transport=WIRE, seq_no=0xFFFFFFFF)
    ctx.check()
    H.assert_all_ranks_equal(oracle, src.download(), want)
    src.free()


def test_poll_timeout_is_reported_and_recoverable(ctxs, oracle):
    """A spin limit of one poll makes some wave give up before its message has
    arrived; every wave still runs to completion, the context reports the
    time-out, and the next launch works."""
    ctx = vr.VirtualRanks(8)
    ins = H.make_inputs(oracle, 8, 1 << 20, 31)
    ctx.set_spin_limit(1)
    timed_out = False
    for algo in ("simple_ring", "small_ring", "bisect"):
        try:
            H.run_allreduce(ctx, algo, ins, transport=WIRE)
        except vr.VRError as e:
            assert e.code == "TIMEOUT"
            timed_out = True
    assert timed_out
    ctx.set_spin_limit(0)
    got, _ = H.run_allreduce(ctx, "simple_ring", ins, transport=WIRE)
    H.assert_all_ranks_equal(oracle, got, oracle.rotated(ins))
    ctx.close()


@pytest.mark.parametrize("fenced", [-1, 0])
def test_config3_bisect_32mib_wire(ctxs, oracle, fenced):
    """The headline shape through scratch: flag words (the library's choice) and the
    reference's 128-byte messages."""
    ins = H.make_inputs(oracle, 8, 16777216, 3000, DIST_NORMAL, 0.0, 0.02)
    ctxs[8].set_tuning(wire_fenced=fenced)
    try:
        got, _ = H.run_allreduce(ctxs[8], "bisect", ins, transport=WIRE)
    finally:
        ctxs[8].set_tuning(wire_fenced=-1)
    H.assert_all_ranks_equal(oracle, got, oracle.bisect(ins))


def test_parallel_defaults_to_wire_and_sweep_sizes(ctxs, oracle):
    for p in range(11, 24, 2):
        n = 1 << p
        ins = H.make_inputs(oracle, 8, n, 5100 + p)
        got, _ = H.run_allreduce(ctxs[8], "parallel", ins)          # default transport
        H.assert_all_ranks_equal(oracle, got, oracle.rotated(ins), "n=%d" % n)


@pytest.mark.parametrize("log2_elems,fenced", [(24, -1), (25, -1), (26, -1), (27, -1), (24, 0), (27, 0)])
def test_config5_parallel_large_sizes(ctxs, oracle, log2_elems, fenced):
    """The sweep's named protocol on its default (wire) transport at 32, 64, 128 and
    256 MiB per rank: N(0,1) inputs, rank 0 compared in full with the rotated-order
    oracle, the other ranks by equality with rank 0.  With the library's own choice of
    format (flag words) and with the reference's 256-byte messages (fenced 0)."""
    n = 1 << log2_elems
    ins = H.make_inputs(oracle, 8, n, 5000 + log2_elems)
    want = oracle.rotated(ins)
    ctxs[8].set_tuning(wire_fenced=fenced)
    try:
        got, _ = H.run_allreduce(ctxs[8], "parallel", ins)          # default transport = wire
    finally:
        ctxs[8].set_tuning(wire_fenced=-1)
    assert oracle.count_mismatch(got[0], want) == 0, n
    for r in range(1, 8):
        assert oracle.count_mismatch(got[r], got[0]) == 0, (n, r)
    assert oracle.count_mismatch(want, oracle.rank_order(ins)) > 1000   # the order matters on this data


def run_allgather_wire(ctx, algo, ins, alias_own_slot=False):
    from gpu_ipc_example_amd.binding import DeviceBuffer
    N, n = ctx.nranks, len(ins[0])
    outs = [DeviceBuffer(N * n * 2 + 64) for _ in range(N)]
    for o in outs:
        o.fill(0x01)
    if alias_own_slot:
        in_ptrs = [outs[r].ptr + r * n * 2 for r in range(N)]
        for r in range(N):
            outs[r].upload(ins[r], r * n * 2)
        srcs = []
    else:
        srcs = [DeviceBuffer(n * 2 + 64) for _ in range(N)]
        for s, a in zip(srcs, ins):
            s.upload(a)
        in_ptrs = [s.ptr for s in srcs]
    ctx.allgather(algo, in_ptrs, [o.ptr for o in outs], n, transport=WIRE)
    ctx.check()
    got = [o.download(np.uint16, N * n) for o in outs]
    for b in outs + srcs:
        b.free()
    return got


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_allgather_wire(ctxs, oracle, nranks, algo):
    for n in (8, 8 * 15, 8 * 1237, 1 << 16, 1 << 20):
        ins = H.make_inputs(oracle, nranks, n, 71 + n, DIST_UNIFORM, -2.0, 2.0)
        want = oracle.allgather(ins)
        for alias in (False, True):
            got = run_allgather_wire(ctxs[nranks], algo, ins, alias)
            for r in range(nranks):
                assert (got[r] == want).all(), (n, r, alias)


@pytest.mark.parametrize("fenced", [0, 1, 3, 4])
@pytest.mark.parametrize("algo", ["simple", "parallel", "bisect", "simple_ring", "simple_pcie",
                                  "simple_pcie_p", "simple_transmit"])
def test_fenced_flag_word_format(oracle, algo, fenced):
    """The Rt64_128 family travels as the reference's messages with a flag in every
    64 bytes (0), or as payload lines + a separate flag word: ordered by agent-scope
    release/acquire fences (1; 3 = payload written through), or by store completion
    with every access at agent scope (4, what the all-to-all flows take when left
    alone).  No assumption about store atomicity in 1, 3 and 4."""
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_fenced=fenced)
    for n in (64, 64 * 129, 1 << 18, 32 * 1001):
        if algo in ("simple_ring", "simple_pcie", "simple_pcie_p") and n % 64:
            continue
        ins = H.make_inputs(oracle, 8, n, 6000 + n)
        for inplace in (True, False):
            got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE, inplace=inplace)
            H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), "%s n=%d" % (algo, n))
    ctx.close()


@pytest.mark.parametrize("fenced", [1, 4])
@pytest.mark.parametrize("algo", ["parallel", "bisect", "simple_pcie"])
def test_flag_word_formats_under_repetition(oracle, algo, fenced):
    """60 launches over the same sinks: slots and flag words are reused with growing
    flag values, and every tenth result is compared with the oracle."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_fenced=fenced)
    n = 64 * 1025
    ins = H.make_inputs(oracle, 8, n, 6900)
    want = H.expected(oracle, algo, ins)
    src = [DeviceBuffer(n * 2) for _ in range(8)]
    dst = [DeviceBuffer(n * 2) for _ in range(8)]
    for b, a in zip(src, ins):
        b.upload(a)
    for it in range(60):
        ctx.allreduce(algo, [b.ptr for b in src], n, outs=[b.ptr for b in dst], transport=WIRE)
        if it % 10 == 9:
            ctx.check()
            for r, b in enumerate(dst):
                assert oracle.count_mismatch(b.download(np.uint16, n), want) == 0, (algo, fenced, it, r)
    for b in src + dst:
        b.free()
    ctx.close()


@pytest.mark.parametrize("algo", ["simple", "parallel", "bisect", "simple_ring", "simple_pcie"])
def test_eight_byte_messages_for_the_128_byte_families(oracle, algo):
    """wire_fenced=2: the Rt64_128 families travel as self-validating 8-byte messages
    (payload dword + flag), which assume nothing beyond 8-byte store atomicity."""
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_fenced=2)
    for n in (64, 64 * 129, 1 << 19):
        ins = H.make_inputs(oracle, 8, n, 6500 + n)
        for inplace in (True, False):
            got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE, inplace=inplace)
            H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), "%s n=%d" % (algo, n))
    with pytest.raises(vr.VRError):
        ctx.set_tuning(wire_fenced=5)
    ctx.close()


@pytest.mark.parametrize("cooperative", [0, 1])
def test_plain_and_cooperative_launch(oracle, cooperative):
    """By default the launch is plain when the occupancy query proves the grid
    co-resident; both forms can be forced."""
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_cooperative=cooperative)
    for algo in ("small", "simple", "bisect", "small_ring"):
        ins = H.make_inputs(oracle, 8, 1 << 18, 6100)
        got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE)
        H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), algo)
    ctx.close()


def test_collective_calls_never_allocate_the_scratch(oracle):
    """The C ABI allocates the wire transport's scratch in vr_ctx_reserve_wire only:
    a wire launch on an unreserved context is an error, not a hidden hipMalloc."""
    import ctypes as C
    from gpu_ipc_example_amd import binding
    L = vr.lib()
    h = C.c_void_p()
    assert L.vr_ctx_create(0, 8, C.byref(h)) == 0
    n = 8 * 4096
    ins = H.make_inputs(oracle, 8, n, 6150)
    src = H.RankBuffers(8, n)
    src.upload(ins)
    seq = C.c_uint32(1)
    table = binding._table(src.ptrs)
    for algo, transport in (("parallel", vr.TRANSPORT_DEFAULT), ("simple", WIRE)):
        rc = L.vr_allreduce(h, None, vr.algo_id(algo), transport, table, None, n, C.byref(seq))
        assert rc == 7 and b"vr_ctx_reserve_wire" in L.vr_last_error_detail()
    assert L.vr_ctx_reserve_wire(h) == 0 and L.vr_ctx_reserve_wire(h) == 0
    assert L.vr_allreduce(h, None, vr.algo_id("parallel"), vr.TRANSPORT_DEFAULT, table, None, n,
                          C.byref(seq)) == 0
    assert L.vr_ctx_check(h, None) == 0
    H.assert_all_ranks_equal(oracle, src.download(), oracle.rotated(ins))
    src.free()
    L.vr_ctx_destroy(h)


@pytest.mark.parametrize("stream_io", [0, 1])
def test_streaming_and_cached_io(oracle, stream_io):
    """Inputs and outputs move with cached or with streaming accesses; ragged
    tails go through the same bounds-checked buffer accesses either way."""
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_stream_io=stream_io)
    for algo in ("small", "parallel", "bisect", "small_ring", "simple_pcie", "simple_transmit"):
        for n in (64 * 1, 64 * 1001, 1 << 19):
            for inplace in (True, False):
                ins = H.make_inputs(oracle, 8, n, 6160 + n)
                got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE, inplace=inplace)
                H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins),
                                         "%s n=%d io=%d" % (algo, n, stream_io))
    ctx.close()


@pytest.mark.parametrize("ahead", [1, 2, 6])
def test_parallel_flow_scatters_running_ahead(oracle, ahead):
    """The parallel flow's senders scatter up to `wire_ahead` steps before they wait
    for a gather; with few wires per rank (a small user grid) every column takes
    dozens of steps and wraps the 8-slot ring many times."""
    ctx = vr.VirtualRanks(8)
    ctx.set_tuning(wire_ahead=ahead)
    n = 8 * 4 * 30011
    ins = H.make_inputs(oracle, 8, n, 6200 + ahead)
    want = oracle.rotated(ins)
    for algo in ("small", "parallel"):
        for grid in (None, (1, 8, 16), (3, 8, 16)):
            for inplace in (True, False):
                got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE, grid=grid, inplace=inplace)
                H.assert_all_ranks_equal(oracle, got, want, "%s grid=%s inplace=%s" % (algo, grid, inplace))
    ctx.close()


def test_sixteen_byte_messages_can_be_swapped_for_eight_byte_ones(oracle):
    """The Rt64_PCIE family sends [d0, d1, flag, flag] in one 16-byte store; with
    wire_msg16=0 it falls back to self-validating 8-byte messages.  Same bits."""
    ctx = vr.VirtualRanks(8)
    n = 8 * 8 * 4099
    ins = H.make_inputs(oracle, 8, n, 6400)
    want = oracle.rotated(ins)
    for msg16 in (1, 0, -1):
        ctx.set_tuning(wire_msg16=msg16)
        for algo in ("small_pcie_p", "small_ring", "small_pcie"):
            for inplace in (True, False):
                got, _ = H.run_allreduce(ctx, algo, ins, transport=WIRE, inplace=inplace)
                H.assert_all_ranks_equal(oracle, got, want, "%s msg16=%d" % (algo, msg16))
    ctx.close()


def test_simple_transmit_ring_sections_wrap(ctxs, oracle):
    """Enough messages per sender to run through the 2 MiB ring sections several
    times in one launch (flag = seqNo + wraps), with small and large grids."""
    n = 8 * (6 << 20) // 2                        # 6 MiB per rank-chunk, 48 MiB per rank
    ins = H.make_inputs(oracle, 8, n, 6300)
    want = oracle.rotated(ins)
    for grid in (None, (2, 4, 16), (64, 64, 16)):
        got, _ = H.run_allreduce(ctxs[8], "simple_transmit", ins, transport=WIRE, grid=grid)
        assert oracle.count_mismatch(got[0], want) == 0, grid
        for r in range(1, 8):
            assert oracle.count_mismatch(got[r], got[0]) == 0, (grid, r)


@pytest.mark.parametrize("algo", ["simple", "bisect", "simple_ring", "small", "simple_transmit",
                                  "small_ring", "small_pcie"])
def test_embedded_flag_formats_under_repetition(ctxs, oracle, algo):
    """Many launches over the same sinks: every 64-byte segment (Rt64_128 family),
    every 8-byte message (Rt64) and every 16-byte message (Rt64_PCIE) must arrive
    whole every time."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    ctx = ctxs[8]
    ctx.set_tuning(wire_fenced=0)          # the reference's embedded-flag messages for every family
    n = 8 * 8192
    ins = H.make_inputs(oracle, 8, n, 6200)
    want = H.expected(oracle, algo, ins)
    src = [DeviceBuffer(n * 2) for _ in range(8)]
    dst = [DeviceBuffer(n * 2) for _ in range(8)]
    for b, a in zip(src, ins):
        b.upload(a)
    for it in range(150):
        ctx.allreduce(algo, [b.ptr for b in src], n, outs=[b.ptr for b in dst], transport=WIRE)
        if it % 10 == 9:
            ctx.check()
            for r, b in enumerate(dst):
                assert oracle.count_mismatch(b.download(np.uint16, n), want) == 0, (algo, it, r)
    ctx.set_tuning(wire_fenced=-1)
    for b in src + dst:
        b.free()
