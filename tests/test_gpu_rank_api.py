"""The per-rank form of the wire transport (vr_allreduce_rank): every rank is its
own launch against caller-owned sinks, the shape one process per GPU would run.
Here the N launches go to N streams of one process.  Results are compared bit
for bit with the oracle, and the bytes the launches leave in the sinks with the
oracle's message layouts (the reference's Rt64 / Rt64_PCIE / Rt64_128 /
Rt64_128_PCIE messages at sub-group size 16, byte for byte)."""
import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from gpu_ipc_example_amd.binding import DeviceBuffer, Stream
from tests import vr_helpers as H
from tests.oracle_lib import WIRE_RT64, WIRE_RT64_128, WIRE_RT64_PCIE, WIRE_RT64_128_PCIE

pytestmark = pytest.mark.gpu
SPIN = 1 << 19          # a rank whose peers never start gives up within a fraction of a second


# Concurrent kernels need distinct hardware queues, of which a process has four:
# the null stream plus three created ones, shared by every rank set of this file.
_POOL = []


def stream_pool():
    if not _POOL:
        _POOL.extend([None, Stream(), Stream(), Stream()])
    return _POOL


class Ranks:
    """N contexts (one per rank, as N processes would hold), N streams, N sink pairs."""

    def __init__(self, nranks):
        self.n = nranks
        self.ctx = [vr.VirtualRanks(nranks) for _ in range(nranks)]
        for c in self.ctx:
            c.set_spin_limit(SPIN)
        self.streams = stream_pool()[:nranks]
        self.sink_bytes = self.ctx[0].rank_scratch_bytes()
        self.scatter = [DeviceBuffer(self.sink_bytes) for _ in range(nranks)]
        self.gather = [DeviceBuffer(self.sink_bytes) for _ in range(nranks)]
        self.zero()

    def zero(self):
        for b in self.scatter + self.gather:
            b.fill(0)

    def handle(self, r):
        return self.streams[r].handle if self.streams[r] else None

    def allreduce(self, algo, ins, seq, inplace=True):
        n = len(ins[0])
        src = H.RankBuffers(self.n, n)
        src.upload(ins)
        dst = None
        if not inplace:
            dst = H.RankBuffers(self.n, n)
            dst.fill(0xAB)
        s0 = [b.ptr for b in self.scatter]
        s1 = [b.ptr for b in self.gather]
        nxt = None
        for r in range(self.n):
            nxt = self.ctx[r].allreduce_rank(algo, r, src.ptrs[r], s0[r], s1[r], s0, s1, self.sink_bytes, n,
                                             seq, out=dst.ptrs[r] if dst else None, stream=self.handle(r))
        for r in range(self.n):           # stops at the first time-out
            self.ctx[r].check(self.handle(r))
        got = (dst or src).download()
        src.free()
        if dst:
            dst.free()
        return got, nxt

    def close(self):
        for b in self.scatter + self.gather:
            b.free()
        for c in self.ctx:
            c.close()


@pytest.fixture(scope="module")
def ranks():
    made = {n: Ranks(n) for n in (2, 4)}
    yield made
    for r in made.values():
        r.close()


@pytest.mark.parametrize("nranks", [2, 4])
@pytest.mark.parametrize("algo", ["simple", "small", "parallel", "bisect", "simple_ring", "small_pcie",
                                  "simple_pcie_p", "simple_transmit"])
def test_rank_launches_match_the_oracle(ranks, oracle, nranks, algo):
    if algo == "bisect" and nranks < 4:
        pytest.skip("bisect needs >= 4 ranks")
    R = ranks[nranks]
    R.zero()                                   # a change of algo needs freshly zeroed sinks
    seq = 1
    for k, n in enumerate((64 * nranks, 64 * nranks * 33, 1 << 20)):
        ins = H.make_inputs(oracle, nranks, n, 8100 + 10 * k + nranks)
        want = H.expected(oracle, algo, ins)
        for inplace in (True, False):
            got, seq2 = R.allreduce(algo, ins, seq, inplace=inplace)
            assert seq2 > seq                  # the sequence number only grows
            seq = seq2
            H.assert_all_ranks_equal(oracle, got, want, "%s N=%d n=%d" % (algo, nranks, n))


@pytest.mark.parametrize("nranks", [2, 4])
@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_rank_allgather(ranks, oracle, nranks, algo):
    """The ring all-gather as one launch per rank, also with a rank's input aliased to
    its own output slot (sequential_transmit.hpp:496-497)."""
    R = ranks[nranks]
    R.zero()
    seq = 1
    s0 = [b.ptr for b in R.scatter]
    s1 = [b.ptr for b in R.gather]
    for n in (8, 8 * 1237, 1 << 18):
        ins = H.make_inputs(oracle, nranks, n, 8500 + n)
        want = oracle.allgather(ins)
        for alias in (False, True):
            outs = [DeviceBuffer(nranks * n * 2) for _ in range(nranks)]
            srcs = []
            for r in range(nranks):
                outs[r].fill(0x01)
                if alias:
                    outs[r].upload(ins[r], r * n * 2)
                else:
                    srcs.append(DeviceBuffer(n * 2))
                    srcs[r].upload(ins[r])
            nxt = seq
            for r in range(nranks):
                inp = outs[r].ptr + r * n * 2 if alias else srcs[r].ptr
                nxt = R.ctx[r].allgather_rank(algo, r, inp, outs[r].ptr, s0[r], s1[r], s0, s1, R.sink_bytes, n,
                                              seq, stream=R.handle(r))
            for r in range(nranks):
                R.ctx[r].check(R.handle(r))
            seq = nxt
            for r in range(nranks):
                assert np.array_equal(outs[r].download(np.uint16, nranks * n), want), (algo, n, r, alias)
            for b in outs + srcs:
                b.free()


LAYOUTS = {
    # algo: (oracle wire kind, payload bytes a wave moves per step, reference messages per wave and step)
    "small": (WIRE_RT64, 1024, 16),
    "simple": (WIRE_RT64_128, 1920, 16),
    "small_pcie_p": (WIRE_RT64_PCIE, 1024, 8),
    "simple_pcie_p": (WIRE_RT64_128_PCIE, 1920, 8),
}


@pytest.mark.parametrize("algo", sorted(LAYOUTS))
def test_sink_bytes_are_the_reference_messages(ranks, oracle, algo):
    """Two ranks, ParallelTransmit, one step: rank 0's wave for chunk 1 scatters its
    wire into rank 1's sink entry (x_id + 0), rank 1 reduces and gathers the sum
    into rank 0's entry (x_id + 1) (parallel_transmit.hpp:47-58, 93, 122).  Each
    2 KiB slot must hold the reference's messages for consecutive pieces of the
    wire's payload, flags included."""
    wire, wire_bytes, msgs = LAYOUTS[algo]
    cap, size = oracle.wire_dwords(wire)
    assert cap * 4 * msgs == wire_bytes and size * 4 * msgs == 2048
    R = ranks[2]
    R.zero()
    for c in R.ctx:
        c.set_tuning(wire_fenced=0)        # the reference's messages (left alone, ParallelTransmit takes flag words)
    wires = 5                                          # wires per chunk, the last one ragged
    chunk_bytes = wire_bytes * (wires - 1) + 16 * 7
    n = 2 * chunk_bytes // 2
    ins = H.make_inputs(oracle, 2, n, 8300)
    seq = 0x1234
    got, _ = R.allreduce(algo, ins, seq)
    want = oracle.rotated(ins)
    H.assert_all_ranks_equal(oracle, got, want)
    scat1 = R.scatter[1].download(np.uint32, R.sink_bytes // 4)
    gath0 = R.gather[0].download(np.uint32, R.sink_bytes // 4)

    def expect_slot(chunk_halves, w):
        """The 2 KiB slot of wire w: the packed messages of its payload pieces."""
        data = np.zeros(wire_bytes // 4, np.uint32)
        piece = chunk_halves.view(np.uint8)[w * wire_bytes:(w + 1) * wire_bytes]
        data.view(np.uint8)[:len(piece)] = piece       # lanes beyond the chunk load zeros
        return np.concatenate([oracle.pack_message(wire, data[m * cap:(m + 1) * cap], seq)
                               for m in range(msgs)])

    half = n // 2
    for w in range(wires):
        x_id = 2 * w                                   # wave 2w + y serves column w
        slot = (x_id + 0) * 8 + 0                      # sender rank 0, step 0
        got_slot = scat1[slot * 512:(slot + 1) * 512]
        assert np.array_equal(got_slot, expect_slot(ins[0][half:], w)), (algo, "scatter", w)
        slot = (x_id + 1) * 8 + 0                      # owner rank 1 gathers into rank 0
        got_slot = gath0[slot * 512:(slot + 1) * 512]
        assert np.array_equal(got_slot, expect_slot(want[half:], w)), (algo, "gather", w)
    for c in R.ctx:
        c.set_tuning(wire_fenced=-1)


def test_rank_call_validates_like_the_constructor(ranks):
    R = ranks[2]
    buf = DeviceBuffer(4096)
    s0 = [b.ptr for b in R.scatter]
    s1 = [b.ptr for b in R.gather]
    c = R.ctx[0]
    with pytest.raises(vr.VRError) as e:                       # allreduce.hpp:110-111
        c.allreduce_rank("simple", 0, buf.ptr + 4, s0[0], s1[0], s0, s1, R.sink_bytes, 64, 1)
    assert e.value.code == "UNALIGNED"
    with pytest.raises(vr.VRError) as e:                       # allreduce.hpp:116-118
        c.allreduce_rank("simple", 0, buf.ptr, s0[0], s1[0], s0, s1, R.sink_bytes, 4 * 3, 1)
    assert e.value.code == "UNEVEN"
    with pytest.raises(vr.VRError) as e:
        c.allreduce_rank("simple", 2, buf.ptr, s0[0], s1[0], s0, s1, R.sink_bytes, 64, 1)
    assert e.value.code == "INVALID"
    with pytest.raises(vr.VRError) as e:                       # sinks smaller than the context needs
        c.allreduce_rank("simple", 0, buf.ptr, s0[0], s1[0], s0, s1, R.sink_bytes // 2, 64, 1)
    assert e.value.code == "INVALID" and "vr_rank_scratch_bytes" in e.value.detail
    with pytest.raises(vr.VRError) as e:
        c.allreduce_rank("simple", 0, buf.ptr, s0[0], s1[0], s0, s1, R.sink_bytes, 64, 0)
    assert e.value.code == "INVALID"
    # the 16-byte-message protocols demand 16-byte alignment (rt64.hpp:3-20 message_t)
    with pytest.raises(vr.VRError) as e:
        c.allreduce_rank("simple_ring", 0, buf.ptr + 8, s0[0], s1[0], s0, s1, R.sink_bytes, 64, 1)
    assert e.value.code == "UNALIGNED"
    buf.free()


@pytest.mark.parametrize("fenced", [-1, 0])
@pytest.mark.parametrize("algo", ["simple", "bisect", "small", "simple_transmit", "parallel"])
def test_eight_byte_aligned_buffers_with_sixteen_byte_chunks(ranks, oracle, algo, fenced):
    """message_t of small / simple / bisect is 8 bytes (rt64.hpp:335, rt64_128.hpp:539):
    an 8-byte-aligned buffer is accepted whatever the chunk length, as by the
    reference's per-rank calcWorkSize, with the reference's messages (fenced 0) and
    with flag words (the library's choice), also when only some ranks' buffers are
    off a 16-byte boundary."""
    R = ranks[4]
    R.zero()
    for c in R.ctx:
        c.set_tuning(wire_fenced=fenced)
    seq = 1
    for n, odd_ranks in ((4 * 64, (0, 1, 2, 3)), (4 * 8 * 1001, (0, 1, 2, 3)), (4 * 8 * 333, (1, 2))):
        ins = H.make_inputs(oracle, 4, n, 8700 + n)
        off = [8 if r in odd_ranks else 16 for r in range(4)]     # 8 bytes off a 16-byte boundary, or on one
        bufs = [DeviceBuffer(n * 2 + 64) for _ in range(4)]
        for r in range(4):
            bufs[r].upload(ins[r], off[r])
        ptrs = [bufs[r].ptr + off[r] for r in range(4)]
        s0 = [b.ptr for b in R.scatter]
        s1 = [b.ptr for b in R.gather]
        nxt = seq
        for r in range(4):
            nxt = R.ctx[r].allreduce_rank(algo, r, ptrs[r], s0[r], s1[r], s0, s1, R.sink_bytes, n, seq,
                                          stream=R.handle(r))
        for r in range(4):
            R.ctx[r].check(R.handle(r))
        seq = nxt
        got = [bufs[r].download(np.uint16, n, off[r]) for r in range(4)]
        H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), "%s n=%d" % (algo, n))
        for b in bufs:
            b.free()
    for c in R.ctx:
        c.set_tuning(wire_fenced=-1)


class Groups:
    """N ranks held by N / k launches of k ranks each (vr_allreduce_ranks), one stream
    per launch: 8 ranks on the 4 hardware queues of one process."""

    def __init__(self, nranks, per_launch):
        self.n, self.k = nranks, per_launch
        self.ctx = vr.VirtualRanks(nranks)
        self.ctx.set_spin_limit(SPIN)
        self.streams = stream_pool()[:nranks // per_launch]
        self.sink_bytes = self.ctx.rank_scratch_bytes()
        self.scatter = [DeviceBuffer(self.sink_bytes) for _ in range(nranks)]
        self.gather = [DeviceBuffer(self.sink_bytes) for _ in range(nranks)]
        self.zero()

    def zero(self):
        for b in self.scatter + self.gather:
            b.fill(0)

    def handle(self, g):
        return self.streams[g].handle if self.streams[g] else None

    def check(self):
        for g in range(len(self.streams)):
            self.ctx.check(self.handle(g))

    def close(self):
        for b in self.scatter + self.gather:
            b.free()
        self.ctx.close()


@pytest.mark.parametrize("nranks,per_launch", [(8, 2), (8, 4), (4, 2)])
@pytest.mark.parametrize("algo", ["simple", "small", "parallel", "bisect", "simple_ring", "small_pcie"])
def test_rank_group_launches(oracle, nranks, per_launch, algo):
    G = Groups(nranks, per_launch)
    s0 = [b.ptr for b in G.scatter]
    s1 = [b.ptr for b in G.gather]
    seq = 1
    for k, n in enumerate((64 * nranks, 64 * nranks * 33, 1 << 20)):
        ins = H.make_inputs(oracle, nranks, n, 8800 + 10 * k + nranks)
        want = H.expected(oracle, algo, ins)
        for inplace in (True, False):
            src = H.RankBuffers(nranks, n)
            src.upload(ins)
            dst = None
            if not inplace:
                dst = H.RankBuffers(nranks, n)
                dst.fill(0xAB)
            nxt = seq
            for g in range(nranks // per_launch):
                first = g * per_launch
                nxt = G.ctx.allreduce_ranks(algo, first, src.ptrs[first:first + per_launch], s0, s1, G.sink_bytes,
                                            n, seq, outs=dst.ptrs[first:first + per_launch] if dst else None,
                                            stream=G.handle(g))
            G.check()
            assert nxt > seq
            seq = nxt
            H.assert_all_ranks_equal(oracle, (dst or src).download(), want,
                                     "%s N=%d k=%d n=%d" % (algo, nranks, per_launch, n))
            src.free()
            if dst:
                dst.free()
    G.close()


@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_rank_group_allgather(oracle, algo):
    G = Groups(8, 2)
    s0 = [b.ptr for b in G.scatter]
    s1 = [b.ptr for b in G.gather]
    seq = 1
    for n in (8, 8 * 1237, 1 << 17):
        ins = H.make_inputs(oracle, 8, n, 8900 + n)
        want = oracle.allgather(ins)
        srcs = [DeviceBuffer(n * 2) for _ in range(8)]
        outs = [DeviceBuffer(8 * n * 2) for _ in range(8)]
        for r in range(8):
            srcs[r].upload(ins[r])
            outs[r].fill(0x01)
        nxt = seq
        for g in range(4):
            nxt = G.ctx.allgather_ranks(algo, 2 * g, [b.ptr for b in srcs[2 * g:2 * g + 2]],
                                        [b.ptr for b in outs[2 * g:2 * g + 2]], s0, s1, G.sink_bytes, n, seq,
                                        stream=G.handle(g))
        G.check()
        seq = nxt
        for r in range(8):
            assert np.array_equal(outs[r].download(np.uint16, 8 * n), want), (algo, n, r)
        for b in srcs + outs:
            b.free()
    G.close()


def test_more_launches_than_hardware_queues_are_refused(oracle):
    """Eight one-rank launches in one process would need eight hardware queues; a
    process has four.  The fifth launch of the collective is refused with the
    remedy instead of ending in a time-out, and so is a second rank on a stream
    that already carries another rank of the same collective."""
    R = Groups(8, 1)                                       # sinks for 8 ranks, context, pool of streams
    R.ctx.set_spin_limit(64)
    n = 8 * 64
    src = H.RankBuffers(8, n)
    src.upload(H.make_inputs(oracle, 8, n, 9000))
    s0 = [b.ptr for b in R.scatter]
    s1 = [b.ptr for b in R.gather]
    pool = stream_pool()
    handles = [p.handle if p else None for p in pool]
    for r in range(4):
        R.ctx.allreduce_rank("simple", r, src.ptrs[r], s0[r], s1[r], s0, s1, R.sink_bytes, n, 7, stream=handles[r])
    extra = Stream()
    with pytest.raises(vr.VRError) as e:
        R.ctx.allreduce_rank("simple", 4, src.ptrs[4], s0[4], s1[4], s0, s1, R.sink_bytes, n, 7, stream=extra.handle)
    assert e.value.code == "INVALID" and "vr_allreduce_ranks" in e.value.detail
    with pytest.raises(vr.VRError) as e:
        R.ctx.allreduce_rank("simple", 5, src.ptrs[5], s0[5], s1[5], s0, s1, R.sink_bytes, n, 7, stream=handles[1])
    assert e.value.code == "INVALID" and "same stream" in e.value.detail
    # the four launches that did start give up after 64 polls and drain
    timed_out = 0
    for r in range(4):
        try:
            R.ctx.check(handles[r])
        except vr.VRError as err:
            assert err.code == "TIMEOUT"
            timed_out += 1
    assert timed_out >= 1
    extra.close()
    src.free()
    R.close()


@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_rank_allgather_with_a_user_grid(ranks, oracle, algo):
    """testAllgather's per-rank form (allreduce.cpp:1191-1213): the -g / -w / -s grid
    changes the launch, never the gathered bytes."""
    R = ranks[4]
    R.zero()
    s0 = [b.ptr for b in R.scatter]
    s1 = [b.ptr for b in R.gather]
    n = 14336
    ins = H.make_inputs(oracle, 4, n, 9100)
    want = oracle.allgather(ins)
    srcs = [DeviceBuffer(n * 2) for _ in range(4)]
    outs = [DeviceBuffer(4 * n * 2) for _ in range(4)]
    for r in range(4):
        srcs[r].upload(ins[r])
    seq = 0xE00F100F
    for groups, subgroups, simd in ((1, 4, 16), (7, 8, 16), (19, 32, 32), (64, 64, 16)):
        for o in outs:
            o.fill(0x01)
        for r in range(4):
            R.ctx[r].allgather_rank_grid(algo, r, srcs[r].ptr, outs[r].ptr, s0[r], s1[r], s0, s1, R.sink_bytes, n,
                                         seq, groups, subgroups, simd, stream=R.handle(r))
        for r in range(4):
            R.ctx[r].check(R.handle(r))
        seq += 100
        for r in range(4):
            assert np.array_equal(outs[r].download(np.uint16, 4 * n), want), (algo, groups, subgroups, r)
    with pytest.raises(vr.VRError) as e:
        R.ctx[0].allgather_rank_grid(algo, 0, srcs[0].ptr, outs[0].ptr, s0[0], s1[0], s0, s1, R.sink_bytes, n,
                                     seq, 4, 2, 16)
    assert e.value.code == "GEOMETRY"
    for b in srcs + outs:
        b.free()


@pytest.mark.parametrize("algo", ["simple", "parallel", "small", "bisect"])
def test_eight_byte_granular_chunks_through_the_rank_calls(ranks, oracle, algo):
    """Chunks that are only a multiple of 8 bytes (and buffers that are only 8-byte
    aligned) take the 8-byte access path on every rank."""
    R = ranks[4]
    R.zero()
    seq = 1
    for n, offset in ((4 * 4 * 1001, 0), (4 * 4 * 33, 8)):
        ins = H.make_inputs(oracle, 4, n, 8600 + n)
        src = H.RankBuffers(4, n, offset)
        src.upload(ins)
        s0 = [b.ptr for b in R.scatter]
        s1 = [b.ptr for b in R.gather]
        nxt = seq
        for r in range(4):
            nxt = R.ctx[r].allreduce_rank(algo, r, src.ptrs[r], s0[r], s1[r], s0, s1, R.sink_bytes, n, seq,
                                          stream=R.handle(r))
        for r in range(4):
            R.ctx[r].check(R.handle(r))
        seq = nxt
        H.assert_all_ranks_equal(oracle, src.download(), H.expected(oracle, algo, ins), "%s n=%d" % (algo, n))
        src.free()


def test_a_rank_without_peers_times_out_and_drains(oracle):
    """Only rank 0 of two is launched: its waves wait for messages that never come,
    give up after the spin limit, and the kernel still finishes."""
    R = Ranks(2)
    R.ctx[0].set_spin_limit(64)
    ins = H.make_inputs(oracle, 2, 1 << 12, 8400)
    src = H.RankBuffers(2, 1 << 12)
    src.upload(ins)
    s0 = [b.ptr for b in R.scatter]
    s1 = [b.ptr for b in R.gather]
    R.ctx[0].allreduce_rank("simple", 0, src.ptrs[0], s0[0], s1[0], s0, s1, R.sink_bytes, 1 << 12, 1)
    with pytest.raises(vr.VRError) as e:
        R.ctx[0].check()
    assert e.value.code == "TIMEOUT"
    src.free()
    R.close()
