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
    # a chunk of 16-byte multiples travels with 16-byte accesses on every rank
    with pytest.raises(vr.VRError) as e:
        c.allreduce_rank("simple", 0, buf.ptr + 8, s0[0], s1[0], s0, s1, R.sink_bytes, 64, 1)
    assert e.value.code == "UNALIGNED" and "16-byte" in e.value.detail
    buf.free()


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
