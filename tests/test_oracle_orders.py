"""Pins the oracle's summation orders.

Pins used (none of them re-types the oracle's own formula):
  * hand-computed known answers that separate rank order / rotated chain /
    pair tree from each other (a dropped rotation, a wrong owner or a wrong
    half mapping fails one of them);
  * the reference's own fixture, fill_pattern, with its closed form
    (i % 32) * N(N+1)/2 (utils.hpp:15-19, allreduce.cpp:537-548);
  * numpy.float16 brute force written as explicit per-chunk loops;
  * the message-level emulators (second restatement, moves 128-byte wires
    through sinks with the device code's index arithmetic).
"""
import numpy as np
import pytest

from tests.oracle_lib import (WIRE_RT64, WIRE_RT64_128, WIRE_RT64_PCIE, WIRE_RT64_128_PCIE, DIST_NORMAL,
                              DIST_UNIFORM)


def h(x):
    return int(np.array([x], np.float16).view(np.uint16)[0])


def const_ranks(values, n):
    return [np.full(n, h(v), np.uint16) for v in values]


def per_chunk(out, nranks):
    chunk = len(out) // nranks
    vals = []
    for c in range(nranks):
        seg = out[c * chunk:(c + 1) * chunk].view(np.float16)
        assert (seg == seg[0]).all()
        vals.append(float(seg[0]))
    return vals


def test_kat_n4_rotated_vs_bisect_vs_rank(oracle):
    ins = const_ranks([2048, 1, 1, 0], 64)
    # chunk 0: ((2048+1)+1)+0 = 2048; chunk 1: ((1+1)+0)+2048 = 2050;
    # chunk 2: ((1+0)+2048)+1 = 2048; chunk 3: ((0+2048)+1)+1 = 2048
    assert per_chunk(oracle.rotated(ins), 4) == [2048, 2050, 2048, 2048]
    # pair sums p0 = 2048+1 = 2048, p1 = 1+0 = 1 -> 2048 everywhere
    assert per_chunk(oracle.bisect(ins), 4) == [2048, 2048, 2048, 2048]
    # ((0+2048)+1)+1+0 = 2048
    assert per_chunk(oracle.rank_order(ins), 4) == [2048, 2048, 2048, 2048]


def test_kat_n8_three_way(oracle):
    ins = const_ranks([2048, 0, 1, 0, 1, 0, 0, 0], 128)
    assert per_chunk(oracle.bisect(ins), 8) == [2048, 2050, 2048, 2048, 2048, 2050, 2048, 2048]
    assert per_chunk(oracle.rotated(ins), 8) == [2048, 2050, 2050, 2048, 2048, 2048, 2048, 2048]
    assert per_chunk(oracle.rank_order(ins), 8) == [2048] * 8


def test_kat_bisect_pair_is_summed_before_chain(oracle):
    # x = (1, 1, 2048, 0): pair tree (1+1) + (2048+0) = 2050; any chain that
    # feeds the ones one at a time into 2048 loses them.
    ins = const_ranks([1, 1, 2048, 0], 64)
    got = per_chunk(oracle.bisect(ins), 4)
    assert got == [2050, 2050, 2050, 2050]
    assert per_chunk(oracle.rotated(ins), 4)[2] == 2048   # ((2048+0)+1)+1


def test_kat_bisect_odd_half_owner(oracle):
    # N=8, only odd ranks non-zero: x1=2048, x3=1, x5=1 -> p = (2048,1,1,0).
    # Second-half chunks (h=1) are owned by odd ranks 1,3,5,7 with l = 0..3.
    ins = const_ranks([0, 2048, 0, 1, 0, 1, 0, 0], 128)
    assert per_chunk(oracle.bisect(ins), 8) == [2048, 2050, 2048, 2048, 2048, 2050, 2048, 2048]


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("n", [128, 256, 384, 1280, 1920, 1024, 2048, 14336, 16384])
def test_fill_pattern_closed_form(oracle, nranks, n):
    """Reference fixture and shape list (test/test_2tile_shapes.sh:4)."""
    ins = [oracle.fill_pattern(r, n) for r in range(nranks)]
    want = ((np.arange(n) % 32) * (nranks * (nranks + 1) // 2)).astype(np.float16).view(np.uint16)
    assert (ins[1].view(np.float16) == ((np.arange(n) % 32) * 2)).all()
    assert (oracle.rank_order(ins) == want).all()
    assert (oracle.rotated(ins) == want).all()
    if nranks >= 4:
        assert (oracle.bisect(ins) == want).all()


def numpy_rotated(ins):
    N, n = len(ins), len(ins[0])
    chunk = n // N
    f = [a.view(np.float16) for a in ins]
    out = np.empty(n, np.float16)
    for c in range(N):
        sl = slice(c * chunk, (c + 1) * chunk)
        acc = f[c][sl].copy()
        for k in range(1, N):
            acc = (f[(c + k) % N][sl] + acc).astype(np.float16)
        out[sl] = acc
    return out.view(np.uint16)


def numpy_bisect(ins):
    N, n = len(ins), len(ins[0])
    B, chunk = N // 2, n // N
    f = [a.view(np.float16) for a in ins]
    out = np.empty(n, np.float16)
    for owner in range(N):                      # walk owners, derive their chunk
        hh, l = owner & 1, owner // 2
        c = hh * B + l
        sl = slice(c * chunk, (c + 1) * chunk)
        pairs = [(f[2 * j][sl] + f[2 * j + 1][sl]).astype(np.float16) for j in range(B)]
        acc = pairs[l]
        for k in range(1, B):
            acc = (pairs[(l + k) % B] + acc).astype(np.float16)
        out[sl] = acc
    return out.view(np.uint16)


def numpy_rank_order(ins):
    acc = np.zeros(len(ins[0]), np.float16)
    for a in ins:
        acc = (acc + a.view(np.float16)).astype(np.float16)
    return acc.view(np.uint16)


@pytest.mark.parametrize("nranks", [2, 4, 8, 16])
@pytest.mark.parametrize("dist", ["n1", "n002", "u1", "wide"])
def test_orders_against_numpy(oracle, nranks, dist):
    n = 16 * nranks * 37
    if dist == "n1":
        ins = [oracle.generate(n, 100 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
    elif dist == "n002":
        ins = [oracle.generate(n, 200 + r, DIST_NORMAL, 0.0, 0.02) for r in range(nranks)]
    elif dist == "u1":
        ins = [oracle.generate(n, 300 + r, DIST_UNIFORM, -1.0, 1.0) for r in range(nranks)]
    else:  # every exponent incl. subnormals and values that overflow when summed
        rng = np.random.default_rng(nranks)
        ins = []
        for r in range(nranks):
            a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
            a[(a & 0x7C00) == 0x7C00] &= 0x83FF          # no inf / nan in the inputs
            ins.append(a)
    with np.errstate(all="ignore"):
        assert oracle.count_mismatch(oracle.rank_order(ins), numpy_rank_order(ins)) == 0
        assert oracle.count_mismatch(oracle.rotated(ins), numpy_rotated(ins)) == 0
        if nranks >= 4:
            assert oracle.count_mismatch(oracle.bisect(ins), numpy_bisect(ins)) == 0
    # the float route and the integer route agree inside the order loops too
    for mode, fn in ((0, oracle.rank_order), (1, oracle.rotated), (2, oracle.bisect)):
        if mode == 2 and nranks < 4:
            continue
        assert oracle.count_mismatch(fn(ins), oracle.order_soft(mode, ins)) == 0


def test_orders_really_differ_on_random_data(oracle):
    """Guards against the three orders collapsing into one implementation."""
    n = 8 * 4096
    ins = [oracle.generate(n, 1 + r, DIST_NORMAL, 0.0, 1.0) for r in range(8)]
    r0, r1, r2 = oracle.rank_order(ins), oracle.rotated(ins), oracle.bisect(ins)
    assert oracle.count_mismatch(r0, r1) > n // 100
    assert oracle.count_mismatch(r1, r2) > n // 100
    assert oracle.count_mismatch(r0, r2) > n // 100
    # chunk 0 of the rotated order starts at rank 0, so it is the rank-order chain
    chunk = n // 8
    assert (r0[:chunk] == r1[:chunk]).all()


def test_shape_rejection(oracle):
    ins = [np.zeros(30, np.uint16) for _ in range(4)]
    with pytest.raises(ValueError):
        oracle.rotated(ins)
    with pytest.raises(ValueError):
        oracle.bisect([np.zeros(30, np.uint16) for _ in range(3)])
    with pytest.raises(ValueError):
        oracle.bisect([np.zeros(32, np.uint16) for _ in range(2)])


def test_allgather_copy_invariant(oracle):
    ins = [oracle.generate(1000, 5 + r, DIST_UNIFORM, -2.0, 2.0) for r in range(4)]
    out = oracle.allgather(ins)
    for r in range(4):
        assert (out[r * 1000:(r + 1) * 1000] == ins[r]).all()


# ---- message-level emulators vs closed forms --------------------------------

GEOMS = [(1, 8), (2, 4), (4, 4), (8, 8), (16, 16), (64, 64), (7, 8), (13, 16)]


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("wire", [WIRE_RT64, WIRE_RT64_128])
def test_emulate_parallel_matches_rotated(oracle, nranks, wire):
    for n in (4 * nranks, 4 * nranks * 15, 16384, 4 * nranks * 1237):
        ins = [oracle.generate(n, 11 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        want = oracle.rotated(ins)
        for g, w in GEOMS:
            if (g * w) % nranks:
                continue
            rc, io = oracle.emulate_parallel(ins, wire, g, w, seq_no=0xE00F100F)
            assert rc == 0
            for r in range(nranks):
                assert (io[r] == want).all(), (n, g, w, r)


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("wire", [WIRE_RT64, WIRE_RT64_128])
def test_emulate_ring_matches_rotated(oracle, nranks, wire):
    for n in (4 * nranks, 4 * nranks * 15, 16384, 4 * nranks * 1237):
        ins = [oracle.generate(n, 21 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        want = oracle.rotated(ins)
        for g, w in GEOMS[:6]:
            rc, io = oracle.emulate_ring(ins, wire, g, w, seq_no=5)
            assert rc == 0
            for r in range(nranks):
                assert (io[r] == want).all(), (n, g, w, r)


ALL_WIRES = [WIRE_RT64, WIRE_RT64_128, WIRE_RT64_PCIE, WIRE_RT64_128_PCIE]


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("wire", ALL_WIRES)
def test_emulate_sequential_matches_rotated(oracle, nranks, wire):
    """SequentialTransmit (sequential_transmit.hpp:83-207) moves other messages through
    other sinks than ParallelTransmit but associates the same way."""
    for n in (8 * nranks, 8 * nranks * 15, 16384, 8 * nranks * 1237):
        ins = [oracle.generate(n, 41 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        want = oracle.rotated(ins)
        for g, w in GEOMS[:6] + [(3, 4)]:
            rc, io = oracle.emulate_sequential(ins, wire, g, w, seq_no=9)
            assert rc == 0
            for r in range(nranks):
                assert (io[r] == want).all(), (n, g, w, r)


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("wire", [WIRE_RT64_PCIE, WIRE_RT64_128_PCIE])
def test_emulate_ring_pcie_wires(oracle, nranks, wire):
    """RingTransmit is instantiated with the 16-byte-message wires (allreduce.cpp:1150-1163)."""
    for n in (8 * nranks, 8 * nranks * 15, 8 * nranks * 1237):
        ins = [oracle.generate(n, 51 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        want = oracle.rotated(ins)
        for g, w in GEOMS[:5]:
            rc, io = oracle.emulate_ring(ins, wire, g, w, seq_no=3)
            assert rc == 0
            for r in range(nranks):
                assert (io[r] == want).all(), (n, g, w, r)


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("wire", [WIRE_RT64_PCIE, WIRE_RT64_128_PCIE])
def test_emulate_allgather_ring_is_a_copy(oracle, nranks, wire):
    """runAllgather (sequential_transmit.hpp:474-516): every output ends up as the
    concatenation of all inputs, also when a rank's input is its own output slot."""
    for n in (8, 8 * 15, 8 * 1237, 16384):
        ins = [oracle.generate(n, 61 + r, DIST_UNIFORM, -2.0, 2.0) for r in range(nranks)]
        want = oracle.allgather(ins)
        for g, w in GEOMS[:5]:
            for alias in (False, True):
                rc, outs = oracle.emulate_allgather_ring(ins, wire, g, w, seq_no=6, alias_own_slot=alias)
                assert rc == 0
                for r in range(nranks):
                    assert (outs[r] == want).all(), (n, g, w, r, alias)


def test_emulators_reject_what_the_reference_cannot_run(oracle):
    ins = [oracle.generate(64, r, DIST_NORMAL, 0.0, 1.0) for r in range(4)]
    assert oracle.emulate_parallel(ins, WIRE_RT64_PCIE, 1, 4)[0] == -2     # no 256-byte layout restated
    assert oracle.emulate_sequential(ins, WIRE_RT64_PCIE, 0, 4)[0] == -3   # empty launch
    assert oracle.emulate_allgather_ring(ins[:3], WIRE_RT64_PCIE, 1, 4)[0] == -2   # 3 ranks: uint32 wrap


@pytest.mark.parametrize("nranks", [4, 8, 16])
def test_emulate_bisect_matches_tree(oracle, nranks):
    for n in (4 * nranks, 4 * nranks * 15, 16384 if nranks != 16 else 16384 * 2, 4 * nranks * 1237):
        ins = [oracle.generate(n, 31 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        want = oracle.bisect(ins)
        for g, w in GEOMS:
            if (g * w) % (nranks // 2):
                continue
            rc, io = oracle.emulate_bisect(ins, g, w, seq_no=77)
            assert rc == 0
            for r in range(nranks):
                assert (io[r] == want).all(), (n, g, w, r)


def test_emulators_reject_geometry_the_reference_cannot_run(oracle):
    ins = [np.zeros(64, np.uint16) for _ in range(8)]
    rc, _ = oracle.emulate_parallel(ins, WIRE_RT64, 1, 4)      # nWires < N -> loopSize 0
    assert rc == -3
    rc, _ = oracle.emulate_bisect(ins, 1, 2)
    assert rc == -3


# ---- chunking ------------------------------------------------------------------

def test_calc_work_size(oracle):
    # allreduce.hpp:108-122
    assert oracle.calc_work_size(0x1000, 16384 * 2, 2, 8) == (0, 16384)
    assert oracle.calc_work_size(0x1004, 16384 * 2, 2, 8)[0] == 1      # unaligned pointer
    assert oracle.calc_work_size(0x1000, 16384 * 2 + 4, 2, 8)[0] == 2  # bytes % msg
    assert oracle.calc_work_size(0x1000, 8 * 9, 8, 8)[0] == 2          # 9 messages over 8 chunks
    assert oracle.calc_work_size(0x1000, 8 * 16, 8, 8) == (0, 16)
    assert oracle.calc_work_size(0x1000, 16 * 8, 8, 16) == (0, 16)
    assert oracle.calc_work_size(0x1008, 16 * 8, 8, 16)[0] == 1
    # all-gather: one chunk (allgather.hpp:104-117)
    assert oracle.calc_work_size(0x1000, 8 * 7, 1, 8) == (0, 56)


def test_generator_is_reproducible_and_distribution_sane(oracle):
    a = oracle.generate(200000, 42, DIST_NORMAL, 0.0, 1.0)
    b = oracle.generate(200000, 42, DIST_NORMAL, 0.0, 1.0)
    assert (a == b).all()
    c = oracle.generate(1000, 42, DIST_NORMAL, 0.0, 1.0)
    assert (c == a[:1000]).all()                       # counter-based: prefixes agree
    f = a.view(np.float16).astype(np.float64)
    assert abs(f.mean()) < 0.01 and abs(f.std() - 1.0) < 0.01
    u = oracle.generate(200000, 43, DIST_UNIFORM, -2.0, 2.0).view(np.float16).astype(np.float64)
    assert u.min() >= -2.0 and u.max() <= 2.0 and abs(u.mean()) < 0.02
    assert abs(u.std() - 4.0 / np.sqrt(12.0)) < 0.01
    s = oracle.generate(200000, 44, DIST_NORMAL, 0.0, 0.02).view(np.float16).astype(np.float64)
    assert abs(s.std() - 0.02) < 0.0005
    assert not (oracle.generate(1000, 45, DIST_NORMAL, 0.0, 1.0) == c).all()
