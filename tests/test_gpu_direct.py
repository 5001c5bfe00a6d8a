"""GPU parity tests (direct transport): HIP path through the C ABI vs the CPU
oracle on the same seeded inputs.  Bit-exact: binary16 sums must match in every
bit (NaNs compare equal to NaNs)."""
import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from tests import vr_helpers as H
from tests.oracle_lib import DIST_NORMAL, DIST_UNIFORM

pytestmark = pytest.mark.gpu


def h(x):
    return int(np.array([x], np.float16).view(np.uint16)[0])


@pytest.fixture(scope="module")
def ctxs():
    made = {n: vr.VirtualRanks(n) for n in (2, 4, 8, 16)}
    yield made
    for c in made.values():
        c.close()


def per_chunk(out, nranks):
    chunk = len(out) // nranks
    vals = []
    for c in range(nranks):
        seg = out[c * chunk:(c + 1) * chunk].view(np.float16)
        assert (seg == seg[0]).all()
        vals.append(float(seg[0]))
    return vals


# ---- known answers that separate the summation orders -------------------------------

def test_kat_n4(ctxs):
    ins = [np.full(256, h(v), np.uint16) for v in (2048, 1, 1, 0)]
    got, _ = H.run_allreduce(ctxs[4], "simple", ins)
    for g in got:
        assert per_chunk(g, 4) == [2048, 2050, 2048, 2048]
    got, _ = H.run_allreduce(ctxs[4], "bisect", ins)
    for g in got:
        assert per_chunk(g, 4) == [2048, 2048, 2048, 2048]
    ins = [np.full(256, h(v), np.uint16) for v in (1, 1, 2048, 0)]
    got, _ = H.run_allreduce(ctxs[4], "bisect", ins)
    for g in got:
        assert per_chunk(g, 4) == [2050, 2050, 2050, 2050]


@pytest.mark.parametrize("algo", ["small", "simple", "bisect", "small_ring", "simple_pcie"])
def test_kat_n8_three_way(ctxs, algo):
    ins = [np.full(1024, h(v), np.uint16) for v in (2048, 0, 1, 0, 1, 0, 0, 0)]
    got, _ = H.run_allreduce(ctxs[8], algo, ins)
    want = ([2048, 2050, 2048, 2048, 2048, 2050, 2048, 2048] if algo == "bisect"
            else [2048, 2050, 2050, 2048, 2048, 2048, 2048, 2048])
    for g in got:
        assert per_chunk(g, 8) == want


# ---- the reference's own fixture and shape list ----------------------------------------

@pytest.mark.parametrize("nranks", [2, 4, 8])
def test_fill_pattern_shapes(ctxs, oracle, nranks):
    for n in (128, 256, 384, 1280, 1920, 1024, 2048, 14336, 16384):   # test_2tile_shapes.sh:4
        ins = [oracle.fill_pattern(r, n) for r in range(nranks)]
        want = ((np.arange(n) % 32) * (nranks * (nranks + 1) // 2)).astype(np.float16).view(np.uint16)
        for algo in ("small", "simple") + (("bisect",) if nranks >= 4 else ()):
            if n % (4 * nranks):
                continue
            got, _ = H.run_allreduce(ctxs[nranks], algo, ins)
            H.assert_all_ranks_equal(oracle, got, want, "%s n=%d" % (algo, n))


@pytest.mark.parametrize("groups", [1, 2, 4, 8, 16, 32, 64, 7, 13, 15, 17, 19])
def test_result_independent_of_grid(ctxs, oracle, groups):
    """test_8tile_shapes.sh sweeps -g x -w; sub-group counts are kept to the
    multiples of 4 that main.cpp:289-291 still accepts."""
    n = 14336
    ins = H.make_inputs(oracle, 8, n, 500)
    for algo in ("small", "bisect"):
        want = H.expected(oracle, algo, ins)
        for subgroups in (4, 8, 32, 64):
            got, _ = H.run_allreduce(ctxs[8], algo, ins, grid=(groups, subgroups, 16))
            H.assert_all_ranks_equal(oracle, got, want, "%s g=%d w=%d" % (algo, groups, subgroups))


def test_grid_validation(ctxs, oracle):
    ins = H.make_inputs(oracle, 8, 1024, 1)
    for bad_w in (1, 2, 6):
        with pytest.raises(vr.VRError) as e:
            H.run_allreduce(ctxs[8], "small", ins, grid=(4, bad_w, 16))
        assert e.value.code == "GEOMETRY"
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[8], "small", ins, grid=(4, 4, 8))
    assert e.value.code == "SUBGROUP"
    got, _ = H.run_allreduce(ctxs[8], "small", ins, grid=(4, 4, 32))
    H.assert_all_ranks_equal(oracle, got, oracle.rotated(ins))


# ---- random data, every algo string, every world size --------------------------------------

@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("algo", H.ROTATED_ALGOS + ("bisect",))
def test_random_all_algos(ctxs, oracle, nranks, algo):
    if algo == "bisect" and nranks < 4:
        pytest.skip("bisect needs >= 4 ranks")
    msg = 16 if ("pcie" in algo or "ring" in algo) else 8
    unit = (msg // 2) * nranks
    for k, n in enumerate((unit, unit * 3, unit * 129, unit * 1000 + unit, 1 << 20)):
        if n % unit:
            n = (n // unit) * unit
        ins = H.make_inputs(oracle, nranks, n, 1000 * nranks + 10 * k)
        want = H.expected(oracle, algo, ins)
        got, _ = H.run_allreduce(ctxs[nranks], algo, ins)
        H.assert_all_ranks_equal(oracle, got, want, "%s N=%d n=%d in-place" % (algo, nranks, n))
        got, kept = H.run_allreduce(ctxs[nranks], algo, ins, inplace=False)
        H.assert_all_ranks_equal(oracle, got, want, "%s N=%d n=%d out-of-place" % (algo, nranks, n))
        for a, b in zip(kept, ins):
            assert (a == b).all(), "out-of-place run modified an input"


def test_bisect_16_ranks(ctxs, oracle):
    for n in (64, 64 * 77, 1 << 18):
        ins = H.make_inputs(oracle, 16, n, 77)
        got, _ = H.run_allreduce(ctxs[16], "bisect", ins)
        H.assert_all_ranks_equal(oracle, got, oracle.bisect(ins))


@pytest.mark.parametrize("algo", ["simple", "bisect"])
def test_eight_byte_granularity(ctxs, oracle, algo):
    """Chunks that are a multiple of 8 bytes but not of 16, and pointers that are
    only 8-byte aligned: both legal for the 8-byte message protocols."""
    for n in (32 * 1, 32 * 3, 32 * 1001):                 # chunk = 4, 12, 4004 halves
        ins = H.make_inputs(oracle, 8, n, 40 + n)
        want = H.expected(oracle, algo, ins)
        got, _ = H.run_allreduce(ctxs[8], algo, ins)
        H.assert_all_ranks_equal(oracle, got, want, "n=%d" % n)
    ins = H.make_inputs(oracle, 8, 1 << 16, 9)
    want = H.expected(oracle, algo, ins)
    got, _ = H.run_allreduce(ctxs[8], algo, ins, offset_bytes=8)
    H.assert_all_ranks_equal(oracle, got, want, "offset 8")
    got, _ = H.run_allreduce(ctxs[8], algo, ins, offset_bytes=8, inplace=False)
    H.assert_all_ranks_equal(oracle, got, want, "offset 8 out-of-place")


def test_runtime_rejections(ctxs, oracle):
    ins = H.make_inputs(oracle, 8, 1 << 12, 3)
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[8], "simple", ins, offset_bytes=4)
    assert e.value.code == "UNALIGNED"
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[8], "simple_ring", ins, offset_bytes=8)      # 16-byte messages
    assert e.value.code == "UNALIGNED"
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[8], "simple", [a[:4 * 8 + 4] for a in ins])
    assert e.value.code == "UNEVEN"
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[2], "bisect", ins[:2])
    assert e.value.code == "TOPOLOGY"
    with pytest.raises(vr.VRError) as e:
        H.run_allreduce(ctxs[16], "simple", H.make_inputs(oracle, 16, 1 << 12, 3))
    assert e.value.code == "TOPOLOGY"
    # empty input: the reference's loop simply does not execute
    empty = [np.zeros(0, np.uint16) for _ in range(8)]
    got, _ = H.run_allreduce(ctxs[8], "simple", empty)
    assert all(len(g) == 0 for g in got)


def test_partial_overlap_is_rejected(ctxs):
    from gpu_ipc_example_amd.binding import DeviceBuffer
    big = DeviceBuffer(1 << 20)
    n = 1 << 12
    bufs = [big.ptr + r * n * 2 for r in range(8)]
    outs = [big.ptr + r * n * 2 + 64 for r in range(8)]
    with pytest.raises(vr.VRError) as e:
        ctxs[8].allreduce("simple", bufs, n, outs=outs)
    assert e.value.code == "OVERLAP"
    big.free()


def test_special_values(ctxs, oracle):
    """Subnormals are kept, overflow goes to infinity, inf-inf gives NaN."""
    rng = np.random.default_rng(11)
    n = 8 * 4096
    ins = []
    for r in range(8):
        a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
        a[(a & 0x7C00) == 0x7C00] &= 0x83FF           # finite inputs, every exponent
        ins.append(a)
    ins[0][:64] = 0x0001                               # smallest subnormals
    ins[1][:64] = 0x8001
    ins[2][64:128] = 0x7BFF                            # +max
    ins[3][64:128] = 0x7BFF
    ins[4][128:192] = 0x7C00                           # +inf and -inf
    ins[5][128:192] = 0xFC00
    for algo in ("simple", "bisect"):
        got, _ = H.run_allreduce(ctxs[8], algo, ins)
        H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), algo)


@pytest.mark.parametrize("nranks", [2, 4, 8])
def test_adds_through_binary32_give_the_same_bits(ctxs, oracle, nranks):
    """f16_wide=1 adds binary16 values as binary32 and rounds back after every add:
    every finite exponent, subnormals, signed zeros, overflow to infinity and
    inf - inf must come out as from the native binary16 add."""
    ctx = ctxs[nranks]
    rng = np.random.default_rng(12 + nranks)
    n = nranks * 8 * 8192
    ins = []
    for r in range(nranks):
        a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
        a[(a & 0x7C00) == 0x7C00] &= 0x83FF
        ins.append(a)
    ins[0][:64] = 0x0001
    ins[1][:64] = 0x8001
    ins[0][64:128] = 0x7BFF
    ins[1][64:128] = 0x7BFF
    ins[0][128:192] = 0x7C00
    ins[1][128:192] = 0xFC00
    ins[0][192:256] = 0x8000                           # -0 + -0 stays -0
    ins[1][192:256] = 0x8000
    for r in range(2, nranks):
        ins[r][:256] = 0x8000
    small = [oracle.generate(n, 900 + r, DIST_NORMAL, 0.0, 1e-4) for r in range(nranks)]   # sums in the subnormal range
    ctx.set_tuning(f16_wide=1)
    try:
        for data in (ins, small):
            for algo in ("simple", "bisect") if nranks >= 4 else ("simple",):
                for unroll in (1, 2):
                    ctx.set_tuning(unroll=unroll)
                    got, _ = H.run_allreduce(ctx, algo, data)
                    H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, data), "%s unroll %d" % (algo, unroll))
    finally:
        ctx.set_tuning(f16_wide=-1, unroll=-1)


# ---- the five benchmark configurations at full size ------------------------------------------------------

def test_config1_two_ranks_simple(ctxs, oracle):
    ins = H.make_inputs(oracle, 2, 16384, 1234, DIST_UNIFORM, -1.0, 1.0)
    got, _ = H.run_allreduce(ctxs[2], "simple", ins, inplace=False)
    want = oracle.rotated(ins)
    assert (want == oracle.rank_order(ins)).all()      # N=2: every order coincides
    H.assert_all_ranks_equal(oracle, got, want)


def test_config2_small_1mib(ctxs, oracle):
    ins = H.make_inputs(oracle, 8, 524288, 2000, DIST_NORMAL, 0.0, 1.0)
    got, _ = H.run_allreduce(ctxs[8], "small", ins)
    H.assert_all_ranks_equal(oracle, got, oracle.rotated(ins))


def test_config3_bisect_32mib(ctxs, oracle):
    ins = H.make_inputs(oracle, 8, 16777216, 3000, DIST_NORMAL, 0.0, 0.02)
    want = oracle.bisect(ins)
    got, _ = H.run_allreduce(ctxs[8], "bisect", ins)
    H.assert_all_ranks_equal(oracle, got, want)
    assert oracle.count_mismatch(want, oracle.rotated(ins)) > 1000   # the tree really differs


@pytest.mark.parametrize("algo,transport", [("bisect", vr.TRANSPORT_DIRECT), ("simple", vr.TRANSPORT_DIRECT),
                                            ("small", vr.TRANSPORT_DIRECT), ("parallel", vr.TRANSPORT_WIRE)])
def test_full_size_closed_form(ctxs, algo, transport):
    """The reference's own fixture at the headline size, checked without the oracle:
    rank r holds (i % 32) * (r + 1), so every order gives (i % 32) * N (N + 1) / 2
    exactly (utils.hpp:15-19, allreduce.cpp:537-548)."""
    n = 16777216
    from gpu_ipc_example_amd import binding
    ins = [binding.fill_pattern(r, n) for r in range(8)]
    want = ((np.arange(n, dtype=np.int64) % 32) * 36).astype(np.float16).view(np.uint16)
    got, _ = H.run_allreduce(ctxs[8], algo, ins, transport=transport)
    for r in range(8):
        assert np.array_equal(got[r], want), (algo, r)


def test_config5_sweep_sizes(ctxs, oracle):
    """4 KiB ... 256 MiB per rank in powers of two; the largest sizes are checked
    on one protocol each to keep host memory and time bounded."""
    for p in range(11, 28):
        n = 1 << p
        algos = ("small", "simple", "bisect") if p <= 22 else (("simple",) if p % 2 else ("bisect",))
        ins = H.make_inputs(oracle, 8, n, 5000 + p)
        for algo in algos:
            got, _ = H.run_allreduce(ctxs[8], algo, ins)
            want = H.expected(oracle, algo, ins)
            # all ranks hold the same bits; compare rank 0 fully and the rest by equality
            assert oracle.count_mismatch(got[0], want) == 0, (algo, n)
            for r in range(1, 8):
                assert oracle.count_mismatch(got[r], got[0]) == 0, (algo, n, r)


def test_multi_stream_copy_yardstick(ctxs, oracle):
    """The all-reduce kernel with the adds removed copies stream k to stream k."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    for nranks, n in ((8, 8 * 8 * 1031), (8, 1 << 22), (4, 4 * 8 * 77), (2, 1 << 16)):
        ins = H.make_inputs(oracle, nranks, n, 5600 + nranks)
        src = H.RankBuffers(nranks, n)
        src.upload(ins)
        dst = H.RankBuffers(nranks, n)
        dst.fill(0x11)
        ctxs[nranks].stream_probe_multi(dst.ptrs, src.ptrs, n * 2)
        ctxs[nranks].sync()
        for a, b in zip(dst.download(), ins):
            assert np.array_equal(a, b), (nranks, n)
        src.free()
        dst.free()
    with pytest.raises(vr.VRError) as e:
        ctxs[8].stream_probe_multi([16] * 8, [16] * 8, 8 * 16 + 16)
    assert e.value.code == "UNEVEN"


# ---- all-gather ---------------------------------------------------------------------------------

def run_allgather(ctx, algo, ins, alias_own_slot=False):
    from gpu_ipc_example_amd.binding import DeviceBuffer
    N, n = ctx.nranks, len(ins[0])
    outs = [DeviceBuffer(N * n * 2 + 64) for _ in range(N)]
    for o in outs:
        o.fill(0x01)                                   # main.cpp:300 memsets the output to 1
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
    ctx.allgather(algo, in_ptrs, [o.ptr for o in outs], n)
    ctx.check()
    got = [o.download(np.uint16, N * n) for o in outs]
    for b in outs + srcs:
        b.free()
    return got


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_allgather(ctxs, oracle, nranks, algo):
    for n in (8, 8 * 15, 8 * 1237, 1 << 16):
        ins = H.make_inputs(oracle, nranks, n, 70 + n, DIST_UNIFORM, -2.0, 2.0)
        want = oracle.allgather(ins)
        for alias in (False, True):
            got = run_allgather(ctxs[nranks], algo, ins, alias)
            for r in range(nranks):
                assert (got[r] == want).all(), (n, r, alias)


@pytest.mark.parametrize("transport", ["direct", "wire"])
@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_allgather_result_independent_of_grid(ctxs, oracle, algo, transport):
    """testAllgather takes the harness's -g / -w / -s grid (allreduce.cpp:1191-1213,
    main.cpp:293-307): the gathered bytes never depend on it, and the grids
    main.cpp or the dispatcher reject are rejected here."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    tr = vr.TRANSPORT_WIRE if transport == "wire" else vr.TRANSPORT_DIRECT
    ctx = ctxs[4]
    n = 14336
    ins = H.make_inputs(oracle, 4, n, 7300, DIST_UNIFORM, -2.0, 2.0)
    want = oracle.allgather(ins)
    srcs = [DeviceBuffer(n * 2) for _ in range(4)]
    outs = [DeviceBuffer(4 * n * 2) for _ in range(4)]
    for s, a in zip(srcs, ins):
        s.upload(a)
    seq = 0xE00F100F
    for groups in (1, 2, 7, 13, 19, 64):
        for subgroups in (4, 8, 32, 64):
            for o in outs:
                o.fill(0x01)
            ctx.allgather_grid(algo, [s.ptr for s in srcs], [o.ptr for o in outs], n, groups, subgroups,
                               simd=32 if groups == 7 else 16, transport=tr, seq_no=seq)
            ctx.check()
            seq += 100
            for r in range(4):
                assert (outs[r].download(np.uint16, 4 * n) == want).all(), (algo, transport, groups, subgroups, r)
    for bad_w, code in ((2, "GEOMETRY"), (6, "GEOMETRY")):
        with pytest.raises(vr.VRError) as e:
            ctx.allgather_grid(algo, [s.ptr for s in srcs], [o.ptr for o in outs], n, 4, bad_w, transport=tr)
        assert e.value.code == code
    with pytest.raises(vr.VRError) as e:
        ctx.allgather_grid(algo, [s.ptr for s in srcs], [o.ptr for o in outs], n, 4, 4, simd=8, transport=tr)
    assert e.value.code == "SUBGROUP"
    with pytest.raises(vr.VRError) as e:
        ctx.allgather_grid("simple", [s.ptr for s in srcs], [o.ptr for o in outs], n, 4, 4, transport=tr)
    assert e.value.code == "ALGO"
    for b in srcs + outs:
        b.free()


def test_config4_allgather_8mib(ctxs, oracle):
    ins = H.make_inputs(oracle, 4, 4194304, 4000, DIST_UNIFORM, -2.0, 2.0)
    want = oracle.allgather(ins)
    got = run_allgather(ctxs[4], "allgather_simple", ins)
    for r in range(4):
        assert (got[r] == want).all()


def test_allgather_rejections(ctxs, oracle):
    ins = H.make_inputs(oracle, 4, 12, 1)                # 24 bytes: not a whole 16-byte message
    with pytest.raises(vr.VRError) as e:
        run_allgather(ctxs[4], "allgather_small", ins)
    assert e.value.code == "UNEVEN"


def test_long_chunks_take_several_launches(ctxs, oracle):
    """A launch addresses a chunk with 32-bit offsets; longer chunks are cut into
    segments.  With the segment forced down to 4 KiB every size here takes several
    launches per chunk, the last one a ragged piece."""
    ctx = ctxs[8]
    ctx.set_tuning(segment_kib=4)
    try:
        for algo, n in (("simple", 8 * 4 * 5000), ("bisect", 8 * 4 * 5000 + 32), ("small", 8 * 8 * 3333),
                        ("simple_ring", 8 * 8 * 2048)):
            ins = H.make_inputs(oracle, 8, n, 5150 + n)
            want = H.expected(oracle, algo, ins)
            got, _ = H.run_allreduce(ctx, algo, ins)
            H.assert_all_ranks_equal(oracle, got, want, "%s n=%d segmented" % (algo, n))
            got, _ = H.run_allreduce(ctx, algo, ins, inplace=False)
            H.assert_all_ranks_equal(oracle, got, want, "%s n=%d segmented out-of-place" % (algo, n))
        ins = H.make_inputs(oracle, 8, 8 * 1237, 99, DIST_UNIFORM, -2.0, 2.0)
        want = oracle.allgather(ins)
        for alias in (False, True):
            got = run_allgather(ctx, "allgather_simple", ins, alias)
            for r in range(8):
                assert (got[r] == want).all(), (r, alias)
    finally:
        ctx.set_tuning(segment_kib=-1)


@pytest.mark.parametrize("nt_store", [0, 1, 2])
@pytest.mark.parametrize("nt_load", [0, 1])
def test_every_cache_policy_gives_the_same_bits(ctxs, oracle, nt_load, nt_store):
    ctx = ctxs[8]
    ctx.set_tuning(nt_load=nt_load, nt_store=nt_store)
    try:
        for unroll in (1, 2, 4):
            ctx.set_tuning(unroll=unroll)
            n = 8 * 4 * 40001                               # ragged last tile at every unroll
            ins = H.make_inputs(oracle, 8, n, 31 + unroll)
            got, _ = H.run_allreduce(ctx, "bisect", ins)
            H.assert_all_ranks_equal(oracle, got, oracle.bisect(ins), "unroll %d" % unroll)
    finally:
        ctx.set_tuning(nt_load=-1, nt_store=-1, unroll=-1)


@pytest.mark.parametrize("nranks", [2, 4, 8, 16])
def test_one_trip_grids_with_a_residency_cap(ctxs, oracle, nranks):
    """A one-trip grid (one tile per work-group) at every block size, vector count and
    residency cap, on sizes whose last tile is ragged, in place and out of place, and
    the all-gather through the same launch path."""
    ctx = ctxs[nranks]
    algo = "bisect" if nranks >= 4 else "simple"
    n = nranks * 4 * 20011
    ins = H.make_inputs(oracle, nranks, n, 9100 + nranks)
    want = H.expected(oracle, algo, ins)
    try:
        for block, unroll, cap, deal in ((64, 1, 4, 1), (256, 1, 2, 2), (512, 1, 2, nranks), (256, 2, 1, 1),
                                         (1024, 4, 1, 2), (128, 2, 8, nranks // 2), (256, 1, 0, 0)):
            ctx.set_tuning(oneshot=1, block=block, unroll=unroll, wgs_per_cu=cap, deal=deal)
            what = "N=%d block=%d unroll=%d cap=%d deal=%d" % (nranks, block, unroll, cap, deal)
            got, _ = H.run_allreduce(ctx, algo, ins)
            H.assert_all_ranks_equal(oracle, got, want, what)
            got, kept = H.run_allreduce(ctx, algo, ins, inplace=False, offset_bytes=8)
            H.assert_all_ranks_equal(oracle, got, want, what + " out of place, 8-byte aligned")
            for a, b in zip(kept, ins):
                assert (a == b).all(), what
        # chunks longer than a launch's segment: several one-trip launches per all-reduce, the last one ragged
        ctx.set_tuning(oneshot=1, block=64, unroll=1, wgs_per_cu=5, deal=1, segment_kib=16)
        got, _ = H.run_allreduce(ctx, algo, ins)
        H.assert_all_ranks_equal(oracle, got, want, "N=%d one-trip in 16 KiB segments" % nranks)
        ctx.set_tuning(segment_kib=-1)
        if nranks <= 8:
            ctx.set_tuning(oneshot=1, block=512, unroll=1, wgs_per_cu=2, deal=2)
            gin = H.make_inputs(oracle, nranks, 8 * 5003, 9200 + nranks, DIST_UNIFORM, -2.0, 2.0)
            gwant = oracle.allgather(gin)
            for alias in (False, True):
                got = run_allgather(ctx, "allgather_simple", gin, alias)
                for r in range(nranks):
                    assert (got[r] == gwant).all(), (nranks, r, alias)
    finally:
        ctx.set_tuning(oneshot=-1, block=-1, unroll=-1, wgs_per_cu=-1, deal=-1, segment_kib=-1)
    # chunk dealing of the persistent grid (which XCDs share a chunk)
    try:
        for deal in (1, 2, nranks):
            ctx.set_tuning(oneshot=0, deal=deal)
            got, _ = H.run_allreduce(ctx, algo, ins)
            H.assert_all_ranks_equal(oracle, got, want, "persistent grid, deal %d" % deal)
    finally:
        ctx.set_tuning(oneshot=-1, deal=-1)
    with pytest.raises(vr.VRError):
        ctx.set_tuning(wgs_per_cu=13)
    with pytest.raises(vr.VRError):
        ctx.set_tuning(deal=3)


@pytest.mark.parametrize("nranks,algo,mib", [(2, "simple", 128), (4, "bisect", 64), (4, "simple", 64),
                                             (4, "bisect", 128), (16, "bisect", 16), (16, "bisect", 32),
                                             (8, "simple", 40), (8, "bisect", 64), (8, "simple", 96)])
def test_streaming_shapes_of_other_rank_counts(ctxs, oracle, nranks, algo, mib):
    """Sizes at which 2, 4 and 16 ranks stream from HBM, where the library launches its
    one-trip grids by itself; out of place (nothing of it fits the memory-side cache)."""
    n = (mib << 20) // 2
    draw = 1 << 20
    ins = [np.tile(a, n // draw) for a in H.make_inputs(oracle, nranks, draw, 9300 + nranks, DIST_NORMAL, 0.0, 0.02)]
    want = H.expected(oracle, algo, ins)
    got, kept = H.run_allreduce(ctxs[nranks], algo, ins, inplace=False)
    assert oracle.count_mismatch(got[0], want) == 0, (nranks, algo)
    for r in range(1, nranks):
        assert oracle.count_mismatch(got[r], got[0]) == 0, (nranks, algo, r)
    for a, b in zip(kept, ins):
        assert (a == b).all()


def test_allgather_one_trip_sizes(ctxs, oracle):
    """All-gather shapes from 64 MiB of output on, where the library launches a one-trip
    grid (eight ranks: with a residency cap), own slot aliased or not."""
    for nranks, n in ((2, 1 << 24), (4, 1 << 22), (8, 1 << 21)):
        ins = H.make_inputs(oracle, nranks, n, 9400 + nranks, DIST_UNIFORM, -2.0, 2.0)
        want = oracle.allgather(ins)
        for alias in (False, True):
            got = run_allgather(ctxs[nranks], "allgather_simple", ins, alias)
            for r in range(nranks):
                assert (got[r] == want).all(), (nranks, r, alias)
    # Runs of consecutive tiles per XCD: forced on a slice whose tile count is no multiple of
    # the group of 8 * run work-groups (the ragged last group keeps its order) and on one
    # shorter than a group.
    ctx = ctxs[4]
    for algo, n in (("allgather_simple", 4 * 1024 * 37 + 8), ("allgather_small", 4 * 1024 * 37 + 24),
                    ("allgather_simple", 1024), ("allgather_simple", 2048 * 8 * 5)):
        ins = H.make_inputs(oracle, 4, n, 9500, DIST_UNIFORM, -2.0, 2.0)
        want = oracle.allgather(ins)
        for block, cap, run in ((64, 4, 2), (256, 4, 8), (128, 0, 256), (64, 8, 16)):
            ctx.set_tuning(oneshot=1, block=block, unroll=1, wgs_per_cu=cap, deal=1, run=run)
            for alias in (False, True):
                got = run_allgather(ctx, algo, ins, alias)
                for r in range(4):
                    assert (got[r] == want).all(), (n, block, cap, run, r, alias)
    ctx.set_tuning(oneshot=-1, block=-1, unroll=-1, wgs_per_cu=-1, deal=-1, run=-1)
    for bad in (3, 512, -2):
        with pytest.raises(vr.VRError):
            ctx.set_tuning(run=bad)


def test_nothing_is_written_past_the_end(ctxs, oracle):
    """The last tile of a chunk hangs over its end; the hardware bounds check of the
    buffer resource must drop those lanes (outputs carry 64 guard bytes here)."""
    from gpu_ipc_example_amd.binding import DeviceBuffer
    N, n = 8, 8 * 4 * 777
    ins = H.make_inputs(oracle, N, n, 5)
    src = H.RankBuffers(N, n)
    src.upload(ins)
    dst = [DeviceBuffer(n * 2 + 4096) for _ in range(N)]
    for d in dst:
        d.fill(0xAB)
    ctxs[N].allreduce("simple", src.ptrs, n, outs=[d.ptr for d in dst])
    ctxs[N].check()
    want = oracle.rotated(ins)
    for d in dst:
        assert oracle.count_mismatch(d.download(np.uint16, n), want) == 0
        assert (d.download(np.uint8, 4096, n * 2) == 0xAB).all()
        d.free()
    src.free()


def test_work_groups_are_dealt_round_robin_over_the_xcds(ctxs):
    """The rank-to-XCD affinity the direct kernels are laid out for: consecutive
    work-groups of a launch go to consecutive XCDs (starting wherever the previous
    launch stopped), so within a launch each XCD serves exactly one of 8 ranks."""
    for _ in range(3):
        ids = ctxs[8].xcc_ids(2048).astype(np.int64)
        assert ids.min() == 0 and ids.max() == 7
        assert (((ids - ids[0]) % 8) == np.arange(2048) % 8).all(), ids[:32]
