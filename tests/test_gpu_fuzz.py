"""Randomised parity sweep: random world size, protocol, transport, element
count, alignment, in/out-of-place choice and launch knobs (cache policy, unroll,
residency, block size, one-trip grids, their residency cap and chunk dealing, segment length, scatter run-ahead, wire format variant, streaming I/O),
each checked bit for bit against
the oracle.  Seeds are fixed, so a failure names a reproducible case."""
import random

import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from tests import vr_helpers as H

pytestmark = pytest.mark.gpu

ALGOS8 = ("small", "simple", "bisect", "parallel", "simple_transmit")
ALGOS16 = ("small_pcie_p", "simple_pcie_p", "small_ring", "simple_ring", "small_pcie", "simple_pcie")


@pytest.mark.parametrize("seed", range(6))
def test_random_cases(oracle, seed):
    rng = random.Random(1000 + seed)
    ctxs = {n: vr.VirtualRanks(n) for n in (2, 4, 8, 16)}
    for case in range(40):
        algo = rng.choice(ALGOS8 + ALGOS16)
        nranks = rng.choice((4, 8, 16) if algo == "bisect" else (2, 4, 8))
        msg_halves = 4 if algo in ALGOS8 else 8
        unit = msg_halves * nranks
        n = unit * rng.choice((1, 2, 3, 5, 17, 63, 64, 65, 257, 1000, 4099, 16384 // unit + 1,
                               rng.randrange(1, 40000)))
        transport = rng.choice((vr.TRANSPORT_DIRECT, vr.TRANSPORT_WIRE))
        inplace = rng.random() < 0.5
        offset = rng.choice((0, 0, 0, 16, 8 if msg_halves == 4 else 16, 32))
        grid = None
        if rng.random() < 0.4:
            grid = (rng.choice((1, 2, 3, 7, 16, 33, 64)), rng.choice((4, 8, 12, 32, 64)), rng.choice((16, 32)))
        knobs = dict(nt_load=rng.choice((-1, 0, 1)), nt_store=rng.choice((-1, 0, 1, 2)),
                     unroll=rng.choice((-1, 1, 2, 4)), segment_kib=rng.choice((-1, -1, 4, 64)),
                     waves_per_cu=rng.choice((-1, 1, 4, 32)), wire_ahead=rng.choice((-1, 1, 3, 6)),
                     wire_fenced=rng.choice((-1, -1, 0, 1, 2)), wire_stream_io=rng.choice((-1, 0, 1)),
                     wire_msg16=rng.choice((-1, 0, 1)), wire_cooperative=rng.choice((-1, -1, 1)))
        # (drawn from a generator of their own, so that the cases above stay what they were)
        rng2 = random.Random(77_000 * seed + case)
        knobs.update(oneshot=rng2.choice((-1, -1, 0, 1)), wgs_per_cu=rng2.choice((-1, 0, 1, 2, 4, 8)),
                     block=rng2.choice((-1, -1, 64, 256, 512, 1024)),
                     deal=rng2.choice((-1, -1, 0, 1, 2, nranks)))
        ctxs[nranks].set_tuning(**knobs)
        ins = H.make_inputs(oracle, nranks, n, 10_000 * seed + 37 * case,
                            p1=rng.choice((0.02, 1.0, 30.0, 3000.0)))
        what = "seed=%d case=%d %s N=%d n=%d transport=%d inplace=%s offset=%d grid=%s knobs=%s" % (
            seed, case, algo, nranks, n, transport, inplace, offset, grid, knobs)
        print(what, flush=True)
        got, kept = H.run_allreduce(ctxs[nranks], algo, ins, inplace=inplace, transport=transport,
                                    offset_bytes=offset, grid=grid)
        H.assert_all_ranks_equal(oracle, got, H.expected(oracle, algo, ins), what)
        if kept is not None:
            for a, b in zip(kept, ins):
                assert (a == b).all(), what
    for c in ctxs.values():
        c.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_allgather_cases(oracle, seed):
    """The all-gather under random launch shapes of the direct transport: one-trip or
    persistent grid, block size, residency cap, sources dealt at a time, tile runs per
    XCD, vectors per lane, own slot aliased or not."""
    from tests.test_gpu_direct import run_allgather
    from tests.oracle_lib import DIST_UNIFORM
    rng = random.Random(5000 + seed)
    ctxs = {n: vr.VirtualRanks(n) for n in (2, 4, 8)}
    for case in range(30):
        nranks = rng.choice((2, 4, 8))
        algo = rng.choice(("allgather_small", "allgather_simple"))
        n = 8 * rng.choice((1, 3, 17, 128, 129, 1000, 4099, 65536 // 8, rng.randrange(1, 60000)))
        alias = rng.random() < 0.4
        knobs = dict(oneshot=rng.choice((-1, 0, 1, 1)), block=rng.choice((-1, 64, 128, 256, 512, 1024)),
                     wgs_per_cu=rng.choice((-1, 0, 1, 3, 8, 12)), deal=rng.choice((-1, 0, 1, 1, 2, nranks)),
                     run=rng.choice((-1, 0, 1, 2, 8, 64, 256)), unroll=rng.choice((-1, 1, 2)),
                     segment_kib=rng.choice((-1, -1, 4, 64)), nt_load=rng.choice((-1, 0, 1)),
                     nt_store=rng.choice((-1, 0, 1, 2)))
        ctxs[nranks].set_tuning(**knobs)
        ins = H.make_inputs(oracle, nranks, n, 20_000 * seed + 41 * case, DIST_UNIFORM, -2.0, 2.0)
        what = "seed=%d case=%d %s N=%d n=%d alias=%s knobs=%s" % (seed, case, algo, nranks, n, alias, knobs)
        print(what, flush=True)
        want = oracle.allgather(ins)
        got = run_allgather(ctxs[nranks], algo, ins, alias)
        for r in range(nranks):
            assert (got[r] == want).all(), (what, r)
    for c in ctxs.values():
        c.close()
