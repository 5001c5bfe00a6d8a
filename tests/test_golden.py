"""The committed golden fixtures (tests/golden/*.npz, written by make_golden.py
from numpy.float16 / torch.bfloat16 arithmetic) against the oracle (CPU) and
against the HIP library through the C ABI (GPU)."""
import os

import numpy as np
import pytest

from tests.oracle_lib import BF16, F16

HERE = os.path.dirname(os.path.abspath(__file__))
MODES = {"rank_order": 0, "rotated": 1, "bisect": 2}


def load(name):
    return np.load(os.path.join(HERE, "golden", name), allow_pickle=False)


def cases(z):
    keys = sorted({k.rsplit("_in", 1)[0] for k in z.files if "_in" in k})
    for key in keys:
        N = int(key[1:].split("_")[0])
        ins = [np.ascontiguousarray(z["%s_in%d" % (key, r)]) for r in range(N)]
        outs = {o: z["%s_%s" % (key, o)] for o in MODES if "%s_%s" % (key, o) in z.files}
        yield key, N, ins, outs


@pytest.mark.parametrize("fname,dtype", [("orders_f16.npz", F16), ("orders_bf16.npz", BF16)])
def test_oracle_reproduces_the_golden_orders(oracle, fname, dtype):
    z = load(fname)
    seen = 0
    for key, N, ins, outs in cases(z):
        for oname, want in outs.items():
            got = oracle.order_dt(dtype, MODES[oname], ins)
            assert oracle.count_mismatch_dt(dtype, got, np.ascontiguousarray(want)) == 0, (key, oname)
            if dtype == F16:     # the fast float-route functions as well
                fast = {0: oracle.rank_order, 1: oracle.rotated, 2: oracle.bisect}[MODES[oname]](ins)
                assert oracle.count_mismatch(fast, np.ascontiguousarray(want)) == 0, (key, oname)
            seen += 1
    assert seen == 4 * 4 * 2 + 3 * 4      # rank+rotated for N=2..16, bisect for N=4..16, 4 data kinds


def test_oracle_reproduces_fill_pattern_sums(oracle):
    z = load("fill_pattern_f16.npz")
    for key in z.files:
        N, n = int(key[1:].split("_")[0]), int(key.split("_n")[1])
        ins = [oracle.fill_pattern(r, n) for r in range(N)]
        want = np.ascontiguousarray(z[key])
        assert (oracle.rank_order(ins) == want).all(), key
        assert (oracle.rotated(ins) == want).all(), key


@pytest.mark.gpu
@pytest.mark.parametrize("fname,dtype", [("orders_f16.npz", F16), ("orders_bf16.npz", BF16)])
def test_gpu_reproduces_the_golden_orders(oracle, fname, dtype):
    import gpu_ipc_example_amd as vr
    from gpu_ipc_example_amd.binding import DeviceBuffer
    z = load(fname)
    ctxs = {}
    for key, N, ins, outs in cases(z):
        if N not in ctxs:
            ctxs[N] = vr.VirtualRanks(N)
            ctxs[N].set_dtype(dtype)
        ctx = ctxs[N]
        n = len(ins[0])
        plans = []
        if N <= 8:
            plans += [(a, "rotated") for a in ("small", "simple", "parallel", "simple_ring", "small_pcie")]
        if N >= 4:
            plans.append(("bisect", "bisect"))
        for algo, oname in plans:
            want = np.ascontiguousarray(outs[oname])
            for transport in (vr.TRANSPORT_DIRECT, vr.TRANSPORT_WIRE):
                bufs = [DeviceBuffer(n * 2) for _ in range(N)]
                for b, a in zip(bufs, ins):
                    b.upload(a)
                ctx.allreduce(algo, [b.ptr for b in bufs], n, transport=transport)
                ctx.check()
                for r, b in enumerate(bufs):
                    got = b.download(np.uint16, n)
                    assert oracle.count_mismatch_dt(dtype, got, want) == 0, (key, algo, transport, r)
                    b.free()
    for c in ctxs.values():
        c.close()
