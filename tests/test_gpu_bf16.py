"""GPU parity for the bfloat16 element type (the reference's other instantiated
type): direct and wire transports against the oracle's bfloat16 orders."""
import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from gpu_ipc_example_amd import binding
from gpu_ipc_example_amd.binding import DeviceBuffer
from tests.oracle_lib import BF16, DIST_NORMAL

pytestmark = pytest.mark.gpu

ALGOS = ("small", "simple", "bisect", "parallel", "small_ring", "simple_ring", "small_pcie",
         "simple_pcie")


def run(ctx, algo, ins, transport, inplace=True):
    n = len(ins[0])
    src = [DeviceBuffer(n * 2) for _ in ins]
    for b, a in zip(src, ins):
        b.upload(a)
    dst = None if inplace else [DeviceBuffer(n * 2) for _ in ins]
    ctx.allreduce(algo, [b.ptr for b in src], n, outs=[b.ptr for b in dst] if dst else None,
                  transport=transport)
    ctx.check()
    got = [b.download(np.uint16, n) for b in (dst or src)]
    for b in src + (dst or []):
        b.free()
    return got


@pytest.mark.parametrize("nranks", [2, 4, 8])
@pytest.mark.parametrize("transport", [vr.TRANSPORT_DIRECT, vr.TRANSPORT_WIRE])
def test_bf16_all_algos(oracle, nranks, transport):
    ctx = vr.VirtualRanks(nranks)
    ctx.set_dtype(binding.DTYPE_BF16)
    for algo in ALGOS:
        if algo == "bisect" and nranks < 4:
            continue
        for n in (8 * nranks, 8 * nranks * 129, 1 << 18):
            for scale in (0.02, 1.0, 3e4):
                ins = [oracle.generate_dt(BF16, n, 42 + r, DIST_NORMAL, 0.0, scale) for r in range(nranks)]
                want = oracle.order_dt(BF16, 2 if algo == "bisect" else 1, ins)
                for inplace in (True, False):
                    got = run(ctx, algo, ins, transport, inplace)
                    for r, g in enumerate(got):
                        assert oracle.count_mismatch_dt(BF16, g, want) == 0, (algo, n, scale, inplace, r)
    ctx.close()


def test_bf16_kat_and_special_values(oracle):
    import torch
    ctx = vr.VirtualRanks(8)
    ctx.set_dtype(binding.DTYPE_BF16)

    def bf(x):
        return int(torch.tensor([x], dtype=torch.bfloat16).view(torch.int16).item()) & 0xFFFF

    ins = [np.full(1024, bf(v), np.uint16) for v in (256, 0, 1, 0, 1, 0, 0, 0)]
    got = run(ctx, "bisect", ins, vr.TRANSPORT_DIRECT)
    want = oracle.order_dt(BF16, 2, ins)
    assert (got[0] == want).all() and got[0][128] == bf(258.0) and got[0][0] == bf(256.0)
    got = run(ctx, "simple", ins, vr.TRANSPORT_DIRECT)
    assert (got[3] == oracle.order_dt(BF16, 1, ins)).all() and got[3][2 * 128] == bf(258.0)
    # every exponent incl. subnormals; sums that overflow to infinity
    rng = np.random.default_rng(3)
    n = 8 * 4096
    ins = []
    for r in range(8):
        a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
        a[(a & 0x7F80) == 0x7F80] &= 0x807F
        ins.append(a)
    ins[0][:64] = 0x0001
    ins[1][:64] = 0x8001
    ins[2][64:128] = 0x7F7F
    ins[3][64:128] = 0x7F7F
    for algo in ("simple", "bisect"):
        for tr in (vr.TRANSPORT_DIRECT, vr.TRANSPORT_WIRE):
            got = run(ctx, algo, ins, tr)
            want = oracle.order_dt(BF16, 2 if algo == "bisect" else 1, ins)
            for g in got:
                assert oracle.count_mismatch_dt(BF16, g, want) == 0, (algo, tr)
    ctx.close()


def test_dtype_switch_on_one_context(oracle):
    ctx = vr.VirtualRanks(8)
    n = 1 << 14
    raw = [oracle.generate(n, 7 + r, DIST_NORMAL, 0.0, 1.0) for r in range(8)]
    ctx.set_dtype(binding.DTYPE_BF16)
    got = run(ctx, "simple", raw, vr.TRANSPORT_DIRECT)          # same bits read as bfloat16
    assert oracle.count_mismatch_dt(BF16, got[0], oracle.order_dt(BF16, 1, raw)) == 0
    ctx.set_dtype(binding.DTYPE_F16)
    got = run(ctx, "simple", raw, vr.TRANSPORT_DIRECT)
    assert oracle.count_mismatch(got[0], oracle.rotated(raw)) == 0
    with pytest.raises(vr.VRError):
        ctx.set_dtype(7)
    ctx.close()


@pytest.mark.parametrize("nranks", [2, 4, 8, 16])
def test_bf16_one_trip_grids_and_streaming_sizes(oracle, nranks):
    """The bfloat16 instantiation under the launches streaming sizes get: forced one-trip grids
    (residency cap, chunk dealing) on ragged sizes, then the library's own choice at 256 MiB of
    inputs, where it streams."""
    ctx = vr.VirtualRanks(nranks)
    ctx.set_dtype(binding.DTYPE_BF16)
    algos = ("bisect",) if nranks == 16 else ("simple",) if nranks == 2 else ("simple", "bisect")
    n = 8 * nranks * 4099
    ins = [oracle.generate_dt(BF16, n, 700 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
    for algo in algos:
        want = oracle.order_dt(BF16, 2 if algo == "bisect" else 1, ins)
        for block, cap, deal in ((64, 5, 1), (256, 2, 2), (128, 0, nranks)):
            ctx.set_tuning(oneshot=1, block=block, unroll=1, wgs_per_cu=cap, deal=deal)
            for inplace in (True, False):
                for r, g in enumerate(run(ctx, algo, ins, vr.TRANSPORT_DIRECT, inplace)):
                    assert oracle.count_mismatch_dt(BF16, g, want) == 0, (algo, block, cap, deal, inplace, r)
        ctx.set_tuning(oneshot=-1, block=-1, unroll=-1, wgs_per_cu=-1, deal=-1)
    n = (256 << 20) // 2 // nranks
    ins = [oracle.generate_dt(BF16, n, 900 + r, DIST_NORMAL, 0.0, 0.02) for r in range(nranks)]
    algo = algos[-1]
    want = oracle.order_dt(BF16, 2 if algo == "bisect" else 1, ins)
    for r, g in enumerate(run(ctx, algo, ins, vr.TRANSPORT_DIRECT, inplace=False)):
        assert oracle.count_mismatch_dt(BF16, g, want) == 0, (algo, "streaming", r)
    ctx.close()
