"""The allocation-free entry point (vr_allreduce_static): a wire-transport
all-reduce whose sinks live in a fixed region of device memory inside the
library's code object.  Checked bit for bit against the existing entry point
(vr_allreduce on the wire transport) on two calls in a row, the second smaller."""
import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from tests import vr_helpers as H

pytestmark = pytest.mark.gpu


def run_pair(oracle, nranks, algo, sizes, seed):
    ctx = vr.VirtualRanks(nranks)
    ctx.reserve_wire()
    for k, n in enumerate(sizes):
        ins = H.make_inputs(oracle, nranks, n, seed + 10 * k)
        # existing entry point, context-owned scratch
        ref = H.RankBuffers(nranks, n)
        ref.upload(ins)
        ctx.allreduce(algo, ref.ptrs, n, transport=vr.TRANSPORT_WIRE)
        ctx.check()
        want = ref.download()
        ref.free()
        # new entry point, in place and out of place
        src = H.RankBuffers(nranks, n)
        src.upload(ins)
        dst = H.RankBuffers(nranks, n)
        dst.fill(0xAB)
        ctx.allreduce_static(algo, src.ptrs, n, outs=dst.ptrs)
        ctx.allreduce_static(algo, src.ptrs, n)
        ctx.check()
        for r, (a, b, w) in enumerate(zip(src.download(), dst.download(), want)):
            assert oracle.count_mismatch(a, w) == 0, (algo, n, r, "in place")
            assert oracle.count_mismatch(b, w) == 0, (algo, n, r, "out of place")
        assert oracle.count_mismatch(want[0], H.expected(oracle, algo, ins)) == 0
        src.free()
        dst.free()
    ctx.close()


@pytest.mark.parametrize("algo", ["parallel", "small", "bisect", "simple_ring", "small_pcie"])
def test_two_calls_in_a_row_second_one_smaller(oracle, algo):
    run_pair(oracle, 8, algo, (64 * 30011, 64 * 129), 7100)


def test_other_rank_counts_share_the_region(oracle):
    run_pair(oracle, 4, "bisect", (1 << 20, 32 * 77), 7200)
    run_pair(oracle, 2, "simple", (1 << 18, 16), 7300)
    run_pair(oracle, 8, "parallel", (1 << 16, 64), 7400)


def test_limits_are_reported(oracle):
    ctx = vr.VirtualRanks(8)
    bufs = H.RankBuffers(8, 64)
    with pytest.raises(vr.VRError) as e:
        ctx.allreduce_static("parallel", bufs.ptrs, (256 << 20) // 2 + 64)
    assert e.value.code == "INVALID" and "bytes per rank" in e.value.detail
    with pytest.raises(vr.VRError) as e:
        ctx.allreduce_static("simple_transmit", bufs.ptrs, 64)
    assert e.value.code == "INVALID"
    ctx.close()
    ctx16 = vr.VirtualRanks(16)
    b16 = H.RankBuffers(16, 128)
    with pytest.raises(vr.VRError) as e:
        ctx16.allreduce_static("bisect", b16.ptrs, 128)
    assert e.value.code == "INVALID" and "ranks" in e.value.detail
    ctx16.close()
    bufs.free()
    b16.free()
