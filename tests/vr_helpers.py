"""Shared plumbing for the GPU parity tests: upload seeded inputs, run the HIP
path through the C ABI, download, compare bit for bit with the oracle."""
import numpy as np

import gpu_ipc_example_amd as vr
from gpu_ipc_example_amd.binding import DeviceBuffer
from tests.oracle_lib import DIST_NORMAL, DIST_UNIFORM

ROTATED_ALGOS = ("small", "simple", "small_pcie_p", "simple_pcie_p", "small_ring", "simple_ring",
                 "small_pcie", "simple_pcie", "simple_transmit")


def make_inputs(oracle, nranks, n, seed, dist=DIST_NORMAL, p0=0.0, p1=1.0):
    return [oracle.generate(n, seed + r, dist, p0, p1) for r in range(nranks)]


def expected(oracle, algo, ins):
    return oracle.bisect(ins) if algo == "bisect" else oracle.rotated(ins)


class RankBuffers:
    """One device allocation per virtual rank (+ optional byte offset to test alignment)."""

    def __init__(self, nranks, n_halves, offset_bytes=0, slack=64):
        self.n, self.off = n_halves, offset_bytes
        self.bufs = [DeviceBuffer(n_halves * 2 + offset_bytes + slack) for _ in range(nranks)]

    @property
    def ptrs(self):
        return [b.ptr + self.off for b in self.bufs]

    def upload(self, arrays):
        for b, a in zip(self.bufs, arrays):
            b.upload(a, self.off)

    def download(self):
        return [b.download(np.uint16, self.n, self.off) for b in self.bufs]

    def fill(self, byte):
        for b in self.bufs:
            b.fill(byte)

    def free(self):
        for b in self.bufs:
            b.free()


def run_allreduce(ctx, algo, ins, inplace=True, transport=vr.TRANSPORT_DEFAULT, offset_bytes=0,
                  grid=None):
    n = len(ins[0])
    src = RankBuffers(ctx.nranks, n, offset_bytes)
    src.upload(ins)
    dst = None
    if not inplace:
        dst = RankBuffers(ctx.nranks, n, offset_bytes)
        dst.fill(0xAB)
    outs = dst.ptrs if dst else None
    if grid:
        ctx.allreduce_grid(algo, src.ptrs, n, grid[0], grid[1], grid[2] if len(grid) > 2 else 16,
                           outs=outs, transport=transport)
    else:
        ctx.allreduce(algo, src.ptrs, n, outs=outs, transport=transport)
    ctx.check()
    got = (dst or src).download()
    kept = src.download() if dst else None
    src.free()
    if dst:
        dst.free()
    return got, kept


def assert_all_ranks_equal(oracle, got, want, what=""):
    for r, g in enumerate(got):
        bad = oracle.count_mismatch(g, want)
        if bad:
            idx = int(np.nonzero(g != want)[0][0])
            raise AssertionError("%s rank %d: %d mismatches, first at %d: got %#06x want %#06x"
                                 % (what, r, bad, idx, int(g[idx]), int(want[idx])))
