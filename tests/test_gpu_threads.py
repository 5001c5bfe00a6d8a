"""One context per host thread: contexts created and used concurrently from
several threads (each on its own stream, direct transport) give the oracle's
bits.  ctypes releases the interpreter lock around every library call, so the
calls of different threads really interleave."""
import threading

import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from gpu_ipc_example_amd.binding import Stream
from tests import vr_helpers as H

pytestmark = pytest.mark.gpu

CASES = [(2, "small", 4096), (4, "simple", 30720), (8, "bisect", 131072), (8, "small_pcie_p", 65536)]


def test_contexts_on_four_threads(oracle):
    start = threading.Barrier(len(CASES))
    errors, results = [], {}

    def worker(k, nranks, algo, n):
        try:
            ins = H.make_inputs(oracle, nranks, n, 4200 + 17 * k)
            want = H.expected(oracle, algo, ins)
            start.wait(timeout=60)
            ctx = vr.VirtualRanks(nranks)          # created while the other threads create theirs
            stream = Stream()
            src = H.RankBuffers(nranks, n)
            dst = H.RankBuffers(nranks, n)
            src.upload(ins)
            bad = 0
            for it in range(25):
                dst.fill(0x5A)
                ctx.allreduce(algo, src.ptrs, n, outs=dst.ptrs, transport=vr.TRANSPORT_DIRECT,
                              stream=stream.handle)
                ctx.check(stream=stream.handle)
                for g in dst.download():
                    bad += oracle.count_mismatch(g, want)
            results[k] = bad
            src.free()
            dst.free()
            stream.close()
            ctx.close()
        except Exception as e:   # reported by the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,) + c) for k, c in enumerate(CASES)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors
    assert results == {k: 0 for k in range(len(CASES))}, results
