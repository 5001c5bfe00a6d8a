"""Host side of the inter-process exchange (no GPU): the AF_UNIX all-gather that
carries the ranks' records (un_allgather, ipc_exchange.cpp:173-265), exercised
through vr_ipc_barrier from several processes at once."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

WORKER = r"""
import ctypes, sys, time
L = ctypes.CDLL(sys.argv[1])
L.vr_ipc_barrier.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_char_p, ctypes.c_int]
L.vr_last_error_detail.restype = ctypes.c_char_p
rank, world, inst, delay = int(sys.argv[2]), int(sys.argv[3]), sys.argv[4].encode(), float(sys.argv[5])
time.sleep(delay * rank)                      # ranks arrive at different times
for gen in (1, 2, 3):
    t0 = time.time()
    rc = L.vr_ipc_barrier(rank, world, inst, gen)
    if rc:
        print("rank", rank, "gen", gen, "rc", rc, L.vr_last_error_detail().decode())
        sys.exit(1)
    print("rank %d gen %d left at %.3f" % (rank, gen, time.time()))
print("ok")
"""


def spawn(world, instance, delay):
    so = os.path.join(ROOT, "gpu_ipc_example_amd", "libvrank_allreduce.so")
    return [subprocess.Popen([sys.executable, "-c", WORKER, so, str(r), str(world), instance, str(delay)],
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            for r in range(world)]


def test_barrier_between_processes():
    for world, delay in ((2, 0.0), (4, 0.15), (8, 0.0)):
        procs = spawn(world, "cpu%d_%d" % (os.getpid(), world), delay)
        outs = []
        for p in procs:
            try:
                out, _ = p.communicate(timeout=60)
            except subprocess.TimeoutExpired:
                p.kill()
                out, _ = p.communicate()
            outs.append((p.returncode, out))
        for rc, out in outs:
            assert rc == 0 and out.strip().endswith("ok"), outs
        # nobody leaves barrier 1 before the last rank has arrived
        if delay:
            left = [float(l.split()[-1]) for _, out in outs for l in out.splitlines() if " gen 1 " in l]
            assert max(left) - min(left) < delay * (world - 1), left


def test_bad_arguments():
    import gpu_ipc_example_amd as vr
    L = vr.lib()
    assert L.vr_ipc_barrier(3, 2, b"x", 1) == 7
    assert L.vr_ipc_barrier(0, 1, b"x", 1) == 0          # a world of one has nobody to wait for
    assert L.vr_ipc_open_all(None, 0, 2, None, None, b"x") == 7
