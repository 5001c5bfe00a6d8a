"""One process per rank on one GPU: every process owns its rank's input and
scratch, the processes exchange IPC handles over AF_UNIX sockets and map each
other's scratch (vr_ipc_open_all <- open_all_ipc_mems, ipc_exchange.cpp:277-311),
and each launches its own rank's wires (vr_allreduce_rank).  The reference's own
arrangement (mpirun -np N ./main), run through the CLI's --rank mode."""
import os
import subprocess

import numpy as np
import pytest

from tests import vr_helpers as H

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "gpu_ipc_example_amd", "vr_main")
_runs = [0]


def run_ranks(world, extra, per_rank=None, timeout=100, ranks_here=1):
    """Start one process per `ranks_here` ranks, wait for all; returns [(returncode, output)]."""
    _runs[0] += 1
    instance = "g%d_%d" % (os.getpid(), _runs[0])
    procs = []
    for r in range(0, world, ranks_here):
        cmd = [CLI, "-r", str(world), "--rank", str(r), "-i", instance] + extra + (per_rank(r) if per_rank else [])
        if ranks_here > 1:
            cmd += ["--ranks-here", str(ranks_here)]
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    out = []
    for p in procs:
        try:
            text, _ = p.communicate(timeout=timeout)
        except subprocess.TimeoutExpired:
            p.kill()                       # exactly the processes started here
            text, _ = p.communicate()
            text += "\n(killed after %d s)" % timeout
        out.append((p.returncode, text))
    return out


@pytest.mark.parametrize("world,algo", [(2, "simple"), (4, "simple"), (2, "small"), (4, "bisect"),
                                        (4, "parallel"), (2, "simple_ring"), (4, "small_pcie"),
                                        (8, "simple"), (8, "bisect")])
def test_fill_pattern_verify_across_processes(world, algo):
    """main.cpp's -v flow in every rank process: fill_pattern inputs, the host sum
    of allreduce.cpp:18-27 as the check."""
    for n in (16384, 14336 * 4):
        res = run_ranks(world, ["-v", "-n", str(n), "-a", algo])
        for r, (rc, text) in enumerate(res):
            assert rc == 0, (algo, n, r, text)
            assert "match the host sum" in text and "Error Compare" not in text, (algo, n, r, text)


@pytest.mark.parametrize("world,algo", [(2, "parallel"), (4, "parallel"), (4, "bisect"), (4, "simple_ring"),
                                        (2, "small"), (8, "parallel"), (8, "bisect")])
def test_seeded_inputs_match_the_oracle_across_processes(oracle, tmp_path, world, algo):
    n = 1 << 20
    seed = 9100 + world
    res = run_ranks(world, ["-n", str(n), "-a", algo, "--seed", str(seed)],
                    per_rank=lambda r: ["--dump", str(tmp_path / ("out%d.bin" % r))])
    for r, (rc, text) in enumerate(res):
        assert rc == 0, (algo, r, text)
    ins = H.make_inputs(oracle, world, n, seed)          # the same generator, rank r seeded with seed + r
    want = H.expected(oracle, algo, ins)
    for r in range(world):
        got = np.fromfile(tmp_path / ("out%d.bin" % r), np.uint16)
        assert len(got) == n and oracle.count_mismatch(got, want) == 0, (algo, r)


@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("algo", ["allgather_small", "allgather_simple"])
def test_allgather_across_processes(oracle, tmp_path, world, algo):
    """benchAllgather per process (main.cpp:110-166, 296-314): output memset to 1, -v
    through verifyAllgather; with and without the -g / -w grid; then seeded inputs
    whose dumped outputs are compared with the oracle's all-gather."""
    for grid in ([], ["-g", "7", "-w", "8"], ["-g", "19", "-w", "32", "-s", "32"]):
        for n in (16384, 14336 * 4):
            res = run_ranks(world, ["-v", "-n", str(n), "-a", algo] + grid)
            for r, (rc, text) in enumerate(res):
                assert rc == 0, (algo, n, grid, r, text)
                assert "gathered elements match" in text and "Error Compare" not in text, (algo, n, grid, r, text)
    n = 1 << 18
    seed = 9300 + world
    res = run_ranks(world, ["-n", str(n), "-a", algo, "--seed", str(seed), "-g", "13", "-w", "8"],
                    per_rank=lambda r: ["--dump", str(tmp_path / ("ag%d.bin" % r))])
    for r, (rc, text) in enumerate(res):
        assert rc == 0, (algo, r, text)
    want = oracle.allgather(H.make_inputs(oracle, world, n, seed))
    for r in range(world):
        got = np.fromfile(tmp_path / ("ag%d.bin" % r), np.uint16)
        assert len(got) == world * n and (got == want).all(), (algo, r)


def test_allgather_timed_run_across_processes():
    res = run_ranks(4, ["-n", "1M", "-a", "allgather_simple", "-g", "16", "-w", "16"])
    for r, (rc, text) in enumerate(res):
        assert rc == 0 and "[%d] Running time: " % r in text, (r, text)


@pytest.mark.parametrize("world,here,algo", [(8, 4, "parallel"), (8, 4, "bisect"), (8, 2, "simple"),
                                             (8, 4, "small_ring"), (4, 2, "simple_pcie"),
                                             (8, 4, "allgather_simple")])
def test_several_ranks_per_process(oracle, tmp_path, world, here, algo):
    """world / here processes, each holding `here` ranks in one launch
    (vr_allreduce_ranks / vr_allgather_ranks) against sinks mapped over IPC."""
    gather = algo.startswith("allgather")
    res = run_ranks(world, ["-v", "-n", "16384", "-a", algo], ranks_here=here)
    for p, (rc, text) in enumerate(res):
        assert rc == 0 and "Error Compare" not in text, (algo, p, text)
        for r in range(p * here, (p + 1) * here):
            assert "[%d] verify: " % r in text and "mismatches" not in text, (algo, r, text)
    n = 1 << 20
    seed = 9400 + world + here
    res = run_ranks(world, ["-n", str(n), "-a", algo, "--seed", str(seed)], ranks_here=here,
                    per_rank=lambda r: ["--dump", str(tmp_path / "grp.bin")])
    for p, (rc, text) in enumerate(res):
        assert rc == 0, (algo, p, text)
    ins = H.make_inputs(oracle, world, n, seed)
    want = oracle.allgather(ins) if gather else H.expected(oracle, algo, ins)
    for r in range(world):
        got = np.fromfile(str(tmp_path / "grp.bin") + ".%d" % r, np.uint16)
        assert len(got) == len(want) and oracle.count_mismatch(got, want) == 0, (algo, r)


def test_timed_run_protocol_across_processes():
    """Without -v: three warm-ups, a barrier, the timed run, one line per rank."""
    res = run_ranks(4, ["-n", "1M", "-a", "simple"])
    for r, (rc, text) in enumerate(res):
        assert rc == 0 and "[%d] Running time: " % r in text, (r, text)


def test_headline_shape_as_eight_processes():
    """8 rank processes, bisect, 32 MiB per rank: the reference's `mpirun -np 8 ./main
    -a bisect -n 16M` on one GPU, with the user grid of its test scripts."""
    res = run_ranks(8, ["-n", "16M", "-a", "bisect"])
    for r, (rc, text) in enumerate(res):
        assert rc == 0 and "[%d] Running time: " % r in text, (r, text)
    print("\n".join(text.strip().splitlines()[-1] for _, text in res))
    res = run_ranks(8, ["-v", "-n", "14336", "-a", "small", "-g", "7", "-w", "8"])
    for r, (rc, text) in enumerate(res):
        assert rc == 0 and "match the host sum" in text, (r, text)


def test_a_missing_rank_is_a_time_out_not_a_hang():
    """Rank 1 of 2 never starts: rank 0 gives up waiting for its record."""
    _runs[0] += 1
    p = subprocess.Popen([CLI, "-r", "2", "--rank", "0", "-i", "lone%d" % os.getpid(), "-v", "-n", "4096",
                          "-a", "simple"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         env=dict(os.environ, VRANK_IPC_TIMEOUT_MS="2000"))
    try:
        text, _ = p.communicate(timeout=60)
    except subprocess.TimeoutExpired:
        p.kill()
        text, _ = p.communicate()
        pytest.fail("rank 0 did not give up: " + text)
    assert p.returncode == 1 and "could not reach rank 1" in text, text
