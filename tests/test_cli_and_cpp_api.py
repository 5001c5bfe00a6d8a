"""The C++ host API (include/vrank/allreduce.hpp) and the vr_main CLI.

CPU part: both build from the committed sources and reject bad arguments with
the reference's texts before touching a GPU.  GPU part: the C++ test program
checks every template against the oracle, and the CLI reproduces the
reference's -v sweep (test/test_8tile_shapes.sh) on fill_pattern inputs."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "gpu_ipc_example_amd", "vr_main")
CPP_TEST = os.path.join(ROOT, "tests", "cpp", "test_host_api")
GRAPH_TEST = os.path.join(ROOT, "tests", "cpp", "test_graph")
LAYOUT_TEST = os.path.join(ROOT, "tests", "cpp", "test_wire_layout")
VERIFY_TEST = os.path.join(ROOT, "tests", "cpp", "test_verify")


def run(cmd, **kw):
    return subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)


def test_cli_and_cpp_test_are_built():
    assert os.path.exists(CLI), "run __graft_entry__.build()"
    assert os.path.exists(CPP_TEST), "run make -C tests/cpp"


def test_wire_sinks_hold_every_slot_the_kernels_index():
    """CPU walk over every flow x rank count x wire count with the kernels' own
    slot functions: each message slot and flag word lies inside the sink."""
    r = run([LAYOUT_TEST], timeout=120)
    assert r.returncode == 0 and " 0 failures" in r.stdout, r.stdout


def test_host_side_checks_of_the_cpp_header():
    """vrank::verifyTransmit / verifyAllReduce / verifyAllgather (allreduce.cpp:519-585,
    832-838) and the element arithmetic under them, against the oracle; CPU only."""
    r = run([VERIFY_TEST], timeout=120)
    assert r.returncode == 0 and "verify ok" in r.stdout, r.stdout[-2000:]


def test_cli_rejects_bad_arguments_like_the_reference():
    r = run([CLI, "-n", "1K", "-a", "tree"])
    assert r.returncode == 1 and "Transmit type not support" in r.stdout
    r = run([CLI, "-n", "1K", "-a", "small", "-g", "4", "-w", "2"])
    assert r.returncode == 1 and "Subgroup numbers must be multiple of 4" in r.stdout
    r = run([CLI, "-n", "1K", "-a", "allgather_small", "-g", "4", "-w", "6"])     # all-gather takes the grid too
    assert r.returncode == 1 and "Subgroup numbers must be multiple of 4" in r.stdout
    r = run([CLI, "--help"])
    assert r.returncode == 0 and "usage" in r.stdout


def test_header_compiles_with_plain_gxx(tmp_path):
    src = tmp_path / "t.cpp"
    src.write_text(
        '#include "vrank/allreduce.hpp"\n'
        "using namespace vrank;\n"
        "static_assert(AllReduce<unsigned short, 8, Rt64, ParallelTransmit>::algo == VR_ALGO_SMALL, \"\");\n"
        "static_assert(AllReduce<unsigned short, 2, Rt64_128, ParallelTransmit>::algo == VR_ALGO_SIMPLE, \"\");\n"
        "static_assert(AllReduce<unsigned short, 8, Rt64_PCIE, RingTransmit>::algo == VR_ALGO_SMALL_RING, \"\");\n"
        "static_assert(AllReduce<unsigned short, 8, Rt64_128_PCIE, SequentialTransmit>::algo == VR_ALGO_SIMPLE_PCIE, \"\");\n"
        "static_assert(AllReduce<unsigned short, 2, Rt64_128, ParallelTransmit>::wireCapacity == 120, \"\");\n"
        "static_assert(bisectPAllReduce<unsigned short, 8>::BiNRanks == 4, \"\");\n"
        "static_assert(AllGather<unsigned short, 4, Rt64_PCIE>::algo == VR_ALGO_ALLGATHER_SMALL, \"\");\n"
        "int main() { return 0; }\n")
    r = run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I", os.path.join(ROOT, "include"), str(src)])
    assert r.returncode == 0, r.stdout


def test_c_abi_header_is_plain_c99_and_links_from_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 and a C program must
    link against the library and resolve the host-only entry points."""
    src = tmp_path / "t.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "vrank_allreduce.h"\n'
        "int main(void) {\n"
        "  int algo = -1; size_t work = 0; vr_geometry g;\n"
        '  if (vr_algo_from_string("bisect", &algo) != VR_OK || algo != VR_ALGO_BISECT) return 1;\n'
        "  const void *bufs[8]; for (int i = 0; i < 8; ++i) bufs[i] = (const void *)0x1000;\n"
        "  if (vr_check_allreduce(algo, 8, bufs, 16777216, &work) != VR_OK || work != 4194304) return 2;\n"
        "  if (vr_launch_geometry(algo, 8, 16777216, &g) != VR_OK || g.steps != 69) return 3;  /* allreduce.hpp:237-248: w = NRanks */\n"
        '  if (strcmp(vr_strerror(VR_ERR_UNEVEN), "We don\'t support non-even divide yet")) return 4;\n'
        '  puts("c ok"); return 0;\n}\n')
    exe = tmp_path / "t"
    lib_dir = os.path.join(ROOT, "gpu_ipc_example_amd")
    r = run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
             str(src), "-o", str(exe), "-L", lib_dir, "-lvrank_allreduce", "-Wl,-rpath," + lib_dir])
    assert r.returncode == 0, r.stdout
    r = run([str(exe)])
    assert r.returncode == 0 and "c ok" in r.stdout, (r.returncode, r.stdout)


@pytest.mark.gpu
def test_direct_transport_replays_correctly_from_a_hip_graph():
    """A captured small -> copy -> bisect sequence, replayed six times with eager
    work and synchronisation in between; every replay is compared with the oracle."""
    assert os.path.exists(GRAPH_TEST), "run make -C tests/cpp"
    r = run([GRAPH_TEST], timeout=120)
    assert r.returncode == 0 and "graph ok" in r.stdout, r.stdout


@pytest.mark.gpu
def test_cpp_host_api_against_oracle():
    r = run([CPP_TEST], timeout=120)
    assert r.returncode == 0 and "host API ok" in r.stdout, r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("world,algo", [(2, "small"), (4, "simple"), (8, "small"), (8, "simple"),
                                        (8, "bisect"), (4, "bisect"), (8, "small_ring"),
                                        (8, "simple_pcie"), (4, "allgather_small"),
                                        (8, "allgather_simple")])
def test_cli_verify_sweep(world, algo):
    """shapes x groups x sub-groups of test/test_8tile_shapes.sh, with the
    sub-group counts main.cpp:289-291 still accepts."""
    shapes = [128, 256, 384, 1280, 1920, 1024, 2048, 14336, 16384]
    msg = 8 if algo in ("small", "simple", "bisect") else 16
    for n in shapes:
        if not algo.startswith("allgather") and n % ((msg // 2) * world):
            continue
        for g, w in ((1, 4), (7, 8), (64, 64), (19, 32)):
            r = run([CLI, "-v", "-n", str(n), "-r", str(world), "-a", algo, "-g", str(g), "-w", str(w)],
                    timeout=60)
            assert r.returncode == 0, r.stdout
            assert "Error Compare" not in r.stdout and "match" in r.stdout, (n, g, w, r.stdout[-400:])


@pytest.mark.gpu
@pytest.mark.parametrize("transport", ["direct", "wire"])
def test_cli_allgather_honours_the_grid(transport):
    """-s is passed on for all-gather algos as for all-reduce ones: a sub-group size the
    dispatcher does not instantiate is rejected (allreduce.cpp:917), 16 and 32 run."""
    base = [CLI, "-v", "-n", "2048", "-r", "4", "-a", "allgather_simple", "-t", transport, "-g", "7", "-w", "8"]
    r = run(base + ["-s", "8"], timeout=60)
    assert r.returncode == 1 and "Unsupported Sub-group size" in r.stdout, r.stdout
    for simd in ("16", "32"):
        r = run(base + ["-s", simd], timeout=60)
        assert r.returncode == 0 and "gathered elements match" in r.stdout, r.stdout


@pytest.mark.gpu
def test_cli_timed_run_prints_the_reference_lines():
    r = run([CLI, "-n", "1M", "-r", "8", "-a", "bisect"], timeout=60)
    assert r.returncode == 0, r.stdout
    assert "---------last run------------------" in r.stdout
    for rank in range(8):
        assert "[%d] Running time: " % rank in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("world,algo", [(2, "small"), (2, "simple"), (2, "simple_ring"),
                                        (2, "small_pcie"), (8, "allgather_small"), (4, "allgather_simple")])
def test_cli_verify_bf16(world, algo):
    """main.cpp:45 builds the reference for bfloat16; the same -v flow here.  -v
    compares with the reference's rank-order host sum, which for bfloat16 only
    coincides with the device order while every partial sum of the pattern is
    exact in 8 bits or the world has two ranks; hence world 2 for the reductions."""
    for n in (2048, 16384):
        for t in ("direct", "wire"):
            r = run([CLI, "-v", "-n", str(n), "-r", str(world), "-a", algo, "--dtype", "bf16", "-t", t],
                    timeout=60)
            assert r.returncode == 0, r.stdout
            assert "Error Compare" not in r.stdout and "match" in r.stdout, (n, t, r.stdout[-300:])
