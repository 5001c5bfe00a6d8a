"""CPU-side tests of the C ABI: the library loads, exports what the header
declares, and the host-only entry points (validation, geometry, parsers,
generators) behave like the reference's host code.  No GPU call is made."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import gpu_ipc_example_amd as vr
from gpu_ipc_example_amd import binding
from tests.oracle_lib import DIST_NORMAL, DIST_UNIFORM

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "vrank_allreduce.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(vr_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 30
    L = C.CDLL(vr.library_path())
    missing = [s for s in sorted(declared) if not hasattr(L, s)]
    assert not missing, missing
    # the Python binding wraps exactly the declared set
    assert set(vr.lib()._signatures) == declared


def test_algo_strings():
    for i, name in enumerate(vr.ALGOS):
        assert vr.algo_id(name) == i
        assert vr.lib().vr_algo_name(i).decode() == name
    with pytest.raises(vr.VRError) as e:
        vr.algo_id("tree")
    assert e.value.code == "ALGO" and e.value.message == "Transmit type not support"
    assert vr.lib().vr_algo_message_bytes(vr.algo_id("small")) == 8
    assert vr.lib().vr_algo_message_bytes(vr.algo_id("simple_ring")) == 16
    assert vr.lib().vr_algo_is_allgather(vr.algo_id("allgather_small")) == 1
    assert vr.algo_id("simple_transmit") == 12 and vr.launch_geometry("simple_transmit", 2, 16384) == (3, 64, 1)


def test_error_texts_are_the_reference_ones():
    L = vr.lib()
    assert L.vr_strerror(1) == b"We only support aligned pointer for now"      # allreduce.hpp:111
    assert L.vr_strerror(2) == b"We don't support non-even divide yet"         # allreduce.hpp:118
    assert L.vr_strerror(3) == b"Transmit type not support"                    # allreduce.cpp:1187
    assert L.vr_strerror(4) == b"Unsupported communication topology"           # allreduce.cpp:880
    assert L.vr_strerror(5) == b"Unsupported Sub-group size"                   # allreduce.cpp:917
    assert L.vr_strerror(6) == b"Subgroup numbers must be multiple of 4"       # main.cpp:290


@pytest.mark.parametrize("algo,msg", [("small", 8), ("simple", 8), ("bisect", 8), ("simple_ring", 16)])
def test_calc_work_size_matches_oracle(oracle, algo, msg):
    nranks = 4 if algo == "bisect" else 2
    base = 0x7F0000001000
    for nelems in (0, 4, 8, 16, 24, 100, 128, 1000, 16384, 16388, 1 << 20):
        for off in (0, 4, 8, 16):
            ptrs = [base + off] * nranks
            rc_o, work_o = oracle.calc_work_size(base + off, nelems * 2, nranks, msg)
            try:
                work = vr.check_allreduce(algo, nranks, ptrs, nelems)
                rc = 0
            except vr.VRError as e:
                rc, work = e.status, None
            assert rc == rc_o, (nelems, off)
            if rc == 0:
                assert work == work_o


def test_unaligned_is_reported_before_uneven():
    with pytest.raises(vr.VRError) as e:
        vr.check_allreduce("small", 2, [0x1004, 0x1000], 7)
    assert e.value.code == "UNALIGNED"
    with pytest.raises(vr.VRError) as e:
        vr.check_allreduce("small", 2, [0x1000, 0x1000], 7)
    assert e.value.code == "UNEVEN"


def test_topology_rules():
    for n in (3, 5, 16):
        with pytest.raises(vr.VRError) as e:
            vr.check_allreduce("small", n, [0x1000] * n, 64 * n)
        assert e.value.code == "TOPOLOGY"
    with pytest.raises(vr.VRError) as e:
        vr.check_allreduce("bisect", 2, [0x1000] * 2, 64)
    assert e.value.code == "TOPOLOGY"
    assert vr.check_allreduce("bisect", 16, [0x1000] * 16, 64 * 16) == 128


def test_absurd_sizes_are_rejected_before_any_arithmetic_overflows():
    with pytest.raises(vr.VRError) as e:
        vr.check_allreduce("small", 8, [0x1000] * 8, (1 << 62) + 32)
    assert e.value.code == "INVALID"


def test_launch_geometry_matches_getLaunchParam():
    # worked by hand from allreduce.hpp:37-62 with PVC constants
    assert vr.launch_geometry("simple", 2, 16384) == (5, 64, 1)       # 137 wires of 120 B, 32 per SS
    assert vr.launch_geometry("small", 8, 524288) == (64, 64, 4)      # 2048 wires of 64 B, 8 per SS
    assert vr.launch_geometry("small", 2, 128) == (1, 64, 1)
    assert vr.launch_geometry("bisect", 8, 16777216) == (64, 64, 69)  # 34953 wires, w = NRanks
    assert vr.launch_geometry("small_ring", 8, 524288) == (16, 64, 1) # 1024 wires of 128 B, 64 per SS
    assert vr.launch_geometry("allgather_small", 4, 4194304) == (64, 64, 16)  # 65536 wires


def test_parse_nelems_like_main_cpp():
    assert vr.parse_nelems("8MB") == 8 * 1024 * 1024
    assert vr.parse_nelems("64K") == 65536
    assert vr.parse_nelems("2G") == 2 << 30
    assert vr.parse_nelems("16384") == 16384
    with pytest.raises(vr.VRError):
        vr.parse_nelems("MB")


def test_host_generators_match_oracle_bit_for_bit(oracle):
    for rank in (0, 1, 7):
        assert (binding.fill_pattern(rank, 4096) == oracle.fill_pattern(rank, 4096)).all()
    for seed, dist, p0, p1 in ((1, DIST_NORMAL, 0.0, 1.0), (9, DIST_NORMAL, 0.0, 0.02),
                               (5, DIST_UNIFORM, -1.0, 1.0), (6, DIST_UNIFORM, -2.0, 2.0)):
        assert (binding.generate(50000, seed, dist, p0, p1) == oracle.generate(50000, seed, dist, p0, p1)).all()


def test_no_device_is_a_clean_error():
    if binding.device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(vr.VRError) as e:
        vr.VirtualRanks(8)
    assert e.value.code == "NO_DEVICE"


def test_launch_plans_of_the_direct_transport():
    """The launches the library picks by itself, as its documentation states them (pure host
    arithmetic behind vr_direct_launch_plan)."""
    MiB = 1 << 20
    plan = vr.direct_launch_plan
    # the headline shape: one-trip grid of one-wave work-groups, five per CU, one chunk at a time,
    # streaming loads, streaming stores written through, adds through binary32; in place alike
    for in_place in (False, True):
        p = plan("bisect", 8, 16 * MiB, in_place)
        assert (p["one_trip"], p["block"], p["unroll"], p["wgs_per_cu"], p["deal"]) == (1, 64, 1, 5, 1)
        assert (p["nt_load"], p["nt_store"], p["f16_wide"]) == (1, 2, 1)
    # other rank counts when streaming
    p = plan("bisect", 4, 32 * MiB, True)
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["deal"], p["f16_wide"]) == (1, 64, 8, 1, 1)
    p = plan("simple", 2, 64 * MiB, True)
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["f16_wide"]) == (1, 512, 2, 0)
    assert (plan("bisect", 16, 8 * MiB, True)["deal"], plan("bisect", 16, 16 * MiB, True)["deal"]) == (2, 1)
    assert plan("bisect", 16, 8 * MiB, True)["wgs_per_cu"] == 4
    # eight ranks: six work-groups per CU for chunks of 16 to 32 MiB
    assert [plan("bisect", 8, n * MiB // 2, True)["wgs_per_cu"] for n in (64, 128, 256, 512)] == [5, 6, 6, 5]
    # everything fits the memory-side cache: persistent grid, cacheable loads, streaming stores
    p = plan("simple", 8, 4 * MiB, True)
    assert (p["one_trip"], p["waves_per_cu"], p["deal"], p["nt_load"], p["nt_store"], p["f16_wide"]) == (0, 4, 8, 0, 1, 0)
    assert plan("simple", 4, 4 * MiB, True)["waves_per_cu"] == 8
    # four ranks, in place, from 96 MiB in all: the one-trip grid with the cacheable policy
    p = plan("bisect", 4, 12 * MiB, True)
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["deal"], p["nt_load"], p["nt_store"]) == (1, 64, 8, 1, 0, 1)
    assert plan("bisect", 4, 11 * MiB, True)["one_trip"] == 0 and plan("bisect", 4, 12 * MiB, False)["one_trip"] == 0
    assert plan("bisect", 8, 6 * MiB, True)["one_trip"] == 0 and plan("simple", 2, 24 * MiB, True)["one_trip"] == 0
    # an in-place footprint of exactly the cache's size streams; one element less does not
    assert plan("bisect", 8, 16 * MiB, True)["nt_load"] == 1 and plan("bisect", 8, 16 * MiB - 64, True)["nt_load"] == 0
    # out of place: inputs about the size of the L2s -> results written through; inputs up to half
    # the cache with a footprint beyond it -> cached loads, results streamed past them
    assert plan("simple", 8, 2 * MiB, False)["nt_store"] == 2 and plan("simple", 8, 1 * MiB, False)["nt_store"] == 1
    p = plan("bisect", 8, 8 * MiB, False)
    assert (p["one_trip"], p["nt_load"], p["nt_store"]) == (0, 0, 2)
    # the latency family: one trip per lane, everything cacheable, up to the size of the cache
    p = plan("small", 8, MiB // 2, True)
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["nt_load"], p["nt_store"]) == (1, 256, 0, 0, 0)
    assert plan("small", 8, 16 * MiB, True)["nt_load"] == 1
    # all-gather: persistent below 32 MiB of output, capped one-trip launches from there on, tile
    # runs (one contiguous eighth of a slice per XCD) up to 32 MiB of inputs
    p = plan("allgather_simple", 4, MiB // 2, False)
    assert (p["one_trip"], p["waves_per_cu"], p["nt_load"], p["nt_store"]) == (0, 32, 0, 2)
    p = plan("allgather_simple", 4, 4 * MiB, False)                     # config 4
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["deal"], p["run"]) == (1, 256, 4, 1, 256)
    p = plan("allgather_simple", 8, 2 * MiB, False)
    assert (p["block"], p["wgs_per_cu"], p["deal"], p["run"]) == (256, 3, 1, 128)
    p = plan("allgather_simple", 8, 8 * MiB, False)
    assert (p["block"], p["wgs_per_cu"], p["deal"], p["run"]) == (128, 6, 1, 1)
    p = plan("allgather_simple", 2, 8 * MiB, False)
    assert (p["one_trip"], p["block"], p["wgs_per_cu"], p["run"]) == (1, 512, 3, 1)
    assert plan("allgather_simple", 4, 16 * MiB, False)["run"] == 1
    with pytest.raises(vr.VRError):
        plan("bisect", 3, 1024, True)
