"""bench.py contract checks that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_bytes_match_the_metric_definition():
    sys.path.insert(0, ROOT)
    import bench
    assert bench.algorithmic_bytes("cfg3") == 2 * 8 * 32 * 2**20          # 2*N*S
    assert bench.algorithmic_bytes("cfg2") == 2 * 8 * 2**20
    assert bench.algorithmic_bytes("cfg4") == 4 * 8 * 2**20 + 4 * 4 * 8 * 2**20   # N*S + N*N*S
    assert bench.WORKLOADS["cfg3"][:3] == (8, "bisect", 16777216)
    assert bench.WORKLOADS["cfg2"][:3] == (8, "small", 524288)
    assert bench.WORKLOADS["cfg4"][:3] == (4, "allgather_simple", 4194304)


def test_measured_traffic_constants_are_the_numbers_in_the_profiles():
    """roofline.traffic is a constant copied from a counter run: the summary under
    profiles/ it names must state exactly that number."""
    sys.path.insert(0, ROOT)
    import bench
    assert bench.MEASURED_TRAFFIC_BYTES
    for (workload, transport), (nbytes, fname) in bench.MEASURED_TRAFFIC_BYTES.items():
        assert workload in bench.WORKLOADS and transport in ("direct", "wire")
        text = open(os.path.join(ROOT, "profiles", fname)).read()
        assert "{:,} B".format(nbytes) in text, (workload, transport, nbytes, fname)
    assert bench.measured_traffic("cfg3", "default") == bench.MEASURED_TRAFFIC_BYTES[("cfg3", "direct")][0]
    assert bench.measured_traffic("cfg3", "wire") == bench.MEASURED_TRAFFIC_BYTES.get(("cfg3", "wire"), (None,))[0]


def test_default_line_carries_the_fixed_sample_and_the_other_configurations():
    """The driver's one line must hold: a kernel-time sample whose size does not depend
    on --steps, the in-place figure on cold sets, config 4, config 5 at three sizes
    and the latency figures measured on the C side.  Checked on the source, so that
    no GPU is needed: every key is one the default path writes."""
    sys.path.insert(0, ROOT)
    import bench
    assert bench.KERNEL_SAMPLE_LAUNCHES >= 200 and bench.KERNEL_SAMPLE_MIN_PAIRS >= 20
    src = open(os.path.join(ROOT, "bench.py")).read()
    for key in ("kernel_us_min", "kernel_us_p50", "kernel_us_p99", "n_pairs", "in_place_cold",
                "cfg4_allgather", "cfg5_sweep_points", "latency_1MiB_per_rank", "host_call_us",
                "back_to_back_us_per_launch", "kernel_trace_p50_us", "same_buffers_cache_warm",
                "hbm_ceilings", "cpu_baseline", "roofline", "inputs_cache_resident", "buffer_sets_rotated",
                "memory_clock", "device_state", "launch"):
        assert '"%s"' % key in src, key
    us, fname = bench.CFG2_KERNEL_TRACE
    text = open(os.path.join(ROOT, "profiles", fname)).read()
    assert ("%.2f" % us) in text, (us, fname)


def test_tiled_inputs_are_the_same_on_both_sides():
    """Workloads above 16 Mi elements per rank repeat a 16 Mi-element draw; the GPU side
    (setup) and the CPU side (cpu_leg) must build the same arrays."""
    sys.path.insert(0, ROOT)
    import bench
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert src.count("min(ne, 1 << 24)") == 2


def test_rotating_sets_keep_the_inputs_out_of_the_memory_side_cache():
    """Streaming stores do not displace cached inputs, so a workload's inputs alone, over all the sets
    its steps rotate through, must exceed the 256 MiB cache: config 4's block rotates 16 sets
    (512 MiB of inputs) and the default set count of every workload is raised alike."""
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert 'setup(vr, binding, name, False, 16)' in src
    assert "(512 << 20) // (n * ne * 2)" in src
