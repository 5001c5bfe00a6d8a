import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: CPU test that takes tens of seconds")
    # Load what is built; compile (hipcc cross-compiles without a GPU) only when a
    # fresh checkout has nothing built yet.
    built = [os.path.join(ROOT, "gpu_ipc_example_amd", "libvrank_allreduce.so"),
             os.path.join(ROOT, "gpu_ipc_example_amd", "vr_main"),
             os.path.join(ROOT, "oracle", "libvr_oracle.so"),
             os.path.join(ROOT, "tests", "cpp", "test_host_api"),
             os.path.join(ROOT, "tests", "cpp", "test_graph"),
             os.path.join(ROOT, "tests", "cpp", "test_wire_layout"),
             os.path.join(ROOT, "tests", "cpp", "test_verify")]
    if not all(os.path.exists(p) for p in built):
        import __graft_entry__
        __graft_entry__.build()


@pytest.fixture(scope="session")
def oracle():
    from tests import oracle_lib

    return oracle_lib.load()
