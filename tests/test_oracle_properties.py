"""Property tests of the oracle (CPU): random shapes and launch geometries, the
closed-form orders against the message-level emulators, and algebraic facts
the arithmetic must satisfy."""
import numpy as np
from hypothesis import given, settings, strategies as st

from tests import oracle_lib
from tests.oracle_lib import WIRE_RT64, WIRE_RT64_128


def _ins(o, nranks, n, seed, scale):
    return [o.generate(n, seed + r, oracle_lib.DIST_NORMAL, 0.0, scale) for r in range(nranks)]


@settings(max_examples=60, deadline=None)
@given(nranks=st.sampled_from([2, 4, 8]), k=st.integers(1, 700), seed=st.integers(0, 2**31),
       scale=st.sampled_from([0.02, 1.0, 100.0, 20000.0]), wire=st.sampled_from([WIRE_RT64, WIRE_RT64_128]),
       cols=st.integers(1, 40), psg_mult=st.integers(1, 3))
def test_parallel_emulator_equals_rotated(nranks, k, seed, scale, wire, cols, psg_mult):
    o = oracle_lib.load()
    n = 4 * nranks * k
    ins = _ins(o, nranks, n, seed, scale)
    rc, io = o.emulate_parallel(ins, wire, cols, nranks * psg_mult, seq_no=seed | 1)
    assert rc == 0
    want = o.rotated(ins)
    assert all(o.count_mismatch(a, want) == 0 for a in io)


@settings(max_examples=40, deadline=None)
@given(nranks=st.sampled_from([4, 8, 16]), k=st.integers(1, 500), seed=st.integers(0, 2**31),
       scale=st.sampled_from([0.02, 1.0, 20000.0]), cols=st.integers(1, 30))
def test_bisect_emulator_equals_tree(nranks, k, seed, scale, cols):
    o = oracle_lib.load()
    n = 4 * nranks * k
    ins = _ins(o, nranks, n, seed, scale)
    rc, io = o.emulate_bisect(ins, cols, nranks // 2 * 2, seq_no=seed | 1)
    assert rc == 0
    want = o.bisect(ins)
    assert all(o.count_mismatch(a, want) == 0 for a in io)


@settings(max_examples=40, deadline=None)
@given(nranks=st.sampled_from([2, 4, 8]), k=st.integers(1, 500), seed=st.integers(0, 2**31),
       wires=st.integers(1, 60))
def test_ring_emulator_equals_rotated(nranks, k, seed, wires):
    o = oracle_lib.load()
    n = 8 * nranks * k
    ins = _ins(o, nranks, n, seed, 1.0)
    rc, io = o.emulate_ring(ins, WIRE_RT64_128, 1, wires, seq_no=seed | 1)
    assert rc == 0
    want = o.rotated(ins)
    assert all(o.count_mismatch(a, want) == 0 for a in io)


@settings(max_examples=200, deadline=None)
@given(a=st.integers(0, 0xFFFF), b=st.integers(0, 0xFFFF))
def test_add_commutes_and_negation_mirrors(a, b):
    o = oracle_lib.load()
    s = o.add_soft(a, b)
    assert o.lib.vro_f16_same(s, o.add_soft(b, a))
    # (-a) + (-b) == -(a + b) for everything that is not NaN
    m = o.add_soft(a ^ 0x8000, b ^ 0x8000)
    is_nan = (s & 0x7C00) == 0x7C00 and (s & 0x3FF)
    if not is_nan and s not in (0x0000,):      # exact cancellation gives +0 on both sides
        assert m == s ^ 0x8000


def test_rotating_the_ranks_rotates_the_chunks():
    """Renaming rank r -> r+1 (and moving chunk c's data to chunk c+1) must leave
    every rotated-order sum unchanged: the order depends on rank-minus-owner only."""
    o = oracle_lib.load()
    N, n = 8, 8 * 512
    ins = _ins(o, N, n, 99, 1.0)
    want = o.rotated(ins)
    chunk = n // N
    shifted = [np.roll(ins[(r - 1) % N], chunk) for r in range(N)]
    got = o.rotated(shifted)
    assert (np.roll(got, -chunk) == want).all()
