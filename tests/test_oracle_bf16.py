"""Pins the oracle's bfloat16 arithmetic and orders.  Independent checker:
torch.bfloat16 CPU arithmetic (float add, round to nearest even)."""
import numpy as np
import pytest
import torch

from tests.oracle_lib import BF16, DIST_NORMAL, DIST_UNIFORM, WIRE_RT64, WIRE_RT64_128


def tb(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def bits(t):
    return t.view(torch.int16).numpy().view(np.uint16)


def bf(x):
    return int(bits(torch.tensor([x], dtype=torch.bfloat16))[0])


@pytest.mark.parametrize("a,b,want", [
    (256.0, 1.0, 256.0),          # 8 significant bits: tie -> even (down)
    (256.0, 3.0, 260.0),          # tie -> even (up)
    (256.0, 2.0, 258.0),
    (1.0, -1.0, 0.0),
    (3.3895313892515355e38, 3.3895313892515355e38, float("inf")),   # max + max
    (1e-40, 1e-40, 2e-40),        # subnormals are kept
])
def test_add_known_answers(oracle, a, b, want):
    assert oracle.lib.vro_bf16_add(bf(a), bf(b)) == bf(want)
    assert oracle.lib.vro_bf16_add(bf(b), bf(a)) == bf(want)


def test_add_against_torch(oracle):
    rng = np.random.default_rng(5)
    n = 400000
    a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
    b[:50000] = a[:50000] ^ 0x8000 ^ rng.integers(0, 4, 50000).astype(np.uint16)   # near cancellation
    want = bits(tb(a) + tb(b))
    got = oracle.order_dt(BF16, 1, [a, b])             # one chunk pair: element-wise a + b
    assert oracle.count_mismatch_dt(BF16, got, want) == 0


def test_conversion_against_torch(oracle):
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-42, 39, 5000),
                        [0.0, -0.0, 1.0, 255.5, 256.5, 257.5, 3.4e38, 3.3961775292304601e38, 1e-45]])
    want = bits(torch.tensor(x, dtype=torch.float64).to(torch.bfloat16))
    for v, w in zip(x, want):
        f32 = np.float32(v)
        if float(f32) != v:      # torch rounds float64 -> bfloat16 in one step as well
            pass
        assert oracle.lib.vro_f64_to_bf16(float(v)) == int(w), v


def torch_rotated(ins):
    N, n = len(ins), len(ins[0])
    chunk = n // N
    f = [tb(a) for a in ins]
    out = torch.empty(n, dtype=torch.bfloat16)
    for c in range(N):
        sl = slice(c * chunk, (c + 1) * chunk)
        acc = f[c][sl].clone()
        for k in range(1, N):
            acc = f[(c + k) % N][sl] + acc
        out[sl] = acc
    return bits(out)


def torch_bisect(ins):
    N, n = len(ins), len(ins[0])
    B, chunk = N // 2, n // N
    f = [tb(a) for a in ins]
    out = torch.empty(n, dtype=torch.bfloat16)
    for owner in range(N):
        hh, l = owner & 1, owner // 2
        c = hh * B + l
        sl = slice(c * chunk, (c + 1) * chunk)
        pairs = [f[2 * j][sl] + f[2 * j + 1][sl] for j in range(B)]
        acc = pairs[l]
        for k in range(1, B):
            acc = pairs[(l + k) % B] + acc
        out[sl] = acc
    return bits(out)


@pytest.mark.parametrize("nranks", [2, 4, 8, 16])
def test_orders_against_torch(oracle, nranks):
    n = 16 * nranks * 41
    for scale in (0.02, 1.0, 1e4):
        ins = [oracle.generate_dt(BF16, n, 700 + r, DIST_NORMAL, 0.0, scale) for r in range(nranks)]
        assert oracle.count_mismatch_dt(BF16, oracle.order_dt(BF16, 1, ins), torch_rotated(ins)) == 0
        if nranks >= 4:
            assert oracle.count_mismatch_dt(BF16, oracle.order_dt(BF16, 2, ins), torch_bisect(ins)) == 0
        acc = torch.zeros(n, dtype=torch.bfloat16)
        for a in ins:
            acc = acc + tb(a)
        assert oracle.count_mismatch_dt(BF16, oracle.order_dt(BF16, 0, ins), bits(acc)) == 0


def test_kat_n8_three_way_bf16(oracle):
    # 256 + 1 ties down, (1 + 1) + 256 = 258: the same vector as the binary16 KAT, scaled
    ins = [np.full(128, bf(v), np.uint16) for v in (256, 0, 1, 0, 1, 0, 0, 0)]
    chunk = 16

    def per_chunk(out):
        return [float(tb(out[c * chunk:c * chunk + 1])[0]) for c in range(8)]

    assert per_chunk(oracle.order_dt(BF16, 2, ins)) == [256, 258, 256, 256, 256, 258, 256, 256]
    assert per_chunk(oracle.order_dt(BF16, 1, ins)) == [256, 258, 258, 256, 256, 256, 256, 256]
    assert per_chunk(oracle.order_dt(BF16, 0, ins)) == [256] * 8


def test_emulators_bf16(oracle):
    for nranks in (4, 8):
        n = 4 * nranks * 333
        ins = [oracle.generate_dt(BF16, n, 800 + r, DIST_NORMAL, 0.0, 1.0) for r in range(nranks)]
        for wire in (WIRE_RT64, WIRE_RT64_128):
            rc, io = oracle.emulate_parallel_dt(BF16, ins, wire, 4, nranks * 2, seq_no=9)
            assert rc == 0
            want = oracle.order_dt(BF16, 1, ins)
            assert all(oracle.count_mismatch_dt(BF16, a, want) == 0 for a in io)
        rc, io = oracle.emulate_bisect_dt(BF16, ins, 4, nranks, seq_no=9)
        assert rc == 0
        want = oracle.order_dt(BF16, 2, ins)
        assert all(oracle.count_mismatch_dt(BF16, a, want) == 0 for a in io)


def test_fill_pattern_bf16_closed_form(oracle):
    # (i % 32) * N(N+1)/2 <= 31 * 36 = 1116 is NOT always representable in 8 bits:
    # the rank-order chain rounds, so compare against the torch chain instead.
    for nranks in (2, 4, 8):
        ins = [oracle.fill_pattern_dt(BF16, r, 256) for r in range(nranks)]
        acc = torch.zeros(256, dtype=torch.bfloat16)
        for a in ins:
            acc = acc + tb(a)
        assert oracle.count_mismatch_dt(BF16, oracle.order_dt(BF16, 0, ins), bits(acc)) == 0
    assert (oracle.fill_pattern_dt(BF16, 1, 64)[:8] == [bf(2.0 * i) for i in range(8)]).all()


def test_host_generators_match_oracle_bf16(oracle):
    from gpu_ipc_example_amd import binding
    assert (binding.fill_pattern(3, 4096, binding.DTYPE_BF16) == oracle.fill_pattern_dt(BF16, 3, 4096)).all()
    for seed, dist, p0, p1 in ((1, DIST_NORMAL, 0.0, 1.0), (5, DIST_UNIFORM, -2.0, 2.0)):
        assert (binding.generate(30000, seed, dist, p0, p1, binding.DTYPE_BF16)
                == oracle.generate_dt(BF16, 30000, seed, dist, p0, p1)).all()
