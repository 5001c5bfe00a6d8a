#!/usr/bin/env python3
"""Writes the golden fixtures in this directory.

Nothing here comes from the oracle or from the HIP library: inputs are drawn with
numpy's PCG64 (seeded), expected outputs are computed with numpy.float16 /
torch.bfloat16 element-wise adds, written out as explicit loops over chunks and
ranks in the summation orders the reference's kernels use

  rank order : ((0 + x0) + x1) + ...                        allreduce.cpp:18-27
  rotated    : chunk c starts at rank c, then c+1, c+2, ...  parallel_transmit.hpp:51-55,104-116
  bisect     : pair sums x_{2j} + x_{2j+1}, chunk c = h*N/2 + l chains pairs l, l+1, ...
                                                             bisect_transmit.hpp:347-424,462-477

plus the reference's own fixture, fill_pattern (utils.hpp:15-19), with its closed
form for binary16.  Files are .npz archives of plain uint16 arrays (bit patterns),
loadable with numpy.load(allow_pickle=False).

Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def add_f16(a, b):
    with np.errstate(all="ignore"):
        return (a.view(np.float16) + b.view(np.float16)).astype(np.float16).view(np.uint16)


def add_bf16(a, b):
    ta = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16)
    return (ta + tb).view(torch.int16).numpy().view(np.uint16)


def orders(ins, add):
    N, n = len(ins), len(ins[0])
    chunk = n // N
    rank = np.zeros(n, np.uint16)
    for x in ins:
        rank = add(rank, x)
    rot = np.empty(n, np.uint16)
    for c in range(N):
        sl = slice(c * chunk, (c + 1) * chunk)
        acc = ins[c][sl].copy()
        for k in range(1, N):
            acc = add(ins[(c + k) % N][sl], acc)
        rot[sl] = acc
    out = {"rank_order": rank, "rotated": rot}
    if N >= 4:
        B = N // 2
        bis = np.empty(n, np.uint16)
        for c in range(N):
            h, l = c // B, c % B
            sl = slice(c * chunk, (c + 1) * chunk)

            def pair(j):
                own = 2 * j + h
                return add(ins[own ^ 1][sl], ins[own][sl])

            acc = pair(l)
            for k in range(1, B):
                acc = add(pair((l + k) % B), acc)
            bis[sl] = acc
        out["bisect"] = bis
    return out


def draw(rng, n, kind, bf16):
    if kind == "all_exponents":
        a = rng.integers(0, 0x10000, n, dtype=np.uint32).astype(np.uint16)
        mask = 0x7F80 if bf16 else 0x7C00
        a[(a & mask) == mask] &= np.uint16(0x8000 | (0x007F if bf16 else 0x03FF))   # finite only
        return a
    x = rng.standard_normal(n) * {"n1": 1.0, "n002": 0.02, "big": 3.0e3}[kind]
    if bf16:
        return torch.tensor(x, dtype=torch.float64).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    with np.errstate(all="ignore"):
        return x.astype(np.float16).view(np.uint16)


def main():
    for name, add, bf16 in (("f16", add_f16, False), ("bf16", add_bf16, True)):
        rng = np.random.Generator(np.random.PCG64(20240611 if not bf16 else 20240612))
        arrays = {}
        for N in (2, 4, 8, 16):
            for kind in ("n1", "n002", "big", "all_exponents"):
                n = 8 * N * 3
                ins = [draw(rng, n, kind, bf16) for _ in range(N)]
                key = "N%d_%s" % (N, kind)
                for r, x in enumerate(ins):
                    arrays["%s_in%d" % (key, r)] = x
                for oname, o in orders(ins, add).items():
                    arrays["%s_%s" % (key, oname)] = o
        np.savez_compressed(os.path.join(HERE, "orders_%s.npz" % name), **arrays)
        print(name, len(arrays), "arrays")

    # fill_pattern: inputs (i % 32) * (rank + 1); binary16 sums are exact for N <= 8
    fp = {}
    for N in (2, 4, 8):
        for n in (128, 256, 384, 1280, 1920, 1024, 2048, 14336, 16384):   # test/test_2tile_shapes.sh:4
            fp["N%d_n%d" % (N, n)] = ((np.arange(n) % 32) * (N * (N + 1) // 2)).astype(np.float16).view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "fill_pattern_f16.npz"), **fp)
    print("fill_pattern", len(fp), "arrays")


if __name__ == "__main__":
    main()
