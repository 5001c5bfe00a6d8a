"""Byte layouts of the four wire formats in the oracle (pack_msg / unpack_msg),
pinned against a register-level model written from the reference's device code:
a message is SubGroupSize = 16 lanes of k dwords, held as k registers of 16 lanes
(component c of lane l = "register c, lane l", the %0(c, l) operands of the inline
assembly); lane l's components land at dwords l*k .. l*k+k-1 of the message.

  Rt64          rt64.hpp:335-341, 566-583   lane = {data, flag}
  Rt64_PCIE     rt64.hpp:3-20, 26-31        lane = {d0, d1, flag, flag}
  Rt64_128      rt64_128.hpp:563-583 (lanes 0..14 load), 640-658 (flags -> (1,7), (1,15)),
                724-731 (shuffle (0,15) <- (1,7)); dead verifier allreduce.cpp:71, 131-133
  Rt64_128_PCIE rt64_128.hpp:33-47 (lanes 0..14 load), 110-117 (flags -> (3,3), (3,7),
                (3,11), (3,15)), 194-203 (shuffle (0,15) <- (3,3), (1,15) <- (3,7),
                (2,15) <- (3,11))
"""
import numpy as np
import pytest

from tests.oracle_lib import WIRE_RT64, WIRE_RT64_128, WIRE_RT64_PCIE, WIRE_RT64_128_PCIE

FLAG = 0xE00F100F
SG = 16


def register_model(wire, payload, flag):
    """regs[c][l] after loadInput, shuffleData, insertFlags; returned lane-major."""
    k = {WIRE_RT64: 2, WIRE_RT64_128: 2, WIRE_RT64_PCIE: 4, WIRE_RT64_128_PCIE: 4}[wire]
    regs = np.zeros((k, SG), np.uint32)
    if wire == WIRE_RT64:                       # one data dword per lane, every lane
        regs[0, :] = payload
        regs[1, :] = flag
    elif wire == WIRE_RT64_PCIE:                # two data dwords per lane, every lane
        regs[0, :] = payload[0::2]
        regs[1, :] = payload[1::2]
        regs[2, :] = flag
        regs[3, :] = flag
    elif wire == WIRE_RT64_128:                 # lanes 0..14 load two dwords each
        for l in range(15):
            regs[0, l], regs[1, l] = payload[2 * l], payload[2 * l + 1]
        regs[0, 15] = regs[1, 7]                # shuffleData
        regs[1, 7] = flag                       # insertFlags
        regs[1, 15] = flag
    else:                                       # lanes 0..14 load four dwords each
        for l in range(15):
            regs[:, l] = payload[4 * l:4 * l + 4]
        regs[0, 15] = regs[3, 3]                # shuffleData
        regs[1, 15] = regs[3, 7]
        regs[2, 15] = regs[3, 11]
        for l in (3, 7, 11, 15):                # insertFlags
            regs[3, l] = flag
    return regs.T.reshape(-1).copy()            # lane l stores its k components contiguously


@pytest.mark.parametrize("wire,cap,size", [(WIRE_RT64, 16, 32), (WIRE_RT64_128, 30, 32),
                                           (WIRE_RT64_PCIE, 32, 64), (WIRE_RT64_128_PCIE, 60, 64)])
def test_pack_matches_the_register_model(oracle, wire, cap, size):
    assert oracle.wire_dwords(wire) == (cap, size)
    rng = np.random.default_rng(wire)
    for trial in range(20):
        payload = (np.arange(cap, dtype=np.uint32) + 1000 * (trial + 1)) if trial == 0 else \
            rng.integers(0, 2**32, cap, dtype=np.uint32)
        msg = oracle.pack_message(wire, payload, FLAG)
        assert np.array_equal(msg, register_model(wire, payload, FLAG))
        rc, back = oracle.unpack_message(wire, msg, FLAG)
        assert rc == 0 and np.array_equal(back, payload)


def test_rt64_128_matches_the_reference_stage_verifier(oracle):
    """allreduce.cpp:71, 131-133: temp[30] = temp[15]; temp[15] = flag; temp[31] = flag."""
    payload = np.arange(30, dtype=np.uint32) + 7
    temp = np.zeros(32, np.uint32)
    temp[:30] = payload
    temp[30] = temp[15]
    temp[15] = FLAG
    temp[31] = FLAG
    assert np.array_equal(oracle.pack_message(WIRE_RT64_128, payload, FLAG), temp)


def test_flag_positions_and_payload_fraction(oracle):
    """Where the flags sit, found by packing an all-zero payload: one per 64 bytes in
    the 128-byte families, every lane in the Rt64 families."""
    want = {WIRE_RT64: list(range(1, 32, 2)),
            WIRE_RT64_PCIE: [i for l in range(16) for i in (4 * l + 2, 4 * l + 3)],
            WIRE_RT64_128: [15, 31],
            WIRE_RT64_128_PCIE: [15, 31, 47, 63]}
    for wire, positions in want.items():
        cap, size = oracle.wire_dwords(wire)
        msg = oracle.pack_message(wire, np.zeros(cap, np.uint32), FLAG)
        assert list(np.nonzero(msg == FLAG)[0]) == positions
        assert cap + len(positions) == size or wire in (WIRE_RT64_128, WIRE_RT64_128_PCIE)
        # every flag position is checked by unpack
        for p in positions:
            bad = msg.copy()
            bad[p] ^= 1
            rc, _ = oracle.unpack_message(wire, bad, FLAG)
            assert rc == -1, (wire, p)
    # 93.75 % payload: 30 of 32 and 60 of 64 dwords
    assert oracle.wire_dwords(WIRE_RT64_128) == (30, 32) and oracle.wire_dwords(WIRE_RT64_128_PCIE) == (60, 64)


def test_displaced_dwords_are_parked_in_the_last_lane(oracle):
    payload = np.arange(60, dtype=np.uint32) + 100
    msg = oracle.pack_message(WIRE_RT64_128_PCIE, payload, FLAG)
    assert (msg[60], msg[61], msg[62]) == (payload[15], payload[31], payload[47])
    assert np.array_equal(np.delete(msg[:60], [15, 31, 47]), np.delete(payload, [15, 31, 47]))
    payload = np.arange(30, dtype=np.uint32) + 100
    msg = oracle.pack_message(WIRE_RT64_128, payload, FLAG)
    assert msg[30] == payload[15]
    assert np.array_equal(np.delete(msg[:30], [15]), np.delete(payload, [15]))
