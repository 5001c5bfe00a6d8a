"""ctypes binding of the CPU oracle (oracle/libvr_oracle.so) for the tests.

The oracle is test infrastructure: only tests, the smoke check and the
benchmark's CPU-baseline leg load it.  Arrays cross the boundary as numpy
uint16 (binary16 bit patterns).
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
SO = os.path.join(ORACLE_DIR, "libvr_oracle.so")

DIST_UNIFORM, DIST_NORMAL = 0, 1
WIRE_RT64, WIRE_RT64_128, WIRE_RT64_PCIE, WIRE_RT64_128_PCIE = 0, 1, 2, 3
ORDER_RANK, ORDER_ROTATED, ORDER_BISECT = 0, 1, 2
F16, BF16 = 0, 1

_u16p = C.POINTER(C.c_uint16)


def _ptr(a):
    assert a.dtype == np.uint16 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_u16p)


def _ptr_array(arrs):
    return (_u16p * len(arrs))(*[_ptr(a) for a in arrs])


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        L = lib
        L.vro_f16_add_soft.restype = C.c_uint16
        L.vro_f16_add_soft.argtypes = [C.c_uint16, C.c_uint16]
        L.vro_f16_add.restype = C.c_uint16
        L.vro_f16_add.argtypes = [C.c_uint16, C.c_uint16]
        L.vro_f16_to_f32.restype = C.c_float
        L.vro_f16_to_f32.argtypes = [C.c_uint16]
        L.vro_f32_to_f16.restype = C.c_uint16
        L.vro_f32_to_f16.argtypes = [C.c_float]
        L.vro_f16_to_f32_soft.restype = C.c_float
        L.vro_f16_to_f32_soft.argtypes = [C.c_uint16]
        L.vro_f32_to_f16_soft.restype = C.c_uint16
        L.vro_f32_to_f16_soft.argtypes = [C.c_float]
        L.vro_f64_to_f16.restype = C.c_uint16
        L.vro_f64_to_f16.argtypes = [C.c_double]
        L.vro_selftest_add.restype = C.c_uint64
        L.vro_selftest_add.argtypes = [C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32)]
        L.vro_fill_pattern.restype = None
        L.vro_fill_pattern.argtypes = [_u16p, C.c_int, C.c_size_t]
        L.vro_generate.restype = None
        L.vro_generate.argtypes = [_u16p, C.c_size_t, C.c_uint64, C.c_int, C.c_double, C.c_double]
        L.vro_calc_work_size.restype = C.c_int
        L.vro_calc_work_size.argtypes = [C.c_size_t, C.c_size_t, C.c_int, C.c_size_t,
                                         C.POINTER(C.c_size_t)]
        for name in ("rank_order", "rotated", "bisect"):
            f = getattr(L, "vro_allreduce_" + name)
            f.restype = C.c_int
            f.argtypes = [_u16p, C.POINTER(_u16p), C.c_int, C.c_size_t]
        L.vro_allreduce_order_soft.restype = C.c_int
        L.vro_allreduce_order_soft.argtypes = [C.c_int, _u16p, C.POINTER(_u16p), C.c_int, C.c_size_t]
        L.vro_allgather.restype = None
        L.vro_allgather.argtypes = [_u16p, C.POINTER(_u16p), C.c_int, C.c_size_t]
        L.vro_count_mismatch.restype = C.c_size_t
        L.vro_count_mismatch.argtypes = [_u16p, _u16p, C.c_size_t]
        for name in ("parallel", "ring", "sequential"):
            f = getattr(L, "vro_emulate_" + name)
            f.restype = C.c_int
            f.argtypes = [C.POINTER(_u16p), C.c_int, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_uint32]
        L.vro_emulate_bisect.restype = C.c_int
        L.vro_emulate_bisect.argtypes = [C.POINTER(_u16p), C.c_int, C.c_size_t, C.c_int, C.c_int,
                                         C.c_uint32]
        L.vro_emulate_allgather_ring.restype = C.c_int
        L.vro_emulate_allgather_ring.argtypes = [C.POINTER(_u16p), C.POINTER(_u16p), C.c_int, C.c_size_t,
                                                 C.c_int, C.c_int, C.c_int, C.c_uint32]
        L.vro_bf16_add.restype = C.c_uint16
        L.vro_bf16_add.argtypes = [C.c_uint16, C.c_uint16]
        L.vro_f64_to_bf16.restype = C.c_uint16
        L.vro_f64_to_bf16.argtypes = [C.c_double]
        L.vro_fill_pattern_dt.restype = None
        L.vro_fill_pattern_dt.argtypes = [C.c_int, _u16p, C.c_int, C.c_size_t]
        L.vro_generate_dt.restype = None
        L.vro_generate_dt.argtypes = [C.c_int, _u16p, C.c_size_t, C.c_uint64, C.c_int, C.c_double,
                                      C.c_double]
        L.vro_allreduce_order_dt.restype = C.c_int
        L.vro_allreduce_order_dt.argtypes = [C.c_int, C.c_int, _u16p, C.POINTER(_u16p), C.c_int,
                                             C.c_size_t]
        L.vro_count_mismatch_dt.restype = C.c_size_t
        L.vro_count_mismatch_dt.argtypes = [C.c_int, _u16p, _u16p, C.c_size_t]
        L.vro_emulate_parallel_dt.restype = C.c_int
        L.vro_emulate_parallel_dt.argtypes = [C.c_int, C.POINTER(_u16p), C.c_int, C.c_size_t, C.c_int,
                                              C.c_int, C.c_int, C.c_uint32]
        L.vro_emulate_bisect_dt.restype = C.c_int
        L.vro_emulate_bisect_dt.argtypes = [C.c_int, C.POINTER(_u16p), C.c_int, C.c_size_t, C.c_int,
                                            C.c_int, C.c_uint32]
        _u32p = C.POINTER(C.c_uint32)
        L.vro_wire_payload_dwords.restype = C.c_int
        L.vro_wire_payload_dwords.argtypes = [C.c_int]
        L.vro_wire_message_dwords.restype = C.c_int
        L.vro_wire_message_dwords.argtypes = [C.c_int]
        L.vro_pack_message.restype = C.c_int
        L.vro_pack_message.argtypes = [C.c_int, _u32p, _u32p, C.c_uint32]
        L.vro_unpack_message.restype = C.c_int
        L.vro_unpack_message.argtypes = [C.c_int, _u32p, _u32p, C.c_uint32]
        L.vro_set_threads.restype = C.c_int
        L.vro_set_threads.argtypes = [C.c_int]

    # ---- scalars ---------------------------------------------------------
    def add_soft(self, a, b):
        return self.lib.vro_f16_add_soft(a, b)

    def add(self, a, b):
        return self.lib.vro_f16_add(a, b)

    # ---- data ------------------------------------------------------------
    def fill_pattern(self, rank, n):
        a = np.empty(n, np.uint16)
        self.lib.vro_fill_pattern(_ptr(a), rank, n)
        return a

    def generate(self, n, seed, dist, p0, p1):
        a = np.empty(n, np.uint16)
        self.lib.vro_generate(_ptr(a), n, seed, dist, p0, p1)
        return a

    def calc_work_size(self, addr, nbytes, nchunks, msg_bytes):
        w = C.c_size_t(0)
        rc = self.lib.vro_calc_work_size(addr, nbytes, nchunks, msg_bytes, C.byref(w))
        return rc, w.value

    # ---- orders ------------------------------------------------------------
    def _order(self, fn, ins):
        n = len(ins[0])
        out = np.empty(n, np.uint16)
        rc = fn(_ptr(out), _ptr_array(ins), len(ins), n)
        if rc:
            raise ValueError("oracle rejected the shape (rc=%d)" % rc)
        return out

    def rank_order(self, ins):
        return self._order(self.lib.vro_allreduce_rank_order, ins)

    def rotated(self, ins):
        return self._order(self.lib.vro_allreduce_rotated, ins)

    def bisect(self, ins):
        return self._order(self.lib.vro_allreduce_bisect, ins)

    def order_soft(self, mode, ins):
        n = len(ins[0])
        out = np.empty(n, np.uint16)
        rc = self.lib.vro_allreduce_order_soft(mode, _ptr(out), _ptr_array(ins), len(ins), n)
        if rc:
            raise ValueError("oracle rejected the shape (rc=%d)" % rc)
        return out

    def allgather(self, ins):
        n = len(ins[0])
        out = np.empty(n * len(ins), np.uint16)
        self.lib.vro_allgather(_ptr(out), _ptr_array(ins), len(ins), n)
        return out

    def count_mismatch(self, a, b):
        assert a.shape == b.shape
        return self.lib.vro_count_mismatch(_ptr(a), _ptr(b), a.size)

    # ---- either element type -----------------------------------------------
    def fill_pattern_dt(self, dtype, rank, n):
        a = np.empty(n, np.uint16)
        self.lib.vro_fill_pattern_dt(dtype, _ptr(a), rank, n)
        return a

    def generate_dt(self, dtype, n, seed, dist, p0, p1):
        a = np.empty(n, np.uint16)
        self.lib.vro_generate_dt(dtype, _ptr(a), n, seed, dist, p0, p1)
        return a

    def order_dt(self, dtype, mode, ins):
        n = len(ins[0])
        out = np.empty(n, np.uint16)
        rc = self.lib.vro_allreduce_order_dt(dtype, mode, _ptr(out), _ptr_array(ins), len(ins), n)
        if rc:
            raise ValueError("oracle rejected the shape (rc=%d)" % rc)
        return out

    def count_mismatch_dt(self, dtype, a, b):
        assert a.shape == b.shape
        return self.lib.vro_count_mismatch_dt(dtype, _ptr(a), _ptr(b), a.size)

    def emulate_parallel_dt(self, dtype, ins, wire, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_parallel_dt(dtype, _ptr_array(io), len(io), len(io[0]), wire, groups,
                                              subgroups, seq_no)
        return rc, io

    def emulate_bisect_dt(self, dtype, ins, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_bisect_dt(dtype, _ptr_array(io), len(io), len(io[0]), groups,
                                            subgroups, seq_no)
        return rc, io

    # ---- emulators (in place on copies) ----------------------------------
    def emulate_parallel(self, ins, wire, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_parallel(_ptr_array(io), len(io), len(io[0]), wire, groups,
                                           subgroups, seq_no)
        return rc, io

    def emulate_ring(self, ins, wire, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_ring(_ptr_array(io), len(io), len(io[0]), wire, groups,
                                       subgroups, seq_no)
        return rc, io

    def emulate_sequential(self, ins, wire, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_sequential(_ptr_array(io), len(io), len(io[0]), wire, groups,
                                             subgroups, seq_no)
        return rc, io

    def emulate_allgather_ring(self, ins, wire, groups, subgroups, seq_no=1, alias_own_slot=False):
        """Returns rc and the N output arrays (N * n halves each), pre-filled with 0x0101
        like main.cpp:300 does.  alias_own_slot: rank r's input is slot r of its output."""
        N, n = len(ins), len(ins[0])
        outs = [np.full(N * n, 0x0101, np.uint16) for _ in range(N)]
        srcs = []
        for r in range(N):
            if alias_own_slot:
                outs[r][r * n:(r + 1) * n] = ins[r]
                srcs.append(outs[r][r * n:(r + 1) * n])     # a view: same memory
            else:
                srcs.append(ins[r].copy())
        rc = self.lib.vro_emulate_allgather_ring(_ptr_array(outs), _ptr_array(srcs), N, n, wire, groups,
                                                 subgroups, seq_no)
        return rc, outs

    def emulate_bisect(self, ins, groups, subgroups, seq_no=1):
        io = [a.copy() for a in ins]
        rc = self.lib.vro_emulate_bisect(_ptr_array(io), len(io), len(io[0]), groups, subgroups,
                                         seq_no)
        return rc, io

    def wire_dwords(self, wire):
        """(payload dwords, message dwords) of one message of the wire format."""
        return self.lib.vro_wire_payload_dwords(wire), self.lib.vro_wire_message_dwords(wire)

    def pack_message(self, wire, payload, flag):
        cap, size = self.wire_dwords(wire)
        payload = np.ascontiguousarray(payload, np.uint32)
        assert len(payload) == cap
        msg = np.zeros(size, np.uint32)
        u32p = C.POINTER(C.c_uint32)
        rc = self.lib.vro_pack_message(wire, msg.ctypes.data_as(u32p), payload.ctypes.data_as(u32p), flag)
        assert rc == 0
        return msg

    def unpack_message(self, wire, msg, flag):
        cap, size = self.wire_dwords(wire)
        msg = np.ascontiguousarray(msg, np.uint32)
        assert len(msg) == size
        payload = np.zeros(cap, np.uint32)
        u32p = C.POINTER(C.c_uint32)
        rc = self.lib.vro_unpack_message(wire, msg.ctypes.data_as(u32p), payload.ctypes.data_as(u32p), flag)
        return rc, payload

    def set_threads(self, n):
        return self.lib.vro_set_threads(n)


_cached = None


def build():
    subprocess.run(["make", "-s", "-C", ORACLE_DIR], check=True)


def load():
    global _cached
    if _cached is None:
        if not os.path.exists(SO):
            build()
        _cached = Oracle(C.CDLL(SO))
    return _cached
