"""ctypes binding of libvrank_allreduce.so (the C ABI in include/vrank_allreduce.h).

No fallback exists: if the shared library is missing or a call fails, an
exception is raised.  Device buffers are plain integers (device addresses), so
callers may hand in ``torch.Tensor.data_ptr()`` values or use the library's own
vr_malloc plumbing through :class:`DeviceBuffer`.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvrank_allreduce.so")

ALGOS = ("small", "simple", "bisect", "parallel", "small_pcie_p", "simple_pcie_p", "small_ring",
         "simple_ring", "small_pcie", "simple_pcie", "allgather_small", "allgather_simple",
         "simple_transmit")
TRANSPORT_DEFAULT, TRANSPORT_DIRECT, TRANSPORT_WIRE = 0, 1, 2

# vr_status -> Python exception class; the texts come from vr_strerror.
STATUS_NAMES = {
    1: "UNALIGNED", 2: "UNEVEN", 3: "ALGO", 4: "TOPOLOGY", 5: "SUBGROUP", 6: "GEOMETRY",
    7: "INVALID", 8: "HIP", 9: "NO_DEVICE", 10: "TIMEOUT", 11: "OVERLAP",
}


class VRError(RuntimeError):
    def __init__(self, status, message, detail):
        super().__init__("%s (%s)" % (message, detail) if detail else message)
        self.status = status
        self.code = STATUS_NAMES.get(status, str(status))
        self.message = message
        self.detail = detail


class Geometry(C.Structure):
    _fields_ = [("groups", C.c_uint32), ("subgroups", C.c_uint32), ("steps", C.c_uint32)]


class LaunchPlan(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("one_trip", "block", "unroll", "waves_per_cu", "wgs_per_cu", "deal", "run",
                                       "nt_load", "nt_store", "f16_wide")]


def library_path():
    return _SO


def build_library(force=False):
    """Compile the gfx950 library in-tree with hipcc (works without a GPU)."""
    args = ["make", "-s", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    if force:
        subprocess.run(args + ["clean"], check=True)
    subprocess.run(args, check=True)


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise ImportError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C gpu_ipc_example_amd/csrc`" % _SO)
    L = C.CDLL(_SO)
    vp, vpp, sz, u32, i = C.c_void_p, C.POINTER(C.c_void_p), C.c_size_t, C.c_uint32, C.c_int
    sig = {
        "vr_ctx_create": (i, [i, i, vpp]),
        "vr_ctx_destroy": (i, [vp]),
        "vr_ctx_reserve_wire": (i, [vp]),
        "vr_ctx_nranks": (i, [vp]),
        "vr_allreduce_rank": (i, [vp, vp, i, i, vp, vp, vp, vp, vpp, vpp, sz, sz, C.POINTER(u32)]),
        "vr_allgather_rank": (i, [vp, vp, i, i, vp, vp, vp, vp, vpp, vpp, sz, sz, C.POINTER(u32)]),
        "vr_allreduce_rank_grid": (i, [vp, vp, i, i, vp, vp, vp, vp, vpp, vpp, sz, sz, u32, u32, u32, u32]),
        "vr_allgather_rank_grid": (i, [vp, vp, i, i, vp, vp, vp, vp, vpp, vpp, sz, sz, u32, u32, u32, u32]),
        "vr_allreduce_ranks": (i, [vp, vp, i, i, i, vpp, vpp, vpp, vpp, sz, sz, C.POINTER(u32)]),
        "vr_allgather_ranks": (i, [vp, vp, i, i, i, vpp, vpp, vpp, vpp, sz, sz, C.POINTER(u32)]),
        "vr_allgather_grid": (i, [vp, vp, i, i, vpp, vpp, sz, u32, u32, u32, u32]),
        "vr_time_allreduce_grouped": (i, [vp, vp, i, i, vpp, vpp, sz, i, i, C.POINTER(C.c_float),
                                          C.POINTER(C.c_double)]),
        "vr_rank_flags_used": (i, [vp, i, sz, u32, u32, C.POINTER(u32)]),
        "vr_rank_scratch_bytes": (i, [vp, C.POINTER(sz)]),
        "vr_allreduce_static": (i, [vp, vp, i, vpp, vpp, sz]),
        "vr_ctx_set_dtype": (i, [vp, i]),
        "vr_ctx_get_dtype": (i, [vp]),
        "vr_fill_pattern_dt": (None, [i, C.POINTER(C.c_uint16), i, sz]),
        "vr_generate_dt": (None, [i, C.POINTER(C.c_uint16), sz, C.c_uint64, i, C.c_double, C.c_double]),
        "vr_algo_from_string": (i, [C.c_char_p, C.POINTER(i)]),
        "vr_algo_name": (C.c_char_p, [i]),
        "vr_algo_is_allgather": (i, [i]),
        "vr_algo_message_bytes": (sz, [i]),
        "vr_check_allreduce": (i, [i, i, vpp, sz, C.POINTER(sz)]),
        "vr_check_allgather": (i, [i, i, vpp, vpp, sz, C.POINTER(sz)]),
        "vr_launch_geometry": (i, [i, i, sz, C.POINTER(Geometry)]),
        "vr_allreduce": (i, [vp, vp, i, i, vpp, vpp, sz, C.POINTER(u32)]),
        "vr_allgather": (i, [vp, vp, i, i, vpp, vpp, sz, C.POINTER(u32)]),
        "vr_allreduce_grid": (i, [vp, vp, i, i, vpp, vpp, sz, u32, u32, u32, u32]),
        "vr_ctx_check": (i, [vp, vp]),
        "vr_ctx_set_spin_limit": (i, [vp, C.c_uint64]),
        "vr_direct_launch_plan": (i, [i, i, sz, i, C.POINTER(LaunchPlan)]),
        "vr_ctx_set_tuning": (i, [vp, C.c_char_p, i]),
        "vr_ctx_get_tuning": (i, [vp, C.c_char_p, C.POINTER(i)]),
        "vr_time_allreduce": (i, [vp, vp, i, i, vpp, vpp, sz, i, C.POINTER(C.c_float)]),
        "vr_time_allgather": (i, [vp, vp, i, i, vpp, vpp, sz, i, C.POINTER(C.c_float)]),
        "vr_time_allreduce_kernel": (i, [vp, vp, i, i, vpp, vpp, sz, i, C.POINTER(C.c_float)]),
        "vr_time_allgather_kernel": (i, [vp, vp, i, i, vpp, vpp, sz, i, C.POINTER(C.c_float)]),
        "vr_time_copy": (i, [vp, vp, vp, vp, sz, i, C.POINTER(C.c_float)]),
        "vr_stream_probe": (i, [vp, vp, i, vp, vp, sz]),
        "vr_stream_probe_multi": (i, [vp, vp, vpp, vpp, sz]),
        "vr_ipc_open_all": (i, [vp, i, i, vpp, C.POINTER(sz), C.c_char_p]),
        "vr_ipc_close_all": (i, [i, i, vpp]),
        "vr_ipc_barrier": (i, [i, i, C.c_char_p, i]),
        "vr_probe_xcc_ids": (i, [vp, u32, C.POINTER(u32)]),
        "vr_fill_pattern": (None, [C.POINTER(C.c_uint16), i, sz]),
        "vr_generate": (None, [C.POINTER(C.c_uint16), sz, C.c_uint64, i, C.c_double, C.c_double]),
        "vr_parse_nelems": (i, [C.c_char_p, C.POINTER(sz)]),
        "vr_device_count": (i, [C.POINTER(i)]),
        "vr_device_name": (i, [i, C.c_char_p, sz]),
        "vr_malloc": (i, [i, sz, vpp]),
        "vr_free": (i, [vp]),
        "vr_memset": (i, [vp, i, sz]),
        "vr_copy_to_device": (i, [vp, vp, sz]),
        "vr_copy_to_host": (i, [vp, vp, sz]),
        "vr_stream_create": (i, [i, vpp]),
        "vr_stream_destroy": (i, [vp]),
        "vr_stream_sync": (i, [vp]),
        "vr_event_create": (i, [vpp]),
        "vr_event_record": (i, [vp, vp]),
        "vr_event_elapsed_ms": (i, [vp, vp, C.POINTER(C.c_float)]),
        "vr_event_destroy": (i, [vp]),
        "vr_strerror": (C.c_char_p, [i]),
        "vr_last_error_detail": (C.c_char_p, []),
        "vr_version": (C.c_char_p, []),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)          # AttributeError here = header and library disagree
        f.restype, f.argtypes = res, args
    L._signatures = sig
    _lib = L
    return L


def _check(status):
    if status != 0:
        L = lib()
        raise VRError(status, L.vr_strerror(status).decode(), L.vr_last_error_detail().decode())


def algo_id(name):
    out = C.c_int(-1)
    _check(lib().vr_algo_from_string(name.encode(), C.byref(out)))
    return out.value


def parse_nelems(text):
    out = C.c_size_t(0)
    _check(lib().vr_parse_nelems(text.encode(), C.byref(out)))
    return out.value


def _table(ptrs):
    return (C.c_void_p * len(ptrs))(*[C.c_void_p(int(p)) for p in ptrs])


def check_allreduce(algo, nranks, ptrs, nelems):
    work = C.c_size_t(0)
    _check(lib().vr_check_allreduce(algo_id(algo), nranks, _table(ptrs), nelems, C.byref(work)))
    return work.value


def launch_geometry(algo, nranks, nelems):
    g = Geometry()
    _check(lib().vr_launch_geometry(algo_id(algo), nranks, nelems, C.byref(g)))
    return g.groups, g.subgroups, g.steps


def direct_launch_plan(algo, nranks, nelems, in_place=True):
    """The launch the direct transport picks for this shape (a dict; no GPU needed)."""
    p = LaunchPlan()
    _check(lib().vr_direct_launch_plan(algo_id(algo), nranks, nelems, int(in_place), C.byref(p)))
    return {k: getattr(p, k) for k, _ in LaunchPlan._fields_}


DTYPE_F16, DTYPE_BF16 = 0, 1


def fill_pattern(rank, n, dtype=DTYPE_F16):
    a = np.empty(n, np.uint16)
    lib().vr_fill_pattern_dt(dtype, a.ctypes.data_as(C.POINTER(C.c_uint16)), rank, n)
    return a


def generate(n, seed, dist, p0, p1, dtype=DTYPE_F16):
    a = np.empty(n, np.uint16)
    lib().vr_generate_dt(dtype, a.ctypes.data_as(C.POINTER(C.c_uint16)), n, seed, dist, p0, p1)
    return a


def device_count():
    n = C.c_int(0)
    _check(lib().vr_device_count(C.byref(n)))
    return n.value


def device_name(device=0):
    buf = C.create_string_buffer(256)
    _check(lib().vr_device_name(device, buf, 256))
    return buf.value.decode()


class DeviceBuffer:
    """A vr_malloc'ed region; `.ptr` is the device address."""

    def __init__(self, nbytes, device=0):
        p = C.c_void_p()
        _check(lib().vr_malloc(device, nbytes, C.byref(p)))
        self.ptr, self.nbytes = p.value, nbytes

    def upload(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes
        _check(lib().vr_copy_to_device(C.c_void_p(self.ptr + offset), arr.ctypes.data_as(C.c_void_p),
                                       arr.nbytes))

    def download(self, dtype=np.uint16, count=None, offset=0):
        item = np.dtype(dtype).itemsize
        if count is None:
            count = (self.nbytes - offset) // item
        out = np.empty(count, dtype)
        _check(lib().vr_copy_to_host(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr + offset),
                                     out.nbytes))
        return out

    def fill(self, byte):
        _check(lib().vr_memset(C.c_void_p(self.ptr), byte, self.nbytes))

    def free(self):
        if self.ptr:
            _check(lib().vr_free(C.c_void_p(self.ptr)))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class VirtualRanks:
    """N virtual ranks on one GPU: the handle every collective call goes through."""

    def __init__(self, nranks, device=0):
        h = C.c_void_p()
        _check(lib().vr_ctx_create(device, nranks, C.byref(h)))
        self._h, self.nranks, self.device = h, nranks, device
        self.seq_no = C.c_uint32(1)

    def close(self):
        if self._h:
            lib().vr_ctx_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_dtype(self, dtype):
        _check(lib().vr_ctx_set_dtype(self._h, dtype))

    def reserve_wire(self):
        """Allocate and zero the wire transport's scratch (idempotent)."""
        _check(lib().vr_ctx_reserve_wire(self._h))

    def _reserve_for(self, algo, transport):
        # The C ABI never allocates inside a collective call; this wrapper reserves
        # the scratch on the first call that will take the wire transport.
        if transport == TRANSPORT_WIRE or (transport == TRANSPORT_DEFAULT and algo == "parallel"):
            self.reserve_wire()

    def rank_scratch_bytes(self):
        out = C.c_size_t(0)
        _check(lib().vr_rank_scratch_bytes(self._h, C.byref(out)))
        return out.value

    def rank_flags_used(self, algo, nelems, groups=0, subgroups=0):
        out = C.c_uint32(0)
        _check(lib().vr_rank_flags_used(self._h, algo_id(algo), nelems, groups, subgroups, C.byref(out)))
        return out.value

    def allreduce_rank(self, algo, rank, inp, scatter, gather, peers0, peers1, sink_bytes, nelems,
                       seq_no, out=None, stream=None):
        """One rank's wires against caller-owned sinks; returns the advanced sequence number."""
        seq = C.c_uint32(seq_no)
        _check(lib().vr_allreduce_rank(self._h, stream, algo_id(algo), rank, C.c_void_p(int(inp)),
                                       C.c_void_p(int(out)) if out else None,
                                       C.c_void_p(int(scatter)), C.c_void_p(int(gather)),
                                       _table(peers0), _table(peers1), sink_bytes, nelems,
                                       C.byref(seq)))
        return seq.value

    def allreduce_rank_grid(self, algo, rank, inp, scatter, gather, peers0, peers1, sink_bytes, nelems,
                            seq_no, groups, subgroups, simd=16, out=None, stream=None):
        _check(lib().vr_allreduce_rank_grid(self._h, stream, algo_id(algo), rank, C.c_void_p(int(inp)),
                                            C.c_void_p(int(out)) if out else None,
                                            C.c_void_p(int(scatter)), C.c_void_p(int(gather)),
                                            _table(peers0), _table(peers1), sink_bytes, nelems, seq_no,
                                            groups, subgroups, simd))

    def allgather_rank(self, algo, rank, inp, out, scatter, gather, peers0, peers1, sink_bytes, nelems,
                       seq_no, stream=None):
        """One rank of the ring all-gather against caller-owned sinks."""
        seq = C.c_uint32(seq_no)
        _check(lib().vr_allgather_rank(self._h, stream, algo_id(algo), rank, C.c_void_p(int(inp)),
                                       C.c_void_p(int(out)), C.c_void_p(int(scatter)),
                                       C.c_void_p(int(gather)), _table(peers0), _table(peers1),
                                       sink_bytes, nelems, C.byref(seq)))
        return seq.value

    def allgather_rank_grid(self, algo, rank, inp, out, scatter, gather, peers0, peers1, sink_bytes, nelems,
                            seq_no, groups, subgroups, simd=16, stream=None):
        _check(lib().vr_allgather_rank_grid(self._h, stream, algo_id(algo), rank, C.c_void_p(int(inp)),
                                            C.c_void_p(int(out)), C.c_void_p(int(scatter)),
                                            C.c_void_p(int(gather)), _table(peers0), _table(peers1),
                                            sink_bytes, nelems, seq_no, groups, subgroups, simd))

    def allreduce_ranks(self, algo, first, inputs, peers0, peers1, sink_bytes, nelems, seq_no, outs=None,
                        stream=None):
        """Ranks [first, first + len(inputs)) in one launch; returns the advanced sequence number."""
        seq = C.c_uint32(seq_no)
        _check(lib().vr_allreduce_ranks(self._h, stream, algo_id(algo), first, len(inputs), _table(inputs),
                                        _table(outs) if outs is not None else None, _table(peers0),
                                        _table(peers1), sink_bytes, nelems, C.byref(seq)))
        return seq.value

    def allgather_ranks(self, algo, first, inputs, outputs, peers0, peers1, sink_bytes, nelems, seq_no,
                        stream=None):
        seq = C.c_uint32(seq_no)
        _check(lib().vr_allgather_ranks(self._h, stream, algo_id(algo), first, len(inputs), _table(inputs),
                                        _table(outputs), _table(peers0), _table(peers1), sink_bytes,
                                        nelems, C.byref(seq)))
        return seq.value

    def allreduce_static(self, algo, bufs, nelems, outs=None, stream=None):
        """Wire-transport all-reduce through the library's fixed scratch region (no allocation)."""
        _check(lib().vr_allreduce_static(self._h, stream, algo_id(algo), _table(bufs),
                                         _table(outs) if outs is not None else None, nelems))

    def set_tuning(self, **kw):
        for k, v in kw.items():
            _check(lib().vr_ctx_set_tuning(self._h, k.encode(), int(v)))

    def get_tuning(self, key):
        v = C.c_int(0)
        _check(lib().vr_ctx_get_tuning(self._h, key.encode(), C.byref(v)))
        return v.value

    def set_spin_limit(self, polls):
        _check(lib().vr_ctx_set_spin_limit(self._h, polls))

    def allreduce(self, algo, bufs, nelems, outs=None, transport=TRANSPORT_DEFAULT, stream=None):
        assert len(bufs) == self.nranks
        self._reserve_for(algo, transport)
        _check(lib().vr_allreduce(self._h, stream, algo_id(algo), transport, _table(bufs),
                                  _table(outs) if outs is not None else None, nelems,
                                  C.byref(self.seq_no)))

    def allreduce_grid(self, algo, bufs, nelems, groups, subgroups, simd=16, outs=None,
                       transport=TRANSPORT_DEFAULT, stream=None, seq_no=0xE00F100F):
        self._reserve_for(algo, transport)
        _check(lib().vr_allreduce_grid(self._h, stream, algo_id(algo), transport, _table(bufs),
                                       _table(outs) if outs is not None else None, nelems, seq_no,
                                       groups, subgroups, simd))

    def allgather(self, algo, inputs, outputs, nelems, transport=TRANSPORT_DEFAULT, stream=None):
        self._reserve_for(algo, transport)
        _check(lib().vr_allgather(self._h, stream, algo_id(algo), transport, _table(inputs),
                                  _table(outputs), nelems, C.byref(self.seq_no)))

    def allgather_grid(self, algo, inputs, outputs, nelems, groups, subgroups, simd=16,
                       transport=TRANSPORT_DEFAULT, stream=None, seq_no=0xE00F100F):
        self._reserve_for(algo, transport)
        _check(lib().vr_allgather_grid(self._h, stream, algo_id(algo), transport, _table(inputs),
                                       _table(outputs), nelems, seq_no, groups, subgroups, simd))

    def check(self, stream=None):
        _check(lib().vr_ctx_check(self._h, stream))

    def sync(self, stream=None):
        _check(lib().vr_stream_sync(stream))

    def time_allreduce(self, algo, bufs, nelems, iters, outs=None, transport=TRANSPORT_DEFAULT,
                       stream=None):
        ms = (C.c_float * iters)()
        self._reserve_for(algo, transport)
        _check(lib().vr_time_allreduce(self._h, stream, algo_id(algo), transport, _table(bufs),
                                       _table(outs) if outs is not None else None, nelems, iters, ms))
        return np.frombuffer(ms, np.float32).copy()

    def time_allreduce_kernel(self, algo, bufs, nelems, iters, outs=None, transport=TRANSPORT_DEFAULT,
                              stream=None):
        """Kernel execution time of each launch (ms), from events attached to the dispatches."""
        ms = (C.c_float * iters)()
        self._reserve_for(algo, transport)
        _check(lib().vr_time_allreduce_kernel(self._h, stream, algo_id(algo), transport, _table(bufs),
                                              _table(outs) if outs is not None else None, nelems, iters, ms))
        return np.frombuffer(ms, np.float32).copy()

    def time_allgather_kernel(self, algo, inputs, outputs, nelems, iters, transport=TRANSPORT_DEFAULT,
                              stream=None):
        ms = (C.c_float * iters)()
        self._reserve_for(algo, transport)
        _check(lib().vr_time_allgather_kernel(self._h, stream, algo_id(algo), transport, _table(inputs),
                                              _table(outputs), nelems, iters, ms))
        return np.frombuffer(ms, np.float32).copy()

    def time_allreduce_grouped(self, algo, bufs, nelems, groups, per_group, outs=None,
                               transport=TRANSPORT_DEFAULT, stream=None):
        """(ms per launch for each group, host microseconds one vr_allreduce call takes), both
        measured inside the library around calls made like any caller's."""
        ms = (C.c_float * groups)()
        host_us = C.c_double(0.0)
        self._reserve_for(algo, transport)
        _check(lib().vr_time_allreduce_grouped(self._h, stream, algo_id(algo), transport, _table(bufs),
                                               _table(outs) if outs is not None else None, nelems,
                                               groups, per_group, ms, C.byref(host_us)))
        return np.frombuffer(ms, np.float32).copy(), host_us.value

    def time_allgather(self, algo, inputs, outputs, nelems, iters, transport=TRANSPORT_DEFAULT,
                       stream=None):
        ms = (C.c_float * iters)()
        self._reserve_for(algo, transport)
        _check(lib().vr_time_allgather(self._h, stream, algo_id(algo), transport, _table(inputs),
                                       _table(outputs), nelems, iters, ms))
        return np.frombuffer(ms, np.float32).copy()

    def stream_probe(self, mode, dst, src, nbytes, stream=None):
        """mode: 0 copy, 1 read only, 2 write only."""
        _check(lib().vr_stream_probe(self._h, stream, mode, C.c_void_p(int(dst)),
                                     C.c_void_p(int(src)), nbytes))

    def stream_probe_multi(self, dsts, srcs, nbytes_each, stream=None):
        """The all-reduce kernel with the adds removed: dsts[k] = srcs[k] for nranks streams."""
        _check(lib().vr_stream_probe_multi(self._h, stream, _table(dsts), _table(srcs), nbytes_each))

    def xcc_ids(self, blocks):
        out = (C.c_uint32 * blocks)()
        _check(lib().vr_probe_xcc_ids(self._h, blocks, out))
        return np.frombuffer(out, np.uint32).copy()

    def time_copy(self, dst, src, nbytes, iters, stream=None):
        ms = (C.c_float * iters)()
        _check(lib().vr_time_copy(self._h, stream, C.c_void_p(int(dst)), C.c_void_p(int(src)), nbytes,
                                  iters, ms))
        return np.frombuffer(ms, np.float32).copy()


class Stream:
    """A non-blocking HIP stream (vr_stream_create); `.handle` is the hipStream_t."""

    def __init__(self, device=0):
        h = C.c_void_p()
        _check(lib().vr_stream_create(device, C.byref(h)))
        self.handle = h

    def sync(self):
        _check(lib().vr_stream_sync(self.handle))

    def close(self):
        if self.handle:
            lib().vr_stream_destroy(self.handle)
            self.handle = None


class EventTimer:
    """Pairs of HIP events recorded on one stream around caller-chosen launches."""

    def __init__(self, pairs, stream=None):
        self.stream, self.events = stream, []
        for _ in range(2 * pairs):
            e = C.c_void_p()
            _check(lib().vr_event_create(C.byref(e)))
            self.events.append(e)

    def start(self, k):
        _check(lib().vr_event_record(self.events[2 * k], self.stream))

    def stop(self, k):
        _check(lib().vr_event_record(self.events[2 * k + 1], self.stream))

    def elapsed_ms(self, count=None):
        count = len(self.events) // 2 if count is None else count
        out = np.empty(count, np.float32)
        ms = C.c_float(0)
        for k in range(count):
            _check(lib().vr_event_elapsed_ms(self.events[2 * k], self.events[2 * k + 1], C.byref(ms)))
            out[k] = ms.value
        return out

    def close(self):
        for e in self.events:
            lib().vr_event_destroy(e)
        self.events = []
