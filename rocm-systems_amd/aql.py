"""ctypes binding of include/mi355_blit_aql.h (the HSA-queue submission path).
No CPU fallback: if the library is missing, loading raises."""
import ctypes as C
import os

from . import build as _build
from .capi import (Desc, Plan, Tuning, PitchedPtr, Dim3, rect_args, BlitError, SUCCESS, ERROR, ERROR_INVALID_ARGUMENT,  # noqa: F401
                   ERROR_NOT_INITIALIZED, ERROR_OUT_OF_RESOURCES)

_U64P = C.POINTER(C.c_uint64)

SIGNATURES = {
    "mi355_aql_create": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "mi355_aql_create_on": (C.c_int, [C.c_uint64, C.c_void_p, C.POINTER(C.c_void_p)]),
    "mi355_aql_destroy": (C.c_int, [C.c_void_p]),
    "mi355_aql_report_queue_error": (C.c_int, [C.c_void_p, C.c_int]),
    "mi355_aql_set_large_transfer_barrier": (C.c_int, [C.c_void_p, C.c_int]),
    "mi355_aql_code_object_acquire": (C.c_int, [C.c_uint64, C.POINTER(C.c_void_p)]),
    "mi355_aql_code_object_release": (C.c_int, [C.c_void_p]),
    "mi355_aql_code_object_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)]),
    "mi355_aql_wait_signal": (C.c_int, [C.c_void_p, C.c_uint64]),
    "mi355_aql_copy_sync": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32]),
    "mi355_aql_fill32_sync": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_size_t]),
    "mi355_aql_note_reference_engine": (C.c_int, [C.c_void_p, C.c_uint32]),
    "mi355_aql_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, _U64P, C.c_uint32, C.c_uint64]),
    "mi355_aql_copy_route": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32, _U64P, C.c_uint32,
                                       C.c_uint64]),
    "mi355_aql_fill32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_size_t, _U64P, C.c_uint32, C.c_uint64]),
    "mi355_aql_copy_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, _U64P, C.c_uint32, C.c_uint64]),
    "mi355_aql_copy_batch_device": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, _U64P, C.c_uint32, C.c_uint64]),
    "mi355_aql_copy_batch_bounded": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, _U64P, C.c_uint32,
                                               C.c_uint64]),
    "mi355_aql_copy_rect": (C.c_int, [C.c_void_p, C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                      C.POINTER(Dim3), C.POINTER(Dim3), _U64P, C.c_uint32, C.c_uint64]),
    "mi355_aql_copy_rect_route": (C.c_int, [C.c_void_p, C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                            C.POINTER(Dim3), C.POINTER(Dim3), C.c_uint32, _U64P, C.c_uint32,
                                            C.c_uint64]),
    "mi355_aql_wait_idle": (C.c_int, [C.c_void_p]),
    "mi355_aql_pending_bytes": (C.c_uint64, [C.c_void_p]),
    "mi355_aql_enable_profiling": (C.c_int, [C.c_void_p, C.c_int]),
    "mi355_aql_get_command_time": (C.c_int, [C.c_void_p, C.c_uint64, _U64P, _U64P, _U64P]),
    "mi355_aql_set_tuning": (C.c_int, [C.c_void_p, C.POINTER(Tuning)]),
    "mi355_aql_last_launch_info": (C.c_int, [C.c_void_p, C.POINTER(Plan)]),
    "mi355_aql_num_cus": (C.c_int, [C.c_void_p]),
    "mi355_aql_set_system_scope_fences": (C.c_int, [C.c_void_p, C.c_int]),
    "mi355_aql_gpu_agent": (C.c_uint64, [C.c_void_p]),
    "mi355_aql_staging": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]),
    "mi355_hsa_memory_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "mi355_hsa_amd_memory_fill": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_size_t]),
    "mi355_hsa_amd_memory_async_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32,
                                                  _U64P, C.c_uint64]),
    "mi355_hsa_amd_memory_async_copy_on_engine": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32,
                                                            _U64P, C.c_uint64, C.c_uint32, C.c_int]),
    "mi355_hsa_amd_memory_copy_engine_status": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_uint32)]),
    "mi355_hsa_amd_memory_async_copy_rect": (C.c_int, [C.c_void_p, C.POINTER(PitchedPtr), C.POINTER(Dim3),
                                                       C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(Dim3),
                                                       C.c_int, C.c_uint32, _U64P, C.c_uint64]),
}

_lib = None


def library_path():
    return _build.AQL_LIB


def load():
    """dlopen lib/libmi355blit_aql.so.  In a process that also uses torch,
    import torch first so that both share one HSA runtime."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with __graft_entry__.build()" % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _deps(deps):
    if not deps:
        return None, 0
    arr = (C.c_uint64 * len(deps))(*deps)
    return arr, len(deps)


class AqlBlit:
    """Owner of one mi355_aql_t handle; methods map 1:1 to the C ABI."""

    backend = "aql"

    def __init__(self, gpu=0, borrowed=None):
        """gpu: ordinal among the GPU agents, on a queue of the engine's own.
        borrowed: a BorrowedQueue instead; the engine then runs on that agent
        and that queue (mi355_aql_create_on) and leaves both alone on close."""
        self.lib = load()
        self.borrowed = borrowed
        h = C.c_void_p()
        if borrowed is not None:
            st = self.lib.mi355_aql_create_on(borrowed.agent, borrowed.queue, C.byref(h))
            what = "mi355_aql_create_on"
        else:
            st = self.lib.mi355_aql_create(gpu, C.byref(h))
            what = "mi355_aql_create"
        if st != SUCCESS:
            raise RuntimeError("%s failed: 0x%x" % (what, st))
        self.handle = h

    def close(self):
        if self.handle:
            st = self.lib.mi355_aql_destroy(self.handle)
            self.handle = None
            if st != SUCCESS:
                raise RuntimeError("mi355_aql_destroy failed: 0x%x" % st)

    def copy_sync(self, dst, src, nbytes, route=0):
        return self.lib.mi355_aql_copy_sync(self.handle, dst, src, nbytes, route)

    def fill32_sync(self, ptr, value, num_dwords):
        return self.lib.mi355_aql_fill32_sync(self.handle, ptr, value, num_dwords)

    def wait_signal(self, signal):
        return self.lib.mi355_aql_wait_signal(self.handle, signal)

    def set_large_transfer_barrier(self, enable):
        return self.lib.mi355_aql_set_large_transfer_barrier(self.handle, 1 if enable else 0)

    def code_object_info(self):
        """(hsa_executable_t.handle the engine's kernels come from, references to it)."""
        exe, users = C.c_uint64(), C.c_uint32()
        st = self.lib.mi355_aql_code_object_info(self.handle, C.byref(exe), C.byref(users))
        if st != SUCCESS:
            raise RuntimeError("mi355_aql_code_object_info failed: 0x%x" % st)
        return exe.value, users.value

    def report_queue_error(self, status=ERROR):
        return self.lib.mi355_aql_report_queue_error(self.handle, status)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def copy(self, dst, src, nbytes, *, deps=None, completion=0, route=None):
        arr, n = _deps(deps)
        if route is not None:
            return self.lib.mi355_aql_copy_route(self.handle, dst, src, nbytes, route, arr, n, completion)
        return self.lib.mi355_aql_copy(self.handle, dst, src, nbytes, arr, n, completion)

    def fill32(self, ptr, value, num_dwords, *, deps=None, completion=0):
        arr, n = _deps(deps)
        return self.lib.mi355_aql_fill32(self.handle, ptr, value, num_dwords, arr, n, completion)

    def copy_batch(self, descs, n, on_device=False, *, deps=None, completion=0):
        arr, nd = _deps(deps)
        addr = descs if isinstance(descs, int) or descs is None else C.cast(descs, C.c_void_p)
        if on_device:
            return self.lib.mi355_aql_copy_batch_device(self.handle, addr, n, arr, nd, completion)
        return self.lib.mi355_aql_copy_batch(self.handle, addr, n, arr, nd, completion)

    def copy_batch_bounded(self, device_descs, n, max_total_bytes, *, deps=None, completion=0):
        """Device-resident descriptors that together move at most max_total_bytes."""
        arr, nd = _deps(deps)
        addr = device_descs if isinstance(device_descs, int) or device_descs is None else C.cast(device_descs, C.c_void_p)
        return self.lib.mi355_aql_copy_batch_bounded(self.handle, addr, n, max_total_bytes, arr, nd, completion)

    def copy_rect(self, dst, dst_offset, src, src_offset, extent, *, deps=None, completion=0, route=None):
        """dst, src: (base, pitch, slice); offsets and extent: (x bytes, y rows, z layers)."""
        arr, n = _deps(deps)
        a = rect_args(dst, dst_offset, src, src_offset, extent)
        if route is not None:
            return self.lib.mi355_aql_copy_rect_route(self.handle, *a, route, arr, n, completion)
        return self.lib.mi355_aql_copy_rect(self.handle, *a, arr, n, completion)

    def synchronize(self):
        return self.lib.mi355_aql_wait_idle(self.handle)

    def pending_bytes(self):
        return self.lib.mi355_aql_pending_bytes(self.handle)

    def last_plan(self):
        p = Plan()
        self.lib.mi355_aql_last_launch_info(self.handle, C.byref(p))
        return p

    def set_tuning(self, **kw):
        if not kw:
            return self.lib.mi355_aql_set_tuning(self.handle, None)
        t = Tuning()
        for k, v in kw.items():
            setattr(t, k, v)
        return self.lib.mi355_aql_set_tuning(self.handle, C.byref(t))

    def set_system_scope_fences(self, on):
        return self.lib.mi355_aql_set_system_scope_fences(self.handle, 1 if on else 0)

    def enable_profiling(self, on):
        return self.lib.mi355_aql_enable_profiling(self.handle, 1 if on else 0)

    # caller policy (hsa_memory_copy / hsa_amd_memory_fill / hsa_amd_memory_async_copy stand-ins)
    def hsa_memory_copy(self, dst, src, nbytes):
        return self.lib.mi355_hsa_memory_copy(self.handle, dst, src, nbytes)

    def hsa_amd_memory_fill(self, ptr, value, count):
        return self.lib.mi355_hsa_amd_memory_fill(self.handle, ptr, value, count)

    def hsa_amd_memory_async_copy(self, dst, src, nbytes, deps=None, completion=0):
        arr, n = _deps(deps)
        return self.lib.mi355_hsa_amd_memory_async_copy(self.handle, dst, src, nbytes, n, arr, completion)

    def hsa_amd_memory_async_copy_on_engine(self, dst, src, nbytes, engine_id, force_copy_on_sdma=False, deps=None,
                                            completion=0):
        arr, n = _deps(deps)
        return self.lib.mi355_hsa_amd_memory_async_copy_on_engine(self.handle, dst, src, nbytes, n, arr, completion,
                                                                  engine_id, 1 if force_copy_on_sdma else 0)

    def hsa_amd_memory_copy_engine_status(self, dst_is_gpu, src_is_gpu):
        """(status, engine_ids_mask)"""
        mask = C.c_uint32(0xdeadbeef)
        st = self.lib.mi355_hsa_amd_memory_copy_engine_status(self.handle, 1 if dst_is_gpu else 0,
                                                              1 if src_is_gpu else 0, C.byref(mask))
        return st, mask.value

    def hsa_amd_memory_async_copy_rect(self, dst, dst_offset, src, src_offset, extent, direction=3, deps=None,
                                       completion=0):
        arr, n = _deps(deps)
        a = rect_args(dst, dst_offset, src, src_offset, extent)
        return self.lib.mi355_hsa_amd_memory_async_copy_rect(self.handle, *a, direction, n, arr, completion)

    def command_time_us(self, completion):
        """Device time of the command that completed `completion`, in microseconds
        (needs enable_profiling(True) before the command was submitted)."""
        a, b, f = C.c_uint64(), C.c_uint64(), C.c_uint64()
        st = self.lib.mi355_aql_get_command_time(self.handle, completion, C.byref(a), C.byref(b), C.byref(f))
        if st != SUCCESS:
            raise RuntimeError("mi355_aql_get_command_time failed: 0x%x" % st)
        return (b.value - a.value) * 1e6 / f.value

    @property
    def num_cus(self):
        return self.lib.mi355_aql_num_cus(self.handle)


class HsaSignals:
    """hsa_signal_create / wait / destroy through ctypes, for callers of the
    AQL path that want completion signals from Python (tests, benchmark)."""

    def __init__(self):
        self.hsa = C.CDLL("libhsa-runtime64.so.1")
        self.hsa.hsa_signal_create.argtypes = [C.c_int64, C.c_uint32, C.c_void_p, _U64P]
        self.hsa.hsa_signal_destroy.argtypes = [C.c_uint64]
        self.hsa.hsa_signal_store_relaxed.argtypes = [C.c_uint64, C.c_int64]
        self.hsa.hsa_signal_store_screlease.argtypes = [C.c_uint64, C.c_int64]
        self.hsa.hsa_signal_load_scacquire.argtypes = [C.c_uint64]
        self.hsa.hsa_signal_load_scacquire.restype = C.c_int64
        self.hsa.hsa_signal_wait_scacquire.argtypes = [C.c_uint64, C.c_int, C.c_int64, C.c_uint64, C.c_int]
        self.hsa.hsa_signal_wait_scacquire.restype = C.c_int64

    def create(self, value=1):
        h = C.c_uint64()
        st = self.hsa.hsa_signal_create(value, 0, None, C.byref(h))
        if st != 0:
            raise RuntimeError("hsa_signal_create failed: 0x%x" % st)
        return h.value

    def destroy(self, s):
        self.hsa.hsa_signal_destroy(s)

    def store(self, s, value):
        self.hsa.hsa_signal_store_screlease(s, value)

    def load(self, s):
        return self.hsa.hsa_signal_load_scacquire(s)

    def wait_below_one(self, s, active=True):
        """Blocks until the signal is < 1 (HSA_SIGNAL_CONDITION_LT = 2)."""
        while self.hsa.hsa_signal_wait_scacquire(s, 2, 1, 0xFFFFFFFFFFFFFFFF, 1 if active else 0) >= 1:
            pass


class BorrowedQueue:
    """An HSA queue made by the caller, the way GpuAgent makes its utility
    queue (hsa_queue_create, 64 packets, HSA_QUEUE_TYPE_MULTI), for an engine to
    run on (AqlBlit(borrowed=...)).  Holds a reference on the runtime for its
    lifetime.  `agent` is hsa_agent_t.handle of GPU `gpu`, `queue` the
    hsa_queue_t* as an int."""

    _AGENT_CB = C.CFUNCTYPE(C.c_int, C.c_uint64, C.c_void_p)
    _ERROR_CB = C.CFUNCTYPE(None, C.c_int, C.c_void_p, C.c_void_p)

    def __init__(self, gpu=0, packets=64):
        hsa = C.CDLL("libhsa-runtime64.so.1")
        self.hsa = hsa
        hsa.hsa_iterate_agents.argtypes = [self._AGENT_CB, C.c_void_p]
        hsa.hsa_agent_get_info.argtypes = [C.c_uint64, C.c_int, C.c_void_p]
        hsa.hsa_queue_create.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, self._ERROR_CB, C.c_void_p, C.c_uint32,
                                         C.c_uint32, C.POINTER(C.c_void_p)]
        hsa.hsa_queue_destroy.argtypes = [C.c_void_p]
        if hsa.hsa_init() != 0:
            raise RuntimeError("hsa_init failed")
        gpus = []

        def visit(agent, _data):
            kind = C.c_int(-1)
            hsa.hsa_agent_get_info(agent, 17, C.byref(kind))  # HSA_AGENT_INFO_DEVICE
            if kind.value == 1:                               # HSA_DEVICE_TYPE_GPU
                gpus.append(agent)
            return 0

        self._visit = self._AGENT_CB(visit)
        hsa.hsa_iterate_agents(self._visit, None)
        if gpu >= len(gpus):
            hsa.hsa_shut_down()
            raise RuntimeError("no GPU agent %d" % gpu)
        self.agent = gpus[gpu]
        self.errors = []
        self._on_error = self._ERROR_CB(lambda status, _queue, _data: self.errors.append(status))
        q = C.c_void_p()
        st = hsa.hsa_queue_create(self.agent, packets, 0, self._on_error  # HSA_QUEUE_TYPE_MULTI
                                  , None, 0xFFFFFFFF, 0xFFFFFFFF, C.byref(q))
        if st != 0:
            hsa.hsa_shut_down()
            raise RuntimeError("hsa_queue_create failed: 0x%x" % st)
        self.queue = q.value

    def close(self):
        if self.queue:
            self.hsa.hsa_queue_destroy(self.queue)
            self.queue = None
            self.hsa.hsa_shut_down()
