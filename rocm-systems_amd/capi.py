"""ctypes binding of include/mi355_blit.h.  Thin on purpose: tests and the
benchmark call the C ABI itself, this file only declares signatures.

There is no CPU fallback: if the library is missing, loading raises."""
import ctypes as C
import os

from . import build as _build

SUCCESS = 0x0
ERROR = 0x1000
ERROR_INVALID_ARGUMENT = 0x1001
ERROR_OUT_OF_RESOURCES = 0x1008
ERROR_NOT_INITIALIZED = 0x100B

KERNEL_COPY = 0
KERNEL_COPY_REALIGN = 1
KERNEL_FILL = 2
KERNEL_COPY_BATCH = 3
KERNEL_COPY_RECT = 4
NOALLOC_MAX_COPIES = 65536
ENGINE_NONE = 0
ENGINE_BLIT_KERNEL = 1
ENGINE_SDMA = 2

STORE_CACHED = 0
STORE_NT = 1
STORE_AGENT_WT = 2
STORE_SYSTEM_WT = 3
ROUTE_DEVICE = 0
ROUTE_HOST_TO_DEVICE = 1
ROUTE_DEVICE_TO_HOST = 2


class Plan(C.Structure):
    _fields_ = [
        ("kernel", C.c_uint32), ("wg_size", C.c_uint32), ("grid", C.c_uint32),
        ("unroll", C.c_uint32), ("nt_load", C.c_uint32), ("store_policy", C.c_uint32),
        ("byte_shift", C.c_uint32), ("lead_vecs", C.c_uint32),
        ("head_bytes", C.c_uint64), ("body_vecs", C.c_uint64), ("tail_bytes", C.c_uint64),
        ("xcd_run", C.c_uint32), ("route", C.c_uint32),
        ("reference_engine", C.c_uint32), ("pieces", C.c_uint32),
    ]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class Tuning(C.Structure):
    _fields_ = [
        ("wg_size", C.c_uint32), ("unroll", C.c_uint32), ("max_grid", C.c_uint32),
        ("nt_load", C.c_uint32), ("store_policy", C.c_uint32), ("xcd_run", C.c_uint32),
        ("batch_prefetch", C.c_uint32), ("batch_staging", C.c_uint32), ("copy_piece_mib", C.c_uint32),
    ]


class Desc(C.Structure):
    _fields_ = [("dst", C.c_void_p), ("src", C.c_void_p), ("bytes", C.c_uint64)]


class PitchedPtr(C.Structure):
    _fields_ = [("base", C.c_void_p), ("pitch", C.c_size_t), ("slice", C.c_size_t)]


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]


class RectPlan(C.Structure):
    _fields_ = [
        ("empty", C.c_uint32), ("linear", C.c_uint32), ("dst", C.c_uint64), ("src", C.c_uint64),
        ("width", C.c_uint64), ("dst_pitch", C.c_uint64), ("dst_slice", C.c_uint64),
        ("src_pitch", C.c_uint64), ("src_slice", C.c_uint64), ("rows", C.c_uint32), ("layers", C.c_uint32),
        ("slots", C.c_uint32), ("unroll", C.c_uint32), ("lanes_per_row", C.c_uint32),
        ("xcd_run", C.c_uint32), ("wg_size", C.c_uint32), ("grid", C.c_uint32),
        ("nt_load", C.c_uint32), ("store_policy", C.c_uint32), ("total_bytes", C.c_uint64),
        ("plain_rows", C.c_uint32), ("route", C.c_uint32),
    ]


def rect_args(dst, dst_offset, src, src_offset, extent):
    """(base, pitch, slice) and (x, y, z) tuples -> ctypes structures; None stays None."""
    def ptr(t):
        return None if t is None else PitchedPtr(*t)

    def dim(t):
        return None if t is None else Dim3(*t)
    return ptr(dst), dim(dst_offset), ptr(src), dim(src_offset), dim(extent)


# every symbol include/mi355_blit.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "mi355_blit_create": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "mi355_blit_destroy": (C.c_int, [C.c_void_p]),
    "mi355_blit_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "mi355_blit_copy_route": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p]),
    "mi355_blit_fill32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_size_t, C.c_void_p]),
    "mi355_blit_copy_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
    "mi355_blit_copy_batch_bounded": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_void_p]),
    "mi355_blit_copy_batch_bounded_noalloc": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_void_p]),
    "mi355_blit_copy_rect": (C.c_int, [C.c_void_p, C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                       C.POINTER(Dim3), C.POINTER(Dim3), C.c_void_p]),
    "mi355_blit_plan_rect": (C.c_int, [C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                       C.POINTER(Dim3), C.POINTER(Dim3), C.POINTER(Tuning), C.POINTER(RectPlan)]),
    "mi355_blit_copy_rect_route": (C.c_int, [C.c_void_p, C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                             C.POINTER(Dim3), C.POINTER(Dim3), C.c_uint32, C.c_void_p]),
    "mi355_blit_plan_rect_route": (C.c_int, [C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                             C.POINTER(Dim3), C.POINTER(Dim3), C.POINTER(Tuning), C.c_uint32,
                                             C.POINTER(RectPlan)]),
    "mi355_blit_signal_complete": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p]),
    "mi355_blit_signal_stamp": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint32, C.c_void_p]),
    "mi355_blit_add_callback": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mi355_blit_synchronize": (C.c_int, [C.c_void_p]),
    "mi355_blit_pending_bytes": (C.c_uint64, [C.c_void_p]),
    "mi355_blit_last_launch_info": (C.c_int, [C.c_void_p, C.POINTER(Plan)]),
    "mi355_blit_plan_copy": (C.c_int, [C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32,
                                       C.POINTER(Tuning), C.POINTER(Plan)]),
    "mi355_blit_plan_copy_route": (C.c_int, [C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32,
                                             C.POINTER(Tuning), C.c_uint32, C.POINTER(Plan)]),
    "mi355_blit_plan_fill": (C.c_int, [C.c_uint64, C.c_uint64, C.c_uint32,
                                       C.POINTER(Tuning), C.POINTER(Plan)]),
    "mi355_blit_plan_copy_pieces": (C.c_uint32, [C.c_uint64, C.c_uint32, C.c_uint32, C.POINTER(Tuning),
                                                 C.POINTER(C.c_uint64)]),
    "mi355_blit_set_tuning": (C.c_int, [C.c_void_p, C.POINTER(Tuning)]),
    "mi355_blit_num_cus": (C.c_int, [C.c_void_p]),
    "mi355_blit_stream": (C.c_void_p, [C.c_void_p]),
    "mi355_blit_status_string": (C.c_char_p, [C.c_int]),
    "mi355_blit_abi_version": (C.c_int, []),
    "mi355_policy_force_sdma_size": (C.c_uint64, []),
    "mi355_policy_same_gpu_engine": (C.c_uint32, [C.c_uint64, C.c_uint64]),
}

_lib = None


def library_path():
    return _build.BLIT_LIB


def load():
    """dlopen lib/libmi355blit.so and declare its signatures.  Import torch
    before calling this in a process that also uses torch, so that both share
    one HIP runtime."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`"
            % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class BlitError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        msg = load().mi355_blit_status_string(status).decode()
        super().__init__("%s failed: 0x%x (%s)" % (what, status, msg))


def check(status, what):
    if status != SUCCESS:
        raise BlitError(status, what)


class Blit:
    """Owner of one mi355_blit_t handle; methods map 1:1 to the C ABI and take
    raw device addresses (ints)."""

    backend = "hip"

    def __init__(self, device=0):
        self.lib = load()
        h = C.c_void_p()
        check(self.lib.mi355_blit_create(device, C.byref(h)), "mi355_blit_create")
        self.handle = h

    def close(self):
        if self.handle:
            st = self.lib.mi355_blit_destroy(self.handle)
            self.handle = None
            check(st, "mi355_blit_destroy")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def copy(self, dst, src, nbytes, stream=None, route=None):
        if route is not None:
            return self.lib.mi355_blit_copy_route(self.handle, dst, src, nbytes, route, stream)
        return self.lib.mi355_blit_copy(self.handle, dst, src, nbytes, stream)

    def fill32(self, ptr, value, num_dwords, stream=None):
        return self.lib.mi355_blit_fill32(self.handle, ptr, value, num_dwords, stream)

    def copy_batch(self, descs, n, on_device=False, stream=None):
        addr = descs if isinstance(descs, int) else C.cast(descs, C.c_void_p)
        return self.lib.mi355_blit_copy_batch(self.handle, addr, n, 1 if on_device else 0, stream)

    def copy_batch_bounded(self, device_descs, n, max_total_bytes, stream=None):
        """Device-resident descriptors that together move at most max_total_bytes."""
        addr = device_descs if isinstance(device_descs, int) or device_descs is None else C.cast(device_descs, C.c_void_p)
        return self.lib.mi355_blit_copy_batch_bounded(self.handle, addr, n, max_total_bytes, stream)

    def copy_batch_bounded_noalloc(self, device_descs, n, max_total_bytes, stream=None):
        """copy_batch_bounded out of the library's fixed scratch array: no allocation."""
        addr = device_descs if isinstance(device_descs, int) or device_descs is None else C.cast(device_descs, C.c_void_p)
        return self.lib.mi355_blit_copy_batch_bounded_noalloc(self.handle, addr, n, max_total_bytes, stream)

    def copy_rect(self, dst, dst_offset, src, src_offset, extent, stream=None, route=None):
        """dst, src: (base, pitch, slice); offsets and extent: (x bytes, y rows, z layers)."""
        a = rect_args(dst, dst_offset, src, src_offset, extent)
        if route is not None:
            return self.lib.mi355_blit_copy_rect_route(self.handle, *a, route, stream)
        return self.lib.mi355_blit_copy_rect(self.handle, *a, stream)

    def synchronize(self):
        return self.lib.mi355_blit_synchronize(self.handle)

    def pending_bytes(self):
        return self.lib.mi355_blit_pending_bytes(self.handle)

    def last_plan(self):
        p = Plan()
        check(self.lib.mi355_blit_last_launch_info(self.handle, C.byref(p)), "last_launch_info")
        return p

    def set_tuning(self, **kw):
        if not kw:
            return self.lib.mi355_blit_set_tuning(self.handle, None)
        t = Tuning()
        for k, v in kw.items():
            setattr(t, k, v)
        return self.lib.mi355_blit_set_tuning(self.handle, C.byref(t))

    @property
    def num_cus(self):
        return self.lib.mi355_blit_num_cus(self.handle)

    @property
    def stream(self):
        return self.lib.mi355_blit_stream(self.handle)


def plan_copy(dst, src, nbytes, num_cus=256, tuning=None, route=None):
    p = Plan()
    t = C.byref(tuning) if tuning is not None else None
    if route is not None:
        st = load().mi355_blit_plan_copy_route(dst, src, nbytes, num_cus, t, route, C.byref(p))
    else:
        st = load().mi355_blit_plan_copy(dst, src, nbytes, num_cus, t, C.byref(p))
    return st, p


def plan_copy_pieces(nbytes, route=0, max_pieces=32, tuning=None):
    """(launches, bytes of each but the last) for a copy of nbytes."""
    piece = C.c_uint64()
    t = C.byref(tuning) if tuning is not None else None
    n = load().mi355_blit_plan_copy_pieces(nbytes, route, max_pieces, t, C.byref(piece))
    return n, piece.value


def plan_rect(dst, dst_offset, src, src_offset, extent, tuning=None, route=None):
    """(status, RectPlan) for a region given as in Blit.copy_rect."""
    out = RectPlan()
    a = rect_args(dst, dst_offset, src, src_offset, extent)
    if route is not None:
        st = load().mi355_blit_plan_rect_route(*a, tuning, route, C.byref(out))
    else:
        st = load().mi355_blit_plan_rect(*a, tuning, C.byref(out))
    return st, out


def plan_fill(ptr, num_dwords, num_cus=256, tuning=None):
    p = Plan()
    st = load().mi355_blit_plan_fill(ptr, num_dwords, num_cus,
                                     C.byref(tuning) if tuning is not None else None, C.byref(p))
    return st, p
