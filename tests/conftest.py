import ctypes as C
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


class KernArgs(C.Union):
    class _Aligned(C.Structure):
        _fields_ = [(n, C.c_uint64) for n in (
            "phase1_src_start", "phase1_dst_start", "phase2_src_start", "phase2_dst_start",
            "phase3_src_start", "phase3_dst_start", "phase4_src_start", "phase4_dst_start",
            "phase4_src_end", "phase4_dst_end")] + [("num_workitems", C.c_uint32)]

    class _Misaligned(C.Structure):
        _fields_ = [(n, C.c_uint64) for n in (
            "phase1_src_start", "phase1_dst_start", "phase2_src_start", "phase2_dst_start",
            "phase2_src_end", "phase2_dst_end")] + [("num_workitems", C.c_uint32)]

    class _Fill(C.Structure):
        _fields_ = [("phase1_dst_start", C.c_uint64), ("phase2_dst_start", C.c_uint64),
                    ("phase2_dst_end", C.c_uint64), ("fill_value", C.c_uint32),
                    ("num_workitems", C.c_uint32)]

    _fields_ = [("copy_aligned", _Aligned), ("copy_misaligned", _Misaligned), ("fill", _Fill),
                ("raw", C.c_uint8 * 96)]


class PitchedPtr(C.Structure):
    _fields_ = [("base", C.c_void_p), ("pitch", C.c_size_t), ("slice", C.c_size_t)]


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]


class Bounds(C.Structure):
    _fields_ = [("dst_lo", C.c_uint64), ("dst_hi", C.c_uint64),
                ("src_lo", C.c_uint64), ("src_hi", C.c_uint64)]


def _declare_oracle(lib):
    u64, u32, vp, sz, i = C.c_uint64, C.c_uint32, C.c_void_p, C.c_size_t, C.c_int
    sig = {
        "oracle_ref_host_fill": (None, [vp, u32, sz]),
        "oracle_ref_validate_copy": (i, [u64, u64, u64, C.POINTER(i)]),
        "oracle_ref_validate_fill": (i, [u64, u64, C.POINTER(i)]),
        "oracle_ref_blit_fill_status": (i, [u64]),
        "oracle_ref_plan_copy": (i, [u64, u64, u64, i, C.POINTER(KernArgs)]),
        "oracle_ref_plan_fill": (None, [u64, u32, u64, i, C.POINTER(KernArgs)]),
        "oracle_ref_grid_size": (u32, [u32]),
        "oracle_ref_exec_copy_aligned": (i, [C.POINTER(KernArgs), C.POINTER(Bounds)]),
        "oracle_ref_exec_copy_misaligned": (i, [C.POINTER(KernArgs), C.POINTER(Bounds)]),
        "oracle_ref_exec_fill": (i, [C.POINTER(KernArgs), C.POINTER(Bounds)]),
        "oracle_ref_blit_copy": (i, [vp, vp, sz, i, C.POINTER(Bounds)]),
        "oracle_ref_blit_fill": (i, [vp, u32, sz, i, C.POINTER(Bounds)]),
        "oracle_ref_same_gpu_uses_blit_kernel": (i, [u64, u64]),
        "oracle_copy_rect": (None, [C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                    C.POINTER(Dim3), C.POINTER(Dim3)]),
        "oracle_ref_validate_rect": (i, [C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr),
                                         C.POINTER(Dim3), C.POINTER(Dim3), i, C.POINTER(i), C.POINTER(i)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def oracle_rect(oracle, dst, dst_offset, src, src_offset, extent):
    """oracle_copy_rect over (base, pitch, slice) and (x, y, z) tuples."""
    oracle.oracle_copy_rect(PitchedPtr(*dst), Dim3(*dst_offset), PitchedPtr(*src), Dim3(*src_offset), Dim3(*extent))


def oracle_validate_rect(oracle, dst, dst_offset, src, src_offset, extent, direction=3):
    """(status, does_work, sdma_alignment_ok) of the reference's argument checks; None = NULL."""
    def ptr(t):
        return None if t is None else PitchedPtr(*t)

    def dim(t):
        return None if t is None else Dim3(*t)
    work, aligned = C.c_int(-1), C.c_int(-1)
    st = oracle.oracle_ref_validate_rect(ptr(dst), dim(dst_offset), ptr(src), dim(src_offset), dim(extent),
                                         direction, C.byref(work), C.byref(aligned))
    return st, work.value, aligned.value


@pytest.fixture(scope="session")
def pkg():
    """The package, with its native parts built: a checkout that has not been
    built yet (the libraries are not kept in the history) is built once here,
    where hipcc is at hand.  Building is not a fallback: the tests still run the
    HIP libraries and nothing else."""
    p = entry.load_package()
    b = p.build
    if not all(os.path.exists(f) for f in (b.BLIT_LIB, b.AQL_LIB, b.ROCR_LIB, b.ORACLE_LIB, b.ROCR_TEST)):
        b.build_all()
    return p


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (oracle/libblit_oracle.so); built on demand here, where
    gcc is at hand.  It never takes the place of the GPU path."""
    p = entry.load_package().build.ORACLE_LIB
    if not os.path.exists(p):
        entry.load_package().build.build_oracle()
    return _declare_oracle(entry.load_oracle())


def host_random(oracle, n, seed):
    a = np.empty(n, dtype=np.uint8)
    oracle.oracle_fill_random(a.ctypes.data, n, seed)
    return a


@pytest.fixture(scope="session")
def rand(oracle):
    return lambda n, seed: host_random(oracle, n, seed)


# ---------------------------------------------------------------- GPU side

@pytest.fixture(scope="session")
def torch_cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: run them with -m gpu on the GPU box")
    return torch


@pytest.fixture(scope="session")
def capi(pkg, torch_cuda):
    # torch first, so that the blit library binds to the HIP runtime torch loaded
    lib_path = pkg.capi.library_path()
    assert os.path.exists(lib_path), (
        "%s is missing: the GPU tests never fall back to a CPU path" % lib_path)
    pkg.capi.load()
    return pkg.capi


@pytest.fixture(scope="session", params=["hip", "aql", "aql_borrowed"])
def blit(request, capi, pkg):
    """The engine under test, once per submission path: HIP stream launches
    (mi355_blit.h), hand-built AQL packets on an HSA queue of the engine's own
    (mi355_aql_create), and the same on a 64-packet queue the caller made, the
    way ROCr hands its utility queue to a blit (mi355_aql_create_on).  All run
    the same kernels."""
    queue = None
    if request.param == "hip":
        b = capi.Blit(0)
    else:
        assert os.path.exists(pkg.aql.library_path()), "AQL library missing: no fallback"
        pkg.aql.load()
        if request.param == "aql_borrowed":
            queue = pkg.aql.BorrowedQueue(0, packets=64)
            b = pkg.aql.AqlBlit(borrowed=queue)
        else:
            b = pkg.aql.AqlBlit(0)
    yield b
    b.close()
    if queue is not None:
        assert queue.errors == [], "the borrowed queue reported errors: %r" % queue.errors
        queue.close()


@pytest.fixture()
def fresh_tuning(blit):
    blit.set_tuning()
    yield blit
    blit.set_tuning()
