"""Host-only checks of the C ABI: the library loads, exports every symbol the
header declares, validates arguments, and its dispatch-sizing functions obey
the plan's invariants.  No compute calls: there is no GPU here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _has_gpu():
    import torch
    return torch.cuda.is_available()


@pytest.fixture(scope="module")
def capi_host(pkg):
    import torch  # noqa: F401  (one HIP runtime per process: torch's first)
    pkg.capi.load()
    return pkg.capi


def test_library_exports_every_declared_symbol(capi_host):
    header = open(os.path.join(ROOT, "include", "mi355_blit.h")).read()
    declared = set(re.findall(r"\b(mi355_(?:blit|policy)_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = C.CDLL(capi_host.library_path())
    for name in sorted(declared):
        assert hasattr(lib, name), "library does not export %s" % name
    # and the ctypes binding declares exactly the same set
    assert declared == set(capi_host.SIGNATURES)


def test_abi_version_and_status_strings(capi_host):
    lib = capi_host.load()
    assert lib.mi355_blit_abi_version() == 4
    assert lib.mi355_blit_status_string(0) == b"success"
    assert lib.mi355_blit_status_string(capi_host.ERROR_INVALID_ARGUMENT) == b"invalid argument"
    assert lib.mi355_blit_status_string(12345) == b"unknown status"


def test_struct_layouts_match_header(capi_host):
    assert C.sizeof(capi_host.Plan) == 8 * 4 + 3 * 8 + 4 * 4
    assert capi_host.Plan.lead_vecs.offset == 28
    assert C.sizeof(capi_host.Tuning) == 36
    assert C.sizeof(capi_host.Desc) == 24


def test_null_handle_is_rejected(capi_host):
    lib = capi_host.load()
    inv = capi_host.ERROR_INVALID_ARGUMENT
    assert lib.mi355_blit_destroy(None) == inv
    assert lib.mi355_blit_copy(None, 16, 32, 8, None) == inv
    assert lib.mi355_blit_fill32(None, 16, 0, 8, None) == inv
    assert lib.mi355_blit_copy_batch(None, None, 0, 0, None) == inv
    assert lib.mi355_blit_synchronize(None) == inv
    assert lib.mi355_blit_pending_bytes(None) == 0
    assert lib.mi355_blit_create(0, None) == inv


def test_create_without_gpu_fails_loudly(capi_host):
    if _has_gpu():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    st = capi_host.load().mi355_blit_create(0, C.byref(h))
    assert st == capi_host.ERROR_NOT_INITIALIZED and not h.value
    with pytest.raises(capi_host.BlitError):
        capi_host.Blit(0)


def _check_copy_plan(p, dst, src, n):
    assert p.head_bytes + 16 * p.body_vecs + p.tail_bytes == n
    assert p.head_bytes <= 15 and p.tail_bytes <= 15
    if p.body_vecs:
        assert (dst + p.head_bytes) % 16 == 0
    assert p.byte_shift == (src - dst) % 4
    assert p.kernel == (1 if p.byte_shift else 0)
    assert p.wg_size % 64 == 0 and 64 <= p.wg_size <= 1024
    assert p.unroll in (1, 2, 4)
    assert p.grid >= 1 and p.grid * p.wg_size < 2 ** 31
    assert p.lead_vecs == ((dst + p.head_bytes) % 256) // 16
    # uncapped: one wave per 256-byte anchored tile plus one for the edges
    tiles = -(-(p.body_vecs + p.lead_vecs) // (64 * p.unroll))
    assert p.grid * (p.wg_size // 64) >= tiles + 1


def test_plan_copy_invariants(capi_host):
    sizes = list(range(0, 70)) + [255, 256, 257, 1023, 1024, 1025, 4096, 65537, (1 << 20) + 3,
                                  (8 << 20) - 1, 8 << 20, (1 << 30), (1 << 32), (1 << 32) + 17]
    for d_off in range(16):
        for s_off in range(16):
            dst, src = 0x7f0000001000 + d_off, 0x7e0000002000 + s_off
            for n in sizes:
                st, p = capi_host.plan_copy(dst, src, n)
                assert st == 0
                _check_copy_plan(p, dst, src, n)


def test_plan_copy_covers_every_tile_when_uncapped(capi_host):
    for n in (1 << 30, (1 << 32) + 5, 12345678):
        for d_off in (0, 16, 48, 240, 251):
            st, p = capi_host.plan_copy(0x7f0000000000 + d_off, 0x7e0000000000, n)
            tiles = -(-(p.body_vecs + p.lead_vecs) // (64 * p.unroll))
            assert p.grid * (p.wg_size // 64) >= tiles + 1


def test_plan_copy_tuning_overrides(capi_host):
    t = capi_host.Tuning(wg_size=512, unroll=4, max_grid=100, nt_load=2, store_policy=capi_host.STORE_NT + 1)
    st, p = capi_host.plan_copy(0x1000, 0x9000, 1 << 30, 256, t)
    assert st == 0 and (p.wg_size, p.unroll, p.grid, p.nt_load, p.store_policy) == (512, 4, 100, 1, capi_host.STORE_NT)
    # nonsense values are ignored rather than launched
    t = capi_host.Tuning(wg_size=100, unroll=3, store_policy=9)
    st, q = capi_host.plan_copy(0x1000, 0x9000, 1 << 30, 256, t)
    st, d = capi_host.plan_copy(0x1000, 0x9000, 1 << 30, 256)
    assert (q.wg_size, q.unroll, q.store_policy) == (d.wg_size, d.unroll, d.store_policy)
    t = capi_host.Tuning(nt_load=1, store_policy=capi_host.STORE_CACHED + 1)
    st, p = capi_host.plan_copy(0x1000, 0x9000, 1 << 30, 256, t)
    assert p.nt_load == 0 and p.store_policy == capi_host.STORE_CACHED


def test_plan_copy_shapes_by_size_and_offset(capi_host):
    """The launch shapes the heuristics pick, and the XCD runs: 576 KiB of
    neighbouring tiles per XCD once a transfer streams from memory."""
    MIB = 1 << 20
    dst = 0x7f0000000000

    def shape(src_off, n):
        st, p = capi_host.plan_copy(dst, 0x7e0000000000 + src_off, n)
        assert st == 0
        return p.wg_size, p.unroll, p.nt_load, p.store_policy, p.xcd_run

    wt, nt, cached = capi_host.STORE_AGENT_WT, capi_host.STORE_NT, capi_host.STORE_CACHED
    for off in (0, 4, 64):                                   # dword-aligned to one another
        assert shape(off, MIB) == (256, 1, 0, cached, 0)
        assert shape(off, 64 * MIB) == (256, 1, 1, wt, 0)
        assert shape(off, 80 * MIB) == (64, 1, 1, wt, 576)      # 576 tiles of 1 KiB
        assert shape(off, 1 << 30) == (64, 1, 1, wt, 576)
    for off in (1, 3, 6):                                    # a byte offset: the realigning kernel
        assert shape(off, MIB) == (512, 1, 0, cached, 0)
        assert shape(off, 16 * MIB) == (256, 2, 1, wt, 0)
        assert shape(off, 48 * MIB) == (64, 2, 1, wt, 288)      # 288 tiles of 2 KiB
        assert shape(off, 256 * MIB) == (64, 2, 1, wt, 288)     # the last-level cache still absorbs the stores
        assert shape(off, 272 * MIB) == (64, 1, 1, nt, 576)
        assert shape(off, 1 << 30) == (64, 1, 1, nt, 576)
    # the run follows the workgroup the tuning asks for; 1 means launch order
    st, p = capi_host.plan_copy(dst, 0x7e0000000000, 1 << 30, 256, capi_host.Tuning(wg_size=256))
    assert p.xcd_run == 144
    st, p = capi_host.plan_copy(dst, 0x7e0000000000, 1 << 30, 256, capi_host.Tuning(xcd_run=1))
    assert p.xcd_run == 0
    st, p = capi_host.plan_copy(dst, 0x7e0000000000, MIB, 256, capi_host.Tuning(xcd_run=40))
    assert p.xcd_run == 40
    # fills store whole lines and share nothing: launch order
    st, p = capi_host.plan_fill(dst, 1 << 28)
    assert st == 0 and p.xcd_run == 0


def test_plan_copy_routes_across_the_host_link(capi_host):
    """A copy one side of which is host memory is cut up like any other (the same
    head / body / tail, the same kernel choice) but launched for the link: 128
    workgroups of 256 at most, in launch order, stores to the host written
    through.  The route of a plan within the device is 0 and changes nothing."""
    MIB = 1 << 20
    dst, src = 0x7f0000000000, 0x7e0000000000
    wt, sys_wt, cached = capi_host.STORE_AGENT_WT, capi_host.STORE_SYSTEM_WT, capi_host.STORE_CACHED
    h2d, d2h = capi_host.ROUTE_HOST_TO_DEVICE, capi_host.ROUTE_DEVICE_TO_HOST
    for off in (0, 3):
        for n in (1, 4096, 512 * 1024 + 5, 3 * MIB, 4 * MIB, 256 * MIB + 1, 1 << 32):
            st, dev = capi_host.plan_copy(dst + 9, src + 9 + off, n)
            assert st == 0 and dev.route == capi_host.ROUTE_DEVICE
            st, same = capi_host.plan_copy(dst + 9, src + 9 + off, n, route=capi_host.ROUTE_DEVICE)
            assert st == 0 and same.as_dict() == dev.as_dict()
            for route, store_small, store_large in ((h2d, cached, wt), (d2h, sys_wt, sys_wt)):
                st, p = capi_host.plan_copy(dst + 9, src + 9 + off, n, route=route)
                assert st == 0 and p.route == route
                # the cut and the kernel do not depend on the route
                for f in ("kernel", "byte_shift", "lead_vecs", "head_bytes", "body_vecs", "tail_bytes"):
                    assert getattr(p, f) == getattr(dev, f), f
                assert (p.wg_size, p.unroll, p.xcd_run) == (256, 1, 0)
                assert p.nt_load == (1 if n >= 4 * MIB else 0)
                assert p.store_policy == (store_large if n >= 4 * MIB else store_small)
                tiles = (p.body_vecs + p.lead_vecs + 63) // 64
                assert p.grid == min(128, (tiles + 1 + 3) // 4)
    # tuning still overrides the cap; an unknown route is refused
    st, p = capi_host.plan_copy(dst, src, 1 << 30, 256, capi_host.Tuning(max_grid=512), route=h2d)
    assert st == 0 and p.grid == 512
    st, p = capi_host.plan_copy(dst, src, 1 << 30, route=3)
    assert st == capi_host.ERROR_INVALID_ARGUMENT


def test_copies_of_several_gib_are_cut_into_pieces(capi_host):
    """Within the device a copy of 1.5 GiB or more goes out as consecutive copies
    of at most 512 MiB (a multiple of 1 MiB each, so every piece keeps the
    alignment of the whole), at most 32 of them and at most what the submission
    path has room for; the pieces tile the copy exactly.  Smaller copies and
    copies over the bus stay one launch."""
    MIB, GIB = 1 << 20, 1 << 30
    for n in (0, 1, GIB, 1536 * MIB - 1):
        assert capi_host.plan_copy_pieces(n) == (1, n)
    for route in (capi_host.ROUTE_HOST_TO_DEVICE, capi_host.ROUTE_DEVICE_TO_HOST):
        assert capi_host.plan_copy_pieces(8 * GIB, route) == (1, 8 * GIB)
    assert capi_host.plan_copy_pieces(1536 * MIB) == (3, 512 * MIB)
    assert capi_host.plan_copy_pieces(2 * GIB) == (4, 512 * MIB)
    assert capi_host.plan_copy_pieces(4 * GIB) == (8, 512 * MIB)
    assert capi_host.plan_copy_pieces(4 * GIB, max_pieces=4) == (4, GIB)
    assert capi_host.plan_copy_pieces(4 * GIB, max_pieces=1) == (1, 4 * GIB)
    assert capi_host.plan_copy_pieces(4 * GIB, max_pieces=0) == (1, 4 * GIB)
    for n in (1536 * MIB + 1, 2 * GIB - 1, 3 * GIB + 12345, 16 * GIB, 16 * GIB + 7, 33 * GIB + 3, 200 * GIB):
        for cap in (32, 7, 2):
            count, piece = capi_host.plan_copy_pieces(n, max_pieces=cap)
            assert 2 <= count <= cap and piece % MIB == 0
            assert (count - 1) * piece < n <= count * piece
            if n <= cap * 512 * MIB:
                assert piece <= 512 * MIB
            # no piece is a sliver beside the others unless the size says so
            assert piece - (n - (count - 1) * piece) < count * MIB
    # tuning: never, or pieces of a given size for anything larger
    T = capi_host.Tuning
    assert capi_host.plan_copy_pieces(64 * GIB, tuning=T(copy_piece_mib=1)) == (1, 64 * GIB)
    assert capi_host.plan_copy_pieces(64 * MIB, tuning=T(copy_piece_mib=64)) == (1, 64 * MIB)
    assert capi_host.plan_copy_pieces(64 * MIB + 1, tuning=T(copy_piece_mib=64)) == (2, 33 * MIB)
    assert capi_host.plan_copy_pieces(GIB, tuning=T(copy_piece_mib=256)) == (4, 256 * MIB)
    assert capi_host.plan_copy_pieces(GIB, capi_host.ROUTE_HOST_TO_DEVICE, tuning=T(copy_piece_mib=256)) == (1, GIB)


def test_plan_fill_invariants(capi_host):
    for off in (0, 4, 8, 12):
        ptr = 0x7f0000000000 + off
        for count in list(range(0, 40)) + [1023, 1024, 1 << 18, (1 << 28), (1 << 30) + 3]:
            st, p = capi_host.plan_fill(ptr, count)
            assert st == 0 and p.kernel == 2
            assert p.head_bytes + 16 * p.body_vecs + p.tail_bytes == 4 * count
            assert p.head_bytes % 4 == 0 and p.tail_bytes % 4 == 0
            assert p.head_bytes <= 12 and p.tail_bytes <= 12
            if p.body_vecs:
                assert (ptr + p.head_bytes) % 16 == 0
            assert p.lead_vecs == ((ptr + p.head_bytes) % 256) // 16
    for off in (1, 2, 3):
        st, _ = capi_host.plan_fill(0x1000 + off, 4)
        assert st == capi_host.ERROR_INVALID_ARGUMENT
    assert capi_host.load().mi355_blit_plan_fill(0x1000, 4, 256, None, None) == capi_host.ERROR_INVALID_ARGUMENT
    assert capi_host.load().mi355_blit_plan_copy(0x1000, 0x2000, 4, 256, None, None) == capi_host.ERROR_INVALID_ARGUMENT


def test_kernel_choice_matches_reference_predicate(capi_host, oracle):
    """Same split as amd_blit_kernel.cpp:716: (src & 3) == (dst & 3)."""
    from conftest import KernArgs
    ka = KernArgs()
    for d in range(16):
        for s in range(16):
            st, p = capi_host.plan_copy(0x10000 + d, 0x90000 + s, 4096)
            ref = oracle.oracle_ref_plan_copy(0x10000 + d, 0x90000 + s, 4096, 256, C.byref(ka))
            assert p.kernel == ref


def test_aql_library_exports_every_declared_symbol(pkg):
    import torch  # noqa: F401
    header = open(os.path.join(ROOT, "include", "mi355_blit_aql.h")).read()
    declared = set(re.findall(r"\b(mi355_(?:aql|hsa)_[a-z0-9_]+)\s*\(", header))
    assert declared and "mi355_hsa_memory_copy" in declared
    lib = C.CDLL(pkg.aql.library_path())
    for name in sorted(declared):
        assert hasattr(lib, name), "library does not export %s" % name
    assert declared == set(pkg.aql.SIGNATURES)
    # the engine-choice policy of mi355_blit.h is exported by this library too
    assert hasattr(lib, "mi355_policy_same_gpu_engine") and hasattr(lib, "mi355_policy_force_sdma_size")


def test_engine_choice_policy_matches_the_reference(capi_host, oracle, monkeypatch):
    """GetBlitObject's choice for a copy within one GPU (amd_gpu_agent.cpp:2390-2397)
    and the flag behind it (flag.h:206-207), against the oracle's restatement."""
    lib = capi_host.load()
    for size in (0, 1, 4096, (128 << 10) - 1, 128 << 10, (1 << 20) - 1, 1 << 20, 1 << 30):
        for flag in (0, 1, 128 << 10, 1 << 20, 1 << 40):
            want = capi_host.ENGINE_BLIT_KERNEL if oracle.oracle_ref_same_gpu_uses_blit_kernel(size, flag) else capi_host.ENGINE_SDMA
            assert lib.mi355_policy_same_gpu_engine(size, flag) == want, (size, flag)
    monkeypatch.delenv("HSA_FORCE_SDMA_SIZE", raising=False)
    assert lib.mi355_policy_force_sdma_size() == 1 << 20
    monkeypatch.setenv("HSA_FORCE_SDMA_SIZE", "131072")
    assert lib.mi355_policy_force_sdma_size() == 131072
    monkeypatch.setenv("HSA_FORCE_SDMA_SIZE", "")
    assert lib.mi355_policy_force_sdma_size() == 1 << 20


def test_aql_code_object_holds_every_kernel_variant(pkg):
    """The stand-alone gfx950 code object names its kernels systematically; the
    AQL engine resolves them by those names."""
    import subprocess
    out = subprocess.run(["/opt/rocm/llvm/bin/llvm-readelf", "-s", pkg.build.HSACO],
                         stdout=subprocess.PIPE, text=True, check=True).stdout
    names = set(re.findall(r"\b(mi355_[a-z0-9_]+)\.kd\b", out))
    for u in (1, 2, 4):
        for l in (0, 1):
            for s in range(4):
                for r in (0, 1):
                    assert "mi355_copy_u%d_l%d_s%d_r%d" % (u, l, s, r) in names
        for s in range(4):
            assert "mi355_fill_u%d_s%d" % (u, s) in names
    for p in (1, 2, 4):
        for l in (0, 1):
            for s in range(4):
                assert "mi355_batch_records_p%d_l%d_s%d" % (p, l, s) in names
    for l in (0, 1):
        for s in range(4):
            assert "mi355_batch_lookup_l%d_s%d" % (l, s) in names
    for n in ("mi355_batch_scan_local", "mi355_batch_scan_top", "mi355_batch_emit_records",
              "mi355_batch_emit_records_lookup", "mi355_signal_complete"):
        assert n in names


def test_aql_create_without_gpu_fails_loudly(pkg):
    if _has_gpu():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    st = pkg.aql.load().mi355_aql_create(0, C.byref(h))
    assert st != 0 and not h.value
