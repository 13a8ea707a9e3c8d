"""Pins the CPU oracle (oracle/blit_oracle.c) before anything is compared with
it: generator streams against committed golden hashes, the fill and copy
oracles against the reference's own known-answer tests and against numpy, and
the restated reference phase split and shaders against closed-form invariants
and against memcpy, brute-forced over every residue class."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from conftest import Bounds, KernArgs

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

ALIGNED, MISALIGNED, FILL = 0, 1, 2
SUCCESS, ERROR, INVALID_ARGUMENT = 0x0, 0x1000, 0x1001


def test_generator_streams_match_golden(oracle, rand):
    with open(os.path.join(GOLDEN, "generator_streams.json")) as f:
        golden = json.load(f)
    for case in golden["streams"]:
        a = rand(case["bytes"], int(case["seed"], 16))
        h = oracle.oracle_fnv1a64(a.ctypes.data, a.size)
        assert "%016x" % h == case["fnv1a64"], case
        assert a[:8].tolist() == case["first8"], case


def test_generator_is_xoshiro256starstar(rand):
    # independent restatement in python ints (splitmix64 seeding, xoshiro256**)
    M = (1 << 64) - 1
    seed = 0xB1170003
    s, x = [], seed
    for _ in range(4):
        x = (x + 0x9E3779B97F4A7C15) & M
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        s.append(z ^ (z >> 31))
    rotl = lambda v, k: ((v << k) | (v >> (64 - k))) & M
    out = bytearray()
    for _ in range(9):
        r = (rotl((s[1] * 5) & M, 7) * 9) & M
        t = (s[1] << 17) & M
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]
        s[2] ^= t; s[3] = rotl(s[3], 45)
        out += r.to_bytes(8, "little")
    assert rand(67, seed).tobytes() == bytes(out[:67])


def test_fnv1a64_known_answers(oracle):
    # published FNV-1a 64 test vectors
    for data, want in ((b"", 0xcbf29ce484222325), (b"a", 0xaf63dc4c8601ec8c),
                       (b"foobar", 0x85944171f73967e8)):
        buf = C.create_string_buffer(data, len(data) or 1)
        assert oracle.oracle_fnv1a64(buf, len(data)) == want


# ---- fill ------------------------------------------------------------------

# rocrtst/samples/async_mem_copy/async_mem_copy.cc:62-65 and the benchmark's pattern
REFERENCE_FILL_VALUES = [0xabcdef12, 0xba5eba11, 0xfeed5a1e, 0xbaadf00d, 0xA5C30F1E]


@pytest.mark.parametrize("value", REFERENCE_FILL_VALUES)
@pytest.mark.parametrize("count", [0, 1, 3, 4, 5, 1023, 4096, 65537])
def test_fill32_known_answer(oracle, value, count):
    """Fill then verify every dword, as async_mem_copy.cc:348-354 does."""
    guard = 64
    buf = np.full(count * 4 + 2 * guard, 0xEE, dtype=np.uint8)
    oracle.oracle_fill32(buf.ctypes.data + guard, value, count)
    assert (buf[:guard] == 0xEE).all() and (buf[guard + 4 * count:] == 0xEE).all()
    body = buf[guard:guard + 4 * count].view("<u4")
    assert (body == value).all()


def test_reference_host_fill_truncates_pattern(oracle):
    """runtime.cpp:657-661 is memset(ptr, value, count*4): only the low byte of
    the pattern survives.  A reference quirk, never used as an expectation."""
    buf = np.zeros(64, dtype=np.uint8)
    oracle.oracle_ref_host_fill(buf.ctypes.data, 0xA5C30F1E, 16)
    assert (buf == 0x1E).all()
    good = np.zeros(64, dtype=np.uint8)
    oracle.oracle_fill32(good.ctypes.data, 0xA5C30F1E, 16)
    assert not np.array_equal(buf, good)
    # the two agree exactly when all four bytes of the pattern are equal
    oracle.oracle_ref_host_fill(buf.ctypes.data, 0x7f7f7f7f, 16)
    oracle.oracle_fill32(good.ctypes.data, 0x7f7f7f7f, 16)
    assert np.array_equal(buf, good)


# ---- copy ------------------------------------------------------------------

@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 4096, 1 << 20, (1 << 20) + 3])
def test_copy_is_memcpy(oracle, rand, n):
    src = rand(n + 32, 0xB1170001)
    dst = np.full(n + 64, 0xEE, dtype=np.uint8)
    oracle.oracle_copy(dst.ctypes.data + 16 + 5, src.ctypes.data + 7, n)
    want = np.full(n + 64, 0xEE, dtype=np.uint8)
    want[21:21 + n] = src[7:7 + n]
    assert np.array_equal(dst, want)


def test_copy_reference_perf_test_case(oracle):
    """memory_async_copy.cc:314-318 + 425: source bytes 1, destination 0,
    memcmp == 0 afterwards, sizes from memory_async_copy.h:207-216 (to 4 MiB here)."""
    for size in [1024 << k for k in range(13)]:
        src = np.full(size, 1, dtype=np.uint8)
        dst = np.zeros(size, dtype=np.uint8)
        oracle.oracle_copy(dst.ctypes.data, src.ctypes.data, size)
        assert dst.tobytes() == src.tobytes()


def test_mt_variants_equal_single_thread(oracle, rand):
    n = (3 << 20) + 13
    src = rand(n, 7)
    a = np.zeros(n, dtype=np.uint8)
    b = np.zeros(n, dtype=np.uint8)
    oracle.oracle_copy(a.ctypes.data, src.ctypes.data, n)
    for t in (1, 3, 8):
        b[:] = 0
        oracle.oracle_copy_mt(b.ctypes.data, src.ctypes.data, n, t)
        assert np.array_equal(a, b)
    cnt = (1 << 18) + 5
    a = np.zeros(cnt, dtype="<u4")
    b = np.zeros(cnt, dtype="<u4")
    oracle.oracle_fill32(a.ctypes.data, 0xA5C30F1E, cnt)
    for t in (1, 3, 8):
        b[:] = 0
        oracle.oracle_fill32_mt(b.ctypes.data, 0xA5C30F1E, cnt, t)
        assert np.array_equal(a, b)


def test_thread_pool_equals_single_thread(oracle, rand):
    """The pooled host path of the CPU baseline (persistent pinned workers, one
    contiguous slice each) against the single-thread oracle: thread counts that
    do and do not divide the size, more threads than 64-byte blocks, guards."""
    import ctypes
    for name, res, args in (("oracle_pool_create", ctypes.c_void_p, [ctypes.c_int]),
                            ("oracle_pool_destroy", None, [ctypes.c_void_p]),
                            ("oracle_pool_threads", ctypes.c_int, [ctypes.c_void_p]),
                            ("oracle_pool_pinned", ctypes.c_int, [ctypes.c_void_p]),
                            ("oracle_pool_first_touch", None, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
                            ("oracle_pool_copy", None, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
                            ("oracle_pool_fill32", None, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_size_t])):
        fn = getattr(oracle, name)
        fn.restype, fn.argtypes = res, args
    guard = 128
    for threads in (1, 2, 7, 16, 33):
        pool = oracle.oracle_pool_create(threads)
        assert pool and oracle.oracle_pool_threads(pool) == threads
        assert 0 <= oracle.oracle_pool_pinned(pool) <= threads
        for n in (0, 1, 63, 64, 65, 1000, (3 << 20) + 13, 1 << 22):
            src = rand(n + 1, 11 + threads)
            got = np.full(n + 2 * guard, 0xEE, dtype=np.uint8)
            want = got.copy()
            oracle.oracle_pool_first_touch(pool, got.ctypes.data + guard, n)
            assert (got[guard:guard + n] == 0).all() and (got[:guard] == 0xEE).all() and (got[guard + n:] == 0xEE).all()
            oracle.oracle_pool_copy(pool, got.ctypes.data + guard, src.ctypes.data, n)
            oracle.oracle_copy(want.ctypes.data + guard, src.ctypes.data, n)
            assert np.array_equal(got, want), (threads, n)
            cnt = n // 4
            oracle.oracle_pool_fill32(pool, got.ctypes.data + guard, 0xA5C30F1E, cnt)
            oracle.oracle_fill32(want.ctypes.data + guard, 0xA5C30F1E, cnt)
            assert np.array_equal(got, want), (threads, n)
        oracle.oracle_pool_destroy(pool)


# ---- API-edge validation -----------------------------------------------------

def test_validate_copy(oracle):
    w = C.c_int()
    assert oracle.oracle_ref_validate_copy(0, 0x1000, 16, C.byref(w)) == INVALID_ARGUMENT and w.value == 0
    assert oracle.oracle_ref_validate_copy(0x1000, 0, 16, C.byref(w)) == INVALID_ARGUMENT and w.value == 0
    assert oracle.oracle_ref_validate_copy(0x1000, 0x2000, 0, C.byref(w)) == SUCCESS and w.value == 0
    assert oracle.oracle_ref_validate_copy(0x1001, 0x2003, 5, C.byref(w)) == SUCCESS and w.value == 1


def test_validate_fill(oracle):
    w = C.c_int()
    assert oracle.oracle_ref_validate_fill(0, 4, C.byref(w)) == INVALID_ARGUMENT
    for off in (1, 2, 3):
        assert oracle.oracle_ref_validate_fill(0x1000 + off, 4, C.byref(w)) == INVALID_ARGUMENT
        # the blit itself answers with plain ERROR (amd_blit_kernel.cpp:791-794)
        assert oracle.oracle_ref_blit_fill_status(0x1000 + off) == ERROR
    assert oracle.oracle_ref_validate_fill(0x1000, 0, C.byref(w)) == SUCCESS and w.value == 0
    assert oracle.oracle_ref_validate_fill(0x1004, 9, C.byref(w)) == SUCCESS and w.value == 1
    assert oracle.oracle_ref_blit_fill_status(0x1004) == SUCCESS


def test_same_gpu_engine_policy(oracle):
    mib = 1 << 20
    assert oracle.oracle_ref_same_gpu_uses_blit_kernel(mib - 1, mib) == 0
    assert oracle.oracle_ref_same_gpu_uses_blit_kernel(mib, mib) == 1
    assert oracle.oracle_ref_same_gpu_uses_blit_kernel(1, 0) == 1  # HSA_FORCE_SDMA_SIZE=0


# ---- the reference's phase split: closed-form invariants ---------------------

def _sizes_around(block):
    s = set(range(0, 20)) | {255, 256, 257, 511, 512, 513}
    for k in (1, 2, 3):
        for d in (-5, -4, -1, 0, 1, 3, 4, 300):
            s.add(k * block + d)
    return sorted(v for v in s if v >= 0)


@pytest.mark.parametrize("num_cus", [1, 256])
def test_plan_copy_aligned_invariants_all_residues(oracle, num_cus):
    W = 64 * 4 * num_cus
    B2 = W * 16
    ka = KernArgs()
    base_d, base_s = 0x7f0000000000, 0x7e0000100000
    sizes = _sizes_around(B2)
    for d_res in range(256):
        # every source residue mod 256 with the same residue mod 4
        for s_res in range(d_res & 3, 256, 4 if num_cus == 1 else 52):
            dst, src = base_d + d_res, base_s + s_res
            for size in sizes:
                k = oracle.oracle_ref_plan_copy(dst, src, size, num_cus, C.byref(ka))
                assert k == ALIGNED
                a = ka.copy_aligned
                p1 = a.phase2_dst_start - a.phase1_dst_start
                p2 = a.phase3_dst_start - a.phase2_dst_start
                p3 = a.phase4_dst_start - a.phase3_dst_start
                p4 = a.phase4_dst_end - a.phase4_dst_start
                assert a.phase1_dst_start == dst and a.phase1_src_start == src
                assert p1 + p2 + p3 + p4 == size
                assert p1 < 256 and (p1 == size or (dst + p1) % 256 == 0)
                assert p2 % B2 == 0 and (size - p1 - p2) < B2
                assert p3 % 4 == 0 and p4 < 4
                assert a.num_workitems == W
                # source bounds move in lock step with destination bounds
                for f in ("phase2", "phase3", "phase4"):
                    assert (getattr(a, f + "_src_start") - src) == (getattr(a, f + "_dst_start") - dst)
                assert a.phase4_src_end - src == size
                # phases 2 and 3 are dword aligned on both sides
                if p2 or p3:
                    assert a.phase2_dst_start % 4 == 0 and a.phase2_src_start % 4 == 0


def test_plan_copy_misaligned_invariants(oracle):
    ka = KernArgs()
    for num_cus in (1, 256):
        W = 64 * 4 * num_cus
        B1 = W * 4
        for d_res in range(16):
            for s_res in range(16):
                if (d_res & 3) == (s_res & 3):
                    continue
                dst, src = 0x7f0000000000 + d_res, 0x7e0000000000 + s_res
                for size in _sizes_around(B1):
                    k = oracle.oracle_ref_plan_copy(dst, src, size, num_cus, C.byref(ka))
                    assert k == MISALIGNED
                    m = ka.copy_misaligned
                    p1 = m.phase2_dst_start - m.phase1_dst_start
                    p2 = m.phase2_dst_end - m.phase2_dst_start
                    assert p1 + p2 == size and p1 % B1 == 0 and p2 < B1
                    assert m.phase2_src_start - src == p1 and m.phase2_src_end - src == size
                    assert m.num_workitems == W


def test_plan_fill_invariants(oracle):
    ka = KernArgs()
    for num_cus in (1, 256):
        W = 64 * num_cus
        B1 = W * 16
        for off in (0, 4, 8, 12, 252):
            ptr = 0x7f0000000000 + off
            for nbytes in _sizes_around(B1):
                count = nbytes // 4
                oracle.oracle_ref_plan_fill(ptr, 0xA5C30F1E, count, num_cus, C.byref(ka))
                f = ka.fill
                p1 = f.phase2_dst_start - f.phase1_dst_start
                p2 = f.phase2_dst_end - f.phase2_dst_start
                assert f.phase1_dst_start == ptr
                assert p1 + p2 == 4 * count and p1 % B1 == 0 and p2 < B1 and p2 % 4 == 0
                assert f.fill_value == 0xA5C30F1E and f.num_workitems == W


def test_reference_constants_on_mi355x(oracle):
    """256 CUs: copy grid 65536 work-items, 1 MiB aligned block, 256 KiB
    misaligned and fill blocks (amd_blit_kernel.cpp:723-734, 759-766, 797-805)."""
    ka = KernArgs()
    oracle.oracle_ref_plan_copy(0x1000000, 0x9000000, 3 << 20, 256, C.byref(ka))
    assert ka.copy_aligned.num_workitems == 65536
    assert ka.copy_aligned.phase3_dst_start - ka.copy_aligned.phase2_dst_start == 3 << 20
    oracle.oracle_ref_plan_copy(0x1000000, 0x9000000, (1 << 20) - 4, 256, C.byref(ka))
    # below one block nothing reaches the dwordx4 loop
    assert ka.copy_aligned.phase3_dst_start == ka.copy_aligned.phase2_dst_start
    oracle.oracle_ref_plan_copy(0x1000001, 0x9000000, (256 << 10) + 5, 256, C.byref(ka))
    assert ka.copy_misaligned.phase2_dst_start - ka.copy_misaligned.phase1_dst_start == 256 << 10
    oracle.oracle_ref_plan_fill(0x1000000, 1, (256 << 10) // 4 + 1, 256, C.byref(ka))
    assert ka.fill.num_workitems == 16384
    assert ka.fill.phase2_dst_start - ka.fill.phase1_dst_start == 256 << 10
    assert oracle.oracle_ref_grid_size(65536) == 65536 and oracle.oracle_ref_grid_size(65) == 128
    assert C.sizeof(KernArgs) == 96


# ---- the reference's shaders, emulated: must equal memcpy / dword fill --------

GUARD = 256


def _run_ref_copy(oracle, rand, d_off, s_off, size, num_cus, seed):
    src = rand(size + 512, seed)
    dst = np.full(size + 2 * GUARD + 512, 0xEE, dtype=np.uint8)
    # place the buffers so that (address & 255) is what the case asks for
    s_addr = src.ctypes.data + ((-src.ctypes.data) % 256) + s_off
    d_addr = dst.ctypes.data + ((-dst.ctypes.data) % 256) + GUARD + d_off
    b = Bounds(d_addr, d_addr + size, s_addr, s_addr + size)
    k = oracle.oracle_ref_blit_copy(d_addr, s_addr, size, num_cus, C.byref(b))
    want = np.full(dst.size, 0xEE, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data + (d_addr - dst.ctypes.data), s_addr, size)
    return k, dst, want


def test_ref_copy_aligned_equals_memcpy_all_dst_residues(oracle, rand):
    """num_cus=1 makes the dwordx4 block 4 KiB, so every phase is exercised."""
    B2 = 256 * 16
    for d_res in range(256):
        s_res = ((d_res * 7) & ~3 | (d_res & 3)) & 255
        for size in (0, 1, 3, 4, 5, 200, 255, 256, 257, B2 - 1, B2, B2 + 1, 2 * B2 + 255 + 7):
            k, got, want = _run_ref_copy(oracle, rand, d_res, s_res, size, 1, d_res * 131 + size)
            assert k == ALIGNED, (d_res, s_res, size)
            assert np.array_equal(got, want), (d_res, s_res, size)


def test_ref_copy_misaligned_equals_memcpy_all_pairs(oracle, rand):
    B1 = 256 * 4
    for d_res in range(16):
        for s_res in range(16):
            if (d_res & 3) == (s_res & 3):
                continue
            for size in (1, 2, 63, 64, 65, B1 - 1, B1, B1 + 1, 3 * B1 + 77):
                k, got, want = _run_ref_copy(oracle, rand, d_res, s_res, size, 1, d_res * 16 + s_res)
                assert k == MISALIGNED
                assert np.array_equal(got, want), (d_res, s_res, size)


@pytest.mark.parametrize("d_off,s_off,size", [
    (0, 0, (2 << 20) + 12345), (3, 7, (1 << 20) + 259), (5, 6, (512 << 10) + 3), (252, 4, 1 << 20)])
def test_ref_copy_at_mi355x_grid(oracle, rand, d_off, s_off, size):
    k, got, want = _run_ref_copy(oracle, rand, d_off, s_off, size, 256, size)
    assert k == (ALIGNED if (d_off & 3) == (s_off & 3) else MISALIGNED)
    assert np.array_equal(got, want)


def test_ref_copy_out_of_bounds_access_is_reported(oracle, rand):
    """The bounds checker itself: a copy whose bounds are one byte short fails."""
    src = rand(4096, 1)
    dst = np.zeros(4096, dtype=np.uint8)
    b = Bounds(dst.ctypes.data, dst.ctypes.data + 999, src.ctypes.data, src.ctypes.data + 1000)
    assert oracle.oracle_ref_blit_copy(dst.ctypes.data, src.ctypes.data, 1000, 1, C.byref(b)) == -1


@pytest.mark.parametrize("num_cus", [1, 256])
def test_ref_fill_equals_dword_fill(oracle, num_cus):
    B1 = 64 * num_cus * 16
    for off in (0, 4, 8, 12):
        for count in (0, 1, 3, 4, 5, B1 // 4 - 1, B1 // 4, B1 // 4 + 1, 2 * B1 // 4 + 37):
            buf = np.full(4 * count + 2 * GUARD + 32, 0xEE, dtype=np.uint8)
            addr = buf.ctypes.data + ((-buf.ctypes.data) % 16) + GUARD + off
            b = Bounds(addr, addr + 4 * count, 0, 0)
            assert oracle.oracle_ref_blit_fill(addr, 0xA5C30F1E, count, num_cus, C.byref(b)) == FILL
            want = np.full(buf.size, 0xEE, dtype=np.uint8)
            oracle.oracle_fill32(want.ctypes.data + (addr - buf.ctypes.data), 0xA5C30F1E, count)
            assert np.array_equal(buf, want), (off, count)
    # a misaligned pointer is rejected before anything is written
    buf = np.zeros(64, dtype=np.uint8)
    addr = buf.ctypes.data + ((-buf.ctypes.data) % 16) + 2
    assert oracle.oracle_ref_blit_fill(addr, 1, 4, num_cus, None) == -1
    assert not buf.any()
