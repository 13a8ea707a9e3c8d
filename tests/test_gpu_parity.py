"""Parity of the gfx950 blit kernels with the CPU oracle, through the C ABI.
Bit-exact: every byte of the destination, guard bands included, must equal
what the oracle (host memcpy / dword fill) leaves on the same seeded inputs."""
import ctypes as C
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD = 256
GUARD_BYTE = 0xEE
FILL_VALUE = 0xA5C30F1E  # the benchmark's pattern
MIB = 1 << 20


class Arena:
    """A device buffer with a host mirror.  Offsets are relative to a 256-byte
    aligned device address, so `off & 15` is the device pointer's alignment."""

    def __init__(self, torch, nbytes, fill=None, host=None):
        self.torch = torch
        self.nbytes = nbytes
        self.t = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda:0")
        self.shift = (-self.t.data_ptr()) % 256
        self.base = self.t.data_ptr() + self.shift
        self.view = self.t[self.shift:self.shift + nbytes]
        if host is not None:
            self.view.copy_(torch.from_numpy(host))
        elif fill is not None:
            self.view.fill_(fill)
        torch.cuda.synchronize()

    def fill(self, lo, hi, value):
        """Set bytes on torch's stream and wait: the blit runs on its own stream."""
        self.view[lo:hi].fill_(value)
        self.torch.cuda.synchronize()

    def host(self, lo=0, hi=None):
        hi = self.nbytes if hi is None else hi
        return self.view[lo:hi].cpu().numpy()


def check_ok(capi, st, what):
    assert st == capi.SUCCESS, "%s returned 0x%x" % (what, st)


def run_copy_case(capi, blit, oracle, src_arena, src_host, dst_arena, s_off, d_off, n):
    """Copy n bytes; compare [d_off-GUARD, d_off+n+GUARD) with the oracle."""
    lo, hi = d_off - GUARD, d_off + n + GUARD
    assert lo >= 0 and hi <= dst_arena.nbytes and s_off + n <= src_arena.nbytes
    dst_arena.fill(lo, hi, GUARD_BYTE)
    check_ok(capi, blit.copy(dst_arena.base + d_off, src_arena.base + s_off, n), "copy")
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst_arena.host(lo, hi)
    want = np.full(hi - lo, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data + GUARD, src_host.ctypes.data + s_off, n)
    if not np.array_equal(got, want):
        bad = np.nonzero(got != want)[0]
        raise AssertionError("copy mismatch s_off=%d d_off=%d n=%d: %d bytes differ, first at %d "
                             "(relative to dst start: %d), plan=%s"
                             % (s_off, d_off, n, bad.size, bad[0], bad[0] - GUARD,
                                blit.last_plan().as_dict()))


@pytest.fixture(scope="module")
def arenas(torch_cuda, rand):
    """64 MiB (+ slack) source with seeded bytes and a destination of the same size."""
    n = 64 * MIB + 2 * MIB
    src_host = rand(n, 0xB1170004)
    src = Arena(torch_cuda, n, host=src_host)
    dst = Arena(torch_cuda, n, fill=GUARD_BYTE)
    return src, src_host, dst


# ---------------------------------------------------------------- aligned copy

@pytest.mark.parametrize("n", [4096 * 4 ** k for k in range(8)])  # 4 KiB .. 64 MiB
def test_aligned_copy_sweep(capi, blit, oracle, arenas, n):
    src, src_host, dst = arenas
    run_copy_case(capi, blit, oracle, src, src_host, dst, 0, GUARD, n)
    p = blit.last_plan()
    assert p.kernel == capi.KERNEL_COPY and p.head_bytes == 0 and p.tail_bytes == 0


def test_reference_perf_sizes(capi, blit, oracle, arenas):
    """Sizes of rocrtst's Memory_Async_Copy (memory_async_copy.h:207-216), to 32 MiB."""
    src, src_host, dst = arenas
    for k in range(16):
        run_copy_case(capi, blit, oracle, src, src_host, dst, 0, GUARD, 1024 << k)


@pytest.mark.parametrize("n", [256 * MIB, 1 << 30])
def test_aligned_copy_large_full_compare(capi, blit, oracle, rand, torch_cuda, n):
    """Headline size, every byte against the oracle."""
    torch = torch_cuda
    src_host = rand(n, 0xB1170003)
    src = Arena(torch, n, host=src_host)
    dst = Arena(torch, n + 2 * GUARD, fill=GUARD_BYTE)
    check_ok(capi, blit.copy(dst.base + GUARD, src.base, n), "copy")
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst.host()
    want = np.full(n + 2 * GUARD, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data + GUARD, src_host.ctypes.data, n)
    assert np.array_equal(got, want)


def test_copy_4gib_properties(capi, blit, oracle, rand, torch_cuda):
    """Maximum sweep size.  A host compare of 4 GiB is slow, so: the source is a
    64 MiB seeded block repeated 64 times; after the copy every 64 MiB slice of
    the destination must hash like the oracle's copy of that block, the device
    compare dst == src must hold, and the guards must be intact."""
    torch = torch_cuda
    n = 4 << 30
    blk = 64 * MIB
    block_host = rand(blk, 0xB1170033)
    src = Arena(torch, n)
    block_dev = torch.from_numpy(block_host).to("cuda:0")
    for i in range(n // blk):
        src.view[i * blk:(i + 1) * blk].copy_(block_dev)
    torch.cuda.synchronize()
    dst = Arena(torch, n + 2 * GUARD, fill=GUARD_BYTE)
    check_ok(capi, blit.copy(dst.base + GUARD, src.base, n), "copy")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert bool((dst.view[:GUARD] == GUARD_BYTE).all()) and bool((dst.view[GUARD + n:] == GUARD_BYTE).all())
    assert torch.equal(dst.view[GUARD:GUARD + n], src.view)
    want = np.empty(blk, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data, block_host.ctypes.data, blk)
    want_hash = oracle.oracle_fnv1a64(want.ctypes.data, 1 << 16)
    for i in (0, 1, 31, 62, 63):
        got = dst.host(GUARD + i * blk, GUARD + (i + 1) * blk)
        assert np.array_equal(got, want), "slice %d differs" % i
        assert oracle.oracle_fnv1a64(got.ctypes.data, 1 << 16) == want_hash
    p = blit.last_plan()
    assert p.grid * (p.wg_size // 64) >= -(-p.body_vecs // (64 * p.unroll))
    # eight launches of 512 MiB, except on a queue the engine does not own
    assert p.pieces == (1 if getattr(blit, "borrowed", None) is not None else 8)


def test_copy_and_fill_beyond_the_largest_grid(capi, fresh_tuning, oracle, rand, torch_cuda):
    """33 GiB, twice.  As one launch (the tuning asks for it; a borrowed queue
    gets one anyway) it has more 1 KiB tiles than a grid can have workgroups (an
    AQL packet counts work-items in 32 bits), so the grid is capped and waves
    take a second tile.  By default it goes out in 32 pieces of a little over
    1 GiB.  Same properties as at 4 GiB, compared on the device in 1 GiB slices,
    with the 64 MiB blocks around the wrap of the grid, or around the seams
    between pieces, also compared on the host."""
    blit = fresh_tuning
    torch = torch_cuda
    gib = 1 << 30
    n = 33 * gib + 12345 * 16
    blk = 64 * MIB
    free, _ = torch.cuda.mem_get_info()
    if free < 2 * n + 4 * gib:
        pytest.skip("needs %d GiB of free device memory" % ((2 * n + 4 * gib) >> 30))
    block_host = rand(blk, 0xB1170034)
    src = Arena(torch, n)
    block_dev = torch.from_numpy(block_host).to("cuda:0")
    for lo in range(0, n, blk):
        m = min(blk, n - lo)
        src.view[lo:lo + m].copy_(block_dev[:m])
    torch.cuda.synchronize()
    dst = Arena(torch, n + 2 * GUARD, fill=GUARD_BYTE)
    want = np.empty(blk, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data, block_host.ctypes.data, blk)
    borrowed = getattr(blit, "borrowed", None) is not None
    for one_launch in (True, False):
        if one_launch:
            blit.set_tuning(copy_piece_mib=1)
        else:
            blit.set_tuning()
            dst.fill(0, n + 2 * GUARD, GUARD_BYTE)
        check_ok(capi, blit.copy(dst.base + GUARD, src.base, n), "copy")
        check_ok(capi, blit.synchronize(), "synchronize")
        p = blit.last_plan()
        if one_launch or borrowed:
            assert p.pieces == 1
            tiles = -(-(p.body_vecs + p.lead_vecs) // (64 * p.unroll))
            waves = p.grid * (p.wg_size // 64)
            assert waves < tiles, "the case is meant to cap the grid: %s" % p.as_dict()
            wrap = waves * 64 * p.unroll * 16 // blk      # the 64 MiB block in which the second round of tiles starts
            blocks = (0, wrap - 1, wrap, wrap + 1, n // blk - 1)
        else:
            count, piece = capi.plan_copy_pieces(n)
            assert p.pieces == count == 32 and gib < piece < gib + 64 * MIB
            # a seam lies inside block k * piece // blk
            blocks = sorted({0, n // blk - 1} | {k * piece // blk for k in (1, 2, 16, 31)})
        assert bool((dst.view[:GUARD] == GUARD_BYTE).all()) and bool((dst.view[GUARD + n:] == GUARD_BYTE).all())
        for lo in range(0, n, gib):
            m = min(gib, n - lo)
            assert torch.equal(dst.view[GUARD + lo:GUARD + lo + m], src.view[lo:lo + m]), \
                "slice at %d GiB differs (one launch: %s)" % (lo >> 30, one_launch)
        for i in blocks:
            got = dst.host(GUARD + i * blk, GUARD + (i + 1) * blk)
            assert np.array_equal(got, want), "block %d differs (one launch: %s)" % (i, one_launch)
    del src
    torch.cuda.empty_cache()
    # the fill, over what the copy left
    count = n // 4
    check_ok(capi, blit.fill32(dst.base + GUARD, FILL_VALUE, count), "fill32")
    check_ok(capi, blit.synchronize(), "synchronize")
    p = blit.last_plan()
    assert p.grid * (p.wg_size // 64) < -(-(p.body_vecs + p.lead_vecs) // (64 * p.unroll)), p.as_dict()
    assert bool((dst.view[:GUARD] == GUARD_BYTE).all()) and bool((dst.view[GUARD + n:] == GUARD_BYTE).all())
    words = dst.view[GUARD:GUARD + n].view(torch.int32)
    pattern = FILL_VALUE - (1 << 32)
    for lo in range(0, count, gib // 4):
        assert bool((words[lo:lo + gib // 4] == pattern).all()), "fill slice at %d GiB differs" % (lo >> 28)


# -------------------------------------------------------------- misaligned copy

def _log_uniform_lengths(rng, k, max_bytes):
    return np.maximum(1, np.floor(2.0 ** (np.log2(max_bytes) * rng.random(k)))).astype(np.int64)


def test_misaligned_all_256_offset_pairs(capi, blit, oracle, arenas):
    """Every (src & 15, dst & 15) pair: 8 lengths drawn log-uniformly from 1 B to
    64 MiB and used as drawn, and one more drawn log-uniformly from 4 MiB to
    64 MiB, so that every pair meets the streaming shapes of the heuristics
    too; destination window and guards compared with the oracle every time."""
    src, src_host, dst = arenas
    rng = np.random.default_rng(0xB1170004)
    for so in range(16):
        for do in range(16):
            lens = list(_log_uniform_lengths(rng, 8, 64 * MIB))
            lens.append(int(4 * MIB * 16.0 ** rng.random()))
            for n in lens:
                n = min(int(n), 64 * MIB)
                run_copy_case(capi, blit, oracle, src, src_host, dst, 512 + so, GUARD + 16 + do, n)
                p = blit.last_plan()
                assert p.byte_shift == (so - do) % 4


def test_misaligned_tiny_lengths_every_pair(capi, blit, oracle, arenas):
    """Lengths 1..40 for every offset pair: all head/tail/body splits near zero.
    Each length has its own 128-byte slot, so one compare covers a pair."""
    src, src_host, dst = arenas
    slot = 128
    span = GUARD + 41 * slot + GUARD
    for so in range(16):
        for do in range(16):
            dst.fill(0, span, GUARD_BYTE)
            want = np.full(span, GUARD_BYTE, dtype=np.uint8)
            for n in range(1, 41):
                d_off = GUARD + n * slot + do
                s_off = 1024 + n * 64 + so
                check_ok(capi, blit.copy(dst.base + d_off, src.base + s_off, n), "copy")
                oracle.oracle_copy(want.ctypes.data + d_off, src_host.ctypes.data + s_off, n)
            check_ok(capi, blit.synchronize(), "synchronize")
            got = dst.host(0, span)
            if not np.array_equal(got, want):
                bad = np.nonzero(got != want)[0]
                raise AssertionError("so=%d do=%d: first bad byte at %d (slot %d)"
                                     % (so, do, bad[0], (bad[0] - GUARD) // slot))


@pytest.mark.parametrize("unroll,wg", [(0, 0), (1, 64), (2, 256), (4, 128)])
def test_every_destination_offset_within_256_bytes(capi, fresh_tuning, oracle, arenas, unroll, wg):
    """Tiles are anchored at 256-byte boundaries of the destination: every
    16-byte step of (dst & 255), plus byte offsets, with lengths around one and
    several tiles, so that the cut first and last tiles meet every shape."""
    blit = fresh_tuning
    src, src_host, dst = arenas
    if unroll:
        blit.set_tuning(unroll=unroll, wg_size=wg)
    tile = 1024 * (unroll or 1)
    lengths = [1, 17, 200, 255, 256, 257, tile - 16, tile, tile + 16, 2 * tile + 5, 5 * tile - 1, 33 * tile + 100]
    for step in range(16):
        for extra, so in ((0, 0), (0, 4), (5, 0), (11, 2)):
            d_off = 2 * GUARD + 16 * step + extra
            for n in lengths:
                run_copy_case(capi, blit, oracle, src, src_host, dst, 2048 + so, d_off, n)
                p = blit.last_plan()
                assert p.lead_vecs == ((dst.base + d_off + p.head_bytes) % 256) // 16


def test_fill_every_destination_offset_within_256_bytes(capi, fresh_tuning, oracle, arenas):
    blit = fresh_tuning
    _, _, dst = arenas
    for unroll in (0, 2, 4):
        if unroll:
            blit.set_tuning(unroll=unroll, wg_size=128)
        tile = 256 * (unroll or 1)  # dwords
        for off in range(0, 256, 4):
            for count in (1, 5, 63, tile - 4, tile, tile + 4, 3 * tile + 7):
                run_fill_case(capi, blit, oracle, dst, 2 * GUARD + off, count, FILL_VALUE ^ off)


@pytest.mark.parametrize("so,do", [(0, 0), (4, 0), (0, 8), (1, 0), (0, 2), (3, 0), (7, 13), (15, 1), (5, 5)])
def test_misaligned_1gib_headline(capi, blit, oracle, rand, torch_cuda, so, do):
    """1 GiB per representative class of ((so-do) & 3, (so-do) & 12); every
    byte against the oracle."""
    torch = torch_cuda
    n = (1 << 30) - 64
    src_host = rand(n + 64, 0xB1170044 + so * 16 + do)
    src = Arena(torch, n + 64, host=src_host)
    dst = Arena(torch, n + 2 * GUARD + 64, fill=GUARD_BYTE)
    check_ok(capi, blit.copy(dst.base + GUARD + do, src.base + so, n), "copy")
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst.host()
    want = np.full(dst.nbytes, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data + GUARD + do, src_host.ctypes.data + so, n)
    assert np.array_equal(got, want)


def test_random_copies_and_shapes(capi, fresh_tuning, oracle, arenas):
    """Seeded random walk over offsets, lengths and launch shapes (the seed and
    case are in the failure message)."""
    blit = fresh_tuning
    src, src_host, dst = arenas
    rng = np.random.default_rng(0xF00D)
    for case in range(600):
        so = int(rng.integers(0, 4096))
        do = GUARD + int(rng.integers(0, 4096))
        n = int(max(1, np.floor(2.0 ** (24 * rng.random()))))  # 1 B .. 16 MiB
        if case % 3 == 0:
            blit.set_tuning()
        else:
            blit.set_tuning(wg_size=int(rng.choice([64, 128, 256, 512, 1024])), unroll=int(rng.choice([1, 2, 4])),
                            nt_load=int(rng.integers(1, 3)), store_policy=int(rng.integers(1, 5)),
                            max_grid=int(rng.choice([0, 0, 3, 64])))
        try:
            run_copy_case(capi, blit, oracle, src, src_host, dst, so, do, n)
        except AssertionError as e:
            raise AssertionError("fuzz case %d (so=%d do=%d n=%d): %s" % (case, so, do, n, e))


def test_copy_8gib_grid_limits(capi, blit, torch_cuda):
    """Twice the largest sweep size: 64-bit indexing and the grid's work-item
    limit (the plan caps the grid, waves then stride over the tiles)."""
    torch = torch_cuda
    n = 8 << 30
    src = Arena(torch, n)
    dst = Arena(torch, n + 2 * GUARD, fill=GUARD_BYTE)
    # a cheap varied pattern: 32-bit counter
    src.view.view(torch.int32).copy_(torch.arange(n // 4, dtype=torch.int32, device="cuda:0"))
    torch.cuda.synchronize()
    check_ok(capi, blit.copy(dst.base + GUARD + 5, src.base + 2, n - 16), "copy")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert torch.equal(dst.view[GUARD + 5:GUARD + 5 + n - 16], src.view[2:2 + n - 16])
    assert bool((dst.view[:GUARD + 5] == GUARD_BYTE).all())
    assert bool((dst.view[GUARD + 5 + n - 16:] == GUARD_BYTE).all())
    p = blit.last_plan()
    assert p.grid * p.wg_size < 2 ** 31
    assert p.pieces == (1 if getattr(blit, "borrowed", None) is not None else 16)


# ------------------------------------------------------------------------- fill

def run_fill_case(capi, blit, oracle, dst, d_off, count, value):
    lo, hi = d_off - GUARD, d_off + 4 * count + GUARD
    dst.fill(lo, hi, GUARD_BYTE)
    check_ok(capi, blit.fill32(dst.base + d_off, value, count), "fill32")
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst.host(lo, hi)
    want = np.full(hi - lo, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_fill32(want.ctypes.data + GUARD, value, count)
    if not np.array_equal(got, want):
        bad = np.nonzero(got != want)[0]
        raise AssertionError("fill mismatch d_off=%d count=%d: %d bytes differ, first at %d, plan=%s"
                             % (d_off, count, bad.size, bad[0] - GUARD, blit.last_plan().as_dict()))


@pytest.mark.parametrize("nbytes", [4096 * 4 ** k for k in range(8)])
def test_fill_sweep(capi, blit, oracle, arenas, nbytes):
    _, _, dst = arenas
    run_fill_case(capi, blit, oracle, dst, GUARD, nbytes // 4, FILL_VALUE)


@pytest.mark.parametrize("value", [0xabcdef12, 0xba5eba11, 0xfeed5a1e, 0xbaadf00d])
def test_fill_reference_patterns(capi, blit, oracle, arenas, value):
    """async_mem_copy.cc:62-65: fill, then every dword must equal the pattern."""
    _, _, dst = arenas
    run_fill_case(capi, blit, oracle, dst, GUARD, MIB // 4, value)


def test_fill_offsets_and_odd_counts(capi, blit, oracle, arenas):
    _, _, dst = arenas
    for off in (0, 4, 8, 12):
        for count in list(range(1, 20)) + [63, 64, 65, 255, 257, 1023, 1025, 65537, (MIB // 4) + 3, (9 * MIB // 4) + 1]:
            run_fill_case(capi, blit, oracle, dst, GUARD + off, count, FILL_VALUE ^ count)


@pytest.mark.parametrize("count", [1 << 26, 1 << 28])  # 256 MiB (a point of the sweep), 1 GiB (the headline)
def test_fill_large_full_compare(capi, blit, oracle, torch_cuda, count):
    torch = torch_cuda
    dst = Arena(torch, 4 * count + 2 * GUARD, fill=GUARD_BYTE)
    # pre-fill with the complement so that an unwritten dword shows
    dst.view[GUARD:GUARD + 4 * count].view(torch.int32).fill_(~FILL_VALUE & 0x7fffffff)
    torch.cuda.synchronize()
    check_ok(capi, blit.fill32(dst.base + GUARD, FILL_VALUE, count), "fill32")
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst.host()
    want = np.full(dst.nbytes, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_fill32(want.ctypes.data + GUARD, FILL_VALUE, count)
    assert np.array_equal(got, want)


def test_fill_4gib_properties(capi, blit, torch_cuda):
    torch = torch_cuda
    count = 1 << 30
    dst = Arena(torch, 4 * count + 2 * GUARD, fill=GUARD_BYTE)
    check_ok(capi, blit.fill32(dst.base + GUARD, FILL_VALUE, count), "fill32")
    check_ok(capi, blit.synchronize(), "synchronize")
    body = dst.view[GUARD:GUARD + 4 * count].view(torch.int32)
    want = FILL_VALUE - (1 << 32)  # as int32
    assert int(body.min()) == want and int(body.max()) == want
    assert bool((dst.view[:GUARD] == GUARD_BYTE).all()) and bool((dst.view[GUARD + 4 * count:] == GUARD_BYTE).all())


# --------------------------------------------------------------- kernel variants

@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("wg", [64, 256, 1024])
def test_every_copy_variant_is_exact(capi, fresh_tuning, oracle, arenas, unroll, wg):
    """Each instantiation (unroll x load policy x store policy x realign) and a
    capped grid (waves striding over tiles) against the oracle."""
    blit = fresh_tuning
    src, src_host, dst = arenas
    n = 3 * MIB + 4321
    for nt_load in (1, 2):
        for policy in range(4):
            for max_grid in (0, 7):
                blit.set_tuning(wg_size=wg, unroll=unroll, nt_load=nt_load, store_policy=policy + 1,
                                max_grid=max_grid)
                for so, do in ((0, 0), (4, 8), (1, 0), (6, 3)):
                    run_copy_case(capi, blit, oracle, src, src_host, dst, 64 + so, GUARD + do, n)
                    p = blit.last_plan()
                    assert (p.wg_size, p.unroll, p.nt_load, p.store_policy) == (wg, unroll, nt_load - 1, policy)
                    if max_grid:
                        assert p.grid == max_grid


@pytest.mark.parametrize("unroll", [1, 2, 4])
def test_every_fill_variant_is_exact(capi, fresh_tuning, oracle, arenas, unroll):
    blit = fresh_tuning
    _, _, dst = arenas
    for wg in (64, 256, 1024):
        for policy in range(4):
            for max_grid in (0, 5):
                blit.set_tuning(wg_size=wg, unroll=unroll, store_policy=policy + 1, max_grid=max_grid)
                for off in (0, 4):
                    run_fill_case(capi, blit, oracle, dst, GUARD + off, (2 * MIB + 1236) // 4, FILL_VALUE)


@pytest.mark.parametrize("xcd_run", [2, 5, 36, 288])
def test_permuted_launches_are_exact(capi, fresh_tuning, oracle, arenas, xcd_run):
    """Launches whose workgroups take their tiles in runs per XCD instead of
    launch order: a permutation of the same tiles, so the same bytes.  Grids
    that are not whole rounds of 8 runs, capped grids (waves striding over
    tiles) and the two copy kernels, the fill and the batch."""
    blit = fresh_tuning
    src, src_host, dst = arenas
    for wg, unroll, max_grid in ((64, 1, 0), (256, 2, 0), (64, 2, 0), (128, 1, 1000), (64, 4, 333)):
        blit.set_tuning(wg_size=wg, unroll=unroll, max_grid=max_grid, xcd_run=xcd_run)
        for so, do, n in ((0, 0, 5 * MIB + 12345), (3, 9, 7 * MIB + 1), (64, 16, 2 * MIB + 77), (1, 0, 40000)):
            run_copy_case(capi, blit, oracle, src, src_host, dst, 64 + so, GUARD + do, n)
            assert blit.last_plan().xcd_run == xcd_run
        run_fill_case(capi, blit, oracle, dst, GUARD + 4, (3 * MIB + 1236) // 4, FILL_VALUE)
        assert blit.last_plan().xcd_run == xcd_run
    blit.set_tuning(xcd_run=xcd_run)
    rng = np.random.default_rng(77 + xcd_run)
    n = 4000
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, max_len=64 << 10)
    dst.fill(0, total, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert blit.last_plan().xcd_run == xcd_run
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))


def test_large_copies_with_the_heuristic_runs(capi, blit, oracle, rand, torch_cuda):
    """At the sizes where the heuristics permute the launch by themselves
    (from 48 MiB with a byte offset, from 80 MiB without): every byte and the
    guards against the oracle."""
    torch = torch_cuda
    n = 160 * MIB + 4099
    src_host = rand(n + 512, 0xB1170077)
    src = Arena(torch, n + 512, host=src_host)
    dst = Arena(torch, n + 1024, fill=GUARD_BYTE)
    for so, do in ((0, 0), (64, 128), (3, 9)):
        run_copy_case(capi, blit, oracle, src, src_host, dst, so, GUARD + do, n)
        p = blit.last_plan()
        assert p.xcd_run == (288 if (so - do) % 4 else 576), p.as_dict()


@pytest.mark.parametrize("so", [0, 1, 2, 3, 7, 64])
def test_offsets_at_the_sizes_of_the_heuristic_runs(capi, blit, oracle, arenas, so):
    """50-60 MiB, where the byte-offset copies (and from 80 MiB the others) are
    launched in XCD runs by the heuristics: every byte shift against destination
    residues that give the first tile a head, a lead or neither."""
    src, src_host, dst = arenas
    for do, n in ((0, 50 * MIB + 1), (5, 49 * MIB + 4321), (16 * 9 + 3, 60 * MIB - 7)):
        run_copy_case(capi, blit, oracle, src, src_host, dst, 256 + so, GUARD + do, n)
        p = blit.last_plan()
        assert p.byte_shift == (so - do) % 4
        assert p.xcd_run == (288 if p.byte_shift else 0), p.as_dict()


# ---------------------------------------------------------------------- batched

def _make_batch(capi, rng, src, dst, n, min_len=64, max_len=256 << 10):
    """Copies carved sequentially: stride = len rounded up to 256 + 256 guard."""
    lens = np.floor(min_len * 2.0 ** (np.log2(max_len / min_len) * rng.random(n))).astype(np.int64)
    so = rng.integers(0, 16, n)
    do = rng.integers(0, 16, n) + 16 * rng.integers(0, 16, n)  # any destination offset within 256 bytes
    stride = ((lens + 255) // 256) * 256 + 512
    offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
    total = int(offs[-1] + stride[-1] + 256)
    assert total <= src.nbytes and total <= dst.nbytes, total
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst.base + int(offs[i] + do[i])
        descs[i].src = src.base + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    return descs, lens, offs, so, do, total


class _Window:
    """An arena from `offset` on, for _make_batch."""

    def __init__(self, arena, offset):
        self.base = arena.base + offset
        self.nbytes = arena.nbytes - offset


def _grid_chunks(p):
    """Chunks a batch launch has waves for: four waves to a 4 KiB chunk."""
    return p.grid * (p.wg_size // 64) // (4 // p.unroll)


def _expect_batch(oracle, src_host, total, lens, offs, so, do):
    want = np.full(total, GUARD_BYTE, dtype=np.uint8)
    for i in range(len(lens)):
        oracle.oracle_copy(want.ctypes.data + int(offs[i] + do[i]),
                           src_host.ctypes.data + int(offs[i] + so[i]), int(lens[i]))
    return want


@pytest.mark.parametrize("n", [1, 2, 63, 1000])
def test_batch_small(capi, blit, oracle, arenas, n):
    src, src_host, dst = arenas
    rng = np.random.default_rng(n)
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n)
    dst.fill(0, total, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))
    assert blit.last_plan().kernel == capi.KERNEL_COPY_BATCH


def test_batch_edge_lengths(capi, blit, oracle, arenas):
    """Zero-length entries, lengths 1..48 and lengths around the 4 KiB chunk."""
    src, src_host, dst = arenas
    lens = [0, 0] + list(range(1, 49)) + [0] + [4095, 4096, 4097, 4096 + 15, 8192, 8193, 12288 + 31, 0]
    n = len(lens)
    rng = np.random.default_rng(99)
    so = rng.integers(0, 16, n)
    do = rng.integers(0, 16, n)
    lens = np.array(lens, dtype=np.int64)
    stride = ((lens + 255) // 256) * 256 + 256
    offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
    total = int(offs[-1] + stride[-1] + 256)
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst.base + int(offs[i] + do[i])
        descs[i].src = src.base + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    dst.fill(0, total, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))


def test_batch_with_copies_beyond_one_mib(capi, blit, oracle, arenas):
    """Copies longer than 1 MiB are cut into pieces at 1 MiB boundaries of the
    destination on the host; mixed here with short ones, at odd offsets."""
    src, src_host, dst = arenas
    lens = [5 * MIB + 3, 77, MIB, MIB + 1, 3 * MIB - 17, 4096, 2 * MIB, 1, 9 * MIB + 12345, 300000]
    so = [3, 0, 1, 15, 7, 2, 0, 9, 5, 11]
    do = [9, 1, 0, 255, 130, 16, 0, 3, 77, 200]
    offs, at = [], 256
    for n in lens:
        offs.append(at)
        at += (n + 255) // 256 * 256 + 512
    total = at + 256
    assert total <= dst.nbytes
    descs = (capi.Desc * len(lens))()
    for i, n in enumerate(lens):
        descs[i].dst = dst.base + offs[i] + do[i]
        descs[i].src = src.base + offs[i] + so[i]
        descs[i].bytes = n
    dst.fill(0, total, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(descs, len(lens)), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    want = _expect_batch(oracle, src_host, total, np.array(lens), np.array(offs), np.array(so), np.array(do))
    assert np.array_equal(dst.host(0, total), want)


def test_batches_in_a_row_with_different_descriptors(capi, blit, oracle, arenas):
    """Eight batches back to back on one engine, each with its own descriptors,
    submitted without waiting in between: the two staging buffers are rewritten
    by the host while earlier batches run, and every batch must still read its
    own descriptors (not a cached image of the buffer's previous content)."""
    src, src_host, dst = arenas
    # disjoint destination windows of 8 MiB, one per batch
    window = 8 * MIB
    batches = []
    for k in range(8):
        rng = np.random.default_rng(9000 + k)
        n = int(rng.integers(200, 1500))
        lens = np.floor(64 * 2.0 ** (10 * rng.random(n))).astype(np.int64)      # 64 B .. 64 KiB
        stride = ((lens + 255) // 256) * 256 + 512
        keep = np.cumsum(stride) + 512 < window
        lens, stride, n = lens[keep], stride[keep], int(keep.sum())
        offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256 + k * window
        so, do = rng.integers(0, 16, n), rng.integers(0, 256, n)
        descs = (capi.Desc * n)()
        for i in range(n):
            descs[i].dst = dst.base + int(offs[i] + do[i])
            descs[i].src = src.base + int(offs[i] + so[i])
            descs[i].bytes = int(lens[i])
        batches.append((descs, n, lens, offs, so, do))
    dst.fill(0, 8 * window, GUARD_BYTE)
    for descs, n, *_ in batches:
        check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    want = np.full(8 * window, GUARD_BYTE, dtype=np.uint8)
    for _, n, lens, offs, so, do in batches:
        for i in range(n):
            oracle.oracle_copy(want.ctypes.data + int(offs[i] + do[i]), src_host.ctypes.data + int(offs[i] + so[i]),
                               int(lens[i]))
    assert np.array_equal(dst.host(0, 8 * window), want)


def test_batch_device_resident_descriptors(capi, blit, oracle, arenas, torch_cuda):
    torch = torch_cuda
    src, src_host, dst = arenas
    n = 777
    rng = np.random.default_rng(4242)
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n)
    raw = np.frombuffer(bytes(descs), dtype=np.uint8).copy()
    descs_dev = torch.from_numpy(raw).to("cuda:0")
    dst.fill(0, total, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch(descs_dev.data_ptr(), n, on_device=True), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))


def _to_device(torch, descs):
    raw = np.frombuffer(bytes(descs), dtype=np.uint8).copy()
    return torch.from_numpy(raw).to("cuda:0")


@pytest.mark.parametrize("n,slack", [(1, 0), (65, 0), (777, 0), (777, 64 * MIB), (3000, 1)])
def test_batch_bounded_device_resident_descriptors(capi, blit, oracle, arenas, torch_cuda, n, slack):
    """Device-resident descriptors with a bound on their total size, exact and
    loose: the per-chunk kernel behind a device-side prefix sum."""
    torch = torch_cuda
    src, src_host, dst = arenas
    rng = np.random.default_rng(5000 + n)
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, max_len=64 << 10)
    descs_dev = _to_device(torch, descs)
    dst.fill(0, total, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch_bounded(descs_dev.data_ptr(), n, int(lens.sum()) + slack), "copy_batch_bounded")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))
    assert blit.last_plan().kernel == capi.KERNEL_COPY_BATCH


def test_batch_bounded_edge_lengths_and_long_copies(capi, blit, oracle, arenas, torch_cuda):
    """Zero-length entries (whole waves of them too), lengths around the 16-byte
    vector and the 4 KiB chunk, and copies of several MiB, which nothing cuts
    into pieces on this path."""
    torch = torch_cuda
    src, src_host, dst = arenas
    lens = ([0] * 70 + list(range(1, 49)) + [0, 4095, 4096, 4097, 4096 + 15, 8192, 8193, 12288 + 31, 0]
            + [5 * MIB + 3, 0, 77, MIB + 1, 3 * MIB - 17] + [0] * 130 + [9, 2 * MIB])
    n = len(lens)
    rng = np.random.default_rng(4711)
    so = rng.integers(0, 16, n)
    do = rng.integers(0, 256, n)
    lens = np.array(lens, dtype=np.int64)
    stride = ((lens + 255) // 256) * 256 + 512
    offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
    total = int(offs[-1] + stride[-1] + 256)
    assert total <= dst.nbytes
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst.base + int(offs[i] + do[i])
        descs[i].src = src.base + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    descs_dev = _to_device(torch, descs)
    dst.fill(0, total, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch_bounded(descs_dev.data_ptr(), n, int(lens.sum())), "copy_batch_bounded")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))


def test_batch_bounded_all_empty_and_arguments(capi, blit, arenas, torch_cuda):
    torch = torch_cuda
    src, _, dst = arenas
    n = 100
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst.base + 512 * i
        descs[i].src = src.base + 512 * i
        descs[i].bytes = 0
    descs_dev = _to_device(torch, descs)
    dst.fill(0, 512 * n, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch_bounded(descs_dev.data_ptr(), n, 1), "copy_batch_bounded")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert (dst.host(0, 512 * n) == GUARD_BYTE).all()
    inv = capi.ERROR_INVALID_ARGUMENT
    assert blit.copy_batch_bounded(descs_dev.data_ptr(), n, 0) == inv
    assert blit.copy_batch_bounded(None, n, 4096) == inv
    assert blit.copy_batch_bounded(descs_dev.data_ptr(), n, 1 << 62) == inv   # more records than 32 bits index
    assert blit.copy_batch_bounded(None, 0, 0) == capi.SUCCESS
    check_ok(capi, blit.synchronize(), "synchronize")


@pytest.mark.parametrize("n,min_len,max_len,bound", [(64, 32 << 10, 64 << 10, 4096), (2100, 8 << 10, 24 << 10, 1),
                                                     (1030, 64, 200 << 10, 50000)])
def test_batch_bound_exceeded_costs_speed_not_bytes(capi, blit, oracle, arenas, torch_cuda, n, min_len, max_len, bound):
    """A bound the descriptors exceed leaves most chunks without a record: the
    copy kernel then finds them through the prefix sums (across groups of 1024
    copies, around copies of no bytes), with fewer waves than chunks.  The
    result is still the full batch, and the guards."""
    torch = torch_cuda
    src, src_host, dst = arenas
    rng = np.random.default_rng(808 + n)
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, min_len=min_len, max_len=max_len)
    for i in range(0, n, 7):       # copies of no bytes share their first chunk with their successor
        descs[i].bytes = 0
        lens[i] = 0
    if n > 1024:
        for i in range(1024 - 3, 1024 + 2):   # also at the end of a group and the start of the next
            descs[i].bytes = 0
            lens[i] = 0
    descs_dev = _to_device(torch, descs)
    dst.fill(0, total, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch_bounded(descs_dev.data_ptr(), n, bound), "copy_batch_bounded")
    check_ok(capi, blit.synchronize(), "synchronize")
    p = blit.last_plan()
    assert _grid_chunks(p) < int((lens // 4096).sum()), "the case is meant to leave chunks without a wave of their own"
    assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do))


def test_batch_unbounded_beyond_what_the_library_assumes(capi, blit, oracle, rand, torch_cuda):
    """Device-resident descriptors without a bound: the grid assumes 32 KiB a
    copy and the record buffer twice that (65,536 records at least).  Four
    copies of 70-80 MiB have 17 times the records: the rest is looked up."""
    torch = torch_cuda
    n = 4
    size = n * 80 * MIB + MIB
    src_host = rand(size, 0xB1170909)
    src = Arena(torch, size, host=src_host)
    dst = Arena(torch, size, fill=GUARD_BYTE)
    rng = np.random.default_rng(909)
    descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, min_len=70 * MIB, max_len=80 * MIB)
    assert int((lens // 4096).sum()) > 65536
    descs_dev = _to_device(torch, descs)
    dst.fill(0, total, GUARD_BYTE)
    torch.cuda.synchronize()
    check_ok(capi, blit.copy_batch(descs_dev.data_ptr(), n, on_device=True), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert _grid_chunks(blit.last_plan()) * 2 < int((lens // 4096).sum())
    got = dst.host(0, total)
    want = _expect_batch(oracle, src_host, total, lens, offs, so, do)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("path", ["hip", "aql"])
def test_batch_unbounded_sizes_itself_by_the_batch_before(capi, pkg, oracle, arenas, torch_cuda, path):
    """Without a bound the first device-resident batch on an engine is launched
    for 8 chunks a copy; its copy kernel leaves the numbers of copies and chunks
    in host memory and the next batch is launched for the same chunks per copy
    less 1.5 %.  Bytes are the oracle's whatever the guess."""
    torch = torch_cuda
    src, src_host, dst = arenas
    eng = capi.Blit(0) if path == "hip" else pkg.aql.AqlBlit(0)
    try:
        rng = np.random.default_rng(4711)
        n = 512
        descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, min_len=60 << 10, max_len=68 << 10)
        chunks = sum((int(d.dst) % 4096 % 256 // 16 * 16 + int(d.bytes) + 4095) // 4096 for d in descs)
        dev = _to_device(torch, descs)
        want = _expect_batch(oracle, src_host, total, lens, offs, so, do)
        grids = []
        for call in range(3):
            dst.fill(0, total, GUARD_BYTE)
            torch.cuda.synchronize()
            check_ok(capi, eng.copy_batch(dev.data_ptr(), n, on_device=True), "copy_batch")
            check_ok(capi, eng.synchronize(), "synchronize")
            grids.append(_grid_chunks(eng.last_plan()))
            assert np.array_equal(dst.host(0, total), want), "call %d" % call
        assert grids[0] == 8 * n
        # 16 or 17 chunks a copy: the second and third launches follow what the first one counted
        assert grids[1] == grids[2] and abs(grids[1] - chunks * 63 // 64 - 1) <= n // 4, (grids, chunks)
        # a batch of short copies next: sized by the long ones once, by itself afterwards
        n2 = 300
        descs2, lens2, offs2, so2, do2, total2 = _make_batch(capi, rng, src, dst, n2, min_len=64, max_len=512)
        dev2 = _to_device(torch, descs2)
        want2 = _expect_batch(oracle, src_host, total2, lens2, offs2, so2, do2)
        for call in range(2):
            dst.fill(0, total2, GUARD_BYTE)
            torch.cuda.synchronize()
            check_ok(capi, eng.copy_batch(dev2.data_ptr(), n2, on_device=True), "copy_batch")
            check_ok(capi, eng.synchronize(), "synchronize")
            grids.append(_grid_chunks(eng.last_plan()))
            assert np.array_equal(dst.host(0, total2), want2), "short copies, call %d" % call
        assert grids[3] > 10 * n2 and grids[4] <= 2 * n2 + 32, grids
    finally:
        eng.close()


def test_batch_of_many_short_copies_is_staged_as_it_is(capi, blit, oracle, arenas, torch_cuda):
    """From 4096 host-resident descriptors of a few KiB on average the host does
    not walk them but stages them as they are, and the GPU takes them from there
    like device-resident ones (sized by the bytes the host added up).  Three
    batches in a row with different descriptors (the two staging buffers and
    the GPU's own copy are reused), copies of no bytes among them; then the
    argument check such a batch still gets."""
    src, src_host, dst = arenas
    for seed, n, max_len in ((1, 4096, 6000), (2, 6001, 3000), (3, 5000, 9000)):
        rng = np.random.default_rng(6100 + seed)
        descs, lens, offs, so, do, total = _make_batch(capi, rng, src, dst, n, min_len=1, max_len=max_len)
        for i in range(0, n, 5):
            descs[i].bytes = 0
            lens[i] = 0
        dst.fill(0, total, GUARD_BYTE)
        check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
        check_ok(capi, blit.synchronize(), "synchronize")
        p = blit.last_plan()
        # the grid follows the host's estimate of the chunk count: a little under it, never far off
        chunks = sum((int(d.dst) % 256 // 16 * 16 + int(d.bytes) + 4095) // 4096 for d in descs if d.bytes)
        assert p.kernel == capi.KERNEL_COPY_BATCH and 0.93 * chunks <= _grid_chunks(p) <= 1.01 * chunks + 2, \
            (p.as_dict(), chunks, int(lens.sum()), n, seed)
        assert np.array_equal(dst.host(0, total), _expect_batch(oracle, src_host, total, lens, offs, so, do)), seed
    # a copy of bytes without a source: refused before anything is launched
    descs[n // 2].src = None
    descs[n // 2].bytes = 8
    dst.fill(0, total, GUARD_BYTE)
    assert blit.copy_batch(descs, n) == capi.ERROR_INVALID_ARGUMENT
    check_ok(capi, blit.synchronize(), "synchronize")
    assert (dst.host(0, total) == GUARD_BYTE).all()
    # all empty: nothing to do
    for i in range(n):
        descs[i].bytes = 0
    check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert (dst.host(0, total) == GUARD_BYTE).all()


def test_batch_65536_copies(capi, blit, oracle, rand, torch_cuda):
    """The benchmark's batch: 65,536 copies, 64 B .. 256 KiB log-uniform, offsets
    0..15 on both sides, carved sequentially out of one arena; all bytes and
    all guards against the oracle."""
    torch = torch_cuda
    n = 65536
    rng = np.random.default_rng(0xB1170005)
    lens = np.floor(64 * 2.0 ** (12 * rng.random(n))).astype(np.int64)
    stride = ((lens + 255) // 256) * 256 + 512
    total = int(stride.sum() + 512)
    src_host = rand(total, 0xB1170005)
    src = Arena(torch, total, host=src_host)
    dst = Arena(torch, total, fill=GUARD_BYTE)
    rng = np.random.default_rng(0xB1170005)
    descs, lens, offs, so, do, total2 = _make_batch(capi, rng, src, dst, n)
    assert total2 <= total
    want = np.full(total, GUARD_BYTE, dtype=np.uint8)
    want[:total2] = _expect_batch(oracle, src_host, total2, lens, offs, so, do)
    # host-resident descriptors both ways -- walked by the host, and staged as
    # they are for the GPU's own prefix sum -- and then as the library chooses
    # (an idle engine gets them as they are)
    for staging in (1, 2, 0):
        blit.set_tuning(**({"batch_staging": staging} if staging else {}))
        dst.fill(0, total, GUARD_BYTE)
        torch.cuda.synchronize()
        check_ok(capi, blit.copy_batch(descs, n), "copy_batch")
        check_ok(capi, blit.synchronize(), "synchronize")
        assert blit.last_plan().kernel == capi.KERNEL_COPY_BATCH
        assert np.array_equal(dst.host(), want), "staging %d" % staging
    blit.set_tuning()
    # the same descriptors resident in device memory: sized by the library's
    # assumption, by the batch before, and by the caller's bound
    descs_dev = _to_device(torch, descs)
    for submit in (lambda: blit.copy_batch(descs_dev.data_ptr(), n, on_device=True),
                   lambda: blit.copy_batch(descs_dev.data_ptr(), n, on_device=True),
                   lambda: blit.copy_batch_bounded(descs_dev.data_ptr(), n, int(lens.sum()))):
        dst.fill(0, total, GUARD_BYTE)
        torch.cuda.synchronize()
        check_ok(capi, submit(), "copy_batch, device-resident descriptors")
        check_ok(capi, blit.synchronize(), "synchronize")
        assert np.array_equal(dst.host(), want)


@pytest.fixture(scope="module")
def batch_arena(capi, oracle, rand, torch_cuda):
    """The benchmark's batch in its arena: 65,536 copies, 64 B .. 256 KiB
    log-uniform, byte offsets 0..15 on both sides, regions spread by
    bench.batch_layout over an 8 GiB source and an 8 GiB destination, so that
    descriptors lie more than 4 GiB apart and the copies are sparse in memory.
    Yields the descriptors and the whole destination as the oracle leaves it
    (every copy by oracle_copy into a buffer of guard bytes), resident on the
    device for the comparisons."""
    import bench
    torch = torch_cuda
    n, arena = 65536, 8 << 30
    lens, so, do, offs, stride = bench.batch_layout(n, arena)
    assert int(offs[-1] + stride[-1]) <= arena and int(offs[-1]) > (7 << 30)
    block = rand(64 * MIB, 0xB1170005)            # the arena's source bytes: this block, repeated
    src = torch.empty(arena + 512, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty(arena + 512, dtype=torch.uint8, device="cuda:0")
    s_sh, d_sh = (-src.data_ptr()) % 256, (-dst.data_ptr()) % 256
    block_dev = torch.from_numpy(block).to("cuda:0")
    for lo in range(0, arena, block.size):
        src[s_sh + lo:s_sh + lo + block.size].copy_(block_dev)
    del block_dev
    # what the oracle leaves in the destination, built and uploaded 1 GiB at a time
    want_dev = torch.empty(arena, dtype=torch.uint8, device="cuda:0")
    part = 1 << 30
    two = np.concatenate([block, block])          # a copy's source bytes may wrap around the block's end
    begin, end = offs + do, offs + do + lens      # destination ranges, ascending and disjoint
    for k in range(arena // part):
        lo, hi = k * part, (k + 1) * part
        want = np.full(part, GUARD_BYTE, dtype=np.uint8)
        # the copies that have bytes in [lo, hi); one that straddles a boundary gives each side its share
        for i in range(int(np.searchsorted(end, lo, side="right")), int(np.searchsorted(begin, hi, side="left"))):
            a, b = max(int(begin[i]), lo), min(int(end[i]), hi)
            s_at = (int(offs[i] + so[i]) + a - int(begin[i])) % block.size
            oracle.oracle_copy(want.ctypes.data + a - lo, two.ctypes.data + s_at, b - a)
        want_dev[lo:hi].copy_(torch.from_numpy(want))
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst.data_ptr() + d_sh + int(offs[i] + do[i])
        descs[i].src = src.data_ptr() + s_sh + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    torch.cuda.synchronize()
    yield descs, n, int(lens.sum()), dst[d_sh:d_sh + arena], want_dev
    del src, dst, want_dev
    torch.cuda.empty_cache()


@pytest.mark.parametrize("descriptors", ["host_walked", "host_as_they_are", "device", "device_bounded"])
def test_batch_65536_copies_in_the_16_gib_arena(capi, blit, batch_arena, torch_cuda, descriptors):
    """Every byte of the 8 GiB destination -- all 65,536 copies, their guard
    bands and everything between them -- against what the oracle leaves."""
    torch = torch_cuda
    descs, n, total, dst, want = batch_arena
    dst.fill_(GUARD_BYTE)
    dev = _to_device(torch, descs) if descriptors.startswith("device") else None
    torch.cuda.synchronize()
    if descriptors.startswith("host"):
        blit.set_tuning(batch_staging=1 if descriptors == "host_walked" else 2)
        st = blit.copy_batch(descs, n)
        blit.set_tuning()
    elif descriptors == "device":
        st = blit.copy_batch(dev.data_ptr(), n, on_device=True)
    else:
        st = blit.copy_batch_bounded(dev.data_ptr(), n, total)
    check_ok(capi, st, "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    if not torch.equal(dst, want):
        part = 1 << 28
        for lo in range(0, dst.numel(), part):
            bad = torch.nonzero(dst[lo:lo + part] != want[lo:lo + part])
            if bad.numel():
                raise AssertionError("destination differs from the oracle's, first at byte %d" % (lo + int(bad[0])))


def test_batch_back_to_back_reuses_staging(capi, blit, oracle, arenas):
    """Two host-descriptor batches in a row share the staging buffers."""
    src, src_host, dst = arenas
    rng = np.random.default_rng(31337)
    d1, l1, o1, s1, e1, t1 = _make_batch(capi, rng, src, dst, 300)
    dst.fill(0, t1, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(d1, 300), "copy_batch")
    # second batch: same regions shifted by a fixed distance past the first
    shift = ((t1 + 255) // 256) * 256
    d2 = (capi.Desc * 200)()
    for i in range(200):
        d2[i].dst = d1[i].dst + shift
        d2[i].src = d1[i].src
        d2[i].bytes = d1[i].bytes
    dst.fill(shift, shift + t1, GUARD_BYTE)
    check_ok(capi, blit.copy_batch(d2, 200), "copy_batch")
    check_ok(capi, blit.synchronize(), "synchronize")
    assert np.array_equal(dst.host(0, t1), _expect_batch(oracle, src_host, t1, l1, o1, s1, e1))
    want2 = np.full(t1, GUARD_BYTE, dtype=np.uint8)
    for i in range(200):
        oracle.oracle_copy(want2.ctypes.data + int(o1[i] + e1[i]), src_host.ctypes.data + int(o1[i] + s1[i]), int(l1[i]))
    assert np.array_equal(dst.host(shift, shift + t1), want2)


@pytest.mark.parametrize("queue", ["own", "borrowed"])
def test_batches_with_signals_between_other_commands(capi, pkg, oracle, arenas, queue):
    """Host-descriptor batches on an AQL engine, back to back and growing (the
    staging and record buffers are replaced on the way), with and without the
    caller's completion signal, one held back by a dependency signal, with a
    linear copy and a device-resident batch in between.  Every batch has a
    stretch of the destination of its own; all are compared with the oracle at
    the end, and the held batch must not have finished before its dependency
    was released."""
    import time
    src, src_host, dst = arenas
    pkg.aql.load()
    sig = pkg.aql.HsaSignals()
    borrowed = pkg.aql.BorrowedQueue(0, packets=64) if queue == "borrowed" else None
    eng = pkg.aql.AqlBlit(borrowed=borrowed) if borrowed is not None else pkg.aql.AqlBlit(0)
    made = []
    try:
        rng = np.random.default_rng(0xB11705EC)
        dst.fill(0, dst.nbytes, GUARD_BYTE)
        want = np.full(dst.nbytes, GUARD_BYTE, dtype=np.uint8)
        at = 0
        keep = []

        def batch(n, max_len, on_device=False, **kw):
            nonlocal at
            descs, lens, offs, so, do, total = _make_batch(capi, rng, _Window(src, at), _Window(dst, at), n, max_len=max_len)
            for i in range(n):
                oracle.oracle_copy(want.ctypes.data + at + int(offs[i] + do[i]),
                                   src_host.ctypes.data + at + int(offs[i] + so[i]), int(lens[i]))
            if on_device:
                dev = src.torch.from_numpy(np.frombuffer(descs, dtype=np.uint8).copy()).to("cuda:0")
                src.torch.cuda.synchronize()
                keep.append(dev)
                check_ok(capi, eng.copy_batch(dev.data_ptr(), n, on_device=True, **kw), "copy_batch")
            else:
                keep.append(descs)
                check_ok(capi, eng.copy_batch(descs, n, **kw), "copy_batch")
            at += (total + 255) // 256 * 256

        for n, max_len in ((40, 4096), (300, 64 << 10), (5, 1 << 20), (3000, 8 << 10), (700, 32 << 10)):
            batch(n, max_len)
        done = sig.create(1)
        made.append(done)
        batch(200, 16 << 10, completion=done)
        sig.wait_below_one(done)
        n_lin = 3 * MIB + 5
        check_ok(capi, eng.copy(dst.base + at + 7, src.base + at + 2, n_lin), "copy")
        oracle.oracle_copy(want.ctypes.data + at + 7, src_host.ctypes.data + at + 2, n_lin)
        at += (n_lin + 7 + 255) // 256 * 256 + 256
        batch(100, 128 << 10)
        dep, held = sig.create(1), sig.create(1)
        made += [dep, held]
        batch(150, 32 << 10, deps=[dep], completion=held)
        batch(60, 8 << 10)          # queued behind the held one
        time.sleep(0.05)
        assert sig.load(held) == 1, "a batch ran before its dependency was released"
        sig.store(dep, 0)
        sig.wait_below_one(held)
        batch(120, 16 << 10, on_device=True)
        batch(90, 64 << 10)
        check_ok(capi, eng.synchronize(), "synchronize")
        assert at <= dst.nbytes
        got = dst.host(0, at)
        if not np.array_equal(got, want[:at]):
            bad = np.nonzero(got != want[:at])[0]
            raise AssertionError("%d bytes differ, first at %d of %d" % (bad.size, bad[0], at))
        assert eng.pending_bytes() == 0
    finally:
        for s_ in made:
            sig.destroy(s_)
        eng.close()
        if borrowed is not None:
            assert borrowed.errors == []
            borrowed.close()


# ---------------------------------------------------------- API edge behaviour

def test_argument_validation(capi, blit, arenas):
    """Same answers as hsa_memory_copy / hsa_amd_memory_fill give at the API
    edge (hsa.cpp:1170-1184, hsa_ext_amd.cpp:237-251)."""
    src, _, dst = arenas
    inv = capi.ERROR_INVALID_ARGUMENT
    assert blit.copy(None, src.base, 16) == inv
    assert blit.copy(dst.base, None, 16) == inv
    assert blit.fill32(None, 1, 4) == inv
    for off in (1, 2, 3):
        assert blit.fill32(dst.base + off, 1, 4) == inv
    # zero size succeeds without touching memory
    dst.fill(0, 64, GUARD_BYTE)
    assert blit.copy(dst.base, src.base, 0) == capi.SUCCESS
    assert blit.fill32(dst.base, 1, 0) == capi.SUCCESS
    assert blit.copy_batch(None, 0) == capi.SUCCESS
    if blit.backend == "hip":
        assert blit.lib.mi355_blit_copy_batch(blit.handle, None, 3, 0, None) == inv
    else:
        assert blit.lib.mi355_aql_copy_batch(blit.handle, None, 3, None, 0, 0) == inv
    bad = (capi.Desc * 1)()
    bad[0].dst, bad[0].src, bad[0].bytes = None, src.base, 8
    assert blit.copy_batch(bad, 1) == inv
    check_ok(capi, blit.synchronize(), "synchronize")
    assert bool((dst.view[:64] == GUARD_BYTE).all())


def test_pending_bytes_zero_is_exact(capi, blit, arenas):
    src, _, dst = arenas
    check_ok(capi, blit.synchronize(), "synchronize")
    assert blit.pending_bytes() == 0
    n = 32 * MIB
    for _ in range(100):  # more commands than ledger slots: back-pressure path
        check_ok(capi, blit.copy(dst.base, src.base, n), "copy")
    pending = blit.pending_bytes()
    assert pending % n == 0 and pending <= 100 * n
    check_ok(capi, blit.synchronize(), "synchronize")
    assert blit.pending_bytes() == 0
    # without a synchronize the count reaches zero by itself once the work is done
    for _ in range(10):
        check_ok(capi, blit.copy(dst.base, src.base, n), "copy")
    import time
    deadline = time.time() + 5.0
    while blit.pending_bytes() != 0 and time.time() < deadline:
        time.sleep(0.001)
    assert blit.pending_bytes() == 0


def test_external_stream_and_ordering(capi, blit, oracle, arenas, torch_cuda):
    """Commands on a caller's stream run in order with that stream's other work."""
    if blit.backend != "hip":
        pytest.skip("streams belong to the HIP-stream path")
    torch = torch_cuda
    src, src_host, dst = arenas
    s = torch.cuda.Stream()
    n = 5 * MIB + 3
    with torch.cuda.stream(s):
        dst.view[:n + 2 * GUARD].fill_(GUARD_BYTE)
        check_ok(capi, blit.fill32(dst.base + GUARD, 0x01020304, n // 4, s.cuda_stream), "fill32")
        check_ok(capi, blit.copy(dst.base + GUARD + 1, src.base + 2, n - 2, s.cuda_stream), "copy")
    s.synchronize()
    want = np.full(n + 2 * GUARD, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_fill32(want.ctypes.data + GUARD, 0x01020304, n // 4)
    oracle.oracle_copy(want.ctypes.data + GUARD + 1, src_host.ctypes.data + 2, n - 2)
    assert np.array_equal(dst.host(0, n + 2 * GUARD), want)


def test_concurrent_submitters(capi, blit, oracle, arenas):
    """Several host threads submit to one handle, as several callers of
    hsa_memory_copy would (the reference serialises them on a mutex)."""
    src, src_host, dst = arenas
    n = MIB + 17
    nthreads, per = 4, 8
    region = ((n + 2 * GUARD + 255) // 256) * 256
    dst.fill(0, nthreads * per * region, GUARD_BYTE)
    errs = []

    def worker(t):
        for j in range(per):
            slot = t * per + j
            st = blit.copy(dst.base + slot * region + GUARD + (slot % 16), src.base + slot * 4096 + (slot % 7), n)
            if st != capi.SUCCESS:
                errs.append(st)

    ths = [threading.Thread(target=worker, args=(t,)) for t in range(nthreads)]
    for t in ths:
        t.start()
    for t in ths:
        t.join()
    assert not errs
    check_ok(capi, blit.synchronize(), "synchronize")
    got = dst.host(0, nthreads * per * region)
    want = np.full(got.size, GUARD_BYTE, dtype=np.uint8)
    for slot in range(nthreads * per):
        oracle.oracle_copy(want.ctypes.data + slot * region + GUARD + (slot % 16),
                           src_host.ctypes.data + slot * 4096 + (slot % 7), n)
    assert np.array_equal(got, want)


def test_create_destroy_many(capi, pkg):
    for _ in range(5):
        b = capi.Blit(0)
        assert b.num_cus > 0 and b.stream
        b.close()
    for _ in range(3):
        a = pkg.aql.AqlBlit(0)
        assert a.num_cus > 0
        a.close()
    with pytest.raises(RuntimeError):
        pkg.aql.AqlBlit(1000)
    h = C.c_void_p()
    assert capi.load().mi355_blit_create(10_000, C.byref(h)) == capi.ERROR_INVALID_ARGUMENT


@pytest.mark.gpu
def test_engines_of_one_agent_share_one_code_object(pkg, oracle, rand, torch_cuda):
    """Three engines on one agent -- the shape of GpuAgent's blits_[] slots, whose
    BlitKernels all run the shaders the agent assembled once
    (amd_gpu_agent.cpp:251-428) -- hold one executable between them, an owner's
    own reference keeps it loaded while no engine exists, and it survives the
    engines' destruction in any order: after each destroy the others still copy
    correctly."""
    torch = torch_cuda
    aql = pkg.aql
    lib = aql.load()
    queue = aql.BorrowedQueue(0)
    n = 3 * MIB + 5
    host = rand(n + 64, 0xB1170077)
    src = torch.from_numpy(host).to("cuda:0")
    dst = torch.empty(n + 64, dtype=torch.uint8, device="cuda:0")

    def copies_right(engine, seed):
        dst.fill_(seed)
        torch.cuda.synchronize()
        assert engine.copy_sync(dst.data_ptr() + 9, src.data_ptr() + 3, n) == 0
        want = np.full(n + 64, seed, dtype=np.uint8)
        oracle.oracle_copy(want.ctypes.data + 9, host.ctypes.data + 3, n)
        assert np.array_equal(dst.cpu().numpy(), want)

    try:
        a = aql.AqlBlit(borrowed=queue)
        exe, base = a.code_object_info()
        # other engines of this test session may be alive on the same agent: they hold the same executable
        assert exe != 0 and base >= 1
        b = aql.AqlBlit(borrowed=queue)       # a second engine on the same queue
        c = aql.AqlBlit(0)                    # and one on a queue of its own
        assert b.code_object_info() == (exe, base + 2) and c.code_object_info() == (exe, base + 2)
        own = C.c_void_p()
        assert lib.mi355_aql_code_object_acquire(queue.agent, C.byref(own)) == 0
        assert a.code_object_info() == (exe, base + 3)
        for engine, seed in ((a, 1), (b, 2), (c, 3)):
            copies_right(engine, seed)
        b.close()
        assert a.code_object_info() == (exe, base + 2)
        copies_right(a, 4)
        copies_right(c, 5)
        a.close()
        copies_right(c, 6)
        c.close()
        # the owner's reference is left: a new engine finds the same executable
        d = aql.AqlBlit(borrowed=queue)
        assert d.code_object_info() == (exe, base + 1)
        copies_right(d, 7)
        d.close()
        assert lib.mi355_aql_code_object_release(own) == 0
        if base == 1:
            # that was the last reference: the handle is gone, and the next engine loads the code afresh
            assert lib.mi355_aql_code_object_release(own) == pkg.capi.ERROR_INVALID_ARGUMENT
        e = aql.AqlBlit(borrowed=queue)
        assert e.code_object_info()[1] == base
        copies_right(e, 8)
        e.close()
        assert lib.mi355_aql_code_object_acquire(0, C.byref(own)) == pkg.capi.ERROR_INVALID_ARGUMENT
    finally:
        queue.close()
