"""Pitched 3-D region copy, the parts that need no GPU: the CPU oracle pinned
against numpy slice assignment, the restated argument checks of the reference
case by case, and the host planning of the library (validation, merging of
contiguous rows, chunk slots) checked by replaying the kernel's slot
arithmetic in numpy and demanding that every byte of the region is written
exactly once and nothing else is."""
import numpy as np
import pytest

from conftest import oracle_rect, oracle_validate_rect

SUCCESS, INVALID_ARGUMENT = 0x0, 0x1001


@pytest.fixture(scope="module")
def capi_host(pkg):
    import torch  # noqa: F401  (one HIP runtime per process: torch's first)
    pkg.capi.load()
    return pkg.capi


def surfaces(rand, seed, shape):
    """Two 3-D byte arrays [layers, rows, pitch], source random, destination 0xEE."""
    z, y, x = shape
    src = rand(z * y * x, seed).reshape(z, y, x)
    dst = np.full((z, y, x), 0xEE, dtype=np.uint8)
    return src, dst


def pitched(a):
    return (a.ctypes.data, a.shape[2], a.shape[1] * a.shape[2])


# ------------------------------------------------------------------ the oracle

@pytest.mark.parametrize("seed", range(12))
def test_oracle_rect_is_numpy_slice_assignment(oracle, rand, seed):
    rng = np.random.default_rng(seed)
    sshape = tuple(int(v) for v in rng.integers(1, [6, 40, 300]))
    dshape = tuple(int(v) for v in rng.integers(1, [6, 40, 300]))
    src, dst = surfaces(rand, seed, sshape)
    dst = np.full(dshape, 0xEE, dtype=np.uint8)
    ext = [int(rng.integers(1, min(sshape[k], dshape[k]) + 1)) for k in range(3)]  # z, y, x
    so = [int(rng.integers(0, sshape[k] - ext[k] + 1)) for k in range(3)]
    do = [int(rng.integers(0, dshape[k] - ext[k] + 1)) for k in range(3)]
    want = dst.copy()
    want[do[0]:do[0] + ext[0], do[1]:do[1] + ext[1], do[2]:do[2] + ext[2]] = \
        src[so[0]:so[0] + ext[0], so[1]:so[1] + ext[1], so[2]:so[2] + ext[2]]
    oracle_rect(oracle, pitched(dst), do[::-1], pitched(src), so[::-1], ext[::-1])
    assert np.array_equal(dst, want)


def test_oracle_rect_empty_range_moves_nothing(oracle, rand):
    src, dst = surfaces(rand, 1, (2, 4, 64))
    for ext in ((0, 2, 2), (8, 0, 2), (8, 2, 0)):
        oracle_rect(oracle, pitched(dst), (0, 0, 0), pitched(src), (0, 0, 0), ext)
    assert (dst == 0xEE).all()


def test_reference_rect_argument_checks(oracle):
    """core/runtime/hsa_ext_amd.cpp:372-405 and amd_blit_sdma.cpp:570-585, one case per branch."""
    d = (0x10000, 512, 512 * 16)
    s = (0x80000, 256, 256 * 32)
    z = (0, 0, 0)
    ok = (64, 4, 2)
    assert oracle_validate_rect(oracle, d, z, s, z, ok) == (SUCCESS, 1, 1)
    for missing in range(5):
        args = [d, z, s, z, ok]
        args[missing] = None
        assert oracle_validate_rect(oracle, *args)[0] == INVALID_ARGUMENT
    assert oracle_validate_rect(oracle, d, z, s, z, ok, direction=0)[0] == INVALID_ARGUMENT  # hsaHostToHost
    for direction in (1, 2, 3):
        assert oracle_validate_rect(oracle, d, z, s, z, ok, direction)[0] == SUCCESS
    for ext in ((0, 4, 2), (64, 0, 2), (64, 4, 0)):
        assert oracle_validate_rect(oracle, d, z, s, z, ext) == (SUCCESS, 0, 1)  # success, nothing submitted
    # width beyond a pitch, on either side
    assert oracle_validate_rect(oracle, d, z, s, (200, 0, 0), ok)[0] == INVALID_ARGUMENT
    assert oracle_validate_rect(oracle, d, (460, 0, 0), s, z, ok)[0] == INVALID_ARGUMENT
    assert oracle_validate_rect(oracle, d, (448, 0, 0), s, (192, 0, 0), ok)[0] == SUCCESS
    # height beyond slice / pitch
    assert oracle_validate_rect(oracle, d, (0, 13, 0), s, z, ok)[0] == INVALID_ARGUMENT
    assert oracle_validate_rect(oracle, d, (0, 12, 0), s, (0, 28, 0), ok)[0] == SUCCESS
    assert oracle_validate_rect(oracle, d, z, s, (0, 29, 0), ok)[0] == INVALID_ARGUMENT
    # no slice: any height passes, but only one layer
    flat_d, flat_s = (d[0], 512, 0), (s[0], 256, 0)
    assert oracle_validate_rect(oracle, flat_d, (0, 1000, 0), flat_s, z, (64, 4, 1))[0] == SUCCESS
    assert oracle_validate_rect(oracle, flat_d, z, s, z, ok)[0] == INVALID_ARGUMENT
    assert oracle_validate_rect(oracle, d, z, flat_s, z, ok)[0] == INVALID_ARGUMENT
    # what only the SDMA packet needs
    assert oracle_validate_rect(oracle, (d[0] + 1, 512, 512 * 16), z, s, z, ok) == (SUCCESS, 1, 0)
    assert oracle_validate_rect(oracle, d, z, (s[0], 258, 258 * 32), z, ok) == (SUCCESS, 1, 0)


# ------------------------------------------------------------ library planning

def replay_narrow_plan(p, dst_bytes, src_bytes, dst_base, src_base):
    """The packed kernel's lane arithmetic: the (row, slot) pairs are numbered
    row by row, lanes_per_row to a row; each takes the 16-byte destination slot
    of that number, or, where the row cuts the slot, the 16 bytes at the row's
    start or end (bytes of the neighbouring slot are then written twice)."""
    written = np.zeros(dst_bytes.size, dtype=np.uint8)
    for n in range(p.rows * p.layers * p.lanes_per_row):
        line, j = divmod(n, p.lanes_per_row)
        layer, y = divmod(line, p.rows)
        d = p.dst + layer * p.dst_slice + y * p.dst_pitch
        s = p.src + layer * p.src_slice + y * p.src_pitch
        slot = d // 16 * 16 + 16 * j
        if slot >= d + p.width:
            continue
        if p.width >= 16:
            lo = min(max(slot, d), d + p.width - 16)
            hi = lo + 16
        else:
            lo, hi = max(slot, d), min(slot + 16, d + p.width)
        do, so = lo - dst_base, s + (lo - d) - src_base
        dst_bytes[do:do + hi - lo] = src_bytes[so:so + hi - lo]
        written[do:do + hi - lo] += 1
    return written


def replay_rect_plan(p, dst_bytes, src_bytes, dst_base, src_base):
    """What the kernel's unit arithmetic moves, with numpy: slot s is unit
    s % slots of merged row s // slots; a unit covers the row's vectors between
    cuts at multiples of 64 * unroll vectors from the 256-byte boundary below
    the row's first vector, the first unit also the head bytes, the last one
    up to 15 vectors more and the tail bytes.  Returns how often each
    destination byte was written."""
    written = np.zeros(dst_bytes.size, dtype=np.uint8)
    unit = 64 * p.unroll
    for line in range(p.rows * p.layers):
        layer, y = divmod(line, p.rows)
        d = p.dst + layer * p.dst_slice + y * p.dst_pitch
        s = p.src + layer * p.src_slice + y * p.src_pitch
        if p.plain_rows:
            # every unit is a plain tile of the row, the last one possibly a partial one
            assert d % 128 == 0 and p.width % 128 == 0 and (s - d) % 4 == 0
            n_vec = p.width // 16
            assert p.slots == (-(-n_vec // unit) if n_vec > 15 + unit else 1)
            for kq in range(p.slots):
                b0 = kq * 16 * unit
                b1 = p.width if kq + 1 == p.slots else (kq + 1) * 16 * unit
                assert b1 - b0 <= 16 * (unit + 15), "the last unit's overflow is at most 15 vectors" 
                do, so = d - dst_base + b0, s - src_base + b0
                dst_bytes[do:do + b1 - b0] = src_bytes[so:so + b1 - b0]
                written[do:do + b1 - b0] += 1
            continue
        head = min((16 - d % 16) % 16, p.width)
        n_vec = (p.width - head) // 16
        lead = ((d + head) % 256) // 16
        n_virtual = n_vec + lead
        units = -(-(n_virtual - 15) // unit) if n_virtual > 15 + unit else 1
        assert units <= p.slots, "a row needs more unit slots than the plan gives it"
        for kq in range(units):
            last = kq + 1 == units
            lo = max(kq * unit, lead)
            hi = n_virtual if last else kq * unit + unit
            assert hi - kq * unit <= unit + 64, "a lane would need more than one extra vector"
            b0 = 0 if kq == 0 else head + 16 * (lo - lead)
            b1 = p.width if last else head + 16 * (hi - lead)
            do, so = d - dst_base + b0, s - src_base + b0
            dst_bytes[do:do + b1 - b0] = src_bytes[so:so + b1 - b0]
            written[do:do + b1 - b0] += 1
    return written


@pytest.mark.parametrize("seed", range(60))
def test_plan_rect_writes_every_byte_once(capi_host, oracle, rand, seed):
    rng = np.random.default_rng(1000 + seed)
    widest = 9000 if seed < 40 else 1300   # the later seeds are mostly packed narrow rows
    sshape = tuple(int(v) for v in rng.integers(1, [4, 12, widest]))
    dshape = tuple(int(v) for v in rng.integers(1, [4, 12, widest]))
    src = rand(int(np.prod(sshape)) + 256, seed)
    dst = np.full(int(np.prod(dshape)) + 256, 0xEE, dtype=np.uint8)
    s_base = src.ctypes.data + int(rng.integers(0, 256))
    d_base = dst.ctypes.data + int(rng.integers(0, 256))
    ext = [int(rng.integers(1, min(sshape[k], dshape[k]) + 1)) for k in range(3)]
    if seed % 5 == 0:  # full-width rows merge
        sshape = (sshape[0], sshape[1], ext[2])
        dshape = (dshape[0], dshape[1], ext[2])
    so = [int(rng.integers(0, sshape[k] - ext[k] + 1)) for k in range(3)]
    do = [int(rng.integers(0, dshape[k] - ext[k] + 1)) for k in range(3)]
    sp = (s_base, sshape[2], sshape[1] * sshape[2])
    dp = (d_base, dshape[2], dshape[1] * dshape[2])
    st, p = capi_host.plan_rect(dp, do[::-1], sp, so[::-1], ext[::-1])
    assert st == SUCCESS and not p.empty
    assert p.total_bytes == ext[0] * ext[1] * ext[2]
    want = dst.copy()
    oracle_rect(oracle, (want.ctypes.data + d_base - dst.ctypes.data,) + dp[1:], do[::-1], sp, so[::-1], ext[::-1])
    if p.linear:
        off_d, off_s = p.dst - dst.ctypes.data, p.src - src.ctypes.data
        got = dst.copy()
        got[off_d:off_d + p.width] = src[off_s:off_s + p.width]
        assert p.width == p.total_bytes
        assert np.array_equal(got, want)
        return
    assert p.rows * p.layers * p.width == p.total_bytes
    got = dst.copy()
    if p.lanes_per_row:
        assert p.grid * (p.wg_size // 64) * 64 >= p.rows * p.layers * p.lanes_per_row
        written = replay_narrow_plan(p, got, src, dst.ctypes.data, src.ctypes.data)
        assert np.array_equal(got, want)
        # every byte of the region at least once, nothing outside it
        assert int((written > 0).sum()) == p.total_bytes and written.max() <= 3
        return
    else:
        assert p.grid * (p.wg_size // 64) >= p.rows * p.layers * p.slots
        written = replay_rect_plan(p, got, src, dst.ctypes.data, src.ctypes.data)
    assert np.array_equal(got, want)
    assert written.max() == 1 and int(written.sum()) == p.total_bytes


@pytest.mark.parametrize("width", [1152, 4096, 4224, 7040, 128 * 77])
def test_plan_rect_plain_rows_write_every_byte_once(capi_host, oracle, rand, width):
    """Rows at 256-byte boundaries of the destination, whole lines wide: the
    short path's tiles cover each row exactly, a partial last unit included."""
    rows, pitch = 9, 16384
    src = rand(rows * pitch + 512, width)
    dst = np.full(rows * pitch + 512, 0xEE, dtype=np.uint8)
    d_base = dst.ctypes.data + (-dst.ctypes.data) % 256
    s_base = src.ctypes.data + (-src.ctypes.data) % 256 + 4
    sp, dp = (s_base, pitch, 0), (d_base, pitch, 0)
    for unroll in (1, 2, 4):
        st, p = capi_host.plan_rect(dp, (256, 1, 0), sp, (8, 0, 0), (width, rows - 1, 1), capi_host.Tuning(unroll=unroll))
        assert st == SUCCESS and p.plain_rows == 1 and p.unroll == unroll
        want = dst.copy()
        oracle_rect(oracle, (want.ctypes.data + d_base - dst.ctypes.data,) + dp[1:], (256, 1, 0), sp, (8, 0, 0),
                    (width, rows - 1, 1))
        got = dst.copy()
        written = replay_rect_plan(p, got, src, dst.ctypes.data, src.ctypes.data)
        assert np.array_equal(got, want)
        assert written.max() == 1 and int(written.sum()) == p.total_bytes


def test_plan_rect_merges_contiguous_rows(capi_host):
    base_d, base_s = 0x7f0000000000, 0x7f1000000000
    # rows as wide as both pitches: one run per layer; layers also contiguous: one run
    st, p = capi_host.plan_rect((base_d, 4096, 4096 * 8), (0, 0, 0), (base_s, 4096, 4096 * 8), (0, 0, 0), (4096, 8, 3))
    assert st == SUCCESS and p.linear and p.width == 4096 * 8 * 3 and p.dst == base_d and p.src == base_s
    # layers apart on one side: three rows of 32 KiB
    st, p = capi_host.plan_rect((base_d, 4096, 4096 * 16), (0, 0, 0), (base_s, 4096, 4096 * 8), (0, 0, 0), (4096, 8, 3))
    assert st == SUCCESS and not p.linear
    assert (p.width, p.rows, p.layers, p.dst_pitch, p.src_pitch) == (4096 * 8, 3, 1, 4096 * 16, 4096 * 8)
    # pitches differ: nothing merges
    st, p = capi_host.plan_rect((base_d, 8192, 8192 * 8), (0, 0, 0), (base_s, 4096, 4096 * 8), (0, 0, 0), (4096, 8, 3))
    assert st == SUCCESS and (p.width, p.rows, p.layers) == (4096, 8, 3)
    # one row per layer: the layers become the rows
    st, p = capi_host.plan_rect((base_d, 8192, 8192 * 8), (0, 2, 1), (base_s, 4096, 4096 * 8), (16, 0, 0), (100, 1, 3))
    assert st == SUCCESS and (p.width, p.rows, p.layers, p.dst_pitch, p.src_pitch) == (100, 3, 1, 8192 * 8, 4096 * 8)
    assert p.dst == base_d + 8192 * 8 + 2 * 8192 and p.src == base_s + 16
    # a single row is a linear copy whatever the pitches
    st, p = capi_host.plan_rect((base_d, 8192, 0), (5, 7, 0), (base_s, 4096, 0), (3, 2, 0), (1000, 1, 1))
    assert st == SUCCESS and p.linear and p.width == 1000
    assert p.dst == base_d + 7 * 8192 + 5 and p.src == base_s + 2 * 4096 + 3


def test_plan_rect_slots_follow_row_alignment(capi_host):
    base_d, base_s = 0x7f0000000000, 0x7f1000000000
    # 4 KiB rows whose every store is a whole cache line: four units of 1 KiB, workgroups of 256
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 64, 1))
    assert st == SUCCESS and (p.slots, p.unroll, p.lanes_per_row, p.wg_size) == (4, 1, 0, 256)
    assert p.grid * (p.wg_size // 64) == 64 * 4
    # 16 bytes off the lines: two units of 2 KiB, workgroups of 128
    st, p = capi_host.plan_rect((base_d, 8192, 0), (16, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 64, 1))
    assert st == SUCCESS and (p.slots, p.unroll, p.lanes_per_row, p.wg_size) == (2, 2, 0, 128)
    assert p.grid * (p.wg_size // 64) == 64 * 2
    # the same rows up to 240 bytes further: the last unit absorbs the spill
    for x in (16, 100, 240):
        st, p = capi_host.plan_rect((base_d, 8192, 0), (x, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 64, 1))
        assert st == SUCCESS and p.slots == 2
    # a pitch that walks through all residues does not change that
    st, p = capi_host.plan_rect((base_d, 4100, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 64, 1))
    assert st == SUCCESS and p.slots == 2
    # but 16 vectors more than two units need a third
    st, p = capi_host.plan_rect((base_d, 8192, 0), (16, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096 + 256, 64, 1))
    assert st == SUCCESS and p.slots == 3
    # rows of up to 64 destination slots are packed, as many to a wave as fit
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (1024, 64, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.slots, p.unroll) == (64, 0, 0)
    st, p = capi_host.plan_rect((base_d, 8192, 0), (1, 0, 0), (base_s, 8192, 0), (0, 0, 0), (1024, 64, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.slots) == (65, 0)   # ragged rows are packed up to 128 slots
    st, p = capi_host.plan_rect((base_d, 8192, 0), (1, 0, 0), (base_s, 8192, 0), (0, 0, 0), (2048, 64, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.slots) == (0, 1)    # 129 slots: one unit of two vectors per lane
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (1, 0, 0), (1024 + 128, 64, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.slots) == (0, 1)    # whole lines with bytes to realign: units
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (512, 64, 1))
    assert st == SUCCESS and p.lanes_per_row == 32 and p.grid * (p.wg_size // 64) == 32
    st, p = capi_host.plan_rect((base_d, 256, 0), (128, 0, 0), (base_s, 256, 0), (64, 0, 0), (64, 4096, 1))
    assert st == SUCCESS and p.lanes_per_row == 4 and p.grid * (p.wg_size // 64) == 256
    st, p = capi_host.plan_rect((base_d, 260, 0), (128, 0, 0), (base_s, 256, 0), (64, 0, 0), (64, 4096, 1))
    assert st == SUCCESS and p.lanes_per_row == 5 and p.grid * (p.wg_size // 64) == 320   # rows at every alignment mod 4
    st, p = capi_host.plan_rect((base_d, 37, 37 * 9), (3, 0, 0), (base_s, 41, 41 * 9), (0, 0, 0), (1, 9, 5))
    assert st == SUCCESS and (p.lanes_per_row, p.rows, p.layers) == (1, 9, 5)
    # packed rows: single-wave workgroups when no two waves can touch one destination line
    st, p = capi_host.plan_rect((base_d, 2048, 0), (0, 0, 0), (base_s, 2048, 0), (0, 0, 0), (1024, 8192, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.wg_size, p.store_policy) == (64, 64, capi_host.STORE_AGENT_WT)
    st, p = capi_host.plan_rect((base_d, 2048, 0), (9, 0, 0), (base_s, 2048, 0), (3, 0, 0), (1000, 8192, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.wg_size, p.store_policy) == (64, 64, capi_host.STORE_NT)
    st, p = capi_host.plan_rect((base_d, 1024, 0), (0, 0, 0), (base_s, 1024, 0), (0, 0, 0), (520, 8192, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.wg_size, p.store_policy) == (33, 256, capi_host.STORE_NT)
    st, p = capi_host.plan_rect((base_d, 260, 0), (0, 0, 0), (base_s, 260, 0), (0, 0, 0), (256, 32768, 1))
    assert st == SUCCESS and p.wg_size == 256                       # neighbouring rows share lines
    # streaming policy from 4 MiB of payload
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 64, 1))
    assert st == SUCCESS and p.nt_load == 0 and p.store_policy == capi_host.STORE_CACHED
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 1024, 1))
    assert st == SUCCESS and p.nt_load == 1 and p.store_policy == capi_host.STORE_AGENT_WT   # whole lines
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4100, 1024, 1))
    assert st == SUCCESS and p.nt_load == 1 and p.store_policy == capi_host.STORE_NT
    # rows tiled like a linear copy take the kernel's short path
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 1024, 1))
    assert st == SUCCESS and p.plain_rows == 1
    st, p = capi_host.plan_rect((base_d, 8192, 0), (256, 0, 0), (base_s, 8192, 0), (4, 0, 0), (4096, 1024, 1))
    assert st == SUCCESS and p.plain_rows == 1                     # 256-byte aligned destination, dword-aligned source
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096 + 128, 1024, 1))
    assert st == SUCCESS and (p.plain_rows, p.slots) == (1, 5)     # whole lines: the last unit is a partial one
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (1024 + 128, 1024, 1))
    assert st == SUCCESS and (p.plain_rows, p.slots) == (1, 1)     # a unit and 8 vectors: one wave's
    st, p = capi_host.plan_rect((base_d, 8192 + 128, 0), (128, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 1024, 1))
    assert st == SUCCESS and p.plain_rows == 1                     # rows at cache-line boundaries
    for d_x, s_x, w, dp in ((64, 0, 4096, 8192), (0, 2, 4096, 8192), (0, 0, 4096 + 64, 8192), (0, 0, 4096, 8192 + 64)):
        st, p = capi_host.plan_rect((base_d, dp, 0), (d_x, 0, 0), (base_s, 8192, 0), (s_x, 0, 0), (w, 1024, 1))
        assert st == SUCCESS and p.plain_rows == 0, (d_x, s_x, w, dp)
    # XCD runs: only from 64 MiB moved, and only where neighbouring waves share cache lines
    assert p.xcd_run == 0                                                                     # 4 MiB
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4100, 32768, 1))
    assert st == SUCCESS and (p.wg_size, p.unroll, p.xcd_run) == (128, 2, 144)               # 144 x 4 KiB
    # ragged rows of 48 KiB and more: the shape of the linear copy with a byte offset
    st, p = capi_host.plan_rect((base_d, 262148, 0), (9, 0, 0), (base_s, 262148, 0), (3, 0, 0), (48 * 1024 - 1, 8192, 1))
    assert st == SUCCESS and (p.wg_size, p.unroll, p.xcd_run, p.store_policy) == (128, 2, 144, capi_host.STORE_NT)
    st, p = capi_host.plan_rect((base_d, 262148, 0), (9, 0, 0), (base_s, 262148, 0), (3, 0, 0), (131065, 8192, 1))
    assert st == SUCCESS and (p.wg_size, p.unroll, p.xcd_run, p.store_policy) == (64, 1, 576, capi_host.STORE_NT)
    st, p = capi_host.plan_rect((base_d, 262148, 0), (9, 0, 0), (base_s, 262148, 0), (3, 0, 0), (131065, 128, 1))
    assert st == SUCCESS and (p.wg_size, p.unroll, p.xcd_run) == (128, 2, 0)                  # 16 MiB: no runs yet
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 32768, 1))
    assert st == SUCCESS and (p.plain_rows, p.wg_size, p.xcd_run) == (1, 64, 576)              # tiled like a linear copy
    st, p = capi_host.plan_rect((base_d, 8192, 0), (128, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 32768, 1))
    assert st == SUCCESS and (p.plain_rows, p.wg_size, p.xcd_run) == (1, 64, 576)              # at a line boundary: plain too
    st, p = capi_host.plan_rect((base_d, 8192, 0), (128, 0, 0), (base_s, 8192, 0), (1, 0, 0), (4096, 32768, 1))
    assert st == SUCCESS and (p.plain_rows, p.wg_size, p.xcd_run) == (0, 256, 0)               # whole lines, bytes to realign
    st, p = capi_host.plan_rect((base_d, 2048, 0), (9, 0, 0), (base_s, 2048, 0), (3, 0, 0), (1000, 1 << 20, 1))
    assert st == SUCCESS and (p.wg_size, p.xcd_run) == (64, 0)                                # waves share no line
    st, p = capi_host.plan_rect((base_d, 1024, 0), (0, 0, 0), (base_s, 1024, 0), (0, 0, 0), (520, 1 << 20, 1))
    assert st == SUCCESS and (p.lanes_per_row, p.wg_size, p.xcd_run) == (33, 256, 144)        # 4 waves x 1 KiB


def test_plan_rect_whole_line_rows_store_policy_follows_the_pitch(capi_host):
    """Rows of whole cache lines are written through L2 when they are under
    1 KiB, or when the destination pitch is a power of two, or a multiple of
    128 KiB while the width is a power of two, or within 3 % of the width; at
    any other pitch their stores are non-temporal
    (rect_whole_lines_write_through)."""
    base_d, base_s = 0x7f0000000000, 0x7f1000000000
    K = 1024
    WT, NT = capi_host.STORE_AGENT_WT, capi_host.STORE_NT
    cases = [
        # width, destination pitch, rows, expected
        (128 * K, 256 * K, 8192, WT), (128 * K, 260 * K, 8192, NT), (128 * K, 384 * K, 8192, WT),
        (128 * K, 192 * K, 8192, NT), (128 * K, 160 * K, 8192, NT), (128 * K, 132 * K, 8192, WT),
        (48 * K, 384 * K, 16384, NT), (96 * K, 384 * K, 8192, NT), (32 * K, 192 * K, 32768, NT), (64 * K, 768 * K, 8192, WT),
        (128 * K, 136 * K + 128, 8192, NT),
        (16 * K, 16 * K + 256, 65536, WT), (16 * K, 20 * K, 65536, NT), (16 * K, 32 * K, 65536, WT),
        (2 * K, 4 * K, 262144, WT), (2 * K, 4352, 262144, NT), (2 * K, 2304, 262144, NT),
        (1 * K, 2 * K, 524288, WT), (1 * K, 2304, 524288, NT),              # the slot kernel, one row a wave
        (512, 2176, 524288, WT), (256, 640, 1 << 20, WT), (128, 384, 1 << 20, WT),
    ]
    for width, pitch, rows, want in cases:
        st, p = capi_host.plan_rect((base_d, pitch, 0), (0, 0, 0), (base_s, pitch, 0), (0, 0, 0), (width, rows, 1))
        assert st == SUCCESS and p.nt_load == 1 and p.store_policy == want, (width, pitch, p.store_policy)
        # the source's pitch plays no part
        st, p = capi_host.plan_rect((base_d, pitch, 0), (0, 0, 0), (base_s, 2 * pitch + 128, 0), (0, 0, 0), (width, rows, 1))
        assert st == SUCCESS and p.store_policy == want, (width, pitch)
    # with bytes to realign the rule is the same; rows that are not whole lines keep non-temporal stores
    st, p = capi_host.plan_rect((base_d, 8448, 0), (0, 0, 0), (base_s, 8448, 0), (1, 0, 0), (4096, 262144, 1))
    assert st == SUCCESS and p.store_policy == NT
    st, p = capi_host.plan_rect((base_d, 8192, 0), (0, 0, 0), (base_s, 8192, 0), (1, 0, 0), (4096, 262144, 1))
    assert st == SUCCESS and p.store_policy == WT
    st, p = capi_host.plan_rect((base_d, 8192, 0), (16, 0, 0), (base_s, 8192, 0), (0, 0, 0), (4096, 262144, 1))
    assert st == SUCCESS and p.store_policy == NT
    # below 4 MiB nothing bypasses the caches, and tuning overrides the rule
    st, p = capi_host.plan_rect((base_d, 4352, 0), (0, 0, 0), (base_s, 4352, 0), (0, 0, 0), (2048, 64, 1))
    assert st == SUCCESS and p.store_policy == capi_host.STORE_CACHED
    st, p = capi_host.plan_rect((base_d, 4352, 0), (0, 0, 0), (base_s, 4352, 0), (0, 0, 0), (2048, 262144, 1),
                                capi_host.Tuning(store_policy=3))
    assert st == SUCCESS and p.store_policy == WT


def test_plan_rect_plain_rows_order_follows_the_pitches(capi_host):
    """Plain rows of a large region run in XCD runs of 576 units, except where
    launch order or longer runs were measured to win
    (rect_plain_rows_in_launch_order, rect_plain_rows_run_units): both pitches
    powers of two and rows of 4 KiB or a multiple of 8 KiB up to 48 KiB that take
    up an eighth to three eighths of a pitch; and, for surfaces of one
    power-of-two pitch, 8 KiB rows at 16 KiB and rows of 16 or 32 KiB at 16 times
    their width (launch order) and rows of 128 KiB and more at 512 KiB and more
    (runs of 2304)."""
    base_d, base_s = 0x7f0000000000, 0x7f1000000000
    K = 1024
    GIB = 1 << 30
    cases = [
        # width, destination pitch, source pitch, units per run (0: launch order)
        (32 * K, 128 * K, 128 * K, 0), (32 * K, 256 * K, 256 * K, 0), (32 * K, 64 * K, 64 * K, 576),
        (32 * K, 512 * K, 512 * K, 0), (32 * K, 128 * K, 256 * K, 0), (32 * K, 32 * K, 128 * K, 0),
        (32 * K, 128 * K, 32 * K, 0), (32 * K, 128 * K + 256, 128 * K, 576), (32 * K, 128 * K, 128 * K + 256, 576),
        (4 * K, 16 * K, 16 * K, 0), (4 * K, 8 * K, 8 * K, 576), (8 * K, 32 * K, 32 * K, 0),
        (12 * K, 64 * K, 64 * K, 576), (24 * K, 64 * K, 64 * K, 0), (48 * K, 128 * K, 128 * K, 0),
        (64 * K, 256 * K, 256 * K, 576), (2 * K, 8 * K, 8 * K, 576), (128 * K, 512 * K, 512 * K, 2304),
        (8 * K, 16 * K, 16 * K, 0), (16 * K, 256 * K, 256 * K, 0), (4 * K, 64 * K, 64 * K, 576),
        (256 * K, 1024 * K, 1024 * K, 2304), (128 * K, 256 * K, 256 * K, 576),
        # any pitch that is not a power of two: runs of 576
        (128 * K, 384 * K, 384 * K, 576), (128 * K, 768 * K, 768 * K, 576), (64 * K, 384 * K, 384 * K, 576),
        (2 * K, 6 * K, 6 * K, 576), (4 * K, 12 * K, 12 * K, 576), (32 * K, 96 * K, 96 * K, 576),
        (48 * K, 384 * K, 384 * K, 576), (12 * K, 192 * K, 192 * K, 576), (128 * K, 260 * K, 260 * K, 576),
        (16 * K, 68 * K, 68 * K, 576),
    ]
    for width, dp, sp, units in cases:
        rows = min(GIB // width, (12 * GIB) // dp)
        st, p = capi_host.plan_rect((base_d, dp, 0), (0, 0, 0), (base_s, sp, 0), (0, 0, 0), (width, rows, 1))
        assert st == SUCCESS and p.plain_rows == 1 and p.wg_size == 64, (width, dp, sp)
        assert p.xcd_run == units, (width, dp, sp, p.xcd_run)
    # x offsets change nothing; several layers, a small region and tuning do
    st, p = capi_host.plan_rect((base_d, 128 * K, 0), (4096, 0, 0), (base_s, 128 * K, 0), (8192, 0, 0), (32 * K, 32768, 1))
    assert st == SUCCESS and (p.plain_rows, p.xcd_run) == (1, 0)
    st, p = capi_host.plan_rect((base_d, 128 * K, 1 << 30), (0, 0, 0), (base_s, 128 * K, 1 << 30), (0, 0, 0),
                                (32 * K, 4096, 4))
    assert st == SUCCESS and (p.plain_rows, p.xcd_run) == (1, 576)
    st, p = capi_host.plan_rect((base_d, 128 * K, 0), (0, 0, 0), (base_s, 128 * K, 0), (0, 0, 0), (32 * K, 32768, 1),
                                capi_host.Tuning(xcd_run=288))
    assert st == SUCCESS and p.xcd_run == 288


def test_plan_rect_routes_across_the_host_link(capi_host):
    """A region one side of which is host memory: the same rows, slots and
    merging, launched as at most 128 workgroups of 256 in launch order, stores
    to the host written through at system scope."""
    h2d, d2h = capi_host.ROUTE_HOST_TO_DEVICE, capi_host.ROUTE_DEVICE_TO_HOST
    d, s = 0x7f0000000000, 0x7e0000000000
    regions = [
        ((d, 262144, 0), (0, 0, 0), (s, 262144, 0), (0, 0, 0), (131072, 8192, 1)),       # plain rows, 1 GiB
        ((d, 20000, 0), (17, 1, 0), (s, 21000, 0), (3001, 0, 0), (16385, 4000, 1)),     # wide rows, any alignment
        ((d, 512, 0), (256, 0, 0), (s, 512, 0), (0, 0, 0), (256, 1 << 20, 1)),          # narrow, whole lines
        ((d, 1024, 0), (3, 0, 0), (s, 1024, 0), (9, 0, 0), (1000, 1 << 18, 1)),         # narrow, sharing lines
    ]
    for dst, do, src, so, ext in regions:
        st, dev = capi_host.plan_rect(dst, do, src, so, ext)
        assert st == 0 and dev.route == capi_host.ROUTE_DEVICE
        for route in (h2d, d2h):
            st, p = capi_host.plan_rect(dst, do, src, so, ext, route=route)
            assert st == 0 and p.route == route
            for f in ("empty", "linear", "dst", "src", "width", "rows", "layers", "lanes_per_row", "total_bytes",
                      "dst_pitch", "src_pitch", "nt_load"):
                assert getattr(p, f) == getattr(dev, f), f
            assert (p.wg_size, p.xcd_run) == (256, 0) and p.grid <= 128
            if p.lanes_per_row == 0:
                assert p.unroll == 1
            if route == d2h:
                assert p.store_policy == capi_host.STORE_SYSTEM_WT
            else:
                assert p.store_policy in (capi_host.STORE_NT, capi_host.STORE_AGENT_WT)
    # a region that merges into one run is a linear copy on the same route
    st, p = capi_host.plan_rect((d, 4096, 4096 * 50), (0, 0, 0), (s, 4096, 4096 * 50), (0, 0, 0), (4096, 50, 2), route=h2d)
    assert st == 0 and p.linear and p.route == h2d
    # tuning still overrides, an unknown route is refused
    st, p = capi_host.plan_rect(*regions[0], capi_host.Tuning(max_grid=1000, wg_size=64, store_policy=2), route=d2h)
    assert st == 0 and (p.wg_size, p.grid, p.store_policy) == (64, 1000, capi_host.STORE_NT)
    st, p = capi_host.plan_rect(*regions[0], route=3)
    assert st == capi_host.ERROR_INVALID_ARGUMENT


def test_plan_rect_validation_matches_reference(capi_host, oracle):
    """Same verdict as the reference's checks on every case, except that the
    SDMA packet's dword alignment is not demanded."""
    rng = np.random.default_rng(7)
    n_bad = 0
    for _ in range(2000):
        d = (0x7f0000000000 + int(rng.integers(0, 64)), int(rng.integers(1, 600)), 0)
        s = (0x7f1000000000 + int(rng.integers(0, 64)), int(rng.integers(1, 600)), 0)
        if rng.integers(0, 3):
            d = (d[0], d[1], d[1] * int(rng.integers(1, 20)))
        if rng.integers(0, 3):
            s = (s[0], s[1], s[1] * int(rng.integers(1, 20)))
        ext = tuple(int(v) for v in rng.integers(0, [500, 16, 4]))
        do = tuple(int(v) for v in rng.integers(0, [200, 10, 3]))
        so = tuple(int(v) for v in rng.integers(0, [200, 10, 3]))
        want, work, _ = oracle_validate_rect(oracle, d, do, s, so, ext)
        st, p = capi_host.plan_rect(d, do, s, so, ext)
        assert st == want, (d, do, s, so, ext)
        if st == SUCCESS:
            assert bool(p.empty) == (work == 0)
        else:
            n_bad += 1
    assert 200 < n_bad < 1800  # the sweep exercises both verdicts
    z = (0, 0, 0)
    ok = ((0x1000, 64, 0), z, (0x2000, 64, 0), z, (8, 2, 1))
    for missing in range(5):
        args = list(ok)
        args[missing] = None
        assert capi_host.plan_rect(*args)[0] == INVALID_ARGUMENT
    assert capi_host.plan_rect((0, 64, 0), z, (0x2000, 64, 0), z, (8, 2, 1))[0] == INVALID_ARGUMENT  # NULL base
    # more rows than the slot index can count
    st, _ = capi_host.plan_rect((0x1000, 8, 8 * 70000), z, (0x2000, 8, 8 * 70000), z, (4, 70000, 70000))
    assert st == INVALID_ARGUMENT
