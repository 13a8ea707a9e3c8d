"""Parity of the pitched 3-D region copy (mi355_blit_copy_rect,
mi355_aql_copy_rect, mi355_hsa_amd_memory_async_copy_rect) with the CPU
oracle, through the C ABI and over both submission paths.  Bit-exact: the
whole destination surface, everything outside the region included, must equal
what oracle_copy_rect leaves on the same seeded inputs."""
import numpy as np
import pytest

from conftest import oracle_rect

pytestmark = pytest.mark.gpu

GUARD_BYTE = 0xEE
MIB = 1 << 20


class Surface:
    """A pitched device surface of [layers, rows, pitch] bytes at a chosen
    address residue modulo 256, with its host image."""

    def __init__(self, torch, shape, residue=0, host=None):
        self.torch = torch
        self.shape = shape
        self.nbytes = int(np.prod(shape))
        self.t = torch.empty(self.nbytes + 512, dtype=torch.uint8, device="cuda:0")
        shift = (residue - self.t.data_ptr()) % 256
        self.base = self.t.data_ptr() + shift
        self.view = self.t[shift:shift + self.nbytes]
        self.t.fill_(GUARD_BYTE)
        if host is not None:
            self.view.copy_(torch.from_numpy(host.reshape(-1)))
        torch.cuda.synchronize()
        self.shift = shift

    def pitched(self, base=None):
        z, y, x = self.shape
        return (self.base if base is None else base, x, y * x)

    def whole(self):
        return self.t.cpu().numpy()


def run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext, so, do, s_res=0, d_res=0, seed=1,
                  flat=False, submit=None):
    """ext, so, do are (x, y, z).  Returns the launch plan."""
    import torch
    src_host = rand(int(np.prod(sshape)), seed)
    src = Surface(torch, sshape, s_res, host=src_host)
    dst = Surface(torch, dshape, d_res)
    sp, dp = src.pitched(), dst.pitched()
    if flat:  # 2-D surfaces may leave the slice pitch at 0
        sp, dp = (sp[0], sp[1], 0), (dp[0], dp[1], 0)
    if submit is None:
        st = blit.copy_rect(dp, do, sp, so, ext)
    else:
        st = submit(dp, do, sp, so, ext)
    assert st == capi.SUCCESS, "copy_rect returned 0x%x" % st
    assert blit.synchronize() == capi.SUCCESS
    got = dst.whole()
    want = np.full(got.size, GUARD_BYTE, dtype=np.uint8)
    oracle_rect(oracle, (want.ctypes.data + dst.shift,) + dp[1:], do, (src_host.ctypes.data,) + sp[1:], so, ext)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, "first mismatch at surface byte %d of %d (%d wrong)" % (
        bad[0] - dst.shift, dst.nbytes, bad.size)
    return blit.last_plan()


CASES = [
    # sshape (z, y, pitch), dshape, extent (x, y, z), src offset, dst offset, src residue, dst residue
    ((1, 16, 300), (1, 12, 517), (100, 7, 1), (13, 2, 0), (5, 3, 0), 0, 0),
    ((1, 16, 300), (1, 12, 517), (100, 7, 1), (13, 2, 0), (5, 3, 0), 7, 201),
    ((4, 9, 1031), (5, 11, 1500), (1000, 5, 3), (31, 4, 1), (499, 6, 2), 3, 9),
    ((1, 64, 131072), (1, 64, 131072), (65536, 64, 1), (0, 0, 0), (65536, 0, 0), 0, 0),
    ((1, 64, 131072), (1, 70, 131072 + 256), (65536, 64, 1), (1, 0, 0), (48, 3, 0), 0, 0),
    ((1, 4096, 256), (1, 4096, 256), (64, 4096, 1), (64, 0, 0), (128, 0, 0), 0, 0),
    ((1, 4096, 256), (1, 4096, 260), (64, 4096, 1), (63, 0, 0), (130, 0, 0), 0, 0),
    ((3, 300, 37), (3, 301, 41), (1, 300, 3), (36, 0, 0), (0, 1, 0), 1, 255),
    ((2, 50, 4096), (2, 50, 4096), (4096, 50, 2), (0, 0, 0), (0, 0, 0), 0, 0),       # merges into one run
    ((2, 64, 4096), (2, 50, 4096), (4096, 50, 2), (0, 14, 0), (0, 0, 0), 0, 16),     # merges into two rows
    ((8, 1, 5000), (8, 3, 6000), (4999, 1, 8), (1, 0, 0), (2, 2, 0), 5, 6),          # one row per layer
    ((1, 1, 70000), (1, 1, 90000), (66000, 1, 1), (1234, 0, 0), (4321, 0, 0), 2, 3),  # a single row
    ((1, 33, 9001), (1, 35, 9473), (8999, 33, 1), (1, 0, 0), (471, 2, 0), 0, 0),
    ((2, 17, 20000), (3, 19, 21000), (16385, 17, 2), (3000, 0, 0), (17, 1, 1), 11, 13),
    ((1, 2048, 4096), (1, 2048, 8192), (2048, 2048, 1), (2048, 0, 0), (4096, 0, 0), 0, 0),  # 4 MiB: streaming
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_rect_cases_are_exact(capi, blit, oracle, rand, case):
    sshape, dshape, ext, so, do, s_res, d_res = CASES[case]
    run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext, so, do, s_res, d_res, seed=0x2EC70000 + case)


def test_rect_flat_surfaces_need_no_slice(capi, blit, oracle, rand):
    run_rect_case(capi, blit, oracle, rand, (1, 40, 3000), (1, 50, 3100), (2999, 40, 1), (1, 0, 0), (99, 10, 0),
                  flat=True, seed=77)


@pytest.mark.parametrize("seed", range(24))
def test_rect_random_regions(capi, fresh_tuning, oracle, rand, seed):
    """Seeded regions with every alignment of bases, pitches, offsets and
    widths, under random launch shapes."""
    blit = fresh_tuning
    rng = np.random.default_rng(0x5EC7 + seed)
    sshape = tuple(int(v) for v in rng.integers(1, [5, 40, 12000]))
    dshape = tuple(int(v) for v in rng.integers(1, [5, 40, 12000]))
    ext = [int(rng.integers(1, min(sshape[k], dshape[k]) + 1)) for k in range(3)]
    so = [int(rng.integers(0, sshape[k] - ext[k] + 1)) for k in range(3)]
    do = [int(rng.integers(0, dshape[k] - ext[k] + 1)) for k in range(3)]
    if seed % 2:
        blit.set_tuning(wg_size=int(rng.choice([64, 128, 256, 512, 1024])), unroll=int(rng.choice([1, 2, 4])),
                        max_grid=int(rng.choice([0, 1, 7, 300])), nt_load=int(rng.integers(0, 3)),
                        store_policy=int(rng.integers(0, 5)))
    run_rect_case(capi, blit, oracle, rand, sshape, dshape, tuple(ext[::-1]), tuple(so[::-1]), tuple(do[::-1]),
                  int(rng.integers(0, 256)), int(rng.integers(0, 256)), seed=0x7EC70000 + seed)


@pytest.mark.parametrize("seed", range(24))
def test_rect_random_narrow_rows(capi, fresh_tuning, oracle, rand, seed):
    """Rows of 1..1100 bytes, the widths that are packed several rows to a wave
    (and the first ones beyond), many rows, every alignment."""
    blit = fresh_tuning
    rng = np.random.default_rng(0xA220 + seed)
    widest = 700 if seed < 16 else 1400
    sshape = tuple(int(v) for v in rng.integers(1, [5, 700, widest]))
    dshape = tuple(int(v) for v in rng.integers(1, [5, 700, widest]))
    ext = [int(rng.integers(1, min(sshape[k], dshape[k]) + 1)) for k in range(3)]
    ext[2] = min(ext[2], 1100)
    if seed % 3 == 0:  # pitches that keep every row at one alignment
        sshape = (sshape[0], sshape[1], (sshape[2] + 15) // 16 * 16)
        dshape = (dshape[0], dshape[1], (dshape[2] + 15) // 16 * 16)
    so = [int(rng.integers(0, sshape[k] - ext[k] + 1)) for k in range(3)]
    do = [int(rng.integers(0, dshape[k] - ext[k] + 1)) for k in range(3)]
    if seed % 2:
        blit.set_tuning(wg_size=int(rng.choice([64, 256, 1024])), max_grid=int(rng.choice([0, 1, 5])),
                        nt_load=int(rng.integers(0, 3)), store_policy=int(rng.integers(0, 5)))
    run_rect_case(capi, blit, oracle, rand, sshape, dshape, tuple(ext[::-1]), tuple(so[::-1]), tuple(do[::-1]),
                  int(rng.integers(0, 256)), int(rng.integers(0, 256)), seed=0x7A220000 + seed)


@pytest.mark.parametrize("width", [1101, 1337, 1600, 1999, 2047])
def test_rect_ragged_rows_wider_than_a_wave(capi, fresh_tuning, oracle, rand, width):
    """Ragged rows of 1101..2047 bytes go to the slot kernel with up to 128
    lanes per row, where a wave holds less than a row and a lane's row within
    the wave is 0 or 1: odd x offsets and pitches, hundreds of rows in 3 layers,
    single waves and large workgroups, capped grids (waves striding over the
    slots) and launches permuted in XCD runs."""
    blit = fresh_tuning
    rows = 211
    sshape, dshape = (3, rows + 9, width + 333), (3, rows + 4, 2 * width + 77)
    ext, so, do = (width, rows, 3), (7 + width % 5, 5, 0), (width - 3, 2, 0)
    for wg, max_grid, xcd_run in ((64, 0, 1), (256, 0, 1), (1024, 0, 1), (64, 1, 1), (256, 5, 1), (64, 0, 3),
                                  (256, 0, 2)):
        blit.set_tuning(wg_size=wg, max_grid=max_grid, xcd_run=xcd_run)
        p = run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext, so, do, 5, 130 + (width & 15),
                          seed=0x7A22F000 + width)
        assert p.kernel == capi.KERNEL_COPY_RECT and p.wg_size == wg
    st, plan = capi.plan_rect((1 << 40, dshape[2], dshape[1] * dshape[2]), do, (1 << 41, sshape[2], sshape[1] * sshape[2]),
                              so, ext, None)
    assert st == capi.SUCCESS
    if width <= 2000:  # 2047 bytes can touch 129 slots: the first width that goes to the unit kernel
        assert 64 < plan.lanes_per_row <= 128 and plan.slots == 0, (
            "the case is meant for the slot kernel with more than a wave per row", plan.lanes_per_row, plan.slots)


@pytest.mark.parametrize("xcd_run", [2, 3, 36])
def test_rect_permuted_launches_are_exact(capi, fresh_tuning, oracle, rand, xcd_run):
    """Both region kernels with their workgroups dealt to the XCDs in runs: a
    permutation of the same row units, so the same bytes.  Grids of a few
    hundred to a few thousand workgroups, not whole rounds of 8 runs."""
    blit = fresh_tuning
    for wg, max_grid in ((64, 0), (256, 0), (128, 50)):
        blit.set_tuning(wg_size=wg, xcd_run=xcd_run, max_grid=max_grid)
        # wide rows: 61 rows of 9001 bytes, 9 units of 1 KiB each
        p = run_rect_case(capi, blit, oracle, rand, (2, 40, 12000), (2, 37, 11003), (9001, 31, 2), (7, 3, 0),
                          (1001, 2, 0), 3, 77, seed=0x7EC7AA00 + xcd_run)
        assert p.kernel == capi.KERNEL_COPY_RECT and p.xcd_run == xcd_run
        # narrow rows: 3 x 500 rows of 333 bytes
        p = run_rect_case(capi, blit, oracle, rand, (3, 600, 517), (3, 550, 400), (333, 500, 3), (13, 20, 0),
                          (5, 31, 0), 9, 130, seed=0x7EC7BB00 + xcd_run)
        assert p.kernel == capi.KERNEL_COPY_RECT and p.xcd_run == xcd_run


@pytest.mark.parametrize("unroll", [1, 2, 4])
def test_rect_plain_rows_are_exact(capi, fresh_tuning, oracle, rand, unroll):
    """Rows tiled like a linear copy (256-byte aligned destination rows, whole
    units, source a multiple of 4 bytes away) take the kernel's short path:
    same bytes, under every launch shape, in launch order and in XCD runs, and
    a region that misses one of the conditions takes the general path."""
    blit = fresh_tuning
    sshape, dshape = (2, 20, 8192), (2, 18, 12288)
    ext, so, do = (4096, 15, 2), (1028, 3, 0), (512, 2, 0)
    for wg, xcd_run, max_grid in ((64, 1, 0), (256, 3, 0), (128, 2, 37), (1024, 1, 0)):
        blit.set_tuning(wg_size=wg, unroll=unroll, xcd_run=xcd_run, max_grid=max_grid)
        p = run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext, so, do, 0, 0, seed=0x7EC7CC00 + unroll)
        assert p.kernel == capi.KERNEL_COPY_RECT and p.unroll == unroll
    t = capi.Tuning(unroll=unroll)
    st, plan = capi.plan_rect((1 << 40, 12288, 12288 * 18), do, (1 << 41, 8192, 8192 * 20), so, ext, t)
    assert st == capi.SUCCESS and plan.plain_rows == 1 and plan.slots == 4096 // (1024 * unroll)
    # rows of whole lines whose last unit is a partial one are plain too
    for width in (4096 - 256, 4096 + 128, 128, 1024 * unroll + 128, 1024 * unroll + 256, 7 * 1024 - 128):
        ext3 = (width, 15, 2)
        st, plan = capi.plan_rect((1 << 40, 12288, 12288 * 18), do, (1 << 41, 8192, 8192 * 20), so, ext3, t)
        if width > 1024:   # narrower rows go to the kernel that packs rows into waves
            n_vec, unit = width // 16, 64 * unroll
            assert st == capi.SUCCESS and plan.plain_rows == 1
            assert plan.slots == (-(-n_vec // unit) if n_vec > 15 + unit else 1)
        for wg, xcd_run in ((64, 1), (256, 3)):
            blit.set_tuning(wg_size=wg, unroll=unroll, xcd_run=xcd_run)
            run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext3, so, do, 0, 0, seed=0x7EC7EE00 + width)
    # one condition off at a time: destination x, source x, width
    for so2, do2, ext2 in (((1028, 3, 0), (576, 2, 0), ext), ((1030, 3, 0), do, ext), (so, do, (4096 - 64, 15, 2))):
        st, plan = capi.plan_rect((1 << 40, 12288, 12288 * 18), do2, (1 << 41, 8192, 8192 * 20), so2, ext2, t)
        assert st == capi.SUCCESS and plan.plain_rows == 0
        blit.set_tuning(unroll=unroll)
        run_rect_case(capi, blit, oracle, rand, sshape, dshape, ext2, so2, do2, 0, 0, seed=0x7EC7DD00 + unroll)


def test_rect_plan_shapes(capi, blit, oracle, rand):
    """What the launch record says: a rect kernel with one wave per 1 KiB of
    row for rows of whole cache lines, a linear copy when the region is one run."""
    p = run_rect_case(capi, blit, oracle, rand, (1, 64, 16384), (1, 64, 16384), (8192, 64, 1), (0, 0, 0), (8192, 0, 0))
    assert p.kernel == capi.KERNEL_COPY_RECT and p.body_vecs == 64 * 8 and p.unroll == 1
    assert p.grid * (p.wg_size // 64) == 64 * 8
    p = run_rect_case(capi, blit, oracle, rand, (1, 64, 8192), (1, 64, 8192), (8192, 64, 1), (0, 0, 0), (0, 0, 0))
    assert p.kernel == capi.KERNEL_COPY


def test_rect_argument_checks(capi, blit, torch_cuda):
    torch = torch_cuda
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    d = (buf.data_ptr(), 256, 256 * 16)
    s = (buf.data_ptr() + (1 << 15), 256, 256 * 16)
    z = (0, 0, 0)
    ok = [d, z, s, z, (64, 4, 2)]
    for missing in range(5):
        args = list(ok)
        args[missing] = None
        assert blit.copy_rect(*args) == capi.ERROR_INVALID_ARGUMENT
    assert blit.copy_rect((0, 256, 0), z, s, z, (64, 4, 1)) == capi.ERROR_INVALID_ARGUMENT
    assert blit.copy_rect(d, (200, 0, 0), s, z, (64, 4, 2)) == capi.ERROR_INVALID_ARGUMENT      # width out of range
    assert blit.copy_rect(d, z, s, (0, 13, 0), (64, 4, 2)) == capi.ERROR_INVALID_ARGUMENT       # height out of range
    assert blit.copy_rect((d[0], 256, 0), z, s, z, (64, 4, 2)) == capi.ERROR_INVALID_ARGUMENT   # slice needed
    for ext in ((0, 4, 2), (64, 0, 2), (64, 4, 0)):
        assert blit.copy_rect(d, z, s, z, ext) == capi.SUCCESS
    assert blit.synchronize() == capi.SUCCESS
    assert int(buf.sum().item()) == 0


def test_rect_one_gib_region(capi, blit, oracle, rand, torch_cuda):
    """8192 rows of 128 KiB out of 256 KiB-pitch surfaces: 1 GiB moved.  The
    whole destination is checked on the device against torch's own strided
    view assignment, and sampled rows against the oracle on the host."""
    torch = torch_cuda
    rows, pitch, width = 8192, 256 * 1024, 128 * 1024
    seedrow = torch.from_numpy(rand(pitch + 4096, 0x16187EC7)).to("cuda:0")
    src = torch.empty(rows * pitch, dtype=torch.uint8, device="cuda:0")
    s2 = src.view(rows, pitch)
    for blk in range(0, rows, 1024):  # every row differs: rotate the seed row
        idx = (torch.arange(blk, blk + 1024, device="cuda:0") * 37 % 4096)[:, None] + \
            torch.arange(pitch, device="cuda:0")[None, :]
        s2[blk:blk + 1024] = seedrow[idx]
        del idx
    dst = torch.full((rows * pitch,), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    so, do = (4096 + 3, 0, 0), (65536 + 16, 0, 0)
    st = blit.copy_rect((dst.data_ptr(), pitch, 0), do, (src.data_ptr(), pitch, 0), so, (width, rows, 1))
    assert st == capi.SUCCESS and blit.synchronize() == capi.SUCCESS
    p = blit.last_plan()
    assert p.kernel == capi.KERNEL_COPY_RECT and p.nt_load == 1
    d2 = dst.view(rows, pitch)
    assert torch.equal(d2[:, do[0]:do[0] + width], s2[:, so[0]:so[0] + width])
    assert bool((d2[:, :do[0]] == GUARD_BYTE).all()) and bool((d2[:, do[0] + width:] == GUARD_BYTE).all())
    for y in (0, 1, 63, 4095, 8190, 8191):
        src_row = s2[y].cpu().numpy()
        want = np.full(pitch, GUARD_BYTE, dtype=np.uint8)
        oracle_rect(oracle, (want.ctypes.data, pitch, 0), (do[0], 0, 0), (src_row.ctypes.data, pitch, 0),
                    (so[0], 0, 0), (width, 1, 1))
        assert np.array_equal(d2[y].cpu().numpy(), want)


def test_rect_merged_rows_beyond_4gib(capi, blit, torch_cuda):
    """Two layers of 4608 contiguous 1 MiB rows: each layer merges into one row
    of 4.5 GiB, more than a 32-bit byte count, 256 bytes off the 256-byte grid."""
    torch = torch_cuda
    row, rows, layers = MIB, 4608, 2
    layer_bytes = row * rows
    s_slice, d_slice = layer_bytes + 4096, layer_bytes + 8192
    src = torch.empty(layers * s_slice + 512, dtype=torch.uint8, device="cuda:0")
    pattern = torch.arange(0, 64 * MIB, dtype=torch.int32, device="cuda:0")
    pattern = (pattern * 2654435761 >> 7).to(torch.uint8)
    for lo in range(0, src.numel(), pattern.numel()):
        m = min(pattern.numel(), src.numel() - lo)
        src[lo:lo + m] = pattern[:m] + (lo >> 26)
    del pattern
    dst = torch.full((layers * d_slice + 512,), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    s_at, d_at = 48, 112
    st = blit.copy_rect((dst.data_ptr() + d_at, row, d_slice), (0, 0, 0), (src.data_ptr() + s_at, row, s_slice),
                        (0, 0, 0), (row, rows, layers))
    assert st == capi.SUCCESS and blit.synchronize() == capi.SUCCESS
    p = blit.last_plan()
    assert p.kernel == capi.KERNEL_COPY_RECT
    for z in range(layers):
        d0, s0 = d_at + z * d_slice, s_at + z * s_slice
        assert torch.equal(dst[d0:d0 + layer_bytes], src[s0:s0 + layer_bytes]), "layer %d" % z
        assert bool((dst[d0 + layer_bytes:d0 + d_slice] == GUARD_BYTE).all()), "gap behind layer %d" % z
    assert bool((dst[:d_at] == GUARD_BYTE).all())


def test_async_copy_rect_stand_in(capi, pkg, oracle, rand, torch_cuda):
    """mi355_hsa_amd_memory_async_copy_rect: the reference's answers at the API
    edge (hsa_ext_amd.cpp:367-410), dependencies honoured, the completion signal
    decremented once, bytes as the oracle's."""
    eng = pkg.aql.AqlBlit(0)
    sig = pkg.aql.HsaSignals()
    try:
        dep, done = sig.create(1), sig.create(1)

        def submit(dp, do, sp, so, ext):
            st = eng.hsa_amd_memory_async_copy_rect(dp, do, sp, so, ext, 3, [dep], done)
            assert sig.load(done) == 1          # blocked behind the dependency
            sig.store(dep, 0)
            sig.wait_below_one(done)
            assert sig.load(done) == 0
            return st
        run_rect_case(capi, eng, oracle, rand, (2, 30, 5000), (2, 31, 5100), (4097, 29, 2), (3, 1, 0), (1, 0, 0),
                      5, 250, seed=99, submit=submit)
        d, s, z, ext = (0x1000, 64, 0), (0x2000, 64, 0), (0, 0, 0), (8, 2, 1)
        f = eng.hsa_amd_memory_async_copy_rect
        assert f(d, z, s, z, ext, 0, None, done) == capi.ERROR_INVALID_ARGUMENT           # hsaHostToHost
        assert f(d, z, s, z, ext, 3, None, 0) == capi.ERROR_INVALID_ARGUMENT              # no completion signal
        for missing in range(5):
            args = [d, z, s, z, ext]
            args[missing] = None
            assert f(*args, 3, None, done) == capi.ERROR_INVALID_ARGUMENT
        arr = (pkg.aql.C.c_uint64 * 1)(dep)
        lib = eng.lib.mi355_hsa_amd_memory_async_copy_rect
        a = pkg.capi.rect_args(d, z, s, z, ext)
        assert lib(eng.handle, *a, 3, 0, arr, done) == capi.ERROR_INVALID_ARGUMENT        # array without a count
        assert lib(eng.handle, *a, 3, 1, None, done) == capi.ERROR_INVALID_ARGUMENT       # count without an array
        sig.store(done, 1)
        assert f(d, z, s, z, (8, 0, 1), 3, None, done) == capi.SUCCESS                    # empty: signal untouched
        assert eng.synchronize() == capi.SUCCESS
        assert sig.load(done) == 1
        sig.destroy(dep)
        sig.destroy(done)
    finally:
        eng.close()


LINK_CASES = [
    # (z, y, pitch) of both surfaces, extent (x, y, z), src offset, dst offset
    ((1, 600, 8192), (4096, 600, 1), (0, 0, 0), (4096, 0, 0)),       # plain rows
    ((2, 90, 20000), (16385, 80, 2), (3001, 3, 0), (17, 9, 0)),      # any alignment, wide rows
    ((1, 5000, 512), (256, 5000, 1), (0, 0, 0), (256, 0, 0)),        # narrow rows of whole lines
    ((3, 700, 261), (100, 650, 3), (13, 20, 0), (150, 1, 0)),        # narrow rows, every alignment
    ((2, 50, 4096), (4096, 50, 2), (0, 0, 0), (0, 0, 0)),            # merges into one run: a linear copy
]


@pytest.mark.parametrize("case", range(len(LINK_CASES)))
def test_rect_across_the_host_link(capi, blit, pkg, oracle, rand, torch_cuda, case):
    """Regions between pinned host surfaces and device surfaces on the routes made
    for the host link, over the HIP path (route argument) and over the stand-in
    for hsa_amd_memory_async_copy_rect (its direction argument): the launch is the
    link's shape and both destination surfaces, guard bytes included, are the
    oracle's."""
    torch = torch_cuda
    shape, ext, so, do = LINK_CASES[case]
    nbytes = int(np.prod(shape))
    pitched = lambda base: (base, shape[2], shape[1] * shape[2])
    payload = rand(nbytes, 0x11CC0000 + case)
    host_in = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    host_in.numpy()[:] = payload
    want_dev = np.full(nbytes, GUARD_BYTE, dtype=np.uint8)
    oracle_rect(oracle, pitched(want_dev.ctypes.data), do, pitched(payload.ctypes.data), so, ext)
    want_out = np.full(nbytes, GUARD_BYTE, dtype=np.uint8)
    oracle_rect(oracle, pitched(want_out.ctypes.data), so, pitched(want_dev.ctypes.data), do, ext)
    eng = pkg.aql.AqlBlit(0)
    sig = pkg.aql.HsaSignals()
    done = sig.create(1)
    try:
        for path in ("hip", "aql"):
            dev = torch.full((nbytes,), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
            host_out = torch.full((nbytes,), GUARD_BYTE, dtype=torch.uint8).pin_memory()
            torch.cuda.synchronize()
            legs = ((capi.ROUTE_HOST_TO_DEVICE, pitched(dev.data_ptr()), do, pitched(host_in.data_ptr()), so),
                    (capi.ROUTE_DEVICE_TO_HOST, pitched(host_out.data_ptr()), so, pitched(dev.data_ptr()), do))
            for route, dp, d_at, sp, s_at in legs:
                if path == "hip":
                    assert blit.copy_rect(dp, d_at, sp, s_at, ext, route=route) == capi.SUCCESS
                    assert blit.synchronize() == capi.SUCCESS
                    p = blit.last_plan()
                else:
                    sig.store(done, 1)
                    assert eng.hsa_amd_memory_async_copy_rect(dp, d_at, sp, s_at, ext, route, None, done) == capi.SUCCESS
                    sig.wait_below_one(done)
                    p = eng.last_plan()
                assert p.route == route and p.wg_size == 256 and p.grid <= 128 and p.xcd_run == 0
                if route == capi.ROUTE_DEVICE_TO_HOST and nbytes >= 4 * MIB:
                    assert p.store_policy == capi.STORE_SYSTEM_WT
            assert np.array_equal(dev.cpu().numpy(), want_dev), path
            assert np.array_equal(host_out.numpy(), want_out), path
    finally:
        sig.destroy(done)
        eng.close()
