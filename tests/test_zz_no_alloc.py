"""The allocation-free batched copy (mi355_blit_copy_batch_bounded_noalloc)
against the entry point it is a variant of (mi355_blit_copy_batch_bounded) and
against the CPU oracle, through the C ABI.  Bit-exact, guard bands included.

Collected last on purpose: the round's GPU run stops at the first failure."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD_BYTE = 0xEE
MIB = 1 << 20


@pytest.fixture(scope="module")
def hip_blit(capi):
    b = capi.Blit(0)
    yield b
    b.close()


def _device_bytes(torch, nbytes, host=None):
    """(tensor, 256-byte aligned view) of nbytes on cuda:0."""
    t = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda:0")
    shift = (-t.data_ptr()) % 256
    v = t[shift:shift + nbytes]
    if host is not None:
        v.copy_(torch.from_numpy(host))
    return t, v


def _carve(capi, rng, src_base, dst_base, n, min_len, max_len, room):
    """n copies carved one behind the other with guard gaps, offsets 0..15 on
    the source side and anywhere within 256 bytes on the destination side."""
    lens = np.floor(min_len * 2.0 ** (np.log2(max_len / min_len) * rng.random(n))).astype(np.int64)
    so = rng.integers(0, 16, n)
    do = rng.integers(0, 256, n)
    stride = ((lens + 255) // 256) * 256 + 512
    offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
    total = int(offs[-1] + stride[-1] + 256)
    assert total <= room, (total, room)
    descs = (capi.Desc * n)()
    for i in range(n):
        descs[i].dst = dst_base + int(offs[i] + do[i])
        descs[i].src = src_base + int(offs[i] + so[i])
        descs[i].bytes = int(lens[i])
    return descs, lens, offs, so, do, total


def _to_device(torch, descs):
    raw = np.frombuffer(bytes(descs), dtype=np.uint8).copy()
    return torch.from_numpy(raw).to("cuda:0")


def _ok(capi, st, what):
    assert st == capi.SUCCESS, "%s returned 0x%x" % (what, st)


def test_noalloc_batch_matches_the_allocating_entry_point_twice_in_a_row(capi, hip_blit, oracle, rand, torch_cuda):
    """Two calls in a row on one GPU, the second with fewer and shorter copies:
    the scratch array keeps the first call's prefix sums and records, and the
    second call must not read any of them.  Each call's destination must equal,
    byte for byte, what mi355_blit_copy_batch_bounded leaves on the same
    descriptors, and what the oracle's memcpy leaves."""
    torch = torch_cuda
    blit = hip_blit
    room = 40 * MIB
    src_host = rand(room, 0xB1170A01)
    _s, src = _device_bytes(torch, room, host=src_host)
    _a, dst_a = _device_bytes(torch, room)   # the allocation-free entry point writes here
    _b, dst_b = _device_bytes(torch, room)   # the existing entry point writes here
    for call, (seed, n, min_len, max_len) in enumerate([(11, 3000, 64, 64 << 10), (12, 700, 1, 9000)]):
        rng = np.random.default_rng(seed)
        descs_a, lens, offs, so, do, total = _carve(capi, rng, src.data_ptr(), dst_a.data_ptr(), n, min_len, max_len, room)
        descs_b = (capi.Desc * n)()
        for i in range(n):
            descs_b[i].dst = descs_a[i].dst - dst_a.data_ptr() + dst_b.data_ptr()
            descs_b[i].src = descs_a[i].src
            descs_b[i].bytes = descs_a[i].bytes
        for i in range(0, n, 9):  # copies of no bytes share their first chunk with their successor
            descs_a[i].bytes = descs_b[i].bytes = 0
            lens[i] = 0
        dev_a, dev_b = _to_device(torch, descs_a), _to_device(torch, descs_b)
        dst_a.fill_(GUARD_BYTE)
        dst_b.fill_(GUARD_BYTE)
        torch.cuda.synchronize()
        bound = int(lens.sum())
        _ok(capi, blit.copy_batch_bounded_noalloc(dev_a.data_ptr(), n, bound), "copy_batch_bounded_noalloc")
        _ok(capi, blit.copy_batch_bounded(dev_b.data_ptr(), n, bound), "copy_batch_bounded")
        _ok(capi, blit.synchronize(), "synchronize")
        got_a = dst_a.cpu().numpy()
        got_b = dst_b.cpu().numpy()
        assert np.array_equal(got_a, got_b), "call %d: differs from mi355_blit_copy_batch_bounded" % call
        want = np.full(room, GUARD_BYTE, dtype=np.uint8)
        for i in range(n):
            oracle.oracle_copy(want.ctypes.data + int(offs[i] + do[i]), src_host.ctypes.data + int(offs[i] + so[i]),
                               int(lens[i]))
        assert np.array_equal(got_a, want), "call %d: differs from the oracle" % call
        assert blit.last_plan().kernel == capi.KERNEL_COPY_BATCH


def test_noalloc_batch_bound_exceeded_and_limits(capi, hip_blit, oracle, rand, torch_cuda):
    """A bound the copies exceed (most chunks without a wave of their own), the
    largest number of copies the scratch holds, one more (refused, nothing
    launched), and the argument checks of the entry point it mirrors."""
    torch = torch_cuda
    blit = hip_blit
    room = 56 * MIB
    src_host = rand(room, 0xB1170A02)
    _s, src = _device_bytes(torch, room, host=src_host)
    _a, dst = _device_bytes(torch, room)

    def run(seed, n, min_len, max_len, bound):
        rng = np.random.default_rng(seed)
        descs, lens, offs, so, do, total = _carve(capi, rng, src.data_ptr(), dst.data_ptr(), n, min_len, max_len, room)
        dev = _to_device(torch, descs)
        dst.fill_(GUARD_BYTE)
        torch.cuda.synchronize()
        _ok(capi, blit.copy_batch_bounded_noalloc(dev.data_ptr(), n, bound or int(lens.sum())), "noalloc")
        _ok(capi, blit.synchronize(), "synchronize")
        want = np.full(room, GUARD_BYTE, dtype=np.uint8)
        for i in range(n):
            oracle.oracle_copy(want.ctypes.data + int(offs[i] + do[i]), src_host.ctypes.data + int(offs[i] + so[i]),
                               int(lens[i]))
        assert np.array_equal(dst.cpu().numpy(), want), (seed, n)
        return dev

    run(21, 2100, 8 << 10, 24 << 10, 1)
    nmax = capi.NOALLOC_MAX_COPIES
    dev = run(22, nmax, 1, 200, 0)
    # one copy more than the scratch has prefix sums for: refused, nothing runs
    dst.fill_(GUARD_BYTE)
    torch.cuda.synchronize()
    assert blit.copy_batch_bounded_noalloc(dev.data_ptr(), nmax + 1, 1 << 20) == capi.ERROR_OUT_OF_RESOURCES
    _ok(capi, blit.synchronize(), "synchronize")
    assert bool((dst == GUARD_BYTE).all())
    inv = capi.ERROR_INVALID_ARGUMENT
    assert blit.copy_batch_bounded_noalloc(dev.data_ptr(), 10, 0) == inv
    assert blit.copy_batch_bounded_noalloc(None, 10, 4096) == inv
    assert blit.copy_batch_bounded_noalloc(dev.data_ptr(), 10, 1 << 62) == inv
    assert blit.copy_batch_bounded_noalloc(None, 0, 0) == capi.SUCCESS
    _ok(capi, blit.synchronize(), "synchronize")
    assert bool((dst == GUARD_BYTE).all())


def test_noalloc_batch_beyond_the_record_capacity(capi, hip_blit, torch_cuda):
    """More 4 KiB chunks than the scratch has records for (2^19): the rest are
    found through the prefix sums.  2.3 GiB in 5 copies; compared on the device
    with what the existing entry point leaves and with the source itself."""
    torch = torch_cuda
    blit = hip_blit
    n = 5
    each = 470 * MIB + 12345
    stride = (each + 4095) // 4096 * 4096 + 4096
    room = n * stride + 4096
    assert n * (each // 4096) > (1 << 19)
    _s, src = _device_bytes(torch, room)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(0xB1170A03)
    src.view(torch.int32)[:] = torch.randint(-2 ** 31, 2 ** 31 - 1, (room // 4,), dtype=torch.int32,
                                             device="cuda:0", generator=g)
    _a, dst_a = _device_bytes(torch, room)
    _b, dst_b = _device_bytes(torch, room)
    descs_a, descs_b = (capi.Desc * n)(), (capi.Desc * n)()
    at = []
    for i in range(n):
        s_off, d_off = i * stride + 256 + 3 * i, i * stride + 256 + 7 * i + 1
        at.append((s_off, d_off))
        for descs, dst in ((descs_a, dst_a), (descs_b, dst_b)):
            descs[i].dst = dst.data_ptr() + d_off
            descs[i].src = src.data_ptr() + s_off
            descs[i].bytes = each
    dev_a, dev_b = _to_device(torch, descs_a), _to_device(torch, descs_b)
    dst_a.fill_(GUARD_BYTE)
    dst_b.fill_(GUARD_BYTE)
    torch.cuda.synchronize()
    _ok(capi, blit.copy_batch_bounded_noalloc(dev_a.data_ptr(), n, n * each), "noalloc")
    _ok(capi, blit.copy_batch_bounded(dev_b.data_ptr(), n, n * each), "copy_batch_bounded")
    _ok(capi, blit.synchronize(), "synchronize")
    assert torch.equal(dst_a, dst_b)
    for s_off, d_off in at:
        assert torch.equal(dst_a[d_off:d_off + each], src[s_off:s_off + each])
        assert bool((dst_a[d_off - 256:d_off] == GUARD_BYTE).all())
        assert bool((dst_a[d_off + each:d_off + each + 256] == GUARD_BYTE).all())
