"""Copy, fill and region copy of the HIP-stream path recorded into a HIP graph:
each is one kernel launch with its arguments by value and no allocation, so a
captured sequence must replay exactly; so must the allocation-free batched
copy, whose four launches take their scratch memory from a static array.  The
graph is replayed several times with the program's own eager work and
synchronisations in between, new source bytes before every replay, and every
replay is checked against the CPU oracle."""
import numpy as np
import pytest

from conftest import oracle_rect

pytestmark = pytest.mark.gpu

GUARD_BYTE = 0xEE
FILL_VALUE = 0x0BADC0DE


def test_captured_commands_replay_exactly(capi, oracle, rand, torch_cuda):
    torch = torch_cuda
    n, s_off, d_off = 3 * (1 << 20) + 77, 3, 9
    rows, width, s_pitch, d_pitch = 300, 1501, 1777, 2049
    fill_dwords = 100_003
    src = torch.empty(n + 64, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty(n + 600, dtype=torch.uint8, device="cuda:0")
    rsrc = torch.empty(rows * s_pitch, dtype=torch.uint8, device="cuda:0")
    rdst = torch.empty(rows * d_pitch, dtype=torch.uint8, device="cuda:0")
    fbuf = torch.empty(4 * fill_dwords + 512, dtype=torch.uint8, device="cuda:0")
    f_at = (-fbuf.data_ptr()) % 4 + 256
    with capi.Blit(0) as blit:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            assert blit.copy(dst.data_ptr() + 256 + d_off, src.data_ptr() + s_off, n, s) == capi.SUCCESS
            assert blit.fill32(fbuf.data_ptr() + f_at, FILL_VALUE, fill_dwords, s) == capi.SUCCESS
            assert blit.copy_rect((rdst.data_ptr(), d_pitch, 0), (5, 0, 0), (rsrc.data_ptr(), s_pitch, 0), (7, 0, 0),
                                  (width, rows, 1), s) == capi.SUCCESS
        # nothing ran and nothing is pending because of the capture
        assert blit.pending_bytes() == 0
        for replay in range(4):
            src_h = rand(n + 64, 0x6EA90000 + replay)
            rsrc_h = rand(rows * s_pitch, 0x6EA91000 + replay)
            src.copy_(torch.from_numpy(src_h))
            rsrc.copy_(torch.from_numpy(rsrc_h))
            dst.fill_(GUARD_BYTE)
            rdst.fill_(GUARD_BYTE)
            fbuf.fill_(GUARD_BYTE)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            want = np.full(n + 600, GUARD_BYTE, dtype=np.uint8)
            oracle.oracle_copy(want.ctypes.data + 256 + d_off, src_h.ctypes.data + s_off, n)
            assert np.array_equal(dst.cpu().numpy(), want), "copy, replay %d" % replay
            want = np.full(4 * fill_dwords + 512, GUARD_BYTE, dtype=np.uint8)
            oracle.oracle_fill32(want.ctypes.data + f_at, FILL_VALUE, fill_dwords)
            assert np.array_equal(fbuf.cpu().numpy(), want), "fill, replay %d" % replay
            want = np.full(rows * d_pitch, GUARD_BYTE, dtype=np.uint8)
            oracle_rect(oracle, (want.ctypes.data, d_pitch, 0), (5, 0, 0), (rsrc_h.ctypes.data, s_pitch, 0), (7, 0, 0),
                        (width, rows, 1))
            assert np.array_equal(rdst.cpu().numpy(), want), "region copy, replay %d" % replay
            # an eager command between replays, on the engine's own stream
            assert blit.copy(dst.data_ptr(), src.data_ptr(), 4096) == capi.SUCCESS
            assert blit.synchronize() == capi.SUCCESS
        del graph


def test_batches_refuse_a_capturing_stream(capi, torch_cuda):
    """The batched copy stages descriptors and orders batches with events, so it
    cannot be recorded into a graph: it must say so instead of recording half of
    itself.  Nothing is launched by the refused calls."""
    torch = torch_cuda
    src = torch.arange(8192, dtype=torch.uint8, device="cuda:0")
    dst = torch.zeros(8192, dtype=torch.uint8, device="cuda:0")
    descs = (capi.Desc * 2)()
    for i in range(2):
        descs[i].dst, descs[i].src, descs[i].bytes = dst.data_ptr() + 4096 * i, src.data_ptr() + 4096 * i, 4000
    dev = torch.from_numpy(np.frombuffer(bytes(descs), dtype=np.uint8).copy()).to("cuda:0")
    with capi.Blit(0) as blit:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            assert blit.copy_batch(descs, 2, False, s) == capi.ERROR_INVALID_ARGUMENT
            assert blit.copy_batch(dev.data_ptr(), 2, True, s) == capi.ERROR_INVALID_ARGUMENT
            assert blit.copy_batch_bounded(dev.data_ptr(), 2, 8000, s) == capi.ERROR_INVALID_ARGUMENT
            assert blit.copy(dst.data_ptr(), src.data_ptr(), 64, s) == capi.SUCCESS
        graph.replay()
        torch.cuda.synchronize()
        assert int(dst[:64].sum()) == sum(range(64)) and int(dst[64:].sum()) == 0
        # the same batch outside a capture goes through
        assert blit.copy_batch(descs, 2, False, None) == capi.SUCCESS
        assert blit.synchronize() == capi.SUCCESS
        assert torch.equal(dst[:4000], src[:4000]) and torch.equal(dst[4096:8096], src[4096:8096])
        del graph


def test_allocation_free_batch_replays_with_new_descriptors(capi, oracle, rand, torch_cuda):
    """mi355_blit_copy_batch_bounded_noalloc is the batched copy for callers
    that cannot allocate, a capturing stream among them: recorded once, the
    graph reads the device-resident descriptors anew at every replay.  Four
    replays with different descriptors and source bytes each, eager work on the
    engine in between, every replay against the oracle."""
    torch = torch_cuda
    n, room = 700, 24 << 20
    src = torch.empty(room, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty(room, dtype=torch.uint8, device="cuda:0")
    dev = torch.zeros(n * 24, dtype=torch.uint8, device="cuda:0")
    bound = 20 << 20
    with capi.Blit(0) as blit:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            assert blit.copy_batch_bounded_noalloc(dev.data_ptr(), n, bound, s) == capi.SUCCESS
        assert blit.pending_bytes() == 0
        for replay in range(4):
            rng = np.random.default_rng(0x6EA92000 + replay)
            src_h = rand(room, 0x6EA93000 + replay)
            lens = np.floor(2.0 ** (17 * rng.random(n))).astype(np.int64)     # 1 B .. 128 KiB
            lens[rng.integers(0, n, 20)] = 0
            stride = ((lens + 255) // 256) * 256 + 512
            offs = np.concatenate([[0], np.cumsum(stride)[:-1]]) + 256
            assert int(offs[-1] + stride[-1]) <= room and int(lens.sum()) <= bound
            so, do = rng.integers(0, 16, n), rng.integers(0, 256, n)
            descs = (capi.Desc * n)()
            want = np.full(room, GUARD_BYTE, dtype=np.uint8)
            for i in range(n):
                descs[i].dst = dst.data_ptr() + int(offs[i] + do[i])
                descs[i].src = src.data_ptr() + int(offs[i] + so[i])
                descs[i].bytes = int(lens[i])
                oracle.oracle_copy(want.ctypes.data + int(offs[i] + do[i]), src_h.ctypes.data + int(offs[i] + so[i]),
                                   int(lens[i]))
            dev.copy_(torch.from_numpy(np.frombuffer(bytes(descs), dtype=np.uint8).copy()))
            src.copy_(torch.from_numpy(src_h))
            dst.fill_(GUARD_BYTE)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(dst.cpu().numpy(), want), "replay %d" % replay
            # eager work between replays: a batch through the allocating entry point and a copy
            assert blit.copy_batch(descs, n) == capi.SUCCESS
            assert blit.copy(dst.data_ptr(), src.data_ptr(), 4096) == capi.SUCCESS
            assert blit.synchronize() == capi.SUCCESS
        del graph
