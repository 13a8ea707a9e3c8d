"""The stand-ins for hsa_memory_copy, hsa_amd_memory_fill and
hsa_amd_memory_async_copy (include/mi355_blit_aql.h, csrc/aql_runtime.cpp):
same answers at the API edge as the reference (hsa.cpp:1170-1184,
hsa_ext_amd.cpp:237-294) and the same routing by pointer ownership as
Runtime::CopyMemory / FillMemory (runtime.cpp:469-664), bytes checked against
the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD = 256
MIB = 1 << 20


@pytest.fixture(scope="module")
def eng(pkg, torch_cuda):
    e = pkg.aql.AqlBlit(0)
    yield e
    e.close()


@pytest.fixture(scope="module")
def signals(pkg, torch_cuda):
    return pkg.aql.HsaSignals()


def _host(n, fill=0xEE):
    return np.full(n, fill, dtype=np.uint8)


@pytest.mark.parametrize("n", [1, 17, 4099, MIB + 3, 9 * MIB + 1])
def test_memory_copy_all_directions(eng, oracle, rand, torch_cuda, n):
    """host->device (unregistered host memory is locked for the GPU), device->device,
    device->host, host->host: one seeded payload goes round and must come back intact."""
    torch = torch_cuda
    payload = rand(n + 16, 0xB1170001)
    dev_a = torch.full((n + 2 * GUARD + 16,), 0xEE, dtype=torch.uint8, device="cuda:0")
    dev_b = torch.full((n + 2 * GUARD + 16,), 0xEE, dtype=torch.uint8, device="cuda:0")
    back = _host(n + 2 * GUARD + 16)
    final = _host(n + 2 * GUARD + 16)
    torch.cuda.synchronize()
    ok = eng.lib.mi355_hsa_memory_copy
    # host (numpy, unknown to the runtime) -> device, odd offsets
    assert ok(eng.handle, dev_a.data_ptr() + GUARD + 3, payload.ctypes.data + 5, n) == 0
    # device -> device
    assert ok(eng.handle, dev_b.data_ptr() + GUARD + 9, dev_a.data_ptr() + GUARD + 3, n) == 0
    # device -> host
    assert ok(eng.handle, back.ctypes.data + GUARD + 1, dev_b.data_ptr() + GUARD + 9, n) == 0
    # host -> host (plain memcpy on the calling thread)
    assert ok(eng.handle, final.ctypes.data + GUARD + 2, back.ctypes.data + GUARD + 1, n) == 0
    want_a = _host(n + 2 * GUARD + 16)
    oracle.oracle_copy(want_a.ctypes.data + GUARD + 3, payload.ctypes.data + 5, n)
    assert np.array_equal(dev_a.cpu().numpy(), want_a)
    want_b = _host(n + 2 * GUARD + 16)
    oracle.oracle_copy(want_b.ctypes.data + GUARD + 9, payload.ctypes.data + 5, n)
    assert np.array_equal(dev_b.cpu().numpy(), want_b)
    want_back = _host(n + 2 * GUARD + 16)
    oracle.oracle_copy(want_back.ctypes.data + GUARD + 1, payload.ctypes.data + 5, n)
    assert np.array_equal(back, want_back)
    want_final = _host(n + 2 * GUARD + 16)
    oracle.oracle_copy(want_final.ctypes.data + GUARD + 2, payload.ctypes.data + 5, n)
    assert np.array_equal(final, want_final)


def test_memory_copy_host_to_host_256_mib(eng, oracle, rand):
    """The reference's own CPU-runnable configuration: 256 MiB of seeded bytes,
    source and destination 64-byte aligned host memory, through the
    hsa_memory_copy stand-in (one memcpy on the calling thread,
    runtime.cpp:507-510); every byte and the guards against the oracle."""
    n = 256 * MIB
    raw_src, raw_dst = rand(n + 64, 0xB1170000), _host(n + 2 * GUARD + 64)
    s_off = (-raw_src.ctypes.data) % 64
    d_off = (-raw_dst.ctypes.data) % 64 + GUARD
    assert (raw_src.ctypes.data + s_off) % 64 == 0 and (raw_dst.ctypes.data + d_off) % 64 == 0
    assert eng.hsa_memory_copy(raw_dst.ctypes.data + d_off, raw_src.ctypes.data + s_off, n) == 0
    want = _host(n + 2 * GUARD + 64)
    oracle.oracle_copy(want.ctypes.data + d_off, raw_src.ctypes.data + s_off, n)
    assert np.array_equal(raw_dst, want)


def test_blocking_forms_and_bounded_wait(eng, oracle, rand, signals, torch_cuda):
    """The blocking copy and fill (their own completion signal, armed and waited
    for under the engine's blocking-call lock, amd_blit_kernel.cpp:614-639,
    787-837) and mi355_aql_wait_signal on a command parked behind a dependency
    that is satisfied later."""
    torch = torch_cuda
    n = MIB + 5
    payload = rand(n, 0xB1170007)
    src = torch.from_numpy(payload).to("cuda:0")
    parked = torch.full((n,), 0xEE, dtype=torch.uint8, device="cuda:0")
    dst = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    assert eng.copy_sync(dst.data_ptr() + GUARD, src.data_ptr(), n) == 0
    assert eng.fill32_sync(dst.data_ptr() + GUARD, 0x01020304, 16) == 0
    assert eng.copy_sync(dst.data_ptr() + GUARD + 64, src.data_ptr() + 64, 1000) == 0
    assert eng.copy_sync(dst.data_ptr(), src.data_ptr(), 0) == 0          # nothing to move: still completes
    assert eng.fill32_sync(dst.data_ptr(), 7, 0) == 0
    assert eng.copy_sync(None, src.data_ptr(), 8) == 0x1001
    assert eng.fill32_sync(dst.data_ptr() + 2, 7, 4) == 0x1001
    want = _host(n + 2 * GUARD)
    oracle.oracle_copy(want.ctypes.data + GUARD, payload.ctypes.data, n)
    oracle.oracle_fill32(want.ctypes.data + GUARD, 0x01020304, 16)
    oracle.oracle_copy(want.ctypes.data + GUARD + 64, payload.ctypes.data + 64, 1000)
    assert np.array_equal(dst.cpu().numpy(), want)
    dep, done = signals.create(1), signals.create(1)
    assert eng.copy(parked.data_ptr(), src.data_ptr(), n, deps=[dep], completion=done) == 0
    assert signals.load(done) == 1
    signals.store(dep, 0)
    assert eng.wait_signal(done) == 0
    assert np.array_equal(parked.cpu().numpy(), payload)
    signals.destroy(dep)
    signals.destroy(done)


def test_async_copy_reports_the_reference_engine(eng, pkg, signals, torch_cuda, monkeypatch):
    """Which engine GetBlitObject would have picked (amd_gpu_agent.cpp:2379-2398)
    is reported beside the launch: SDMA below HSA_FORCE_SDMA_SIZE, the blit
    kernel from there on, SDMA across the host link."""
    torch = torch_cuda
    capi = pkg.capi
    a = torch.zeros(4 * MIB, dtype=torch.uint8, device="cuda:0")
    b = torch.zeros(4 * MIB, dtype=torch.uint8, device="cuda:0")
    pinned = torch.zeros(4 * MIB, dtype=torch.uint8, pin_memory=True)
    torch.cuda.synchronize()
    done = signals.create(1)

    def engine_of(dst, src, n):
        signals.store(done, 1)
        assert eng.hsa_amd_memory_async_copy(dst, src, n, completion=done) == 0
        assert eng.wait_signal(done) == 0
        return eng.last_plan().reference_engine

    monkeypatch.delenv("HSA_FORCE_SDMA_SIZE", raising=False)
    assert engine_of(b.data_ptr(), a.data_ptr(), 4096) == capi.ENGINE_SDMA
    assert engine_of(b.data_ptr(), a.data_ptr(), MIB - 1) == capi.ENGINE_SDMA
    assert engine_of(b.data_ptr(), a.data_ptr(), MIB) == capi.ENGINE_BLIT_KERNEL
    assert engine_of(b.data_ptr(), pinned.data_ptr(), 2 * MIB) == capi.ENGINE_SDMA
    monkeypatch.setenv("HSA_FORCE_SDMA_SIZE", str(128 << 10))
    assert engine_of(b.data_ptr(), a.data_ptr(), (128 << 10) - 1) == capi.ENGINE_SDMA
    assert engine_of(b.data_ptr(), a.data_ptr(), 128 << 10) == capi.ENGINE_BLIT_KERNEL
    monkeypatch.setenv("HSA_FORCE_SDMA_SIZE", "0")
    assert engine_of(b.data_ptr(), a.data_ptr(), 1) == capi.ENGINE_BLIT_KERNEL
    signals.destroy(done)


def test_packet_log(pkg, signals, torch_cuda, monkeypatch, capfd):
    """MI355_BLIT_LOG_PKTS=1: one line per barrier and dispatch packet with the
    fields the reference logs (amd_blit_kernel.cpp:681-702, 903-923)."""
    import re
    torch = torch_cuda
    a = torch.zeros(MIB, dtype=torch.uint8, device="cuda:0")
    b = torch.zeros(MIB, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    monkeypatch.setenv("MI355_BLIT_LOG_PKTS", "1")
    e = pkg.aql.AqlBlit(0)
    try:
        dep, done = signals.create(0), signals.create(1)
        capfd.readouterr()
        assert e.copy(b.data_ptr(), a.data_ptr(), MIB, deps=[dep], completion=done) == 0
        assert e.wait_signal(done) == 0
        err = capfd.readouterr().err
        signals.destroy(dep)
        signals.destroy(done)
    finally:
        e.close()
    barrier = re.search(r"HWq=0x[0-9a-f]+, id=\d+, Barrier Header = 0x[0-9a-f]+ \(type=3, barrier=0, acquire=0, release=0\), "
                        r"dep_signal=\[0x%x 0x0 0x0 0x0 0x0\], completion_signal=0x0 rptr=\d+, wptr=(\d+)" % dep, err)
    assert barrier, err
    dispatch = re.search(r"Dispatch Header = 0x[0-9a-f]+ \(type=2, barrier=1, acquire=2, release=2\), setup=1, "
                         r"grid=\[(\d+), 1, 1\], workgroup=\[(\d+), 1, 1\], private_seg_size=0, group_seg_size=0, "
                         r"kernel_obj=0x[0-9a-f]+, kernarg_address=0x[0-9a-f]+, completion_signal=0x%x rptr=\d+, wptr=(\d+)"
                         % done, err)
    assert dispatch, err
    assert int(dispatch.group(3)) == int(barrier.group(1)) + 1
    assert int(dispatch.group(1)) % int(dispatch.group(2)) == 0


def test_barrier_bit_of_large_transfers(pkg, signals, torch_cuda, monkeypatch, capfd):
    """Without dependencies a blit's dispatch packet has the barrier bit clear, as
    the reference's has (amd_blit_kernel.cpp:870-882) -- except transfers of
    4 MiB and more on an engine's own queue, which wait for the queue to drain.
    An engine on a borrowed queue keeps the reference's packets; either default
    can be changed."""
    import re
    torch = torch_cuda
    n = 8 * MIB
    a = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    b = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    monkeypatch.setenv("MI355_BLIT_LOG_PKTS", "1")

    def barrier_bits(engine):
        """barrier bit of the dispatch packets of a 64 KiB copy, an 8 MiB copy and an 8 MiB fill"""
        out = []
        for submit in (lambda c: engine.copy(b.data_ptr(), a.data_ptr(), 65536, completion=c),
                       lambda c: engine.copy(b.data_ptr(), a.data_ptr(), n, completion=c),
                       lambda c: engine.fill32(b.data_ptr(), 7, n // 4, completion=c)):
            done = signals.create(1)
            capfd.readouterr()
            assert submit(done) == 0
            assert engine.wait_signal(done) == 0
            m = re.search(r"Dispatch Header = 0x[0-9a-f]+ \(type=2, barrier=(\d)", capfd.readouterr().err)
            signals.destroy(done)
            assert m
            out.append(int(m.group(1)))
        return out

    own = pkg.aql.AqlBlit(0)
    queue = pkg.aql.BorrowedQueue(0)
    try:
        assert barrier_bits(own) == [0, 1, 1]
        assert own.set_large_transfer_barrier(False) == 0
        assert barrier_bits(own) == [0, 0, 0]
        borrowed = pkg.aql.AqlBlit(borrowed=queue)
        try:
            assert barrier_bits(borrowed) == [0, 0, 0]
            assert borrowed.set_large_transfer_barrier(True) == 0
            assert barrier_bits(borrowed) == [0, 1, 1]
        finally:
            borrowed.close()
    finally:
        own.close()
        queue.close()


def test_long_copies_go_out_in_pieces_except_where_they_must_not(pkg, signals, torch_cuda):
    """A copy of 1.5 GiB or more within the device is several dispatches on an
    engine's own queue (the completion signal on the last), one on a borrowed
    queue unless asked otherwise, and one while the queue's profiling is on, so
    that the stamps in the completion signal cover the whole command."""
    torch = torch_cuda
    n = 2 << 30
    a = torch.empty(n + 64, dtype=torch.uint8, device="cuda:0")
    b = torch.zeros(n + 64, dtype=torch.uint8, device="cuda:0")
    a.view(torch.int32)[:n // 4].copy_(torch.arange(n // 4, dtype=torch.int32, device="cuda:0"))
    torch.cuda.synchronize()

    def run(engine, want_pieces):
        b.zero_()
        torch.cuda.synchronize()
        done = signals.create(1)
        assert engine.copy(b.data_ptr() + 5, a.data_ptr() + 1, n - 16, completion=done) == 0
        assert engine.wait_signal(done) == 0
        assert signals.load(done) == 0
        # the signal says the whole copy is done, not a piece of it
        assert torch.equal(b[5:5 + n - 16], a[1:1 + n - 16])
        assert engine.last_plan().pieces == want_pieces
        return done

    own = pkg.aql.AqlBlit(0)
    queue = pkg.aql.BorrowedQueue(0)
    try:
        signals.destroy(run(own, 4))
        assert own.enable_profiling(True) == 0
        done = run(own, 1)
        us = own.command_time_us(done)
        signals.destroy(done)
        assert 500.0 < us < 1500.0, us        # 2 GiB at 6-7 TB/s is 620-720 us: the whole command, not a quarter
        assert own.enable_profiling(False) == 0
        signals.destroy(run(own, 4))
        borrowed = pkg.aql.AqlBlit(borrowed=queue)
        try:
            signals.destroy(run(borrowed, 1))
            assert borrowed.set_large_transfer_barrier(True) == 0
            signals.destroy(run(borrowed, 4))
        finally:
            borrowed.close()
    finally:
        own.close()
        queue.close()


def test_kernarg_ring_in_host_memory(pkg, capi, oracle, rand, torch_cuda, monkeypatch):
    """MI355_BLIT_HOST_KERNARGS=1 keeps every kernarg slot in host memory, as the
    reference does (amd_blit_kernel.cpp:565-569): a small copy, a copy of many
    workgroups, a fill and a batch against the oracle."""
    torch = torch_cuda
    monkeypatch.setenv("MI355_BLIT_HOST_KERNARGS", "1")
    e = pkg.aql.AqlBlit(0)
    try:
        n = 24 * MIB + 13
        payload = rand(n + 64, 0xB1170009)
        src = torch.from_numpy(payload).to("cuda:0")
        dst = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        for size, s_off, d_off in ((4099, 3, 9), (n, 5, 2)):
            dst.fill_(0xEE)
            torch.cuda.synchronize()
            assert e.copy(dst.data_ptr() + GUARD + d_off, src.data_ptr() + s_off, size) == 0
            assert e.synchronize() == 0
            want = _host(n + 2 * GUARD)
            oracle.oracle_copy(want.ctypes.data + GUARD + d_off, payload.ctypes.data + s_off, size)
            assert np.array_equal(dst.cpu().numpy(), want), size
        dst.fill_(0xEE)
        torch.cuda.synchronize()
        assert e.fill32(dst.data_ptr() + GUARD + 4, 0xabcdef12, (n - 8) // 4) == 0
        assert e.synchronize() == 0
        want = _host(n + 2 * GUARD)
        oracle.oracle_fill32(want.ctypes.data + GUARD + 4, 0xabcdef12, (n - 8) // 4)
        assert np.array_equal(dst.cpu().numpy(), want)
        # a batch: 300 copies of 1 .. 200,000 bytes at byte offsets
        rng = np.random.default_rng(99)
        m = 300
        descs = (capi.Desc * m)()
        dst.fill_(0xEE)
        torch.cuda.synchronize()
        want = _host(n + 2 * GUARD)
        at = GUARD
        for i in range(m):
            ln = int(rng.integers(1, 80000))
            so, do = int(rng.integers(0, 16)), int(rng.integers(0, 16))
            descs[i].dst = dst.data_ptr() + at + do
            descs[i].src = src.data_ptr() + at + so
            descs[i].bytes = ln
            oracle.oracle_copy(want.ctypes.data + at + do, payload.ctypes.data + at + so, ln)
            at += (ln + 15 + 255) // 256 * 256 + 256
        assert at < n
        assert e.copy_batch(descs, m) == 0
        assert e.synchronize() == 0
        assert np.array_equal(dst.cpu().numpy(), want)
    finally:
        e.close()


def test_memory_copy_pinned_host(eng, oracle, rand, torch_cuda):
    """Host memory allocated through the runtime (pinned) needs no locking."""
    torch = torch_cuda
    n = 3 * MIB + 7
    pinned = torch.empty(n + 64, dtype=torch.uint8, pin_memory=True)
    payload = rand(n + 64, 0xB1170002)
    pinned.numpy()[:] = payload
    dev = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    assert eng.hsa_memory_copy(dev.data_ptr() + GUARD, pinned.data_ptr() + 1, n) == 0
    want = _host(n + 2 * GUARD)
    oracle.oracle_copy(want.ctypes.data + GUARD, payload.ctypes.data + 1, n)
    assert np.array_equal(dev.cpu().numpy(), want)
    out = torch.full((n + 64,), 0xEE, dtype=torch.uint8).pin_memory()
    assert eng.hsa_memory_copy(out.data_ptr() + 2, dev.data_ptr() + GUARD, n) == 0
    assert np.array_equal(out.numpy()[2:2 + n], payload[1:1 + n]) and out.numpy()[0] == 0xEE


@pytest.mark.parametrize("n,s_off,d_off", [(1, 0, 0), (4099, 3, 9), (MIB + 3, 5, 0), (5 * MIB + 77, 0, 4),
                                          (40 * MIB + 1, 13, 6)])
def test_copies_across_the_host_link_are_exact(eng, capi, oracle, rand, torch_cuda, n, s_off, d_off):
    """Host to device and device to host on the routes made for the link (pinned
    host memory, both submission paths): the launch is the link's shape, the bytes
    are the oracle's and the guard bytes stay."""
    torch = torch_cuda
    h2d, d2h = capi.ROUTE_HOST_TO_DEVICE, capi.ROUTE_DEVICE_TO_HOST
    payload = rand(n + 64, 0xB1170021)
    pinned = torch.empty(n + 64, dtype=torch.uint8, pin_memory=True)
    pinned.numpy()[:] = payload
    want_dev = _host(n + 2 * GUARD)
    oracle.oracle_copy(want_dev.ctypes.data + GUARD + d_off, payload.ctypes.data + s_off, n)
    want_out = _host(n + 2 * GUARD)
    oracle.oracle_copy(want_out.ctypes.data + GUARD + s_off, want_dev.ctypes.data + GUARD + d_off, n)
    with capi.Blit(0) as blit:
        for path in ("aql", "hip"):
            dev = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
            out = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8).pin_memory()
            torch.cuda.synchronize()
            for route, dst, src in ((h2d, dev.data_ptr() + GUARD + d_off, pinned.data_ptr() + s_off),
                                    (d2h, out.data_ptr() + GUARD + s_off, dev.data_ptr() + GUARD + d_off)):
                if path == "aql":
                    assert eng.copy(dst, src, n, route=route) == 0
                    assert eng.synchronize() == 0
                    p = eng.last_plan()
                else:
                    assert blit.copy(dst, src, n, route=route) == 0
                    assert blit.synchronize() == 0
                    p = blit.last_plan()
                assert p.route == route and p.wg_size == 256 and p.grid <= 128 and p.xcd_run == 0
                assert p.byte_shift == ((s_off - d_off) & 3 if route == h2d else (d_off - s_off) & 3)
            assert np.array_equal(dev.cpu().numpy(), want_dev), path
            assert np.array_equal(out.numpy(), want_out), path
    assert eng.copy(dev.data_ptr(), pinned.data_ptr(), 16, route=3) == capi.ERROR_INVALID_ARGUMENT


def test_caller_policy_takes_the_route_the_placements_give(eng, signals, capi, rand, torch_cuda):
    """hsa_memory_copy classifies both pointers anyway and routes every size; the
    asynchronous copy has no agents in its signature and looks the pointers up
    from 1 MiB on, where the launch shape starts to depend on the route."""
    torch = torch_cuda
    n = 2 * MIB
    pinned = torch.empty(n, dtype=torch.uint8, pin_memory=True)
    pinned.numpy()[:] = rand(n, 0xB1170022)
    dev = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    dev2 = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    assert eng.hsa_memory_copy(dev.data_ptr(), pinned.data_ptr(), n) == 0
    assert eng.last_plan().route == capi.ROUTE_HOST_TO_DEVICE
    assert eng.hsa_memory_copy(pinned.data_ptr(), dev.data_ptr(), 4096) == 0
    assert eng.last_plan().route == capi.ROUTE_DEVICE_TO_HOST
    assert eng.hsa_memory_copy(dev2.data_ptr(), dev.data_ptr(), n) == 0
    assert eng.last_plan().route == capi.ROUTE_DEVICE
    done = signals.create(1)
    for dst, src, size, route in ((dev2.data_ptr(), pinned.data_ptr(), n, capi.ROUTE_HOST_TO_DEVICE),
                                  (pinned.data_ptr(), dev.data_ptr(), n, capi.ROUTE_DEVICE_TO_HOST),
                                  (dev2.data_ptr(), dev.data_ptr(), n, capi.ROUTE_DEVICE),
                                  (dev2.data_ptr(), pinned.data_ptr(), n // 4, capi.ROUTE_DEVICE)):
        signals.store(done, 1)
        assert eng.hsa_amd_memory_async_copy(dst, src, size, None, done) == 0
        signals.wait_below_one(done)
        assert eng.last_plan().route == route
    signals.destroy(done)
    assert torch.equal(dev2.cpu(), pinned) and torch.equal(dev.cpu(), pinned)


def test_memory_copy_api_edge(eng, torch_cuda):
    """hsa.cpp:1174-1180"""
    torch = torch_cuda
    dev = torch.zeros(64, dtype=torch.uint8, device="cuda:0")
    inv = 0x1001
    assert eng.hsa_memory_copy(None, dev.data_ptr(), 8) == inv
    assert eng.hsa_memory_copy(dev.data_ptr(), None, 8) == inv
    assert eng.hsa_memory_copy(dev.data_ptr(), dev.data_ptr() + 32, 0) == 0


@pytest.mark.parametrize("value", [0xabcdef12, 0xA5C30F1E])
def test_memory_fill_device_and_host(eng, oracle, torch_cuda, value):
    """Device memory goes to the blit; plain host memory is filled on the host
    with the whole 32-bit pattern (the reference's memset there truncates it)."""
    torch = torch_cuda
    count = MIB // 4 + 3
    dev = torch.full((4 * count + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    off = GUARD + (-(dev.data_ptr() + GUARD)) % 4
    assert eng.hsa_amd_memory_fill(dev.data_ptr() + off, value, count) == 0
    want = _host(4 * count + 2 * GUARD)
    oracle.oracle_fill32(want.ctypes.data + off, value, count)
    assert np.array_equal(dev.cpu().numpy(), want)
    host = _host(4 * count + 2 * GUARD)
    hoff = GUARD + (-(host.ctypes.data + GUARD)) % 4
    assert eng.hsa_amd_memory_fill(host.ctypes.data + hoff, value, count) == 0
    want = _host(4 * count + 2 * GUARD)
    oracle.oracle_fill32(want.ctypes.data + hoff, value, count)
    assert np.array_equal(host, want)
    # what the reference's host fallback would have left instead
    quirk = _host(4 * count + 2 * GUARD)
    oracle.oracle_ref_host_fill(quirk.ctypes.data + hoff, value, count)
    assert not np.array_equal(host, quirk)


def test_memory_fill_api_edge(eng, torch_cuda):
    """hsa_ext_amd.cpp:241-247"""
    torch = torch_cuda
    dev = torch.zeros(64, dtype=torch.uint8, device="cuda:0")
    base = dev.data_ptr() + (-dev.data_ptr()) % 4
    inv = 0x1001
    assert eng.hsa_amd_memory_fill(None, 1, 4) == inv
    for off in (1, 2, 3):
        assert eng.hsa_amd_memory_fill(base + off, 1, 4) == inv
    assert eng.hsa_amd_memory_fill(base, 1, 0) == 0
    torch.cuda.synchronize()
    assert not dev.cpu().numpy().any()


def test_async_copy_api_edge_and_completion(eng, signals, oracle, rand, torch_cuda):
    """hsa_ext_amd.cpp:253-294: argument checks, size 0 leaves the signal alone,
    a real copy decrements it once; dependencies hold the copy back."""
    torch = torch_cuda
    n = 2 * MIB + 5
    payload = rand(n, 0xB1170003)
    src = torch.from_numpy(payload).to("cuda:0")
    dst = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    inv = 0x1001
    done = signals.create(1)
    dep = signals.create(1)
    f = eng.lib.mi355_hsa_amd_memory_async_copy
    assert f(eng.handle, None, src.data_ptr(), n, 0, None, done) == inv
    assert f(eng.handle, dst.data_ptr(), None, n, 0, None, done) == inv
    assert f(eng.handle, dst.data_ptr(), src.data_ptr(), n, 1, None, done) == inv      # count without array
    one = (C.c_uint64 * 1)(dep)
    assert f(eng.handle, dst.data_ptr(), src.data_ptr(), n, 0, one, done) == inv       # array without count
    assert f(eng.handle, dst.data_ptr(), src.data_ptr(), n, 0, None, 0) == inv         # no completion signal
    assert f(eng.handle, dst.data_ptr(), src.data_ptr(), 0, 0, None, done) == 0
    assert signals.load(done) == 1                                                     # untouched
    # a copy behind an unsatisfied dependency
    assert f(eng.handle, dst.data_ptr() + GUARD, src.data_ptr(), n, 1, one, done) == 0
    import time
    time.sleep(0.05)
    assert signals.load(done) == 1
    torch.cuda.synchronize()
    assert bool((dst == 0xEE).all())
    signals.store(dep, 0)
    signals.wait_below_one(done, active=False)
    assert signals.load(done) == 0
    want = _host(n + 2 * GUARD)
    oracle.oracle_copy(want.ctypes.data + GUARD, payload.ctypes.data, n)
    assert np.array_equal(dst.cpu().numpy(), want)
    signals.destroy(done)
    signals.destroy(dep)


def _stock_agents():
    """(hsa library, GPU agent handles, CPU agent handles) of the runtime the process runs on."""
    hsa = C.CDLL("libhsa-runtime64.so.1")
    gpus, cpus = [], []
    CB = C.CFUNCTYPE(C.c_int, C.c_uint64, C.c_void_p)

    def visit(agent, _):
        dev = C.c_int(-1)
        hsa.hsa_agent_get_info(C.c_uint64(agent), 17, C.byref(dev))     # HSA_AGENT_INFO_DEVICE
        (gpus if dev.value == 1 else cpus).append(agent)                 # HSA_DEVICE_TYPE_GPU == 1
        return 0
    cb = CB(visit)
    hsa.hsa_agent_get_info.argtypes = [C.c_uint64, C.c_int, C.c_void_p]
    hsa.hsa_iterate_agents.argtypes = [CB, C.c_void_p]
    assert hsa.hsa_iterate_agents(cb, None) == 0
    return hsa, gpus, cpus


def test_copy_engine_status_matches_the_installed_runtime(eng, torch_cuda):
    """hsa_amd_memory_copy_engine_status (hsa_ext_amd.cpp:341-352, runtime.cpp:603-613,
    amd_gpu_agent.cpp:1181-1243): the same statuses and, with no copy in flight,
    the same mask of free engines as the runtime itself reports for this GPU."""
    torch_cuda.cuda.synchronize()
    inv_agent = 0x1004
    assert eng.hsa_amd_memory_copy_engine_status(True, True) == (inv_agent, 0)
    assert eng.hsa_amd_memory_copy_engine_status(False, False) == (inv_agent, 0)
    assert eng.lib.mi355_hsa_amd_memory_copy_engine_status(eng.handle, 1, 0, None) == 0x1001
    h2d = eng.hsa_amd_memory_copy_engine_status(True, False)
    d2h = eng.hsa_amd_memory_copy_engine_status(False, True)
    assert h2d == d2h
    try:
        hsa, gpus, cpus = _stock_agents()
        f = hsa.hsa_amd_memory_copy_engine_status
    except (OSError, AttributeError) as e:
        pytest.skip("no loadable libhsa-runtime64 with the entry point: %s" % e)
    f.argtypes = [C.c_uint64, C.c_uint64, C.POINTER(C.c_uint32)]
    gpu = eng.lib.mi355_aql_gpu_agent(eng.handle)
    assert gpu in gpus and cpus
    mask = C.c_uint32(0)
    st = f(gpu, cpus[0], C.byref(mask))                                   # destination GPU, source host
    assert (st, mask.value) == h2d
    st = f(cpus[0], gpu, C.byref(mask))
    assert (st, mask.value) == d2h
    assert f(gpu, gpu, C.byref(mask)) == inv_agent


def test_async_copy_on_engine(eng, signals, oracle, rand, torch_cuda):
    """hsa_amd_memory_async_copy_on_engine within the GPU (hsa_ext_amd.cpp:296-339,
    runtime.cpp:585-601, amd_gpu_agent.cpp:1110-1179): the engine must be one
    existing engine, and the copy then runs on the blit kernel all the same."""
    torch = torch_cuda
    n = MIB + 77
    payload = rand(n, 0xB1170009)
    src = torch.from_numpy(payload).to("cuda:0")
    dst = torch.full((n + 2 * GUARD,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    inv = 0x1001
    done = signals.create(1)
    st, free_mask = eng.hsa_amd_memory_copy_engine_status(True, False)
    assert st == 0 and free_mask & 1
    d, s = dst.data_ptr() + GUARD, src.data_ptr()
    f = eng.hsa_amd_memory_async_copy_on_engine
    assert f(None, s, n, 1, completion=done) == inv
    assert f(d, None, n, 1, completion=done) == inv
    assert f(d, s, n, 1, completion=0) == inv
    assert f(d, s, n, 0, completion=done) == inv                    # no engine named
    assert f(d, s, n, 3, completion=done) == inv                    # two engines named
    assert f(d, s, n, 1 << 31, completion=done) == inv              # an engine the GPU does not have
    assert f(d, s, 0, 3, completion=done) == 0                      # size 0 succeeds before the engine is looked at
    assert f(d, s, n, 1, force_copy_on_sdma=True, completion=done) == 0x1008   # no SDMA behind this library
    assert signals.load(done) == 1
    torch.cuda.synchronize()
    assert bool((dst == 0xEE).all())
    assert f(d, s, n, 1, completion=done) == 0
    signals.wait_below_one(done, active=False)
    want = _host(n + 2 * GUARD)
    oracle.oracle_copy(want.ctypes.data + GUARD, payload.ctypes.data, n)
    assert np.array_equal(dst.cpu().numpy(), want)
    signals.destroy(done)
