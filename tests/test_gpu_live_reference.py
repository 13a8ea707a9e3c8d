"""The installed ROCr beside this engine.  The HSA runtime the process already
runs on (libhsa-runtime64 of the ROCm image) is a binary build of the
reference: its hsa_memory_copy / hsa_amd_memory_fill on same-GPU device
pointers go through AMD::BlitKernel and the CopyAligned / CopyMisaligned / Fill
shaders (core/runtime/runtime.cpp:513, amd_gpu_agent.cpp:951, 1285).  Both are
given the same seeded inputs, misaligned offsets and odd lengths included
(cases no test of the reference holds a vector for), and must leave the same
bytes, which must also be the CPU oracle's.  Its hsa_amd_memory_async_copy_rect
(SDMA engines) is the reference for the region copy in the same way."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD = 256
GUARD_BYTE = 0xEE
MIB = 1 << 20


@pytest.fixture(scope="module")
def stock(torch_cuda):
    """hsa_memory_copy / hsa_amd_memory_fill of the runtime torch loaded."""
    try:
        hsa = C.CDLL("libhsa-runtime64.so.1")
        hsa.hsa_init.restype = C.c_int
        hsa.hsa_shut_down.restype = C.c_int
        hsa.hsa_memory_copy.restype = C.c_int
        hsa.hsa_memory_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        hsa.hsa_amd_memory_fill.restype = C.c_int
        hsa.hsa_amd_memory_fill.argtypes = [C.c_void_p, C.c_uint32, C.c_size_t]
    except (OSError, AttributeError) as e:
        pytest.skip("no loadable libhsa-runtime64 beside the engine: %s" % e)
    if hsa.hsa_init() != 0:
        pytest.skip("hsa_init of the installed runtime failed")
    yield hsa
    hsa.hsa_shut_down()


def device_pair(torch, nbytes):
    a = torch.full((nbytes + 512,), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    b = torch.full((nbytes + 512,), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    return a, b, a.data_ptr() + (-a.data_ptr()) % 256, b.data_ptr() + (-b.data_ptr()) % 256


COPY_CASES = [
    # source offset, destination offset, bytes
    (0, 0, 4096), (0, 0, MIB), (0, 0, 16 * MIB + 4),
    (3, 9, 1), (3, 9, 15), (3, 9, 255), (3, 9, 4099), (3, 9, MIB + 17), (3, 9, 32 * MIB - 61),
    (1, 0, 70001), (0, 1, 70001), (2, 2, 70001), (7, 5, 262144 + 3), (5, 7, 1048576 + 1),
    (4, 8, 3 * MIB + 4), (12, 4, 3 * MIB + 2), (15, 15, 999), (255, 1, 5 * MIB + 13), (129, 130, 8 * MIB),
]


@pytest.mark.parametrize("s_off,d_off,n", COPY_CASES)
def test_copy_leaves_the_bytes_the_installed_runtime_leaves(capi, blit, stock, oracle, rand, torch_cuda,
                                                            s_off, d_off, n):
    torch = torch_cuda
    src_h = rand(n + 512, 0x11FE0000 + n % 65521)
    src = torch.from_numpy(src_h).to("cuda:0")
    sbase = src.data_ptr()
    ours, theirs, obase, tbase = device_pair(torch, n + 2 * GUARD + 256)
    torch.cuda.synchronize()
    assert stock.hsa_memory_copy(tbase + GUARD + d_off, sbase + s_off, n) == 0
    assert blit.copy(obase + GUARD + d_off, sbase + s_off, n) == capi.SUCCESS
    assert blit.synchronize() == capi.SUCCESS
    torch.cuda.synchronize()
    lo_o, lo_t = obase - ours.data_ptr(), tbase - theirs.data_ptr()
    span = n + 2 * GUARD + 256
    got = ours[lo_o:lo_o + span].cpu().numpy()
    ref = theirs[lo_t:lo_t + span].cpu().numpy()
    assert np.array_equal(got, ref), "differs from the installed runtime's copy"
    want = np.full(span, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_copy(want.ctypes.data + GUARD + d_off, src_h.ctypes.data + s_off, n)
    assert np.array_equal(ref, want), "the installed runtime's copy differs from the oracle"


@pytest.mark.parametrize("d_off,count,value", [
    (0, 1, 0xabcdef12), (4, 3, 0xba5eba11), (8, 1023, 0xfeed5a1e), (12, 65537, 0xbaadf00d),
    (0, 4 * MIB, 0xA5C30F1E), (252, 2 * MIB + 1, 0x01020304),
])
def test_fill_leaves_the_dwords_the_installed_runtime_leaves(capi, blit, stock, oracle, torch_cuda,
                                                             d_off, count, value):
    torch = torch_cuda
    n = 4 * count
    ours, theirs, obase, tbase = device_pair(torch, n + 2 * GUARD + 256)
    torch.cuda.synchronize()
    assert stock.hsa_amd_memory_fill(tbase + GUARD + d_off, value, count) == 0
    assert blit.fill32(obase + GUARD + d_off, value, count) == capi.SUCCESS
    assert blit.synchronize() == capi.SUCCESS
    torch.cuda.synchronize()
    lo_o, lo_t = obase - ours.data_ptr(), tbase - theirs.data_ptr()
    span = n + 2 * GUARD + 256
    got = ours[lo_o:lo_o + span].cpu().numpy()
    ref = theirs[lo_t:lo_t + span].cpu().numpy()
    assert np.array_equal(got, ref), "differs from the installed runtime's fill"
    want = np.full(span, GUARD_BYTE, dtype=np.uint8)
    oracle.oracle_fill32(want.ctypes.data + GUARD + d_off, value, count)
    assert np.array_equal(ref, want), "the installed runtime's fill differs from the oracle"


def test_api_edge_answers_match_the_installed_runtime(capi, blit, stock, torch_cuda):
    """NULL pointers, zero sizes and a misaligned fill pointer: same statuses."""
    torch = torch_cuda
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    p = buf.data_ptr()
    assert stock.hsa_memory_copy(None, p, 16) == blit.copy(None, p, 16) == capi.ERROR_INVALID_ARGUMENT
    assert stock.hsa_memory_copy(p, None, 16) == blit.copy(p, None, 16) == capi.ERROR_INVALID_ARGUMENT
    assert stock.hsa_memory_copy(p, p + 64, 0) == blit.copy(p, p + 64, 0) == capi.SUCCESS
    assert stock.hsa_amd_memory_fill(None, 1, 4) == blit.fill32(None, 1, 4) == capi.ERROR_INVALID_ARGUMENT
    assert stock.hsa_amd_memory_fill(p + 2, 1, 4) == blit.fill32(p + 2, 1, 4) == capi.ERROR_INVALID_ARGUMENT
    assert stock.hsa_amd_memory_fill(p, 1, 0) == blit.fill32(p, 1, 0) == capi.SUCCESS
    assert blit.synchronize() == capi.SUCCESS


RECT_CASES = [
    # source shape (layers, rows, pitch), destination shape, extent (x bytes, y, z), source offset, destination offset:
    # bases, pitches, offsets and widths multiples of 4, which is all the reference's SDMA packet accepts
    ((1, 16, 512), (1, 12, 1024), (256, 7, 1), (64, 2, 0), (128, 3, 0)),
    ((4, 9, 1032), (5, 11, 1500), (1000, 5, 3), (32, 4, 1), (496, 6, 2)),
    ((1, 64, 131072), (1, 64, 131072), (65536, 64, 1), (0, 0, 0), (65536, 0, 0)),
    ((3, 300, 516), (3, 310, 400), (332, 250, 3), (12, 20, 0), (4, 31, 0)),
    ((2, 40, 12000), (2, 37, 11004), (9000, 31, 2), (8, 3, 0), (1000, 2, 0)),
]


@pytest.mark.parametrize("case", range(len(RECT_CASES)))
def test_rect_copy_leaves_the_bytes_the_installed_runtime_leaves(capi, blit, oracle, rand, torch_cuda, pkg, case):
    """hsa_amd_memory_async_copy_rect of the installed runtime (SDMA engines:
    amd_gpu_agent.cpp:1255-1283, amd_blit_sdma.cpp:564-636) beside this engine's
    shader on the same seeded surfaces: both destination surfaces, everything
    outside the region included, must be equal, and equal to the oracle's.  The
    reference's tests hold no vector for region copies; this is the check
    against its own implementation."""
    from conftest import PitchedPtr, Dim3, oracle_rect
    torch = torch_cuda
    try:
        hsa = C.CDLL("libhsa-runtime64.so.1")
        f = hsa.hsa_amd_memory_async_copy_rect
    except (OSError, AttributeError) as e:
        pytest.skip("no loadable libhsa-runtime64 with the entry point: %s" % e)
    f.restype = C.c_int
    f.argtypes = [C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(PitchedPtr), C.POINTER(Dim3), C.POINTER(Dim3),
                  C.c_uint64, C.c_int, C.c_uint32, C.c_void_p, C.c_uint64]
    sshape, dshape, ext, so, do = RECT_CASES[case]
    src_h = rand(int(np.prod(sshape)), 0x11FE7000 + case)
    src = torch.from_numpy(src_h).to("cuda:0")
    ours = torch.full((int(np.prod(dshape)),), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    theirs = torch.full((int(np.prod(dshape)),), GUARD_BYTE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    assert src.data_ptr() % 4 == 0 and ours.data_ptr() % 4 == 0 and theirs.data_ptr() % 4 == 0
    sp = (src.data_ptr(), sshape[2], sshape[1] * sshape[2])
    signals = pkg.aql.HsaSignals()
    done = signals.create(1)
    # the GPU agent of the installed runtime: the one that owns the destination
    aql = pkg.aql.AqlBlit(0)
    gpu = aql.lib.mi355_aql_gpu_agent(aql.handle)
    aql.close()
    dp_t = (theirs.data_ptr(), dshape[2], dshape[1] * dshape[2])
    st = f(PitchedPtr(*dp_t), Dim3(*do), PitchedPtr(*sp), Dim3(*so), Dim3(*ext), gpu, 3, 0, None, done)
    if st != 0:
        signals.destroy(done)
        pytest.skip("the installed runtime has no engine for region copies here: status 0x%x" % st)
    signals.wait_below_one(done, active=False)
    signals.destroy(done)
    dp_o = (ours.data_ptr(), dshape[2], dshape[1] * dshape[2])
    assert blit.copy_rect(dp_o, do, sp, so, ext) == capi.SUCCESS
    assert blit.synchronize() == capi.SUCCESS
    torch.cuda.synchronize()
    got, ref = ours.cpu().numpy(), theirs.cpu().numpy()
    assert np.array_equal(got, ref), "differs from the installed runtime's region copy"
    want = np.full(got.size, GUARD_BYTE, dtype=np.uint8)
    oracle_rect(oracle, (want.ctypes.data,) + dp_o[1:], do, (src_h.ctypes.data,) + sp[1:], so, ext)
    assert np.array_equal(ref, want), "the installed runtime's region copy differs from the oracle"
