"""The installed ROCr beside this engine.  The HSA runtime the process already
runs on (libhsa-runtime64 of the ROCm image) is a binary build of the
reference: its hsa_memory_copy / hsa_amd_memory_fill on same-GPU device
pointers go through AMD::BlitKernel and the CopyAligned / CopyMisaligned / Fill
shaders (core/runtime/runtime.cpp:513, amd_gpu_agent.cpp:951, 1285).  Both are
given the same seeded inputs, misaligned offsets and odd lengths included
(cases no test of the reference holds a vector for), and must leave the same
bytes, which must also be the CPU oracle's."""
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
