"""The C++ core::Blit adapter (rocm-systems_amd/csrc/rocr_blit.{h,cpp}).

CPU part: the adapter library and its native test driver are built, load, and
export the interface.  GPU part: the native driver
(tests/cpp/test_rocr_blit.cpp) runs every case against the CPU oracle; it is a
separate process because it drives the engine through HSA signals the way a
ROCr caller does."""
import os
import re
import subprocess

import pytest


def _paths(pkg):
    b = pkg.build
    return b.ROCR_LIB, b.ROCR_TEST


def test_adapter_is_built_and_exports_the_interface(pkg):
    lib, exe = _paths(pkg)
    assert os.path.exists(lib) and os.path.exists(exe), "run __graft_entry__.build() first"
    syms = subprocess.run(["nm", "-DC", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    for cls in ("BlitKernelGfx950", "BlitKernelGfx950Aql"):
        for member in ("Initialize(rocr::core::Agent const&)", "Destroy(rocr::core::Agent const&)",
                       "SubmitLinearCopyCommand(void*, void const*, unsigned long)",
                       "SubmitLinearFillCommand(void*, unsigned int, unsigned long)",
                       "SubmitBatchCopyCommand", "EnableProfiling(bool)", "PendingBytes()"):
            assert "rocr::AMD::%s::%s" % (cls, member) in syms, (cls, member)
    # the asynchronous overload with dependency, completion and gang signals
    assert re.search(r"BlitKernelGfx950::SubmitLinearCopyCommand\(void\*, void const\*, unsigned long, "
                     r"std::vector<rocr::core::Signal\*.*rocr::core::Signal&, std::vector<rocr::core::Signal\*", syms)


def test_adapter_interface_mirrors_reference_blit_h():
    """Every pure virtual of core::Blit (core/inc/blit.h:52-122) is declared with
    the same name and parameter list in the local restatement."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "rocm-systems_amd", "csrc", "rocr_blit.h")).read()
    blit = text[text.index("class Blit {"):text.index("}  // namespace core")]
    flat = re.sub(r"\s+", " ", blit)
    for decl in (
            "virtual hsa_status_t Destroy(const core::Agent& agent) = 0;",
            "virtual hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size) = 0;",
            "virtual hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size, "
            "std::vector<core::Signal*>& dep_signals, core::Signal& out_signal, "
            "std::vector<core::Signal*>& gang_signals) = 0;",
            "virtual hsa_status_t SubmitLinearFillCommand(void* ptr, uint32_t value, size_t num) = 0;",
            "virtual hsa_status_t EnableProfiling(bool enable) = 0;",
            "virtual bool isSDMA() const { return false; }",
            "virtual uint64_t PendingBytes() = 0;",
            "virtual void GangLeader(bool gang_leader) = 0;",
            "virtual bool GangLeader() const { return false; }"):
        assert decl in flat, decl


def test_native_driver_lists_its_cases(pkg):
    _, exe = _paths(pkg)
    out = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, text=True, check=True).stdout.split()
    for engine in ("_hip", "_aql"):
        assert "dependencies_6" + engine in out and "async_copy_blocked_wait" + engine in out
    assert "profiling_timestamps_aql" in out and "copy_rect_with_signal_aql" in out and len(out) >= 25


@pytest.mark.gpu
def test_native_driver_passes_on_gpu(pkg, torch_cuda):
    _, exe = _paths(pkg)
    cases = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, text=True, check=True).stdout.split()
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-4000:]
    for case in cases:
        assert "PASS " + case + "\n" in proc.stdout, "case %s did not pass" % case
    assert "FAIL" not in proc.stdout
