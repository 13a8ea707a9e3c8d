"""Runs tests/cpp/test_kernels_on_cpu.cpp: the blit kernels themselves, compiled
for the host over a lock-step lane emulation, launched with the product's own
plans.  Pins what no GPU test can: that no load of a copy leaves the aligned
dwords that hold a requested source byte (the reference's shaders mask their
edge accesses and never over-read either, blit_copyAligned.s:108-128, 236-256),
and no store the destination range -- for the linear copy over all 256 offset
pairs and every length up to 1100 bytes and around the tile sizes, the fill, the
batched copy on both descriptor paths and the region kernels.  Built with
AddressSanitizer and UBSan; nothing here needs a GPU."""
import os
import subprocess

SHARDS = 4


def _exe(pkg):
    exe = pkg.build.KERNELS_ON_CPU_TEST
    if not os.path.exists(exe):
        pkg.build.build_kernels_on_cpu_test()
    return exe


def test_planted_over_read_is_found(pkg):
    """Every dword load moved up by four bytes: the realigning copy's fetch of
    the dword behind its last vector then leaves the source, and the checker
    must say so in every case (and report nothing for the kernels as built)."""
    proc = subprocess.run([_exe(pkg), "--self-test"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "moved up by 4 bytes found in 192" in proc.stdout, proc.stdout[-2000:]


def test_kernels_touch_only_what_the_command_names(pkg):
    exe = _exe(pkg)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    procs = [subprocess.Popen([exe, "--shard", "%d/%d" % (i, SHARDS)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                              text=True, env=env) for i in range(SHARDS)]
    for i, proc in enumerate(procs):
        out, _ = proc.communicate(timeout=1200)
        assert proc.returncode == 0, "shard %d:\n%s" % (i, out[-4000:])
        assert out.strip().endswith("0 failures"), out[-2000:]
