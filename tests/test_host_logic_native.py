"""Runs tests/cpp/test_host_logic.cpp: the plans of copies, fills and region
copies checked over 300,000 seeded cases each in a native binary built with
AddressSanitizer and UBSan (host code only; nothing here needs a GPU)."""
import os
import subprocess


def test_host_arithmetic_under_sanitizers(pkg):
    exe = pkg.build.HOST_LOGIC_TEST
    if not os.path.exists(exe):
        pkg.build.build_host_logic_test()
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([exe, "300000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600,
                          env=env)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert proc.stdout.strip().endswith("0 failures")
