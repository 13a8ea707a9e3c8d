"""The core::Blit adapter compiled against ROCr's own headers.  In this
repository csrc/rocr_blit.h carries stand-ins for core::Agent, core::Queue and
core::Signal and repeats core::Blit; with MI355_ROCR_IN_TREE defined it takes
the real core/inc/{blit,agent,queue,signal}.h instead.  This test compiles the
adapter (csrc/rocr_blit_aql.cpp) and a caller shaped like GpuAgent::
CreateBlitKernel (tests/cpp/rocr_in_tree_check.cpp) that way, to objects: every
`override` must match a pure virtual of the real interface, the class must be
concrete, and the members the adapter calls on the real Agent / Queue / Signal
must exist with those signatures.  Needs the reference tree (the headers are not
part of an installed ROCm); skipped where it is absent."""
import os
import subprocess
import tempfile

import pytest

REF = "/root/reference/projects/rocr-runtime"
RT = os.path.join(REF, "runtime", "hsa-runtime")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rocm-systems_amd", "csrc")


@pytest.mark.skipif(not os.path.exists(os.path.join(RT, "core", "inc", "blit.h")),
                    reason="ROCr's internal headers (the reference tree) are not on this machine")
@pytest.mark.parametrize("source", [os.path.join(CSRC, "rocr_blit_aql.cpp"),
                                    os.path.join(ROOT, "tests", "cpp", "rocr_in_tree_check.cpp")])
def test_adapter_compiles_against_the_real_interface(source):
    with tempfile.TemporaryDirectory() as tmp:
        cmd = ["g++", "-std=c++17", "-c", "-Wall", "-Werror=overloaded-virtual", "-DMI355_ROCR_IN_TREE",
               "-I", RT, "-I", os.path.join(RT, "inc"), "-I", os.path.dirname(RT),
               "-I", os.path.join(REF, "libhsakmt", "include"), "-I", "/opt/rocm/include",
               "-I", os.path.join(ROOT, "include"), "-I", CSRC,
               "-o", os.path.join(tmp, "out.o"), source]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
        assert proc.returncode == 0, proc.stdout[-6000:]
        assert os.path.getsize(os.path.join(tmp, "out.o")) > 0
