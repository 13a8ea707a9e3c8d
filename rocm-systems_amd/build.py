"""Compile recipe for the native parts.  Everything is built in-tree with
hipcc / gcc; nothing is fetched."""
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
INCLUDE = os.path.join(ROOT, "include")
ORACLE_DIR = os.path.join(ROOT, "oracle")

BLIT_LIB = os.path.join(LIB_DIR, "libmi355blit.so")
AQL_LIB = os.path.join(LIB_DIR, "libmi355blit_aql.so")
HSACO = os.path.join(LIB_DIR, "mi355_blit_gfx950.hsaco")
ROCR_LIB = os.path.join(LIB_DIR, "libmi355blit_rocr.so")
ROCR_TEST = os.path.join(LIB_DIR, "test_rocr_blit")
ORACLE_LIB = os.path.join(ORACLE_DIR, "libblit_oracle.so")
HOST_LOGIC_TEST = os.path.join(LIB_DIR, "test_host_logic")
KERNELS_ON_CPU_TEST = os.path.join(LIB_DIR, "test_kernels_on_cpu")
XCD_PROGRESS = os.path.join(LIB_DIR, "xcd_progress")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    # hipcc may pair float ops into packed-FP32 instructions; keep them scalar
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    exe = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build the gfx950 blit library")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def build_blit():
    """HIP kernels + C ABI -> lib/libmi355blit.so"""
    os.makedirs(LIB_DIR, exist_ok=True)
    _run([_hipcc()] + HIPCC_FLAGS + [
        "-shared", "-I", INCLUDE, "-I", CSRC,
        "-o", BLIT_LIB, os.path.join(CSRC, "blit_capi.hip"),
    ])
    return BLIT_LIB


def build_aql():
    """Stand-alone gfx950 code object + the HSA-only AQL engine ->
    lib/mi355_blit_gfx950.hsaco, lib/libmi355blit_aql.so"""
    os.makedirs(LIB_DIR, exist_ok=True)
    _run([_hipcc()] + HIPCC_FLAGS + [
        "--cuda-device-only", "--no-gpu-bundle-output", "-I", INCLUDE, "-I", CSRC,
        "-o", HSACO, os.path.join(CSRC, "blit_code_object.hip"),
    ])
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-shared",
          "-I", INCLUDE, "-I", CSRC, "-I", os.path.join(ROCM, "include"),
          "-DHSACO_PATH=\"%s\"" % HSACO,
          "-o", AQL_LIB, os.path.join(CSRC, "aql_capi.cpp"), os.path.join(CSRC, "aql_runtime.cpp"),
          os.path.join(CSRC, "hsaco_embed.S"),
          "-L", os.path.join(ROCM, "lib"), "-lhsa-runtime64", "-lpthread",
          "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return AQL_LIB


def build_rocr_adapter():
    """C++ core::Blit adapter over the C ABI + public HSA signals ->
    lib/libmi355blit_rocr.so, and its native test driver."""
    src = os.path.join(CSRC, "rocr_blit.cpp")
    if not os.path.exists(src):
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    common = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-I", INCLUDE, "-I", CSRC,
              "-I", os.path.join(ROCM, "include")]
    link = ["-L", LIB_DIR, "-lmi355blit", "-lmi355blit_aql", "-L", os.path.join(ROCM, "lib"), "-lhsa-runtime64",
            "-lpthread", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    _run(["g++"] + common + ["-shared", "-o", ROCR_LIB, src, os.path.join(CSRC, "rocr_blit_aql.cpp")] + link)
    return ROCR_LIB


def build_rocr_test():
    """Native test driver of the adapter (links the CPU oracle as its checker)."""
    test_src = os.path.join(ROOT, "tests", "cpp", "test_rocr_blit.cpp")
    if not (os.path.exists(test_src) and os.path.exists(ROCR_LIB)):
        return None
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__",
          "-I", INCLUDE, "-I", CSRC, "-I", os.path.join(ROCM, "include"),
          "-o", ROCR_TEST, test_src,
          "-L", LIB_DIR, "-lmi355blit_rocr", "-lmi355blit", "-lmi355blit_aql",
          "-L", ORACLE_DIR, "-lblit_oracle",
          "-L", os.path.join(ROCM, "lib"), "-lhsa-runtime64", "-lamdhip64", "-lpthread",
          "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,$ORIGIN/../../oracle",
          "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return ROCR_TEST


def build_host_logic_test():
    """Native test of the host arithmetic (plans of copies, fills and region
    copies) under AddressSanitizer and UBSan; host code only, the CPU oracle
    compiled in as its checker."""
    test_src = os.path.join(ROOT, "tests", "cpp", "test_host_logic.cpp")
    if not os.path.exists(test_src):
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    _run(["g++", "-O1", "-g", "-Wall", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
          "-static-libasan", "-static-libubsan", "-I", INCLUDE, "-I", CSRC,
          "-o", HOST_LOGIC_TEST, "-x", "c", os.path.join(ORACLE_DIR, "blit_oracle.c"),
          "-x", "c++", "-std=c++17", test_src, "-lpthread"])
    return HOST_LOGIC_TEST


def build_kernels_on_cpu_test():
    """The blit kernels compiled for the host over tests/cpp/lane_emulation.h
    (lanes in lock step, every access checked), under AddressSanitizer and
    UBSan."""
    test_src = os.path.join(ROOT, "tests", "cpp", "test_kernels_on_cpu.cpp")
    if not os.path.exists(test_src):
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    _run(["g++", "-O1", "-g", "-std=c++17", "-Wall", "-Wno-unknown-pragmas", "-fsanitize=address,undefined",
          "-fno-sanitize-recover=all", "-static-libasan", "-static-libubsan", "-I", INCLUDE, "-I", CSRC,
          "-I", os.path.join(ROOT, "tests", "cpp"), "-o", KERNELS_ON_CPU_TEST, test_src])
    return KERNELS_ON_CPU_TEST


def build_oracle():
    """CPU oracle (test infrastructure) -> oracle/libblit_oracle.so"""
    _run(["make", "-C", ORACLE_DIR, "-B", "libblit_oracle.so"])
    return ORACLE_LIB


def build_xcd_progress():
    """GPU diagnostic: the XCD every workgroup of a launch runs on and how far
    apart the XCDs drift in one long copy (tests/cpp/xcd_progress.hip)."""
    src = os.path.join(ROOT, "tests", "cpp", "xcd_progress.hip")
    if not os.path.exists(src):
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    _run([_hipcc()] + flags + ["-I", INCLUDE, "-I", CSRC, "-o", XCD_PROGRESS, src])
    return XCD_PROGRESS


def build_all():
    out = [build_blit(), build_aql()]
    r = build_rocr_adapter()
    if r:
        out.append(r)
    out.append(build_oracle())
    for t in (build_rocr_test(), build_host_logic_test(), build_kernels_on_cpu_test(), build_xcd_progress()):
        if t:
            out.append(t)
    return out


if __name__ == "__main__":
    for path in build_all():
        print("built", path)
