"""What the compiler made of the kernels, read from this build's own gfx950
code object: every body access must be a global_* instruction (a generic
pointer would give flat_*, which pays the aperture check and counts against
both memory counters), and every 16-byte store must carry the cache policy its
kernel is named for (a hint that got lost in the optimizer costs 10-15 % at
1 GiB and no test of the bytes can see it)."""
import collections
import os
import re
import shutil
import subprocess

import pytest

OBJDUMP = "/opt/rocm/llvm/bin/llvm-objdump"


@pytest.fixture(scope="module")
def kernels(pkg):
    code_object = os.path.join(os.path.dirname(pkg.capi.library_path()), "mi355_blit_gfx950.hsaco")
    if not (os.path.exists(OBJDUMP) or shutil.which("llvm-objdump")):
        pytest.skip("no llvm-objdump in this image")
    assert os.path.exists(code_object), code_object
    tool = OBJDUMP if os.path.exists(OBJDUMP) else shutil.which("llvm-objdump")
    text = subprocess.run([tool, "-d", "--no-show-raw-insn", code_object], check=True, capture_output=True,
                          text=True).stdout
    out = collections.OrderedDict()
    name = None
    for line in text.splitlines():
        m = re.match(r"^[0-9a-f]+ <(mi355_[a-z0-9_]+)>:", line)
        if m:
            name = m.group(1)
            out[name] = []
        elif name and line.startswith("\t"):
            out[name].append(line.split("//")[0].strip())
    assert len(out) > 100, "kernels found: %d" % len(out)
    return out


def test_no_flat_memory_instructions(kernels):
    for name, body in kernels.items():
        flat = [i for i in body if i.startswith("flat_")]
        if name == "mi355_signal_complete":
            continue   # one system-scope atomic on an HSA signal in host memory
        assert not flat, "%s: %s" % (name, flat[:3])


def test_store_policies_are_what_the_names_say(kernels):
    want = {"0": "", "1": "nt", "2": "sc1", "3": "sc0 sc1"}
    checked = 0
    for name, body in kernels.items():
        m = re.search(r"_s([0-3])(_r[01])?$", name)
        if not m or not name.startswith(("mi355_copy_", "mi355_fill_", "mi355_batch_records_", "mi355_batch_lookup_",
                                         "mi355_rect_")):
            continue
        stores = [i for i in body if i.startswith("global_store_dwordx4")]
        assert stores, name
        for i in stores:
            bits = " ".join(w for w in i.split("off", 1)[1].split() if w in ("nt", "sc0", "sc1")) if "off" in i else ""
            assert bits == want[m.group(1)], "%s: %s" % (name, i)
        checked += 1
    assert checked >= 100


def test_load_policies_are_what_the_names_say(kernels):
    for name, body in kernels.items():
        m = re.search(r"_l([01])_s[0-3]", name)
        if not m:
            continue
        loads = [i for i in body if i.startswith("global_load_dwordx4")]
        assert loads, name
        for i in loads:
            assert (" nt" in i) == (m.group(1) == "1"), "%s: %s" % (name, i)
