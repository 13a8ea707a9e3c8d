"""The assumption behind the launch permutation of the blit kernels
(xcd_workgroup, csrc/blit_args.h): workgroup b of a launch runs on XCD b % 8.
tests/cpp/xcd_progress.hip runs a copy of the product's shape whose workgroups
note the XCD they run on; it is a process of its own because it is a HIP
program, not a call into the library."""
import json
import os
import subprocess

import pytest


@pytest.mark.gpu
def test_workgroup_b_runs_on_xcd_b_mod_8(pkg):
    exe = pkg.build.XCD_PROGRESS
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    out = subprocess.run([exe, "1", "576"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-2000:]
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    # every residue has one XCD of its own, and every noting workgroup confirms it
    assert sorted(rec["xcc_of_residue"]) == list(range(8)), rec
    assert rec["agree"] == rec["noting_workgroups"] == 8 * (1 << 20) // 512, rec
    # the XCDs stay within a few thousand workgroups of one another over 1 GiB
    assert max(rec["spread_thousand_workgroups"][:-1]) < 8.0, rec


def test_xcd_progress_is_built(pkg):
    assert os.path.exists(pkg.build.XCD_PROGRESS), "run __graft_entry__.build() first"
