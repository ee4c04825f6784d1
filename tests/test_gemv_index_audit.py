"""CPU audit of the GEMV tile's index arithmetic (tests/gemv_index_audit.cpp over
elutq_amd/csrc/hlq_gemv_index.h, the header the kernel itself computes its runs, LDS offsets and staging
indices with): every slice and wave -- waves without a run included -- of planes 1-4 x groups 64/128 x 1-16
waves x every slice length x 0-4 handed-over slices x {one tile, runs of column blocks per workgroup} stays
inside the dynamic LDS the launcher allocates and inside the documented buffers.  The same audit with the
staged-chunk read replayed without its clamp must report violations (it did read one element past the
staging area before the clamp existed), which shows the audit covers that access."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def audit_exe(tmp_path_factory):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("audit") / "gemv_index_audit")
    subprocess.run([gxx, "-O2", "-std=c++17", "-I", os.path.join(ROOT, "elutq_amd", "csrc"), "-o", exe,
                    os.path.join(ROOT, "tests", "gemv_index_audit.cpp")], check=True)
    return exe


def test_every_access_of_the_gemv_tile_stays_in_bounds(audit_exe):
    res = subprocess.run([audit_exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    assert re.search(r"^violations 0$", res.stdout, re.M)
    shapes = int(re.search(r"^shapes (\d+) checks (\d+)$", res.stdout, re.M).group(1))
    assert shapes > 100_000


def test_the_audit_flags_the_unclamped_staged_read(audit_exe):
    res = subprocess.run([audit_exe, "--unclamped-stage"], capture_output=True, text=True)
    assert res.returncode == 1
    cats = dict(re.findall(r"^category (\S+) (\d+)$", res.stdout, re.M))
    assert set(cats) == {"lds-stage"} and int(cats["lds-stage"]) > 0
    # the offender is a wave without a run: its first k is the end of the slice
    assert "VIOLATION lds-stage" in res.stdout
