"""The index arithmetic of the kernels that normalise rows into LDS, swept on the host over every shape their
launchers admit (tests/layout_sweep.cpp, built here with g++ and the address and undefined-behaviour checks
of the compiler, as the reference builds its own C++ for its sanitizer job: CMakeLists.txt:19-22,
.github/workflows/ci.yml:29-40).  The kernels take these addresses from the same header the sweep includes."""

import os
import subprocess
import tempfile
from pathlib import Path

import pytest

HERE = Path(__file__).resolve().parent


@pytest.fixture(scope="module")
def sweep_output():
    out_dir = Path(tempfile.gettempdir()) / f"bitwise_amd_plain_{os.getuid()}"
    out_dir.mkdir(exist_ok=True)
    exe = out_dir / f"layout_sweep_{os.getpid()}"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                    str(HERE / "layout_sweep.cpp"), "-o", str(exe)], check=True)
    try:
        p = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600)
    finally:
        exe.unlink(missing_ok=True)
    assert "ERROR: AddressSanitizer" not in p.stderr and "runtime error" not in p.stderr, p.stderr[-3000:]
    return p.returncode, p.stdout


def test_every_admitted_shape_stays_inside_its_row_and_its_lds(sweep_output):
    rc, out = sweep_output
    lines = out.splitlines()
    fails = [l for l in lines if l.startswith("FAIL") and "removed variant" not in l]
    assert rc == 0 and not fails, "\n".join(fails[:20])
    counts = {l.split()[1]: int(l.split()[2]) for l in lines if l.startswith("ok ") and len(l.split()) == 3}
    # each part of the sweep ran, over a number of addresses that says it was not empty
    assert counts["row-vectors-8"] > 1e4 and counts["row-vectors-16"] > 5e4 and counts["mid-ring"] > 3e4
    assert counts["mid-norm-rows"] > 1e7 and counts["decode-rows"] > 1e7
    assert "ok in-library failures 0" in out


def test_the_sweep_can_fail_and_what_it_says_of_the_variant_that_was_taken_out(sweep_output):
    """The same checks applied to what is not in the library: a load that is not clamped into its row is found
    (so the checks can fail), and rows of 4096 in 16-row blocks would have been refused at the launch."""
    _, out = sweep_output
    notes = [l for l in out.splitlines() if l.startswith("note removed-variant")]
    assert any("16 rows x 4096 in 16-row blocks: 197632 bytes" in l and "refused" in l for l in notes)
    assert any("unclamped" in l and "8192 loads leave their row" in l for l in notes)
    assert any("clamped, 16 rows x 2048" in l and l.endswith(" 0 failures") for l in notes)
