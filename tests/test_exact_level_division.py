"""The quantise kernels divide a group's range by the level count with three float operations
instead of an IEEE division (kivi_quant.hip, ``group_scale`` with ``LevelDiv``) where that is
exact: for 2^b - 1 levels, b = 1..8.  ``tests/exact_level_division.c`` compares the two over the
non-negative finite floats; this runs it over every 4099th of them plus the smallest and largest
ones (the full range, stride 1, takes minutes and found no mismatch)."""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def _build(tmp_path):
    exe = str(tmp_path / "exact_level_division")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-o", exe, os.path.join(HERE, "exact_level_division.c"), "-lm", "-lpthread"],
                   check=True)
    return exe


def test_three_operation_division_by_the_level_counts_is_exact_on_a_sample(tmp_path):
    exe = _build(tmp_path)
    for stride in ("4099", "65537"):
        out = subprocess.run([exe, stride], capture_output=True, text=True)
        sys.stdout.write(out.stdout)
        assert out.returncode == 0, out.stdout
        assert out.stdout.count("0 mismatches") == 8
