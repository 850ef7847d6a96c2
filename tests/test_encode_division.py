"""The FP8 row-encode kernel replaces the per-element IEEE divide by a reciprocal plus one
fused correction step; this CPU test checks that sequence against the IEEE quotient on a
sample of all (row maximum, element) pairs (the full space is a one-minute run of the same
program with stride 1)."""
import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))


def test_division_free_quotient_is_correctly_rounded():
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "markstein_check")
        subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe, os.path.join(HERE, "markstein_check.c"), "-lm"],
                       check=True)
        out = subprocess.run([exe, "61"], check=True, capture_output=True, text=True).stdout
    checked, bad = int(out.split()[1]), int(out.split()[3])
    assert checked > 1_000_000 and bad == 0
