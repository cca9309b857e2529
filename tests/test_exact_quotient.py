"""The division of SOFIE_I8OUT_I8_DQQ formed from the rounded reciprocal (sofie_amd/csrc/exact_quotient.hpp) against the
processor's IEEE division: every float of the sixteen binades around the divisor (2^-4 <= |v / q| < 2^11, both signs) for
twenty divisors, random operands over the whole admitted range, the reciprocal against quad precision, and the divisors and
scales that must be refused.  A formula with one Newton correction less than needed, or none, fails here (the uncorrected
product differs from the quotient for a third of the operands)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_quotient_by_reciprocal_equals_ieee_division(tmp_path):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    exe = str(tmp_path / "quotient_check")
    flags = ["-O2", "-ffp-contract=off", "-std=c++17"]
    with open("/proc/cpuinfo") as f:
        if " fma " in f.read():
            flags.append("-mfma")  # hardware fused multiply-add; without it libm's (equally exact) one runs, ten times slower
    subprocess.run([gxx] + flags + ["-I" + os.path.join(ROOT, "sofie_amd", "csrc"), os.path.join(ROOT, "tests", "quotient_check.cxx"), "-o", exe],
                   check=True)
    r = subprocess.run([exe, "7"], stdout=subprocess.PIPE, text=True, timeout=900)
    lines = r.stdout.strip().splitlines()
    assert r.returncode == 0, r.stdout
    rows = [l.split() for l in lines if not l.startswith("reciprocals")]
    assert len(rows) == 20
    for q, tried, bad in rows:
        assert int(tried) > 250_000_000 and int(bad) == 0, (q, tried, bad)
    recip = [l.split() for l in lines if l.startswith("reciprocals")][0]
    assert int(recip[1]) == 2_000_000 and int(recip[2]) == 0
