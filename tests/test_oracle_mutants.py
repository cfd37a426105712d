"""The pins of tests/test_oracle_pins.py must tell the checker from a nearly right one: the checker's source carries eight
deliberate slips (ORC_MUTATE = 1..8 in oracle/mascot_oracle.c: MuPPET's scale index with a ceiling for the floor, the index
one too large, the half step of either quantisation bound with the wrong sign, the quantised error truncated instead of rounded; AFP's scale
with a floor for the ceiling; the MuPPET ladder with a threshold 10 % lower or a window one epoch short).  Each is built
into a library of its own and the pin tests are run against it in a child process: at least one pin must fail.  The
unmodified source built the same way must pass, so a failure is the slip's doing."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCE = os.path.join(ROOT, "oracle", "mascot_oracle.c")
CFLAGS = ["-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-Wall", "-Wno-unknown-pragmas", "-mavx2", "-mf16c"]
SLIPS = {1: "MuPPET scale index: ceiling for floor", 2: "MuPPET scale index one too large", 3: "MuPPET upper bound: half step with the wrong sign",
         4: "MuPPET lower bound: half step with the wrong sign", 5: "MuPPET quantised error truncated", 6: "AFP scale: floor for ceiling",
         7: "ladder threshold 10 % lower", 8: "ladder window one epoch short"}


def run_pins(tmp_path, slip):
    out = tmp_path / ("slip%d" % slip)
    out.mkdir()
    for name, extra in (("liboracle.so", []), ("liboracle_soft.so", ["-DORC_SOFT_HALF"])):
        subprocess.check_call(["gcc"] + CFLAGS + extra + ["-DORC_MUTATE=%d" % slip, SOURCE, "-o", str(out / name), "-lm"])
    env = dict(os.environ, ORACLE_BUILD_DIR=str(out))
    return subprocess.run([sys.executable, "-m", "pytest", os.path.join(HERE, "test_oracle_pins.py"), "-x", "-q", "-p", "no:cacheprovider"],
                          cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_unmodified_checker_passes_its_pins(tmp_path):
    r = run_pins(tmp_path, 0)
    assert r.returncode == 0, r.stdout[-2000:]


@pytest.mark.parametrize("slip", sorted(SLIPS))
def test_every_slip_fails_a_pin(tmp_path, slip):
    r = run_pins(tmp_path, slip)
    assert r.returncode == 1, "slip %d (%s) went unnoticed by the pins:\n%s" % (slip, SLIPS[slip], r.stdout[-2000:])
    assert " failed" in r.stdout
