"""The C++ host side (mograd_amd/host/mograd_exec.hpp): the reference's dispatch surface
restated for a compiled caller.  Its test driver (tests/host_cpp/selftest.cpp) runs the
reference's golden vectors, closed forms, exact integer products and error conditions
through the C++ exec functions; here it is built, its rule table is compared with the Python
mirror's, and on a GPU it is run."""
import os
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
DRIVER = ROOT / "tests" / "host_cpp" / "selftest"


@pytest.fixture(scope="module")
def driver():
    if not DRIVER.exists():
        subprocess.run(["make", "-C", str(DRIVER.parent)], check=True, capture_output=True)
    return DRIVER


def test_rule_table_matches_the_python_mirror(driver):
    # No GPU: the driver only prints its table.  Same op types, same exec function names,
    # same order as mograd_amd.runtime.SCHEDULER_RULES.
    from mograd_amd.runtime import SCHEDULER_RULES

    out = subprocess.run([str(driver), "rules"], check=True, capture_output=True, text=True).stdout
    got = [tuple(line.split()) for line in out.splitlines()]
    want = [(op, "sum" if fn.__name__ == "sum" else fn.__name__) for op, fn in SCHEDULER_RULES.items()]
    assert got == want


def test_missing_library_is_an_error(driver):
    # The host side has no fallback: without the library it must fail, before touching a GPU.
    env = dict(os.environ, MOGRAD_HIP_SO=str(ROOT / "mograd_amd" / "no_such_library.so"))
    proc = subprocess.run([str(driver), "run"], env=env, capture_output=True, text=True)
    assert proc.returncode == 3
    assert "cannot load" in (proc.stderr + proc.stdout)


@pytest.mark.gpu
def test_cases_pass_on_the_gpu(driver):
    env = dict(os.environ, MOGRAD_HIP_SO=str(ROOT / "mograd_amd" / "libmograd_hip.so"))
    proc = subprocess.run([str(driver), "run"], env=env, capture_output=True, text=True, timeout=110)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout[-2000:]
    lines = proc.stdout.splitlines()
    assert sum(l.startswith("PASS ") for l in lines) >= 22 and not any(l.startswith("FAIL ") for l in lines)
