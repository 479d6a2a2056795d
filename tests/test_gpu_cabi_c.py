"""Runs tests/cabi_parity and tests/cabi_objects, the parity checks written in plain C against include/eri_optim8.h
and include/eri_adam8bit.h: device steps through the C ABI against the CPU oracle, bit for bit, with no Python or
torch in the process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("mode", ["eri", "l2", "bnb"])
def test_c_program_matches_the_oracle(dtype, mode):
    exe = os.path.join(HERE, "cabi_parity")
    # normally built beforehand by __graft_entry__.build(); make does nothing then, and rebuilds a program
    # that is older than the header it was compiled against (the row structs are passed by layout)
    subprocess.check_call(["make", "-s", "-C", HERE, "cabi_parity"])
    out = subprocess.run([exe, dtype, mode], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count("bit-exact") == 5 and out.stdout.strip().endswith("ok")


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("flavour", ["list", "functional"])
def test_c_program_over_the_optimizer_objects_matches_the_oracle(dtype, flavour):
    """The list optimizer (with a parameter that sits out a step) and the functional optimizer (update_many into
    alternating output sets), parameters, gradients and states out of three lanes of the device pool."""
    exe = os.path.join(HERE, "cabi_objects")
    subprocess.check_call(["make", "-s", "-C", HERE, "cabi_objects"])
    out = subprocess.run([exe, dtype, flavour], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count("bit-exact") == 4 and out.stdout.strip().endswith("ok")
