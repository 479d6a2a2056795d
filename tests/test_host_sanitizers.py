"""The host side of the library under AddressSanitizer, UndefinedBehaviorSanitizer and the leak checker, on the CPU.

tests/san_host.mk rebuilds the two host translation units with the sanitizers (host code only) into
tests/_san/libsan_host.so and links tests/san_host against it; the program feeds the state-file parsers a
directory of mutated files and walks the argument checks of the launch table, the functional optimizer and the
pool.  A Python process cannot host a sanitized library (the sanitizer's allocator has to be in place before the
first allocation of the process), which is why this runs as a program of its own."""
import os
import subprocess

import pytest

from test_host_objects_cpu import mutated_state_files

HERE = os.path.dirname(os.path.abspath(__file__))


def test_host_code_is_clean_under_the_sanitizers(tmp_path):
    if not os.path.exists(os.path.join(HERE, "san_host.mk")):
        pytest.skip("the sanitizer build rules are not part of this copy of the tree (they stay off machines with a GPU)")
    count = 600
    for k, (use_st, blob) in enumerate(mutated_state_files(count, seed=4321)):
        (tmp_path / ("%03d.%s" % (k, "st" if use_st else "bc"))).write_bytes(blob)
    subprocess.check_call(["make", "-s", "-C", HERE, "-f", "san_host.mk", "san_host"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:halt_on_error=1", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    out = subprocess.run([os.path.join(HERE, "san_host"), str(tmp_path), str(count)], capture_output=True, text=True,
                         timeout=600, env=env)
    text = out.stdout + out.stderr
    assert out.returncode == 0, text[-4000:]
    for marker in ("AddressSanitizer", "LeakSanitizer", "runtime error:"):
        assert marker not in text, text[-4000:]
    assert out.stdout.strip().endswith("ok")
