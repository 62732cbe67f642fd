"""The threaded host logic (slot cache, prefetch ring, submission service, completion timeline, tagged readback)
under ThreadSanitizer and AddressSanitizer/UBSan: host-only g++ builds of the library's own sources, driven by the
programs under tests/cpp/sanitize (`make -C shrike_amd/csrc tsan|asan`). A report fails the run."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("target", ["tsan", "asan"])
def test_threaded_host_logic_is_clean_under(target):
    out = subprocess.run(["make", "-C", os.path.join(ROOT, "shrike_amd", "csrc"), target], capture_output=True, text=True,
                         env=dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66", ASAN_OPTIONS="detect_leaks=1"))
    text = out.stdout + out.stderr
    if "unexpected memory mapping" in text or "ASLR" in text and out.returncode != 0:
        pytest.skip("the sanitizer runtime cannot map its shadow memory in this environment")
    assert out.returncode == 0, text[-3000:]
    assert "WARNING: ThreadSanitizer" not in text and "ERROR: AddressSanitizer" not in text and "runtime error" not in text, text[-3000:]
    assert text.count("== ") == 3
