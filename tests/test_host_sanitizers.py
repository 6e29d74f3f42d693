"""The repository's HOST code under AddressSanitizer + UndefinedBehaviorSanitizer and under ThreadSanitizer (the
reference has the same for its own host code: .bazelrc:108-115 `--config=asan`, kv_cache_manager/client/test/asan_runner.py).

`make -C tests/cpp sanitize` compiles oracle/kvcm_oracle.c, the library's host-only translation units
(csrc/kvcm_file.hip, csrc/kvcm_host.hip, csrc/kvcm_host_idx.h) and include/kvcm_hip.hpp with a plain host compiler
over a host stand-in of the HIP runtime (tests/cpp/sanitize/fake_hip.cpp), twice, and runs tests/cpp/sanitize/
sanitize_host.cpp in both builds: 16 concurrent callers of a file store, a store destroyed while a transfer is inside
it, the blocking cell pool, the index-list walk, the oracle's threaded forms. No GPU code is involved."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.timeout(600)
def test_host_code_is_clean_under_asan_ubsan_and_tsan():
    if shutil.which("g++") is None or shutil.which("make") is None:
        pytest.skip("no host compiler")
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "sanitize"], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=580)
    tail = proc.stdout[-4000:]
    assert proc.returncode == 0, tail
    assert proc.stdout.count("sanitize_host: all scenarios passed") == 2, tail
    assert "runtime error" not in proc.stdout and "Sanitizer" not in proc.stdout.replace("ThreadSanitizer: reported", ""), tail
