"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer (host code only): `make -C oracle
asan` builds the oracle source with a driver that calls every function on ragged and edge-case shapes
with exactly-sized heap buffers and compares its two GEMM / convolution tiers; any finding aborts it."""
import os
import subprocess

import oracle_lib as O


def test_oracle_is_clean_under_asan_and_ubsan():
    subprocess.check_call(["make", "-C", O.ORACLE_DIR, "-B", "asan"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0:verify_asan_link_order=0"
    r = subprocess.run([os.path.join(O.ORACLE_DIR, "oracle_asan")], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "asan_driver: ok" in r.stdout
