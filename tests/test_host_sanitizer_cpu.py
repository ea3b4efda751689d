"""The C-ABI front (argument validation, batch slicing, status texts, tunables) built for the host
alone, with stand-in launchers that record what they are asked to launch, and the plain-C oracle,
run under AddressSanitizer and UndefinedBehaviorSanitizer (tests/host_sanitizer/).  No GPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_layer_under_address_and_ub_sanitizers(tmp_path):
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host_sanitizer"), "check", "OUT=%s" % tmp_path],
                         capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "host sanitizer run ok" in res.stdout
    assert "runtime error" not in res.stderr and "AddressSanitizer" not in res.stderr
