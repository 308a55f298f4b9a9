"""The host code of the library under AddressSanitizer and UndefinedBehaviorSanitizer: tests/sanitize/format_driver.cc
drives the format builders through the C-ABI (random matrices through all fourteen skeletons, dense operators,
division of sub-blocks and columns, the forms of the tile template, two-strip graphs with fused and carried kernels,
kernel source generation; no GPU).  The build takes a few minutes, so the test runs only with ASX_SANITIZE=1."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sanitize")


@pytest.mark.skipif(os.environ.get("ASX_SANITIZE") != "1", reason="set ASX_SANITIZE=1 to build and run the sanitizer driver (a few minutes)")
def test_format_builders_under_address_and_undefined_behaviour_sanitizers():
    subprocess.run(["bash", os.path.join(HERE, "build.sh")], check=True, timeout=1800)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1")
    p = subprocess.run([os.path.join(HERE, "build", "format_driver"), "8"], capture_output=True, text=True, timeout=1800, env=env)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-4000:]
    assert "ERROR: AddressSanitizer" not in p.stderr and "runtime error" not in p.stderr, p.stderr[-4000:]
    last = p.stdout.strip().splitlines()[-1]
    assert last.startswith("done:") and last.endswith(" 0 api errors") and int(last.split()[1]) > 100, last
