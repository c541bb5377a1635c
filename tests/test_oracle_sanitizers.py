"""The plain-C oracle under AddressSanitizer + UndefinedBehaviorSanitizer (host code only): built
from oracle/polar_oracle.c and a small driver, run as a child process."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.mark.parametrize("san", ["address,undefined", "undefined"])
def test_c_oracle_is_clean_under_sanitizers(tmp_path, san):
    exe = str(tmp_path / "oracle_san")
    cmd = ["gcc", "-O1", "-g", "-std=c11", "-ffp-contract=off", "-fno-omit-frame-pointer", "-fsanitize=" + san,
           "-fno-sanitize-recover=all", "-static-libasan", "-static-libubsan",
           os.path.join(ROOT, "oracle", "polar_oracle.c"), os.path.join(HERE, "oracle_san_main.c"), "-o", exe, "-lm"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    if build.returncode != 0:
        pytest.skip("sanitizer runtime not available to gcc here: " + build.stderr[-300:])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=120)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert run.stdout.startswith("checksum ") and "runtime error" not in run.stderr
