"""The CPU oracle under AddressSanitizer and UndefinedBehaviorSanitizer (host code only): a C
driver (tests/c/oracle_sanitized.c) calls every oracle function on exactly sized heap buffers,
edge shapes included; the sanitized build must run clean and print the same checksum as the
plain -O3 build."""
import os
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent


def test_oracle_runs_clean_under_sanitizers():
    subprocess.run(["make", "-C", os.fspath(HERE / "c"), "all"], check=True, capture_output=True)
    environment = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1",
                       UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="2")
    outputs = []
    for name in ("oracle_plain", "oracle_sanitized"):
        done = subprocess.run([os.fspath(HERE / "c" / "build" / name)], capture_output=True, text=True,
                              timeout=300, env=environment)
        assert done.returncode == 0, done.stderr[-2000:]
        assert "Sanitizer" not in done.stderr and "runtime error" not in done.stderr, done.stderr[-2000:]
        outputs.append(done.stdout.strip())
    assert outputs[0] == outputs[1] and outputs[0].startswith("oracle checksum")
