"""The hand-over protocol of the one-launch MLP (csrc/q4_chain.hip) modelled with host threads
under the thread sanitizer (tests/c/chain_protocol_model.cpp): counters that are never reset,
the last step's extra count, launch-order dispatch onto few places, and the bounded wait ending
a launch whose consumers cannot be served."""
import os
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent


def test_chain_protocol_model_runs_clean():
    subprocess.run(["make", "-C", os.fspath(HERE / "c"), os.fspath(HERE / "c" / "build" / "chain_protocol_model")],
                   check=True, capture_output=True)
    done = subprocess.run([os.fspath(HERE / "c" / "build" / "chain_protocol_model")], capture_output=True, text=True,
                          timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert "ThreadSanitizer" not in done.stderr, done.stderr[-2000:]
    assert done.stdout.strip() == "chain model ok"
