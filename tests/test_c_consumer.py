"""The boundary from C: tests/c/h3_projection_consumer.c implements the reference's own C ABI
for this path, minimax_h3_m3_run_q4_projection_bf16 (minimax_h3_m3_gemm.h:58-66), on top of
include/mi355q.h.  It must compile as strict C11 (-Wall -Wextra -Wpedantic -Werror) and link
against libmi355q; on a GPU it runs as a process of its own on seeded bf16 data and its bf16
output is compared with the oracle."""
import os
import subprocess
import sys
import tempfile
from pathlib import Path

import numpy as np
import pytest

from conftest import bf16_bits, bf16_to_f32, q4_relative_error

HERE = Path(__file__).resolve().parent
BINARY = HERE / "c" / "build" / "h3_projection_consumer"


def build():
    subprocess.run(["make", "-C", os.fspath(HERE / "c")], check=True, capture_output=True)
    assert BINARY.exists()


def write_case(path, quants, scales, biases, x_bits, N, K, M):
    with open(path, "wb") as stream:
        stream.write(np.array([N, K, M], dtype=np.uint32).tobytes())
        for plane in (quants, scales, biases, x_bits):
            stream.write(np.ascontiguousarray(plane).tobytes())


def test_consumer_compiles_as_strict_c11_and_links(engine):
    """Link check on any machine: a fresh build with -Werror, and the program starts (without a
    GPU the context cannot be created: status 1 and the library's message, not a crash)."""
    subprocess.run(["make", "-B", "-C", os.fspath(HERE / "c")], check=True, capture_output=True)
    N, K, M = 16, 64, 1
    quants, scales, biases = engine.synth_q4_affine(3, 0.02, N, K, engine.META_BF16_PLANES)
    with tempfile.TemporaryDirectory() as folder:
        case, out = Path(folder) / "case.bin", Path(folder) / "out.bin"
        write_case(case, quants, scales, biases, np.zeros((M, K), dtype=np.uint16), N, K, M)
        done = subprocess.run([os.fspath(BINARY), os.fspath(case), os.fspath(out)], capture_output=True, text=True,
                              timeout=120)
        if done.returncode != 0:  # no gfx950 device here
            assert done.returncode == 1 and "status 1" in done.stderr
        bad = subprocess.run([os.fspath(BINARY)], capture_output=True, text=True, timeout=60)
        assert bad.returncode == 64


@pytest.mark.gpu
@pytest.mark.parametrize("M", [11, 32])
def test_consumer_process_matches_oracle(engine, oracle, M):
    """A fresh process: N = 1024, K = 5376 (the H3 projection width), the reference's boundary
    input x_i = bf16(((i % 29) - 14) / 32) (minimax_h3_m3_real_gemm.c:59-65) at M = 11 rows (the
    reference's own batch; exact weights) and 32 rows (the matrix-instruction path, weights
    rounded to fp16); bf16 outputs against the oracle, gate 2^-8 (the output rounding)."""
    if not BINARY.exists():
        build()
    N, K = 1024, 5376
    quants, scales, biases = engine.synth_q4_affine(17, 0.02, N, K, engine.META_BF16_PLANES)
    i = np.arange(M * K)
    x = (((i % 29) - 14) / 32.0).astype(np.float32).reshape(M, K)
    x_bits = bf16_bits(x).reshape(M, K)
    assert np.array_equal(bf16_to_f32(x_bits), x)  # the recipe's values are exact in bf16
    with tempfile.TemporaryDirectory() as folder:
        case, out = Path(folder) / "case.bin", Path(folder) / "out.bin"
        write_case(case, quants, scales, biases, x_bits, N, K, M)
        print(f"consumer process M={M}", flush=True)
        done = subprocess.run([os.fspath(BINARY), os.fspath(case), os.fspath(out)], capture_output=True, text=True,
                              timeout=120)
        assert done.returncode == 0, done.stderr
        assert "gpu_ms=" in done.stdout
        y = bf16_to_f32(np.fromfile(out, dtype=np.uint16).reshape(M, N))
    rounding = oracle.W_ROUND_F16 if M > 16 else oracle.W_EXACT
    ref = oracle.q4_linear(quants, scales, biases, oracle.META_BF16_PLANES, N, K, x_bits, oracle.X_BF16, M,
                           weight_rounding=rounding)
    assert q4_relative_error(y, ref) <= 2.0 ** -8
    # the call refuses what the reference refuses: a column count that is no multiple of 64 -> status 2
    with tempfile.TemporaryDirectory() as folder:
        case, out = Path(folder) / "case.bin", Path(folder) / "out.bin"
        write_case(case, quants[:16 * 48], scales[:16], biases[:16], x_bits[:1, :96], 16, 96, 1)
        done = subprocess.run([os.fspath(BINARY), os.fspath(case), os.fspath(out)], capture_output=True, text=True,
                              timeout=120)
        assert done.returncode == 2 and "status 2" in done.stderr
