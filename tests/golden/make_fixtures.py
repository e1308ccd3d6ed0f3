"""Writes the golden vectors under tests/golden/ from the reference's own compiled C
(oracle/_ref, built by oracle/Makefile from the sources under the reference tree).
Run in the build container only; the committed .npz files are what the tests read
where the reference tree is absent.  Inputs are seeded; nothing here imports or
executes the reference's Python.

    python tests/golden/make_fixtures.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT / "oracle"))
sys.path.insert(0, str(ROOT / "tests"))
import oracle  # noqa: E402
from sym128 import output_block, pack_sym128  # noqa: E402

HERE = Path(__file__).resolve().parent


def sym128_fixture():
    ref = oracle.ref_qwen35()
    assert ref is not None, "oracle/_ref is not built"
    rng = np.random.default_rng(20250101)
    rows, cols = 12, 384
    weights = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    weights[3, 128:256] = 0.0  # an all-zero group (scale falls back to 1)
    records = pack_sym128(weights)
    blocked = output_block(records, 4)
    x = rng.standard_normal(cols).astype(np.float32)
    out = {"weights": weights, "records": records.reshape(-1), "blocked": blocked, "x": x}
    for name, data, flag in (("rowmajor", records.reshape(-1), 0), ("blocked", blocked, 1)):
        y = np.empty(rows, dtype=np.float32)
        ref.ref_qwen35_q4_gemv(data.ctypes.data, flag, rows, cols, x.ctypes.data, y.ctypes.data)
        out[f"y_{name}"] = y
        dq = np.empty((rows, cols), dtype=np.float32)
        for r in range(rows):
            ref.ref_qwen35_dequantize_q4_row(data.ctypes.data, flag, rows, cols, r, dq[r].ctypes.data)
        out[f"dequant_{name}"] = dq
    np.savez_compressed(HERE / "sym128_q4_gemv.npz", **out)


def w8a8_fixture():
    ref = oracle.ref_minimindo()
    assert ref is not None, "oracle/_ref is not built"
    rng = np.random.default_rng(20250102)
    M, K, N = 7, 160, 24
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[2] = 0.0                      # all-zero token: zero codes, scale 0
    x[3, :8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.0, -127.0]  # exact .5 ties after scaling
    x[3, 8:] = 0.0
    x[3, 6] = 127.0
    q = np.empty((M, K), dtype=np.int8)
    scales = np.empty(M, dtype=np.float32)
    for m in range(M):
        scales[m] = ref.ref_minimindo_quantize_i8(x[m].ctypes.data, q[m].ctypes.data, K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    rows = oracle.q8_weight_quantize(w)
    bias = rng.standard_normal(N).astype(np.float32)
    out_bias = np.empty((M, N), dtype=np.float32)
    out_nobias = np.empty((M, N), dtype=np.float32)
    ref.ref_minimindo_matrix_sequence_i8_quantized(rows.ctypes.data, N, K, q.ctypes.data,
                                                   scales.ctypes.data, M, out_bias.ctypes.data,
                                                   bias.ctypes.data)
    ref.ref_minimindo_matrix_sequence_i8_quantized(rows.ctypes.data, N, K, q.ctypes.data,
                                                   scales.ctypes.data, M, out_nobias.ctypes.data, None)
    dots = np.array([[ref.ref_minimindo_q8_i8_dot(rows[n * (4 + K) + 4:].ctypes.data, q[m].ctypes.data, K)
                      for n in range(N)] for m in range(M)], dtype=np.int32)
    np.savez_compressed(HERE / "w8a8_minimindo.npz", x=x, q=q, scales=scales, w=w, rows=rows, bias=bias,
                        out_bias=out_bias, out_nobias=out_nobias, dots=dots)


def q8rows_f32_fixture():
    """The reference's q8_matvec / q8_matmul_sequence (minimindo_thinker.c:181-213) on seeded inputs."""
    ref = oracle.ref_thinker()
    assert ref is not None, "oracle/_ref is not built"
    rng = np.random.default_rng(20250103)
    N, K, M = 40, 192, 3
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    w[5] = 0.0  # all-zero row: scale 1, zero codes
    rows = oracle.q8_weight_quantize(w)
    x = rng.standard_normal((M, K)).astype(np.float32)
    out = np.empty((M, N), dtype=np.float32)
    ref.ref_thinker_q8_matmul_sequence(rows.ctypes.data, N, K, x.ctypes.data, M, out.ctypes.data)
    out_one = np.empty((1, N), dtype=np.float32)
    ref.ref_thinker_q8_matmul_sequence(rows.ctypes.data, N, K, x[1].ctypes.data, 1, out_one.ctypes.data)
    np.savez_compressed(HERE / "q8rows_f32_thinker.npz", rows=rows, x=x, out=out, out_one=out_one)


def mimi_conv_fixture():
    """The reference's causal_q8_windows and stream_conv1d (minimindo_mimi.c:552-598,869-917): two
    consecutive chunks of a stream (the second starts from the history the first left), kernel 7
    and kernel 1, and a chunk shorter than the history."""
    ref = oracle.ref_mimi()
    assert ref is not None, "oracle/_ref is not built"
    rng = np.random.default_rng(20250104)
    out = {}
    for tag, (C, O, kernel, lengths) in {"k7": (16, 24, 7, (9, 4, 12)), "k1": (32, 8, 1, (5,))}.items():
        w = (rng.standard_normal((O, C * kernel)) * 0.05).astype(np.float32)
        rows = oracle.q8_weight_quantize(w)
        bias = rng.standard_normal(O).astype(np.float32)
        history = np.zeros((C, max(kernel - 1, 1)), dtype=np.float32)[:, :kernel - 1].copy()
        out[f"{tag}_rows"], out[f"{tag}_bias"] = rows, bias
        out[f"{tag}_shape"] = np.array([C, O, kernel], dtype=np.int64)
        for index, length in enumerate(lengths):
            x = rng.standard_normal((C, length)).astype(np.float32)
            if index == 1:
                x[:, 1] = 0.0
            before = history.copy()
            q = np.empty((length, C * kernel), dtype=np.int8)
            scales = np.empty(length, dtype=np.float32)
            history_arg = before.ctypes.data if kernel > 1 else None
            assert ref.ref_mimi_causal_q8_windows(x.ctypes.data, history_arg, C, kernel, length, q.ctypes.data,
                                                  scales.ctypes.data) == 0
            y = np.empty((O, length), dtype=np.float32)
            state = history.copy() if kernel > 1 else np.zeros(1, dtype=np.float32)
            assert ref.ref_mimi_stream_conv1d(rows.ctypes.data, bias.ctypes.data, C, O, kernel, state.ctypes.data,
                                              x.ctypes.data, length, y.ctypes.data) == 0
            if kernel > 1:
                history = state
            for name, value in (("x", x), ("history_before", before), ("q", q), ("scales", scales), ("y", y),
                                ("history_after", history.copy())):
                out[f"{tag}_{index}_{name}"] = value
    np.savez_compressed(HERE / "mimi_stream_conv.npz", **out)


if __name__ == "__main__":
    sym128_fixture()
    w8a8_fixture()
    q8rows_f32_fixture()
    mimi_conv_fixture()
    print("wrote", sorted(p.name for p in HERE.glob("*.npz")))
