"""Pins the oracle's W8A8 path (reference: minimindo_audio_encoder.c:138-306) against the
reference's own compiled C (live via oracle/_ref where built, golden vectors elsewhere), plus
integer brute force and the closed forms of the activation quantizer."""
from pathlib import Path

import numpy as np
import pytest

GOLDEN = Path(__file__).resolve().parent / "golden" / "w8a8_minimindo.npz"


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN, allow_pickle=False)


def test_quantize_i8_matches_reference_golden(oracle, golden):
    q, scales = oracle.quantize_i8(golden["x"])
    assert np.array_equal(q, golden["q"])
    assert np.array_equal(scales.view(np.uint32), golden["scales"].view(np.uint32))
    assert scales[2] == 0.0 and not q[2].any()          # all-zero token
    assert q[3, 6] == 127 and q[3, 7] == -127           # +-max -> +-127
    assert list(q[3, :6]) == [0, 2, 2, 0, -2, -2]       # x*inv = .5, 1.5, 2.5: ties to even


def test_linear_matches_reference_golden_bitwise(oracle, golden):
    N, K = golden["w"].shape
    for bias, key in ((golden["bias"], "out_bias"), (None, "out_nobias")):
        out, acc = oracle.w8a8_linear(golden["rows"], N, K, golden["q"], golden["scales"], bias, threads=2)
        assert np.array_equal(acc, golden["dots"])
        assert np.array_equal(out.view(np.uint32), golden[key].view(np.uint32))


def test_int32_accumulators_equal_integer_matmul(oracle, golden):
    N, K = golden["w"].shape
    w8 = golden["rows"].reshape(N, 4 + K)[:, 4:].view(np.int8).astype(np.int64)
    expect = golden["q"].astype(np.int64) @ w8.T
    assert np.array_equal(golden["dots"].astype(np.int64), expect)
    # K = 1024 worst case stays inside int32 and inside fp32's exact integers
    assert 127 * 127 * 1024 < 2 ** 24


def test_live_reference_build(oracle):
    ref = oracle.ref_minimindo()
    if ref is None:
        pytest.skip("oracle/_ref not built here (the reference tree is absent)")
    rng = np.random.default_rng(21)
    M, K, N = 9, 1024, 48
    x = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    q, scales = oracle.quantize_i8(x)
    for m in range(M):
        qr = np.empty(K, dtype=np.int8)
        s = ref.ref_minimindo_quantize_i8(x[m].ctypes.data, qr.ctypes.data, K)
        assert np.array_equal(qr, q[m]) and np.float32(s) == scales[m]
    rows = oracle.q8_weight_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    bias = rng.standard_normal(N).astype(np.float32)
    expect = np.empty((M, N), dtype=np.float32)
    ref.ref_minimindo_matrix_sequence_i8_quantized(rows.ctypes.data, N, K, q.ctypes.data,
                                                   scales.ctypes.data, M, expect.ctypes.data,
                                                   bias.ctypes.data)
    out, _ = oracle.w8a8_linear(rows, N, K, q, scales, bias)
    assert np.array_equal(out.view(np.uint32), expect.view(np.uint32))


Q8_PAYLOAD_CASES = ("normal", "ties", "halves", "wide")


@pytest.mark.parametrize("case", Q8_PAYLOAD_CASES)
def test_weight_quantizer_matches_reference_payload_bytes(oracle, engine, case):
    """orc_q8_weight_quantize and the library's host quantizer mi355q_quantize_w8_rows against the
    record bytes the reference's own q8_payload produced (compile_minimindo_sensevoice_image.py:
    38-46; tests/golden/q8_payload.npz, written by make_q8_payload_fixture.py): N(0,0.02) rows with
    an all-zero and a constant row, quotients on and one float32 step beside every .5, exact
    halves at scale 1, and row maxima from 1e-30 to 1e30 with subnormal entries.  Byte for byte."""
    golden = np.load(GOLDEN.with_name("q8_payload.npz"), allow_pickle=False)
    w, records = golden[f"{case}_w"], golden[f"{case}_records"]
    N, K = w.shape
    assert np.array_equal(oracle.q8_weight_quantize(w).reshape(-1), records)
    mine = np.empty(N * (4 + K), dtype=np.uint8)
    status = engine.library().mi355q_quantize_w8_rows(w.ctypes.data, N, K, mine.ctypes.data)
    assert status == 0 and np.array_equal(mine, records)


def test_reference_payload_fixture_tells_plausible_mistakes_apart():
    """The fixture is only a pin if the likely wrong restatements disagree with it somewhere:
    multiplying by 1/scale instead of dividing, rounding halves away from zero and dividing in
    double each differ from the recorded bytes.  (max/127 computed in float32 or in double and
    then rounded cannot differ: 1/127 has a binary period of seven bits, so no quotient of a
    24-bit maximum sits close enough to a float32 midpoint for the second rounding to matter.)"""
    golden = np.load(GOLDEN.with_name("q8_payload.npz"), allow_pickle=False)
    wrong = {"reciprocal": 0, "half_away": 0, "double_division": 0}
    for case in Q8_PAYLOAD_CASES:
        w = golden[f"{case}_w"]
        N, K = w.shape
        records = golden[f"{case}_records"].reshape(N, 4 + K)
        scale = records[:, :4].copy().view(np.float32).reshape(N)
        q = records[:, 4:].view(np.int8)
        maximum = np.abs(w).max(axis=1)
        with np.errstate(all="ignore"):
            wrong["reciprocal"] += int((np.clip(np.rint(w * (np.float32(1) / scale)[:, None]), -127, 127) != q).sum())
            away = np.sign(w) * np.floor(np.abs(w / scale[:, None]) + np.float32(0.5))
            wrong["half_away"] += int((np.clip(away, -127, 127) != q).sum())
            in_double = np.rint(w.astype(np.float64) / (maximum.astype(np.float64) / 127.0)[:, None])
            wrong["double_division"] += int((np.clip(np.nan_to_num(in_double), -127, 127) != q).sum())
    assert all(count > 0 for count in wrong.values()), wrong


def test_q8rows_f32_matches_reference_golden_bitwise(oracle):
    """orc_q8rows_f32_linear against the reference's own q8_matvec / q8_matmul_sequence
    (minimindo_thinker.c:181-213, compiled from where it lies; golden vectors committed), bit
    for bit, and live against oracle/_ref where that is built."""
    golden = np.load(GOLDEN.with_name("q8rows_f32_thinker.npz"), allow_pickle=False)
    M, K = golden["x"].shape
    N = golden["out"].shape[1]
    out = oracle.q8rows_f32_linear(golden["rows"], N, K, golden["x"])
    assert np.array_equal(out.view(np.uint32), golden["out"].view(np.uint32))
    one = oracle.q8rows_f32_linear(golden["rows"], N, K, golden["x"][1:2])
    assert np.array_equal(one.view(np.uint32), golden["out_one"].view(np.uint32))
    assert not out[:, 5].any()  # the all-zero row
    ref = oracle.ref_thinker()
    if ref is not None:
        rng = np.random.default_rng(5)
        w = (rng.standard_normal((24, 128)) * 0.02).astype(np.float32)
        rows = oracle.q8_weight_quantize(w)
        x = rng.standard_normal((5, 128)).astype(np.float32)
        live = np.empty((5, 24), dtype=np.float32)
        ref.ref_thinker_q8_matmul_sequence(rows.ctypes.data, 24, 128, x.ctypes.data, 5, live.ctypes.data)
        assert np.array_equal(oracle.q8rows_f32_linear(rows, 24, 128, x).view(np.uint32), live.view(np.uint32))


def test_mimi_stream_conv_matches_reference_golden_bitwise(oracle):
    """orc_causal_q8_windows + orc_w8a8_conv against the reference's own causal_q8_windows and
    stream_conv1d (minimindo_mimi.c:552-598,869-917; golden vectors of consecutive stream
    chunks, committed), bit for bit; the pair windows of the transposed convolution against a
    direct numpy construction."""
    golden = np.load(GOLDEN.with_name("mimi_stream_conv.npz"), allow_pickle=False)
    for tag, chunks in (("k7", 3), ("k1", 1)):
        C, O, kernel = (int(v) for v in golden[f"{tag}_shape"])
        for index in range(chunks):
            x = golden[f"{tag}_{index}_x"]
            history = golden[f"{tag}_{index}_history_before"] if kernel > 1 else None
            q, scales = oracle.causal_q8_windows(x, history, kernel)
            assert np.array_equal(q, golden[f"{tag}_{index}_q"])
            assert np.array_equal(scales.view(np.uint32), golden[f"{tag}_{index}_scales"].view(np.uint32))
            y = oracle.w8a8_conv(golden[f"{tag}_rows"], O, C * kernel, q, scales, golden[f"{tag}_bias"])
            assert np.array_equal(y.view(np.uint32), golden[f"{tag}_{index}_y"].view(np.uint32))
    rng = np.random.default_rng(8)
    x = rng.standard_normal((6, 5)).astype(np.float32)
    history = rng.standard_normal(6).astype(np.float32)
    q, scales = oracle.causal_q8_windows(x, history, 0, pairs=True)
    previous = np.concatenate([history[:, None], x[:, :-1]], axis=1)
    windows = np.concatenate([x.T, previous.T], axis=1)
    expect_q, expect_scales = oracle.quantize_i8(windows)
    assert np.array_equal(q, expect_q) and np.array_equal(scales, expect_scales)
