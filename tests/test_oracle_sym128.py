"""Pins the oracle's symmetric group-128 Q4 path (reference: qwen35_task.c:286-362,426-450)
against the reference's own compiled C: live through oracle/_ref where it was built, and through
the golden vectors that build wrote (tests/golden/sym128_q4_gemv.npz) everywhere else.  Also the
layout property the reference's own unit test asserts (tests/test_q4_output_block.py) and the
lossless re-expression as affine group-64."""
from pathlib import Path

import numpy as np
import pytest

from sym128 import output_block, pack_sym128

GOLDEN = Path(__file__).resolve().parent / "golden" / "sym128_q4_gemv.npz"


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN, allow_pickle=False)


def test_gemv_matches_reference_golden_bitwise(oracle, golden):
    rows, cols = golden["weights"].shape
    for name, flag in (("rowmajor", 0), ("blocked", 1)):
        data = golden["records"] if flag == 0 else golden["blocked"]
        y = oracle.sym128_gemv(data, flag, rows, cols, golden["x"], threads=2)
        assert np.array_equal(y.view(np.uint32), golden[f"y_{name}"].view(np.uint32)), name
        for r in range(rows):
            out = np.empty(cols, dtype=np.float32)
            oracle.lib().orc_sym128_dequantize_row(data.ctypes.data, flag, cols, r, out.ctypes.data)
            assert np.array_equal(out.view(np.uint32), golden[f"dequant_{name}"][r].view(np.uint32))
    # both record orders describe the same matrix
    assert np.array_equal(golden["y_rowmajor"], golden["y_blocked"])


def test_gemv_matches_live_reference_build(oracle):
    ref = oracle.ref_qwen35()
    if ref is None:
        pytest.skip("oracle/_ref not built here (the reference tree is absent)")
    rng = np.random.default_rng(11)
    for rows, cols in ((4, 128), (16, 1024), (40, 640)):
        records = pack_sym128(rng.standard_normal((rows, cols)).astype(np.float32) * 0.03)
        x = rng.standard_normal(cols).astype(np.float32)
        for flag, data in ((0, records.reshape(-1)), (1, output_block(records, 4))):
            expect = np.empty(rows, dtype=np.float32)
            ref.ref_qwen35_q4_gemv(data.ctypes.data, flag, rows, cols, x.ctypes.data, expect.ctypes.data)
            got = oracle.sym128_gemv(data, flag, rows, cols, x)
            assert np.array_equal(got.view(np.uint32), expect.view(np.uint32))


def test_output_block_layout_as_in_reference_unit_test():
    """weights and expected permutation of tests/test_q4_output_block.py:19-31."""
    values = np.arange(8 * 256, dtype=np.float32).reshape(8, 256)
    records = pack_sym128(np.sin(values * np.float32(0.017)))
    blocked = output_block(records, 4)
    expected = records.reshape(2, 4, 2, 66).transpose(0, 2, 1, 3)
    assert np.array_equal(blocked.reshape(2, 2, 4, 66), expected)
    with pytest.raises(ValueError):
        output_block(records[:6], 4)


def test_dequantized_row_reproduces_gemv(oracle, golden):
    """dequantize_q4_row is the round trip the runtime itself uses (qwen35_task.c:426-450):
    x . dequant(row) must equal the GEMV up to the order of the fp32 sums."""
    dq = golden["dequant_rowmajor"].astype(np.float64)
    expect = dq @ golden["x"].astype(np.float64)
    assert np.allclose(golden["y_rowmajor"], expect, rtol=0, atol=2e-5)
    # and the quantizer's error stays below half a step of each group's (bf16-rounded) scale
    w = golden["weights"]
    records = golden["records"].reshape(w.shape[0], -1, 66)
    scale_bits = records[..., 0].astype(np.uint32) | (records[..., 1].astype(np.uint32) << 8)
    scale = (scale_bits << 16).view(np.float32).astype(np.float64)
    step = np.repeat(scale, 128, axis=1)
    assert np.all(np.abs(dq - w) <= step * (0.5 + 8 * 2.0 ** -8) + 1e-9)


def test_sym128_to_affine_is_lossless(oracle, golden):
    rows, cols = golden["weights"].shape
    for flag, data in ((0, golden["records"]), (1, golden["blocked"])):
        quants, scales, biases = oracle.sym128_to_affine(data, flag, rows, cols)
        x = golden["x"].reshape(1, cols)
        affine = oracle.q4_linear(quants, scales, biases, oracle.META_BF16_PLANES, rows, cols, x,
                                  oracle.X_F32, 1)
        exact = golden["dequant_rowmajor"].astype(np.float64) @ golden["x"].astype(np.float64)
        assert np.allclose(affine[0], exact, rtol=1e-13, atol=1e-13)


def test_batched_form_with_bias(oracle, golden):
    rows, cols = golden["weights"].shape
    rng = np.random.default_rng(5)
    batch = rng.standard_normal((3, cols)).astype(np.float32)
    bias = rng.standard_normal(rows).astype(np.float32)
    out = np.empty((3, rows), dtype=np.float32)
    records = golden["records"]  # keep the array alive while C reads it
    oracle.lib().orc_sym128_gemm(records.ctypes.data, batch.ctypes.data, 3, cols, rows,
                                 bias.ctypes.data, out.ctypes.data, 2)
    expect = batch.astype(np.float64) @ golden["dequant_rowmajor"].astype(np.float64).T + bias
    assert np.allclose(out, expect, atol=3e-5)
