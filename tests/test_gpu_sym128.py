"""GPU parity of the symmetric group-128 Q4 path (66-byte records of compiler/q4_image.py, read by
q4_gemv, qwen35_task.c:318-362, and by whisper's grouped linear, whisper_turbo_encoder.c:127-176):
prepare-time mapping to the affine layout, and the two entry points that carry the reference's
hook signatures.

Truth is the exact dequantized matrix (bf16 scale times the integer code, exact in fp32) multiplied
in float64; the oracle's fp32 restatement of the reference loop and the golden vectors written by
the reference's own C are compared against the same truth on the same metric.
Gate: max_i |y_i - ref_i| / max(|ref_i|, 1e-2*rms(ref)) <= 1e-3.
"""
from pathlib import Path

import numpy as np
import pytest

from conftest import q4_relative_error
from sym128 import output_block, pack_sym128

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-3
GOLDEN = Path(__file__).resolve().parent / "golden" / "sym128_q4_gemv.npz"


def dequantized(oracle, records, order, N, K):
    out = np.empty((N, K), dtype=np.float32)
    for row in range(N):
        oracle.lib().orc_sym128_dequantize_row(records.ctypes.data, int(order), K, row,
                                               out[row].ctypes.data)
    return out.astype(np.float64)


def test_golden_vectors_of_the_reference_build(engine, oracle, gpu):
    """The fixture holds what the reference's own q4_gemv returned for both record orders."""
    golden = np.load(GOLDEN, allow_pickle=False)
    N, K = golden["weights"].shape
    x = golden["x"]
    for name, order in (("rowmajor", engine.SYM128_ROW_MAJOR), ("blocked", engine.SYM128_OUTPUT_BLOCKED)):
        records = golden["records"] if order == engine.SYM128_ROW_MAJOR else golden["blocked"]
        weight = gpu.sym128_prepare(records, N, K, order)
        try:
            print(f"sym128 golden {name}", flush=True)
            y = gpu.q4_linear(weight, x[None, :], engine.F32, engine.F32)[0]
        finally:
            weight.destroy()
        truth = golden[f"dequant_{name}"].astype(np.float64) @ x.astype(np.float64)
        assert q4_relative_error(y, truth) <= TOLERANCE
        # the reference's fp32 loop and this kernel differ from each other by rounding only
        assert q4_relative_error(y, golden[f"y_{name}"].astype(np.float64)) <= TOLERANCE


@pytest.mark.parametrize("N,K,M", [(3584, 1024, 1), (248, 2560, 1), (100, 128, 3), (1024, 1024, 8),
                                   (640, 1280, 40)])
@pytest.mark.parametrize("order", [0, 1])
def test_prepare_and_linear(engine, oracle, gpu, N, K, M, order):
    """Config-1 shape (K=1024, N=3584, M=1) and ragged ones, both record orders, fp32 in and out;
    M=40 takes the matrix-instruction GEMM.  Its weights are fp16(scale * v): exact for these
    records (a bf16 scale times an integer of at most three bits fits fp16's eleven), and fp32
    activations go in as (value, remainder) pairs, so the exact product is the truth at every M."""
    rng = np.random.default_rng(N + K + M)
    grid = pack_sym128(rng.standard_normal((N, K)).astype(np.float32) * 0.03)
    records = output_block(grid, 4) if order else np.ascontiguousarray(grid).reshape(-1)
    x = rng.standard_normal((M, K)).astype(np.float32)
    weight = gpu.sym128_prepare(records, N, K, order)
    try:
        print(f"sym128 case N={N} K={K} M={M} order={order}", flush=True)
        assert engine.library().mi355q_q4_weight_image_bytes(weight.handle) == records.size
        y = gpu.q4_linear(weight, x, engine.F32, engine.F32)
    finally:
        weight.destroy()
    w = dequantized(oracle, records, order, N, K)
    truth = x.astype(np.float64) @ w.T
    assert q4_relative_error(y, truth) <= TOLERANCE
    if M == 1:
        restated = oracle.sym128_gemv(records, order, N, K, x[0])
        assert q4_relative_error(y[0], restated.astype(np.float64)) <= TOLERANCE


def test_prepare_rejects_bad_shapes(engine, gpu):
    records = np.zeros(66 * 8, dtype=np.uint8)
    for N, K, order in ((4, 192, 0), (0, 128, 0), (6, 128, 1), (4, 128, 7)):
        with pytest.raises(engine.Mi355qError) as info:
            gpu.sym128_prepare(records, N, K, order)
        assert info.value.status == engine.ERROR_INVALID


@pytest.mark.parametrize("rows", [1, 5, 64])
def test_bias_row_through_the_residual(engine, oracle, gpu, rows):
    """MI355Q_RESIDUAL_IS_BIAS adds one row [N] to every output row, on the streaming kernel
    (rows 1 and 5) and on the GEMM (64 rows)."""
    N, K = 200, 512
    quants, meta_a, meta_b = engine.synth_q4_affine(3, 0.02, N, K, engine.META_BF16_PLANES)
    x = np.stack([engine.synth_normal_f16(11 + r, 1.0, K) for r in range(rows)])
    bias = engine.synth_normal_f32(5, 1.0, N)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        print(f"bias case rows={rows}", flush=True)
        plain = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        biased = gpu.q4_linear(weight, x, engine.F16, engine.F32, bias, engine.F32, residual_is_bias=True)
    finally:
        weight.destroy()
    assert np.array_equal(biased, plain + bias[None, :])


def test_hook_signatures(engine, oracle, gpu):
    """mi355q_hook_q4_gemm / _gemv: raw record pointer per call, host fp32 in and out, weights
    prepared once per pointer; compared with the oracle's restatement of linear_grouped and q4_gemv."""
    rng = np.random.default_rng(12)
    N, K = 384, 1280
    grid = pack_sym128(rng.standard_normal((N, K)).astype(np.float32) * 0.03)
    records = np.ascontiguousarray(grid).reshape(-1)
    blocked = output_block(grid, 4)
    bias = rng.standard_normal(N).astype(np.float32)
    try:
        for rows in (1, 6, 150):
            x = rng.standard_normal((rows, K)).astype(np.float32)
            print(f"hook gemm rows={rows}", flush=True)
            expect = np.empty((rows, N), dtype=np.float32)
            oracle.lib().orc_sym128_gemm(records.ctypes.data, x.ctypes.data, rows, K, N, bias.ctypes.data,
                                         expect.ctypes.data, 2)
            got = engine.hook_q4_gemm(records, x, N, bias)
            again = engine.hook_q4_gemm(records, x, N, None)  # cached weight, no bias
            assert np.array_equal(got, again + bias[None, :])
            # (more than 8 fp32 rows take the matrix-instruction GEMM: fp32 rows as (value, remainder)
            # pairs, weights fp16(scale * v), which is exact for these records: the same gate)
            assert q4_relative_error(got, expect.astype(np.float64)) <= TOLERANCE
        x = rng.standard_normal(K).astype(np.float32)
        for order, data in ((engine.SYM128_ROW_MAJOR, records), (engine.SYM128_OUTPUT_BLOCKED, blocked)):
            print(f"hook gemv order={order}", flush=True)
            got = engine.hook_q4_gemv(data, order, N, x)
            expect = oracle.sym128_gemv(data, order, N, K, x)
            assert q4_relative_error(got, expect.astype(np.float64)) <= TOLERANCE
        with pytest.raises(engine.Mi355qError) as info:
            engine.hook_q4_gemv(records, 0, N, np.zeros(K + 64, dtype=np.float32))
        assert info.value.status == engine.ERROR_INVALID
    finally:
        engine.hook_release()
