"""The reference's own known-answer inputs through the GPU path (C ABI), gated on the oracle.

The reference's benchmarks build their matrices and activations from closed formulas and check
their GPU kernels against scalar C on them (qwen38_m3.m:64-87,567-580,753-763;
minimax_h3_m3_gemm.m:75-104, recorded max error 0.0025806427 on O(1) outputs,
models/minimax-h3/targets/apple-m3-pro/results.json:210).  These inputs differ in kind from the
N(0, 0.02) synthetic weights of the other tests: uniformly random codes, scales of 0.0035-0.0277
and biases near -7.5 scales, activations that are smooth (sin/cos) or take 17 values.
"""
import numpy as np
import pytest

import recipes
from conftest import bf16_bits, q4_relative_error

pytestmark = pytest.mark.gpu


def check(y, ref, tolerance=1e-3):
    y = np.asarray(y, dtype=np.float64)
    assert np.all(np.isfinite(y))
    error = q4_relative_error(y, ref)
    assert error <= tolerance, f"relative error {error:.3e}"
    return error


@pytest.mark.parametrize("name,N,K", [("gate", 17408, 5120), ("up", 17408, 5120), ("down", 5120, 17408)])
def test_qwen38_recipe_decode(engine, oracle, gpu, name, N, K):
    """M = 1 (the reference checks its GEMV kernels on exactly this, 8 rows; here every row):
    exact weights, fp16 activation, fp32 out; then the fp16 output the bench configuration uses."""
    quants, meta = recipes.qwen38_weights(oracle, recipes.QWEN38_SEEDS[name], N, K)
    x = recipes.qwen38_activation(1, K)
    weight = gpu.q4_prepare(quants, meta, None, N, K, engine.META_F16_INTERLEAVED)
    try:
        print(f"qwen38 recipe {name} M=1", flush=True)
        y32 = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        y16 = gpu.q4_linear(weight, x, engine.F16, engine.F16)
    finally:
        weight.destroy()
    ref = oracle.q4_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x, oracle.X_F16, 1)
    check(y32, ref)
    check(y16, ref)
    # the reference's own loop (sequential fp32) on its eight checked rows agrees to its recorded scale
    lib = oracle.lib()
    for row in range(8):
        one = lib.orc_q4_dot_f16x_seq(quants.ctypes.data, meta.ctypes.data, x.ctypes.data, row, K // 64)
        assert abs(one - float(y32[0, row])) <= 2.6e-3


@pytest.mark.parametrize("M", [2, 8, 32])
def test_qwen38_recipe_batches(engine, oracle, gpu, M):
    """The gate matrix against M rows of the activation formula: the verify kernel (exact
    weights) for M <= 16 and the GEMM (weights rounded to fp16) at M = 32."""
    N, K = 17408, 5120
    quants, meta = recipes.qwen38_weights(oracle, recipes.QWEN38_SEEDS["gate"], N, K)
    x = recipes.qwen38_activation(M, K)
    weight = gpu.q4_prepare(quants, meta, None, N, K, engine.META_F16_INTERLEAVED)
    try:
        print(f"qwen38 recipe gate M={M}", flush=True)
        y = gpu.q4_linear(weight, x, engine.F16, engine.F32)
    finally:
        weight.destroy()
    rounding = oracle.W_ROUND_F16 if M > 16 else oracle.W_EXACT
    ref = oracle.q4_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x, oracle.X_F16, M,
                           weight_rounding=rounding)
    check(y, ref)


def test_h3_recipe_decode_and_projection(engine, oracle, gpu):
    """The H3 closed-form GEMM, K = 5376 (an odd number of 128-column steps: 42), N = 14336:
    M = 1 with fp32 input and output, and M = 32 with bf16 input and output as
    minimax_h3_m3_run_q4_projection_bf16 takes them (minimax_h3_m3_gemm.h:58-66), against the
    oracle's fp16-weight flavour, which is how the reference's own check evaluates the weight
    (gemm_reference, minimax_h3_m3_gemm.m:87-104)."""
    N, K = recipes.H3_N, recipes.H3_K
    quants, meta = recipes.h3_weights()
    weight = gpu.q4_prepare(quants, meta, None, N, K, engine.META_F16_INTERLEAVED)
    try:
        x1 = recipes.h3_input(1)
        print("h3 recipe M=1", flush=True)
        y1 = gpu.q4_linear(weight, x1, engine.F32, engine.F32)
        x32 = recipes.h3_input(32)
        print("h3 recipe M=32 bf16", flush=True)
        y32 = gpu.q4_linear(weight, bf16_bits(x32).reshape(32, K), engine.BF16, engine.BF16)
    finally:
        weight.destroy()
    exact = oracle.q4_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x1, oracle.X_F32, 1)
    check(y1, exact)
    # the reference's scalar check on its first eight rows: fp16 weight, sequential fp32; the
    # exact-weight GPU result sits within the error the reference recorded for its own kernel
    seq = oracle.q4_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x1, oracle.X_F32, 1,
                           weight_rounding=oracle.W_ROUND_F16, accumulate=oracle.ACC_F32_SEQUENTIAL,
                           rows=(0, 8))[:, :8]
    assert float(np.max(np.abs(seq - y1[:, :8]))) <= 2 * 0.0025806427
    rounded = oracle.q4_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x32, oracle.X_F32, 32,
                               weight_rounding=oracle.W_ROUND_F16)
    got = (y32.astype(np.uint32) << 16).view(np.float32)
    check(got, rounded, tolerance=2.0 ** -8)  # bf16 output rounding dominates
