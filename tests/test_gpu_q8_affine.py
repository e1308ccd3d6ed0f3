"""GPU parity of the affine-Q8 g64 linear (one Q4 weight of twice the columns, mi355q_q8_linear) against the oracle.

Format and reference arithmetic: minimax_h3_q8_gemm_bf16_meta (minimax_h3_attention.metal:594-676),
u8 quants[N][K], bf16 scales/biases [N][K/64], weight = scale * q + bias.
Gate for M <= 16 (weights kept exact): max_i |y_i - ref_i| / max(|ref_i|, 1e-2*rms(ref)) <= 1e-3
against the exact weight with double accumulation.  The GEMM path (M > 16) has two forms.  When the
columns are whole 128-column steps, a kernel multiplies the bytes themselves with the weight rounded
as the reference rounds it, half(scale*q+bias): gate max_i |y_i - ref_i| <= 1e-5 * rms(ref) against
the oracle with that rounding (what is left is the order of the fp32 additions and the rare double
rounding of the reference's fp32 multiply-add).  Otherwise, and under option q8_gemm=doubled, the Q4
kernels run on the doubled weight and round the two nibble halves of a weight to fp16 separately:
within fp16 rounding of the exact weight but not of the reference's rounding, so the gate there is the
distance to the exact-weight result, max_i |y_i - ref_i| <= 2e-3 * rms(ref) (the bound the Q4 GEMM
tests report for fp16-rounded weights), with the reference's own rounding held to the same bound for
comparison."""
import numpy as np
import pytest

from conftest import bf16_bits, q4_relative_error

pytestmark = pytest.mark.gpu


def make_q8(engine, seed, N, K, meta_kind):
    """Seeded N(0, 0.02) weights, min/max affine 8-bit per group of 64 (metadata rounded first)."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K // 64, 64)) * 0.02).astype(np.float32)
    lo, hi = w.min(axis=2), w.max(axis=2)
    scale = np.where(hi > lo, (hi - lo) / 255.0, 1.0).astype(np.float32)
    if meta_kind == engine.META_BF16_PLANES:
        scale_bits, bias_bits = bf16_bits(scale), bf16_bits(lo)
        scale_r = (scale_bits.astype(np.uint32) << 16).view(np.float32)
        bias_r = (bias_bits.astype(np.uint32) << 16).view(np.float32)
        meta_a, meta_b = scale_bits.reshape(-1), bias_bits.reshape(-1)
    else:
        scale_r, bias_r = scale.astype(np.float16).astype(np.float32), lo.astype(np.float16).astype(np.float32)
        meta_a = np.stack([scale_r.astype(np.float16).view(np.uint16), bias_r.astype(np.float16).view(np.uint16)],
                          axis=-1).reshape(-1)
        meta_b = None
    q = np.clip(np.rint((w - bias_r[..., None]) / scale_r[..., None]), 0, 255).astype(np.uint8)
    return np.ascontiguousarray(q.reshape(-1)), np.ascontiguousarray(meta_a), meta_b


@pytest.mark.parametrize("N,K,M,meta", [(100, 192, 1, "META_BF16_PLANES"), (256, 1024, 1, "META_F16_INTERLEAVED"),
                                        (1024, 3072, 4, "META_BF16_PLANES"), (320, 8704, 8, "META_BF16_PLANES"),
                                        (528, 1536, 64, "META_BF16_PLANES"), (1088, 640, 200, "META_F16_INTERLEAVED"),
                                        # K not a whole number of 128-column steps: the rows are written twice first
                                        (272, 320, 40, "META_BF16_PLANES"),
                                        # long rows, K splits: the activation row starts over inside a split
                                        (560, 2176, 150, "META_BF16_PLANES"),
                                        # one tile and one step; a ragged second tile under many row blocks
                                        (16, 128, 17, "META_F16_INTERLEAVED"), (17, 256, 1000, "META_BF16_PLANES")])
def test_q8_affine_linear(engine, oracle, gpu, force, N, K, M, meta):
    meta_kind = getattr(engine, meta)
    quants, meta_a, meta_b = make_q8(engine, 3, N, K, meta_kind)
    x = np.stack([engine.synth_normal_f32(70 + m, 1.0, K) for m in range(M)]).astype(np.float16)
    residual = engine.synth_normal_f32(99, 1.0, M * N).reshape(M, N)
    weight = gpu.q8_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"q8 affine N={N} K={K} M={M} meta={meta}", flush=True)
        assert engine.library().mi355q_q8_weight_image_bytes(weight) == N * K + N * (K // 64) * 4
        y = gpu.q8_linear(weight, N, x, engine.F16, engine.F32)
        y16 = gpu.q8_linear(weight, N, x, engine.F16, engine.F16)
        with_residual = gpu.q8_linear(weight, N, x, engine.F16, engine.F32, residual, engine.F32)
        force("q8_gemm", "doubled")
        doubled = gpu.q8_linear(weight, N, x, engine.F16, engine.F32)
    finally:
        gpu.q8_destroy(weight)
    exact = oracle.q8_affine_linear(quants, meta_a, meta_b, meta_kind, N, K, x, engine.F16, M)
    if M <= 16:
        assert q4_relative_error(y, exact) <= 1e-3
        assert q4_relative_error(y16, exact) <= 1e-3
        assert q4_relative_error(with_residual, exact + residual) <= 1e-3
    else:
        rounded = oracle.q8_affine_linear(quants, meta_a, meta_b, meta_kind, N, K, x, engine.F16, M,
                                          weight_rounding=oracle.W_ROUND_F16)
        rms = np.sqrt(np.mean(exact * exact, axis=1, keepdims=True))
        ours = float(np.max(np.abs(y - exact) / rms))
        theirs = float(np.max(np.abs(rounded - exact) / rms))
        on_doubled = float(np.max(np.abs(doubled - exact) / rms))
        to_theirs = float(np.max(np.abs(y - rounded) / rms))
        print(f"distance to exact weights / rms: this library {ours:.2e} (doubled weight {on_doubled:.2e}), "
              f"half(scale*q+bias) {theirs:.2e}; this library to half(scale*q+bias) {to_theirs:.2e}", flush=True)
        assert ours <= 2e-3 and theirs <= 2e-3 and on_doubled <= 2e-3
        assert float(np.max(np.abs(with_residual - (exact + residual)) / rms)) <= 2e-3
        if K % 128 == 0:  # the kernel on the bytes themselves: the reference's own rounding of a weight
            assert to_theirs <= 1e-5
            assert float(np.max(np.abs(y16 - rounded) / rms)) <= 2e-3  # fp16 outputs
            assert float(np.max(np.abs(with_residual - (rounded + residual)) / rms)) <= 1e-5
        else:
            assert np.array_equal(y, doubled)


def test_q8rows_f32_against_reference_golden(engine, oracle, gpu):
    """Q8 rows x fp32 activations (mi355q_q8rows_weight_prepare + mi355q_q8_linear) against the
    golden vectors of the reference's own q8_matvec / q8_matmul_sequence
    (minimindo_thinker.c:181-213).  The reference adds in double and rounds once; here the
    integer-weighted sum is accumulated in fp32 from activations carried as fp16 value +
    remainder: the Q4 gate, max_i |y_i - ref_i| / max(|ref_i|, 1e-2*rms(ref)) <= 1e-3."""
    import pathlib
    golden = np.load(pathlib.Path(__file__).parent / "golden" / "q8rows_f32_thinker.npz", allow_pickle=False)
    M, K = golden["x"].shape
    N = golden["out"].shape[1]
    weight = gpu.q8rows_prepare(golden["rows"], N, K)
    try:
        print("q8 rows golden case", flush=True)
        y = gpu.q8_linear(weight, N, golden["x"], engine.F32, engine.F32)
        one = gpu.q8_linear(weight, N, golden["x"][1:2], engine.F32, engine.F32)
    finally:
        gpu.q8_destroy(weight)
    error = q4_relative_error(y, golden["out"])
    print(f"relative error vs the reference's C: {error:.2e}", flush=True)
    assert error <= 1e-3
    assert q4_relative_error(one, golden["out_one"]) <= 1e-3
    assert not y[:, 5].any()  # the all-zero row


@pytest.mark.parametrize("N,K,M", [(768, 768, 1), (2048, 768, 6), (768, 2048, 40)])
def test_q8rows_f32_shapes(engine, oracle, gpu, N, K, M):
    """MiniMind-sized projections (hidden 768) at M = 1, a short sequence, and a sequence long
    enough for the GEMM path (M > 8 rows of fp32), with a per-column bias added after the scale."""
    rng = np.random.default_rng(N + K + M)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    rows = oracle.q8_weight_quantize(w)
    x = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    weight = gpu.q8rows_prepare(rows, N, K)
    try:
        print(f"q8 rows N={N} K={K} M={M}", flush=True)
        y = gpu.q8_linear(weight, N, x, engine.F32, engine.F32)
        _call_bias = engine.library().mi355q_q8_linear
        biased = np.empty((M, N), dtype=np.float32)
        message = __import__("ctypes").create_string_buffer(256)
        status = _call_bias(gpu.handle, weight, x.ctypes.data, engine.F32, M, biased.ctypes.data, engine.F32,
                            bias.ctypes.data, engine.F32, engine.RESIDUAL_IS_BIAS, message, 256)
        assert status == 0, message.value
    finally:
        gpu.q8_destroy(weight)
    ref = oracle.q8rows_f32_linear(rows, N, K, x).astype(np.float64)
    if M <= 8:
        assert q4_relative_error(y, ref) <= 1e-3
        assert q4_relative_error(biased, ref + bias) <= 1e-3
    else:
        # the GEMM path rounds fp32 activations to fp16 once per call (2^-11 per element): the
        # gate is the distance relative to the row's rms, as for the other fp16-operand paths
        rms = np.sqrt(np.mean(ref * ref, axis=1, keepdims=True))
        assert float(np.max(np.abs(y - ref) / rms)) <= 2e-3
        assert float(np.max(np.abs(biased - (ref + bias)) / rms)) <= 2e-3


@pytest.mark.parametrize("forced", ["0,1", "2,2", "3,1", "6,1", "6,3", "7,2", "8,2"])
def test_q8_affine_under_every_gemm_kernel(engine, oracle, gpu, forced, force):
    """The activation row starts over at the weight's second half of columns in each of the three
    matrix kernels' addressing; every GEMM variant (first kernel, pipelined 16 / 17 / 20 tiles,
    with and without K splits) on a Q8 weight whose doubled row is ten steps long."""
    force("q8_gemm", "doubled")
    force("q4_gemm", forced)
    N, K, M = 560, 640, 150
    meta_kind = engine.META_BF16_PLANES
    quants, meta_a, meta_b = make_q8(engine, 11, N, K, meta_kind)
    x = np.stack([engine.synth_normal_f32(170 + m, 1.0, K) for m in range(M)]).astype(np.float16)
    weight = gpu.q8_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"q8 affine forced={forced}", flush=True)
        y = gpu.q8_linear(weight, N, x, engine.F16, engine.F32)
    finally:
        gpu.q8_destroy(weight)
    exact = oracle.q8_affine_linear(quants, meta_a, meta_b, meta_kind, N, K, x, engine.F16, M)
    rms = np.sqrt(np.mean(exact * exact, axis=1, keepdims=True))
    assert float(np.max(np.abs(y - exact) / rms)) <= 2e-3


@pytest.mark.parametrize("x_type", ["F16", "BF16", "F32"])
@pytest.mark.parametrize("forced", [None, "9,1", "9,2", "9,5", "10,1", "10,3"])
def test_q8_affine_byte_kernel(engine, oracle, gpu, forced, x_type, force):
    """The GEMM kernel on the bytes themselves, with and without K splits, on a shape with a ragged
    last block of tiles (35 = 2 x 16 + 3), a ragged last block of rows (150 = 128 + 22) and a
    number of steps (17) that no split divides; fp16, bf16 and fp32 activations, fp16 metadata,
    a residual, fp16 and bf16 outputs.  Against the oracle with the reference's rounding of a
    weight, half(scale*q+bias)."""
    if forced is not None:
        force("q4_gemm", forced)
    N, K, M = 560, 2176, 150
    meta_kind = engine.META_F16_INTERLEAVED
    quants, meta_a, meta_b = make_q8(engine, 12, N, K, meta_kind)
    x32 = np.stack([engine.synth_normal_f32(270 + m, 1.0, K) for m in range(M)])
    x_dtype = getattr(engine, x_type)
    if x_type == "F16":
        x = x32.astype(np.float16)
        seen = x.astype(np.float32)
    elif x_type == "BF16":
        x = bf16_bits(x32)
        seen = (x.astype(np.uint32) << 16).view(np.float32)
    else:
        x = seen = x32
    residual = engine.synth_normal_f32(98, 1.0, M * N).reshape(M, N)
    weight = gpu.q8_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"q8 byte kernel forced={forced} x={x_type}", flush=True)
        y = gpu.q8_linear(weight, N, x, x_dtype, engine.F32)
        y16 = gpu.q8_linear(weight, N, x, x_dtype, engine.F16)
        ybf = gpu.q8_linear(weight, N, x, x_dtype, engine.BF16)
        with_residual = gpu.q8_linear(weight, N, x, x_dtype, engine.F32, residual, engine.F32)
    finally:
        gpu.q8_destroy(weight)
    rounded = oracle.q8_affine_linear(quants, meta_a, meta_b, meta_kind, N, K, seen, engine.F32, M,
                                      weight_rounding=oracle.W_ROUND_F16)
    rms = np.sqrt(np.mean(rounded * rounded, axis=1, keepdims=True))
    distance = float(np.max(np.abs(y - rounded) / rms))
    print(f"distance to the oracle with half(scale*q+bias) weights / rms: {distance:.2e}", flush=True)
    # fp16 and bf16 activations enter the matrix units exactly (bf16 after a power-of-two scaling of the
    # row); fp32 ones as fp16 value + remainder, 2^-22 relative per element
    assert distance <= 1e-5
    assert float(np.max(np.abs(with_residual - (rounded + residual)) / rms)) <= 1e-5
    assert float(np.max(np.abs(y16.astype(np.float64) - rounded) / rms)) <= 2e-3
    bf = (ybf.astype(np.uint32) << 16).view(np.float32) if ybf.dtype == np.uint16 else ybf
    assert float(np.max(np.abs(bf.astype(np.float64) - rounded) / rms)) <= 1.6e-2


def test_q8rows_byte_kernel_matches_doubled_weight(engine, oracle, gpu, force):
    """Q8 rows on the GEMM path: integer weights v = byte - 128 are exact in fp16 in both forms (the
    bytes themselves with {1, -128}; the nibble halves with {16, -128} and {1, 0}), so the two forms
    differ only in the order of the fp32 additions."""
    N, K, M = 400, 1280, 72
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    rows = oracle.q8_weight_quantize(w)
    x = rng.standard_normal((M, K)).astype(np.float16)
    weight = gpu.q8rows_prepare(rows, N, K)
    try:
        print("q8 rows, byte kernel and doubled weight", flush=True)
        native = gpu.q8_linear(weight, N, x, engine.F16, engine.F32)
        force("q8_gemm", "doubled")
        doubled = gpu.q8_linear(weight, N, x, engine.F16, engine.F32)
    finally:
        gpu.q8_destroy(weight)
    ref = oracle.q8rows_f32_linear(rows, N, K, x.astype(np.float32)).astype(np.float64)
    rms = np.sqrt(np.mean(ref * ref, axis=1, keepdims=True))
    assert float(np.max(np.abs(native - ref) / rms)) <= 5e-5
    assert float(np.max(np.abs(doubled - ref) / rms)) <= 5e-5
