"""GPU parity of the W8A8 path against the CPU oracle and the reference's golden vectors:
int8 codes, scales, int32 accumulators and fp32 outputs must all be bit-exact."""
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden" / "w8a8_minimindo.npz"


def check(engine, oracle, gpu, M, K, N, seed, bias=True):
    x = engine.synth_normal_f32(seed, 1.0, M * K).reshape(M, K)
    rows = engine.synth_w8_rows(seed + 1, 0.02, N, K)
    b = engine.synth_normal_f32(seed + 2, 1.0, N) if bias else None
    print(f"w8a8 case M={M} K={K} N={N} bias={bias}", flush=True)
    q, scales = gpu.quantize_i8(x)
    q_ref, s_ref = oracle.quantize_i8(x)
    assert np.array_equal(q, q_ref)
    assert np.array_equal(scales.view(np.uint32), s_ref.view(np.uint32))
    weight = gpu.w8a8_prepare(rows, N, K)
    try:
        out, acc = gpu.w8a8_linear(weight, N, q, scales, b)
    finally:
        gpu.w8a8_destroy(weight)
    out_ref, acc_ref = oracle.w8a8_linear(rows, N, K, q_ref, s_ref, b)
    assert acc.tobytes() == acc_ref.tobytes()          # the memcmp gate on the int32 accumulators
    assert np.array_equal(out.view(np.uint32), out_ref.view(np.uint32))


def test_config5(engine, oracle, gpu):
    """Headline configuration 5 (SenseVoice encoder projection): M=64, K=1024, N=4096."""
    check(engine, oracle, gpu, 64, 1024, 4096, 31)


@pytest.mark.parametrize("M,K,N", [(1, 16, 16), (3, 48, 20), (17, 560, 100), (40, 512, 2048),
                                   (130, 2048, 512), (64, 1024, 4100), (5, 1024, 40), (17, 3072, 1000),
                                   (33, 1024, 16400), (64, 2048, 12304)])
def test_shapes(engine, oracle, gpu, M, K, N):
    """Tile counts of 1 to 1025 (the launch takes one tile per workgroup unless option "w8a8" asks
    for more: test_tiles_per_workgroup_give_the_same_bits), K of one to three 1024-column rounds
    and ragged ones, row counts that end inside a fragment."""
    check(engine, oracle, gpu, M, K, N, 7 + M, bias=(M % 2 == 0))


@pytest.mark.parametrize("M,K,N,channel_major", [(64, 1024, 4096, False), (21, 2048, 530, True),
                                                 (9, 1024, 4100, False), (40, 560, 4100, True)])
def test_tiles_per_workgroup_give_the_same_bits(engine, oracle, gpu, force, M, K, N, channel_major):
    """One to four weight tiles per workgroup (option "w8a8"; the default launch takes one): the
    multi-tile kernels share the activation registers between their tiles and keep one partial sum
    area per tile in LDS.  Every setting gives the one-tile launch's bits and the oracle's; N = 4100
    is 257 tiles, so with two, three and four tiles a workgroup the last workgroup's tiles partly
    do not exist; M = 9, 21 and 40 fall into the one-, two- and four-fragment row blocks."""
    x = engine.synth_normal_f32(5, 1.0, M * K).reshape(M, K)
    rows = engine.synth_w8_rows(6, 0.02, N, K)
    bias = engine.synth_normal_f32(7, 1.0, N)
    q, scales = gpu.quantize_i8(x)
    weight = gpu.w8a8_prepare(rows, N, K)
    results = {}
    try:
        print(f"w8a8 tiles per workgroup M={M} K={K} N={N} channel_major={channel_major}", flush=True)
        results["default"] = gpu.w8a8_linear(weight, N, q, scales, bias, channel_major=channel_major)
        for tiles in ("1", "2", "3", "4"):
            force("w8a8", tiles)
            results[tiles] = gpu.w8a8_linear(weight, N, q, scales, bias, channel_major=channel_major)
    finally:
        gpu.w8a8_destroy(weight)
    out_ref, acc_ref = oracle.w8a8_linear(rows, N, K, q, scales, bias)
    if channel_major:
        out_ref = oracle.w8a8_conv(rows, N, K, q, scales, bias)
    assert np.any(acc_ref != 0)
    for name, (out, acc) in results.items():
        assert acc.tobytes() == acc_ref.tobytes(), name
        assert np.array_equal(out.view(np.uint32), out_ref.view(np.uint32)), name


@pytest.mark.parametrize("tiles", ["2", "3", "4"])
def test_shared_activation_launch_with_several_tiles_per_workgroup(engine, oracle, gpu, force, tiles):
    """Three weights in one launch (workgroup ranges map to weights) with several tiles per
    workgroup: the first workgroup of a weight starts at that weight's first tile whatever the
    tile counts in front of it (here 257, 7 and 33 tiles)."""
    M, K, widths = 23, 560, (4100, 100, 528)
    x = engine.synth_normal_f32(171, 1.0, M * K).reshape(M, K)
    q, scales = oracle.quantize_i8(x)
    rows = [engine.synth_w8_rows(180 + i, 0.02, N, K) for i, N in enumerate(widths)]
    biases = [engine.synth_normal_f32(190 + i, 1.0, N) for i, N in enumerate(widths)]
    weights = [gpu.w8a8_prepare(r, N, K) for r, N in zip(rows, widths)]
    try:
        print(f"w8a8 shared activation, {tiles} tiles per workgroup", flush=True)
        force("w8a8", tiles)
        results = gpu.w8a8_linear_multi(weights, widths, q, scales, biases)
    finally:
        for weight in weights:
            gpu.w8a8_destroy(weight)
    for i, N in enumerate(widths):
        out_ref, acc_ref = oracle.w8a8_linear(rows[i], N, K, q, scales, biases[i])
        assert results[i][1].tobytes() == acc_ref.tobytes()
        assert np.array_equal(results[i][0].view(np.uint32), out_ref.view(np.uint32))


def test_reference_golden_vectors(engine, gpu):
    g = np.load(GOLDEN, allow_pickle=False)
    x, rows, bias = g["x"], g["rows"], g["bias"]
    N, K = g["w"].shape
    q, scales = gpu.quantize_i8(x)
    assert np.array_equal(q, g["q"]) and np.array_equal(scales.view(np.uint32), g["scales"].view(np.uint32))
    weight = gpu.w8a8_prepare(rows, N, K)
    try:
        out, acc = gpu.w8a8_linear(weight, N, q, scales, bias)
        out2, _ = gpu.w8a8_linear(weight, N, q, scales, None)
    finally:
        gpu.w8a8_destroy(weight)
    assert np.array_equal(acc, g["dots"])
    assert np.array_equal(out.view(np.uint32), g["out_bias"].view(np.uint32))
    assert np.array_equal(out2.view(np.uint32), g["out_nobias"].view(np.uint32))


def test_saturating_inputs_keep_int32_exact(engine, oracle, gpu):
    """+-127 codes against +-127 weights at K=2048: |acc| = 33,032,192 > 2^24, still exact in int32."""
    M, K, N = 16, 2048, 32
    x = np.ones((M, K), dtype=np.float32)
    x[1::2] *= -1
    w = np.ones((N, K), dtype=np.float32) * 0.5
    w[::3] *= -1
    rows = np.empty(N * (4 + K), dtype=np.uint8)
    assert engine.library().mi355q_quantize_w8_rows(w.ctypes.data, N, K, rows.ctypes.data) == 0
    q, scales = gpu.quantize_i8(x)
    assert set(np.unique(q)) == {-127, 127}
    weight = gpu.w8a8_prepare(rows, N, K)
    try:
        out, acc = gpu.w8a8_linear(weight, N, q, scales, None)
    finally:
        gpu.w8a8_destroy(weight)
    assert np.max(np.abs(acc)) == 127 * 127 * K
    out_ref, acc_ref = oracle.w8a8_linear(rows, N, K, q, scales, None)
    assert np.array_equal(acc, acc_ref) and np.array_equal(out.view(np.uint32), out_ref.view(np.uint32))


def test_argument_errors(engine, gpu):
    rows = engine.synth_w8_rows(1, 0.02, 16, 24)
    with pytest.raises(engine.Mi355qError) as info:
        gpu.w8a8_prepare(rows, 16, 24)  # 24 is not a multiple of 16
    assert info.value.status == engine.ERROR_INVALID


@pytest.mark.parametrize("M,K,widths", [(64, 1024, (4096, 4096, 4096)), (23, 560, (512, 100, 36, 512)),
                                        (5, 48, (20, 16))])
def test_projections_sharing_one_activation(engine, oracle, gpu, M, K, widths):
    """q, k and v of an encoder layer multiply the same quantized activation
    (minimindo_audio_encoder.c:400-403): one launch for all of them gives, per weight, the bits of
    the single call (and of the oracle)."""
    x = engine.synth_normal_f32(71, 1.0, M * K).reshape(M, K)
    q, scales = oracle.quantize_i8(x)
    rows = [engine.synth_w8_rows(80 + i, 0.02, N, K) for i, N in enumerate(widths)]
    biases = [engine.synth_normal_f32(90 + i, 1.0, N) if i != 1 else None for i, N in enumerate(widths)]
    weights = [gpu.w8a8_prepare(r, N, K) for r, N in zip(rows, widths)]
    try:
        print(f"w8a8 shared activation M={M} K={K} widths={widths}", flush=True)
        results = gpu.w8a8_linear_multi(weights, widths, q, scales, biases)
        for i, N in enumerate(widths):
            out_ref, acc_ref = oracle.w8a8_linear(rows[i], N, K, q, scales, biases[i])
            assert results[i][1].tobytes() == acc_ref.tobytes()
            assert np.array_equal(results[i][0].view(np.uint32), out_ref.view(np.uint32))
            single, _ = gpu.w8a8_linear(weights[i], N, q, scales, biases[i])
            assert np.array_equal(single.view(np.uint32), results[i][0].view(np.uint32))
    finally:
        for weight in weights:
            gpu.w8a8_destroy(weight)


def test_shared_activation_needs_equal_columns(engine, gpu):
    rows_a = engine.synth_w8_rows(1, 0.02, 32, 64)
    rows_b = engine.synth_w8_rows(2, 0.02, 32, 128)
    a, b = gpu.w8a8_prepare(rows_a, 32, 64), gpu.w8a8_prepare(rows_b, 32, 128)
    try:
        with pytest.raises(engine.Mi355qError) as caught:
            gpu.w8a8_linear_multi([a, b], (32, 32), np.zeros((2, 64), np.int8), np.ones(2, np.float32))
        assert caught.value.status == 2
    finally:
        gpu.w8a8_destroy(a)
        gpu.w8a8_destroy(b)
