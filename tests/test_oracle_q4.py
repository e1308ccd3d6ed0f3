"""Pins the oracle's affine-Q4 dot (reference: qwen38_m3.m:102-121,
qwen38_m3_layer.m:354-393, minimax_h3_m3_real_gemm.c:25-42,
minimax_h3_m3_gemm.m:75-104) with checks that do not restate its loop:
a numpy float64 matrix product on independently unpacked codes, closed forms
that isolate the scale, the bias and the nibble/byte/group index mapping, and the
reference's deterministic synthetic fixtures regenerated from their formulas."""
import numpy as np
import pytest

from conftest import bf16_bits, bf16_to_f32


def unpack_codes(quants, N, K):
    """[N][K] integer codes from the packed plane, via the uint32 view the packer
    documents (qwen38_m3_pack.c:618-637): element k%8 at bits 4*(k%8) of word k/8."""
    words = np.frombuffer(np.ascontiguousarray(quants).tobytes(), dtype="<u4").reshape(N, K // 8)
    shifts = (4 * np.arange(8, dtype=np.uint32))[None, None, :]
    return ((words[:, :, None] >> shifts) & 15).reshape(N, K).astype(np.float64)


def dense_weights(quants, meta_a, meta_b, meta_kind, N, K):
    codes = unpack_codes(quants, N, K)
    if meta_kind == 0:
        meta = np.asarray(meta_a).reshape(N, K // 64, 2)
        scale = meta[..., 0].copy().view(np.float16).astype(np.float64)
        bias = meta[..., 1].copy().view(np.float16).astype(np.float64)
    else:
        scale = bf16_to_f32(meta_a).reshape(N, K // 64).astype(np.float64)
        bias = bf16_to_f32(meta_b).reshape(N, K // 64).astype(np.float64)
    return np.repeat(scale, 64, axis=1) * codes + np.repeat(bias, 64, axis=1)


def random_image(rng, N, K, meta_kind):
    quants = rng.integers(0, 256, size=N * K // 2, dtype=np.uint8)
    scale = (rng.random(N * K // 64) * 0.01 + 0.001).astype(np.float32)
    bias = (rng.standard_normal(N * K // 64) * 0.05).astype(np.float32)
    if meta_kind == 0:
        meta = np.empty(N * K // 64 * 2, dtype=np.uint16)
        meta[0::2] = scale.astype(np.float16).view(np.uint16)
        meta[1::2] = bias.astype(np.float16).view(np.uint16)
        return quants, meta, None
    return quants, bf16_bits(scale), bf16_bits(bias)


@pytest.mark.parametrize("meta_kind", [0, 1])
@pytest.mark.parametrize("x_kind", ["f16", "f32", "bf16"])
def test_truth_flavour_equals_float64_matmul(oracle, meta_kind, x_kind):
    rng = np.random.default_rng(3)
    N, K, M = 37, 320, 3
    quants, meta_a, meta_b = random_image(rng, N, K, meta_kind)
    x32 = rng.standard_normal((M, K)).astype(np.float32)
    if x_kind == "f16":
        x, kind, xd = x32.astype(np.float16), oracle.X_F16, x32.astype(np.float16).astype(np.float64)
    elif x_kind == "bf16":
        x, kind = bf16_bits(x32).reshape(M, K), oracle.X_BF16
        xd = bf16_to_f32(x).astype(np.float64)
    else:
        x, kind, xd = x32, oracle.X_F32, x32.astype(np.float64)
    y = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x, kind, M)
    expect = xd @ dense_weights(quants, meta_a, meta_b, meta_kind, N, K).T
    # the oracle adds the K terms one by one in double, numpy in blocks: ~1e-15 relative
    assert np.allclose(y, expect, rtol=1e-12, atol=1e-12)
    seq = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x, kind, M,
                           accumulate=oracle.ACC_F32_SEQUENTIAL)
    assert np.max(np.abs(seq - expect)) < 2e-4  # fp32 sequential sum of 320 O(0.1) terms


def test_rows_window_and_threads(oracle):
    rng = np.random.default_rng(4)
    N, K = 64, 128
    quants, meta_a, meta_b = random_image(rng, N, K, 0)
    x = rng.standard_normal((1, K)).astype(np.float16)
    full = oracle.q4_linear(quants, meta_a, meta_b, 0, N, K, x, oracle.X_F16, 1, threads=3)
    part = oracle.q4_linear(quants, meta_a, meta_b, 0, N, K, x, oracle.X_F16, 1, rows=(10, 20))
    assert np.array_equal(part[0, 10:20], full[0, 10:20]) and not part[0, :10].any()
    with pytest.raises(ValueError):
        oracle.q4_linear(quants[: N * 48], meta_a, None, 0, N, 96, x, oracle.X_F16, 1)


def test_closed_forms(oracle):
    """all codes equal c  =>  y = (s*c + b) * sum(x);   s = 0  =>  y = sum_g b_g * sum_g(x);
    one hot nibble       =>  y - baseline = s * c * x[k] for exactly the right k."""
    rng = np.random.default_rng(5)
    N, K = 4, 256
    groups = K // 64
    x = (rng.integers(-8, 9, size=(1, K)) / 8.0).astype(np.float16)  # exact binary fractions
    xs = x.astype(np.float64)
    s, b, c = np.float16(0.0078125), np.float16(-0.0625), 11
    meta = np.tile(np.array([s.view(np.uint16), b.view(np.uint16)], dtype=np.uint16), N * groups)
    quants = np.full(N * K // 2, c | (c << 4), dtype=np.uint8)
    y = oracle.q4_linear(quants, meta, None, 0, N, K, x, oracle.X_F16, 1)
    assert np.allclose(y, (float(s) * c + float(b)) * xs.sum(), rtol=0, atol=1e-12)
    # zero scale, per-group biases
    biases = (np.arange(N * groups) - 5) / 64.0
    meta0 = np.zeros(N * groups * 2, dtype=np.uint16)
    meta0[1::2] = biases.astype(np.float16).view(np.uint16)
    y0 = oracle.q4_linear(rng.integers(0, 256, N * K // 2, dtype=np.uint8), meta0, None, 0, N, K,
                          x, oracle.X_F16, 1)
    expect0 = (biases.reshape(N, groups) * xs.reshape(groups, 64).sum(axis=1)[None, :]).sum(axis=1)
    assert np.allclose(y0[0], expect0, atol=1e-12)
    # single hot nibble at every (row, k) of a small sweep: isolates byte/nibble/group mapping
    metab = np.tile(np.array([s.view(np.uint16), 0], dtype=np.uint16), N * groups)
    for row, k in [(0, 0), (0, 1), (1, 62), (1, 63), (2, 64), (2, 129), (3, 255), (3, 190)]:
        hot = np.zeros(N * K // 2, dtype=np.uint8)
        hot[row * K // 2 + k // 2] = 9 << (4 * (k % 2))
        yh = oracle.q4_linear(hot, metab, None, 0, N, K, x, oracle.X_F16, 1)
        expect = np.zeros(N)
        expect[row] = float(s) * 9 * xs[0, k]
        assert np.allclose(yh[0], expect, atol=1e-15), (row, k)


def test_h3_synthetic_fixture_weight_rounding(oracle):
    """The reference's closed-form synthetic GEMM (minimax_h3_m3_gemm.m:75-104): code bytes,
    metadata and inputs from formulas; its CPU reference rounds the weight to fp16.  Regenerated
    here with numpy and compared with the oracle's fp16-weight flavour on the first rows; the
    exact-weight flavour must differ from it by no more than the recorded GPU-vs-CPU error scale
    (0.0026 on O(1..10) outputs, results.json:210)."""
    K, N, groups = 5376, 16, 84
    index = np.arange(N * K // 2, dtype=np.uint32)
    block = index >> 5
    low = (index * 5 + block * 3 + 3) & 15
    high = (index * 7 + block * 11 + 11) & 15
    quants = (low | (high << 4)).astype(np.uint8)
    blocks = np.arange(N * groups)
    phase = (blocks % 7).astype(np.float32)
    scale = (np.float32(0.0175) + phase * np.float32(0.0017)).astype(np.float16)
    bias = (np.float32(-0.1875) + phase * np.float32(0.0078125)).astype(np.float16)
    meta = np.empty(N * groups * 2, dtype=np.uint16)
    meta[0::2], meta[1::2] = scale.view(np.uint16), bias.view(np.uint16)
    k = np.arange(K, dtype=np.uint32)
    x = ((((k * 13 + 17) % 17).astype(np.int32) - 8) * 0.0625).astype(np.float32).reshape(1, K)
    codes = unpack_codes(quants, N, K)
    w16 = (np.repeat(scale.astype(np.float32).reshape(N, groups), 64, axis=1) * codes.astype(np.float32)
           + np.repeat(bias.astype(np.float32).reshape(N, groups), 64, axis=1)).astype(np.float16)
    expect = x.astype(np.float64) @ w16.astype(np.float64).T
    got = oracle.q4_linear(quants, meta, None, 0, N, K, x, oracle.X_F32, 1,
                           weight_rounding=oracle.W_ROUND_F16)
    assert np.allclose(got, expect, atol=1e-10)
    seq = oracle.q4_linear(quants, meta, None, 0, N, K, x, oracle.X_F32, 1,
                           weight_rounding=oracle.W_ROUND_F16, accumulate=oracle.ACC_F32_SEQUENTIAL)
    assert np.max(np.abs(seq - expect)) < 1e-3
    exact = oracle.q4_linear(quants, meta, None, 0, N, K, x, oracle.X_F32, 1)
    assert np.max(np.abs(exact - expect)) < 0.02


def test_qwen38_synthetic_recipe_and_bf16_weight_flavour(oracle):
    """xorshift32 weights and sin/cos activation of the Qwen3.8 bench (qwen38_m3.m:64-87,567-572),
    8 rows of the 5120-column gate matrix; bf16-weight flavour against numpy (real_gemm.c:25-42)."""
    K, N = 5120, 8
    groups = K // 64
    state = np.uint32(0x36A110C)
    quants = np.empty(N * groups * 32, dtype=np.uint8)
    meta = np.empty(N * groups * 2, dtype=np.uint16)

    def nxt(s):
        s ^= (s << np.uint32(13)) & np.uint32(0xFFFFFFFF)
        s ^= s >> np.uint32(17)
        s ^= (s << np.uint32(5)) & np.uint32(0xFFFFFFFF)
        return np.uint32(s)

    with np.errstate(over="ignore"):
        for g in range(N * groups):
            for byte in range(32):
                state = nxt(state)
                quants[g * 32 + byte] = np.uint8(int(state) & 0xFF)
            state = nxt(state)
            scale = np.float32(0.0035) + np.float32(0.00025) * np.float32(int(state) & 7)
            bias = np.float32(-7.5) * scale + np.float32(0.0002) * np.float32((g % 5) - 2)
            meta[2 * g] = np.float16(scale).view(np.uint16)
            meta[2 * g + 1] = np.float16(bias).view(np.uint16)
    i = np.arange(K, dtype=np.float32)
    x = (np.float32(0.75) * np.sin(np.float32(0.013) * i) + np.float32(0.20) * np.cos(np.float32(0.031) * i))
    x = x.astype(np.float16).reshape(1, K)
    expect = x.astype(np.float64) @ dense_weights(quants, meta, None, 0, N, K).T
    got = oracle.q4_linear(quants, meta, None, 0, N, K, x, oracle.X_F16, 1)
    assert np.allclose(got, expect, rtol=1e-12, atol=1e-12)
    lib = oracle.lib()
    one = lib.orc_q4_dot_f16x_seq(quants.ctypes.data, meta.ctypes.data, x.ctypes.data, 3, groups)
    assert abs(one - expect[0, 3]) < 5e-5
    # bf16 planes + bf16-rounded weight
    s = bf16_bits(meta[0::2].copy().view(np.float16).astype(np.float32))
    b = bf16_bits(meta[1::2].copy().view(np.float16).astype(np.float32))
    xb = bf16_bits(x.astype(np.float32)).reshape(1, K)
    codes = unpack_codes(quants, N, K).astype(np.float32)
    w = (np.repeat(bf16_to_f32(s).reshape(N, groups), 64, axis=1) * codes
         + np.repeat(bf16_to_f32(b).reshape(N, groups), 64, axis=1)).astype(np.float32)
    wb = bf16_to_f32(bf16_bits(w)).astype(np.float64)
    expect_b = bf16_to_f32(xb).astype(np.float64) @ wb.T
    got_b = oracle.q4_linear(quants, s, b, 1, N, K, xb, oracle.X_BF16, 1,
                             weight_rounding=oracle.W_ROUND_BF16)
    assert np.allclose(got_b, expect_b, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("meta_kind", [0, 1])
def test_dequantize_row_equals_numpy_float32(oracle, meta_kind):
    """orc_q4_dequantize_row (qwen38_global.metal:13-29) against numpy float32 arithmetic — a
    rounded multiply, then a rounded add, numpy never fuses them — on codes unpacked through the
    uint32 view; a wrong nibble, byte, group or plane index changes some element."""
    rng = np.random.default_rng(11)
    N, K = 23, 448
    quants, meta_a, meta_b = random_image(rng, N, K, meta_kind)
    codes = unpack_codes(quants, N, K).astype(np.float32)
    if meta_kind == 0:
        meta = np.asarray(meta_a).reshape(N, K // 64, 2)
        scale = meta[..., 0].copy().view(np.float16).astype(np.float32)
        bias = meta[..., 1].copy().view(np.float16).astype(np.float32)
    else:
        scale = bf16_to_f32(meta_a).reshape(N, K // 64)
        bias = bf16_to_f32(meta_b).reshape(N, K // 64)
    expect = np.repeat(scale, 64, axis=1) * codes + np.repeat(bias, 64, axis=1)
    assert expect.dtype == np.float32
    rows = [0, 7, 22, 7]
    got = oracle.q4_dequantize_rows(quants, meta_a, meta_b, meta_kind, K, rows)
    assert np.array_equal(got.view(np.uint32), expect[rows].view(np.uint32))


def test_q8_affine_matches_numpy_float64(oracle):
    """orc_q8_affine_linear (u8 codes, one per byte) against a float64 matrix product on the codes
    read straight from the byte array; a single hot code at eight (row, k) positions isolates the
    index mapping (byte (n*K/64 + g)*64 + k, minimax_h3_attention.metal:631-634)."""
    rng = np.random.default_rng(11)
    N, K, M = 37, 320, 3
    quants = rng.integers(0, 256, size=N * K, dtype=np.uint8)
    scales = (rng.random(N * (K // 64), dtype=np.float32) * 0.01 + 0.001).astype(np.float16)
    biases = (rng.standard_normal(N * (K // 64)).astype(np.float32) * 0.1).astype(np.float16)
    meta = np.stack([scales.view(np.uint16), biases.view(np.uint16)], axis=-1).reshape(-1)
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (scales.astype(np.float64).reshape(N, -1, 1) * quants.reshape(N, -1, 64).astype(np.float64)
         + biases.astype(np.float64).reshape(N, -1, 1)).reshape(N, K)
    expect = x.astype(np.float64) @ w.T
    got = oracle.q8_affine_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x, oracle.X_F16, M)
    assert np.max(np.abs(got - expect)) <= 1e-9 * np.max(np.abs(expect))
    for n, k in [(0, 0), (0, 63), (0, 64), (5, 131), (36, 319), (17, 1), (20, 200), (36, 0)]:
        hot = np.zeros(N * K, dtype=np.uint8)
        hot[n * K + k] = 200
        one = np.stack([np.float16(1.0).view(np.uint16), np.float16(0.0).view(np.uint16)])
        meta_one = np.tile(one, N * (K // 64))
        y = oracle.q8_affine_linear(hot, meta_one, None, oracle.META_F16_INTERLEAVED, N, K, x, oracle.X_F16, M)
        expect_hot = np.zeros((M, N))
        expect_hot[:, n] = 200.0 * x[:, k].astype(np.float64)
        assert np.array_equal(y, expect_hot)
    seq = oracle.q8_affine_linear(quants, meta, None, oracle.META_F16_INTERLEAVED, N, K, x, oracle.X_F16, M,
                                  accumulate=oracle.ACC_F32_SEQUENTIAL)
    assert np.max(np.abs(seq - expect)) <= 1e-4 * np.max(np.abs(expect))


def test_recipe_generators_agree(oracle):
    """The C generator of the Qwen3.8 benchmark's xorshift32 matrices (used by the GPU tests at
    full size) against the step-by-step numpy restatement of the same recipe on the first 700
    groups of each seed, and the activation formula's first values against Python floats."""
    import math

    import recipes
    for seed in recipes.QWEN38_SEEDS.values():
        quants, meta = recipes.qwen38_weights(oracle, seed, 8, 5120)
        slow_q, slow_m = recipes.qwen38_weights_numpy(seed, 640)
        assert np.array_equal(quants, slow_q) and np.array_equal(meta, slow_m)
    scales = meta[0::2].view(np.float16).astype(np.float32)
    assert scales.min() >= 0.0035 - 1e-5 and scales.max() <= 0.0035 + 7 * 0.00025 + 1e-5
    x = recipes.qwen38_activation(2, 5120)
    for i in (0, 1, 77, 5119, 5120, 10239):
        expect = 0.75 * math.sin(np.float32(0.013) * np.float32(i)) + 0.20 * math.cos(np.float32(0.031) * np.float32(i))
        assert abs(float(x.reshape(-1)[i]) - expect) <= 1e-3
    h3 = recipes.h3_input(2)
    assert h3[0, 0] == np.float32(0.0625 * (17 % 17 - 8)) and h3[1, 0] == np.float32(0.0625 * ((13 * 5376 + 17) % 17 - 8))
    assert set(np.unique(h3 * 16).astype(int)) <= set(range(-8, 9))
