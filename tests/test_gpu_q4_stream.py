"""GPU parity of the weight-streaming affine-Q4 linear (1..16 activation rows)
against the CPU oracle, through the C ABI.

Gate (Q4, fp32 accumulation): max_i |y_i - ref_i| / max(|ref_i|, 1e-2*rms(ref)) <= 1e-3,
where ref is the oracle's exact-weight, double-accumulated result
(reference semantics: qwen38_m3.m:102-121, weights not rounded).
"""
import numpy as np
import pytest

from conftest import bf16_bits, q4_relative_error

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-3


def make_x(engine, seed, M, K, x_dtype):
    rows = [engine.synth_normal_f32(seed + 1000 * m, 1.0, K) for m in range(M)]
    x32 = np.stack(rows)
    if x_dtype == engine.F16:
        return x32.astype(np.float16)
    if x_dtype == engine.BF16:
        return bf16_bits(x32)
    return x32


def run_case(engine, oracle, gpu, N, K, M, meta_kind, x_dtype, y_dtype, seed=7, residual=False):
    quants, meta_a, meta_b = engine.synth_q4_affine(seed, 0.02, N, K, meta_kind)
    x = make_x(engine, seed + 1, M, K, x_dtype)
    res = None
    if residual:
        res = engine.synth_normal_f32(seed + 2, 1.0, M * N).reshape(M, N)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"case N={N} K={K} M={M} meta={meta_kind} x={x_dtype} y={y_dtype} res={residual}",
              flush=True)
        y = gpu.q4_linear(weight, x, x_dtype, y_dtype, res, engine.F32)
    finally:
        weight.destroy()
    ref = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x, x_dtype, M)
    if residual:
        ref = ref + res.astype(np.float64)
    if y_dtype == engine.BF16:
        y = (y.astype(np.uint32) << 16).view(np.float32)
        tolerance = 2.0 ** -8  # bf16 output rounding dominates
    else:
        tolerance = TOLERANCE
    error = q4_relative_error(y, ref)
    assert np.all(np.isfinite(np.asarray(y, dtype=np.float64)))
    assert error <= tolerance, f"relative error {error:.3e}"
    return error


def test_config1_gemv_fp16(engine, oracle, gpu):
    """Headline configuration 1 (the reference's own CPU-runnable case): K=1024, N=3584, M=1, fp16 scale/bias, fp16 x, fp16 y."""
    run_case(engine, oracle, gpu, 3584, 1024, 1, engine.META_F16_INTERLEAVED, engine.F16, engine.F16)


@pytest.mark.parametrize("N,K", [(16, 64), (48, 64), (100, 192), (33, 1024), (257, 1088),
                                 (16480, 512)])
@pytest.mark.parametrize("M", [1, 2, 3, 8, 16])
def test_edge_shapes(engine, oracle, gpu, N, K, M):
    run_case(engine, oracle, gpu, N, K, M, engine.META_F16_INTERLEAVED, engine.F16, engine.F32)


@pytest.mark.parametrize("name,N,K", [("q", 6144, 5120), ("kv", 1024, 5120), ("o", 5120, 6144),
                                      ("gate_up", 17408, 5120), ("down", 5120, 17408)])
@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_27b_layer_shapes(engine, oracle, gpu, name, N, K, M):
    """Headline configurations 2 and 3 (27B layer shapes, decode and verify): bf16 scale/bias, fp16 activations, fp16 output."""
    run_case(engine, oracle, gpu, N, K, M, engine.META_BF16_PLANES, engine.F16, engine.F16,
             seed=11)


@pytest.mark.parametrize("M", [1, 3, 8])
def test_fp32_activations(engine, oracle, gpu, M):
    """fp32 x (the reference's cpu_q4_dot_float, qwen38_m3_layer.m:375-393) with a residual
    (qwen38_q4.metal:163-191)."""
    run_case(engine, oracle, gpu, 5120, 17408 if M == 1 else 2048, M,
             engine.META_F16_INTERLEAVED, engine.F32, engine.F32, residual=True)


@pytest.mark.parametrize("M", [2, 6])
def test_fp32_activations_long_rows(engine, oracle, gpu, M):
    """fp32 x on long rows with few tiles: the rows are cut in K slices that different workgroups
    take (M = 6 runs as twelve fp16 rows, the widest activation slots), and K = 17472 is an odd
    multiple of 64, so the last step has only its lower half."""
    run_case(engine, oracle, gpu, 528, 17472, M, engine.META_BF16_PLANES, engine.F32, engine.F32,
             seed=23, residual=True)


@pytest.mark.parametrize("y_dtype", ["F16", "BF16", "F32"])
def test_bf16_activations_and_outputs(engine, oracle, gpu, y_dtype):
    """bf16 activations and outputs (minimax_h3_m3_run_q4_projection_bf16)."""
    run_case(engine, oracle, gpu, 1000, 1536, 5, engine.META_BF16_PLANES, engine.BF16,
             getattr(engine, y_dtype))


def test_repeat_calls_are_bitwise_stable(engine, gpu):
    """Split-K partial sums are added in a fixed order: same bytes every call."""
    N, K, M = 5120, 17408, 4
    quants, meta_a, meta_b = engine.synth_q4_affine(3, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 5, M, K, engine.F16)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        first = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        for _ in range(5):
            again = gpu.q4_linear(weight, x, engine.F16, engine.F32)
            assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
    finally:
        weight.destroy()


def test_back_to_back_launches_of_mixed_row_counts(engine, oracle, gpu):
    """Launches with different numbers of activation rows lay LDS out differently (a wave's
    activation slots grow with the rows).  Many of them back to back on one weight, the workgroups
    of one launch taking over the LDS of the previous one's: every result equals the first of its
    kind bit for bit, and the first of each kind passes the usual gate."""
    N, K = 1536, 2112  # K: an odd multiple of 64
    quants, meta_a, meta_b = engine.synth_q4_affine(31, 0.02, N, K, engine.META_BF16_PLANES)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        inputs = {M: make_x(engine, 40 + M, M, K, engine.F16) for M in (1, 2, 5, 8, 16)}
        first = {}
        for M, x in inputs.items():
            first[M] = gpu.q4_linear(weight, x, engine.F16, engine.F32)
            ref = oracle.q4_linear(quants, meta_a, meta_b, engine.META_BF16_PLANES, N, K, x, engine.F16, M)
            assert q4_relative_error(first[M], ref) <= TOLERANCE
        for _ in range(20):
            for M in (16, 1, 8, 2, 5):
                again = gpu.q4_linear(weight, inputs[M], engine.F16, engine.F32)
                assert np.array_equal(first[M].view(np.uint32), again.view(np.uint32)), f"M={M}"
    finally:
        weight.destroy()


def test_argument_errors(engine, gpu):
    quants, meta_a, meta_b = engine.synth_q4_affine(1, 0.02, 16, 64, engine.META_F16_INTERLEAVED)
    with pytest.raises(engine.Mi355qError) as info:
        gpu.q4_prepare(quants, meta_a, None, 16, 96, engine.META_F16_INTERLEAVED)
    assert info.value.status == engine.ERROR_INVALID
    with pytest.raises(engine.Mi355qError) as info:
        gpu.q4_prepare(quants, meta_a, None, 16, 64, engine.META_BF16_PLANES)
    assert info.value.status == engine.ERROR_INVALID
    weight = gpu.q4_prepare(quants, meta_a, None, 16, 64, engine.META_F16_INTERLEAVED)
    try:
        with pytest.raises(engine.Mi355qError) as info:
            gpu.q4_linear(weight, np.zeros((0, 64), np.float16), engine.F16)
        assert info.value.status == engine.ERROR_INVALID
    finally:
        weight.destroy()


@pytest.mark.parametrize("M", [1, 3, 8])
def test_shared_activation_multi_launch(engine, oracle, gpu, M):
    """q|k|v-style call: three weights of different row counts, one launch, same x; each output
    must pass the oracle gate, repeat bit for bit on a second call, and agree with the
    single-weight call to fp32 summation-order noise (the split of the columns over waves
    depends on how many tiles a launch carries, so the order of the partial sums may differ)."""
    K = 1536
    rows = [640, 100, 1024]
    images = [engine.synth_q4_affine(60 + i, 0.02, N, K, engine.META_BF16_PLANES)
              for i, N in enumerate(rows)]
    x = make_x(engine, 70, M, K, engine.F16)
    weights = [gpu.q4_prepare(q, a, b, N, K, engine.META_BF16_PLANES)
               for (q, a, b), N in zip(images, rows)]
    try:
        print(f"multi case M={M}", flush=True)
        together = gpu.q4_linear_multi(weights, x, engine.F16, engine.F32)
        for (q, a, b), N, w, y in zip(images, rows, weights, together):
            alone = gpu.q4_linear(w, x, engine.F16, engine.F32)
            assert q4_relative_error(alone, y.astype(np.float64)) <= 1e-4
            ref = oracle.q4_linear(q, a, b, engine.META_BF16_PLANES, N, K, x, engine.F16, M)
            assert q4_relative_error(y, ref) <= TOLERANCE
        again = gpu.q4_linear_multi(weights, x, engine.F16, engine.F32)
        for first, second in zip(together, again):
            assert np.array_equal(first.view(np.uint32), second.view(np.uint32))
        mixed = gpu.q4_prepare(*engine.synth_q4_affine(1, 0.02, 32, 512, engine.META_BF16_PLANES),
                               32, 512, engine.META_BF16_PLANES)
        with pytest.raises(engine.Mi355qError) as info:
            gpu.q4_linear_multi([weights[0], mixed], x, engine.F16, engine.F32)
        assert info.value.status == engine.ERROR_INVALID
        mixed.destroy()
    finally:
        for w in weights:
            w.destroy()


@pytest.mark.parametrize("N,K,M,x_dtype", [(1000, 1536, 1, "F16"), (1000, 1536, 3, "F16"),
                                           (2048, 1024, 8, "BF16"), (640, 8704, 8, "F16"),
                                           (640, 8704, 4, "F32"), (17408, 5120, 1, "F16"),
                                           (4096, 4096, 1, "F16"), (5120, 2048, 1, "F16"),
                                           (3200, 1024, 2, "F16")])
def test_fused_gate_up_silu(engine, oracle, gpu, N, K, M, x_dtype):
    """MI355Q_FUSE_GATE_UP_SILU: y = silu(gate . x) * (up . x) in one launch
    (qwen38_q4_gate_up_silu, qwen38_q4.metal:129-151), against the oracle's two exact-weight dots
    combined in float64; (640, 8704) is cut in K slices, so the reduction kernel applies the
    nonlinearity there; N = 3200 .. 5120 at one row is the range where the unfused launch would
    take sixteen waves per tile, which the paired tiles of the fused launch do not have.  Also
    through the sequence call, with device pointers."""
    x_dtype = getattr(engine, x_dtype)
    gate_image = engine.synth_q4_affine(21, 0.02, N, K, engine.META_BF16_PLANES)
    up_image = engine.synth_q4_affine(22, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 23, M, K, x_dtype)
    gate = gpu.q4_prepare(*gate_image, N, K, engine.META_BF16_PLANES)
    up = gpu.q4_prepare(*up_image, N, K, engine.META_BF16_PLANES)
    x_ptr = y_ptr = None
    try:
        print(f"fused case N={N} K={K} M={M} x={x_dtype}", flush=True)
        y = gpu.q4_gate_up_silu(gate, up, x, x_dtype, engine.F32)
        x_ptr, y_ptr = gpu.to_device(x), gpu.alloc(M * N * 4)
        calls = engine.make_calls([([(gate, y_ptr), (up, None)], x_ptr, x_dtype, M, engine.F32, engine.F32,
                                    engine.FUSE_GATE_UP_SILU)])
        gpu.q4_sequence(calls)
        gpu.sync()
        queued = gpu.download(y_ptr, (M, N), np.float32)
        with pytest.raises(engine.Mi355qError) as info:  # three targets cannot be fused
            gpu.q4_sequence(engine.make_calls([([(gate, y_ptr), (up, y_ptr), (up, y_ptr)], x_ptr, x_dtype, M,
                                                engine.F32, engine.F32, engine.FUSE_GATE_UP_SILU)]))
        assert info.value.status == engine.ERROR_INVALID
    finally:
        for pointer in (x_ptr, y_ptr):
            if pointer:
                gpu.free(pointer)
        gate.destroy()
        up.destroy()
    g = oracle.q4_linear(*gate_image, engine.META_BF16_PLANES, N, K, x, x_dtype, M)
    u = oracle.q4_linear(*up_image, engine.META_BF16_PLANES, N, K, x, x_dtype, M)
    reference = g / (1.0 + np.exp(-g)) * u
    assert q4_relative_error(y, reference) <= TOLERANCE
    assert np.array_equal(y.view(np.uint32), queued.view(np.uint32))


@pytest.mark.parametrize("meta_kind", ["META_F16_INTERLEAVED", "META_BF16_PLANES"])
@pytest.mark.parametrize("N,K", [(1000, 5120), (33, 192)])
def test_dequant_rows_embedding_lookup(engine, oracle, gpu, meta_kind, N, K):
    """mi355q_q4_dequant_rows reads rows back out of the stream tiles: bit-exact with the oracle's
    scale * q + bias in fp32, and with its fp16 / bf16 roundings (the reference's embedding kernel
    writes half, qwen38_global.metal:13-29).  Ragged shapes exercise partial tiles and half steps."""
    meta_kind = getattr(engine, meta_kind)
    image = engine.synth_q4_affine(31, 0.02, N, K, meta_kind)
    rows = np.array([0, N - 1, 17 % N, N // 2, 0], dtype=np.uint32)
    weight = gpu.q4_prepare(*image, N, K, meta_kind)
    try:
        print(f"dequant rows N={N} K={K} meta={meta_kind}", flush=True)
        as_f32 = gpu.q4_dequant_rows(weight, rows, engine.F32)
        as_f16 = gpu.q4_dequant_rows(weight, rows, engine.F16)
        as_bf16 = gpu.q4_dequant_rows(weight, rows, engine.BF16)
        with pytest.raises(engine.Mi355qError) as info:
            gpu.q4_dequant_rows(weight, [N], engine.F32)
        assert info.value.status == engine.ERROR_INVALID
    finally:
        weight.destroy()
    expect = oracle.q4_dequantize_rows(*image, meta_kind, K, rows)
    assert np.array_equal(as_f32.view(np.uint32), expect.view(np.uint32))
    assert np.array_equal(as_f16.view(np.uint16), expect.astype(np.float16).view(np.uint16))
    assert np.array_equal(as_bf16, bf16_bits(expect).reshape(as_bf16.shape))


def test_lm_head_sized_gemv(engine, oracle, gpu):
    """The largest linear of the model, 248320 x 5120 (698 MB, qwen38_q4_lm_head,
    qwen38_global.metal:39-61), fp16 activations and fp32 logits: three 48-row windows of the
    output against the oracle, and the untouched logits between them against a second call
    (bitwise repeatability)."""
    N, K = 248320, 5120
    rng = np.random.default_rng(5)
    quants = rng.integers(0, 256, size=N * K // 2, dtype=np.uint8)
    meta = np.empty(N * (K // 64) * 2, dtype=np.uint16)
    meta[0::2] = (rng.random(N * (K // 64), dtype=np.float32) * 0.01 + 0.001).astype(np.float16).view(np.uint16)
    meta[1::2] = (rng.standard_normal(N * (K // 64), dtype=np.float32) * 0.05).astype(np.float16).view(np.uint16)
    x = make_x(engine, 3, 1, K, engine.F16)
    weight = gpu.q4_prepare(quants, meta, None, N, K, engine.META_F16_INTERLEAVED)
    try:
        print("lm head case", flush=True)
        y = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        again = gpu.q4_linear(weight, x, engine.F16, engine.F32)
    finally:
        weight.destroy()
    assert np.array_equal(y.view(np.uint32), again.view(np.uint32))
    assert np.all(np.isfinite(y))
    for begin in (0, 124111, N - 48):
        ref = oracle.q4_linear(quants, meta, None, engine.META_F16_INTERLEAVED, N, K, x, engine.F16, 1,
                               rows=(begin, begin + 48))[:, begin:begin + 48]
        assert q4_relative_error(y[:, begin:begin + 48], ref) <= TOLERANCE


@pytest.mark.parametrize("M,x_dtype,meta_kind", [(1, "F16", "META_F16_INTERLEAVED"), (4, "F16", "META_BF16_PLANES"),
                                                 (8, "F16", "META_BF16_PLANES"), (2, "F32", "META_BF16_PLANES")])
def test_row_subsets(engine, oracle, gpu, M, x_dtype, meta_kind):
    """mi355q_q4_linear_rows, the restricted-vocabulary head (qwen38_q4_lm_head over a low-id
    prefix, qwen38_q4_lm_head_gathered over listed ids; qwen38_global.metal:39-96): a prefix
    that ends inside a tile and a gathered list (unsorted, with repeats, first and last row,
    a count that is no multiple of 16) must equal the same rows of the full linear, and the
    oracle on those rows, to the usual tolerance.  K=8704 is cut in slices at M=8."""
    x_dtype, meta_kind = getattr(engine, x_dtype), getattr(engine, meta_kind)
    N, K = 1000, 8704 if M == 8 else 1536
    quants, meta_a, meta_b = engine.synth_q4_affine(31, 0.02, N, K, meta_kind)
    x = make_x(engine, 32, M, K, x_dtype)
    rng = np.random.default_rng(33)
    ids = np.concatenate([[N - 1, 0, 17, 17], rng.integers(0, N, size=71)]).astype(np.uint32)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"row subsets M={M} x={x_dtype} meta={meta_kind}", flush=True)
        full = gpu.q4_linear(weight, x, x_dtype, engine.F32)
        prefix = gpu.q4_linear_rows(weight, None, x, x_dtype, engine.F32, count=203)
        gathered = gpu.q4_linear_rows(weight, ids, x, x_dtype, engine.F32)
        gathered16 = gpu.q4_linear_rows(weight, ids, x, x_dtype, engine.F16)
        with pytest.raises(engine.Mi355qError):
            gpu.q4_linear_rows(weight, np.array([N], dtype=np.uint32), x, x_dtype, engine.F32)
        with pytest.raises(engine.Mi355qError):
            gpu.q4_linear_rows(weight, None, x, x_dtype, engine.F32, count=N + 1)
    finally:
        weight.destroy()
    ref = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x, x_dtype, M)
    assert prefix.shape == (M, 203) and gathered.shape == (M, ids.size)
    assert q4_relative_error(full, ref) <= TOLERANCE
    assert q4_relative_error(prefix, ref[:, :203]) <= TOLERANCE
    assert q4_relative_error(gathered, ref[:, ids]) <= TOLERANCE
    assert q4_relative_error(gathered16, ref[:, ids]) <= TOLERANCE
    # the same arithmetic as the full linear; only the split of K over waves may differ
    assert q4_relative_error(prefix, full[:, :203].astype(np.float64)) <= 1e-4
    assert q4_relative_error(gathered, full[:, ids].astype(np.float64)) <= 1e-4


@pytest.mark.parametrize("M", [1, 4])
def test_row_subsets_with_three_tiles_per_workgroup(engine, oracle, gpu, force, M):
    """A prefix and a gathered list of rows under the three-tile launch shape (what a restricted
    vocabulary of 33 to 49 thousand rows takes): the same values as the library's own shape for
    these small subsets, bit for bit (which workgroup computes a tile does not change its sums
    as long as the waves and K slices are the same), and the oracle's to the tolerance."""
    kind = engine.META_BF16_PLANES
    N, K = 1000, 1536
    quants, meta_a, meta_b = engine.synth_q4_affine(34, 0.02, N, K, kind)
    x = make_x(engine, 35, M, K, engine.F16)
    rng = np.random.default_rng(36)
    ids = np.concatenate([[N - 1, 0, 17, 17], rng.integers(0, N, size=90)]).astype(np.uint32)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, kind)
    try:
        print(f"row subsets, three tiles per workgroup, M={M}", flush=True)
        results = {}
        for shape in ("3,2,4", "1,2,4"):
            force("q4_stream", shape)
            results[shape] = (gpu.q4_linear_rows(weight, None, x, engine.F16, engine.F32, count=203),
                              gpu.q4_linear_rows(weight, ids, x, engine.F16, engine.F32))
    finally:
        weight.destroy()
    ref = oracle.q4_linear(quants, meta_a, meta_b, kind, N, K, x, engine.F16, M)
    prefix, gathered = results["3,2,4"]
    assert q4_relative_error(prefix, ref[:, :203]) <= TOLERANCE
    assert q4_relative_error(gathered, ref[:, ids]) <= TOLERANCE
    assert np.array_equal(prefix.view(np.uint32), results["1,2,4"][0].view(np.uint32))
    assert np.array_equal(gathered.view(np.uint32), results["1,2,4"][1].view(np.uint32))


def test_row_subset_with_device_ids(engine, oracle, gpu):
    """Row ids that already live on the GPU (MI355Q_SOURCE_DEVICE, asynchronous call): an id past
    the matrix yields 0 instead of being refused, the rest equals the host-id call bit for bit."""
    N, K, M = 777, 1024, 2
    quants, meta_a, meta_b = engine.synth_q4_affine(61, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 62, M, K, engine.F16)
    ids = np.array([5, N - 1, N + 3, 0, 400, 2**31, 17], dtype=np.uint32)
    good = ids < N
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    pointers = []
    try:
        print("row subset, device ids", flush=True)
        host = gpu.q4_linear_rows(weight, ids[good], x, engine.F16, engine.F32)
        ids_ptr, x_ptr = gpu.to_device(ids), gpu.to_device(x)
        y_ptr = gpu.alloc(M * ids.size * 4)
        pointers += [ids_ptr, x_ptr, y_ptr]
        gpu.q4_linear_rows_device(weight, ids_ptr, ids.size, x_ptr, engine.F16, M, y_ptr, engine.F32)
        gpu.sync()
        y = gpu.download(y_ptr, (M, ids.size), np.float32)
    finally:
        for pointer in pointers:
            gpu.free(pointer)
        weight.destroy()
    assert not y[:, ~good].any()
    assert np.array_equal(y[:, good].view(np.uint32), host.view(np.uint32))


def test_activation_range(engine, oracle, gpu):
    """Activations far from fp16's range.  Rows that are not fp16 are scaled by a power of two
    per row before they are split into fp16 pieces, so the gate holds whatever the row's
    magnitude: fp32 rows of magnitude 1e4, 1e-3 and 1e-6 (unscaled, the remainders of the last
    two would be fp16 subnormals or zero), a row with two entries beyond 65504 (which would be
    infinities in fp16), and the same rows as bf16."""
    N, K = 512, 1024
    quants, meta_a, meta_b = engine.synth_q4_affine(91, 0.02, N, K, engine.META_BF16_PLANES)
    base = make_x(engine, 92, 4, K, engine.F32)
    x = np.stack([base[0] * np.float32(1e4), base[1] * np.float32(1e-3), base[2] * np.float32(1e-6), base[3]])
    x[3, 5], x[3, 77] = np.float32(1e5), np.float32(-2.5e5)
    x_bf = bf16_bits(x).reshape(4, K)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        print("activation range case", flush=True)
        y = gpu.q4_linear(weight, x, engine.F32, engine.F32)
        y_bf = gpu.q4_linear(weight, x_bf, engine.BF16, engine.F32)
        y_one = gpu.q4_linear(weight, x[2:3], engine.F32, engine.F32)
    finally:
        weight.destroy()
    assert np.all(np.isfinite(y)) and np.all(np.isfinite(y_bf))
    ref = oracle.q4_linear(quants, meta_a, meta_b, engine.META_BF16_PLANES, N, K, x, engine.F32, 4)
    assert q4_relative_error(y, ref) <= TOLERANCE
    assert q4_relative_error(y_one, ref[2:3]) <= TOLERANCE
    ref_bf = oracle.q4_linear(quants, meta_a, meta_b, engine.META_BF16_PLANES, N, K, x_bf, engine.BF16, 4)
    assert q4_relative_error(y_bf, ref_bf) <= TOLERANCE


SLICED_CASES = [
    # name, [N per target], K, M, x dtype, fused gate-up-silu
    ("small", [320], 8704, 8, "F16", False),
    ("down_m1", [5120], 17408, 1, "F16", False),
    ("down_m2", [5120], 17408, 2, "F16", False),
    ("down_m4", [5120], 17408, 4, "F16", False),
    ("down_m8", [5120], 17408, 8, "F16", False),
    ("down_m4_f32", [5120], 17408, 4, "F32", False),
    ("three_targets", [640, 320, 336], 8704, 8, "F16", False),
    ("fused_silu", [640, 640], 8704, 8, "F16", True),
]


@pytest.mark.parametrize("name,rows,K,M,x_dtype,fused", SLICED_CASES, ids=[c[0] for c in SLICED_CASES])
def test_slices_added_in_kernel_match_second_kernel(engine, oracle, gpu, name, rows, K, M, x_dtype, fused):
    """K slices are added by the last workgroup of a column to arrive, which needs the
    workgroups of a column on one XCD (probed when a context is created).  The probe must
    say so on this GPU, and the same context with the in-kernel addition switched off (a
    second kernel adds the slices) must give the same bits: both add in slice order.
    Cases: the 27B down projection at every verify row count, fp32 activations (row pairs),
    a sliced launch of three weights, and the fused gate-up-SiLU launch whose nonlinearity the
    adding workgroup applies.  Repeated calls (the arrival counters return to zero) and a
    recorded graph's replays stay bitwise equal too."""
    shared, xcds = gpu.probe_xcd_columns()
    print(f"sliced case {name}: xcds={xcds} columns_share_xcd={shared}", flush=True)
    assert shared and xcds >= 1
    x_dtype = getattr(engine, x_dtype)
    kind = engine.META_BF16_PLANES
    images = [engine.synth_q4_affine(41 + i, 0.02, N, K, kind) for i, N in enumerate(rows)]
    x = make_x(engine, 42, M, K, x_dtype)
    ctx = engine.Context(0)
    weights = [ctx.q4_prepare(*image, N, K, kind) for image, N in zip(images, rows)]
    pointers, graph = [], None
    try:
        x_ptr = ctx.to_device(x)
        outputs = 1 if fused else len(rows)
        y_ptr = [ctx.alloc(M * N * 4) for N in rows[:outputs]]
        pointers = [x_ptr] + y_ptr
        targets = [(w, y_ptr[i] if i < outputs else None) for i, w in enumerate(weights)]
        calls = engine.make_calls([(targets, x_ptr, x_dtype, M, engine.F32, engine.F32,
                                    engine.FUSE_GATE_UP_SILU if fused else 0)])

        def run(launch):
            for pointer, N in zip(y_ptr, rows):
                ctx.upload(pointer, np.zeros((M, N), dtype=np.float32))
            launch()
            ctx.sync()
            return [ctx.download(pointer, (M, N), np.float32) for pointer, N in zip(y_ptr, rows)]

        ctx.set_option("trace", "1")
        in_kernel = [run(lambda: ctx.q4_sequence(calls)) for _ in range(3)]
        ctx.set_option("trace", None)
        graph = ctx.q4_sequence_record(calls)
        replays = [run(lambda: ctx.graph_launch(graph)) for _ in range(3)]
        ctx.set_option("in_kernel_slices", "0")
        second_kernel = [run(lambda: ctx.q4_sequence(calls)) for _ in range(2)]
    finally:
        if graph is not None:
            ctx.graph_destroy(graph)
        for pointer in pointers:
            ctx.free(pointer)
        for w in weights:
            w.destroy()
        ctx.close()
    for label, runs in (("in-kernel", in_kernel), ("graph replay", replays), ("second kernel", second_kernel)):
        for index, outputs_of_run in enumerate(runs):
            for got, first in zip(outputs_of_run, in_kernel[0]):
                assert np.array_equal(got.view(np.uint32), first.view(np.uint32)), f"{label} run {index}"
    refs = [oracle.q4_linear(*image, kind, N, K, x, x_dtype, M) for image, N in zip(images, rows)]
    if fused:
        refs = [refs[0] / (1.0 + np.exp(-refs[0])) * refs[1]]
    for got, ref in zip(in_kernel[0], refs):
        assert q4_relative_error(got, ref) <= TOLERANCE


def test_recorded_sequence_replays(engine, oracle, gpu):
    """mi355q_q4_sequence_record / mi355q_graph_launch: three calls (shared-x pair at M=1, an fp32
    activation that goes through the conversion kernel, an M=8 call that is cut in K slices and
    reduced) recorded into one graph; every replay, with eager work and synchronisation in between
    and fresh inputs, must equal the eager sequence bit for bit.  A graph is refused once the
    context has reallocated a staging buffer (a context of its own, so that what other tests did
    to the shared one does not decide whether the last call grows a buffer)."""
    gpu = engine.Context(0)  # the fixture only decides whether the test runs at all
    K1, N1, K2, N2 = 1536, 640, 8704, 320
    images = [engine.synth_q4_affine(80 + i, 0.02, n, k, engine.META_BF16_PLANES)
              for i, (n, k) in enumerate([(N1, K1), (N1, K1), (N2, K2), (N2, K2)])]
    weights = [gpu.q4_prepare(*image, n, k, engine.META_BF16_PLANES)
               for image, (n, k) in zip(images, [(N1, K1), (N1, K1), (N2, K2), (N2, K2)])]
    pointers, graph = [], None
    try:
        x1 = make_x(engine, 1, 1, K1, engine.F16)
        x2 = make_x(engine, 2, 2, K2, engine.F32)
        x3 = make_x(engine, 3, 8, K2, engine.F16)
        x_ptr = [gpu.to_device(x) for x in (x1, x2, x3)]
        y_shapes = [(1, N1), (1, N1), (2, N2), (8, N2)]
        y_ptr = [gpu.alloc(m * n * 4) for m, n in y_shapes]
        pointers = x_ptr + y_ptr
        calls = engine.make_calls([
            ([(weights[0], y_ptr[0]), (weights[1], y_ptr[1])], x_ptr[0], engine.F16, 1, engine.F32),
            ((weights[2], y_ptr[2]), x_ptr[1], engine.F32, 2, engine.F32),
            ((weights[3], y_ptr[3]), x_ptr[2], engine.F16, 8, engine.F32)])

        def outputs():
            gpu.sync()
            return [gpu.download(p, shape, np.float32) for p, shape in zip(y_ptr, y_shapes)]

        print("recorded sequence case", flush=True)
        graph = gpu.q4_sequence_record(calls)
        for replay in range(3):
            # new activations, an eager run as the expectation, outputs wiped, then the replay
            for pointer, x, seed in zip(x_ptr, (x1, x2, x3), (11, 12, 13)):
                gpu.upload(pointer, make_x(engine, seed + 10 * replay, x.shape[0], x.shape[1],
                                           engine.F32 if x.dtype == np.float32 else engine.F16))
            gpu.q4_sequence(calls)
            expect = outputs()
            for pointer, shape in zip(y_ptr, y_shapes):
                gpu.upload(pointer, np.zeros(shape, dtype=np.float32))
            gpu.graph_launch(graph)
            got = outputs()
            for a, b in zip(got, expect):
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"replay {replay}"
            assert all(np.any(a != 0) for a in got)
        # a host-pointer call larger than any before it grows a staging buffer: the graph is stale
        big = gpu.q4_linear(weights[3], make_x(engine, 5, 16, K2, engine.F16), engine.F16, engine.F32)
        assert big.shape == (16, N2)
        with pytest.raises(engine.Mi355qError) as info:
            gpu.graph_launch(graph)
        assert info.value.status == engine.ERROR_INVALID
    finally:
        if graph is not None:
            gpu.graph_destroy(graph)
        for pointer in pointers:
            gpu.free(pointer)
        for w in weights:
            w.destroy()
        gpu.close()


HALF_CASES = [
    # name, [N per target], K, M, x dtype, residual
    ("o_m1", [5120], 6144, 1, "F16", False),
    ("o_m2_residual", [5120], 6144, 2, "F16", True),
    ("down_m1", [5120], 17408, 1, "F16", False),
    ("down_m2_bf16", [5120], 17408, 2, "BF16", True),
    ("ragged_m1", [1000], 1536, 1, "F16", False),
    ("ragged_m3", [1000], 1536, 3, "F16", True),
    ("m4", [528], 2048, 4, "BF16", False),
    ("three_targets_m2", [640, 328, 16], 1024, 2, "F16", True),
]


@pytest.mark.parametrize("name,rows,K,M,x_dtype,with_residual", HALF_CASES, ids=[c[0] for c in HALF_CASES])
def test_half_tile_form(engine, oracle, gpu, force, name, rows, K, M, x_dtype, with_residual):
    """The half-tile form of the streaming launch (eight rows of a tile and two 128-column steps at
    a time per workgroup; what o_proj and down_proj of the 27B layer take at one and two rows):
    forced on for every shape here, against the oracle and against the whole-tile launch of the
    same call (which adds the same products in another order: equal within the gate, and a
    second launch of the half-tile form repeats its own bits)."""
    x_dtype = getattr(engine, x_dtype)
    kind = engine.META_BF16_PLANES
    images = [engine.synth_q4_affine(400 + i, 0.02, N, K, kind) for i, N in enumerate(rows)]
    weights = [gpu.q4_prepare(*image, N, K, kind) for image, N in zip(images, rows)]
    x = make_x(engine, 410, M, K, x_dtype)
    residuals = [engine.synth_normal_f32(420 + i, 1.0, M * N).reshape(M, N) if with_residual else None
                 for i, N in enumerate(rows)]
    pointers = []
    try:
        print(f"half tile case {name}", flush=True)
        x_ptr = gpu.to_device(x)
        y_ptrs = [gpu.alloc(M * N * 4) for N in rows]
        r_ptrs = [gpu.to_device(r) if r is not None else None for r in residuals]
        pointers = [x_ptr] + y_ptrs + [p for p in r_ptrs if p]
        calls = engine.make_calls([([(w, y, r) for w, y, r in zip(weights, y_ptrs, r_ptrs)], x_ptr, x_dtype, M,
                                    engine.F32, engine.F32)])
        results = {}
        for mode in ("0", "1", "1 again"):
            force("half_tiles", mode[0])
            for y_ptr, N in zip(y_ptrs, rows):
                gpu.upload(y_ptr, np.full((M, N), np.nan, dtype=np.float32))
            gpu.q4_sequence(calls)
            gpu.sync()
            results[mode] = [gpu.download(y_ptr, (M, N), np.float32) for y_ptr, N in zip(y_ptrs, rows)]
    finally:
        for pointer in pointers:
            gpu.free(pointer)
        for weight in weights:
            weight.destroy()
    for i, N in enumerate(rows):
        reference = oracle.q4_linear(*images[i], kind, N, K, x, x_dtype, M)
        if with_residual:
            reference = reference + residuals[i]
        assert q4_relative_error(results["1"][i], reference) <= TOLERANCE
        assert q4_relative_error(results["0"][i], reference) <= TOLERANCE
        assert np.array_equal(results["1"][i].view(np.uint32), results["1 again"][i].view(np.uint32))


THREE_TILE_CASES = [
    # name, rows of the targets, K, M, x dtype, residual, forced launch shape
    ("gate_up_sized_m8", (17408, 17408), 640, 8, "F16", False, None),   # chosen by the library itself: 2176 tiles
    ("ragged_tiles_m4", (1000, 520), 1024, 4, "F16", True, "3,2,4"),    # 63 and 33 tiles: last workgroups of one and two tiles
    ("bf16_rows_m16", (1000,), 704, 16, "BF16", False, "3,2,4"),        # sixteen rows, odd number of 64-column groups
    ("fp32_rows_m5", (808, 808, 200), 1536, 5, "F32", True, "3,2,4"),   # ten operand rows (value, remainder)
    ("k_slices_m8", (600,), 4096, 8, "F16", False, "3,2,4,2"),          # two K slices added inside the kernel
]


@pytest.mark.parametrize("name,rows,K,M,x_dtype,with_residual,forced", THREE_TILE_CASES,
                         ids=[c[0] for c in THREE_TILE_CASES])
def test_three_tiles_per_workgroup(engine, oracle, gpu, force, name, rows, K, M, x_dtype, with_residual, forced):
    """Three tiles per workgroup (what gate|up of the 27B layer takes from four rows on, so that its
    workgroups fit the compute units in one round): against the oracle, and bit for bit against the
    launch with two tiles per workgroup (tiles do not meet: which workgroup computes a tile cannot
    change its sums)."""
    x_dtype = getattr(engine, x_dtype)
    kind = engine.META_BF16_PLANES
    images = [engine.synth_q4_affine(500 + i, 0.02, N, K, kind) for i, N in enumerate(rows)]
    weights = [gpu.q4_prepare(*image, N, K, kind) for image, N in zip(images, rows)]
    x = make_x(engine, 510, M, K, x_dtype)
    residuals = [engine.synth_normal_f32(520 + i, 1.0, M * N).reshape(M, N) if with_residual else None
                 for i, N in enumerate(rows)]
    pointers = []
    try:
        print(f"three tile case {name}", flush=True)
        x_ptr = gpu.to_device(x)
        y_ptrs = [gpu.alloc(M * N * 4) for N in rows]
        r_ptrs = [gpu.to_device(r) if r is not None else None for r in residuals]
        pointers = [x_ptr] + y_ptrs + [p for p in r_ptrs if p]
        calls = engine.make_calls([([(w, y, r) for w, y, r in zip(weights, y_ptrs, r_ptrs)], x_ptr, x_dtype, M,
                                    engine.F32, engine.F32)])
        results = {}
        two = "2,2,4" + (forced[5:] if forced and len(forced) > 5 else "")
        for mode, shape in (("three", forced), ("two", two)):
            force("q4_stream", shape)
            for y_ptr, N in zip(y_ptrs, rows):
                gpu.upload(y_ptr, np.full((M, N), np.nan, dtype=np.float32))
            gpu.q4_sequence(calls)
            gpu.sync()
            results[mode] = [gpu.download(y_ptr, (M, N), np.float32) for y_ptr, N in zip(y_ptrs, rows)]
    finally:
        for pointer in pointers:
            gpu.free(pointer)
        for weight in weights:
            weight.destroy()
    for i, N in enumerate(rows):
        reference = oracle.q4_linear(*images[i], kind, N, K, x, x_dtype, M)
        if with_residual:
            reference = reference + residuals[i]
        assert q4_relative_error(results["three"][i], reference) <= TOLERANCE
        assert np.array_equal(results["three"][i].view(np.uint32), results["two"][i].view(np.uint32))
