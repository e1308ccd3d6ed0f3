"""GPU parity of the prefill GEMM (M > 16) against the CPU oracle, through the C ABI.

The GEMM rounds each weight to fp16 before an fp16 x fp16 multiply with fp32 accumulation
(as the reference's batched kernels and its scalar check do, minimax_h3_m3_gemm.m:87-104), so
the gate compares with the oracle's fp16-weight flavour in double accumulation:
max_i |y_i - ref_i| / max(|ref_i|, 1e-2*rms(ref)) <= 1e-3.  The distance to the exact-weight
result is reported against rms(ref) (the weight rounding itself, ~2^-12 per weight)."""
import numpy as np
import pytest

from conftest import bf16_bits, q4_relative_error

pytestmark = pytest.mark.gpu


def make_x(engine, seed, M, K):
    return engine.synth_normal_f32(seed, 1.0, M * K).reshape(M, K)


def run_case(engine, oracle, gpu, N, K, M, meta_kind, x_dtype, y_dtype, columns=None, seed=5,
             residual=False):
    quants, meta_a, meta_b = engine.synth_q4_affine(seed, 0.02, N, K, meta_kind)
    x32 = make_x(engine, seed + 1, M, K)
    if x_dtype == engine.F16:
        x = x32.astype(np.float16)
        x_ref, x_kind = x, oracle.X_F16
    elif x_dtype == engine.BF16:
        x = bf16_bits(x32).reshape(M, K)
        # the kernel multiplies fp16: bf16 values in fp16's normal range convert exactly
        x_ref, x_kind = x, oracle.X_BF16
    else:
        x = x32
        x_ref, x_kind = x32, oracle.X_F32  # fp32 rows go in as (value, remainder) pairs: not rounded
    res = engine.synth_normal_f32(seed + 2, 1.0, M * N).reshape(M, N) if residual else None
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, meta_kind)
    try:
        print(f"gemm case N={N} K={K} M={M} meta={meta_kind} x={x_dtype} y={y_dtype}", flush=True)
        y = gpu.q4_linear(weight, x, x_dtype, y_dtype, res, engine.F32)
    finally:
        weight.destroy()
    windows = columns if columns else [(0, N)]
    if isinstance(windows, tuple):
        windows = [windows]
    assert np.all(np.isfinite(np.asarray(y, dtype=np.float64)))
    if y_dtype == engine.BF16:
        y = (y.astype(np.uint32) << 16).view(np.float32)
    error = 0.0
    for lo, hi in windows:
        ref = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x_ref, x_kind, M,
                               weight_rounding=oracle.W_ROUND_F16, rows=(lo, hi))[:, lo:hi]
        exact = oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x_ref, x_kind, M,
                                 rows=(lo, hi))[:, lo:hi]
        if residual:
            ref, exact = ref + res[:, lo:hi], exact + res[:, lo:hi]
        got = np.asarray(y, dtype=np.float64)[:, lo:hi]
        window_error = q4_relative_error(got, ref)
        tolerance = 2.0 ** -8 if y_dtype == engine.BF16 else 1e-3
        assert window_error <= tolerance, f"columns {lo}..{hi}: relative error {window_error:.3e}"
        rms = np.sqrt(np.mean(exact * exact))
        drift = float(np.max(np.abs(got - exact)) / rms)
        # a bf16 output adds its own rounding: half an ulp (2^-9 relative) of the largest output
        limit = 2e-3 + (2.0 ** -9 * float(np.max(np.abs(exact)) / rms) if y_dtype == engine.BF16 else 0.0)
        assert drift <= limit, f"columns {lo}..{hi}: vs exact weights {drift:.3e}"
        error = max(error, window_error)
    return error


@pytest.mark.parametrize("N,K,M", [(256, 128, 17), (512, 1024, 64), (272, 192, 130), (100, 64, 33),
                                   (1040, 2048, 257)])
@pytest.mark.parametrize("meta_kind", [0, 1])
def test_small_shapes(engine, oracle, gpu, N, K, M, meta_kind):
    run_case(engine, oracle, gpu, N, K, M, meta_kind, engine.F16, engine.F32)


def geometry_windows(N):
    """16-column windows (whole weight tiles) placed by the launch geometry of the GEMM kernels:
    a workgroup takes 16, 17 (16 + one tile shared by its four waves) or 20 consecutive tiles,
    four or five per wave.  Tiles 0, 5, 10 and 15 fall to the four waves of the first workgroup
    whichever of the three it is; tile 16 is the shared seventeenth tile of the first 17-tile
    workgroup; the others sit in an interior workgroup (its shared tile, and a tile of its last
    wave) and in the last workgroup, down to the last (possibly partly filled) tile."""
    tiles = (N + 15) // 16
    middle = tiles // 17 // 2
    picks = {0, 5, 10, 15, 16, 17 * middle + 16, 17 * middle + 13, 20 * (tiles // 20 // 2) + 19,
             16 * (tiles // 16 // 2) + 7, tiles - 20, tiles - 17, tiles - 1}
    return [(16 * t, min(16 * t + 16, N)) for t in sorted(t for t in picks if 0 <= t < tiles)]


@pytest.mark.parametrize("M", [512, 2048])
@pytest.mark.parametrize("N,K", [(17408, 5120), (5120, 17408)])
def test_prefill_shapes(engine, oracle, gpu, N, K, M):
    """Headline configuration 4 (27B MLP shapes at prefill row counts): bf16 scale/bias, fp16
    activations, fp16 output.  The oracle checks every row of x at full K on a dozen 16-column
    windows chosen from the launch geometry (see geometry_windows); the rest of the output is
    checked for finiteness and, below, against the streaming kernel."""
    run_case(engine, oracle, gpu, N, K, M, engine.META_BF16_PLANES, engine.F16, engine.F16,
             columns=geometry_windows(N))


def test_agrees_with_streaming_kernel_rows(engine, gpu):
    """Size-independent property: row m of the GEMM equals the M=1 streaming result for x[m]
    up to the fp16 weight rounding (the streaming kernel keeps the weight exact)."""
    N, K, M = 5120, 17408, 512
    quants, meta_a, meta_b = engine.synth_q4_affine(9, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 10, M, K).astype(np.float16)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        big = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        for m in (0, 255, 511):
            one = gpu.q4_linear(weight, x[m:m + 1], engine.F16, engine.F32)
            rms = float(np.sqrt(np.mean(one.astype(np.float64) ** 2)))
            assert float(np.max(np.abs(big[m] - one[0]))) <= 2e-3 * rms
    finally:
        weight.destroy()


@pytest.mark.parametrize("x_dtype,y_dtype", [("F32", "F32"), ("BF16", "BF16"), ("F16", "F16")])
def test_dtypes_and_residual(engine, oracle, gpu, x_dtype, y_dtype):
    run_case(engine, oracle, gpu, 384, 512, 40, engine.META_F16_INTERLEAVED, getattr(engine, x_dtype),
             getattr(engine, y_dtype), residual=True)


@pytest.mark.parametrize("forced", [None, "0,1", "3,2", "6,1", "7,2"])
def test_activation_range(engine, oracle, gpu, force, forced):
    """Activations far from fp16's range on the matrix-instruction path (64 rows): fp32 and bf16
    rows of magnitude 1e4, 1e-3 and 1e-6 and rows with entries beyond 65504.  Rows that are not
    fp16 are scaled by a power of two per row and fp32 rows go in as (value, remainder) pairs, so
    the gate against the fp16-weight oracle on the caller's own x holds whatever the magnitude
    (the reference keeps fp32 activations at any row count: whisper_turbo_encoder.c:128-176,
    qwen38_m3_layer.m:375-393); with a residual and through a K split."""
    N, K, M = 528, 1536, 64
    if forced:
        force("q4_gemm", forced)
    quants, meta_a, meta_b = engine.synth_q4_affine(191, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 192, M, K).copy()
    scales = np.ones(M, dtype=np.float32)
    scales[0::4], scales[1::4], scales[2::4] = 1e4, 1e-3, 1e-6
    x *= scales[:, None]
    x[3, 5], x[3, 77], x[7, 1000] = np.float32(1e5), np.float32(-2.5e5), np.float32(7e4)
    x_bf = bf16_bits(x).reshape(M, K)
    res = engine.synth_normal_f32(193, 1.0, M * N).reshape(M, N) * scales[:, None]
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    try:
        print(f"gemm activation range case forced={forced}", flush=True)
        y = gpu.q4_linear(weight, x, engine.F32, engine.F32, res, engine.F32)
        y_bf = gpu.q4_linear(weight, x_bf, engine.BF16, engine.F32)
    finally:
        weight.destroy()
    assert np.all(np.isfinite(y)) and np.all(np.isfinite(y_bf))
    ref = oracle.q4_linear(quants, meta_a, meta_b, engine.META_BF16_PLANES, N, K, x, oracle.X_F32, M,
                           weight_rounding=oracle.W_ROUND_F16) + res
    assert q4_relative_error(y, ref) <= 1e-3
    ref_bf = oracle.q4_linear(quants, meta_a, meta_b, engine.META_BF16_PLANES, N, K, x_bf, oracle.X_BF16, M,
                              weight_rounding=oracle.W_ROUND_F16)
    assert q4_relative_error(y_bf, ref_bf) <= 1e-3


@pytest.mark.parametrize("forced", ["0,1", "1,2", "2,1", "3,1", "3,3", "4,1", "5,2", "6,1", "6,3", "7,1", "7,2", "8,1", "8,2"])
def test_forced_decompositions(engine, oracle, gpu, forced, force):
    """Every kernel variant the host heuristic can pick (rows per block, tiles per wave, odd
    tile on the last wave), with and without K splits."""
    force("q4_gemm", forced)
    run_case(engine, oracle, gpu, 1104, 2176, 150, engine.META_BF16_PLANES, engine.F16, engine.F32)


@pytest.mark.parametrize("forced", ["6,1", "7,1", "7,2", "8,1"])
@pytest.mark.parametrize("K", [128, 256, 384, 640])
def test_pipelined_kernel_short_rows(engine, oracle, gpu, forced, K, force):
    """The pipelined kernel fetches three steps ahead and rotates its registers over three
    steps: rows of one to five 128-column steps exercise its prologue, the clamped fetches past
    the end and both remainder steps (alone and under a K split)."""
    force("q4_gemm", forced)
    run_case(engine, oracle, gpu, 560, K, 70, engine.META_BF16_PLANES, engine.F16, engine.F32)


@pytest.mark.parametrize("forced", ["6,1", "7,2", "8,1"])
@pytest.mark.parametrize("y_dtype", ["F16", "F32", "BF16"])
def test_pipelined_kernel_rows_of_odd_width(engine, oracle, gpu, forced, y_dtype, force):
    """N % 4 != 0: the pipelined kernel's four-at-once stores do not apply and every output leaves
    on its own (also the last, partly filled tile)."""
    force("q4_gemm", forced)
    run_case(engine, oracle, gpu, 1102, 384, 150, engine.META_BF16_PLANES, engine.F16,
             getattr(engine, y_dtype), residual=(y_dtype == "F32"))


@pytest.mark.parametrize("forced", ["6,1", "7,2", "8,2"])
@pytest.mark.parametrize("y_dtype,width", [("F16", 2), ("F32", 4), ("BF16", 2)])
def test_pipelined_kernel_output_alignment(engine, gpu, forced, y_dtype, width, force):
    """A device output pointer that is not 16-byte aligned takes the element-wise stores and must
    give the same bits as the aligned call."""
    force("q4_gemm", forced)
    N, K, M = 1104, 384, 150
    quants, meta_a, meta_b = engine.synth_q4_affine(21, 0.02, N, K, engine.META_BF16_PLANES)
    x = make_x(engine, 22, M, K).astype(np.float16)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, engine.META_BF16_PLANES)
    x_ptr = gpu.to_device(x)
    y_ptr = gpu.alloc(M * N * width + 64)
    kind = {2: np.uint16, 4: np.uint32}[width]
    try:
        outputs = []
        for shift in (0, width):  # aligned, then one element further
            print(f"gemm alignment case forced={forced} y={y_dtype} shift={shift}", flush=True)
            calls = engine.make_calls([((weight, y_ptr + shift), x_ptr, engine.F16, M, getattr(engine, y_dtype))])
            gpu.q4_sequence(calls)
            gpu.sync()
            outputs.append(gpu.download(y_ptr + shift, (M, N), kind))
        assert np.array_equal(outputs[0], outputs[1])
        assert np.any(outputs[0] != 0)
    finally:
        gpu.free(x_ptr)
        gpu.free(y_ptr)
        weight.destroy()


@pytest.mark.parametrize("N,K,M,splits", [(17408, 5120, 512, 1), (1104, 2176, 150, 2), (560, 384, 70, 1)])
def test_hand_scheduled_loads_match_compiler_managed_loads(engine, gpu, force, N, K, M, splits):
    """The pipelined kernel issues its weight loads as asm statements and waits for them with its
    own counted s_waitcnt; a second build of the same kernel (the 17-tile shape) uses ordinary loads
    whose waits the compiler places.  Same bits, or a wait no longer covers its loads."""
    kind = engine.META_BF16_PLANES
    quants, meta_a, meta_b = engine.synth_q4_affine(61, 0.02, N, K, kind)
    x = make_x(engine, 62, M, K).astype(np.float16)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, kind)
    try:
        force("q4_gemm", f"7,{splits}")
        print(f"gemm load forms N={N} K={K} M={M} splits={splits}", flush=True)
        scheduled = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        force("gemm_loads", "plain")
        plain = gpu.q4_linear(weight, x, engine.F16, engine.F32)
    finally:
        weight.destroy()
    assert np.array_equal(scheduled.view(np.uint32), plain.view(np.uint32))
    assert np.any(scheduled != 0)



@pytest.mark.parametrize("N,K,M,forced", [(1104, 2176, 400, "6,2"), (1104, 2176, 150, "7,3"), (5120, 640, 300, "8,1"),
                                          (560, 384, 70, "6,1")])
def test_block_order_does_not_change_the_bits(engine, gpu, force, N, K, M, forced):
    """The pipelined kernel either takes its blocks in launch order or renumbers them so that the
    row blocks of one tile block run on one XCD (numbers of blocks that are and are not multiples
    of eight, with K splits, ragged last blocks): every block is computed exactly once either way,
    so the outputs are the same bits."""
    kind = engine.META_BF16_PLANES
    quants, meta_a, meta_b = engine.synth_q4_affine(71, 0.02, N, K, kind)
    x = make_x(engine, 72, M, K).astype(np.float16)
    weight = gpu.q4_prepare(quants, meta_a, meta_b, N, K, kind)
    try:
        force("q4_gemm", forced)
        print(f"gemm block order N={N} K={K} M={M} forced={forced}", flush=True)
        force("gemm_order", "launch")
        in_launch_order = gpu.q4_linear(weight, x, engine.F16, engine.F32)
        force("gemm_order", "xcd")
        renumbered = gpu.q4_linear(weight, x, engine.F16, engine.F32)
    finally:
        weight.destroy()
    assert np.array_equal(in_launch_order.view(np.uint32), renumbered.view(np.uint32))
    assert np.any(renumbered != 0)
