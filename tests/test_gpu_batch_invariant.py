"""Decode-identical verify batches: with the context option "batch_invariant" = "1", row m of an
M-row call of the streaming linear (M <= 8, or 4 rows of fp32) is bit for bit the one-row call on
x[m] - what the reference's exact batched kernels give and its parity test asserts
(qwen38_prefill.metal:5-9,142-248; tests/qwen38_m3_prefill_parity_test.c:115-199).  Without the
option the launch shape follows the row count and the rows agree only within the tolerance."""
import numpy as np
import pytest

from conftest import q4_relative_error

pytestmark = pytest.mark.gpu

LAYER = {"q": (6144, 5120), "k": (1024, 5120), "o": (5120, 6144), "gate": (17408, 5120), "down": (5120, 17408)}


@pytest.fixture(scope="module")
def weights(engine, gpu):
    kind = engine.META_BF16_PLANES
    images = {name: engine.synth_q4_affine(300 + i, 0.02, N, K, kind) for i, (name, (N, K)) in enumerate(LAYER.items())}
    prepared = {name: gpu.q4_prepare(*images[name], *LAYER[name], kind) for name in LAYER}
    yield images, prepared
    for weight in prepared.values():
        weight.destroy()


@pytest.mark.parametrize("name", list(LAYER))
@pytest.mark.parametrize("M", [2, 4, 8])
def test_rows_of_a_batch_equal_one_row_calls(engine, oracle, gpu, force, weights, name, M):
    """The five 27B shapes (down is cut in K slices), fp16 activations."""
    images, prepared = weights
    N, K = LAYER[name]
    x = np.stack([engine.synth_normal_f16(900 + m, 1.0, K) for m in range(M)])
    print(f"batch invariant {name} M={M}", flush=True)
    force("batch_invariant", "1")
    batch = gpu.q4_linear(prepared[name], x, engine.F16, engine.F32)
    for m in range(M):
        one = gpu.q4_linear(prepared[name], x[m:m + 1], engine.F16, engine.F32)
        assert np.array_equal(batch[m].view(np.uint32), one[0].view(np.uint32)), f"row {m}"
    reference = oracle.q4_linear(*images[name], engine.META_BF16_PLANES, N, K, x, oracle.X_F16, M)
    assert q4_relative_error(batch, reference) <= 1e-3


@pytest.mark.parametrize("M", [2, 4, 8])
def test_shared_activation_and_fused_launches(engine, gpu, force, weights, M):
    """q|k in one launch, and the fused gate|up-SiLU pair (here gate with itself)."""
    _, prepared = weights
    x = np.stack([engine.synth_normal_f16(950 + m, 1.0, 5120) for m in range(M)])
    force("batch_invariant", "1")
    print(f"batch invariant multi and fused M={M}", flush=True)
    batch = gpu.q4_linear_multi([prepared["q"], prepared["k"]], x, engine.F16, engine.F32)
    fused = gpu.q4_gate_up_silu(prepared["gate"], prepared["gate"], x, engine.F16, engine.F32)
    for m in range(M):
        one = gpu.q4_linear_multi([prepared["q"], prepared["k"]], x[m:m + 1], engine.F16, engine.F32)
        for got, want in zip(batch, one):
            assert np.array_equal(got[m].view(np.uint32), want[0].view(np.uint32)), f"row {m}"
        one = gpu.q4_gate_up_silu(prepared["gate"], prepared["gate"], x[m:m + 1], engine.F16, engine.F32)
        assert np.array_equal(fused[m].view(np.uint32), one[0].view(np.uint32)), f"fused row {m}"


@pytest.mark.parametrize("M", [2, 4])
def test_fp32_rows(engine, gpu, force, weights, M):
    """fp32 activations travel as (value, remainder) pairs: up to four rows stay within eight."""
    _, prepared = weights
    x = np.stack([engine.synth_normal_f32(970 + m, 1.0, 17408) for m in range(M)])
    force("batch_invariant", "1")
    print(f"batch invariant fp32 down M={M}", flush=True)
    batch = gpu.q4_linear(prepared["down"], x, engine.F32, engine.F32)
    for m in range(M):
        one = gpu.q4_linear(prepared["down"], x[m:m + 1], engine.F32, engine.F32)
        assert np.array_equal(batch[m].view(np.uint32), one[0].view(np.uint32)), f"row {m}"


def test_without_the_option_shapes_follow_the_row_count(engine, gpu, weights):
    """The default picks the fastest launch shape per row count: rows agree within the tolerance,
    and for o_proj at eight rows (four waves instead of eight) not bit for bit - which is what the
    option is for."""
    _, prepared = weights
    x = np.stack([engine.synth_normal_f16(990 + m, 1.0, 6144) for m in range(8)])
    batch = gpu.q4_linear(prepared["o"], x, engine.F16, engine.F32)
    one = gpu.q4_linear(prepared["o"], x[3:4], engine.F16, engine.F32)
    assert q4_relative_error(batch[3:4], one.astype(np.float64)) <= 1e-3
    assert not np.array_equal(batch[3].view(np.uint32), one[0].view(np.uint32))
