"""GPU tests of the one-launch MLP: gate|up with SiLU and the down projection that reads its
output, queued as two consecutive calls of a sequence, go out as one kernel whose second half
waits, 128 columns at a time, for the first half's outputs (the reference encodes the two
kernels into one command buffer, qwen38_m3_layer.m:314-336; qwen38_q4.metal:129-191).

The one-launch form is behind the context option "chain" = "1".  Gates: the one-launch pair is
bit-equal to the same two calls as two launches of whole tiles (the launch shapes the pair shares;
option "half_tiles" = "0" keeps the two-launch form on them), and both match the oracle: h = silu(gate . x) * (up . x) rounded to fp16, and
y = down . h (+ residual) on the GPU's own h, within the Q4 gate of 1e-3."""
import numpy as np
import pytest

from conftest import q4_relative_error

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-3
BF16 = "META_BF16_PLANES"
F16M = "META_F16_INTERLEAVED"


class Mlp:
    """gate, up [hidden -> inner] and down [inner -> hidden] on the GPU, with device buffers."""

    def __init__(self, engine, gpu, hidden, inner, meta_kind, max_rows, seed=50):
        self.engine, self.gpu, self.hidden, self.inner, self.meta_kind = engine, gpu, hidden, inner, meta_kind
        self.images = [engine.synth_q4_affine(seed + i, 0.02, N, K, meta_kind)
                       for i, (N, K) in enumerate(((inner, hidden), (inner, hidden), (hidden, inner)))]
        self.weights = [gpu.q4_prepare(*image, N, K, meta_kind)
                        for image, (N, K) in zip(self.images, ((inner, hidden), (inner, hidden), (hidden, inner)))]
        self.x = np.stack([engine.synth_normal_f16(seed + 10 + m, 1.0, hidden) for m in range(max_rows)])
        self.residual = np.stack([engine.synth_normal_f32(seed + 40 + m, 1.0, hidden) for m in range(max_rows)])
        self.x_ptr = gpu.to_device(self.x)
        self.residual_ptr = gpu.to_device(self.residual)
        self.h_ptr = gpu.alloc(max_rows * inner * 2)
        self.y_ptr = gpu.alloc(max_rows * hidden * 4)

    def calls(self, M, residual=False):
        engine = self.engine
        gate, up, down = self.weights
        target = (down, self.y_ptr, self.residual_ptr) if residual else (down, self.y_ptr)
        return engine.make_calls([
            ([(gate, self.h_ptr), (up, None)], self.x_ptr, engine.F16, M, engine.F16, engine.F32,
             engine.FUSE_GATE_UP_SILU),
            (target, self.h_ptr, engine.F16, M, engine.F32, engine.F32)])

    def run(self, M, residual=False):
        """(h, y) of one pass; the buffers are poisoned first so that nothing survives from a previous one."""
        gpu = self.gpu
        gpu.upload(self.h_ptr, np.full(M * self.inner, 0x7E00, dtype=np.uint16))  # fp16 NaN
        gpu.upload(self.y_ptr, np.full(M * self.hidden, np.nan, dtype=np.float32))
        gpu.q4_sequence(self.calls(M, residual))
        gpu.sync()
        return (gpu.download(self.h_ptr, (M, self.inner), np.float16),
                gpu.download(self.y_ptr, (M, self.hidden), np.float32))

    def check_against_oracle(self, oracle, M, h, y, residual=False):
        kind = getattr(self.engine, self.meta_kind) if isinstance(self.meta_kind, str) else self.meta_kind
        g = oracle.q4_linear(*self.images[0], kind, self.inner, self.hidden, self.x[:M], oracle.X_F16, M)
        u = oracle.q4_linear(*self.images[1], kind, self.inner, self.hidden, self.x[:M], oracle.X_F16, M)
        assert q4_relative_error(h.astype(np.float64), g / (1.0 + np.exp(-g)) * u) <= TOLERANCE
        reference = oracle.q4_linear(*self.images[2], kind, self.hidden, self.inner, h, oracle.X_F16, M)
        if residual:
            reference = reference + self.residual[:M].astype(np.float64)
        assert q4_relative_error(y, reference) <= TOLERANCE

    def destroy(self):
        for pointer in (self.x_ptr, self.residual_ptr, self.h_ptr, self.y_ptr):
            self.gpu.free(pointer)
        for weight in self.weights:
            weight.destroy()


@pytest.fixture(scope="module")
def mlp_27b(engine, gpu):
    mlp = Mlp(engine, gpu, 5120, 17408, engine.META_BF16_PLANES, 8)
    yield mlp
    mlp.destroy()


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_27b_mlp_one_launch_equals_two(engine, oracle, gpu, force, mlp_27b, M):
    """The 27B MLP: one launch for the pair wherever the two linears' launch shapes allow it
    (four-wave workgroups for both: at four rows the down projection takes eight), bit-equal to
    the two launches, both right."""
    print(f"chained 27B MLP M={M}", flush=True)
    before = gpu.get("chained_launches")
    force("half_tiles", "0")
    h0, y0 = mlp_27b.run(M, residual=True)
    assert gpu.get("chained_launches") == before  # off unless asked for
    force("chain", "1")
    h1, y1 = mlp_27b.run(M, residual=True)
    chained = gpu.get("chained_launches") - before
    assert chained == (0 if M == 4 else 1)
    assert np.array_equal(h1.view(np.uint16), h0.view(np.uint16))
    assert np.array_equal(y1.view(np.uint32), y0.view(np.uint32))
    mlp_27b.check_against_oracle(oracle, M, h1, y1, residual=True)


def test_repeated_and_alternating_shapes(engine, oracle, gpu, force, mlp_27b):
    """The step counters count launches and are never reset between launches of one shape; a pair
    of another shape in between starts them over.  Every pass gives the first pass's bits."""
    small = Mlp(engine, gpu, 1024, 12288, engine.META_F16_INTERLEAVED, 2, seed=90)
    try:
        print("chained passes, two shapes alternating", flush=True)
        force("chain", "1")
        before = gpu.get("chained_launches")
        first_big = mlp_27b.run(1)
        first_small = small.run(2)
        assert gpu.get("chained_launches") == before + 2
        for index in range(6):
            for mlp, rows, first in ((mlp_27b, 1, first_big), (small, 2, first_small), (mlp_27b, 1, first_big)):
                h, y = mlp.run(rows)
                assert np.array_equal(h.view(np.uint16), first[0].view(np.uint16)), index
                assert np.array_equal(y.view(np.uint32), first[1].view(np.uint32)), index
        small.check_against_oracle(oracle, 2, *first_small)
    finally:
        small.destroy()


def test_bounded_wait_gives_up_and_reports(engine, gpu, force, mlp_27b):
    """The consumers' wait is bounded: asked to wait for a count the producers cannot reach, every
    wave gives up after the configured polls, the kernel ends, and the next wait on the stream
    reports status 1.  The launches after it are right again."""
    print("chained 27B MLP with the announcement withheld", flush=True)
    force("chain", "1")
    h_good, y_good = mlp_27b.run(1)
    force("chain_withhold", "1")
    force("chain_spin_limit", "40")
    before = gpu.get("chained_launches")
    with pytest.raises(engine.Mi355qError) as info:
        mlp_27b.run(1)
    assert info.value.status == engine.ERROR_RUNTIME
    assert gpu.get("chained_launches") == before + 1
    gpu.set_option("chain_withhold", None)
    gpu.set_option("chain_spin_limit", None)
    h, y = mlp_27b.run(1)
    assert np.array_equal(h.view(np.uint16), h_good.view(np.uint16))
    assert np.array_equal(y.view(np.uint32), y_good.view(np.uint32))


def test_pairs_that_stay_two_launches(engine, gpu, force, mlp_27b):
    """fp32 output of the first call, another activation pointer for the second, or a graph
    being recorded: two launches, as before."""
    gate, up, down = mlp_27b.weights
    h32 = gpu.alloc(17408 * 4)
    force("chain", "1")
    try:
        before = gpu.get("chained_launches")
        gpu.q4_sequence(engine.make_calls([
            ([(gate, h32), (up, None)], mlp_27b.x_ptr, engine.F16, 1, engine.F32, engine.F32, engine.FUSE_GATE_UP_SILU),
            ((down, mlp_27b.y_ptr), mlp_27b.h_ptr, engine.F16, 1, engine.F32, engine.F32)]))
        gpu.sync()
        graph = gpu.q4_sequence_record(mlp_27b.calls(1))
        gpu.graph_launch(graph)
        gpu.sync()
        gpu.graph_destroy(graph)
        # the recording ran the calls once for real (one chained launch); the capture itself did not chain
        assert gpu.get("chained_launches") == before + 1
    finally:
        gpu.free(h32)
