"""GPU: the Mimi decoder's streaming convolution (quantized causal windows + channel-major W8A8
product) through the C ABI, bit-exact against golden vectors of the reference's own C
(causal_q8_windows, stream_conv1d: minimindo_mimi.c:552-598,869-917) and against the oracle
at a decoder-sized shape."""
import pathlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = pathlib.Path(__file__).parent / "golden" / "mimi_stream_conv.npz"


def test_stream_conv_matches_reference_golden_bitwise(engine, gpu):
    golden = np.load(GOLDEN, allow_pickle=False)
    for tag, chunks in (("k7", 3), ("k1", 1)):
        C, O, kernel = (int(v) for v in golden[f"{tag}_shape"])
        weight = gpu.w8a8_prepare(golden[f"{tag}_rows"], O, C * kernel)
        try:
            for index in range(chunks):
                print(f"mimi conv {tag} chunk {index}", flush=True)
                x = golden[f"{tag}_{index}_x"]
                history = golden[f"{tag}_{index}_history_before"] if kernel > 1 else None
                q, scales = gpu.causal_q8_windows(x, history, kernel)
                assert np.array_equal(q, golden[f"{tag}_{index}_q"])
                assert np.array_equal(scales.view(np.uint32), golden[f"{tag}_{index}_scales"].view(np.uint32))
                y, _ = gpu.w8a8_linear(weight, O, q, scales, golden[f"{tag}_bias"], channel_major=True)
                assert np.array_equal(y.view(np.uint32), golden[f"{tag}_{index}_y"].view(np.uint32))
        finally:
            gpu.w8a8_destroy(weight)


@pytest.mark.parametrize("pairs", [False, True])
def test_decoder_sized_conv_against_oracle(engine, oracle, gpu, pairs):
    """512 channels, kernel 7 (3584 columns) -> 1024 outputs over 50 positions, and the
    two-sample windows of a transposed convolution (1024 columns)."""
    rng = np.random.default_rng(17)
    C, O, kernel, L = 512, 1024, 7, 50
    columns = C * (2 if pairs else kernel)
    x = rng.standard_normal((C, L)).astype(np.float32)
    x[:, 3] = 0.0
    history = rng.standard_normal((C, 1 if pairs else kernel - 1)).astype(np.float32)
    rows = oracle.q8_weight_quantize((rng.standard_normal((O, columns)) * 0.02).astype(np.float32))
    bias = rng.standard_normal(O).astype(np.float32)
    weight = gpu.w8a8_prepare(rows, O, columns)
    try:
        print(f"mimi conv sized pairs={pairs}", flush=True)
        q, scales = gpu.causal_q8_windows(x, history, kernel, pairs=pairs)
        y, acc = gpu.w8a8_linear(weight, O, q, scales, bias, channel_major=True)
    finally:
        gpu.w8a8_destroy(weight)
    expect_q, expect_scales = oracle.causal_q8_windows(x, history, kernel, pairs=pairs)
    assert np.array_equal(q, expect_q)
    assert np.array_equal(scales.view(np.uint32), expect_scales.view(np.uint32))
    expect = oracle.w8a8_conv(rows, O, columns, expect_q, expect_scales, bias)
    assert np.array_equal(y.view(np.uint32), expect.view(np.uint32))
