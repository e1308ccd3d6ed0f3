"""Pins the oracle's number-format conversions against independent implementations:
numpy's float16 (exhaustive over all 65536 bit patterns, and on random / boundary
fp32 inputs) and a numpy integer restatement + torch.bfloat16 for bf16."""
import numpy as np
import pytest

from conftest import bf16_bits


def test_f16_to_f32_exhaustive(oracle):
    lib = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    expect = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.orc_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(expect)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), expect[~nan].view(np.uint32))


def test_f32_to_f16_roundtrip_exhaustive(oracle):
    lib = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    values = bits.view(np.float16).astype(np.float32)
    for b, v in zip(bits.tolist(), values.tolist()):
        if v != v:
            assert (lib.orc_f32_to_f16(v) & 0x7C00) == 0x7C00 and (lib.orc_f32_to_f16(v) & 0x3FF)
        else:
            assert lib.orc_f32_to_f16(v) == b


def test_f32_to_f16_rounding_matches_numpy(oracle):
    lib = oracle.lib()
    rng = np.random.default_rng(0)
    samples = [rng.standard_normal(20000).astype(np.float32) * s
               for s in (1.0, 1e-3, 1e-5, 1e-7, 3e4, 7e4)]
    # exact ties and their neighbours around every fp16 spacing
    halves = np.arange(0, 65535, dtype=np.uint16).view(np.float16).astype(np.float64)
    finite = halves[np.isfinite(halves)]
    mid = ((finite[:-1] + finite[1:]) / 2).astype(np.float32)[::7]
    samples += [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e9, -1e9, np.inf, -np.inf,
                          2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -26], dtype=np.float32)]
    values = np.concatenate(samples).astype(np.float32)
    with np.errstate(over="ignore"):
        expect = values.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f32_to_f16(float(v)) for v in values], dtype=np.uint16)
    assert np.array_equal(got, expect)


def test_bf16_conversions(oracle):
    lib = oracle.lib()
    rng = np.random.default_rng(1)
    values = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 0.05,
        # ties: low 16 bits exactly 0x8000 with even and odd kept bit
        np.array([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x3F807FFF, 0xBF808000, 0x00008000, 0x7F7FFFFF],
                 dtype=np.uint32).view(np.float32),
    ])
    expect = bf16_bits(values)
    got = np.array([lib.orc_f32_to_bf16(float(v)) for v in values], dtype=np.uint16)
    assert np.array_equal(got, expect)
    torch = pytest.importorskip("torch")
    finite = values[np.isfinite(values) & (np.abs(values) < 1e38)]
    via_torch = torch.from_numpy(finite.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bf16_bits(finite), via_torch)
    back = np.array([lib.orc_bf16_to_f32(int(b)) for b in expect[:1000]], dtype=np.float32)
    assert np.array_equal(back.view(np.uint32), expect[:1000].astype(np.uint32) << 16)
