"""The C-ABI library loads without a GPU, exports every symbol the headers declare, and
answers bad arguments with status 2 and a message instead of crashing."""
import ctypes
import re
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[1]


def declared_functions():
    names = set()
    for header in ("mi355q.h", "mi355q_synth.h"):
        text = (ROOT / "include" / header).read_text()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(mi355q_[a-z0-9_]+)\s*\(", text))
    return names


def test_every_declared_symbol_is_exported_and_bound(engine):
    lib = engine.library()
    declared = declared_functions()
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    assert declared == set(engine.SIGNATURES), declared ^ set(engine.SIGNATURES)


def test_null_arguments_are_rejected_without_a_device(engine):
    lib = engine.library()
    err = ctypes.create_string_buffer(128)
    assert lib.mi355q_context_create(0, None, err, len(err)) == engine.ERROR_INVALID
    assert err.value
    assert lib.mi355q_context_create(-1, ctypes.byref(ctypes.c_void_p()), None, 0) == engine.ERROR_INVALID
    assert lib.mi355q_sync(None, err, len(err)) == engine.ERROR_INVALID
    assert lib.mi355q_q4_linear(None, None, None, 0, 1, None, 0, None, 0, 0, err, len(err)) == engine.ERROR_INVALID
    out = ctypes.c_void_p()
    assert lib.mi355q_q4_weight_prepare(None, None, None, None, 16, 64, 0, 0, ctypes.byref(out), err,
                                        len(err)) == engine.ERROR_INVALID
    lib.mi355q_context_destroy(None)
    lib.mi355q_q4_weight_destroy(None)
    assert lib.mi355q_q4_weight_image_bytes(None) == 0


def test_synthetic_inputs_are_deterministic_and_well_formed(engine):
    a = engine.synth_normal_f32(9, 0.02, 100001)
    b = engine.synth_normal_f32(9, 0.02, 100001)
    assert np.array_equal(a, b) and not np.array_equal(a, engine.synth_normal_f32(10, 0.02, 100001))
    assert abs(float(a.mean())) < 3e-4 and abs(float(a.std()) - 0.02) < 3e-4
    h = engine.synth_normal_f16(9, 0.02, 4096)
    assert np.array_equal(h, a[:4096].astype(np.float16))
    for kind in (engine.META_F16_INTERLEAVED, engine.META_BF16_PLANES):
        quants, meta_a, meta_b = engine.synth_q4_affine(3, 0.02, 24, 192, kind)
        w = engine.synth_normal_f32(3, 0.02, 24 * 192).reshape(24, 192)
        q2, a2, b2 = engine.quantize_q4_affine(w, kind)
        assert np.array_equal(quants, q2) and np.array_equal(meta_a, a2)
        assert (meta_b is None and b2 is None) or np.array_equal(meta_b, b2)
    assert engine.library().mi355q_quantize_q4_affine(w.ctypes.data, 24, 100, 0, quants.ctypes.data,
                                                      meta_a.ctypes.data, None) == engine.ERROR_INVALID


def test_affine_quantizer_error_bound(engine, oracle):
    """|w - (s*q + b)| <= s/2 (+ metadata rounding) inside each group: dequantize with the oracle."""
    N, K = 16, 256
    w = engine.synth_normal_f32(5, 0.02, N * K).reshape(N, K)
    for kind in (engine.META_F16_INTERLEAVED, engine.META_BF16_PLANES):
        quants, meta_a, meta_b = engine.quantize_q4_affine(w, kind)
        eye = np.eye(K, dtype=np.float32)
        dense = oracle.q4_linear(quants, meta_a, meta_b, kind, N, K, eye, oracle.X_F32, K).T
        step = (w.reshape(N, K // 64, 64).max(-1) - w.reshape(N, K // 64, 64).min(-1)) / 15.0
        bound = np.repeat(step, 64, axis=1) * (0.5 + 15 * 2.0 ** -8) + 2.0 ** -8 * np.abs(w).max()
        assert np.all(np.abs(dense - w) <= bound)
        codes = np.frombuffer(quants.tobytes(), dtype=np.uint8)
        assert ((codes & 15).max() == 15 or (codes >> 4).max() == 15) and ((codes & 15).min() == 0)
