"""ctypes loader for the CPU oracle (oracle/mi355q_oracle.c) and, where it was
built, the reference's own compiled C (oracle/_ref).  TEST INFRASTRUCTURE ONLY:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg,
never by the engine.
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ORACLE_PATH = HERE / "libmi355q_oracle.so"
REF_QWEN35_PATH = HERE / "_ref" / "libref_qwen35.so"
REF_MINIMINDO_PATH = HERE / "_ref" / "libref_minimindo.so"

META_F16_INTERLEAVED, META_BF16_PLANES = 0, 1
X_F16, X_F32, X_BF16 = 0, 1, 2
W_EXACT, W_ROUND_F16, W_ROUND_BF16 = 0, 1, 2
ACC_F32_SEQUENTIAL, ACC_F64 = 0, 1

_c = ctypes
_vp, _u32, _sz, _int = _c.c_void_p, _c.c_uint32, _c.c_size_t, _c.c_int
_libs: dict = {}


def _p(array):
    if array is None:
        return None
    assert array.flags["C_CONTIGUOUS"]
    return array.ctypes.data_as(_vp)


def lib() -> ctypes.CDLL:
    if "oracle" not in _libs:
        if not ORACLE_PATH.exists():
            raise FileNotFoundError(f"{ORACLE_PATH} is not built; run `make -C {HERE}`")
        l = ctypes.CDLL(os.fspath(ORACLE_PATH))
        l.orc_f32_to_f16.restype, l.orc_f32_to_f16.argtypes = _c.c_uint16, [_c.c_float]
        l.orc_f16_to_f32.restype, l.orc_f16_to_f32.argtypes = _c.c_float, [_c.c_uint16]
        l.orc_f32_to_bf16.restype, l.orc_f32_to_bf16.argtypes = _c.c_uint16, [_c.c_float]
        l.orc_bf16_to_f32.restype, l.orc_bf16_to_f32.argtypes = _c.c_float, [_c.c_uint16]
        l.orc_q4_linear.restype = _int
        l.orc_q4_linear.argtypes = [_vp, _vp, _vp, _int, _u32, _u32, _vp, _int, _u32, _int,
                                    _int, _u32, _u32, _vp, _int]
        l.orc_q8_affine_linear.restype = _int
        l.orc_q8_affine_linear.argtypes = [_vp, _vp, _vp, _int, _u32, _u32, _vp, _int, _u32, _int, _int, _vp]
        l.orc_q8rows_f32_linear.restype = None
        l.orc_q8rows_f32_linear.argtypes = [_vp, _u32, _u32, _vp, _u32, _vp]
        l.orc_causal_q8_windows.restype = None
        l.orc_causal_q8_windows.argtypes = [_vp, _vp, _u32, _u32, _u32, _int, _vp, _vp]
        l.orc_w8a8_conv.restype = None
        l.orc_w8a8_conv.argtypes = [_vp, _u32, _u32, _vp, _vp, _u32, _vp, _vp]
        l.orc_q4_dot_f16x_seq.restype = _c.c_float
        l.orc_q4_dot_f16x_seq.argtypes = [_vp, _vp, _vp, _sz, _sz]
        l.orc_q4_dot_f32x_seq.restype = _c.c_float
        l.orc_q4_dot_f32x_seq.argtypes = [_vp, _vp, _vp, _sz, _sz]
        l.orc_q4_dequantize_row.restype = _int
        l.orc_q4_dequantize_row.argtypes = [_vp, _vp, _vp, _int, _u32, _u32, _vp]
        l.orc_sym128_gemv.restype = None
        l.orc_sym128_gemv.argtypes = [_vp, _int, _u32, _u32, _vp, _vp, _int]
        l.orc_sym128_dequantize_row.restype = None
        l.orc_sym128_dequantize_row.argtypes = [_vp, _int, _u32, _u32, _vp]
        l.orc_sym128_to_affine.restype = None
        l.orc_sym128_to_affine.argtypes = [_vp, _int, _u32, _u32, _vp, _vp, _vp]
        l.orc_sym128_gemm.restype = None
        l.orc_sym128_gemm.argtypes = [_vp, _vp, _sz, _sz, _sz, _vp, _vp, _int]
        l.orc_quantize_i8.restype = _c.c_float
        l.orc_quantize_i8.argtypes = [_vp, _vp, _u32]
        l.orc_i8_dot.restype = _c.c_int32
        l.orc_i8_dot.argtypes = [_vp, _vp, _u32]
        l.orc_w8a8_linear.restype = None
        l.orc_w8a8_linear.argtypes = [_vp, _u32, _u32, _vp, _vp, _u32, _vp, _vp, _vp, _int]
        l.orc_q8_weight_quantize.restype = None
        l.orc_q8_weight_quantize.argtypes = [_vp, _u32, _u32, _vp]
        l.orc_recipe_qwen38_weights.restype = None
        l.orc_recipe_qwen38_weights.argtypes = [_u32, _sz, _vp, _vp]
        l.orc_probe_read_gib_per_s.restype = _c.c_double
        l.orc_probe_read_gib_per_s.argtypes = [_sz, _int, _c.c_double, _vp]
        _libs["oracle"] = l
    return _libs["oracle"]


def ref_qwen35():
    """The reference's compiled q4_gemv / dequantize_q4_row, or None if not built."""
    if "qwen35" not in _libs:
        if not REF_QWEN35_PATH.exists():
            return None
        l = ctypes.CDLL(os.fspath(REF_QWEN35_PATH))
        l.ref_qwen35_q4_gemv.restype = None
        l.ref_qwen35_q4_gemv.argtypes = [_vp, _int, _u32, _u32, _vp, _vp]
        l.ref_qwen35_dequantize_q4_row.restype = None
        l.ref_qwen35_dequantize_q4_row.argtypes = [_vp, _int, _u32, _u32, _u32, _vp]
        _libs["qwen35"] = l
    return _libs["qwen35"]


def ref_minimindo():
    """The reference's compiled W8A8 functions, or None if not built."""
    if "minimindo" not in _libs:
        if not REF_MINIMINDO_PATH.exists():
            return None
        l = ctypes.CDLL(os.fspath(REF_MINIMINDO_PATH))
        l.ref_minimindo_quantize_i8.restype = _c.c_float
        l.ref_minimindo_quantize_i8.argtypes = [_vp, _vp, _u32]
        l.ref_minimindo_q8_i8_dot.restype = _c.c_int32
        l.ref_minimindo_q8_i8_dot.argtypes = [_vp, _vp, _u32]
        l.ref_minimindo_matrix_sequence_i8_quantized.restype = None
        l.ref_minimindo_matrix_sequence_i8_quantized.argtypes = [_vp, _u32, _u32, _vp, _vp,
                                                                 _u32, _vp, _vp]
        _libs["minimindo"] = l
    return _libs["minimindo"]


def ref_mimi():
    """The reference's compiled streaming convolution (minimindo_mimi.c), or None if not built."""
    if "mimi" not in _libs:
        path = REF_MINIMINDO_PATH.with_name("libref_mimi.so")
        if not path.exists():
            return None
        l = ctypes.CDLL(os.fspath(path))
        l.ref_mimi_causal_q8_windows.restype = _int
        l.ref_mimi_causal_q8_windows.argtypes = [_vp, _vp, _u32, _u32, _u32, _vp, _vp]
        l.ref_mimi_stream_conv1d.restype = _int
        l.ref_mimi_stream_conv1d.argtypes = [_vp, _vp, _u32, _u32, _u32, _vp, _vp, _u32, _vp]
        _libs["mimi"] = l
    return _libs["mimi"]


def ref_thinker():
    """The reference's compiled Q8-row x fp32 product (minimindo_thinker.c), or None if not built."""
    if "thinker" not in _libs:
        path = REF_MINIMINDO_PATH.with_name("libref_thinker.so")
        if not path.exists():
            return None
        l = ctypes.CDLL(os.fspath(path))
        l.ref_thinker_q8_matmul_sequence.restype = None
        l.ref_thinker_q8_matmul_sequence.argtypes = [_vp, _u32, _u32, _vp, _u32, _vp]
        _libs["thinker"] = l
    return _libs["thinker"]


# ---- convenience wrappers ---------------------------------------------------

def q4_linear(quants, meta_a, meta_b, meta_kind, N, K, x, x_kind, M,
              weight_rounding=W_EXACT, accumulate=ACC_F64, rows=None, threads=0):
    """y [M][N] float64; rows=(begin,end) restricts the computed output rows
    (the rest is left at zero)."""
    x = np.ascontiguousarray(x)
    y = np.zeros((M, N), dtype=np.float64)
    begin, end = rows if rows is not None else (0, N)
    status = lib().orc_q4_linear(_p(quants), _p(meta_a), _p(meta_b), meta_kind, N, K, _p(x),
                                 x_kind, M, weight_rounding, accumulate, begin, end, _p(y),
                                 threads)
    if status != 0:
        raise ValueError(f"orc_q4_linear status {status}")
    return y


def q8_affine_linear(quants, meta_a, meta_b, meta_kind, N, K, x, x_kind, M,
                     weight_rounding=W_EXACT, accumulate=ACC_F64):
    """Affine Q8 g64 (u8 quants [N][K]): y [M][N] float64."""
    x = np.ascontiguousarray(x)
    y = np.zeros((M, N), dtype=np.float64)
    status = lib().orc_q8_affine_linear(_p(quants), _p(meta_a), _p(meta_b), meta_kind, N, K, _p(x), x_kind, M,
                                        weight_rounding, accumulate, _p(y))
    if status != 0:
        raise ValueError(f"orc_q8_affine_linear status {status}")
    return y


def q8rows_f32_linear(records, N, K, x):
    """Q8 rows (fp32 scale + K int8 each) x fp32 x [M][K] -> fp32 [M][N]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty((x.shape[0], N), dtype=np.float32)
    lib().orc_q8rows_f32_linear(_p(records), N, K, _p(x), x.shape[0], _p(out))
    return out


def q4_dequantize_rows(quants, meta_a, meta_b, meta_kind, K, rows):
    """fp32 [len(rows)][K]: scale * q + bias, unrounded."""
    out = np.empty((len(rows), K), dtype=np.float32)
    for i, row in enumerate(rows):
        status = lib().orc_q4_dequantize_row(_p(quants), _p(meta_a), _p(meta_b), meta_kind, K, int(row),
                                             _p(out[i]))
        if status != 0:
            raise ValueError(f"orc_q4_dequantize_row status {status}")
    return out


def sym128_gemv(records, output_blocked, rows, columns, x, threads=0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(rows, dtype=np.float32)
    lib().orc_sym128_gemv(_p(records), int(output_blocked), rows, columns, _p(x), _p(y), threads)
    return y


def sym128_to_affine(records, output_blocked, rows, columns):
    groups = rows * (columns // 64)
    quants = np.empty(groups * 32, dtype=np.uint8)
    scales = np.empty(groups, dtype=np.uint16)
    biases = np.empty(groups, dtype=np.uint16)
    lib().orc_sym128_to_affine(_p(records), int(output_blocked), rows, columns, _p(quants),
                               _p(scales), _p(biases))
    return quants, scales, biases


def quantize_i8(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    q = np.empty((M, K), dtype=np.int8)
    scales = np.empty(M, dtype=np.float32)
    for m in range(M):
        scales[m] = lib().orc_quantize_i8(_p(x[m]), _p(q[m]), K)
    return q, scales


def w8a8_linear(weights, N, K, q, x_scales, bias=None, threads=0):
    M = q.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.int32)
    lib().orc_w8a8_linear(_p(weights), N, K, _p(np.ascontiguousarray(q)),
                          _p(np.ascontiguousarray(x_scales, dtype=np.float32)), M, _p(bias),
                          _p(out), _p(acc), threads)
    return out, acc


def causal_q8_windows(x, history, kernel, pairs=False):
    """x [channels][length] fp32 -> (q [length][columns] int8, scales [length])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    channels, length = x.shape
    columns = channels * (2 if pairs else kernel)
    q = np.empty((length, columns), dtype=np.int8)
    scales = np.empty(length, dtype=np.float32)
    if history is not None:
        history = np.ascontiguousarray(history, dtype=np.float32)
    lib().orc_causal_q8_windows(_p(x), _p(history), channels, kernel, length, int(pairs), _p(q), _p(scales))
    return q, scales


def w8a8_conv(weights, N, K, q, x_scales, bias=None):
    """Channel-major [N][M] output of the streaming convolution's W8A8 product."""
    M = q.shape[0]
    out = np.empty((N, M), dtype=np.float32)
    lib().orc_w8a8_conv(_p(weights), N, K, _p(np.ascontiguousarray(q)),
                        _p(np.ascontiguousarray(x_scales, dtype=np.float32)), M, _p(bias), _p(out))
    return out


def q8_weight_quantize(w):
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    rows = np.empty(N * (4 + K), dtype=np.uint8)
    lib().orc_q8_weight_quantize(_p(w), N, K, _p(rows))
    return rows


def probe_read_gib_per_s(nbytes=256 << 20, threads=1, seconds=0.5):
    """Host read bandwidth (GiB/s) at `threads` threads, the reference's target-probe measurement."""
    return lib().orc_probe_read_gib_per_s(nbytes, threads, seconds, None)

