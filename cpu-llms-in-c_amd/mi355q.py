"""ctypes binding of libmi355q.so (include/mi355q.h, include/mi355q_synth.h).

Used by the tests, the smoke check and bench.py.  It only loads the library
that `make -C cpu-llms-in-c_amd/csrc` (or __graft_entry__.build) has built in
cpu-llms-in-c_amd/lib; there is no fallback of any kind: a missing library or a
missing GPU raises.
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path

import numpy as np

PACKAGE_DIR = Path(__file__).resolve().parent
LIBRARY_PATH = PACKAGE_DIR / "lib" / "libmi355q.so"

OK, ERROR_RUNTIME, ERROR_INVALID = 0, 1, 2
F16, F32, BF16 = 0, 1, 2
META_F16_INTERLEAVED, META_BF16_PLANES = 0, 1
X_DEVICE, Y_DEVICE, RESIDUAL_DEVICE, ASYNC, SOURCE_DEVICE, RESIDUAL_IS_BIAS = 1, 2, 4, 8, 16, 32
W8A8_CHANNEL_MAJOR, WINDOWS_PAIRS = 128, 256
FUSE_GATE_UP_SILU = 64
SYM128_ROW_MAJOR, SYM128_OUTPUT_BLOCKED = 0, 1

_c = ctypes
_u32, _u64, _sz, _int = _c.c_uint32, _c.c_uint64, _c.c_size_t, _c.c_int
_vp, _cp = _c.c_void_p, _c.c_char_p
_err = (_c.c_char_p, _c.c_size_t)


class DeviceInfo(_c.Structure):
    _fields_ = [
        ("name", _c.c_char * 128),
        ("arch", _c.c_char * 32),
        ("compute_units", _int),
        ("wavefront", _int),
        ("hbm_bytes", _sz),
        ("lds_per_workgroup", _sz),
        ("clock_mhz", _int),
        ("memory_clock_mhz", _int),
        ("memory_bus_bits", _int),
    ]


class Q4Target(_c.Structure):
    _fields_ = [("weight", _vp), ("y", _vp), ("residual", _vp)]


class W8a8Target(_c.Structure):
    _fields_ = [("weight", _vp), ("bias", _vp), ("out", _vp), ("acc", _vp)]


class Q4Call(_c.Structure):
    _fields_ = [("x", _vp), ("M", _u32), ("x_dtype", _int), ("y_dtype", _int),
                ("residual_dtype", _int), ("target_count", _u32), ("targets", Q4Target * 4),
                ("flags", _u32)]


# name -> (restype, argtypes): every symbol the two headers declare
SIGNATURES = {
    "mi355q_context_create": (_int, [_int, _c.POINTER(_vp), *_err]),
    "mi355q_context_destroy": (None, [_vp]),
    "mi355q_context_info": (_int, [_vp, _c.POINTER(DeviceInfo), *_err]),
    "mi355q_context_set_option": (_int, [_vp, _cp, _cp, *_err]),
    "mi355q_context_get": (_int, [_vp, _cp, _c.POINTER(_u64), *_err]),
    "mi355q_sync": (_int, [_vp, *_err]),
    "mi355q_device_alloc": (_int, [_vp, _sz, _c.POINTER(_vp), *_err]),
    "mi355q_device_free": (_int, [_vp, _vp, *_err]),
    "mi355q_upload": (_int, [_vp, _vp, _vp, _sz, *_err]),
    "mi355q_download": (_int, [_vp, _vp, _vp, _sz, *_err]),
    "mi355q_timer_begin": (_int, [_vp, *_err]),
    "mi355q_timer_end": (_int, [_vp, _c.POINTER(_c.c_double), *_err]),
    "mi355q_profile_begin": (_int, [_vp, *_err]),
    "mi355q_profile_end": (_int, [_vp, _c.POINTER(_c.c_double), _c.POINTER(_u64), *_err]),
    "mi355q_profile_durations": (_int, [_vp, _vp, _sz, _c.POINTER(_sz), *_err]),
    "mi355q_probe_read_bandwidth": (_int, [_vp, _sz, _sz, _int, _int, _c.POINTER(_c.c_double), *_err]),
    "mi355q_probe_mfma_rate": (_int, [_vp, _int, _int, _c.POINTER(_c.c_double), *_err]),
    "mi355q_q4_weight_prepare": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _int, _u32,
                                        _c.POINTER(_vp), *_err]),
    "mi355q_sym128_weight_prepare": (_int, [_vp, _vp, _u32, _u32, _int, _u32, _c.POINTER(_vp), *_err]),
    "mi355q_q4_weight_destroy": (None, [_vp]),
    "mi355q_q4_weight_image_bytes": (_sz, [_vp]),
    "mi355q_probe_xcd_columns": (_int, [_vp, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), *_err]),
    "mi355q_q4_weight_shape": (None, [_vp, ctypes.POINTER(_u32), ctypes.POINTER(_u32)]),
    "mi355q_q38_image_open": (_int, [_vp, _vp, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p), *_err]),
    "mi355q_q38_image_close": (None, [_vp]),
    "mi355q_q38_image_kind": (_int, [_vp]),
    "mi355q_q38_kind_name": (ctypes.c_char_p, [_int]),
    "mi355q_q38_image_version": (_u32, [_vp]),
    "mi355q_q38_image_layer_index": (_u32, [_vp]),
    "mi355q_q38_image_linear_count": (ctypes.c_size_t, [_vp]),
    "mi355q_q38_image_linear": (ctypes.c_void_p, [_vp, ctypes.c_size_t, ctypes.POINTER(ctypes.c_char_p)]),
    "mi355q_q38_image_find": (ctypes.c_void_p, [_vp, ctypes.c_char_p]),
    "mi355q_q38_layout_field": (_int, [_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_char_p),
                                       ctypes.POINTER(_u32), ctypes.POINTER(_u32)]),
    "mi355q_q8_weight_prepare": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _int, _u32, ctypes.POINTER(ctypes.c_void_p), *_err]),
    "mi355q_q8rows_weight_prepare": (_int, [_vp, _vp, _u32, _u32, _u32, ctypes.POINTER(ctypes.c_void_p), *_err]),
    "mi355q_q8_weight_destroy": (None, [_vp]),
    "mi355q_q8_weight_image_bytes": (ctypes.c_size_t, [_vp]),
    "mi355q_q8_linear": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _int, _vp, _int, _u32, *_err]),
    "mi355q_causal_q8_windows": (_int, [_vp, _vp, _vp, _u32, _u32, _u32, _vp, _vp, _u32, *_err]),
    "mi355q_q4_dequant_rows": (_int, [_vp, _vp, _vp, _u32, _vp, _int, _u32, *_err]),
    "mi355q_q4_linear_rows": (_int, [_vp, _vp, _vp, _u32, _vp, _int, _u32, _vp, _int, _u32, *_err]),
    "mi355q_q4_linear": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _int, _vp, _int, _u32, *_err]),
    "mi355q_q4_linear_noalloc": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _int, _vp, _int, _u32, *_err]),
    "mi355q_q4_linear_multi": (_int, [_vp, _c.POINTER(Q4Target), _u32, _vp, _int, _u32, _int, _int,
                                      _u32, *_err]),
    "mi355q_q4_linear_sequence": (_int, [_vp, _c.POINTER(Q4Call), _sz, *_err]),
    "mi355q_hook_q4_gemm": (_int, [_vp, _vp, _sz, _sz, _sz, _vp, _vp]),
    "mi355q_hook_q4_gemv": (_int, [_vp, _int, _sz, _sz, _vp, _vp]),
    "mi355q_hook_last_error": (_int, [_c.c_char_p, _sz]),
    "mi355q_hook_release": (None, []),
    "mi355q_q4_sequence_record": (_int, [_vp, _c.POINTER(Q4Call), _sz, _c.POINTER(_vp), *_err]),
    "mi355q_graph_launch": (_int, [_vp, _vp, *_err]),
    "mi355q_graph_destroy": (None, [_vp]),
    "mi355q_w8a8_weight_prepare": (_int, [_vp, _vp, _u32, _u32, _u32, _c.POINTER(_vp), *_err]),
    "mi355q_w8a8_weight_destroy": (None, [_vp]),
    "mi355q_quantize_i8": (_int, [_vp, _vp, _u32, _u32, _vp, _vp, _u32, *_err]),
    "mi355q_w8a8_linear": (_int, [_vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp, _u32, *_err]),
    "mi355q_w8a8_linear_multi": (_int, [_vp, _vp, _u32, _vp, _vp, _u32, _u32, *_err]),
    "mi355q_synth_normal_f32": (None, [_u64, _c.c_float, _sz, _vp]),
    "mi355q_synth_normal_f16": (None, [_u64, _c.c_float, _sz, _vp]),
    "mi355q_quantize_q4_affine": (_int, [_vp, _u32, _u32, _int, _vp, _vp, _vp]),
    "mi355q_synth_q4_affine": (_int, [_u64, _c.c_float, _u32, _u32, _int, _vp, _vp, _vp]),
    "mi355q_quantize_w8_rows": (_int, [_vp, _u32, _u32, _vp]),
    "mi355q_synth_w8_rows": (_int, [_u64, _c.c_float, _u32, _u32, _vp]),
}

_library = None


class Mi355qError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"mi355q status {status}: {message}")
        self.status = status
        self.message = message


def library() -> ctypes.CDLL:
    """Loads libmi355q.so (once) and types every exported function."""
    global _library
    if _library is None:
        if not LIBRARY_PATH.exists():
            raise FileNotFoundError(
                f"{LIBRARY_PATH} is not built; run `make -C {PACKAGE_DIR / 'csrc'}`")
        lib = ctypes.CDLL(os.fspath(LIBRARY_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(lib, name)
            function.restype = restype
            function.argtypes = argtypes
        _library = lib
    return _library


def _ptr(array):
    if array is None:
        return None
    if isinstance(array, (int, ctypes.c_void_p)):
        return array
    assert array.flags["C_CONTIGUOUS"]
    return array.ctypes.data_as(ctypes.c_void_p)


def _call(function, *args):
    error = ctypes.create_string_buffer(512)
    status = function(*args, error, len(error))
    if status != OK:
        raise Mi355qError(status, error.value.decode(errors="replace"))


_NP_DTYPE = {F16: np.float16, F32: np.float32, BF16: np.uint16}


class Q4Weight:
    def __init__(self, context: "Context", handle, N: int, K: int):
        self.context, self.handle, self.N, self.K = context, handle, N, K

    @property
    def image_bytes(self) -> int:
        return library().mi355q_q4_weight_image_bytes(self.handle)

    def destroy(self):
        if self.handle:
            library().mi355q_q4_weight_destroy(self.handle)
            self.handle = None


class Q38Image:
    """An opened Qwen3.8 image file: its linears as prepared weights (owned by the image)."""

    def __init__(self, context: "Context", handle):
        lib = library()
        self.context, self.handle = context, handle
        self.kind = lib.mi355q_q38_kind_name(lib.mi355q_q38_image_kind(handle)).decode()
        self.version = lib.mi355q_q38_image_version(handle)
        self.layer_index = lib.mi355q_q38_image_layer_index(handle)
        self.linears = {}
        for index in range(lib.mi355q_q38_image_linear_count(handle)):
            name = ctypes.c_char_p()
            weight = ctypes.c_void_p(lib.mi355q_q38_image_linear(handle, index, ctypes.byref(name)))
            N, K = _u32(), _u32()
            lib.mi355q_q4_weight_shape(weight, ctypes.byref(N), ctypes.byref(K))
            self.linears[name.value.decode()] = Q4Weight(context, weight, N.value, K.value)

    def close(self):
        if self.handle:
            library().mi355q_q38_image_close(self.handle)
            self.handle = None
            for weight in self.linears.values():
                weight.handle = None  # freed with the image


def q38_layout_fields(kind: int) -> dict:
    """{field name: (byte offset, size)} the loader reads from a header of that kind."""
    lib, fields, index = library(), {}, 0
    while True:
        name, offset, size = ctypes.c_char_p(), _u32(), _u32()
        if lib.mi355q_q38_layout_field(kind, index, ctypes.byref(name), ctypes.byref(offset), ctypes.byref(size)):
            return fields
        fields[name.value.decode()] = (offset.value, size.value)
        index += 1


class Context:
    """One engine context (one HIP stream) on one GPU."""

    def __init__(self, device: int = 0):
        self.lib = library()
        handle = ctypes.c_void_p()
        _call(self.lib.mi355q_context_create, device, ctypes.byref(handle))
        self.handle = handle

    def close(self):
        if self.handle:
            self.lib.mi355q_context_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def info(self) -> DeviceInfo:
        info = DeviceInfo()
        _call(self.lib.mi355q_context_info, self.handle, ctypes.byref(info))
        return info

    def set_option(self, name: str, value: str | None):
        """Experiment knob of this context (see mi355q_context_set_option); None clears it."""
        _call(self.lib.mi355q_context_set_option, self.handle, name.encode(),
              None if value is None else value.encode())

    def get(self, name: str) -> int:
        """A counter of the context: "chained_launches", "staging_bytes", "staging_generation"."""
        value = ctypes.c_uint64()
        _call(self.lib.mi355q_context_get, self.handle, name.encode(), ctypes.byref(value))
        return int(value.value)

    def sync(self):
        _call(self.lib.mi355q_sync, self.handle)

    def alloc(self, nbytes: int) -> int:
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_device_alloc, self.handle, nbytes, ctypes.byref(out))
        return out.value

    def free(self, pointer: int):
        _call(self.lib.mi355q_device_free, self.handle, pointer)

    def upload(self, pointer: int, array: np.ndarray):
        array = np.ascontiguousarray(array)
        _call(self.lib.mi355q_upload, self.handle, pointer, _ptr(array), array.nbytes)

    def to_device(self, array: np.ndarray) -> int:
        pointer = self.alloc(max(array.nbytes, 16))
        self.upload(pointer, array)
        return pointer

    def download(self, pointer: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        _call(self.lib.mi355q_download, self.handle, _ptr(out), pointer, out.nbytes)
        return out

    def timer_begin(self):
        _call(self.lib.mi355q_timer_begin, self.handle)

    def timer_end(self) -> float:
        ms = ctypes.c_double()
        _call(self.lib.mi355q_timer_end, self.handle, ctypes.byref(ms))
        return ms.value

    def profile_begin(self):
        _call(self.lib.mi355q_profile_begin, self.handle)

    def profile_end(self):
        """(sum of kernel durations in ms, number of kernel launches)"""
        ms, launches = ctypes.c_double(), ctypes.c_uint64()
        _call(self.lib.mi355q_profile_end, self.handle, ctypes.byref(ms), ctypes.byref(launches))
        return ms.value, launches.value

    def profile_durations(self) -> np.ndarray:
        """Per-launch kernel durations (us) of the profile that just ended, in launch order."""
        count = ctypes.c_size_t()
        _call(self.lib.mi355q_profile_durations, self.handle, None, 0, ctypes.byref(count))
        out = np.empty(count.value, dtype=np.float64)
        _call(self.lib.mi355q_profile_durations, self.handle, _ptr(out), out.size, ctypes.byref(count))
        return out

    def probe_read_bandwidth(self, nbytes: int = 2 << 30, repeats: int = 5, variant: int = 1,
                             launch_bytes: int = 0) -> float:
        gbs = ctypes.c_double()
        _call(self.lib.mi355q_probe_read_bandwidth, self.handle, nbytes, launch_bytes, repeats, variant,
              ctypes.byref(gbs))
        return gbs.value

    def probe_mfma_rate(self, valu_per_mfma: int = 0, repeats: int = 3) -> float:
        tflops = ctypes.c_double()
        _call(self.lib.mi355q_probe_mfma_rate, self.handle, valu_per_mfma, repeats, ctypes.byref(tflops))
        return tflops.value

    # ---- affine Q4 ----
    def q4_prepare(self, quants, meta_a, meta_b, N: int, K: int, meta_kind: int,
                   flags: int = 0) -> Q4Weight:
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_q4_weight_prepare, self.handle, _ptr(quants), _ptr(meta_a),
              _ptr(meta_b), N, K, meta_kind, flags, ctypes.byref(out))
        return Q4Weight(self, out, N, K)

    def sym128_prepare(self, records, N: int, K: int, record_order: int = SYM128_ROW_MAJOR,
                       flags: int = 0) -> Q4Weight:
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_sym128_weight_prepare, self.handle, _ptr(records), N, K, record_order,
              flags, ctypes.byref(out))
        return Q4Weight(self, out, N, K)

    # ---- affine Q8 (one Q4 weight of twice the columns) ----
    def q8_prepare(self, quants, meta_a, meta_b, N: int, K: int, meta_kind: int):
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_q8_weight_prepare, self.handle, _ptr(quants), _ptr(meta_a), _ptr(meta_b), N, K,
              meta_kind, 0, ctypes.byref(out))
        return out

    def q8rows_prepare(self, records, N: int, K: int):
        """Records [N][4 + K]: fp32 scale then K int8 per output row."""
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_q8rows_weight_prepare, self.handle, _ptr(records), N, K, 0, ctypes.byref(out))
        return out

    def q8_destroy(self, weight):
        self.lib.mi355q_q8_weight_destroy(weight)

    def q8_linear(self, weight, N: int, x: np.ndarray, x_dtype: int, y_dtype: int = F32,
                  residual: np.ndarray | None = None, residual_dtype: int = F32) -> np.ndarray:
        x = np.ascontiguousarray(x)
        M = x.shape[0]
        y = np.empty((M, N), dtype=_NP_DTYPE[y_dtype])
        _call(self.lib.mi355q_q8_linear, self.handle, weight, _ptr(x), x_dtype, M, _ptr(y), y_dtype,
              _ptr(residual), residual_dtype, 0)
        return y

    def q8_linear_device(self, weight, x_ptr: int, x_dtype: int, M: int, y_ptr: int, y_dtype: int = F32,
                         asynchronous: bool = True):
        _call(self.lib.mi355q_q8_linear, self.handle, weight, ctypes.c_void_p(x_ptr), x_dtype, M,
              ctypes.c_void_p(y_ptr), y_dtype, None, F32, X_DEVICE | Y_DEVICE | (ASYNC if asynchronous else 0))

    def q38_image_open(self, image_bytes) -> Q38Image:
        """Opens the bytes of a .q38delta / .q38att / .q38global / .q38mtp file."""
        data = np.ascontiguousarray(np.frombuffer(image_bytes, dtype=np.uint8))
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_q38_image_open, self.handle, _ptr(data), data.size, ctypes.byref(out))
        return Q38Image(self, out)

    def probe_xcd_columns(self):
        """(columns_share_xcd, xcds): see mi355q_probe_xcd_columns."""
        shared, xcds = ctypes.c_int(), ctypes.c_int()
        _call(self.lib.mi355q_probe_xcd_columns, self.handle, ctypes.byref(shared), ctypes.byref(xcds))
        return bool(shared.value), xcds.value

    def q4_dequant_rows(self, weight: Q4Weight, rows, out_dtype: int = F32) -> np.ndarray:
        rows = np.ascontiguousarray(rows, dtype=np.uint32)
        out = np.empty((rows.size, weight.K), dtype=_NP_DTYPE[out_dtype])
        _call(self.lib.mi355q_q4_dequant_rows, self.handle, weight.handle, _ptr(rows), rows.size, _ptr(out),
              out_dtype, 0)
        return out

    def q4_linear(self, weight: Q4Weight, x: np.ndarray, x_dtype: int, y_dtype: int = F32,
                  residual: np.ndarray | None = None, residual_dtype: int = F32,
                  residual_is_bias: bool = False) -> np.ndarray:
        """Host-array convenience form: x [M][K] -> y [M][N]."""
        x = np.ascontiguousarray(x)
        M = x.shape[0]
        y = np.empty((M, weight.N), dtype=_NP_DTYPE[y_dtype])
        _call(self.lib.mi355q_q4_linear, self.handle, weight.handle, _ptr(x), x_dtype, M,
              _ptr(y), y_dtype, _ptr(residual), residual_dtype,
              RESIDUAL_IS_BIAS if residual_is_bias else 0)
        return y

    def q4_linear_rows(self, weight: Q4Weight, rows, x: np.ndarray, x_dtype: int, y_dtype: int = F32,
                       count: int | None = None) -> np.ndarray:
        """The linear restricted to output rows `rows` (ids), or to the first `count` rows when
        rows is None: x [M][K] -> y [M][len(rows) or count]."""
        x = np.ascontiguousarray(x)
        M = x.shape[0]
        if rows is not None:
            rows = np.ascontiguousarray(rows, dtype=np.uint32)
            count = rows.size
        y = np.empty((M, count), dtype=_NP_DTYPE[y_dtype])
        _call(self.lib.mi355q_q4_linear_rows, self.handle, weight.handle, _ptr(rows), count, _ptr(x), x_dtype,
              M, _ptr(y), y_dtype, 0)
        return y

    def q4_linear_rows_device(self, weight: Q4Weight, rows_ptr: int | None, count: int, x_ptr: int,
                              x_dtype: int, M: int, y_ptr: int, y_dtype: int, asynchronous: bool = True):
        flags = X_DEVICE | Y_DEVICE | SOURCE_DEVICE | (ASYNC if asynchronous else 0)
        _call(self.lib.mi355q_q4_linear_rows, self.handle, weight.handle, rows_ptr, count, x_ptr, x_dtype, M,
              y_ptr, y_dtype, flags)

    def q4_gate_up_silu(self, gate: Q4Weight, up: Q4Weight, x: np.ndarray, x_dtype: int,
                        y_dtype: int = F32) -> np.ndarray:
        """Host-array form of the fused call: silu(gate . x) * (up . x), [M][N]."""
        x = np.ascontiguousarray(x)
        M = x.shape[0]
        y = np.empty((M, gate.N), dtype=_NP_DTYPE[y_dtype])
        targets = (Q4Target * 2)()
        targets[0].weight, targets[0].y = gate.handle, y.ctypes.data
        targets[1].weight = up.handle
        _call(self.lib.mi355q_q4_linear_multi, self.handle, targets, 2, _ptr(x), x_dtype, M, y_dtype, F32,
              FUSE_GATE_UP_SILU)
        return y

    def q4_linear_multi(self, weights, x: np.ndarray, x_dtype: int, y_dtype: int = F32):
        """Host-array form of the shared-x call: returns one y per weight."""
        x = np.ascontiguousarray(x)
        M = x.shape[0]
        ys = [np.empty((M, w.N), dtype=_NP_DTYPE[y_dtype]) for w in weights]
        targets = (Q4Target * len(weights))()
        for slot, w, y in zip(targets, weights, ys):
            slot.weight, slot.y, slot.residual = w.handle, y.ctypes.data, None
        _call(self.lib.mi355q_q4_linear_multi, self.handle, targets, len(weights), _ptr(x), x_dtype, M,
              y_dtype, F32, 0)
        return ys

    def q4_linear_device(self, weight: Q4Weight, x_ptr: int, x_dtype: int, M: int, y_ptr: int,
                         y_dtype: int, residual_ptr: int | None = None,
                         residual_dtype: int = F32, asynchronous: bool = True):
        flags = X_DEVICE | Y_DEVICE | RESIDUAL_DEVICE | (ASYNC if asynchronous else 0)
        _call(self.lib.mi355q_q4_linear, self.handle, weight.handle, x_ptr, x_dtype, M, y_ptr,
              y_dtype, residual_ptr, residual_dtype, flags)

    def q4_linear_noalloc(self, weight: Q4Weight, x_ptr: int, x_dtype: int, M: int, y_ptr: int,
                          y_dtype: int, residual_ptr: int | None = None, residual_dtype: int = F32,
                          asynchronous: bool = False, residual_is_bias: bool = False):
        """The entry point that allocates nothing; device pointers only."""
        flags = (ASYNC if asynchronous else 0) | (RESIDUAL_IS_BIAS if residual_is_bias else 0)
        _call(self.lib.mi355q_q4_linear_noalloc, self.handle, weight.handle, x_ptr, x_dtype, M, y_ptr,
              y_dtype, residual_ptr, residual_dtype, flags)

    # ---- W8A8 ----
    def w8a8_prepare(self, rows: np.ndarray, N: int, K: int):
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_w8a8_weight_prepare, self.handle, _ptr(rows), N, K, 0, ctypes.byref(out))
        return out

    def w8a8_destroy(self, weight):
        self.lib.mi355q_w8a8_weight_destroy(weight)

    def quantize_i8(self, x: np.ndarray):
        x = np.ascontiguousarray(x, dtype=np.float32)
        M, K = x.shape
        q = np.empty((M, K), dtype=np.int8)
        scales = np.empty(M, dtype=np.float32)
        _call(self.lib.mi355q_quantize_i8, self.handle, _ptr(x), M, K, _ptr(q), _ptr(scales), 0)
        return q, scales

    def w8a8_linear(self, weight, N: int, q: np.ndarray, x_scales: np.ndarray, bias=None,
                    channel_major: bool = False):
        """out [M][N] (or [N][M] with the streaming convolution's epilogue) and the int32 sums [M][N]."""
        q = np.ascontiguousarray(q, dtype=np.int8)
        M = q.shape[0]
        out = np.empty((N, M) if channel_major else (M, N), dtype=np.float32)
        acc = np.empty((M, N), dtype=np.int32)
        _call(self.lib.mi355q_w8a8_linear, self.handle, weight, _ptr(q),
              _ptr(np.ascontiguousarray(x_scales, dtype=np.float32)), M, _ptr(bias), _ptr(out),
              _ptr(acc), W8A8_CHANNEL_MAJOR if channel_major else 0)
        return out, acc

    def w8a8_linear_multi(self, weights, widths, q: np.ndarray, x_scales: np.ndarray, biases=None):
        """One launch for up to four weights that share q: list of (out [M][N], acc [M][N])."""
        q = np.ascontiguousarray(q, dtype=np.int8)
        M = q.shape[0]
        biases = biases if biases is not None else [None] * len(weights)
        biases = [None if b is None else np.ascontiguousarray(b, dtype=np.float32) for b in biases]
        results = [(np.empty((M, N), dtype=np.float32), np.empty((M, N), dtype=np.int32)) for N in widths]
        targets = (W8a8Target * len(weights))()
        for slot, weight, bias, (out, acc) in zip(targets, weights, biases, results):
            slot.weight, slot.bias, slot.out, slot.acc = weight, _ptr(bias), _ptr(out), _ptr(acc)
        _call(self.lib.mi355q_w8a8_linear_multi, self.handle, targets, len(weights), _ptr(q),
              _ptr(np.ascontiguousarray(x_scales, dtype=np.float32)), M, 0)
        return results

    def w8a8_linear_multi_device(self, weights, q_ptr: int, scales_ptr: int, M: int, bias_ptrs, out_ptrs,
                                 acc_ptrs=None, asynchronous: bool = True):
        targets = (W8a8Target * len(weights))()
        for index, slot in enumerate(targets):
            slot.weight, slot.bias, slot.out = weights[index], bias_ptrs[index], out_ptrs[index]
            slot.acc = acc_ptrs[index] if acc_ptrs else None
        _call(self.lib.mi355q_w8a8_linear_multi, self.handle, targets, len(weights), q_ptr, scales_ptr, M,
              X_DEVICE | Y_DEVICE | (ASYNC if asynchronous else 0))

    def causal_q8_windows(self, x: np.ndarray, history, kernel: int, pairs: bool = False):
        """x [channels][length] fp32 -> (q [length][columns] int8, scales [length])."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        channels, length = x.shape
        columns = channels * (2 if pairs else kernel)
        q = np.empty((length, columns), dtype=np.int8)
        scales = np.empty(length, dtype=np.float32)
        if history is not None:
            history = np.ascontiguousarray(history, dtype=np.float32)
        _call(self.lib.mi355q_causal_q8_windows, self.handle, _ptr(x), _ptr(history), channels, kernel, length,
              _ptr(q), _ptr(scales), WINDOWS_PAIRS if pairs else 0)
        return q, scales

    def quantize_i8_device(self, x_ptr: int, M: int, K: int, q_ptr: int, scales_ptr: int,
                           asynchronous: bool = True):
        _call(self.lib.mi355q_quantize_i8, self.handle, x_ptr, M, K, q_ptr, scales_ptr,
              X_DEVICE | Y_DEVICE | (ASYNC if asynchronous else 0))

    def w8a8_linear_device(self, weight, q_ptr: int, scales_ptr: int, M: int, bias_ptr, out_ptr: int,
                           acc_ptr=None, asynchronous: bool = True):
        _call(self.lib.mi355q_w8a8_linear, self.handle, weight, q_ptr, scales_ptr, M, bias_ptr, out_ptr,
              acc_ptr, X_DEVICE | Y_DEVICE | (ASYNC if asynchronous else 0))

    def q4_sequence_record(self, calls):
        """Records the calls into a graph (running them once); returns the graph handle."""
        out = ctypes.c_void_p()
        _call(self.lib.mi355q_q4_sequence_record, self.handle, calls, len(calls), ctypes.byref(out))
        return out

    def graph_launch(self, graph):
        _call(self.lib.mi355q_graph_launch, self.handle, graph)

    def graph_destroy(self, graph):
        self.lib.mi355q_graph_destroy(graph)

    def q4_sequence(self, calls):
        """calls: a ctypes array of Q4Call (build once, reuse)."""
        _call(self.lib.mi355q_q4_linear_sequence, self.handle, calls, len(calls))


def make_calls(items):
    """items: iterable of (targets, x_ptr, x_dtype, M, y_dtype[, residual_dtype[, flags]]) where targets is
    a Q4Weight with its y pointer `(weight, y_ptr[, residual_ptr])` or a list of up to four of them
    (one launch, shared x)."""
    items = list(items)
    array = (Q4Call * len(items))()
    for slot, item in zip(array, items):
        targets, x_ptr, x_dtype, M, y_dtype = item[:5]
        if isinstance(targets, tuple):
            targets = [targets]
        slot.x, slot.M, slot.x_dtype, slot.y_dtype = x_ptr, M, x_dtype, y_dtype
        slot.residual_dtype = item[5] if len(item) > 5 else F32
        slot.flags = item[6] if len(item) > 6 else 0
        slot.target_count = len(targets)
        for index, target in enumerate(targets):
            slot.targets[index].weight = target[0].handle
            slot.targets[index].y = target[1]
            slot.targets[index].residual = target[2] if len(target) > 2 else None
    return array


# ---- entry points with the reference's hook signatures ----------------------

def _hook_check(status: int):
    if status != 0:
        message = ctypes.create_string_buffer(256)
        library().mi355q_hook_last_error(message, len(message))
        raise Mi355qError(status, message.value.decode(errors="replace"))


def hook_q4_gemm(records: np.ndarray, x: np.ndarray, N: int, bias=None) -> np.ndarray:
    """output[r][n] = bias[n] + sum_k w[n][k] x[r][k]; records stay alive with the caller."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, K = x.shape
    out = np.empty((rows, N), dtype=np.float32)
    _hook_check(library().mi355q_hook_q4_gemm(_ptr(records), _ptr(x), rows, K, N, _ptr(bias), _ptr(out)))
    return out


def hook_q4_gemv(records: np.ndarray, record_order: int, N: int, x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(N, dtype=np.float32)
    _hook_check(library().mi355q_hook_q4_gemv(_ptr(records), record_order, N, x.size, _ptr(x), _ptr(out)))
    return out


def hook_release():
    library().mi355q_hook_release()


# ---- synthetic inputs (host side) ------------------------------------------

def synth_normal_f32(seed: int, sigma: float, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.float32)
    library().mi355q_synth_normal_f32(seed, sigma, count, _ptr(out))
    return out


def synth_normal_f16(seed: int, sigma: float, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.float16)
    library().mi355q_synth_normal_f16(seed, sigma, count, _ptr(out))
    return out


def _q4_planes(N: int, K: int, meta_kind: int):
    groups = N * (K // 64)
    quants = np.empty(groups * 32, dtype=np.uint8)
    if meta_kind == META_F16_INTERLEAVED:
        return quants, np.empty(groups * 2, dtype=np.uint16), None
    return quants, np.empty(groups, dtype=np.uint16), np.empty(groups, dtype=np.uint16)


def quantize_q4_affine(w: np.ndarray, meta_kind: int):
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    quants, meta_a, meta_b = _q4_planes(N, K, meta_kind)
    status = library().mi355q_quantize_q4_affine(_ptr(w), N, K, meta_kind, _ptr(quants),
                                                 _ptr(meta_a), _ptr(meta_b))
    if status != OK:
        raise Mi355qError(status, "quantize_q4_affine: bad shape")
    return quants, meta_a, meta_b


def synth_q4_affine(seed: int, sigma: float, N: int, K: int, meta_kind: int):
    quants, meta_a, meta_b = _q4_planes(N, K, meta_kind)
    status = library().mi355q_synth_q4_affine(seed, sigma, N, K, meta_kind, _ptr(quants),
                                              _ptr(meta_a), _ptr(meta_b))
    if status != OK:
        raise Mi355qError(status, "synth_q4_affine: bad shape")
    return quants, meta_a, meta_b


def synth_w8_rows(seed: int, sigma: float, N: int, K: int) -> np.ndarray:
    rows = np.empty(N * (4 + K), dtype=np.uint8)
    status = library().mi355q_synth_w8_rows(seed, sigma, N, K, _ptr(rows))
    if status != OK:
        raise Mi355qError(status, "synth_w8_rows: bad shape")
    return rows
