"""mi355q_q4_linear_noalloc (the entry point that allocates nothing) against mi355q_q4_linear,
through the C ABI, bit for bit: same kernels and launch shapes, but converted activations,
slice partial sums and arrival counters live in the library's fixed device array.

The non-allocating call runs first on a fresh context and must leave the context's staging
buffers as they were (none).  Two calls in a row on each weight, the second with a smaller input, so that what the first
call left in the shared array (larger partial sums, counters, converted rows) must not leak
into the second.  Runs alone in a fresh process and after the other tests alike: it makes its
own context and cares nothing for what ran before.
"""
import numpy as np
import pytest

from conftest import q4_relative_error

pytestmark = pytest.mark.gpu


def make_x(engine, seed, M, K, x_dtype):
    x32 = np.stack([engine.synth_normal_f32(seed + 1000 * m, 1.0, K) for m in range(M)])
    return x32.astype(np.float16) if x_dtype == engine.F16 else x32


CASES = [
    # name, N, K, x dtype, residual, (M of the first call, M of the second, smaller, call)
    ("down_sliced_f16", 5120, 17408, "F16", False, (8, 1)),
    ("down_sliced_f32_residual", 5120, 17408, "F32", True, (4, 2)),
    ("few_tiles_long_rows", 528, 17472, "F32", False, (6, 1)),
    ("gate_unsliced", 17408, 5120, "F16", False, (2, 1)),
    ("o_half_tiles_at_one_row", 5120, 6144, "F16", True, (2, 1)),
    ("ragged_small", 100, 192, "F32", True, (8, 3)),
]


@pytest.mark.parametrize("name,N,K,x_dtype,with_residual,rows", CASES, ids=[c[0] for c in CASES])
def test_noalloc_matches_ordinary_call_bitwise(engine, oracle, name, N, K, x_dtype, with_residual, rows):
    x_dtype = getattr(engine, x_dtype)
    kind = engine.META_BF16_PLANES
    quants, meta_a, meta_b = engine.synth_q4_affine(71, 0.02, N, K, kind)
    ctx = engine.Context(0)
    weight = ctx.q4_prepare(quants, meta_a, meta_b, N, K, kind)
    pointers = []
    try:
        for call, M in enumerate(rows):
            print(f"noalloc case {name} call {call} M={M}", flush=True)
            x = make_x(engine, 72 + call, M, K, x_dtype)
            residual = engine.synth_normal_f32(73 + call, 1.0, M * N).reshape(M, N) if with_residual else None
            x_ptr, y_ptr, z_ptr = ctx.to_device(x), ctx.alloc(M * N * 4), ctx.alloc(M * N * 4)
            r_ptr = ctx.to_device(residual) if with_residual else None
            pointers += [p for p in (x_ptr, y_ptr, z_ptr, r_ptr) if p]
            for pointer in (y_ptr, z_ptr):
                ctx.upload(pointer, np.full((M, N), np.nan, dtype=np.float32))
            # the non-allocating call first, on a context whose staging buffers the ordinary call has
            # not yet grown for this size: it must not touch them (nothing allocated, nothing freed)
            staging = (ctx.get("staging_bytes"), ctx.get("staging_generation"))
            ctx.q4_linear_noalloc(weight, x_ptr, x_dtype, M, z_ptr, engine.F32, r_ptr, engine.F32)
            assert (ctx.get("staging_bytes"), ctx.get("staging_generation")) == staging
            if call == 0:
                assert staging == (0, 0)  # a fresh context: the library has allocated no staging at all
            ctx.q4_linear_device(weight, x_ptr, x_dtype, M, y_ptr, engine.F32, r_ptr, engine.F32,
                                 asynchronous=False)
            expect = ctx.download(y_ptr, (M, N), np.float32)
            got = ctx.download(z_ptr, (M, N), np.float32)
            assert np.array_equal(got.view(np.uint32), expect.view(np.uint32)), f"call {call} (M={M})"
            ref = oracle.q4_linear(quants, meta_a, meta_b, kind, N, K, x, x_dtype, M)
            if with_residual:
                ref = ref + residual
            assert q4_relative_error(got, ref) <= 1e-3
    finally:
        for pointer in pointers:
            ctx.free(pointer)
        weight.destroy()
        ctx.close()


def test_noalloc_refuses_what_does_not_fit(engine):
    """Sizes beyond the fixed array, host-style misuse and profiling are refused with status 2
    and a message; nothing is launched."""
    kind = engine.META_BF16_PLANES
    ctx = engine.Context(0)
    N, K = 16, 40960  # 8 fp32 rows -> 16 fp16 rows * 40960 * 2 bytes = 1.25 MiB of converted x
    weight = ctx.q4_prepare(*engine.synth_q4_affine(5, 0.02, N, K, kind), N, K, kind)
    x_ptr, y_ptr = ctx.alloc(8 * K * 4), ctx.alloc(17 * N * 4)
    try:
        ctx.upload(x_ptr, np.zeros((8, K), dtype=np.float32))
        with pytest.raises(engine.Mi355qError) as info:
            ctx.q4_linear_noalloc(weight, x_ptr, engine.F32, 8, y_ptr, engine.F32)
        assert info.value.status == engine.ERROR_INVALID and "exceed" in info.value.message
        ctx.q4_linear_noalloc(weight, x_ptr, engine.F32, 4, y_ptr, engine.F32)  # half of it fits
        with pytest.raises(engine.Mi355qError) as info:  # more rows than the streaming kernel takes
            ctx.q4_linear_noalloc(weight, x_ptr, engine.F16, 17, y_ptr, engine.F32)
        assert info.value.status == engine.ERROR_INVALID
        ctx.profile_begin()
        try:
            with pytest.raises(engine.Mi355qError) as info:
                ctx.q4_linear_noalloc(weight, x_ptr, engine.F16, 1, y_ptr, engine.F32)
            assert info.value.status == engine.ERROR_INVALID
        finally:
            ctx.profile_end()
    finally:
        ctx.free(x_ptr)
        ctx.free(y_ptr)
        weight.destroy()
        ctx.close()
