"""mgn_matmul_q_static: the matmul on the library's static workspace (no device allocation in
the call) against mgn_matmul_q, through the C ABI, on shapes whose K is cut into parts."""
import numpy as np
import pytest

from helpers import Q4, Q8, bits
from meganeura_amd import capi, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def free_device_bytes():
    """hipMemGetInfo's free figure, straight from the HIP runtime the library itself is linked to."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def both(ctx, orc, fmt, m, k, n, seed, with_d):
    x = synth.normal(seed, m * k).reshape(m, k)
    w = synth.normal(seed + 1, k * n, 0.02).reshape(k, n)
    d = synth.normal(seed + 2, m * n).reshape(m, n) if with_d else None
    wt, a = ctx.weight(fmt, w), ctx.upload(x)
    db = ctx.upload(d) if with_d else None
    c_ref, c_new = ctx.buffer(m * n * 4), ctx.buffer(m * n * 4)
    ctx.matmul_q(a, wt, c_ref, m, db)
    ref = c_ref.download(np.float32, m * n).reshape(m, n)
    ctx.sync()
    before = free_device_bytes()
    ctx.matmul_q_static(a, wt, c_new, m, db)
    ctx.sync()
    assert free_device_bytes() == before, "the static entry point must not change the device's free memory"
    got = c_new.download(np.float32, m * n).reshape(m, n)
    want = orc.matmul_f32(x, orc.dequantize(fmt, orc.quantize(fmt, w), k, n), d)
    for buf in (a, c_ref, c_new, wt) + ((db,) if with_d else ()):
        buf.free()
    # same plan, same kernels, partial sums added in part order: bit-identical to mgn_matmul_q,
    # and both within the matmul bar of the oracle (1e-3 relative or 1e-4 absolute)
    assert np.array_equal(bits(got), bits(ref)), (fmt, m, k, n)
    orc.assert_close(got, want, 1e-3, 1e-4)


# (first call, second call with a smaller input); every first shape keeps partial sums in the workspace
PAIRS = [
    ((Q4, 4, 14336, 518), (Q4, 3, 12288, 64)),       # decode kernel, K parts across workgroups
    ((Q8, 16, 4096, 2048), (Q8, 6, 4096, 300)),      # tiled kernel, K parts across workgroups
    ((Q4, 16, 14336, 4096), (Q4, 1, 576, 192)),      # C5 at M = 16, then a shape with no workspace at all
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_workspace_matches_the_allocating_entry_point(ctx, orc, first, second):
    assert capi.matmul_plan(*first).workspace_bytes > 0
    assert capi.matmul_plan(*first).workspace_bytes <= capi.STATIC_WORKSPACE_BYTES
    both(ctx, orc, *first, seed=901, with_d=True)
    both(ctx, orc, *second, seed=907, with_d=False)


def test_static_workspace_tolerates_what_an_earlier_call_left(ctx, orc):
    """All contexts of a device share the static array and it keeps the last call's contents.  A
    call that gave up half-way (forced here with a zero spin limit) leaves partial sums behind and
    counters that may not be zero; the next call must still come out right."""
    fmt, m, k, n = Q4, 16, 14336, 4096
    w = synth.normal(931, k * n, 0.02).reshape(k, n)
    x = synth.normal(932, m * k).reshape(m, k)
    wt, a, c = ctx.weight(fmt, w), ctx.upload(x), ctx.buffer(m * n * 4)
    ctx.set_spin_limit(0)
    try:
        ctx.matmul_q_static(a, wt, c, m)
        with pytest.raises(capi.MgnError) as e:
            ctx.sync()
        assert e.value.status == capi.ETIMEOUT
    finally:
        ctx.set_spin_limit(1 << 20)
    for h in (wt, a, c):
        h.free()
    both(ctx, orc, Q8, 16, 4096, 2048, seed=941, with_d=False)   # tiled kernel, K parts
    both(ctx, orc, Q4, 4, 14336, 518, seed=943, with_d=True)     # decode kernel, K parts


def test_static_workspace_refuses_what_does_not_fit(ctx):
    fmt, m, k, n = Q4, 512, 8192, 2304
    plan = capi.matmul_plan(fmt, m, k, n)
    assert plan.workspace_bytes > capi.STATIC_WORKSPACE_BYTES, "pick a shape whose K parts exceed the static workspace"
    wt = ctx.weight(fmt, synth.normal(5, k * n, 0.02).reshape(k, n))
    a, c = ctx.buffer(m * k * 4), ctx.buffer(m * n * 4)
    with pytest.raises(capi.MgnError, match="static") as e:
        ctx.matmul_q_static(a, wt, c, m)
    assert e.value.status == capi.EUNSUPPORTED
    ctx.matmul_q(a, wt, c, m)  # the allocating entry point takes it
    ctx.sync()
    for buf in (a, c, wt):
        buf.free()
