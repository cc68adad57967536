"""The five BASELINE configurations at their real shapes, against the oracle."""
import numpy as np
import pytest

from helpers import Q4, Q8, bits
from meganeura_amd import capi, synth
from test_gpu_parity import ABS, REL, ROUTES, run_matmul

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def assert_dequant_bits(orc, wt, fmt, packed, k, n):
    """The device's dequantized weight against the oracle's, bit for bit, at the weight's full size
    (the kernel's block indexing depends on the size: every element is compared, none sampled)."""
    got = bits(wt.dequantize())
    want = bits(orc.dequantize(fmt, packed, k, n))
    assert got.shape == want.shape == (k, n)
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        r, c = bad[0]
        raise AssertionError(f"{len(bad)} of {k * n} dequantized elements differ; first at [{r}, {c}]: "
                             f"{got[r, c]:#010x} != {want[r, c]:#010x}")


def check(ctx, orc, fmt, x, w, d=None, f16=False, routes=("auto",), check_weight=True):
    k, n = w.shape
    packed = orc.quantize(fmt, w)
    wt = ctx.weight(fmt, w)
    if check_weight:
        assert (wt.export_ref() == packed).all()
        assert_dequant_bits(orc, wt, fmt, packed, k, n)
    xo = x.astype(np.float16).astype(np.float32) if f16 else x
    want = orc.matmul_packed(fmt, xo, packed, n, d)
    for route in routes:
        got = run_matmul(ctx, fmt, x, wt, ROUTES[route], d=d, f16=f16)
        orc.assert_close(got, want, REL, ABS)
    wt.free()


def test_c1_q8_gemv_mlp_up(ctx, orc):
    check(ctx, orc, Q8, synth.activations(1, 1, 576), synth.weights(1, 576, 1536), routes=("auto", "generic"))


@pytest.mark.parametrize("name,k,n,resid", [
    ("q", 576, 576, False), ("k", 576, 192, False), ("v", 576, 192, False), ("o", 576, 576, True),
    ("gate", 576, 1536, False), ("up", 576, 1536, False), ("gate+up", 576, 3072, False), ("down", 1536, 576, True),
])
def test_c2_q4_decode_layer_set(ctx, orc, name, k, n, resid):
    which = sum(map(ord, name))
    x = synth.activations(2, 1, k, which=which)
    w = synth.weights(2, k, n, which=which)
    d = synth.activations(2, 1, n, which=which + 1) if resid else None
    check(ctx, orc, Q4, x, w, d)


def test_c3_q4_lm_head(ctx, orc):
    check(ctx, orc, Q4, synth.activations(3, 1, 576), synth.weights(3, 576, 49152))


def test_c4_q4_prefill_mlp(ctx, orc):
    x = synth.activations(4, 512, 1024)
    check(ctx, orc, Q4, x, synth.weights(4, 1024, 3072), f16=True)
    x2 = synth.activations(4, 512, 3072, which=1)
    check(ctx, orc, Q4, x2, synth.weights(4, 3072, 1024, which=1), f16=True)


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("k,n", [(4096, 14336), (14336, 4096)])
def test_c5_llama_ffn(ctx, orc, fmt, k, n):
    w = synth.weights(5, k, n, which=k)
    packed = orc.quantize(fmt, w)
    wt = ctx.weight(fmt, w)
    assert (wt.export_ref() == packed).all()
    del w
    assert_dequant_bits(orc, wt, fmt, packed, k, n)
    for m in (1, 4, 16):
        x = synth.activations(5, m, k, which=m)
        want = orc.matmul_packed(fmt, x, packed, n)
        got = run_matmul(ctx, fmt, x, wt)
        orc.assert_close(got, want, REL, ABS)
        if m == 16:
            # a context that was promised activations in the fp16 range may take the 32x32x16 kernel:
            # that route on the same shape, forced so that it runs whatever the planner prefers
            ctx.set_activation_range(True)
            try:
                orc.assert_close(run_matmul(ctx, fmt, x, wt), want, REL, ABS)
                orc.assert_close(run_matmul(ctx, fmt, x, wt, ROUTES["gemm_mfma"]), want, REL, ABS)
            finally:
                ctx.set_activation_range(False)
    wt.free()
