"""Parity of the HIP path against the CPU oracle, through the C ABI.

Bars: dequantized weights and packed bytes bit-exact; matmul outputs within
1e-3 relative OR 1e-4 absolute of the f32 sequential-k result on the oracle's
dequantized weights (helper semantics of tests/gemv_parity.rs:61-72)."""
import numpy as np
import pytest

from helpers import Q4, Q8, bits, ref_test_inputs_q4_matmul
from meganeura_amd import capi, synth

pytestmark = pytest.mark.gpu

REL, ABS = 1e-3, 1e-4


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def run_matmul(ctx, fmt, x, w_or_weight, route=capi.ROUTE_AUTO, d=None, f16=False):
    m, k = x.shape
    weight = w_or_weight if isinstance(w_or_weight, capi.Weight) else ctx.weight(fmt, w_or_weight)
    n = weight.cols
    a = ctx.upload(x.astype(np.float16) if f16 else x)
    c = ctx.buffer(m * n * 4)
    dbuf = ctx.upload(d) if d is not None else None
    ctx.set_route(route)
    try:
        (ctx.matmul_q_f16a if f16 else ctx.matmul_q)(a, weight, c, m, dbuf)
        out = c.download(np.float32, m * n).reshape(m, n)
    finally:
        ctx.set_route(capi.ROUTE_AUTO)
        a.free(); c.free()
        if dbuf is not None:
            dbuf.free()
        if weight is not w_or_weight:
            weight.free()
    return out


# ---- weights: bit-exact ------------------------------------------------------------------

@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("shape", [(32, 1), (64, 7), (576, 192), (1536, 576), (1024, 300)])
def test_device_weight_is_bit_exact(ctx, orc, fmt, shape):
    k, n = shape
    w = synth.normal(7 + k + n, k * n, 0.02).reshape(k, n)
    want_packed = orc.quantize(fmt, w)
    want = orc.dequantize(fmt, want_packed, k, n)
    wt = ctx.weight(fmt, w)
    assert (bits(wt.dequantize()) == bits(want)).all()
    assert (wt.export_ref() == want_packed).all()
    wt.free()
    # the same weight from pre-packed bytes and from the device-side quantizer
    wt = ctx.weight_from_packed(fmt, want_packed, k, n)
    assert (bits(wt.dequantize()) == bits(want)).all()
    wt.free()
    src = ctx.upload(w)
    wt = ctx.weight_from_device(fmt, src, k, n)
    assert (wt.export_ref() == want_packed).all()
    wt.free(); src.free()
    # and from the same matrix stored [N, K], as a matmul_bt operand keeps it
    wt = ctx.weight_nk(fmt, np.ascontiguousarray(w.T))
    assert (wt.export_ref() == want_packed).all()
    wt.free()


def test_device_quantizer_matches_golden_vectors(ctx):
    from helpers import check_golden_packed, golden_vectors
    vectors, _ = golden_vectors()
    for name, fmt, w, entry in vectors:
        src = ctx.upload(w)
        for wt in (ctx.weight(fmt, w), ctx.weight_from_device(fmt, src, *w.shape)):
            check_golden_packed(name, wt.export_ref(), entry)
            deq = wt.dequantize().reshape(-1)
            for idx, bits_ in entry.get("dequant_f32_bits", {}).items():
                assert int(deq[int(idx)].view(np.uint32)) == bits_, name
            wt.free()
        src.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_device_weight_extreme_scales(ctx, orc, fmt):
    # half-subnormal scales must decode as the half crate does (kept, not flushed),
    # and the device quantizer must agree on ties, zero and constant blocks
    rng = np.random.default_rng(12)
    k, n = 64, 48
    w = rng.standard_normal((k, n)).astype(np.float32)
    w[:, 0] *= 1e-6
    w[:, 1] *= 3e-8
    w[:, 2] *= 1e3
    w[:, 3] = 0.0
    w[:, 4] = 0.375
    w[:32, 5] = np.linspace(0, 15, 32, dtype=np.float32)
    w[:32, 6] = np.arange(32, dtype=np.float32) * 0.5
    w[0, 7] = 127.0
    w[1:5, 7] = [0.5, 2.5, -0.5, -2.5]
    want_packed = orc.quantize(fmt, w)
    want = orc.dequantize(fmt, want_packed, k, n)
    wt = ctx.weight(fmt, w)
    assert (bits(wt.dequantize()) == bits(want)).all()
    wt.free()
    src = ctx.upload(w)
    wt = ctx.weight_from_device(fmt, src, k, n)
    assert (wt.export_ref() == want_packed).all()
    assert (bits(wt.dequantize()) == bits(want)).all()
    wt.free(); src.free()


def test_weight_errors(ctx):
    with pytest.raises(capi.MgnError, match="multiple of 32"):
        ctx.weight(Q4, np.zeros((48, 8), np.float32))
    wt = ctx.weight(Q4, np.zeros((64, 8), np.float32))
    a = ctx.buffer(4 * 10)
    c = ctx.buffer(4 * 8)
    with pytest.raises(capi.MgnError, match="smaller"):
        ctx.matmul_q(a, wt, c, 1)
    a.free(); c.free(); wt.free()


# ---- matmul: every route at small and ragged shapes ----------------------------------------

# (route, m, k, n) combinations of the tests below that a forced kernel family refuses, each with
# the reason; every other combination must run and match the oracle (the automatic route never refuses)
REFUSED = {
    # the vector-ALU GEMV keeps all K groups of a column in one workgroup and the staged activations in LDS
    ("gemv_valu", 4, 14336, 518), ("gemv_valu", 3, 12288, 64), ("gemv_valu", 1, 18944, 132),
    ("gemv_valu", 4, 11008, 260), ("gemv_valu", 3, 13824, 70), ("gemv_valu", 4, 14336, 70),
    # both GEMV kernels serve at most four activation rows
    ("gemv_valu", 6, 1024, 300), ("gemv_mfma", 6, 1024, 300), ("gemv_valu", 16, 4096, 2048), ("gemv_mfma", 16, 4096, 2048),
}

ROUTES = {"generic": capi.ROUTE_GENERIC, "gemv_valu": capi.ROUTE_GEMV_VALU, "gemv_mfma": capi.ROUTE_GEMV_MFMA,
          "gemm_mfma": capi.ROUTE_GEMM_MFMA, "tile_mfma": capi.ROUTE_TILE_MFMA, "auto": capi.ROUTE_AUTO}


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("route", ["generic", "gemv_valu", "gemv_mfma", "gemm_mfma", "tile_mfma", "auto"])
@pytest.mark.parametrize("m,k,n", [
    (1, 32, 1), (1, 64, 3), (1, 576, 192), (1, 576, 577), (1, 1536, 576), (1, 1024, 100),
    (2, 576, 65), (3, 2048, 130), (4, 4096, 257), (1, 14336, 64), (1, 3072, 1024),
    # K a multiple of 512 (full steps only) with a ragged last quad, waves without a quad, several quads per wave
    (2, 512, 2055), (1, 512, 32774),
    # four rows of a long K: the GEMV kernel cuts K into parts for different workgroups
    (4, 14336, 518), (3, 12288, 64),
    # K splits that do not share the 16-block steps evenly, with a partial last step
    (1, 11008, 132), (2, 11040, 66),
    # K parts that are not even: 37 and 21.5 steps of 16 blocks
    (1, 18944, 132), (4, 11008, 260), (3, 13824, 70),
    # one full step plus 2, 1, 4 leftover blocks and very many columns: the quads of a wave share a
    # step for the leftovers (Q4); ragged last quad, last wave with fewer than four quads
    (1, 576, 40000), (2, 544, 33001), (4, 640, 36002), (3, 576, 49153),
])
def test_small_m_routes(ctx, orc, fmt, route, m, k, n):
    x = synth.normal(1000 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(2000 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(3000 + n, m * n).reshape(m, n)
    if (route, m, k, n) in REFUSED:
        with pytest.raises(capi.MgnError, match="does not support"):
            run_matmul(ctx, fmt, x, w, ROUTES[route])
        return
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    got = run_matmul(ctx, fmt, x, w, ROUTES[route])
    got_d = run_matmul(ctx, fmt, x, w, ROUTES[route], d=d)
    orc.assert_close(got, orc.matmul_f32(x, deq), REL, ABS)
    orc.assert_close(got_d, orc.matmul_f32(x, deq, d), REL, ABS)


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n", [(1, 576, 192), (1, 4096, 257), (3, 1024, 100), (4, 14336, 70), (2, 11040, 66)])
def test_small_m_fp16_activations(ctx, orc, fmt, m, k, n):
    """mgn_matmul_q_f16a at decode sizes: the GEMV kernel widens the halves while it stages the
    activations; the oracle multiplies the rounded values."""
    x = synth.normal(21 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(22 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(23 + n, m * n).reshape(m, n)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    x16 = x.astype(np.float16).astype(np.float32)
    for route in ("generic", "gemv_mfma", "auto"):
        got = run_matmul(ctx, fmt, x, w, ROUTES[route], d=d, f16=True)
        orc.assert_close(got, orc.matmul_f32(x16, deq, d), REL, ABS)


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n", [(5, 64, 70), (6, 1024, 2048), (16, 576, 130), (17, 256, 64), (64, 128, 96), (130, 96, 67),
                                   (70, 2048, 200), (40, 4128, 48), (33, 1056, 530)])  # row groups with K parts, ragged K
def test_larger_m(ctx, orc, fmt, m, k, n):
    x = synth.normal(11 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(12 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(13 + n, m * n).reshape(m, n)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    for route in ("generic", "gemm_mfma", "tile_mfma", "auto"):
        got = run_matmul(ctx, fmt, x, w, ROUTES[route], d=d)
        orc.assert_close(got, orc.matmul_f32(x, deq, d), REL, ABS)
        # fp16 activations: the oracle multiplies the rounded values
        x16 = x.astype(np.float16).astype(np.float32)
        got = run_matmul(ctx, fmt, x, w, ROUTES[route], f16=True)
        orc.assert_close(got, orc.matmul_f32(x16, deq), REL, ABS)


def _random_shapes(count, seed=0x4D474E51):
    """Seeded shapes across every route's territory: M from the GEMV sizes to several row tiles,
    K any multiple of 32 up to past the K-part thresholds, N ragged more often than not."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = int(rng.choice([1, 1, 1, 2, 2, 3, 4, 4, 5, 8, 15, 16, 17, 31, 33, 70]))
        k = 32 * int(rng.choice([rng.integers(1, 20), rng.integers(20, 160), rng.integers(160, 640)]))
        budget = 60_000_000 // (m * k)  # keeps the oracle's triple loop short
        n = int(min(rng.choice([rng.integers(1, 40), rng.integers(40, 700), rng.integers(700, 9000)]), max(1, budget)))
        out.append((m, k, n))
    return out


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n", _random_shapes(40))
def test_random_shapes_on_the_automatic_route(ctx, orc, fmt, m, k, n):
    """What a caller gets without choosing a kernel, on shapes nobody picked by hand; the
    generic kernel on the same inputs is the second opinion.  With and without a residual,
    and from fp16 activations."""
    x = synth.normal(31 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(32 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(33 + n, m * n).reshape(m, n)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    weight = ctx.weight(fmt, w)
    try:
        want = orc.matmul_f32(x, deq)
        orc.assert_close(run_matmul(ctx, fmt, x, weight), want, REL, ABS)
        orc.assert_close(run_matmul(ctx, fmt, x, weight, ROUTES["generic"]), want, REL, ABS)
        orc.assert_close(run_matmul(ctx, fmt, x, weight, d=d), orc.matmul_f32(x, deq, d), REL, ABS)
        x16 = x.astype(np.float16).astype(np.float32)
        orc.assert_close(run_matmul(ctx, fmt, x, weight, f16=True), orc.matmul_f32(x16, deq), REL, ABS)
    finally:
        weight.free()


def test_reference_q4_matmul_correctness_inputs(ctx, orc):
    # tests/gpu_smoke.rs:2681-2771 (m=6, k=1024, n=2048; the reference's own bar is abs 0.1)
    a, b = ref_test_inputs_q4_matmul()
    packed = orc.quantize(Q4, b)
    want = orc.matmul_packed(Q4, a, packed, 2048)
    for route in ("generic", "auto"):
        got = run_matmul(ctx, Q4, a, b, ROUTES[route])
        assert np.abs(got - want).max() < 0.1
        orc.assert_close(got, want, REL, ABS)
    # and row by row through the M=1 route
    for r in (0, 5):
        got = run_matmul(ctx, Q4, a[r:r + 1], b)
        orc.assert_close(got, want[r:r + 1], REL, ABS)


def test_linearity_and_zero_input(ctx):
    # size-independent properties: W(0) = 0; W(x + y) = W(x) + W(y) to rounding; W(2x) = 2 W(x) exactly
    k, n = 4096, 1024
    w = synth.weights(5, k, n)
    wt = ctx.weight(Q4, w)
    x = synth.activations(5, 1, k)
    y = synth.activations(5, 1, k, which=1)
    fx = run_matmul(ctx, Q4, x, wt)
    assert (run_matmul(ctx, Q4, np.zeros_like(x), wt) == 0).all()
    assert (run_matmul(ctx, Q4, 2 * x, wt) == 2 * fx).all()
    fy = run_matmul(ctx, Q4, y, wt)
    fxy = run_matmul(ctx, Q4, x + y, wt)
    assert np.abs(fxy - (fx + fy)).max() < 2e-4
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n,route", [(16, 4096, 2048, "gemm_mfma"), (4, 14336, 1024, "gemv_mfma"), (16, 14336, 1024, "tile_mfma")])
def test_split_k_is_repeatable(ctx, orc, fmt, m, k, n, route):
    """Few tiles and a long K: the tiled kernel splits K across workgroups and the last
    one to arrive adds the partial tiles in part order (the GEMV kernel does the same when
    four rows of a long K do not fit in LDS).  Alternating two inputs makes a
    partial tile left over from the previous call wrong for this one, so a stale read
    shows; the result must also be the same bits every time."""
    w = synth.normal(91 + fmt, k * n, 0.02).reshape(k, n)
    wt = ctx.weight(fmt, w)
    packed = orc.quantize(fmt, w)
    xs = [synth.normal(92 + i, m * k, 1.0).reshape(m, k) for i in range(2)]
    bufs = [ctx.upload(x) for x in xs]
    c = ctx.buffer(m * n * 4)
    ctx.set_route(ROUTES[route])
    try:
        first = []
        for i in range(2):
            ctx.matmul_q(bufs[i], wt, c, m, None)
            first.append(c.download(np.float32, m * n).reshape(m, n))
            orc.assert_close(first[i], orc.matmul_packed(fmt, xs[i], packed, n), REL, ABS)
        for it in range(40):
            i = it & 1
            ctx.matmul_q(bufs[i], wt, c, m, None)
            got = c.download(np.float32, m * n).reshape(m, n)
            assert (bits(got) == bits(first[i])).all(), f"call {it} differs from the first call with the same input"
    finally:
        ctx.set_route(capi.ROUTE_AUTO)
        for b in bufs:
            b.free()
        c.free()
        wt.free()


def _rms_norm_f32(x, g, eps):
    # src/shaders/rms_norm.wgsl:1-57 in f32: x * rsqrt(mean(x^2) + eps) * weight
    ms = (x.astype(np.float64) ** 2).mean(1, keepdims=True)
    r = (1.0 / np.sqrt(ms + eps)).astype(np.float32)
    return (x * r) * g


def _swiglu_f32(gate_up):
    k = gate_up.shape[1] // 2
    gate, up = gate_up[:, :k], gate_up[:, k:]
    sig = (1.0 / (1.0 + np.exp(-gate.astype(np.float64)))).astype(np.float32)
    return gate * sig * up


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n,resid", [(1, 576, 576, False), (1, 576, 3072, False), (2, 576, 192, True),
                                         (1, 4096, 1024, True), (1, 1536, 576, True)])
def test_fused_prologues(ctx, orc, fmt, m, k, n, resid):
    """rms_norm -> matmul and swiglu_concat -> matmul in one launch, against the two steps
    done separately on the CPU (pointwise op in f32 with numpy, then the oracle's matmul)."""
    w = synth.normal(500 + k + n, k * n, 0.02).reshape(k, n)
    packed = orc.quantize(fmt, w)
    wt = ctx.weight(fmt, w)
    assert ctx.can_fuse(wt, m)
    d = synth.normal(501, m * n, 1.0).reshape(m, n) if resid else None
    dbuf = ctx.upload(d) if resid else None
    c = ctx.buffer(m * n * 4)
    # rms_norm
    x = synth.normal(502 + m, m * k, 3.0).reshape(m, k)
    g = 1.0 + 0.25 * synth.normal(503, k, 1.0)
    xb, gb = ctx.upload(x), ctx.upload(g)
    ctx.matmul_q_rms_norm(xb, gb, 1e-5, wt, c, m, dbuf)
    got = c.download(np.float32, m * n).reshape(m, n)
    orc.assert_close(got, orc.matmul_packed(fmt, _rms_norm_f32(x, g, 1e-5), packed, n, d), REL, ABS)
    # swiglu over gate | up
    gu = synth.normal(504 + m, m * 2 * k, 1.5).reshape(m, 2 * k)
    gub = ctx.upload(gu)
    ctx.matmul_q_swiglu(gub, wt, c, m, dbuf)
    got = c.download(np.float32, m * n).reshape(m, n)
    orc.assert_close(got, orc.matmul_packed(fmt, _swiglu_f32(gu), packed, n, d), REL, ABS)
    for b in (xb, gb, gub, c) + ((dbuf,) if resid else ()):
        b.free()
    wt.free()


def test_fused_prologue_is_refused_where_it_cannot_run(ctx):
    k, n = 576, 64
    wt = ctx.weight(Q4, synth.normal(510, k * n, 0.02).reshape(k, n))
    x = ctx.upload(synth.normal(511, 8 * k, 1.0))
    g = ctx.upload(np.ones(k, np.float32))
    c = ctx.buffer(8 * n * 4)
    assert not ctx.can_fuse(wt, 8)
    with pytest.raises(capi.MgnError) as e:
        ctx.matmul_q_rms_norm(x, g, 1e-5, wt, c, 8)
    assert e.value.status == capi.EUNSUPPORTED
    short = ctx.upload(np.ones(k - 1, np.float32))
    with pytest.raises(capi.MgnError) as e:
        ctx.matmul_q_rms_norm(x, short, 1e-5, wt, c, 1)
    assert e.value.status == capi.EINVAL
    for b in (x, g, c, short):
        b.free()
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,ns", [(1, 576, (576, 192, 192)), (2, 576, (64, 6)), (1, 4096, (1024, 132, 4096)), (1, 64, (8, 4, 12))])
def test_batched_matmuls_share_one_launch(ctx, orc, fmt, m, k, ns):
    """Up to three weights on the same activations in one launch (q, k, v), with and without
    a prologue and residuals.  The K split is planned for the whole batch, so the summation
    order may differ from the single-weight launch: compared at the matmul bar, not bitwise."""
    x = synth.normal(700 + k, m * k, 1.0).reshape(m, k)
    xb = ctx.upload(x)
    ws = [synth.normal(701 + j, k * n, 0.02).reshape(k, n) for j, n in enumerate(ns)]
    wts = [ctx.weight(fmt, w) for w in ws]
    ds = [synth.normal(710 + j, m * n, 1.0).reshape(m, n) if j == 1 else None for j, n in enumerate(ns)]
    dbs = [ctx.upload(d) if d is not None else None for d in ds]
    cs = [ctx.buffer(m * n * 4) for n in ns]
    single = ctx.buffer(m * max(ns) * 4)
    ctx.set_route(capi.ROUTE_GEMV_MFMA)
    try:
        ctx.matmul_q_batch(xb, list(zip(wts, cs, dbs)), m)
        for j, n in enumerate(ns):
            got = cs[j].download(np.float32, m * n).reshape(m, n)
            orc.assert_close(got, orc.matmul_packed(fmt, x, orc.quantize(fmt, ws[j]), n, ds[j]), REL, ABS)
            ctx.matmul_q(xb, wts[j], single, m, dbs[j])
            orc.assert_close(single.download(np.float32, m * n).reshape(m, n), got, REL, ABS)
        # with the norm folded in
        g = ctx.upload(1.0 + 0.25 * synth.normal(720, k, 1.0))
        ctx.matmul_q_batch(xb, list(zip(wts, cs, dbs)), m, capi.PROLOGUE_RMS_NORM, g, 1e-5)
        for j, n in enumerate(ns):
            got = cs[j].download(np.float32, m * n)
            ctx.matmul_q_rms_norm(xb, g, 1e-5, wts[j], single, m, dbs[j])
            orc.assert_close(single.download(np.float32, m * n), got, REL, ABS)
        g.free()
    finally:
        ctx.set_route(capi.ROUTE_AUTO)
    # different K in one batch is an argument error
    other = ctx.weight(fmt, synth.normal(730, 2 * k * 8, 0.02).reshape(2 * k, 8))
    with pytest.raises(capi.MgnError) as e:
        ctx.matmul_q_batch(xb, [(wts[0], cs[0], None), (other, cs[1], None)], m)
    assert e.value.status == capi.EINVAL
    other.free()
    for b in [xb, single] + cs + [d for d in dbs if d is not None]:
        b.free()
    for w in wts:
        w.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_weight_file_round_trip(ctx, orc, fmt, tmp_path):
    """save -> load gives the same weight byte for byte; foreign, truncated and inconsistent
    files are refused with a status, never loaded."""
    k, n = 576, 130
    w = synth.normal(950 + fmt, k * n, 0.02).reshape(k, n)
    wt = ctx.weight(fmt, w)
    path = tmp_path / "w.mgnq"
    wt.save(path)
    raw = path.read_bytes()
    assert raw[:4] == b"MGNQ" and len(raw) == 40 + len(orc.quantize(fmt, w))
    assert (np.frombuffer(raw[40:], np.uint8) == orc.quantize(fmt, w)).all()
    back = ctx.load_weight(path)
    assert (back.fmt, back.rows, back.cols) == (fmt, k, n)
    assert (back.export_ref() == wt.export_ref()).all()
    x = synth.normal(951, k, 1.0).reshape(1, k)
    assert (bits(run_matmul(ctx, fmt, x, back)) == bits(run_matmul(ctx, fmt, x, wt))).all()
    back.free()
    wt.free()
    with pytest.raises(capi.MgnError) as e:
        ctx.load_weight(tmp_path / "missing.mgnq")
    assert e.value.status == capi.ENOTFOUND
    for name, data in (("foreign", b"GGUF" + raw[4:]), ("truncated", raw[:-7]), ("version", raw[:4] + b"\x02\0\0\0" + raw[8:]),
                       ("shape", raw[:16] + (k + 32).to_bytes(8, "little") + raw[24:])):
        p = tmp_path / name
        p.write_bytes(data)
        with pytest.raises(capi.MgnError) as e:
            ctx.load_weight(p)
        assert e.value.status == capi.EINVAL, name


UNARY = {"relu": capi.UNARY_RELU, "sigmoid": capi.UNARY_SIGMOID, "neg": capi.UNARY_NEG, "silu": capi.UNARY_SILU}


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("route", ["generic", "gemv_valu", "gemv_mfma", "gemm_mfma", "tile_mfma", "auto"])
@pytest.mark.parametrize("m,k,n", [(1, 576, 192), (4, 14336, 70), (6, 1024, 300), (16, 4096, 2048)])
def test_unary_epilogues(ctx, orc, fmt, route, m, k, n):
    """C = f(A x W + D) in the matmul's own launch: every operation the reference folds into a
    matmul (Relu, Sigmoid, Neg, Silu; compile.rs:915-1035), a chain of two, with and without the
    residual, on every kernel family (K parts and split-K shapes included)."""
    x = synth.normal(31 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(32 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(33 + n, m * n).reshape(m, n)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    plain = orc.matmul_f32(x, deq)
    plain_d = orc.matmul_f32(x, deq, d)
    wt = ctx.weight(fmt, w)
    a = ctx.upload(x)
    db = ctx.upload(d)
    c = ctx.buffer(m * n * 4)
    ctx.set_route(ROUTES[route])
    try:
        for chain, with_d in ((("relu",), False), (("sigmoid",), True), (("neg",), False), (("silu",), True),
                              (("relu", "neg"), True), ((), False)):
            if (route, m, k, n) in REFUSED:
                with pytest.raises(capi.MgnError, match="does not support"):
                    ctx.matmul_q_epilogue(a, wt, c, m, [UNARY[o] for o in chain], db if with_d else None)
                continue
            ctx.matmul_q_epilogue(a, wt, c, m, [UNARY[o] for o in chain], db if with_d else None)
            got = c.download(np.float32, m * n).reshape(m, n)
            want = plain_d if with_d else plain
            for o in chain:
                want = orc.unary(o, want)
            orc.assert_close(got, want, REL, ABS)
    finally:
        ctx.set_route(capi.ROUTE_AUTO)
        a.free(); db.free(); c.free(); wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,k,n", [(1, 576, 192), (3, 4096, 257), (6, 1024, 300), (33, 96, 67), (70, 2048, 40)])
def test_transposed_activations(ctx, orc, fmt, m, k, n):
    """mgn_matmul_q_at: A arrives as [K, M] (the MatMulAT / FusedMatMulATAdd dispatches); the result
    is the plain matmul on A^T, with the residual and an epilogue, and a second call with a larger
    M (the staging area grows) leaves the first result's inputs alone."""
    x = synth.normal(41 + m + k + n, m * k).reshape(m, k)
    w = synth.normal(42 + m + k + n, k * n, 0.02).reshape(k, n)
    d = synth.normal(43 + n, m * n).reshape(m, n)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    weight = ctx.weight(fmt, w)
    a_t = ctx.upload(np.ascontiguousarray(x.T))
    dbuf = ctx.upload(d)
    c = ctx.buffer(m * n * 4)
    try:
        ctx.matmul_q_at(a_t, weight, c, m)
        orc.assert_close(c.download(np.float32, m * n).reshape(m, n), orc.matmul_f32(x, deq), REL, ABS)
        ctx.matmul_q_at(a_t, weight, c, m, d=dbuf, ops=[capi.UNARY_NEG, capi.UNARY_RELU])
        want = orc.unary("relu", orc.unary("neg", orc.matmul_f32(x, deq, d)))
        orc.assert_close(c.download(np.float32, m * n).reshape(m, n), want, REL, ABS)
        # a taller A^T right behind it: the staging area is replaced while nothing reads it
        m2 = m + 40
        x2 = synth.normal(44 + m + k + n, m2 * k).reshape(m2, k)
        a2 = ctx.upload(np.ascontiguousarray(x2.T))
        c2 = ctx.buffer(m2 * n * 4)
        ctx.matmul_q_at(a2, weight, c2, m2)
        ctx.matmul_q_at(a_t, weight, c, m)
        orc.assert_close(c2.download(np.float32, m2 * n).reshape(m2, n), orc.matmul_f32(x2, deq), REL, ABS)
        orc.assert_close(c.download(np.float32, m * n).reshape(m, n), orc.matmul_f32(x, deq), REL, ABS)
        a2.free(); c2.free()
        with pytest.raises(capi.MgnError):  # A^T shorter than K x m
            ctx.matmul_q_at(a_t, weight, c, m + 1)
    finally:
        a_t.free(); dbuf.free(); c.free(); weight.free()


def test_epilogue_arguments_are_checked(ctx):
    wt = ctx.weight(Q4, synth.normal(970, 64 * 8, 0.02).reshape(64, 8))
    a = ctx.buffer(4 * 64)
    c = ctx.buffer(4 * 8)
    with pytest.raises(capi.MgnError) as e:
        ctx.matmul_q_epilogue(a, wt, c, 1, [capi.UNARY_RELU] * 9)
    assert e.value.status == capi.EINVAL
    with pytest.raises(capi.MgnError) as e:
        ctx.matmul_q_epilogue(a, wt, c, 1, [7])
    assert e.value.status == capi.EINVAL
    a.free(); c.free(); wt.free()


def test_matmul_loop_is_the_same_calls_in_a_row(ctx, orc):
    """mgn_matmul_q_loop enqueues call i on weights[i % count]: after five steps over two
    weights the output is what the first weight gives (bit for bit the single call's)."""
    k, n, m = 576, 192, 1
    ws = [synth.normal(960 + j, k * n, 0.02).reshape(k, n) for j in range(2)]
    wts = [ctx.weight(Q4, w) for w in ws]
    x = synth.normal(962, m * k).reshape(m, k)
    a = ctx.upload(x)
    c = ctx.buffer(m * n * 4)
    ctx.matmul_q(a, wts[0], c, m)
    single = c.download(np.float32, m * n)
    ctx.matmul_q_loop(a, wts, c, m, 4)
    assert (bits(c.download(np.float32, m * n)) != bits(single)).any()  # the fourth call ran on the other weight
    ctx.matmul_q_loop(a, wts, c, m, 5)
    assert (bits(c.download(np.float32, m * n)) == bits(single)).all()
    orc.assert_close(single.reshape(m, n), orc.matmul_packed(Q4, x, orc.quantize(Q4, ws[0]), n), REL, ABS)
    a.free(); c.free()
    for w in wts:
        w.free()


def test_engine_clock_probes_return_plausible_figures(ctx):
    """mgn_engine_clock_mhz (a measurement aid): the shader clock against the 100 MHz counter, from one
    idle wave and under a matrix-instruction load on every CU, with the load's cycles per round; the
    probes use the head of the split-K workspace and must leave the context usable."""
    idle = ctx.engine_clock_mhz()
    loaded, cycles = ctx.engine_probe()
    assert 500.0 < idle < 4000.0 and 500.0 < loaded < 4000.0
    assert 64.0 <= cycles < 5000.0  # at least the eight matrix instructions of a round, at 8 cycles each
    ctx.sync()


def test_weight_read_loop_leaves_results_alone(ctx, orc):
    """mgn_weight_read_loop (a timing aid: plain reads of the packed bytes) runs on weights of
    both formats, the smallest included, and a K-part matmul enqueued right behind it, whose
    partial sums use the workspace the probe's sink lives in, still gives the oracle's result."""
    with pytest.raises(capi.MgnError):
        ctx.weight_read_loop([], 3)
    tiny = ctx.weight(Q8, synth.normal(975, 32, 0.02).reshape(32, 1))
    ctx.weight_read_loop([tiny], 3)
    ctx.weight_read_loop([tiny], 3, pattern=1)
    with pytest.raises(capi.MgnError):
        ctx.weight_read_loop([tiny], 1, pattern=2)
    m, k, n = 4, 14336, 70
    for fmt in (Q4, Q8):
        w = synth.normal(976 + fmt, k * n, 0.02).reshape(k, n)
        x = synth.normal(978, m * k).reshape(m, k)
        wt = ctx.weight(fmt, w)
        a = ctx.upload(x)
        c = ctx.buffer(m * n * 4)
        ctx.weight_read_loop([wt, tiny], 7)
        ctx.weight_read_loop([wt, tiny], 4, pattern=1)
        ctx.matmul_q(a, wt, c, m)
        ctx.weight_read_loop([wt], 2)
        ctx.weight_read_loop([wt], 2, pattern=1)
        got = c.download(np.float32, m * n).reshape(m, n)
        orc.assert_close(got, orc.matmul_packed(fmt, x, orc.quantize(fmt, w), n), REL, ABS)
        a.free(); c.free(); wt.free()
    tiny.free()


def test_zero_rows_is_a_no_op(ctx):
    wt = ctx.weight(Q4, synth.normal(970, 64 * 8, 0.02).reshape(64, 8))
    a = ctx.buffer(4 * 64)
    c = ctx.upload(np.full(8, 7.0, np.float32))
    ctx.matmul_q(a, wt, c, 0)
    ctx.matmul_q_f16a(a, wt, c, 0)
    assert (c.download(np.float32, 8) == 7.0).all()
    a.free(); c.free(); wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m", [1, 4])
def test_a_column_with_infinite_scales_stays_on_its_own(ctx, orc, fmt, m):
    """K = 576 is 18 blocks: the GEMV kernel's second 16-block step reads past the end of a
    column into the next one's blocks (against zero activations).  Scales of +inf in column 1
    must make column 1 non-finite and leave every other column as it was."""
    k, n = 576, 8
    bpc = k // 32
    w = synth.normal(990, k * n, 0.02).reshape(k, n)
    x = synth.normal(991 + m, m * k, 1.0).reshape(m, k)
    packed = orc.quantize(fmt, w).copy()
    clean = orc.matmul_packed(fmt, x, packed, n)
    for kb in range(bpc):
        blk = 1 * bpc + kb
        if fmt == Q4:
            packed[blk * 4:blk * 4 + 2] = (0x00, 0x7C)  # d = +inf
        else:
            packed[blk * 36:blk * 36 + 2] = (0x00, 0x7C)
    wt = ctx.weight_from_packed(fmt, packed, k, n)
    a = ctx.upload(x)
    c = ctx.buffer(m * n * 4)
    ctx.set_route(capi.ROUTE_GEMV_MFMA)
    try:
        ctx.matmul_q(a, wt, c, m)
        got = c.download(np.float32, m * n).reshape(m, n)
    finally:
        ctx.set_route(capi.ROUTE_AUTO)
        a.free(); c.free(); wt.free()
    assert not np.isfinite(got[:, 1]).any()
    keep = [j for j in range(n) if j != 1]
    orc.assert_close(got[:, keep], clean[:, keep], REL, ABS)


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,route", [(1, "gemv_mfma"), (4, "gemv_mfma"), (16, "gemm_mfma"), (16, "tile_mfma"), (40, "tile_mfma")])
def test_activations_and_weights_with_a_large_mean(ctx, orc, fmt, m, route):
    """All-positive activations against weights whose blocks sit far from zero: the format's
    additive part (block minimum x sum of activations) and the scaled quant sums are then both
    large and the kernels keep them in separate accumulators or centre them.  Checked against
    the f64 product of the dequantized weights at the matmul bar."""
    k, n = 8192, 160
    x = np.abs(synth.normal(980 + m, m * k, 1.0)).reshape(m, k) + np.float32(0.5)
    w = (synth.normal(981, k * n, 0.02) + np.float32(0.3)).reshape(k, n)
    w[:, 1::2] -= np.float32(0.6)  # every other column far below zero
    packed = orc.quantize(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, packed, k, n))
    got = run_matmul(ctx, fmt, x, w, ROUTES[route])
    orc.assert_close(got, want, REL, ABS)


def assert_close_rowwise(got, want, x):
    """The matmul bar with its absolute part scaled by each row's activation magnitude: the
    reference's 1e-4 is meant for activations of order one, and a row scaled by s has outputs and
    errors scaled by s."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    rms = np.sqrt((np.asarray(x, np.float64) ** 2).mean(axis=1, keepdims=True))
    err = np.abs(got - want)
    ok = (err <= REL * np.abs(want)) | (err <= ABS * rms)
    assert np.isfinite(got).all()
    assert ok.all(), f"{(~ok).sum()} of {ok.size} outside the bar; worst {err.max():.3e} at row {np.unravel_index(err.argmax(), err.shape)[0]}"


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_weights_with_huge_minima_and_scales_stay_on_the_matrix_cores(ctx, orc, fmt):
    """Blocks whose minimum (Q4) or scale (Q8) is far beyond anything a model holds.  The 16x16x32
    tiled kernel multiplies the block's m (or scale) as the fp16 value it is stored as, against
    block means that stay below 2^12, so no weight is out of its range; the automatic route
    takes it for weights the faster 32x32x16 kernel cannot hold -- however the weight was created."""
    m, k, n = 16, 256, 96
    w = synth.normal(990 + fmt, k * n, 0.02).reshape(k, n)
    w[32:64, 5] = np.linspace(-5000.0, -4990.0, 32, dtype=np.float32)   # block minimum -5000
    w[64:96, 7] = np.linspace(-3000.0, 3000.0, 32, dtype=np.float32)    # Q8 scale 23.6
    w[96:128, 9] = np.linspace(-60000.0, 60000.0, 32, dtype=np.float32)  # near the largest half
    x = synth.normal(991, m * k, 1.0).reshape(m, k)
    packed = orc.quantize(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, packed, k, n))
    src = ctx.upload(w)
    for wt in (ctx.weight(fmt, w), ctx.weight_from_device(fmt, src, k, n), ctx.weight_from_packed(fmt, packed, k, n)):
        for route in ("auto", "tile_mfma"):
            got = run_matmul(ctx, fmt, x, wt, ROUTES[route])
            assert np.isfinite(got).all()
            # the huge columns' outputs are of order 1e5: relative bar there, absolute elsewhere
            orc.assert_close(got, want, REL, ABS)
        # the 32x32x16 kernel feeds 32 x m (Q8: 4096 x scale) to the matrix cores as fp16 and refuses the weight
        with pytest.raises(capi.MgnError, match="does not support"):
            run_matmul(ctx, fmt, x, wt, ROUTES["gemm_mfma"])
        got1 = run_matmul(ctx, fmt, x[:1], wt, ROUTES["gemv_mfma"])
        orc.assert_close(got1, want[:1], REL, ABS)
        wt.free()
    src.free()
    # the verdict is the weight's own: an ordinary weight created next is taken by the 32x32x16 kernel
    tame = synth.normal(992 + fmt, k * n, 0.02).reshape(k, n)
    tame_packed = orc.quantize(fmt, tame)
    tame_want = orc.matmul_f64(x, orc.dequantize(fmt, tame_packed, k, n))
    src = ctx.upload(tame)
    for wt in (ctx.weight(fmt, tame), ctx.weight_from_device(fmt, src, k, n), ctx.weight_from_packed(fmt, tame_packed, k, n)):
        orc.assert_close(run_matmul(ctx, fmt, x, wt, ROUTES["gemm_mfma"]), tame_want, REL, ABS)
        wt.free()
    src.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_rows_whose_activation_images_exceed_the_workspace_run_in_blocks(ctx, orc, fmt):
    """The general 16x16x32 kernel keeps the converted activations of a launch in the context's 16 MiB
    workspace (17.25 KiB per 16 rows x 256 elements of f32 activations).  300 rows of K = 16384 need
    21 MB: the rows go out in blocks, one launch pair each, with the residual and the epilogue
    applied per block.  The last block is shorter than the others and ends off a multiple of 16."""
    m, k, n = 300, 16384, 48
    plan = capi.matmul_plan(fmt, m, k, n)
    assert plan.route == capi.ROUTE_TILE_MFMA and plan.quads_per_wave >= 2
    w = synth.normal(980 + fmt, k * n, 0.02).reshape(k, n)
    x = synth.normal(981, m * k, 1.0).reshape(m, k)
    x[7] *= np.float32(3.0e7)   # a row far outside the fp16 range, in the first block
    x[299] *= np.float32(1e-9)  # and a tiny one in the last
    d = synth.normal(982, m * n, 1.0).reshape(m, n)
    packed = orc.quantize(fmt, w)
    want = np.asarray(orc.matmul_f64(x, orc.dequantize(fmt, packed, k, n)), np.float64)
    wt = ctx.weight(fmt, w)
    a, dd, c = ctx.upload(x), ctx.upload(d), ctx.buffer(m * n * 4)
    ctx.matmul_q(a, wt, c, m)
    assert_close_rowwise(c.download(np.float32, m * n).reshape(m, n), want, x)
    ctx.matmul_q(a, wt, c, m, d=dd)
    got = c.download(np.float32, m * n).reshape(m, n)
    rows = np.ones(m, bool)
    rows[[7, 299]] = False  # (their products dwarf or vanish beside a residual of order one)
    assert_close_rowwise(got[rows], want[rows] + d[rows], x[rows])
    assert np.allclose(got[299], d[299], rtol=0, atol=1e-6)
    for b in (a, dd, c):
        b.free()
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_all_zero_columns_give_exactly_the_residual(ctx, orc, fmt):
    """Columns of zeros (the padding of an lm_head, a pruned unit) come out as the residual, bit
    for bit, on every kernel, and zero blocks inside live columns leave those within the bar.  The
    reference's Q8 quantizer gives an all-zero block the scale 1.0 (src/runtime.rs:2171), about a
    thousand times its neighbours': a kernel that forms scale * (sum (q + 128) x - 128 sum x) with
    that scale leaves rounding of the size of an ordinary output there.  Such weights still export
    to the bytes they were made from and dequantize as the oracle does."""
    k, n = 2080, 150
    w = synth.normal(1301, k * n, 0.02).reshape(k, n)
    zero_cols = [0, 77, n - 1]
    for j in zero_cols:
        w[:, j] = 0.0
    w[64:96, 5] = 0.0
    w[2048:2080, 140] = 0.0
    w[0:512, 33] = 0.0
    packed = orc.quantize(fmt, w)
    deq = orc.dequantize(fmt, packed, k, n)
    weights = [ctx.weight_from_packed(fmt, packed, k, n), ctx.weight(fmt, w)]
    src = ctx.upload(w)
    weights.append(ctx.weight_from_device(fmt, src, k, n))
    for wt in weights:
        assert (wt.export_ref() == packed).all()
        assert (bits(wt.dequantize()) == bits(deq)).all()
    wt = weights[0]
    for m in (1, 3, 6, 16, 40, 70):
        x = synth.normal(1302 + m, m * k, 1.0).reshape(m, k)
        d = synth.normal(1303 + m, m * n).reshape(m, n)
        for f16 in (False, True):
            xin = x.astype(np.float16).astype(np.float32) if f16 else x
            want = orc.matmul_f64(xin, deq, d)
            for route in ("generic", "gemv_mfma", "gemm_mfma", "tile_mfma", "auto"):
                if (route == "gemv_mfma" and m > 4) or (route in ("gemm_mfma", "tile_mfma") and m < 5):
                    continue
                got = run_matmul(ctx, fmt, x, wt, ROUTES[route], d=d, f16=f16)
                assert (bits(got[:, zero_cols]) == bits(d[:, zero_cols])).all(), (m, f16, route)
                orc.assert_close(got, want, REL, ABS)
    for wt in weights:
        wt.free()
    src.free()


def test_q8_zero_blocks_with_foreign_scales_round_trip(ctx, orc):
    """All-zero Q8 blocks with scales the reference's quantizer never writes (0, -0, anything)
    come back byte for byte and dequantize to zeros."""
    k, n = 64, 8
    w = synth.normal(1311, k * n, 0.02).reshape(k, n)
    w[:, :6] = 0.0
    packed = orc.quantize(Q8, w).copy()
    blocks = packed.reshape(-1, 36)
    for b, scale_bits in enumerate([0x0000, 0x8000, 0x3C00, 0x1234, 0x3555, 0xBC00]):
        assert not blocks[b, 4:].any()
        blocks[b, 0], blocks[b, 1] = scale_bits & 0xFF, scale_bits >> 8
    wt = ctx.weight_from_packed(Q8, packed, k, n)
    assert (wt.export_ref() == packed).all()
    assert (bits(wt.dequantize()) == bits(orc.dequantize(Q8, packed, k, n))).all()
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("m,route", [(1, "gemv_mfma"), (2, "gemv_mfma"), (4, "gemv_mfma"), (16, "tile_mfma"), (40, "tile_mfma"),
                                     (16, "gemm_mfma"), (40, "gemm_mfma"), (1, "auto"), (16, "auto"), (40, "auto")])
def test_the_error_scales_with_the_activations(ctx, orc, fmt, f16, m, route):
    """The same activations times 1e-4 .. 3e3 stay within the bar scaled by that factor, on every
    matrix-core kernel.  Two things this pins: block sums of small fp16 activations (a mean kept as
    an fp16 pair loses the sum's low bits from about 1e-3 down), and the one-row Q4 kernel's
    integer digits for blocks whose largest magnitude lies in [2^11, 2^12), where the block's own
    power of two is 1 (1000 and 3000 put most blocks there).  f32 activations on the 32x32x16
    kernel are left out below 1e-2: it does not rescale them and says so."""
    k, n = 1280, 208
    w = synth.normal(1201, k * n, 0.02).reshape(k, n)
    base = synth.normal(1202 + m, m * k, 1.0).reshape(m, k)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    wt = ctx.weight(fmt, w)
    for mag in (1e-4, 1e-3, 1e-2, 1.0, 1000.0, 3000.0):
        if route == "gemm_mfma" and not f16 and mag < 1e-2:
            continue
        x = base * np.float32(mag)
        if f16:
            x = x.astype(np.float16).astype(np.float32)
        got = run_matmul(ctx, fmt, x, wt, ROUTES[route], f16=f16)
        assert_close_rowwise(got, orc.matmul_f64(x, deq), x)
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,route", [(16, "tile_mfma"), (40, "tile_mfma"), (70, "tile_mfma"), (40, "auto")])
def test_fp16_block_sums_at_both_ends_of_the_range(ctx, orc, fmt, m, route):
    """The 16x16x32 kernels carry a block's mean activation as an fp16 pair (the mean cut to fp16,
    and the rest times 2^11).  Rows that put the pair at its limits: every element at 60000 (block
    sums of 1.9e6, means near the largest half), alternating +-65504, every element the smallest
    subnormal half (the mean IS the smallest half), a single smallest half per block (the mean, 2^-29,
    lives in the low part alone), and ordinary rows between them."""
    k, n = 1024, 96
    w = synth.normal(1401, k * n, 0.02).reshape(k, n) + np.float32(0.01)  # (minima and byte bias well away from zero)
    x = synth.normal(1402 + m, m * k, 1.0).reshape(m, k)
    tiny = np.float32(2.0 ** -24)
    x[0, :] = 60000.0
    x[1, 0::2], x[1, 1::2] = 65504.0, -65504.0
    x[2, :] = tiny
    x[3, :] = 0.0
    x[3, 5::32] = tiny
    x[4, :] = 0.0
    x[4, 0::32], x[4, 1::32] = 65504.0, tiny
    x = x.astype(np.float16).astype(np.float32)
    deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n)
    wt = ctx.weight(fmt, w)
    got = run_matmul(ctx, fmt, x, wt, ROUTES[route], f16=True)
    assert_close_rowwise(got, orc.matmul_f64(x, deq), x)
    # the additive part alone must come out: rows 2 and 3 against what the sums times the minima give
    want = orc.matmul_f64(x, deq)
    for r in (2, 3):
        assert np.abs(got[r] - want[r]).max() <= 2e-3 * np.abs(want[r]).max(), r
    wt.free()


def weight_scaled_bar(got, want, x, factor, abs_bar=ABS):
    """The matmul bar for weights scaled by `factor`: outputs and errors scale with it, so the
    absolute part does too (and with each row's activation magnitude)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    rms = np.sqrt((np.asarray(x, np.float64) ** 2).mean(axis=1, keepdims=True))
    err = np.abs(got - want)
    ok = (err <= REL * np.abs(want)) | (err <= abs_bar * factor * rms)
    assert np.isfinite(got).all()
    return ok, err


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m,route", [(1, "gemv_mfma"), (4, "gemv_mfma"), (9, "tile_mfma"), (49, "tile_mfma"), (9, "gemm_mfma"),
                                     (49, "gemm_mfma"), (1, "auto"), (9, "auto"), (49, "auto")])
def test_the_error_scales_with_the_weights(ctx, orc, fmt, m, route):
    """Weights of N(0, 0.02) times 1e-6 .. 1e3 on every matrix-core kernel: block scales and minima
    from fp16 subnormals up to values near the largest half.  The result must stay within the bar
    scaled by the factor.  (Q8 scales that are fp16 subnormals, block maxima below 0.0077, once cost
    the 16x16x32 kernels 2 .. 8 times the bar with f32 activations: the matrix cores drop low product
    bits of a subnormal operand, and the byte bias term -128 * scale * sum(x) hands them the scales.
    Those kernels now multiply the constants by a power of two first.)"""
    k, n = 1280, 208
    base_w = synth.normal(1301, k * n, 0.02).reshape(k, n)
    x = synth.normal(1302 + m, m * k, 1.0).reshape(m, k)
    for factor in (1e-6, 1e-5, 1e-3, 1e-2, 1.0, 30.0, 1e3):
        w = (base_w * np.float32(factor)).astype(np.float32)
        packed = orc.quantize(fmt, w)
        want = orc.matmul_f64(x, orc.dequantize(fmt, packed, k, n))
        wt = ctx.weight(fmt, w)
        try:
            if route == "gemm_mfma":
                # the 32x32x16 kernel takes a weight only while its block constants fit fp16 operands;
                # beyond that the forced route is refused and the automatic one goes elsewhere
                try:
                    got = run_matmul(ctx, fmt, x, wt, ROUTES[route])
                except capi.MgnError as e:
                    assert factor >= 30.0 and e.status == capi.EINVAL, (factor, str(e))
                    continue
            else:
                got = run_matmul(ctx, fmt, x, wt, ROUTES[route])
            ok, err = weight_scaled_bar(got, want, x, factor, ABS)
            assert ok.all(), (f"factor {factor}: {(~ok).sum()} of {ok.size} outside the bar; worst {err.max():.3e} "
                              f"= {err.max() / factor:.3e} x factor")
        finally:
            wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m", [5, 16])
def test_a_slice_beyond_2_to_the_100_gives_a_non_finite_row(ctx, orc, fmt, m):
    """The rescaling kernels scale every (row, 256-element slice) by a power of two; from 2^100 on
    they do not, and the truncating fp16 conversion would clamp such a value to 65504: a finite,
    wrong result.  The row's sums over that slice are made non-finite instead (the reference's f32
    arithmetic would still be exact there: that magnitude is outside what this library carries,
    and it must say so rather than return a number).  The other rows are untouched."""
    k, n = 768, 112
    w = synth.normal(1401, k * n, 0.02).reshape(k, n)
    x = synth.normal(1402 + m, m * k, 1.0).reshape(m, k)
    x[1, 300] = np.float32(1e31)
    x[3, 10] = np.float32(-3e35)
    wt = ctx.weight(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, orc.quantize(fmt, w), k, n))
    for route in ("tile_mfma", "auto"):
        got = run_matmul(ctx, fmt, x, wt, ROUTES[route])
        assert not np.isfinite(got[1]).any() and not np.isfinite(got[3]).any()
        rest = [r for r in range(m) if r not in (1, 3)]
        assert_close_rowwise(got[rest], want[rest], x[rest])
    wt.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_a_block_beyond_2_to_the_100_gives_a_non_finite_row_on_the_gemv(ctx, orc, fmt, m):
    """The same on the GEMV kernels, which rescale per 32-element block: a block that holds a finite
    magnitude of 2^100 or more makes its row non-finite on the fp16 forms (M = 2..4, Q8) as on the
    one-row Q4 kernel's integer digits; the other rows stay within the bar."""
    k, n = 1024, 96
    w = synth.normal(1411, k * n, 0.02).reshape(k, n)
    x = synth.normal(1412 + m, m * k, 1.0).reshape(m, k)
    x[m - 1, 77] = np.float32(-2e33)
    wt = ctx.weight(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, orc.quantize(fmt, w), k, n))
    for route in ("gemv_mfma", "auto"):
        got = run_matmul(ctx, fmt, x, wt, ROUTES[route])
        assert not np.isfinite(got[m - 1]).any(), route
        if m > 1:
            assert_close_rowwise(got[:m - 1], want[:m - 1], x[:m - 1])
    wt.free()


@pytest.mark.parametrize("seed,shared", [(11, False), (12, False), (13, True)])
def test_random_shapes_magnitudes_and_hand_over_forms(ctx, orc, seed, shared):
    """A seeded random sweep of the kind that found the per-XCD residency limit: 120 shapes per
    seed over both formats, M from 1 to 1000, K from 32 to 16000, N from 1 to 30000, f32 and fp16
    activations of several magnitudes, weights of several magnitudes and offsets, with and without a
    residual, on the automatic route; one seed on a context that shares its device (K parts added
    up by the last part only).  Every result within the matmul bar, with its absolute part scaled
    by the magnitudes at hand; no launch may end in a give-up."""
    rng = np.random.default_rng(seed)
    ctx.set_shared_device(shared)
    try:
        done = 0
        while done < 120:
            fmt = int(rng.integers(0, 2))
            m = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 200, 513, 1000]))
            k = 32 * int(rng.choice([rng.integers(1, 12), rng.integers(12, 100), rng.integers(100, 500)]))
            n = int(rng.choice([rng.integers(1, 40), rng.integers(40, 600), rng.integers(600, 5000), rng.integers(5000, 30000)]))
            if m * k * n > 1.5e9 or k * n > 6.0e7:
                continue
            f16 = bool(rng.integers(0, 2))
            resid = bool(rng.integers(0, 2))
            scale = float(rng.choice([1.0, 1e-2, 1e-4, 300.0]))
            wscale = float(rng.choice([0.03, 0.03, 1e-5, 30.0]))
            woff = float(rng.choice([0.0, 0.0, 1.0, -3.0])) * wscale
            w = (rng.standard_normal((k, n)) * wscale + woff).astype(np.float32)
            x = (rng.standard_normal((m, k)) * scale).astype(np.float32)
            xa = x.astype(np.float16).astype(np.float32) if f16 else x
            d = (rng.standard_normal((m, n)) * scale).astype(np.float32) if resid else None
            deq = orc.dequantize(fmt, orc.quantize(fmt, w), k, n).astype(np.float64)
            want = xa.astype(np.float64) @ deq + (d.astype(np.float64) if resid else 0.0)
            got = run_matmul(ctx, fmt, x, w, d=d, f16=f16).astype(np.float64)
            xr = np.sqrt((xa.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
            typ = xr * np.sqrt((deq ** 2).mean(axis=0, keepdims=True)) * np.sqrt(k) + 1e-30 + (np.abs(d) if resid else 0.0)
            err = np.abs(got - want)
            where = f"seed {seed} shape {done}: fmt {fmt} m {m} k {k} n {n} f16 {f16} resid {resid} scale {scale} wscale {wscale} woff {woff}"
            assert np.isfinite(got).all(), where
            assert (err <= REL * np.abs(want) + ABS * typ).all(), where + f" worst {(err / typ).max():.2e} of typical"
            done += 1
    finally:
        ctx.set_shared_device(False)


def test_shares_are_planned_only_when_every_xcd_holds_its_workgroups():
    """Every part adds up a share only if all workgroups are resident at once, and that is decided
    per XCD: 17 column groups of 14 parts are 238 workgroups on 256 CUs, but XCD 0 would get three
    groups = 42 workgroups on its 32 CUs.  Such a launch keeps the single reader (its workspace
    holds 13 parts' tiles, not 14); 16 groups of 14 parts fit and take the shares."""
    slot = 8 * 2 * 1024  # a workgroup's tiles: 8 waves x one pair of 16-column tiles x 1 KiB
    p = capi.matmul_plan(Q4, 16, 14336, 17 * 256)
    assert (p.route, p.k_parts, p.grid[1], p.grid[2]) == (capi.ROUTE_TILE_MFMA, 14, 17, 1)
    assert p.workspace_bytes == 13 * 17 * slot
    p = capi.matmul_plan(Q4, 16, 14336, 16 * 256)
    assert (p.k_parts, p.grid[1]) == (14, 16) and p.workspace_bytes == 14 * 16 * slot


@pytest.mark.parametrize("fmt,m,k,n", [(Q4, 16, 14336, 1024), (Q8, 9, 8192, 512), (Q4, 16, 2048, 4096), (Q4, 16, 14336, 17 * 256)])
def test_k_parts_added_up_by_shares_or_by_the_last_part_agree(ctx, orc, fmt, m, k, n):
    """Shapes whose K parts are added up by all parts, a share each (the whole grid resident at
    once), against the same call on a context that shares its device, where the part dispatched
    last adds the others up: both within the bar, each repeatable bit for bit, and the two orders
    of summation within a few ulps of each other."""
    w = synth.normal(1501 + k, k * n, 0.02).reshape(k, n)
    x = synth.normal(1502 + m, m * k, 1.0).reshape(m, k)
    wt = ctx.weight(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, orc.quantize(fmt, w), k, n))
    assert capi.matmul_plan(fmt, m, k, n).k_parts > 1
    shares = [run_matmul(ctx, fmt, x, wt, ROUTES["auto"]) for _ in range(3)]
    ctx.set_shared_device(True)
    try:
        last = [run_matmul(ctx, fmt, x, wt, ROUTES["auto"]) for _ in range(3)]
    finally:
        ctx.set_shared_device(False)
    for got in (shares, last):
        assert (bits(got[0]) == bits(got[1])).all() and (bits(got[0]) == bits(got[2])).all()
        orc.assert_close(got[0], want, REL, ABS)
    np.testing.assert_allclose(shares[0], last[0], rtol=2e-5, atol=2e-5)
    wt.free()


@pytest.mark.parametrize("fmt,m,k,n", [(Q4, 16, 4096, 2048), (Q8, 9, 4096, 1024), (Q4, 4, 14336, 518), (Q8, 3, 12288, 64)])
def test_a_reader_that_gives_up_is_reported_and_the_context_recovers(ctx, orc, fmt, m, k, n):
    """K cut into parts for different workgroups: the part that adds the others up polls the
    hand-over workspace for their sums, and its wait is bounded.  With a limit of zero polls it
    looks at nothing and gives up at once: every kernel still ends, the next synchronising call
    returns MGN_ETIMEOUT, the library empties the workspace again, and the same matmul with the
    default limit comes out right."""
    plan = capi.matmul_plan(fmt, m, k, n)
    assert plan.k_parts > 1 and plan.route in (capi.ROUTE_GEMV_MFMA, capi.ROUTE_TILE_MFMA)
    w = synth.normal(1501, k * n, 0.02).reshape(k, n)
    x = synth.normal(1502, m * k, 1.0).reshape(m, k)
    wt, a, c = ctx.weight(fmt, w), ctx.upload(x), ctx.buffer(m * n * 4)
    want = orc.matmul_packed(fmt, x, orc.quantize(fmt, w), n)
    try:
        ctx.set_spin_limit(0)
        ctx.matmul_q(a, wt, c, m)
        ctx.matmul_q(a, wt, c, m)
        with pytest.raises(capi.MgnError) as e:
            ctx.sync()
        assert e.value.status == capi.ETIMEOUT
        ctx.sync()  # reported once
    finally:
        ctx.set_spin_limit(1 << 20)
    for _ in range(3):
        ctx.matmul_q(a, wt, c, m)
        orc.assert_close(c.download(np.float32, m * n).reshape(m, n), want, REL, ABS)
    for h in (wt, a, c):
        h.free()


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("m", [5, 16, 40])
def test_activations_of_any_magnitude_on_the_rescaling_tiled_kernel(ctx, orc, fmt, m):
    """f32 activations are scaled per (row, 256-element slice) by a power of two before they are
    split into fp16 pairs: rows of magnitude 1e-20, 1e-4, 1 and 1e6 side by side, an outlier of
    2e5 in an ordinary row and a value near the largest float all come out within the bar of the
    f64 product (absolute part scaled by the row's magnitude).  The reference computes in f32."""
    k, n = 1280, 208
    w = synth.normal(995, k * n, 0.02).reshape(k, n)
    x = synth.normal(996 + m, m * k, 1.0).reshape(m, k)
    mags = np.array([1e-20, 1e-4, 1.0, 1e6, 3e-3, 1e12, 1e-9], np.float32)
    for r in range(m):
        x[r] *= mags[r % len(mags)]
    x[2, 17] = np.float32(2.0e5)      # outlier in a row of order one
    x[m - 1, 300] = np.float32(1e30)  # dominates its row and its slice
    packed = orc.quantize(fmt, w)
    want = orc.matmul_f64(x, orc.dequantize(fmt, packed, k, n))
    wt = ctx.weight(fmt, w)
    for route in ("tile_mfma", "generic"):
        assert_close_rowwise(run_matmul(ctx, fmt, x, wt, ROUTES[route]), want, x)
    # the 32x32x16 kernel splits activations into fp16 pairs without rescaling: it flags such data
    # and the next synchronising call fails loudly instead of handing back wrong numbers
    with pytest.raises(capi.MgnError) as e:
        run_matmul(ctx, fmt, x, wt, ROUTES["gemm_mfma"])
    assert e.value.status == capi.ERANGE
    ctx.sync()  # reported once; the context keeps working
    # the automatic route assumes nothing about f32 activations and keeps them off that kernel ...
    assert_close_rowwise(run_matmul(ctx, fmt, x, wt, capi.ROUTE_AUTO), want, x)
    # ... unless the context was promised that they lie in the fp16 range: then the promise is checked
    # wherever it is relied on (a shape the rescaling kernel takes anyway just comes out right)
    ctx.set_activation_range(True)
    try:
        if capi.matmul_plan(fmt, m, k, n, fp16_range=True).route == capi.ROUTE_GEMM_MFMA:
            with pytest.raises(capi.MgnError) as e:
                run_matmul(ctx, fmt, x, wt, capi.ROUTE_AUTO)
            assert e.value.status == capi.ERANGE
            ctx.sync()
        else:
            assert_close_rowwise(run_matmul(ctx, fmt, x, wt, capi.ROUTE_AUTO), want, x)
        tame = synth.normal(997 + m, m * k, 1.0).reshape(m, k)
        oracle_tame = orc.matmul_f64(tame, orc.dequantize(fmt, packed, k, n))
        assert_close_rowwise(run_matmul(ctx, fmt, tame, wt, capi.ROUTE_AUTO), oracle_tame, tame)
    finally:
        ctx.set_activation_range(False)
    # non-finite activations give non-finite outputs in their own rows only
    x[1, 5] = np.float32(np.inf)
    x[3, 700] = np.float32(np.nan)
    got = run_matmul(ctx, fmt, x, wt, ROUTES["tile_mfma"])
    assert not np.isfinite(got[1]).any() and not np.isfinite(got[3]).any()
    rest = [r for r in range(m) if r not in (1, 3)]
    assert_close_rowwise(got[rest], want[rest], x[rest])
    wt.free()
