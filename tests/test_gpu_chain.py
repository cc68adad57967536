"""mgn_chain_*: a chain of dependent one-row matmuls in one launch, against numpy pointwise
operations + the oracle's matmul on the oracle's dequantized weights, through the C ABI."""
import numpy as np
import pytest

from helpers import Q4, Q8
from meganeura_amd import capi, synth

pytestmark = pytest.mark.gpu

REL, ABS = 1e-3, 1e-4


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def deq(orc, w):
    k, n = w.shape
    return orc.dequantize(Q4, orc.quantize(Q4, w), k, n)


def rms_norm(x, g, eps):
    # src/shaders/rms_norm.wgsl:1-57
    x64 = x.astype(np.float64)
    return (x64 / np.sqrt((x64 ** 2).mean() + eps) * g).astype(np.float32)


def test_a_context_on_a_shared_device_refuses_chains(ctx, orc):
    """mgn_ctx_set_shared_device: a chain's workgroups all wait for each other, which needs the
    device to themselves; on a shared device the chain is refused and the caller launches the
    stages one by one."""
    k, n = 576, 576
    wt = ctx.weight(Q4, synth.normal(3001, k * n, 0.02).reshape(k, n))
    a, c = ctx.upload(synth.normal(3002, k, 1.0)), ctx.buffer(n * 4)
    ctx.set_shared_device(True)
    try:
        with pytest.raises(capi.MgnError) as e:
            ctx.chain([dict(w=wt, a=a, c=c)])
        assert e.value.status == capi.EUNSUPPORTED
    finally:
        ctx.set_shared_device(False)
    ch = ctx.chain([dict(w=wt, a=a, c=c)])
    ch.run()
    ctx.sync()
    ch.free()
    for h in (a, c, wt):
        h.free()


def swiglu(gate_up, k):
    # src/shaders/swiglu_concat.wgsl:20-32
    g, u = gate_up[:, :k].astype(np.float64), gate_up[:, k:].astype(np.float64)
    return (g / (1.0 + np.exp(-g)) * u).astype(np.float32)


@pytest.mark.parametrize("hidden,inter", [(576, 1536), (1024, 3072), (2048, 5632)])
def test_ffn_chain_matches_the_oracle(ctx, orc, hidden, inter):
    """rms_norm -> gate | up, then SwiGLU -> down + residual: two stages, one launch, the second
    stage's activations made by the first.  Five launches in a row: consecutive launches
    alternate between the chain's two sets of hand-over slots."""
    x = synth.activations(3, 1, hidden)
    wgu, wd = synth.weights(5, hidden, 2 * inter), synth.weights(6, inter, hidden)
    g = (1.0 + synth.normal(7, hidden, 0.1)).astype(np.float32)
    Wgu, Wd, bx, bg = ctx.weight(Q4, wgu), ctx.weight(Q4, wd), ctx.upload(x), ctx.upload(g)
    bgu, by = ctx.buffer(2 * inter * 4), ctx.buffer(hidden * 4)
    ch = ctx.chain([dict(w=Wgu, a=bx, c=bgu, prologue=capi.PROLOGUE_RMS_NORM, norm_weight=bg, eps=1e-5),
                    dict(w=Wd, a=bgu, c=by, prologue=capi.PROLOGUE_SWIGLU, d=bx)])
    want_gu = orc.matmul_f32(rms_norm(x, g, 1e-5), deq(orc, wgu))
    want_y = orc.matmul_f32(swiglu(want_gu, inter), deq(orc, wd), x)
    for _ in range(5):
        ch.run()
        orc.assert_close(by.download(np.float32, hidden).reshape(1, -1), want_y, REL, ABS)
        orc.assert_close(bgu.download(np.float32, 2 * inter).reshape(1, -1), want_gu, REL, ABS)
    ch.free()
    for h in (Wgu, Wd, bx, bg, bgu, by):
        h.free()


def test_decode_layers_chain_matches_the_oracle(ctx, orc):
    """Three SmolLM2-shaped decode layers (models/smollm2.rs:392-405 without the attention core) as
    ONE launch of 18 stages: q, k, v and the o-projection of a layer are independent and share the
    workgroups; gate | up waits for o, down for gate | up, the next layer for down.  A unary
    operation rides on one of the stages."""
    hidden, kv, inter, layers = 576, 192, 1536, 3
    x_ref = synth.activations(2, 1, hidden, which=0)
    attn = synth.activations(2, 1, hidden, which=1)
    g1 = (1.0 + synth.normal(11, hidden, 0.1)).astype(np.float32)
    bx, battn, bg = ctx.upload(x_ref), ctx.upload(attn), ctx.upload(g1)
    stages, keep, checks = [], [bx, battn, bg], []
    bxl = bx
    for l in range(layers):
        shapes = [("q", hidden, hidden), ("k", hidden, kv), ("v", hidden, kv), ("o", hidden, hidden),
                  ("gu", hidden, 2 * inter), ("d", inter, hidden)]
        ws = {nm: synth.weights(2, kk, nn, which=(l * 7 + j) % 7) for j, (nm, kk, nn) in enumerate(shapes)}
        W = {nm: ctx.weight(Q4, w) for nm, w in ws.items()}
        out = {nm: ctx.buffer(nn * 4) for nm, _, nn in shapes}
        for nm in ("q", "k", "v"):
            stages.append(dict(w=W[nm], a=bxl, c=out[nm], prologue=capi.PROLOGUE_RMS_NORM, norm_weight=bg, eps=1e-5,
                               ops=[capi.UNARY_RELU] if nm == "k" else []))
        stages.append(dict(w=W["o"], a=battn, c=out["o"], d=bxl))
        stages.append(dict(w=W["gu"], a=out["o"], c=out["gu"], prologue=capi.PROLOGUE_RMS_NORM, norm_weight=bg, eps=1e-5))
        stages.append(dict(w=W["d"], a=out["gu"], c=out["d"], prologue=capi.PROLOGUE_SWIGLU, d=out["o"]))
        n1 = rms_norm(x_ref, g1, 1e-5)
        q_ref = orc.matmul_f32(n1, deq(orc, ws["q"]))
        k_ref = np.maximum(orc.matmul_f32(n1, deq(orc, ws["k"])), 0.0)
        h_ref = orc.matmul_f32(attn, deq(orc, ws["o"]), x_ref)
        gu_ref = orc.matmul_f32(rms_norm(h_ref, g1, 1e-5), deq(orc, ws["gu"]))
        x_ref = orc.matmul_f32(swiglu(gu_ref, inter), deq(orc, ws["d"]), h_ref)
        checks += [(out["q"], q_ref), (out["k"], k_ref), (out["o"], h_ref), (out["d"], x_ref)]
        keep += list(W.values()) + list(out.values())
        bxl = out["d"]
    ch = ctx.chain(stages)
    for _ in range(4):
        ch.run()
        for buf, want in checks:
            orc.assert_close(buf.download(np.float32, want.size).reshape(1, -1), want, REL, ABS)
    ch.free()
    for h in keep:
        h.free()


def test_what_a_chain_does_not_serve_is_refused(ctx):
    k, n = 576, 192
    w4 = ctx.weight(Q4, synth.weights(2, k, n))
    w8 = ctx.weight(Q8, synth.weights(2, k, n))
    wsq = ctx.weight(Q4, synth.weights(2, k, k))
    a, b, c = ctx.buffer(k * 4), ctx.buffer(k * 4), ctx.buffer(n * 4)
    for stages, m in (([dict(w=w8, a=a, c=c)], 1),                                   # Q8
                      ([dict(w=w4, a=a, c=c)], 2),                                   # two rows
                      ([dict(w=w4, a=a, c=c), dict(w=w4, a=b, c=c)], 1),             # two stages write one buffer
                      ([dict(w=w4, a=a, c=c), dict(w=wsq, a=b, c=a)], 1)):           # a stage overwrites another's input
        with pytest.raises(capi.MgnError) as e:
            ctx.chain(stages, m)
        assert e.value.status == capi.EUNSUPPORTED
    with pytest.raises(capi.MgnError) as e:
        ctx.chain([dict(w=w4, a=c, c=a)])   # the activations are shorter than K
    assert e.value.status == capi.EINVAL
    for h in (w4, w8, wsq, a, b, c):
        h.free()


def test_a_chain_reader_that_gives_up_is_reported_and_the_chain_recovers(ctx, orc):
    """The wait for another workgroup's outputs is bounded.  With a limit of zero polls a reader
    looks at nothing and gives up at once: the launch still ends, the next synchronising call
    returns MGN_ETIMEOUT and empties the chain's slots again, and the next launches are right."""
    hidden, inter = 576, 1536
    x = synth.activations(3, 1, hidden)
    wgu, wd = synth.weights(5, hidden, 2 * inter), synth.weights(6, inter, hidden)
    Wgu, Wd, bx = ctx.weight(Q4, wgu), ctx.weight(Q4, wd), ctx.upload(x)
    bgu, by = ctx.buffer(2 * inter * 4), ctx.buffer(hidden * 4)
    ch = ctx.chain([dict(w=Wgu, a=bx, c=bgu), dict(w=Wd, a=bgu, c=by, prologue=capi.PROLOGUE_SWIGLU, d=bx)])
    want = orc.matmul_f32(swiglu(orc.matmul_f32(x, deq(orc, wgu)), inter), deq(orc, wd), x)
    ch.run()
    orc.assert_close(by.download(np.float32, hidden).reshape(1, -1), want, REL, ABS)
    ctx.set_spin_limit(0)
    try:
        ch.run()
        ch.run()
        with pytest.raises(capi.MgnError) as e:
            ctx.sync()
        assert e.value.status == capi.ETIMEOUT
    finally:
        ctx.set_spin_limit(1 << 20)
    for _ in range(3):
        ch.run()
        orc.assert_close(by.download(np.float32, hidden).reshape(1, -1), want, REL, ABS)
    ch.free()
    for h in (Wgu, Wd, bx, bgu, by):
        h.free()
