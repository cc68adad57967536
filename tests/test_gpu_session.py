"""The Graph / Session surface end to end on the GPU, written after the
reference's own tests (tests/gpu_smoke.rs, tests/gemv_parity.rs)."""
import numpy as np
import pytest

from helpers import Q4, Q8, gemv_parity_inputs, golden_ratio_weights, ref_test_inputs_q4_matmul
from meganeura_amd import capi, synth
from meganeura_amd.graph import Graph, ShaderEntry, build_inference_session

pytestmark = pytest.mark.gpu


def test_q4_matmul_correctness(orc):
    # tests/gpu_smoke.rs:2681-2771
    m, k, n = 6, 1024, 2048
    g = Graph()
    a = g.input("a", [m, k])
    b = g.parameter_q4("b", [k, n])
    g.set_outputs([g.matmul(a, b)])
    sess = build_inference_session(g)
    a_data, b_data = ref_test_inputs_q4_matmul()
    sess.set_input("a", a_data)
    sess.set_parameter("b", b_data)
    sess.step()
    sess.wait()
    out = sess.read_output(m * n)
    b_deq = orc.dequantize(Q4, orc.quantize(Q4, b_data), k, n)
    cpu = orc.matmul_f32(a_data, b_deq).reshape(-1)
    assert not np.isnan(out).any()
    assert np.abs(cpu - out).max() < 0.1
    orc.assert_close(out, cpu, 1e-3, 1e-4)
    sess.close()


@pytest.mark.parametrize("quant", ["q4", "q8"])
@pytest.mark.parametrize("k,n,seed", [(64, 64, 1), (576, 576, 2), (576, 1536, 3), (1536, 576, 4), (576, 49152, 5), (64, 66, 6)])
def test_gemv_shapes(orc, quant, k, n, seed):
    # tests/gemv_parity.rs:74-130 shapes, with the weight quantized
    fmt = Q4 if quant == "q4" else Q8
    a, b = gemv_parity_inputs(k, n, seed)
    g = Graph()
    an = g.input("a", [1, k])
    bn = (g.parameter_q4 if quant == "q4" else g.parameter_q8)("b", [k, n])
    g.set_outputs([g.matmul(an, bn)])
    sess = build_inference_session(g)
    gemv = [d for d in sess.plan() if d.shader == ShaderEntry.MatMulGemv]
    assert len(gemv) == (1 if n % 4 == 0 else 0)
    sess.set_input("a", a)
    sess.set_parameter("b", b)
    sess.step()
    sess.wait()
    gpu = sess.read_output(n)
    cpu = orc.matmul_f32(a, orc.dequantize(fmt, orc.quantize(fmt, b), k, n)).reshape(-1)
    orc.assert_close(gpu, cpu, 1e-3, 1e-4)
    sess.close()


@pytest.mark.parametrize("k,n,seed", [(1536, 576, 100), (576, 576, 101), (2048, 720, 102)])
def test_gemv_add_shapes(orc, k, n, seed):
    # tests/gemv_parity.rs:133-196: MatMul + Add fuses and takes the GemvAdd entry at M = 1
    a, b = gemv_parity_inputs(k, n, seed)
    d = np.sin(np.arange(n, dtype=np.float32) * np.float32(0.01)).reshape(1, n)
    g = Graph()
    an = g.input("a", [1, k])
    bn = g.parameter_q4("b", [k, n])
    dn = g.parameter("d", [1, n])
    g.set_outputs([g.add(g.matmul(an, bn), dn)])
    sess = build_inference_session(g)
    assert [x.shader for x in sess.plan()] == [ShaderEntry.MatMulGemvAdd]
    sess.set_input("a", a)
    sess.set_parameter("b", b)
    sess.set_parameter("d", d)
    sess.step()
    sess.wait()
    gpu = sess.read_output(n)
    cpu = orc.matmul_f32(a, orc.dequantize(Q4, orc.quantize(Q4, b), k, n), d).reshape(-1)
    orc.assert_close(gpu, cpu, 1e-3, 1e-4)
    sess.close()


def _silu_mul(gate, up):
    gate = gate.astype(np.float32)
    sig = np.float32(1) / (np.float32(1) + np.exp(-gate, dtype=np.float32))
    return gate * sig * up


@pytest.mark.parametrize("seq,hidden,ffn", [(1, 576, 1536), (6, 1024, 3072)])
def test_q4_mlp_block_with_fused_gate_up(orc, seq, hidden, ffn):
    # the MLP half of tests/gpu_smoke.rs:2824-2835 (q4_layer_nan_hunt), with values checked:
    # x + down(swiglu(gate(h), up(h))), gate/up fused into one wide matmul on a derived weight
    g = Graph()
    x = g.input("x", [seq, hidden])
    ln = g.parameter("ln2", [hidden])
    h = g.rms_norm(x, ln, 1e-6)
    gate = g.matmul(h, g.parameter_q4("wg", [hidden, ffn]))
    up = g.matmul(h, g.parameter_q4("wu", [hidden, ffn]))
    act = g.swiglu(gate, up)
    out = g.add(x, g.matmul(act, g.parameter_q4("wd", [ffn, hidden])))
    g.set_outputs([out])
    sess = build_inference_session(g)
    shaders = [d.shader for d in sess.plan()]
    mm = ShaderEntry.MatMulGemv if seq == 1 else ShaderEntry.MatMul
    mma = ShaderEntry.MatMulGemvAdd if seq == 1 else ShaderEntry.FusedMatMulAdd
    assert shaders == [ShaderEntry.RmsNorm, mm, ShaderEntry.SwiGLUConcat, mma]

    xv = synth.normal(77, seq * hidden).reshape(seq, hidden)
    wg = golden_ratio_weights(hidden * ffn).reshape(hidden, ffn) * np.float32(0.1)
    wu = synth.normal(78, hidden * ffn, 0.02).reshape(hidden, ffn)
    wd = synth.normal(79, ffn * hidden, 0.02).reshape(ffn, hidden)
    sess.set_input("x", xv)
    sess.set_parameter("ln2", np.ones(hidden, np.float32))
    sess.set_parameter("wg", wg)
    sess.set_parameter("wu", wu)
    sess.set_parameter("wd", wd)
    with pytest.raises(KeyError, match="unknown parameter"):
        sess.set_parameter("nope", wd)
    sess.step()
    sess.wait()
    got = sess.read_output(seq * hidden).reshape(seq, hidden)

    deq = lambda w: orc.dequantize(Q4, orc.quantize(Q4, w), *w.shape)
    hn = xv * (np.float32(1) / np.sqrt((xv.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-6)).astype(np.float32)
    gate_o = orc.matmul_f64(hn, deq(wg))
    up_o = orc.matmul_f64(hn, deq(wu))
    want = orc.matmul_f64(_silu_mul(gate_o, up_o), deq(wd), xv)
    assert np.isfinite(got).all()
    # three chained ops: compare with a bar scaled to the block's output, not the single-matmul bar
    orc.assert_close(got, want, 2e-3, 2e-4)

    # setting one source again re-quantizes the derived weight (src/runtime.rs:2347-2406)
    sess.set_parameter("wu", np.zeros_like(wu))
    sess.step()
    sess.wait()
    got0 = sess.read_output(seq * hidden).reshape(seq, hidden)
    orc.assert_close(got0, xv, 1e-5, 1e-5)
    sess.close()


def test_q8_session_and_stepping_twice(orc):
    m, k, n = 1, 576, 1536
    g = Graph()
    a = g.input("a", [m, k])
    b = g.parameter_q8("b", [k, n])
    g.set_outputs([g.matmul(a, b)])
    sess = build_inference_session(g)
    w = synth.weights(1, k, n)
    deq = orc.dequantize(Q8, orc.quantize(Q8, w), k, n)
    sess.set_parameter("b", w)
    for which in (0, 1):
        x = synth.activations(1, m, k, which=which)
        sess.set_input("a", x)
        sess.step()
        sess.wait()
        orc.assert_close(sess.read_output(n), orc.matmul_f32(x, deq), 1e-3, 1e-4)
    sess.close()


def test_f32_weight_matmul_is_refused():
    g = Graph()
    a = g.input("a", [1, 64])
    b = g.parameter("b", [64, 64])
    g.set_outputs([g.matmul(a, b)])
    with pytest.raises(capi.MgnError, match="quantized path"):
        build_inference_session(g)


def _decode_layer_graph(hidden, inter, fmt_param):
    """SmolLM2-style decode layer without the attention core (models/smollm2.rs:340-414):
    norm -> q/k/v projections; o-projection + residual; norm -> gate, up -> swiglu -> down + residual."""
    g = Graph()
    x = g.input("x", [1, hidden])
    attn = g.input("attn", [1, hidden])
    n1 = g.rms_norm(x, g.parameter("norm1", [hidden]), 1e-5)
    q = g.matmul(n1, fmt_param(g, "wq", [hidden, hidden]))
    kk = g.matmul(n1, fmt_param(g, "wk", [hidden, hidden // 3]))
    v = g.matmul(n1, fmt_param(g, "wv", [hidden, hidden // 3]))
    h = g.add(g.matmul(attn, fmt_param(g, "wo", [hidden, hidden])), x)
    n2 = g.rms_norm(h, g.parameter("norm2", [hidden]), 1e-5)
    gate = g.matmul(n2, fmt_param(g, "wg", [hidden, inter]))
    up = g.matmul(n2, fmt_param(g, "wu", [hidden, inter]))
    out = g.add(g.matmul(g.swiglu(gate, up), fmt_param(g, "wd", [inter, hidden])), h)
    g.set_outputs([out, q, kk, v])
    return g


def test_graph_replay_matches_individual_launches(orc):
    """A step replayed as one captured HIP graph gives the same bits as the same step
    launched dispatch by dispatch: replayed several times, with fresh inputs, eager work and
    synchronisation in between."""
    hidden, inter = 576, 1536
    g = _decode_layer_graph(hidden, inter, lambda gr, name, shape: gr.parameter_q4(name, shape))
    sess = build_inference_session(g)
    shapes = {"wq": (hidden, hidden), "wk": (hidden, hidden // 3), "wv": (hidden, hidden // 3), "wo": (hidden, hidden),
              "wg": (hidden, inter), "wu": (hidden, inter), "wd": (inter, hidden)}
    for i, (name, (k, n)) in enumerate(shapes.items()):
        sess.set_parameter(name, synth.normal(300 + i, k * n, 0.02))
    sess.set_parameter("norm1", 1.0 + 0.1 * synth.normal(310, hidden, 1.0))
    sess.set_parameter("norm2", 1.0 + 0.1 * synth.normal(311, hidden, 1.0))
    sizes = [hidden, hidden, hidden // 3, hidden // 3]

    def run(seed):
        sess.set_input("x", synth.normal(seed, hidden, 1.0))
        sess.set_input("attn", synth.normal(seed + 1000, hidden, 1.0))
        sess.step()
        sess.wait()
        return [sess.read_output_by_index(i, n) for i, n in enumerate(sizes)]

    sess.set_graph_replay(False)
    sess.set_chains(False)      # launch by launch: what the graph records (a chain launch is never recorded)
    want = {seed: run(seed) for seed in (1, 2, 3)}
    assert not sess.graph_active()
    sess.set_graph_replay(True)
    run(2)                      # every kernel has run before: captured right away
    assert sess.graph_active()
    scratch = capi.Context(0)   # unrelated eager work on the same device between replays
    for it in range(9):
        seed = 1 + it % 3
        got = run(seed)
        for a, b in zip(got, want[seed]):
            assert (a.view(np.uint32) == b.view(np.uint32)).all(), f"replay {it} differs from the eager step"
        buf = scratch.upload(synth.normal(50 + it, 4096, 1.0))
        scratch.sync()
        buf.free()
    scratch.close()
    # a new weight invalidates the captured step; the next steps run eagerly, then re-capture
    sess.set_parameter("wq", synth.normal(400, hidden * hidden, 0.02))
    assert not sess.graph_active()
    sess.set_graph_replay(True)
    first = run(1)              # launch by launch
    assert not sess.graph_active()
    second = run(1)             # captured here
    assert sess.graph_active()
    third = run(1)
    for a, b, c in zip(first, second, third):
        assert (a.view(np.uint32) == b.view(np.uint32)).all() and (a.view(np.uint32) == c.view(np.uint32)).all()
    assert (first[0].view(np.uint32) != want[1][1].view(np.uint32)).any()  # q really uses the new weight
    sess.close()


def test_decode_layer_fuses_norm_and_swiglu_into_the_matmuls(orc):
    """9 dispatches in the plan, 4 kernel launches per step: both norms and the SwiGLU ride on
    the matmuls that read them, and q, k, v share one launch; with chains (the default) those
    four go out as ONE launch.  Same numbers as the unfused step within the matmul bar."""
    hidden, inter = 576, 1536
    g = _decode_layer_graph(hidden, inter, lambda gr, name, shape: gr.parameter_q4(name, shape))
    sess = build_inference_session(g)
    shapes = {"wq": (hidden, hidden), "wk": (hidden, hidden // 3), "wv": (hidden, hidden // 3), "wo": (hidden, hidden),
              "wg": (hidden, inter), "wu": (hidden, inter), "wd": (inter, hidden)}
    for i, (name, (k, n)) in enumerate(shapes.items()):
        sess.set_parameter(name, synth.normal(600 + i, k * n, 0.02))
    sess.set_parameter("norm1", 1.0 + 0.1 * synth.normal(610, hidden, 1.0))
    sess.set_parameter("norm2", 1.0 + 0.1 * synth.normal(611, hidden, 1.0))
    sess.set_input("x", synth.normal(612, hidden, 1.0))
    sess.set_input("attn", synth.normal(613, hidden, 1.0))
    sizes = [hidden, hidden, hidden // 3, hidden // 3]
    plan = [d.shader for d in sess.plan()]
    assert len(plan) == 9 and plan.count(ShaderEntry.RmsNorm) == 2 and plan.count(ShaderEntry.SwiGLUConcat) == 1
    assert sess.num_launches() == 1
    chained = []
    for _ in range(3):  # consecutive steps alternate between the chain's two sets of hand-over slots
        sess.step()
        sess.wait()
        chained.append([sess.read_output_by_index(i, n) for i, n in enumerate(sizes)])
    sess.set_chains(False)
    assert sess.num_launches() == 4
    sess.step()
    sess.wait()
    fused = [sess.read_output_by_index(i, n) for i, n in enumerate(sizes)]
    for step in chained:
        for a, b in zip(step, fused):
            assert np.isfinite(a).all()
            orc.assert_close(a, b, 1e-3, 1e-4)
    sess.set_graph_replay(True)   # a replayed graph would run a chain on one set of slots every time
    sess.set_chains(True)
    assert sess.num_launches() == 4
    sess.set_graph_replay(False)
    assert sess.num_launches() == 1
    sess.set_fusion(False)
    assert sess.num_launches() == 9
    sess.step()
    sess.wait()
    plain = [sess.read_output_by_index(i, n) for i, n in enumerate(sizes)]
    for a, b in zip(fused, plain):
        assert np.isfinite(a).all()
        orc.assert_close(a, b, 1e-3, 1e-4)
    sess.close()


@pytest.mark.parametrize("quant", ["q4", "q8"])
@pytest.mark.parametrize("m,k,n", [(6, 1024, 300), (1, 576, 192), (1, 576, 49152), (2, 1536, 64)])
def test_unary_ops_behind_a_quantized_matmul(orc, quant, m, k, n):
    """relu(x W + r) then -silu(.): for M > 1 the compiler folds both into the matmul dispatch
    (compile.rs:915-1035); for M = 1 they stay dispatches of their own in the plan and the
    matmul's launch applies them.  One launch either way, same numbers as launched one by one."""
    fmt = Q4 if quant == "q4" else Q8
    g = Graph()
    x = g.input("x", [m, k])
    r = g.input("r", [m, n])
    w = (g.parameter_q4 if fmt == Q4 else g.parameter_q8)("w", [k, n])
    h = g.neg(g.silu(g.relu(g.add(g.matmul(x, w), r))))
    g.set_outputs([h])
    sess = build_inference_session(g)
    xv = synth.normal(700 + m + k, m * k).reshape(m, k)
    rv = synth.normal(701 + n, m * n).reshape(m, n)
    wv = synth.normal(702 + k + n, k * n, 0.02).reshape(k, n)
    sess.set_input("x", xv)
    sess.set_input("r", rv)
    sess.set_parameter("w", wv)
    plan = sess.plan()
    if m == 1 and n % 4 == 0:
        assert [d.shader for d in plan] == [ShaderEntry.MatMulGemvAdd, ShaderEntry.Relu, ShaderEntry.Silu, ShaderEntry.Neg]
    else:
        assert [d.shader for d in plan] == [ShaderEntry.FusedMatMulAdd] and len(plan[0].epilogue) == 3
    assert sess.num_launches() == 1
    sess.step()
    sess.wait()
    got = sess.read_output(m * n)
    want = orc.matmul_f32(xv, orc.dequantize(fmt, orc.quantize(fmt, wv), k, n), rv)
    for op in ("relu", "silu", "neg"):
        want = orc.unary(op, want)
    orc.assert_close(got, want.reshape(-1), 1e-3, 1e-4)
    sess.set_fusion(False)
    assert sess.num_launches() == len(plan)
    sess.step()
    sess.wait()
    orc.assert_close(sess.read_output(m * n), want.reshape(-1), 1e-3, 1e-4)
    sess.close()


def test_norm_with_another_reader_is_not_folded():
    # the normed activations are also an output: the RmsNorm dispatch must run on its own
    hidden = 576
    g = Graph()
    x = g.input("x", [1, hidden])
    n1 = g.rms_norm(x, g.parameter("norm", [hidden]), 1e-5)
    q = g.matmul(n1, g.parameter_q4("wq", [hidden, hidden]))
    g.set_outputs([q, n1])
    sess = build_inference_session(g)
    sess.set_parameter("wq", synth.normal(620, hidden * hidden, 0.02))
    sess.set_parameter("norm", np.ones(hidden, np.float32))
    assert sess.num_launches() == 2
    xv = synth.normal(621, hidden, 2.0)
    sess.set_input("x", xv)
    sess.step()
    sess.wait()
    got = sess.read_output_by_index(1, hidden)
    want = xv / np.sqrt((xv.astype(np.float64) ** 2).mean() + 1e-5)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    sess.close()


@pytest.mark.parametrize("quant", ["q4", "q8"])
@pytest.mark.parametrize("m,k,n", [(1, 576, 49152), (1, 64, 66), (6, 128, 200)])
def test_matmul_bt_with_quantized_table(orc, quant, m, k, n):
    """Weight-tied lm_head: logits = x @ embed^T with embed[vocab, hidden] quantized
    (models/smollm2.rs:413-414).  The table is blocked along hidden (K), so the result is the
    plain quantized matmul against embed^T."""
    fmt = Q4 if quant == "q4" else Q8
    g = Graph()
    x = g.input("x", [m, k])
    e = (g.parameter_q4 if quant == "q4" else g.parameter_q8)("embed", [n, k])
    g.set_outputs([g.matmul_bt(x, e)])
    sess = build_inference_session(g)
    (d,) = sess.plan()
    assert d.shader == (ShaderEntry.MatMulGemvBT if m == 1 else ShaderEntry.MatMulBT)
    embed = synth.normal(900 + n, n * k, 0.02).reshape(n, k)
    xv = synth.normal(901 + k, m * k, 1.0).reshape(m, k)
    sess.set_parameter("embed", embed)
    sess.set_input("x", xv)
    sess.step()
    sess.wait()
    got = sess.read_output(m * n).reshape(m, n)
    want = orc.matmul_packed(fmt, xv, orc.quantize(fmt, np.ascontiguousarray(embed.T)), n)
    orc.assert_close(got, want, 1e-3, 1e-4)
    sess.close()


@pytest.mark.parametrize("quant", ["q4", "q8"])
@pytest.mark.parametrize("m,k,n", [(1, 64, 66), (6, 128, 200), (40, 576, 96)])
def test_matmul_at_and_fused_add_forms(orc, quant, m, k, n):
    """matmul_at (a stored [K, M]) alone, with a residual and a relu folded in, and matmul_bt
    with a residual: each is one dispatch of the plan, as in the reference
    (src/optimize.rs:724-767, src/compile.rs:1423-1445, 1526-1574), and equals the plain
    quantized matmul on the transposed operand."""
    fmt = Q4 if quant == "q4" else Q8
    param = "parameter_q4" if quant == "q4" else "parameter_q8"
    g = Graph()
    xt = g.input("xt", [k, m])
    x = g.input("x", [m, k])
    r = g.input("r", [m, n])
    w = getattr(g, param)("w", [k, n])
    e = getattr(g, param)("e", [n, k])
    g.set_outputs([g.matmul_at(xt, w), g.relu(g.add(g.matmul_at(xt, w), r)), g.add(r, g.matmul_bt(x, e))])
    sess = build_inference_session(g)
    assert [d.shader for d in sess.plan()] == [ShaderEntry.MatMulAT, ShaderEntry.FusedMatMulATAdd, ShaderEntry.FusedMatMulBTAdd]
    wv = synth.normal(910 + n, k * n, 0.02).reshape(k, n)
    ev = synth.normal(911 + n, n * k, 0.02).reshape(n, k)
    xv = synth.normal(912 + k, m * k, 1.0).reshape(m, k)
    rv = synth.normal(913 + k, m * n, 1.0).reshape(m, n)
    sess.set_parameter("w", wv)
    sess.set_parameter("e", ev)
    sess.set_input("xt", np.ascontiguousarray(xv.T))
    sess.set_input("x", xv)
    sess.set_input("r", rv)
    plain = orc.matmul_packed(fmt, xv, orc.quantize(fmt, wv), n)
    fused = np.maximum(orc.matmul_packed(fmt, xv, orc.quantize(fmt, wv), n, rv), 0.0)
    bt = orc.matmul_packed(fmt, xv, orc.quantize(fmt, np.ascontiguousarray(ev.T)), n, rv)
    # plain launches (the second step finds the staging area in place), then the step captured
    # as a graph and replayed
    for step in range(5):
        if step == 2:
            sess.set_graph_replay(True)
        sess.step()
        sess.wait()
        orc.assert_close(sess.read_output_by_index(0, m * n).reshape(m, n), plain, 1e-3, 1e-4)
        orc.assert_close(sess.read_output_by_index(1, m * n).reshape(m, n), fused, 1e-3, 1e-4)
        orc.assert_close(sess.read_output_by_index(2, m * n).reshape(m, n), bt, 1e-3, 1e-4)
    sess.close()


@pytest.mark.parametrize("k", [15392, 16000, 16384])
def test_siblings_that_plan_alone_but_not_together_run_as_separate_launches(orc, k):
    """q, k, v with a long K and few columns: each weight alone has a one-launch plan with a
    fused norm, three of them in one launch have none (the launch is planned for the columns of
    the whole batch).  The step must fall back to fewer weights per launch, not fail."""
    n = 544
    g = Graph()
    x = g.input("x", [1, k])
    h = g.rms_norm(x, g.parameter("norm", [k]), 1e-5)
    outs = [g.matmul(h, g.parameter_q4(name, [k, n])) for name in ("wq", "wk", "wv")]
    g.set_outputs(outs)
    sess = build_inference_session(g)
    ws = {name: synth.normal(700 + i + k, k * n, 0.02).reshape(k, n) for i, name in enumerate(("wq", "wk", "wv"))}
    for name, w in ws.items():
        sess.set_parameter(name, w)
    gamma = (1.0 + 0.1 * synth.normal(710, k, 1.0)).astype(np.float32)
    xs = synth.normal(711 + k, k, 1.0)
    sess.set_parameter("norm", gamma)
    sess.set_input("x", xs)
    sess.step()
    sess.wait()
    x64 = xs.astype(np.float64)
    normed = (x64 / np.sqrt((x64 * x64).mean() + 1e-5) * gamma).astype(np.float32).reshape(1, k)
    for i, name in enumerate(("wq", "wk", "wv")):
        got = sess.read_output_by_index(i, n)
        want = orc.matmul_f32(normed, orc.dequantize(Q4, orc.quantize(Q4, ws[name]), k, n))
        orc.assert_close(got.reshape(1, n), want, 1e-3, 1e-4)
    sess.close()
