"""CPU-side checks of the shipped library: the C ABI loads and exports every
declared symbol, the host quantizers equal the oracle byte for byte, and the
graph compiler routes matmuls as the reference does.  No GPU call is made."""
import ctypes
import os
import re

import numpy as np
import pytest

from helpers import Q4, Q8, bits, gemv_parity_inputs
from meganeura_amd import capi, synth
from meganeura_amd.graph import Graph, ShaderEntry, WeightFormat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(capi.LIB_PATH)
    declared = set()
    for header, listed in (("mgn_hip.h", capi.HIP_SYMBOLS), ("mgn_bench.h", capi.BENCH_SYMBOLS),
                           ("mgn_session.h", capi.SESSION_SYMBOLS)):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        here = set(re.findall(r"\b(mgn_[a-z0-9_]+)\s*\(", text))
        assert here == set(listed), header
        declared |= here
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert capi.load().mgn_built_for() == b"gfx950"


def test_no_product_file_touches_the_oracle():
    for base, _, files in os.walk(os.path.join(ROOT, "meganeura_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "liboracle" not in text and "import oracle" not in text and "from oracle" not in text, f


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("shape", [(32, 1), (64, 7), (576, 192), (1536, 100), (4096, 33)])
def test_host_quantizer_equals_oracle(orc, fmt, shape):
    k, n = shape
    w = synth.normal(100 + k + n + fmt, k * n, 0.02).reshape(k, n)
    w[0, 0] = 0.0
    if n > 2:
        w[:32, 1] = 0.25          # constant block
        w[:32, 2] = 0.0           # zero block
    packed = capi.quantize_ref(fmt, w)
    want = orc.quantize(fmt, w)
    assert packed.size == capi.packed_size(fmt, k, n) == want.size
    assert (packed == want).all()
    got = capi.dequantize_ref(fmt, packed, k, n)
    assert (bits(got) == bits(orc.dequantize(fmt, want, k, n))).all()


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_host_quantizer_extreme_values(orc, fmt):
    rng = np.random.default_rng(4)
    k, n = 64, 40
    w = rng.standard_normal((k, n)).astype(np.float32)
    w[:, 0] *= 1e-7       # f16-subnormal scales
    w[:, 1] *= 1e-10      # scales that round to zero in f16
    w[:, 2] *= 1e4
    w[:, 3] *= 1e6        # scales overflow f16 -> inf
    w[5, 4] = np.nan
    w[6, 5] = np.inf
    w[7, 6] = -np.inf
    w[:, 7] = np.float32(1e-45)
    w[:32, 8] = np.linspace(0, 15, 32, dtype=np.float32)   # exact ties at .5 steps
    w[:32, 9] = np.arange(32, dtype=np.float32) * 0.5
    with np.errstate(all="ignore"):
        packed = capi.quantize_ref(fmt, w)
        want = orc.quantize(fmt, w)
        assert (packed == want).all()
        a = capi.dequantize_ref(fmt, packed, k, n)
        b = orc.dequantize(fmt, want, k, n)
    nan = np.isnan(b)
    assert (np.isnan(a) == nan).all() and (bits(a)[~nan] == bits(b)[~nan]).all()


def test_host_quantizer_rejects_ragged_rows():
    # src/runtime.rs:2037-2040: "Q4 requires rows (K dim) to be a multiple of 32"
    with pytest.raises(capi.MgnError):
        capi.quantize_ref(Q4, np.zeros((48, 4), np.float32))
    with pytest.raises(capi.MgnError):
        capi.quantize_ref(Q8, np.zeros((31, 4), np.float32))
    assert capi.packed_size(Q4, 576, 1536) == 552960   # src/graph.rs:52-68
    assert capi.packed_size(Q8, 576, 1536) == 995328
    assert capi.packed_size(Q4, 4096, 14336) == 36700160


def test_context_creation_fails_cleanly_without_gpu():
    lib = capi.load()
    h = ctypes.c_void_p()
    st = lib.mgn_ctx_create(10_000, ctypes.byref(h))
    assert st != capi.OK and not h.value
    assert lib.mgn_last_error(None)


# ---- routing: tests/gemv_parity.rs:32-52, 157-174 -------------------------------------

def _plan(m, k, n, quant="q4", add=False):
    g = Graph()
    a = g.input("a", [m, k])
    b = {"q4": g.parameter_q4, "q8": g.parameter_q8, "f32": g.parameter}[quant]("b", [k, n])
    out = g.matmul(a, b)
    if add:
        out = g.add(out, g.parameter("d", [m, n]))
    g.set_outputs([out])
    return g.compile()


@pytest.mark.parametrize("quant", ["q4", "q8", "f32"])
def test_m1_routes_to_gemv_iff_n_multiple_of_4(quant):
    fmt = {"q4": WeightFormat.Q4, "q8": WeightFormat.Q8, "f32": WeightFormat.F32}[quant]
    for n in (576, 1536, 49152, 192):
        (d,) = _plan(1, 576, n, quant)
        assert d.shader == ShaderEntry.MatMulGemv and d.workgroups == [n // 4, 1, 1]
        assert d.params == [1, 576, n, 0] and d.weight_format == fmt
    (d,) = _plan(1, 64, 66, quant)
    assert d.shader == ShaderEntry.MatMul and d.workgroups == [2, 1, 1]
    (d,) = _plan(6, 1024, 2048, quant)
    assert d.shader == ShaderEntry.MatMul and d.workgroups == [32, 1, 1] and d.params == [6, 1024, 2048, 0]
    (d,) = _plan(512, 1024, 3072, quant)
    assert d.workgroups == [48, 8, 1]


def test_matmul_add_fuses_and_routes():
    (d,) = _plan(1, 1536, 576, "q4", add=True)
    assert d.shader == ShaderEntry.MatMulGemvAdd and d.workgroups == [144, 1, 1]
    (d,) = _plan(4, 1536, 576, "q8", add=True)
    assert d.shader == ShaderEntry.FusedMatMulAdd and d.weight_format == WeightFormat.Q8


def test_matmul_that_is_an_output_is_not_fused():
    g = Graph()
    a = g.input("a", [1, 64])
    b = g.parameter_q4("b", [64, 64])
    mm = g.matmul(a, b)
    out = g.add(mm, g.parameter("d", [1, 64]))
    g.set_outputs([out, mm])
    shaders = [d.shader for d in g.compile()]
    assert shaders == [ShaderEntry.MatMulGemv, ShaderEntry.Add]


def test_unary_after_a_tiled_matmul_becomes_its_epilogue():
    # src/compile.rs:3498-3512 (test_compile_fused), with the weight quantized: one MatMul dispatch
    # that carries the Relu; a chain folds one by one; the M = 1 entries are left alone
    # (compile.rs:971-983 lists the tiled entries only)
    from meganeura_amd.graph import EpilogueOp
    g = Graph()
    x = g.input("x", [4, 800])
    h = g.relu(g.matmul(x, g.parameter_q4("w", [800, 128])))
    g.set_outputs([h])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.MatMul and d.weight_format == WeightFormat.Q4 and d.epilogue == [EpilogueOp.Relu]

    g = Graph()
    x = g.input("x", [4, 800])
    mm = g.add(g.matmul(x, g.parameter_q8("w", [800, 128])), g.input("r", [4, 128]))
    g.set_outputs([g.neg(g.silu(mm))])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.FusedMatMulAdd and d.epilogue == [EpilogueOp.Silu, EpilogueOp.Neg]

    g = Graph()
    x = g.input("x", [1, 800])
    g.set_outputs([g.sigmoid(g.matmul(x, g.parameter_q4("w", [800, 128])))])
    plan = g.compile()
    assert [d.shader for d in plan] == [ShaderEntry.MatMulGemv, ShaderEntry.Sigmoid] and plan[0].epilogue == []
    assert plan[1].workgroups == [1, 1, 1] and plan[1].params == [128, 0, 0, 0]


def test_unary_is_not_folded_when_the_matmul_result_is_needed():
    # a second reader, or the result being a graph output (the reference does not look at outputs
    # there and would leave such an output unwritten)
    for keep in ("reader", "output"):
        g = Graph()
        x = g.input("x", [4, 800])
        mm = g.matmul(x, g.parameter_q4("w", [800, 128]))
        r = g.relu(mm)
        outs = [r, g.add(mm, g.input("r", [4, 128]))] if keep == "reader" else [r, mm]
        g.set_outputs(outs)
        plan = g.compile()
        assert plan[0].shader == ShaderEntry.MatMul and plan[0].epilogue == []
        assert ShaderEntry.Relu in [d.shader for d in plan]


def test_all_unary_entries():
    # src/compile.rs:3515-3531 (test_compile_all_unary_ops)
    g = Graph()
    x = g.input("x", [4, 8])
    g.set_outputs([g.relu(x), g.sigmoid(x), g.neg(x), g.silu(x)])
    plan = g.compile()
    assert [d.shader for d in plan] == [ShaderEntry.Relu, ShaderEntry.Sigmoid, ShaderEntry.Neg, ShaderEntry.Silu]
    assert all(d.params == [32, 0, 0, 0] and d.workgroups == [1, 1, 1] for d in plan)


def test_swiglu_of_two_matmuls_becomes_one_wide_matmul():
    # src/optimize.rs:776-879; the concatenated weight keeps the Q4 dtype (848-854)
    g = Graph()
    h = g.input("h", [1, 576])
    gate = g.matmul(h, g.parameter_q4("w_gate", [576, 1536]))
    up = g.matmul(h, g.parameter_q4("w_up", [576, 1536]))
    act = g.swiglu(gate, up)
    down = g.matmul(act, g.parameter_q4("w_down", [1536, 576]))
    out = g.add(g.input("resid", [1, 576]), down)
    g.set_outputs([out])
    plan = g.compile()
    assert [d.shader for d in plan] == [ShaderEntry.MatMulGemv, ShaderEntry.SwiGLUConcat, ShaderEntry.MatMulGemvAdd]
    assert plan[0].params == [1, 576, 3072, 0] and plan[0].weight_format == WeightFormat.Q4
    assert plan[1].params[:2] == [1536, 1536]
    assert plan[2].params == [1, 1536, 576, 0]


def test_graph_builder_errors():
    g = Graph()
    a = g.input("a", [2, 64])
    b = g.parameter_q4("b", [32, 8])
    with pytest.raises(ValueError, match="inner dimensions"):
        g.matmul(a, b)
    with pytest.raises(ValueError, match="matching shapes"):
        g.add(a, b)
    v = g.parameter("v", [64])
    with pytest.raises(ValueError, match="2D"):
        g.matmul(a, v)
    assert g.rms_norm(a, v, 1e-6) >= 0


def test_nk_quantizer_equals_quantizing_the_transpose(orc):
    """A weight stored [N, K] (matmul_bt operand) is blocked along K: the bytes are those of
    the reference quantizer applied to the transposed [K, N] matrix."""
    from meganeura_amd import capi, synth
    for fmt in (0, 1):
        for n, k in ((5, 64), (192, 576), (1, 32)):
            w_nk = synth.normal(800 + n + k, n * k, 0.02).reshape(n, k)
            w_nk[0, :32] = 0.25  # a constant block
            got = capi.quantize_ref_nk(fmt, w_nk)
            assert (got == orc.quantize(fmt, np.ascontiguousarray(w_nk.T))).all()
    with pytest.raises(capi.MgnError):
        capi.quantize_ref_nk(0, np.zeros((4, 48), np.float32))


def test_matmul_bt_lowering_and_mixed_use():
    # src/compile.rs:1447-1485: GemvBT at M = 1 and K % 4 == 0, params [m, n, k, 0]
    from meganeura_amd.graph import Graph, ShaderEntry, WeightFormat
    g = Graph()
    x = g.input("x", [1, 576])
    e = g.parameter_q4("embed", [49152, 576])
    g.set_outputs([g.matmul_bt(x, e)])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.MatMulGemvBT and d.workgroups == [49152, 1, 1]
    assert d.params == [1, 49152, 576, 0] and d.weight_format == WeightFormat.Q4
    g = Graph()
    x = g.input("x", [6, 64])
    e = g.parameter_q8("e", [70, 64])
    g.set_outputs([g.matmul_bt(x, e)])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.MatMulBT and d.workgroups == [2, 1, 1] and d.params == [6, 70, 64, 0]
    with pytest.raises(ValueError, match="K dimensions must match"):
        g2 = Graph()
        g2.matmul_bt(g2.input("x", [1, 64]), g2.parameter_q4("e", [64, 32]))
    # one quantized parameter, both orientations: its blocks can only run one way
    g3 = Graph()
    x = g3.input("x", [1, 64])
    e = g3.parameter_q4("e", [64, 64])
    g3.set_outputs([g3.matmul(x, e), g3.matmul_bt(x, e)])
    with pytest.raises(ValueError, match="both matmul and matmul_bt"):
        g3.compile()


def test_matmul_at_and_fused_add_forms_lowering():
    # src/compile.rs:1423-1445, 1526-1574: A stored [K, M]; always the tiled entry; params
    # [m, n, k, 0]; Add(MatMulAT) and Add(MatMulBT) fuse like Add(MatMul) (src/optimize.rs:724-767)
    from meganeura_amd.graph import EpilogueOp, Graph, ShaderEntry, WeightFormat
    g = Graph()
    xt = g.input("xt", [64, 1])
    w = g.parameter_q8("w", [64, 132])
    g.set_outputs([g.matmul_at(xt, w)])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.MatMulAT and d.workgroups == [3, 1, 1]
    assert d.params == [1, 132, 64, 0] and d.weight_format == WeightFormat.Q8
    g = Graph()
    xt = g.input("xt", [96, 70])
    r = g.input("r", [70, 40])
    w = g.parameter_q4("w", [96, 40])
    g.set_outputs([g.relu(g.add(r, g.matmul_at(xt, w)))])
    (d,) = g.compile()
    assert d.shader == ShaderEntry.FusedMatMulATAdd and d.workgroups == [1, 2, 1] and d.params == [70, 40, 96, 0]
    assert d.epilogue == [EpilogueOp.Relu]
    g = Graph()
    x = g.input("x", [1, 64])
    r = g.input("r", [1, 48])
    e = g.parameter_q4("e", [48, 64])
    g.set_outputs([g.add(g.matmul_bt(x, e), r)])
    (d,) = g.compile()  # no GEMV form of the fused BT entry in the reference
    assert d.shader == ShaderEntry.FusedMatMulBTAdd and d.workgroups == [1, 1, 1] and d.params == [1, 48, 64, 0]
    with pytest.raises(ValueError, match="K dimensions must match"):
        g2 = Graph()
        g2.matmul_at(g2.input("x", [32, 4]), g2.parameter_q4("w", [64, 8]))
    # matmul and matmul_at read a parameter the same way; matmul_at and matmul_bt do not
    g3 = Graph()
    w = g3.parameter_q4("w", [64, 64])
    g3.set_outputs([g3.matmul(g3.input("x", [2, 64]), w), g3.matmul_at(g3.input("xt", [64, 2]), w)])
    assert [d.shader for d in g3.compile()] == [ShaderEntry.MatMul, ShaderEntry.MatMulAT]
    g4 = Graph()
    w = g4.parameter_q4("w", [64, 64])
    g4.set_outputs([g4.matmul_at(g4.input("xt", [64, 2]), w), g4.matmul_bt(g4.input("x", [2, 64]), w)])
    with pytest.raises(ValueError, match="both matmul and matmul_bt"):
        g4.compile()


def test_host_quantizer_matches_golden_vectors():
    from helpers import check_golden_packed, golden_vectors
    vectors, _ = golden_vectors()
    for name, fmt, w, entry in vectors:
        packed = capi.quantize_ref(fmt, w)
        check_golden_packed(name, packed, entry)
        deq = capi.dequantize_ref(fmt, packed, *w.shape).reshape(-1)
        for idx, bits_ in entry.get("dequant_f32_bits", {}).items():
            assert int(deq[int(idx)].view(np.uint32)) == bits_, name


def test_a_c_program_links_against_the_library(tmp_path):
    """The boundary is C: a C99 translation unit includes both headers, links the shared library
    and calls the entries that need no device (sizes, host quantizer, planner, graph lowering)."""
    import os
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler here")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.join(root, "meganeura_amd")
    src = tmp_path / "consumer.c"
    src.write_text(r"""
#include <stdio.h>
#include <string.h>
#include "mgn_hip.h"
#include "mgn_session.h"
int main(void) {
  float w[32];
  unsigned char packed[20];
  float back[32];
  int i;
  mgn_plan_info plan;
  mgn_graph* g;
  int x, p, y;
  for (i = 0; i < 32; i++) w[i] = (float)(i - 16) * 0.1f;           /* src/runtime.rs:2223-2226 */
  if (mgn_packed_size(MGN_FMT_Q4, 32, 1) != 20 || mgn_packed_size(MGN_FMT_Q8, 64, 3) != 216) return 1;
  if (mgn_quantize_ref(MGN_FMT_Q4, w, 32, 1, packed) != MGN_OK) return 2;
  if (packed[0] != 0x9D || packed[1] != 0x32 || packed[2] != 0x66 || packed[3] != 0xBE) return 3;
  if (mgn_dequantize_ref(MGN_FMT_Q4, packed, 32, 1, back) != MGN_OK) return 4;
  for (i = 0; i < 32; i++) if (back[i] - w[i] > 0.3f || w[i] - back[i] > 0.3f) return 5;
  if (mgn_matmul_q_plan(MGN_FMT_Q4, 1, 4096, 14336, 0, 256, &plan) != MGN_OK) return 6;
  if (plan.route != MGN_ROUTE_GEMV_MFMA || plan.grid[0] != 256) return 7;
  g = mgn_graph_new();
  x = mgn_graph_input(g, "x", 1, 64);
  p = mgn_graph_parameter_q4(g, "w", 64, 8);
  y = mgn_graph_matmul(g, x, p);
  if (x < 0 || p < 0 || y < 0) return 8;
  if (mgn_graph_matmul(g, x, x) >= 0 || strlen(mgn_graph_last_error(g)) == 0) return 9;  /* 64 != 1 */
  mgn_graph_free(g);
  puts("ok");
  return 0;
}
""")
    exe = tmp_path / "consumer"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(root, "include"), str(src), "-o", str(exe),
                    "-L", libdir, "-lmgn_hip", "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and out.stdout.strip() == "ok", (out.returncode, out.stdout, out.stderr)
