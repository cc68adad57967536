"""Pins the CPU oracle before anything is compared against it.

Expected bytes below were derived by hand / with numpy's own float16 and are
literals; none of them comes from the oracle.  Reference citations are relative
to the reference checkout.
"""
import numpy as np
import pytest

Q4, Q8 = 0, 1


# ---- committed golden vectors ------------------------------------------------------

def test_golden_vectors(orc):
    from helpers import check_golden_packed, golden_vectors
    vectors, f16 = golden_vectors()
    assert len(vectors) >= 7
    for name, fmt, w, entry in vectors:
        packed = orc.quantize(fmt, w)
        check_golden_packed(name, packed, entry)
        deq = orc.dequantize(fmt, packed, *w.shape).reshape(-1)
        for idx, bits_ in entry.get("dequant_f32_bits", {}).items():
            assert int(deq[int(idx)].view(np.uint32)) == bits_, name
    for bits_, val in f16["decode"].items():
        assert orc.f16_bits_to_f32(int(bits_, 16)) == np.float32(val)


# ---- f16 conversion ------------------------------------------------------------

def test_f16_decode_reference_bit_patterns(orc):
    # src/runtime.rs:2269-2290 (q4_decode_f16_matches_half_crate)
    want = {0x3C00: 1.0, 0x4000: 2.0, 0x3800: 0.5, 0xBC00: -1.0, 0x0000: 0.0, 0x7BFF: 65504.0}
    for bits, val in want.items():
        assert orc.f16_bits_to_f32(bits) == np.float32(val)


def test_f16_decode_exhaustive_vs_numpy(orc):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_bits_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    assert (got[~nan].view(np.uint32) == want[~nan].view(np.uint32)).all()


def test_f16_encode_roundtrip_and_ties(orc):
    # every half value encodes back to itself
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    for b, v in zip(bits[::7], vals[::7]):
        if np.isnan(v):
            continue
        assert orc.f32_to_f16_bits(v) == int(b)
    # ties: 1 + 2^-11 is halfway between 0x3C00 and 0x3C01 -> even (0x3C00);
    # 1 + 3*2^-11 is halfway between 0x3C01 and 0x3C02 -> even (0x3C02)
    assert orc.f32_to_f16_bits(1.0 + 2.0**-11) == 0x3C00
    assert orc.f32_to_f16_bits(1.0 + 3 * 2.0**-11) == 0x3C02
    assert orc.f32_to_f16_bits(np.nextafter(np.float32(1.0 + 2.0**-11), np.float32(2))) == 0x3C01
    assert orc.f32_to_f16_bits(65520.0) == 0x7C00  # rounds up to inf
    assert orc.f32_to_f16_bits(65519.0) == 0x7BFF
    assert orc.f32_to_f16_bits(2.0**-24) == 0x0001
    assert orc.f32_to_f16_bits(2.0**-25) == 0x0000  # tie to even (zero)
    assert orc.f32_to_f16_bits(1.5 * 2.0**-24) == 0x0002  # tie to even
    assert orc.f32_to_f16_bits(-0.0) == 0x8000
    assert orc.f32_to_f16_bits(np.inf) == 0x7C00


def test_f16_encode_random_vs_numpy(orc):
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.standard_normal(3000).astype(np.float32) * 0.02,
        rng.standard_normal(3000).astype(np.float32) * 1e-6,   # half subnormals
        rng.standard_normal(3000).astype(np.float32) * 3e4,    # near overflow
        rng.integers(0, 2**32, 3000, dtype=np.uint32).view(np.float32),
    ])
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    for v, w in zip(x, want):
        if np.isnan(v):
            assert (orc.f32_to_f16_bits(v) & 0x7C00) == 0x7C00 and (orc.f32_to_f16_bits(v) & 0x3FF)
        else:
            assert orc.f32_to_f16_bits(v) == int(w), v


# ---- Q4 known answers -------------------------------------------------------------

def _ramp():
    # src/runtime.rs:2223-2226: data[i] = (i as f32 - 16.0) * 0.1
    return ((np.arange(32, dtype=np.float32) - np.float32(16)) * np.float32(0.1)).reshape(32, 1)


def test_q4_known_answer_ramp(orc):
    packed = orc.quantize(Q4, _ramp())
    assert packed.size == 20
    want = bytes.fromhex("9d3266be" "00112233445566778899aabbccddeeff")
    assert packed.tobytes() == want
    deq = orc.dequantize(Q4, packed, 32, 1).reshape(-1)
    assert deq[0].view(np.uint32) == 0xBFCCC000  # nibble 0 -> m_f16 exactly (-1.599609375)
    assert deq[2].view(np.uint32) == 0xBFB24C00
    # src/runtime.rs:2231-2241: the reference's own bar
    assert np.abs(deq - _ramp().reshape(-1)).max() < 0.3
    assert abs(float(np.abs(deq - _ramp().reshape(-1)).max()) - 0.100366235) < 1e-7


def test_q4_roundtrip_matrix_reference_test(orc):
    # src/runtime.rs:2245-2266 (q4_roundtrip_matrix)
    data = (((np.arange(128) % 17).astype(np.float32) - np.float32(8)) * np.float32(0.05)).reshape(32, 4)
    deq = orc.dequantize(Q4, orc.quantize(Q4, data), 32, 4)
    assert np.abs(deq - data).max() < 0.3


def test_q4_ties_round_half_away_from_zero(orc):
    # min 0, max 15 -> d = 1, m = 0; 0.5 -> 1 and 2.5 -> 3 (half-even would give 0 and 2)
    blk = np.zeros((32, 1), np.float32)
    blk[1, 0] = 15.0
    blk[2, 0] = 0.5
    blk[3, 0] = 2.5
    blk[4, 0] = 1.5
    packed = orc.quantize(Q4, blk)
    assert packed[:4].tobytes() == bytes.fromhex("003c0000")  # d=1.0, m=0.0
    assert packed[4] == 0xF0 and packed[5] == 0x31 and packed[6] == 0x02


def test_q4_uses_unrounded_scale_for_nibbles(orc):
    # src/runtime.rs:2084-2088: nibbles come from the f32 d, not from the stored f16 d.
    # Block min 0, max 3.1: d32 = 0.20666666, d16 = 0.20666504 (< d32).  The two values
    # below (f32 bit patterns) sit just under j + 0.5 steps of d32: the f32 scale gives
    # nibbles 6 and 12, the f16-rounded scale would give 7 and 13.
    blk = np.zeros((32, 1), np.float32)
    blk[31, 0] = np.float32(3.1)
    blk[5, 0] = np.array([1068233303], np.uint32).view(np.float32)[0]   # 1.3433331
    blk[8, 0] = np.array([1076188500], np.uint32).view(np.float32)[0]   # 2.583333
    packed = orc.quantize(Q4, blk)
    assert packed[:4].tobytes() == bytes.fromhex("9d320000")
    assert (packed[4 + 2] >> 4) == 6
    assert (packed[4 + 4] & 0xF) == 12
    assert (packed[4 + 15] >> 4) == 15


def test_q4_constant_block_and_zero_block(orc):
    for val, mbits in ((0.0, 0x0000), (0.375, 0x3600), (-2.0, 0xC000)):
        blk = np.full((32, 1), val, np.float32)
        packed = orc.quantize(Q4, blk)
        # src/runtime.rs:2068-2072: degenerate block -> d = 1.0 (0x3C00), nibbles all 0
        assert packed[:2].tobytes() == bytes.fromhex("003c")
        assert int(packed[2]) | (int(packed[3]) << 8) == mbits
        assert not packed[4:].any()
        assert (orc.dequantize(Q4, packed, 32, 1) == np.float32(val)).all()


def test_q4_layout_column_blocked_soa(orc):
    # src/runtime.rs:2049-2058,2078-2083: block id = col*bpc + blk; dm words first, nibbles after
    rng = np.random.default_rng(3)
    rows, cols = 96, 5
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    packed = orc.quantize(Q4, w)
    nb = 3 * cols
    assert packed.size == nb * 20
    for col in range(cols):
        for blk in range(3):
            single = orc.quantize(Q4, w[blk * 32:(blk + 1) * 32, col:col + 1].copy())
            b = col * 3 + blk
            assert packed[b * 4:b * 4 + 4].tobytes() == single[:4].tobytes()
            assert packed[nb * 4 + b * 16:nb * 4 + b * 16 + 16].tobytes() == single[4:].tobytes()


def test_q4_invariants_random(orc):
    rng = np.random.default_rng(11)
    rows, cols = 256, 24
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    packed = orc.quantize(Q4, w)
    deq = orc.dequantize(Q4, packed, rows, cols)
    nb = (rows // 32) * cols
    dm = packed[:nb * 4].view(np.uint32)
    d16 = (dm & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
    m16 = (dm >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
    wb = w.reshape(rows // 32, 32, cols).transpose(2, 0, 1).reshape(nb, 32)  # [block, i]
    db = deq.reshape(rows // 32, 32, cols).transpose(2, 0, 1).reshape(nb, 32)
    mn, mx = wb.min(1), wb.max(1)
    d32 = (mx - mn) / np.float32(15)
    # stored values are the f16 roundings of f32 d and m
    assert (d16 == d32.astype(np.float16).astype(np.float32)).all()
    assert (m16 == mn.astype(np.float16).astype(np.float32)).all()
    # block min decodes to m_f16 exactly, block max to 15*d_f16 + m_f16
    assert (db[np.arange(nb), wb.argmin(1)] == m16).all()
    assert (db[np.arange(nb), wb.argmax(1)] == np.float32(15) * d16 + m16).all()
    # error bound per element
    bound = d16 / 2 + 15 * np.abs(d32 - d16) + np.abs(mn - m16) + 1e-7
    assert (np.abs(db - wb) <= bound[:, None]).all()
    # every decoded value is nibble*d16 + m16 for an integer nibble in 0..15
    nibs = np.rint((db - m16[:, None]) / d16[:, None])
    assert nibs.min() >= 0 and nibs.max() <= 15
    assert (nibs.astype(np.float32) * d16[:, None] + m16[:, None] == db).all()


def test_q4_column_independence_concat(orc):
    # what makes the fused gate|up weight equal to separately quantized halves
    # (src/optimize.rs:842-854, src/runtime.rs:2373-2406)
    rng = np.random.default_rng(5)
    a = rng.standard_normal((64, 8)).astype(np.float32)
    b = rng.standard_normal((64, 8)).astype(np.float32)
    whole = orc.dequantize(Q4, orc.quantize(Q4, np.hstack([a, b])), 64, 16)
    assert (whole[:, :8] == orc.dequantize(Q4, orc.quantize(Q4, a), 64, 8)).all()
    assert (whole[:, 8:] == orc.dequantize(Q4, orc.quantize(Q4, b), 64, 8)).all()


def test_rows_must_be_multiple_of_32(orc):
    # src/runtime.rs:2037-2040, 2145-2148
    with pytest.raises(ValueError):
        orc.quantize(Q4, np.zeros((33, 2), np.float32))
    with pytest.raises(ValueError):
        orc.quantize(Q8, np.zeros((31, 2), np.float32))


def test_nan_and_inf_inputs_do_not_crash(orc):
    blk = np.linspace(-1, 1, 32, dtype=np.float32).reshape(32, 1)
    blk[3, 0] = np.nan
    p = orc.quantize(Q4, blk)
    assert (p[4 + 1] >> 4) == 0  # NaN -> nibble 0 (Rust `as u8` of NaN)
    q = orc.quantize(Q8, blk)
    assert q[4 + 3] == 0
    blk[3, 0] = np.inf
    orc.quantize(Q4, blk)
    orc.quantize(Q8, blk)


# ---- Q8 known answers (the reference holds no Q8 test: these are all there is) --------

def test_q8_known_answer_ramp(orc):
    packed = orc.quantize(Q8, _ramp())
    assert packed.size == 36
    q = [-127, -119, -111, -103, -95, -87, -79, -71, -64, -56, -48, -40, -32, -24, -16, -8,
         0, 8, 16, 24, 32, 40, 48, 56, 64, 71, 79, 87, 95, 103, 111, 119]
    want = bytes.fromhex("73220000") + np.array(q, np.int8).tobytes()
    assert packed.tobytes() == want
    deq = orc.dequantize(Q8, packed, 32, 1).reshape(-1)
    s16 = np.array([0x2273], np.uint16).view(np.float16).astype(np.float32)[0]
    assert (deq == np.array(q, np.float32) * s16).all()


def test_q8_ties_round_half_away_from_zero(orc):
    blk = np.zeros((32, 1), np.float32)
    blk[0, 0] = 127.0  # scale = 1, inv = 1
    blk[1:5, 0] = [0.5, 2.5, -0.5, -2.5]
    packed = orc.quantize(Q8, blk)
    assert packed[:4].tobytes() == bytes.fromhex("003c0000")
    assert packed[4:9].view(np.int8).tolist() == [127, 1, 3, -1, -3]


def test_q8_zero_block_and_layout(orc):
    packed = orc.quantize(Q8, np.zeros((32, 1), np.float32))
    assert packed[:4].tobytes() == bytes.fromhex("003c0000") and not packed[4:].any()
    rng = np.random.default_rng(9)
    rows, cols = 64, 3
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    packed = orc.quantize(Q8, w)
    assert packed.size == 36 * 2 * cols
    blocks = packed.reshape(-1, 36)
    assert not blocks[:, 2:4].any()  # pad bytes stay zero
    assert np.abs(blocks[:, 4:].view(np.int8).astype(int)).max() <= 127
    for col in range(cols):
        for blk in range(2):
            single = orc.quantize(Q8, w[blk * 32:(blk + 1) * 32, col:col + 1].copy())
            assert blocks[col * 2 + blk].tobytes() == single.tobytes()
    # each block's absmax element maps to +-127
    deq = orc.dequantize(Q8, packed, rows, cols)
    s16 = blocks[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    wb = w.reshape(2, 32, cols).transpose(2, 0, 1).reshape(-1, 32)
    db = deq.reshape(2, 32, cols).transpose(2, 0, 1).reshape(-1, 32)
    amax = np.abs(wb).max(1)
    assert (s16 == (amax / np.float32(127)).astype(np.float16).astype(np.float32)).all()
    assert (np.abs(db[np.arange(db.shape[0]), np.abs(wb).argmax(1)]) == np.float32(127) * s16).all()
    assert (np.abs(db - wb) <= (s16 / 2 + 127 * np.abs(amax / np.float32(127) - s16))[:, None] + 1e-7).all()


# ---- matmul ground truth ------------------------------------------------------------

def test_matmul_known_answers_from_reference_tests(orc):
    # tests/gpu_smoke.rs:130-168 style: small integer-valued matmul has an exact answer
    a = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    b = np.array([[7, 8], [9, 10], [11, 12]], np.float32)
    want = np.array([[58, 64], [139, 154]], np.float32)
    assert (orc.matmul_f32(a, b) == want).all()
    assert (orc.matmul_f64(a, b) == want).all()
    d = np.array([[1, -1], [0.5, 2]], np.float32)
    assert (orc.matmul_f32(a, b, d) == want + d).all()
    # a transposed operand or swapped index must fail this: non-square, non-symmetric
    assert orc.matmul_f32(a, b).shape == (2, 2)


def test_matmul_f32_is_sequential_k_without_fma(orc):
    # order matters: (1e8 + 1) - 1e8 in f32, k ascending -> 0; any reordering that adds
    # 1 and -1e8... differently would give 1.  Also a product whose fused form differs.
    a = np.array([[1.0, 1.0, 1.0]], np.float32)
    b = np.array([[1e8], [1.0], [-1e8]], np.float32)
    assert orc.matmul_f32(a, b)[0, 0] == 0.0
    x = np.float32(1 + 2**-12)
    a = np.array([[x, 1.0]], np.float32)
    b = np.array([[x], [-np.float32(x * x)]], np.float32)
    assert orc.matmul_f32(a, b)[0, 0] == 0.0  # an FMA would leave the rounding error of x*x


def test_matmul_matches_python_loop_tiny(orc):
    rng = np.random.default_rng(1)
    a = rng.standard_normal((3, 40)).astype(np.float32)
    b = rng.standard_normal((40, 5)).astype(np.float32)
    want = np.zeros((3, 5), np.float32)
    for r in range(3):
        for c in range(5):
            s = np.float32(0)
            for k in range(40):
                s = np.float32(s + np.float32(a[r, k] * b[k, c]))
            want[r, c] = s
    assert (orc.matmul_f32(a, b) == want).all()
    assert np.abs(orc.matmul_f64(a, b) - (a.astype(np.float64) @ b.astype(np.float64))).max() < 1e-6


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_packed_and_tiled_matmul_equal_plain(orc, fmt):
    rng = np.random.default_rng(2)
    m, k, n = 6, 128, 70  # ragged: n not a multiple of 64, m < 64
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    d = rng.standard_normal((m, n)).astype(np.float32)
    packed = orc.quantize(fmt, w)
    deq = orc.dequantize(fmt, packed, k, n)
    want = orc.matmul_f32(a, deq, d)
    assert (orc.matmul_packed(fmt, a, packed, n, d) == want).all()
    assert (orc.matmul_packed(fmt, a, packed, n, d, tiled=True) == want).all()
    assert (orc.matmul_packed(fmt, a, packed, n) == orc.matmul_f32(a, deq)).all()


def test_q4_matmul_correctness_reference_inputs(orc):
    # tests/gpu_smoke.rs:2681-2771 inputs (m=6,k=1024,n=2048): the f32 and f64 sums over the
    # dequantized weights agree far inside the reference's own 0.1 bar
    m, k, n = 6, 1024, 2048
    i = np.arange(m * k)
    a = (((i % 7).astype(np.float32) - np.float32(3)) * np.float32(0.5)).reshape(m, k)
    i = np.arange(k * n)
    b = ((i % 11).astype(np.float32) - np.float32(5)) * np.float32(0.3)
    b = np.where(i % 1000 == 0, b * np.float32(5), b).astype(np.float32).reshape(k, n)
    packed = orc.quantize(Q4, b)
    deq = orc.dequantize(Q4, packed, k, n)
    c32 = orc.matmul_packed(Q4, a, packed, n)
    c64 = orc.matmul_f64(a, deq)
    assert np.abs(c32 - c64).max() < 0.1
    orc.assert_close(c32, c64, 1e-3, 1e-4)
