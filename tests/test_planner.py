"""The launch planner on the host: mgn_matmul_q_plan tells what mgn_matmul_q would launch for a
shape without touching a device.  Swept over decode and prefill shapes, the geometry must cover
every column and every K block exactly once, stay inside the hardware limits (threads, LDS) and
inside the context's workspace, and put the BASELINE configurations on the kernels built for them."""
import itertools

import pytest

from meganeura_amd import capi

Q4, Q8 = 0, 1
GENERIC, GEMV_VALU, GEMV_MFMA, GEMM_MFMA, TILE_MFMA = 1, 2, 3, 4, 5
WORKSPACE = 16 << 20
COUNTERS = 4096

KS = [32, 64, 96, 480, 512, 544, 576, 960, 1024, 1536, 2048, 3072, 4096, 5120, 8192, 11008, 11040, 12288, 14336,
      16384, 28672, 32768, 65536]
NS = [1, 3, 4, 64, 100, 192, 576, 1027, 3072, 4096, 14336, 49152, 151936]
MS = [1, 2, 3, 4, 5, 8, 16, 17, 64, 512]


def ceil_div(a, b):
    return -(-a // b)


def check_gemv(p, fmt, m, k, n):
    mrows = m if m <= 2 else 4
    bpc = k // 32
    assert m <= 4
    assert p.threads == 64 * p.k_splits * p.waves_n <= 1024
    assert p.lds_bytes <= 150 * 1024
    assert p.k_parts >= 1 and p.grid[1] == p.k_parts and p.grid[2] == 1
    steps_all = ceil_div(bpc, 16)
    if p.k_parts > 1:
        # parts of a whole number of 16-block steps, none of them empty; their kernels always mask
        steps_total = ceil_div(steps_all, p.k_parts)
        assert (p.k_parts - 1) * steps_total < steps_all
        assert p.full_steps == 0 and p.quads_per_wave == 1
        assert p.workspace_bytes == (p.k_parts - 1) * mrows * n * 4 <= WORKSPACE  # the last part keeps its own sums
    elif p.tail_blocks:
        # full steps plus a few leftover blocks that the wave's quads share one more step for
        assert fmt == Q4 and p.k_splits == 1 and p.full_steps == 1 and p.workspace_bytes == 0
        assert bpc == 16 * p.steps + p.tail_blocks and p.tail_blocks in (1, 2, 4)
        assert p.quads_per_wave * p.tail_blocks <= 16
        steps_total = p.steps
    else:
        steps_total = steps_all
        assert p.workspace_bytes == 0
        assert p.full_steps == int(bpc % 16 == 0 and p.k_splits * p.steps == steps_total)
    assert 1 <= p.steps <= 8
    assert p.k_splits * p.steps >= steps_total          # all of K is walked
    assert (p.k_splits - 1) * p.steps < steps_total      # no K split without a step of its own
    nquads = ceil_div(n, 4)
    per_wg = p.waves_n * p.quads_per_wave
    assert p.grid[0] * per_wg >= nquads                  # every column has a wave
    assert (p.grid[0] - 1) * per_wg < nquads             # no workgroup without a column
    if p.quads_per_wave > 1:
        assert p.k_splits == 1 and p.steps * p.quads_per_wave + (1 if p.tail_blocks else 0) <= 8


def check_gemm(p, fmt, m, k, n, f16):
    rows = 32 if f16 or m > 16 else 16  # f32 rows travel as fp16 pairs: 16 per tile up to M = 16, 32 beyond
    bpc = k // 32
    assert p.grid[2] == ceil_div(m, rows)
    assert p.threads == 64 * p.k_splits * p.waves_n <= 512
    assert p.k_splits in (1, 2)
    assert p.lds_bytes <= 160 * 1024
    n_tiles = ceil_div(n, 32)
    assert p.grid[1] * p.waves_n >= n_tiles and (p.grid[1] - 1) * p.waves_n < n_tiles
    chunks = ceil_div(bpc, 8 * p.k_splits)
    assert p.grid[0] == p.k_parts >= 1
    assert p.k_parts * p.steps >= chunks and (p.k_parts - 1) * p.steps < chunks
    if p.k_parts > 1:
        assert p.workspace_bytes == p.k_parts * p.grid[2] * rows * n * 4 <= WORKSPACE
        assert p.grid[1] * p.grid[2] <= COUNTERS
    else:
        assert p.workspace_bytes == 0


def check_tile(p, fmt, m, k, n, f16):
    """MGN_ROUTE_TILE_MFMA: tiles of 16 columns, K in slices of 256 elements, `full_steps` row tiles of 16 rows
    per workgroup.  quads_per_wave == 0: the form that keeps the activation images in LDS (grid, as the plan
    reports it: (K parts, column groups, row groups of 16 or 32 rows); launched with the groups in x, rounded
    up to a multiple of 8, and the parts in y), 8 waves with one or two pairs of tiles each, parts of
    4 slices; row groups of 32 only with fp16 activations); otherwise the general form (grid = (K parts, column groups, row groups),
    `k_splits` waves per tile) in `quads_per_wave` launches over blocks of rows."""
    nslices, n_tiles = ceil_div(k, 256), ceil_div(n, 16)
    assert p.lds_bytes <= 160 * 1024 and p.threads <= 512
    rows = 16 * p.full_steps
    assert p.grid[1] * p.waves_n >= n_tiles and (p.grid[1] - 1) * p.waves_n < n_tiles
    assert p.grid[0] == p.k_parts >= 1
    if p.quads_per_wave == 0:
        assert p.threads == 512 and p.full_steps in (1, 2)
        if m > 32:  # beyond 32 rows only with few K parts and small partial tiles
            assert p.k_parts <= 4 and p.workspace_bytes <= 8 << 20 and (fmt == Q4 or m >= 128)
        assert p.grid[2] * rows >= m and (p.grid[2] - 1) * rows < m
        assert p.steps == 4 and p.waves_n in (16, 32)
        assert p.full_steps == 1 or f16  # row groups of 32 are for fp16 activations
        assert p.k_parts == ceil_div(nslices, p.steps)
        # partial tiles in whole workgroup slots: 8 waves x (pairs x 2 tiles x row tiles) float4 per lane;
        # the parts meet without counters.  Either the last part adds the others up and keeps its own
        # tiles, or -- when the whole grid is resident at once (256 CUs here) and the parts are five or
        # more, or the workgroups fill at most two thirds of the chip -- every part adds up a share and
        # the workspace holds all parts' tiles.
        slot = 8 * (p.waves_n // 16) * 2 * p.full_steps * 1024
        # (resident at once is a matter of every XCD: it gets every eighth group with all its parts, on 32 CUs)
        wgs = p.k_parts * p.grid[1] * p.grid[2]
        per_xcd = ceil_div(p.grid[1] * p.grid[2], 8) * p.k_parts
        shares = p.k_parts >= 2 and per_xcd <= 32 and (p.k_parts >= 5 or 3 * wgs <= 2 * 256)
        partial = (p.k_parts if shares else p.k_parts - 1) * p.grid[2] * p.grid[1] * slot
        assert p.workspace_bytes == partial <= WORKSPACE
    else:
        assert p.full_steps in (1, 2, 4) and p.k_splits in (1, 2, 4) and p.threads == 64 * p.k_splits * p.waves_n
        assert p.k_parts * p.steps * p.k_splits >= nslices
        assert p.quads_per_wave * p.grid[2] * rows >= m          # the launches' row groups cover every row
        if p.quads_per_wave == 1:
            assert (p.grid[2] - 1) * rows < m
        assert p.workspace_bytes <= WORKSPACE
        if p.k_parts > 1:
            assert p.grid[1] * p.grid[2] <= COUNTERS


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_plans_cover_the_problem_and_respect_the_limits(fmt):
    routes = set()
    for m, k, n in itertools.product(MS, KS, NS):
        if (k // 32) * n >= 0x7FFFFFFF:
            continue
        # activations: f32 of any magnitude (a context's default), fp16, f32 promised to lie in the fp16 range
        for f16, promised in ((False, False), (True, False), (False, True)):
            p = capi.matmul_plan(fmt, m, k, n, f16, fp16_range=promised)
            where = f"fmt={fmt} m={m} k={k} n={n} f16={f16} promised={promised} route={p.route}"
            routes.add(p.route)
            try:
                assert p.route in (GENERIC, GEMV_VALU, GEMV_MFMA, GEMM_MFMA, TILE_MFMA)
                if m > 4 and not f16 and not promised:
                    # nothing is assumed about f32 activations: the rescaling kernels (their lanes address the
                    # weight with 32-bit offsets; beyond 2^32 elements the scalar route is the one left)
                    assert p.route == (TILE_MFMA if k * n < 1 << 32 else GENERIC)
                elif m > 4:
                    assert p.route in (GEMM_MFMA, TILE_MFMA)
                if f16:
                    assert p.route != GEMV_VALU  # the vector-ALU GEMV reads f32 activations only
                if p.route == GEMV_MFMA:
                    check_gemv(p, fmt, m, k, n)
                elif p.route == GEMM_MFMA:
                    check_gemm(p, fmt, m, k, n, f16)
                elif p.route == TILE_MFMA:
                    check_tile(p, fmt, m, k, n, f16)
            except AssertionError as e:
                raise AssertionError(where) from e
    assert {GEMV_MFMA, GEMM_MFMA, TILE_MFMA} <= routes


def test_baseline_configurations_take_the_kernels_built_for_them():
    gemv = [(Q8, 1, 576, 1536), (Q4, 1, 576, 576), (Q4, 1, 576, 192), (Q4, 1, 576, 3072), (Q4, 1, 1536, 576),
            (Q4, 1, 576, 49152)]
    for fmt in (Q4, Q8):
        for m in (1, 4):
            gemv += [(fmt, m, 4096, 14336), (fmt, m, 14336, 4096)]
    for fmt, m, k, n in gemv:
        assert capi.matmul_plan(fmt, m, k, n).route == GEMV_MFMA, (fmt, m, k, n)
    for fmt in (Q4, Q8):
        # the LDS-resident form is the faster kernel here whatever the activations (one round of workgroups, 4 K parts)
        for promised in (False, True):
            p = capi.matmul_plan(fmt, 16, 4096, 14336, fp16_range=promised)
            assert p.route == TILE_MFMA and p.quads_per_wave == 0 and list(p.grid) == [4, 56, 1]
            p = capi.matmul_plan(fmt, 16, 14336, 4096, fp16_range=promised)   # 14 K parts, still one round
            assert p.route == TILE_MFMA and p.quads_per_wave == 0 and list(p.grid) == [14, 16, 1]
        # elsewhere the 32x32 kernel is ahead, and runs when the activations are fp16 or promised to be in its range
        assert capi.matmul_plan(fmt, 16, 5120, 14336, fp16_range=True).route == GEMM_MFMA  # 0.55 of a round of workgroups
        assert capi.matmul_plan(fmt, 16, 4096, 49152, fp16_range=True).route == TILE_MFMA  # 1.5 rounds, all but full
        assert capi.matmul_plan(fmt, 16, 4096, 4096, fp16_range=True).route == GEMM_MFMA   # a quarter of the CUs
        # 17 rows on 14336 x 4096: two pairs of tiles per wave keep it to one round; Q8 cannot park its quants then
        assert capi.matmul_plan(fmt, 17, 14336, 4096, fp16_range=True).route == (TILE_MFMA if fmt == Q4 else GEMM_MFMA)
        assert capi.matmul_plan(fmt, 17, 8192, 14336, fp16_range=True).route == GEMM_MFMA  # two rounds of workgroups
        assert capi.matmul_plan(fmt, 17, 8192, 4096, fp16_range=True).route == TILE_MFMA   # 8 K parts, one round
        assert capi.matmul_plan(fmt, 17, 4096, 4096, fp16_range=True).route == TILE_MFMA   # two row groups of 16, one round
        assert capi.matmul_plan(fmt, 16, 14336, 4096).route == TILE_MFMA
    big = capi.matmul_plan(Q4, 512, 14336, 4096)   # images of 512 rows x 14336 exceed the 16 MiB workspace: several launches
    assert big.route == TILE_MFMA and big.quads_per_wave > 1
    # prefill with f32 activations (what the reference's Session hands over): row groups on the LDS-resident form,
    # also on a context that was promised the fp16 range (it measured faster than the 32x32 kernel there)
    for promised in (False, True):
        p = capi.matmul_plan(Q4, 512, 1024, 3072, fp16_range=promised)
        assert p.route == TILE_MFMA and p.quads_per_wave == 0 and p.k_parts == 1 and p.grid[2] == 32
    up = capi.matmul_plan(Q4, 512, 1024, 3072, True)  # fp16 activations, C4 up-projection: row groups of 32
    assert up.route == TILE_MFMA and up.quads_per_wave == 0 and up.full_steps == 2 and list(up.grid) == [1, 12, 16]
    down = capi.matmul_plan(Q4, 512, 3072, 1024, True)  # C4 down-projection: three K parts, three quarters of a round
    assert down.route == TILE_MFMA and down.quads_per_wave == 0 and list(down.grid) == [3, 4, 16]
    assert capi.matmul_plan(Q4, 128, 3072, 3072, fp16_range=True).route == GEMM_MFMA  # a second round would stay half empty
    assert capi.matmul_plan(Q8, 512, 1024, 3072, True).route == GEMM_MFMA
    head = capi.matmul_plan(Q4, 1, 4096, 14336)
    assert (head.grid[0], head.threads, head.steps, head.k_splits, head.full_steps) == (256, 896, 8, 1, 1)
    tall = capi.matmul_plan(Q4, 4, 14336, 4096)
    assert tall.k_parts == 4 and tall.workspace_bytes == 3 * 4 * 4096 * 4  # three parts hand their sums to the fourth
    # K = 18944 is 37 steps of 16 blocks: more activation chunks than a workgroup has threads for
    assert capi.matmul_plan(Q4, 1, 18944, 3584).route == GEMV_MFMA
    assert capi.matmul_plan(Q4, 4, 11008, 4096).k_parts >= 2


def test_edge_shapes_of_the_gpu_parity_tests_stay_on_the_gemv_kernel():
    """tests/test_gpu_parity.py::test_small_m_routes skips a route that refuses a shape; these are
    the shapes it lists for the sake of the MFMA GEMV's special cases, so that route must take them."""
    for m, k, n in [(2, 512, 2055), (1, 512, 32774), (4, 14336, 518), (3, 12288, 64), (1, 11008, 132), (2, 11040, 66),
                    (1, 18944, 132), (4, 11008, 260), (3, 13824, 70), (1, 576, 577), (4, 4096, 257), (1, 14336, 64)]:
        for fmt in (Q4, Q8):
            p = capi.matmul_plan(fmt, m, k, n)
            assert p.route == GEMV_MFMA, (fmt, m, k, n)
    assert capi.matmul_plan(Q4, 4, 14336, 518).k_parts > 1
    assert capi.matmul_plan(Q4, 1, 18944, 132).k_parts > 1
    assert capi.matmul_plan(Q4, 1, 11008, 132).full_steps == 0
    assert capi.matmul_plan(Q4, 1, 512, 32774).quads_per_wave == 4
    # lm_head of SmolLM2-135M: 18 blocks = one full step + 2 leftover blocks shared by the wave's four quads
    lm = capi.matmul_plan(Q4, 1, 576, 49152)
    assert (lm.steps, lm.quads_per_wave, lm.tail_blocks, lm.full_steps) == (1, 4, 2, 1)
    assert capi.matmul_plan(Q8, 1, 576, 49152).tail_blocks == 0  # Q8 keeps its two steps
    assert capi.matmul_plan(Q4, 1, 608, 49152).tail_blocks == 0  # 3 leftover blocks do not divide the slots


def test_shapes_no_weight_can_have_are_refused():
    for args in ((Q4, 1, 100, 8), (Q4, 0, 64, 8), (Q4, 1, 0, 8), (Q4, 1, 64, 0), (7, 1, 64, 8)):
        with pytest.raises(capi.MgnError):
            capi.matmul_plan(*args)
