"""GPU parity of the count-sketch kernels against the CPU oracle, through the C-ABI library
(ctypes) and the product classes that wrap it.  Buckets, signs and query results must be bit
exact.  Updates on a plan add in the oracle's order and must be bit exact too; updates without a
plan (float atomics in no fixed order, as in the reference) are compared at 1e-5 relative."""
import ctypes

import numpy as np
import pytest
import torch

from _helpers import assert_close, to_np

pytestmark = pytest.mark.gpu

A, B = 994443, 609478


@pytest.fixture(scope="module")
def lib():
    from conef_amd import _lib
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return _lib.load()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("d,w", [(1, 1), (700, 65), (5760, 1152), (4096, 409), (200_000, 130_000),
                                 (1_300_000, 130_000), (100_000, 1), (300_000, 2 ** 30), (1000, 3)])
def test_device_hash_bit_exact(lib, oracle, d, w):
    bucket = torch.empty(d, dtype=torch.int32, device="cuda")
    sign = torch.empty(d, dtype=torch.int32, device="cuda")
    for (a, b, sa, sb) in [(A, B, A + 2, B + 3), (9171025, 2171464, 9171025 + 8, 2171464 + 7)]:
        rc = lib.conef_hash_table_i32(bucket.data_ptr(), sign.data_ptr(), d, w, a, b, sa, sb, 0)
        assert rc == 0
        torch.cuda.synchronize()
        ob, osg = oracle.hash_table(d, w, a, b, sa, sb)
        np.testing.assert_array_equal(to_np(bucket), ob)
        np.testing.assert_array_equal(to_np(sign), osg)


SHAPES = [  # n, d, sketch_size   (row shape: short rows;  tile shape: long rows)
    (1, 1, 0.5), (3, 17, 0.3), (16, 27, 0.5), (64, 576, 0.2), (7, 650, 0.1), (33, 1024, 0.1),
    (40, 5760, 0.2), (5, 40_003, 0.1), (5, 100_000, 0.1), (2, 65_537, 0.5), (3, 8191, 1.0),
]


@pytest.mark.parametrize("n,d,ss", SHAPES)
def test_query_bit_exact(oracle, n, d, ss):
    from conef_amd.compressors.CountSketch import DenseCS
    rng = np.random.RandomState(n * 7 + d)
    cs = DenseCS(n, d, ss)
    o = oracle.DenseCS(n, d, ss)
    assert cs.range == o.range
    o.cs[:] = rng.randn(n, o.range).astype(np.float32)
    cs.cs.copy_(dev(o.cs))
    x = (rng.randn(n, d) * 1e-3).astype(np.float32)
    xd = dev(x)
    cs.query(xd, 1 - 0.9)
    o.query(x, 1 - 0.9)
    np.testing.assert_array_equal(to_np(xd), x)


@pytest.mark.parametrize("n,d,ss", [(5, 130_000, 0.1), (40, 650, 0.1), (640, 5760, 0.2), (3, 17, 0.3), (7, 4099, 0.25),
                                    (8, 40_000, 0.1), (3, 100_000, 0.2), (1, 65_536, 0.1), (6, 30_002, 0.3)])
def test_query_hashed_and_table_entry_points_agree(oracle, n, d, ss):
    """conef_cs_query_f32 hashes every column, conef_cs_query_planned_f32 reads bucket and sign from the
    plan's table (binned and row-list plans) and, given a binned plan's workspace, gathers the cells of
    all (at most 8) rows of a column at once from an interleaved copy of the sketch: all must give the
    oracle's bits; a plan built for other seeds is refused."""
    from conef_amd import _lib
    from conef_amd._plan import SketchPlan
    lib = _lib.load()
    rng = np.random.RandomState(n + d)
    w = max(int(d * ss), 1)
    cs = (rng.randn(n, w)).astype(np.float32)
    x = (rng.randn(n, d) * 1e-3).astype(np.float32)
    want = x.copy()
    oracle.cs_query(want, cs, np.float32(0.1))
    csd = dev(cs)
    a, b = 994443, 609478
    hashed, table = dev(x), dev(x)
    assert lib.conef_cs_query_f32(hashed.data_ptr(), csd.data_ptr(), n, d, w, 0.1, a, b, 0) == 0
    plan = SketchPlan.shared(n, d, w, a, b, torch.device("cuda", 0))
    assert lib.conef_cs_query_planned_f32(table.data_ptr(), csd.data_ptr(), plan.host_ptr, plan.device.data_ptr(), None,
                                          n, d, w, 0.1, a, b, 0) == 0
    np.testing.assert_array_equal(to_np(hashed), want)
    np.testing.assert_array_equal(to_np(table), want)
    if not plan.in_place:                      # a binned plan has a workspace: the interleaved form where the shape allows
        inter = dev(x)
        assert lib.conef_cs_query_planned_f32(inter.data_ptr(), csd.data_ptr(), plan.host_ptr, plan.device.data_ptr(),
                                              plan.workspace.data_ptr(), n, d, w, 0.1, a, b, 0) == 0
        np.testing.assert_array_equal(to_np(inter), want)
    other = SketchPlan.shared(n, d, w, a, b, torch.device("cuda", 0), sign_seeds=(a + 4, b + 5))
    assert lib.conef_cs_query_planned_f32(table.data_ptr(), csd.data_ptr(), other.host_ptr, other.device.data_ptr(), None,
                                          n, d, w, 0.1, a, b, 0) == -1
    assert lib.conef_cs_query_planned_f32(table.data_ptr(), csd.data_ptr(), plan.host_ptr, plan.device.data_ptr(), None,
                                          n, d, w + 1, 0.1, a, b, 0) == -1


@pytest.mark.parametrize("n,d,ss", SHAPES)
@pytest.mark.parametrize("beta", [0.9, 1.0])
def test_update_parity(oracle, n, d, ss, beta):
    from conef_amd.compressors.CountSketch import DenseCS
    rng = np.random.RandomState(n * 11 + d)
    cs = DenseCS(n, d, ss)
    o = oracle.DenseCS(n, d, ss)
    for step in range(3):                      # state carried across steps
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        cs.update(dev(v), beta)
        o.update(v, beta)
        assert_close(cs.cs, o.cs, what="sketch after update %d" % step)
    cs.clean(0.5)
    o.clean(0.5)
    assert_close(cs.cs, o.cs, what="clean")
    cs.clean(0)
    assert float(cs.cs.abs().max()) == 0.0


def test_update_raw_abi_aliasing_rules(lib):
    n, d, w = 4, 100_000, 10_000           # tile shape: in place is refused
    assert lib.conef_cs_update_inplace_ok(n, d, w) == 0
    v = torch.zeros(n, d, device="cuda")
    cs = torch.zeros(n, w, device="cuda")
    assert lib.conef_cs_update_f32(v.data_ptr(), cs.data_ptr(), cs.data_ptr(), n, d, w, 0.9, A, B, 0) == -1
    assert lib.conef_cs_update_inplace_ok(64, 576, 115) == 1
    assert lib.conef_cs_update_f32(v.data_ptr(), cs.data_ptr(), cs.data_ptr(), n, d, 0, 0.9, A, B, 0) == -1
    assert lib.conef_cs_query_f32(0, cs.data_ptr(), n, d, w, 0.1, A, B, 0) == -1
    assert lib.conef_cs_query_f32(v.data_ptr(), cs.data_ptr(), 0, d, w, 0.1, A, B, 0) == 0   # empty input


def test_exact_recovery_on_device(oracle):
    # W >= m with an injective hash sample: unsketch(sketch(v)) == v bit for bit
    from conef_amd.compressors.CountSketch import DenseCS
    w = 4096
    bucket, _ = oracle.hash_table(600, w)
    d, seen = 0, set()
    while int(bucket[d]) not in seen:
        seen.add(int(bucket[d]))
        d += 1
    cs = DenseCS(2, d, w / d + 1e-9)
    assert cs.range == w
    v = torch.randn(2, d, device="cuda")
    cs.update(v, 1.0)
    x = torch.zeros_like(v)
    cs.query(x, 1.0)
    assert torch.equal(x, v)


@pytest.mark.parametrize("n,d,ss", [(3, 17, 0.3), (64, 576, 0.2), (5, 100_000, 0.1)])
def test_half_sketch_parity(oracle, n, d, ss):
    from conef_amd.compressors.halfCountSketch import DenseCS as HalfCS
    rng = np.random.RandomState(d)
    cs = HalfCS(n, d, ss)
    o = oracle.HalfDenseCS(n, d, ss)
    for step in range(3):
        v = (rng.randn(n, d) * 1e-2).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        got, want = to_np(cs.cs).astype(np.float32), o.cs.astype(np.float32)
        # one fp16 ulp of slack on top of the fp32 tolerance: a value on a rounding boundary may
        # land either side when the fp32 accumulation order differs
        assert np.abs(got - want).max() <= 2 ** -10 * np.abs(want).max()
        o.cs = to_np(cs.cs).copy()           # keep both on the same fp16 state for the next step
    x = (rng.randn(n, d) * 1e-2).astype(np.float32)
    xd = dev(x)
    cs.query(xd, 0.1)
    o.query(x, 0.1)
    np.testing.assert_array_equal(to_np(xd), x)
    cs.clean(0.5)
    o.clean(0.5)
    np.testing.assert_array_equal(to_np(cs.cs), o.cs)


@pytest.mark.parametrize("n,d,ss", [(3, 17, 0.3), (64, 576, 0.2), (5, 50_000, 0.1), (641, 1028, 0.2), (1, 4096, 0.1)])
def test_hash3_parity(oracle, n, d, ss):
    from conef_amd.compressors.CountSketchHash3 import DenseCSHash3
    rng = np.random.RandomState(d + 1)
    cs = DenseCSHash3(n, d, ss)
    o = oracle.DenseCSHash3(n, d, ss)
    for step in range(3):
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        for k, (g, want) in enumerate(zip((cs.cs0, cs.cs1, cs.cs2), (o.cs0, o.cs1, o.cs2))):
            assert_close(g, want, what="cs%d step %d" % (k, step))
        for g, want in zip((cs.cs0, cs.cs1, cs.cs2), (o.cs0, o.cs1, o.cs2)):
            want[:] = to_np(g)                 # same state on both sides before the query
    x = (rng.randn(n, d) * 1e-3).astype(np.float32)
    xd = dev(x)
    cs.query(xd, 0.1)
    o.query(x, 0.1)
    np.testing.assert_array_equal(to_np(xd), x)


@pytest.mark.parametrize("n,d,ss", [(3, 17, 0.3), (64, 576, 0.2), (640, 5760, 0.2), (5, 50_000, 0.1), (2100, 650, 0.1),
                                    (1, 1, 0.5), (7, 24_576, 0.05)])
def test_hash3_update_on_plans_is_bit_exact(oracle, n, d, ss):
    """With a plan per sketch the three-hash update has no atomics: every cell receives the
    serial definition's terms in its order, so all three sketches match the oracle bit for bit,
    step after step."""
    from conef_amd.compressors.CountSketchHash3 import DenseCSHash3
    rng = np.random.RandomState(n + d)
    cs = DenseCSHash3(n, d, ss)
    assert cs.plans() is not None and len(cs.plans()) == 3
    o = oracle.DenseCSHash3(n, d, ss)
    for step in range(3):
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        for k, (g, want) in enumerate(zip((cs.cs0, cs.cs1, cs.cs2), (o.cs0, o.cs1, o.cs2))):
            np.testing.assert_array_equal(to_np(g), want, err_msg="cs%d step %d" % (k, step))


def test_hash3_without_plans_uses_atomics(oracle, monkeypatch):
    from conef_amd.compressors.CountSketchHash3 import DenseCSHash3
    monkeypatch.setenv("CONEF_PLAN", "0")
    rng = np.random.RandomState(3)
    n, d, ss = 6, 3000, 0.2
    cs = DenseCSHash3(n, d, ss)
    assert cs.plans() is None
    o = oracle.DenseCSHash3(n, d, ss)
    v = (rng.randn(n, d) * 1e-3).astype(np.float32)
    cs.update(dev(v), 0.9)
    o.update(v, 0.9)
    for g, want in zip((cs.cs0, cs.cs1, cs.cs2), (o.cs0, o.cs1, o.cs2)):
        assert_close(g, want, what="atomic three-hash update")


def test_state_dict_round_trip():
    from conef_amd.compressors.CountSketch import DenseCS
    cs = DenseCS(4, 100, 0.2)
    cs.update(torch.randn(4, 100, device="cuda"), 0.9)
    sd = cs.state_dict()
    other = DenseCS(4, 100, 0.2)
    other.load_state_dict(sd)
    assert torch.equal(other.cs, cs.cs)
    with pytest.raises(ValueError):
        DenseCS(4, 101, 0.2).load_state_dict(sd)


def test_rejects_host_tensors():
    from conef_amd.compressors.CountSketch import DenseCS
    cs = DenseCS(2, 10, 0.5)
    with pytest.raises(ValueError):
        cs.update(torch.zeros(2, 10), 0.9)
    with pytest.raises(ValueError):
        cs.query(torch.zeros(2, 11, device="cuda"), 0.1)


# ---- long rows: the planned (atomic-free) path is deterministic and follows the oracle's order ----

PLANNED_SHAPES = [  # (n, d, sketch_size, kind): 0 = binned long rows, 1 = row lists, 2 = row lists in column panels
    (5, 40_003, 0.1, 0), (5, 100_000, 0.1, 0), (2, 65_537, 0.5, 0), (1, 300_001, 0.05, 0), (8, 30_000, 0.9, 0), (5, 24_577, 0.004, 0),
    (8, 20_000, 0.9, 0), (3, 8191, 1.0, 1), (8, 20_000, 0.05, 1), (1, 1, 0.5, 1), (3, 17, 0.3, 1), (64, 576, 0.2, 1), (40, 5760, 0.2, 1),
    (2100, 650, 0.1, 1), (4099, 1024, 0.1, 1), (7, 24_576, 0.05, 1), (33, 1023, 2.0, 1), (20_000, 66, 0.1, 1),
    # long rows and more than 8 of them (the reference kernel takes any N and D, CountSketch.py:27-67,143-158):
    # the binned passes over groups of 8 rows (a last group of 1..7), and the panels for tall matrices
    (16, 50_000, 0.1, 0), (9, 100_000, 0.1, 0), (11, 40_003, 0.1, 0), (64, 200_000, 0.1, 0), (23, 30_002, 0.9, 0),
    (600, 25_088, 0.1, 2), (257, 30_001, 0.4, 2), (1030, 40_000, 0.01, 2), (513, 24_578, 0.5, 2)]


@pytest.mark.parametrize("n,d,ss,kind", PLANNED_SHAPES)
def test_planned_update_bit_exact(oracle, n, d, ss, kind):
    from conef_amd.compressors.CountSketch import DenseCS
    rng = np.random.RandomState(d)
    cs = DenseCS(n, d, ss)
    assert cs.plan() is not None and cs.plan().kind == kind
    o = oracle.DenseCS(n, d, ss)
    for step in range(3):
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        np.testing.assert_array_equal(to_np(cs.cs), o.cs)


@pytest.mark.parametrize("n,d,ss", [(2100, 650, 0.1), (33, 1023, 0.3), (64, 576, 0.2), (1, 2, 0.5), (3, 5, 0.5)])
def test_planned_update_unaligned_start(oracle, n, d, ss):
    """Row lists read a tile as one flat run; the tensor may start 4, 8 or 12 bytes past a 16-byte
    boundary (a parameter in the middle of a bucket)."""
    from conef_amd.compressors.CountSketch import DenseCS
    rng = np.random.RandomState(n + d)
    cs = DenseCS(n, d, ss)
    o = oracle.DenseCS(n, d, ss)
    for off in (1, 2, 3):
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        arena = torch.zeros(n * d + 8, device="cuda")
        vd = arena[off:off + n * d].view(n, d)
        vd.copy_(dev(v))
        cs.update(vd, 0.9)
        o.update(v, 0.9)
        np.testing.assert_array_equal(to_np(cs.cs), o.cs)
        np.testing.assert_array_equal(to_np(vd), v)                       # the input is only read


@pytest.mark.parametrize("chunk,tbin", [(1024, 64), (2048, 512), (8192, 256), (4096, 128)])
def test_planned_update_any_tiling(oracle, monkeypatch, chunk, tbin):
    from conef_amd.compressors.CountSketch import DenseCS
    monkeypatch.setenv("CONEF_PLAN_CHUNK", str(chunk))
    monkeypatch.setenv("CONEF_PLAN_BIN", str(tbin))
    n, d, ss = 5, 130_001, 0.1
    cs = DenseCS(n, d, ss)
    h = cs.plan().header()
    assert (h["chunk_cols"], h["bin_buckets"]) == (chunk, tbin)
    o = oracle.DenseCS(n, d, ss)
    v = (np.random.RandomState(1).randn(n, d) * 1e-3).astype(np.float32)
    for _ in range(2):
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
    np.testing.assert_array_equal(to_np(cs.cs), o.cs)


@pytest.mark.parametrize("n,d,ss", [(3, 17, 0.3), (64, 576, 0.2), (2100, 650, 0.1), (40, 5760, 0.2)])
def test_unplanned_row_kernels_still_match(oracle, monkeypatch, n, d, ss):
    """The entry points that take no plan (one wavefront per row, LDS atomics) stay in the library."""
    from conef_amd.compressors.CountSketch import DenseCS
    monkeypatch.setenv("CONEF_PLAN", "0")
    cs = DenseCS(n, d, ss)
    assert cs.plan() is None
    o = oracle.DenseCS(n, d, ss)
    rng = np.random.RandomState(n)
    for _ in range(2):
        v = (rng.randn(n, d) * 1e-3).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        assert_close(cs.cs, o.cs, what="row kernel without a plan")


@pytest.mark.parametrize("n,d,ss", [(3, 17, 0.3), (64, 576, 0.2), (2100, 650, 0.1)])
def test_half_sketch_on_a_plan_bit_exact(oracle, n, d, ss):
    from conef_amd.compressors.halfCountSketch import DenseCS as HalfCS
    cs = HalfCS(n, d, ss)
    assert cs.plan() is not None
    o = oracle.HalfDenseCS(n, d, ss)
    rng = np.random.RandomState(d)
    for _ in range(3):
        v = (rng.randn(n, d) * 1e-2).astype(np.float32)
        cs.update(dev(v), 0.9)
        o.update(v, 0.9)
        np.testing.assert_array_equal(to_np(cs.cs), o.cs)


def test_atomic_fallback_still_matches(oracle, monkeypatch):
    from conef_amd.compressors.CountSketch import DenseCS
    monkeypatch.setenv("CONEF_PLAN", "0")
    n, d, ss = 5, 100_000, 0.1
    cs = DenseCS(n, d, ss)
    assert cs.plan() is None
    o = oracle.DenseCS(n, d, ss)
    v = (np.random.RandomState(2).randn(n, d) * 1e-3).astype(np.float32)
    cs.update(dev(v), 0.9)
    o.update(v, 0.9)
    assert_close(cs.cs, o.cs, what="atomic path")
    big = DenseCS(12, 100_000, 0.1)          # the same kernel at 12 rows, where a plan would have been found
    assert big.plan() is None
    ob = oracle.DenseCS(12, 100_000, 0.1)
    v = (np.random.RandomState(3).randn(12, 100_000) * 1e-3).astype(np.float32)
    big.update(dev(v), 0.9)
    ob.update(v, 0.9)
    assert_close(big.cs, ob.cs, what="atomic path, 12 rows")


def test_a_shape_without_a_plan_says_so_once(monkeypatch, caplog):
    """No shape falls back to float atomics silently: a sketch that finds no plan logs a warning,
    once per shape."""
    import logging
    from conef_amd.compressors import CountSketch
    monkeypatch.setattr(CountSketch.SketchPlan, "applicable", staticmethod(lambda *a, **k: False))
    CountSketch._WARNED.discard((6, 3000, 600))
    with caplog.at_level(logging.WARNING):
        for _ in range(3):
            cs = CountSketch.DenseCS(6, 3000, 0.2)
            assert cs.plan() is None
    hits = [r for r in caplog.records if "float atomics" in r.getMessage()]
    assert len(hits) == 1 and "[6, 3000]" in hits[0].getMessage()


def test_full_vgg_fc_layer_on_panels_bit_exact(oracle):
    """[4096, 25088] (the first fully connected layer of VGG-16): a row is too long for whole row
    lists, the matrix tall enough for the panels."""
    from conef_amd.compressors.CountSketch import DenseCS
    n, d, ss = 4096, 25_088, 0.1
    cs = DenseCS(n, d, ss)
    assert cs.plan() is not None and cs.plan().kind == 2
    o = oracle.DenseCS(n, d, ss)
    gen = torch.Generator(device="cuda").manual_seed(9)
    for step in range(2):
        v = torch.randn(n, d, generator=gen, device="cuda") * 1e-3
        cs.update(v, 0.9)
        o.update(to_np(v), 0.9)
        np.testing.assert_array_equal(to_np(cs.cs), o.cs)


@pytest.mark.parametrize("n,d,ss,kind", [(600, 25_088, 0.1, 2), (257, 30_001, 0.4, 2), (16, 50_000, 0.1, 0),
                                         (9, 100_000, 0.1, 0), (19, 40_003, 0.3, 0)])
def test_randblock_step_on_panels_and_row_groups_bit_exact(oracle, n, d, ss, kind):
    """The fused RandomBlock + sketch step (RandomBlock_hook.py:190,216-243,272-280) on the plans for
    long rows of a matrix with more than 8 of them: block, zeros, payload and the new sketch against
    the oracle's fused step, bit for bit, with a block that wraps around the end and one that does not."""
    from conef_amd.compressors.CountSketch import DenseCS
    rng = np.random.RandomState(n + d)
    cs = DenseCS(n, d, ss)
    assert cs.plan() is not None and cs.plan().kind == kind
    ocs = np.zeros((n, cs.range), np.float32)
    numel = n * d
    block = max(1, int(0.1 * numel))
    for step, start in enumerate([numel - block // 3, 12_345, 7 * d + 3]):
        x = (rng.randn(n, d) * 1e-3).astype(np.float32)
        xd = dev(x)
        payload = torch.empty(block, device="cuda")
        cs.randblock_step(xd, payload, start, block, 1 - 0.9, 0.9)
        opay = np.empty(block, np.float32)
        oracle.randblock_conef_step(x, ocs, opay, start, block, 1 - 0.9, 0.9)
        np.testing.assert_array_equal(to_np(xd), x, err_msg="decompressed gradient, step %d" % step)
        np.testing.assert_array_equal(to_np(payload), opay, err_msg="payload, step %d" % step)
        np.testing.assert_array_equal(to_np(cs.cs), ocs, err_msg="sketch, step %d" % step)
