"""CPU-only checks of the native boundary: the library is built in-tree, loads, exports every
entry point include/conef_hip.h declares with the arity the Python binding uses, rejects bad
arguments before touching a GPU, and its hash (compiled for the host from the same source the
kernels use) agrees with the oracle bit for bit.  No device compute is called here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "conef_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|int64_t)\s+(conef_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args == "void" else len([a for a in args.split(",") if a.strip()])
    return out


@pytest.fixture(scope="module")
def lib():
    from conef_amd import _lib
    return _lib.load()


def test_header_library_and_binding_agree(lib):
    from conef_amd import _lib
    decl = declared_functions()
    assert len(decl) >= 30
    assert set(decl) == set(_lib.SIGNATURES), set(decl) ^ set(_lib.SIGNATURES)
    raw = ctypes.CDLL(_lib.LIBPATH)
    for name, nargs in decl.items():
        assert hasattr(raw, name), "library does not export %s" % name
        assert nargs == len(_lib.SIGNATURES[name]), name
    assert lib.conef_version() == 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from conef_amd import _lib
    monkeypatch.setattr(_lib, "_handle", None)
    monkeypatch.setattr(_lib, "LIBPATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.ConefLibraryError, match="no CPU fallback"):
        _lib.load()


def test_argument_validation_without_gpu(lib):
    # all of these are refused on the host before any launch
    assert lib.conef_cs_query_f32(1, 1, 1, 1, 0, 0.1, 1, 1, 0) == -1            # w < 1
    assert lib.conef_cs_query_f32(0, 0, 2, 2, 4, 0.1, 1, 1, 0) == -1            # null pointers
    assert lib.conef_cs_update_f32(1, 1, 1, -1, 1, 1, 0.9, 1, 1, 0) == -1
    assert lib.conef_randblock_ef_step_f32(1, 1, 1, 10, 10, 1, 0) == -1         # start == numel
    assert lib.conef_randblock_ef_step_f32(1, 1, 1, 10, 0, 11, 0) == -1         # block > numel
    assert lib.conef_randblock_unbiased_step_f32(1, 1, 10, 0, 1, 0.0, 0) == -1  # prob must be > 0
    assert lib.conef_gram_schmidt_f32(1, 10, 33, 0.0, 0, 0, 0) == -1            # rank above 32
    assert lib.conef_gram_schmidt_f32(1, 100_000, 8, 0.0, 0, 0, 0) == -1        # too large for LDS: needs the workspace
    assert lib.conef_psgd_mtp_f32(1, 1, 1, 640, 5760, 4, 0, 0, 0) == -1         # several row slabs: needs the workspace
    assert lib.conef_psgd_workspace_bytes(640, 5760, 4) >= 4 * 5760 * 4
    assert lib.conef_psgd_workspace_bytes(0, 5, 1) == -1
    assert lib.conef_psgd_mq_f32(1, 1, 1, 4, 4, 0, 0, 0, 0) == -1
    assert lib.conef_topk_sparsify_f32(1, 100, 10, 0, 0, 0) == -1               # no workspace
    assert lib.conef_topk_sparsify_f32(1, 100, 100, 0, 0, 0) == 0               # k >= numel: nothing to do
    assert lib.conef_topk_workspace_bytes(1 << 20) >= 4 * 1024
    # the round that orthogonalises the next round's Q factors: its flags need the second buffers and the answer slot
    from conef_amd import _lib
    items = (_lib.PsgdItem * 1)()
    made = ctypes.c_int32(7)
    assert lib.conef_psgd_round_ahead_f32(items, 1, 0, 0, 0.0, 0.0, 0.0, 1, 1, None, 2, ctypes.byref(made), 0, 0, 0) == -1
    assert made.value == 0
    assert lib.conef_psgd_round_ahead_f32(items, 1, 0, 0, 0.0, 0.0, 0.0, 1, 1, None, 1, None, 0, 0, 0) == -1
    assert lib.conef_psgd_round_ahead_f32(items, 0, 0, 0, 0.0, 0.0, 0.0, 1, 1, None, 0, None, 0, 0, 0) == 0     # empty bucket
    assert lib.conef_psgd_round_ahead_f32(items, 1, 0, 4, 0.0, 0.0, 0.0, 1, 1, None, 0, None, 0, 0, 0) == -1    # pqt_mode
    # the one-call-per-bucket random-block step: every item is checked before anything is enqueued
    rb = (_lib.RandBlockItem * 2)()
    for it in rb:
        it.x, it.payload, it.err, it.n, it.m, it.start, it.block = 1, 1, 1, 4, 10, 3, 4
    assert lib.conef_randblock_step_batch_f32(rb, 2, 3, 0.1, 0.9, 1, 1, 0) == -1        # unknown mode
    assert lib.conef_randblock_step_batch_f32(rb, -1, 0, 0.1, 0.9, 1, 1, 0) == -1
    assert lib.conef_randblock_step_batch_f32(None, 1, 0, 0.1, 0.9, 1, 1, 0) == -1
    assert lib.conef_randblock_step_batch_f32(rb, 0, 1, 0.1, 0.9, 1, 1, 0) == 0         # a bucket without matrices
    rb[1].start = 40
    assert lib.conef_randblock_step_batch_f32(rb, 2, 0, 0.1, 0.9, 1, 1, 0) == -1        # start == numel in the second item
    rb[1].start, rb[1].err = 3, None
    assert lib.conef_randblock_step_batch_f32(rb, 2, 1, 0.1, 0.9, 1, 1, 0) == -1        # dense mode without an error tensor
    assert lib.conef_randblock_step_batch_f32(rb, 2, 2, 0.1, 0.9, 1, 1, 0) == -1        # sketched mode without sketches
    # the top-k entry point that allocates nothing: argument checks come before any device call
    assert lib.conef_topk_sparsify_noalloc_f32(1, 1 << 32, 10, 0) == -2                 # beyond its stated maximum
    assert lib.conef_topk_sparsify_noalloc_f32(1, 100, 0, 0) == -1
    assert lib.conef_topk_sparsify_noalloc_f32(None, 100, 10, 0) == -1
    assert lib.conef_topk_sparsify_noalloc_f32(1, 100, 100, 0) == 0                     # k >= numel: nothing to do
    with pytest.raises(ValueError, match="stated maximum"):
        _lib.check(-2, "conef_topk_sparsify_noalloc_f32")
    # shapes: short rows may update in place, the flat 25 MB bucket may not
    assert lib.conef_cs_update_inplace_ok(640, 5760, 1152) == 1
    assert lib.conef_cs_update_inplace_ok(5, 1_300_000, 130_000) == 0


@pytest.mark.parametrize("d,w", [(1, 1), (1000, 7), (70_000, 65), (5760, 1152), (200_000, 130_000),
                                 (100_000, 1 << 30), (300_000, 3), (65_536, 2), (50_000, 99_991)])
def test_shipped_hash_matches_oracle_on_host(lib, oracle, d, w):
    for (a, b, sa, sb) in [(994443, 609478, 994445, 609481), (4113759, 2949676, 4113763, 2949681),
                           (9171025, 2171464, 9171033, 2171468), (9171025, 2171464, 9171033, 2171471)]:
        bucket = np.empty(d, np.int32)
        sign = np.empty(d, np.int32)
        assert lib.conef_hash_table_host_i32(bucket.ctypes.data, sign.ctypes.data, d, w, a, b, sa, sb) == 0
        ob, osg = oracle.hash_table(d, w, a, b, sa, sb)
        np.testing.assert_array_equal(bucket, ob)
        np.testing.assert_array_equal(sign, osg)


def test_fast_modulo_near_multiples(lib, oracle):
    # widths chosen so that many hash values sit next to a multiple of w, where a quotient
    # estimated in floating point is most likely to be off by one
    for w in (1, 2, 3, 7, 1000, 65_535, 65_536, 65_537, (1 << 30) - 1, 1 << 30):
        d = 20_000
        bucket = np.empty(d, np.int32)
        sign = np.empty(d, np.int32)
        assert lib.conef_hash_table_host_i32(bucket.ctypes.data, sign.ctypes.data, d, w, 1, 0, 3, 5) == 0
        ob, osg = oracle.hash_table(d, w, 1, 0, 3, 5)
        np.testing.assert_array_equal(bucket, ob)
        np.testing.assert_array_equal(sign, osg)


def test_states_and_host_logic_need_no_gpu():
    from conef_amd.RandomBlock_hook import RandomBlockState
    from conef_amd.UnbiasedRandomBlock_hook import UnbiasedRandomBlockState
    from conef_amd.hPowerSGD_hook import hPowerSGDState
    from conef_amd.powerSGD_hook import PowerSGDState, _should_compress
    with pytest.raises(ValueError, match="Expect `start_compression_iter` > 1"):
        RandomBlockState(None, start_compression_iter=1)
    with pytest.raises(ValueError, match="Expect `use_error_feedback` = True if `use_error_compression`"):
        RandomBlockState(None, start_compression_iter=2, use_error_feedback=False, use_error_compression=True)
    with pytest.raises(ValueError, match="Expect `start_compression_iter` > 1"):
        UnbiasedRandomBlockState(None, start_compression_iter=1)
    for cls in (PowerSGDState, hPowerSGDState):
        with pytest.raises(ValueError, match="Expect `start_powerSGD_iter` > 1"):
            cls(None, start_powerSGD_iter=1)
        cls(None, start_powerSGD_iter=1, use_error_feedback=False, warm_start=False)
    s = RandomBlockState(None, start_compression_iter=2)
    assert (s.compression_ratio, s.beta, s.sketch_size, s.use_error_feedback, s.use_error_compression) == \
        (0.1, 0.9, 0.5, True, False)
    assert [int(s.rng.choice(6_500_000)) for _ in range(2)] == [6413414, 6423388]
    # the hooks draw block offsets with randint(0, n): the stream choice(n) draws from for an int n
    # (RandomBlock_hook.py:218, UnbiasedRandomBlock_hook.py:157), on every size class of the generator
    a, b = np.random.RandomState(42), np.random.RandomState(42)
    sizes = [6_500_000, 33278 * 650, 2600 * 650, 17, 1, 2, 255, 256, 65_536, 2 ** 31 - 1, 2 ** 31 + 5, 2 ** 33 + 1] * 20
    assert [int(a.choice(n)) for n in sizes] == [int(b.randint(0, n)) for n in sizes]
    p = PowerSGDState(None, start_powerSGD_iter=2)
    assert (p.matrix_approximation_rank, p.min_compression_rate, p.warm_start, p.beta, p.sketch_size) == \
        (1, 2, True, 0.9, 0.5)
    assert int(p.rng.randint(1_000_000_000)) == 209652396
    assert hPowerSGDState(None, start_powerSGD_iter=2).topk_ratio == 0.4
    # BERT's [2,1024] pooler-adjacent weight is not worth compressing at rank 8, [1024,1024] is
    assert _should_compress(2, 1024, 2, 2) == (False, 2048, 2052)
    assert _should_compress(1024, 1024, 8, 2)[0] is True
    assert p.compression_stats() == (0, 0, 0)


def test_hooks_refuse_host_tensors():
    import torch
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from _helpers import FakeGradBucket
    from conef_amd.RandomBlock_hook import RandomBlock_hook, RandomBlockState
    from conef_amd.powerSGD_hook import PowerSGDState, powerSGD_hook
    st = RandomBlockState(None, start_compression_iter=2)
    g = torch.zeros(40)
    out = RandomBlock_hook(st, FakeGradBucket(g, [(4, 10)])).wait()      # warm-up: identity all-reduce
    assert out is g and st.iter == 1
    st.iter = 2
    with pytest.raises(ValueError, match="no CPU path"):
        RandomBlock_hook(st, FakeGradBucket(g, [(4, 10)]))
    ps = PowerSGDState(None, start_powerSGD_iter=2)
    ps.iter = 2
    with pytest.raises(ValueError, match="no CPU path"):
        powerSGD_hook(ps, FakeGradBucket(g, [(4, 10)]))


def test_plans_are_shared_and_released():
    """One plan per (shape, seeds, tiling, device), however many sketches ask for it; release()
    drops the pool without invalidating a plan somebody still holds."""
    import torch
    import conef_amd
    from conef_amd import _pools
    from conef_amd._plan import SketchPlan
    conef_amd.release()
    cpu = torch.device("cpu")
    p1 = SketchPlan.shared(40, 650, 65, 994443, 609478, cpu)
    p2 = SketchPlan.shared(40, 650, 65, 994443, 609478, cpu)
    p3 = SketchPlan.shared(40, 650, 65, 994443, 609478, cpu, sign_seeds=(7, 9))
    p4 = SketchPlan.shared(5, 130_000, 13_000, 994443, 609478, cpu)
    assert p1 is p2 and p3 is not p1
    assert p1.kind == SketchPlan.ROWLIST and p1.workspace_bytes == 0
    assert p4.kind == SketchPlan.BINNED and p4.workspace_bytes >= 4 * 5 * 130_000
    held = _pools.held_bytes()
    assert held["plans"] == p1.device.numel() + p3.device.numel() + p4.device.numel() and held["staging"] == 0
    with pytest.raises(ValueError):       # long rows in more groups of 8 than a grid dimension holds: no plan
        SketchPlan.shared(8 * 65536, 100_000, 100_000, 994443, 609478, cpu)
    with pytest.raises(ValueError):                                       # ... remembered, not rebuilt
        SketchPlan.shared(8 * 65536, 100_000, 100_000, 994443, 609478, cpu)
    conef_amd.release()
    assert _pools.held_bytes()["plans"] == 0
    assert p1.header()["w"] == 65                                        # still valid for its holder
    assert SketchPlan.shared(40, 650, 65, 994443, 609478, cpu) is not p1


def test_threaded_oracle_step_is_the_single_threaded_one(oracle):
    """The CPU baseline spreads the sketch rows over host threads: same bits as the fused C step."""
    rng = np.random.RandomState(3)
    n, m, w, block = 5, 20_000, 2_000, 9_000
    x0 = (rng.randn(n, m) * 1e-3).astype(np.float32)
    cs_a = (rng.randn(n, w) * 1e-3).astype(np.float32)
    cs_b = cs_a.copy()
    for start in (95_000, 12_345):              # one block that wraps, one that does not
        xa, xb = x0.copy(), x0.copy()
        pa, pb = np.empty(block, np.float32), np.empty(block, np.float32)
        oracle.randblock_conef_step(xa, cs_a, pa, start, block, 0.1, 0.9)
        oracle.randblock_conef_step_threaded(xb, cs_b, pb, start, block, 0.1, 0.9, threads=3)
        np.testing.assert_array_equal(xa, xb)
        np.testing.assert_array_equal(pa, pb)
        np.testing.assert_array_equal(cs_a, cs_b)


def test_one_launch_round_qualification_and_workspace(lib):
    """Which buckets the one-launch PowerSGD round takes, and the records it asks workspace for: host
    logic, nothing is launched (the pointers are never followed without a plan to check)."""
    import ctypes
    from conef_amd._lib import PsgdItem

    def items_for(shapes, rank):
        arr = (PsgdItem * len(shapes))()
        for k, (n, m) in enumerate(shapes):
            arr[k].x = arr[k].err = arr[k].p = arr[k].q = 256 * (k + 1)     # non-null, 16-byte aligned, never followed
            arr[k].n, arr[k].m, arr[k].r = n, m, min(rank, n, m)
        return arr

    def slices(n, m):
        s = 1 if n * m <= 10240 else min(-(-n * m // 4608), 16, n)
        rows_per = -(-n // s)
        return -(-n // rows_per)

    def records(n, m, r):
        s = slices(n, m)
        return 0 if s == 1 else -(-(n * r + s * r * m) // 32) * 32

    small = [(16, 27), (32, 288), (10, 64)]
    arr = items_for(small, 2)
    assert lib.conef_psgd_round_small_fits(arr, len(small), 0, 0, 994443, 609478) == 1
    assert lib.conef_psgd_round_small_fits(arr, len(small), 1, 1, 994443, 609478) == 1
    assert lib.conef_psgd_round_small_fits(arr, len(small), 2, 2, 994443, 609478) == 0     # no sketch, no plan
    assert lib.conef_psgd_round_small_fits(arr, len(small), 2, 1, 994443, 609478) == 0     # modes 2 come together
    assert lib.conef_psgd_round_small_workspace_bytes(arr, len(small)) == 0
    sliced = [(64, 576), (64, 288), (37, 301), (16, 2304), (20, 2000)]
    arr = items_for(sliced, 2)
    assert lib.conef_psgd_round_small_fits(arr, len(sliced), 1, 1, 994443, 609478) == 1
    assert lib.conef_psgd_round_small_workspace_bytes(arr, len(sliced)) == 8 * sum(records(n, m, 2) for n, m in sliced)
    assert lib.conef_psgd_batch_workspace_bytes(arr, len(sliced)) >= lib.conef_psgd_round_small_workspace_bytes(arr, len(sliced))
    # beyond sixteen slices' worth of elements, above rank 8, more than 24 matrices, more than 128 workgroups
    assert lib.conef_psgd_round_small_fits(items_for([(128, 577)], 2), 1, 0, 0, 994443, 609478) == 0
    assert lib.conef_psgd_round_small_fits(items_for([(64, 64)], 16), 1, 0, 0, 994443, 609478) == 0
    assert lib.conef_psgd_round_small_fits(items_for([(8, 8)] * 25, 2), 25, 0, 0, 994443, 609478) == 0
    assert lib.conef_psgd_round_small_fits(items_for([(64, 1024)] * 10, 2), 10, 0, 0, 994443, 609478) == 0
    assert lib.conef_psgd_round_small_fits(items_for([(64, 1024)] * 8, 2), 8, 0, 0, 994443, 609478) == 1
    # a slice that does not fit LDS with its factors: one row of 30000 columns
    assert lib.conef_psgd_round_small_fits(items_for([(2, 30000)], 2), 1, 0, 0, 994443, 609478) == 0
    # the round itself refuses what does not qualify, and a workspace that is too small, before any launch
    arr = items_for(sliced, 2)
    assert lib.conef_psgd_round_small_f32(arr, len(sliced), 1, 1, 0.0, 0.0, 0.0, 994443, 609478, None, 0, None) != 0
    assert lib.conef_psgd_round_small_f32(items_for([(128, 577)], 2), 1, 0, 0, 0.0, 0.0, 0.0, 994443, 609478, None, 0, None) != 0
