"""Pins the CPU oracle (oracle/conef_oracle.c) before anything is compared with it.

The reference ships no tests and no golden vectors, and its sketch kernels need CuPy/NVRTC, so
each oracle function is pinned by (a) known answers derived independently of the C code,
(b) brute force with an explicit dense signed selection matrix in float64, and (c) special
cases the mathematics fixes.  Each check is chosen so that a plausible slip (logical instead of
arithmetic shift, sign taken before the modulo, decay applied once per bucket instead of once
per colliding element, transposed operand) fails it.
"""
import json
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
A, B = 994443, 609478


# ------------------------------------------------------------------- hash --

def test_hash_known_answers_survey(oracle):
    # CountSketch.py:7-18 with (a,b) = (994443, 609478): values worked out by hand-independent
    # arithmetic when the reference was surveyed.
    pre = [1551950793, 1023706841, 849916109, 1606745146, 761103557, 1492328880, 551956319, 185564866]
    mod = [10793, 86841, 106109, 75146, 83557, 58880, 106319, 54866]
    sign_bits = [0, 1, 0, 1, 0, 1, 1, 1]
    assert [oracle.mix(i) for i in range(8)] == pre
    assert [oracle.hash_bucket(i, 130000) for i in range(8)] == mod
    assert [oracle.hash_bucket(i, 130000, A + 2, B + 3) & 1 for i in range(8)] == sign_bits
    bucket, sign = oracle.hash_table(8, 130000)
    assert bucket.tolist() == mod
    assert sign.tolist() == [1 if s else -1 for s in sign_bits]


def test_hash_golden_file(oracle):
    kat = json.load(open(os.path.join(HERE, "golden", "hash_kat.json")))
    for name, s in kat["seeds"].items():
        for v, pre in zip(kat["values"], s["mix"]):
            assert oracle.mix(v, s["a"], s["b"]) == pre, (name, v)
        for w in kat["widths"]:
            for v, want in zip(kat["values"], s["mod"][str(w)]):
                assert oracle.hash_bucket(v, w, s["a"], s["b"]) == want, (name, v, w)


def test_hash_not_textbook_fmix32(oracle):
    # With logical shifts (murmur3 fmix32) the value for i=1 would differ; the reference's
    # signed `h` makes the shifts arithmetic.
    def fmix_logical(v):
        h = (A * v + B) & 0xFFFFFFFF
        h ^= h >> 16
        h = (h * 0x85EBCA6B) & 0xFFFFFFFF
        h ^= h >> 13
        h = (h * 0xC2B2AE35) & 0xFFFFFFFF
        h ^= h >> 16
        return h
    diffs = sum(fmix_logical(i) != oracle.mix(i) for i in range(64))
    assert diffs > 0


def test_hash_invariants(oracle):
    rng = np.random.RandomState(7)
    for w in (1, 2, 65, 130000, 2 ** 30):
        for v in rng.randint(0, 2 ** 31 - 1, size=2000):
            h = oracle.mix(int(v))
            assert h >= 0
            assert 0 <= oracle.hash_bucket(int(v), w) < w
    bucket, sign = oracle.hash_table(500, 1)
    assert (bucket == 0).all() and (sign == -1).all()      # W=1: every sign bit is 0


def test_median3(oracle):
    import itertools
    for trip in itertools.permutations([-1.5, 0.25, 3.0]):
        assert oracle.median3(*trip) == 0.25
    assert oracle.median3(2.0, 2.0, -1.0) == 2.0


# ------------------------------------------------------------ count sketch --

def dense_selection(d, w, oracle, a=A, b=B, sa=None, sb=None):
    bucket, sign = oracle.hash_table(d, w, a, b, sa, sb)
    S = np.zeros((d, w), dtype=np.float64)
    S[np.arange(d), bucket] = sign
    return S


@pytest.mark.parametrize("n,d,w", [(3, 17, 5), (1, 64, 64), (4, 33, 1), (2, 40, 7)])
def test_query_against_dense_matrix(oracle, n, d, w):
    rng = np.random.RandomState(n * 100 + d)
    x0 = rng.randn(n, d).astype(np.float32)
    cs = rng.randn(n, w).astype(np.float32)
    alpha = np.float32(0.1)
    S = dense_selection(d, w, oracle)
    want = x0.astype(np.float64) + float(alpha) * cs.astype(np.float64) @ S.T
    x = x0.copy()
    oracle.cs_query(x, cs, alpha)
    np.testing.assert_allclose(x, want, rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("n,d,w,beta", [(3, 17, 5, 0.9), (2, 64, 9, 0.5), (4, 33, 1, 0.9), (2, 50, 50, 0.0)])
def test_update_against_dense_matrix(oracle, n, d, w, beta):
    # cs' = cs * (1 - (1-beta) * c) + V S, c_j = number of columns hashing to j: the decay is
    # applied once per colliding element (CountSketch.py:63-64), not once per bucket.
    rng = np.random.RandomState(n * 1000 + d + w)
    v = rng.randn(n, d).astype(np.float32)
    cs0 = rng.randn(n, w).astype(np.float32)
    S = dense_selection(d, w, oracle)
    c = np.abs(S).sum(axis=0)
    b32 = float(np.float32(beta))
    want = cs0.astype(np.float64) * (1.0 - (1.0 - b32) * c) + v.astype(np.float64) @ S
    cs = cs0.copy()
    oracle.cs_update(v, cs, beta)
    np.testing.assert_allclose(cs, want, rtol=1e-5, atol=2e-6)
    if w < d:                      # guards the check itself: with collisions c_j > 1 somewhere,
        assert c.max() > 1         # so "decay once per bucket" would give another answer
        wrong = cs0.astype(np.float64) * b32 + v.astype(np.float64) @ S
        assert np.abs(wrong - want).max() > 1e-3


def test_update_beta_one_is_linear_sketch(oracle):
    rng = np.random.RandomState(3)
    n, d, w = 3, 200, 23
    S = dense_selection(d, w, oracle)
    v1 = rng.randn(n, d).astype(np.float32)
    v2 = rng.randn(n, d).astype(np.float32)
    cs_a = np.zeros((n, w), np.float32)
    oracle.cs_update(v1, cs_a, 1.0)
    np.testing.assert_allclose(cs_a, v1.astype(np.float64) @ S, rtol=1e-5, atol=1e-6)
    # linearity: sketch(v1) then sketch(v2) on top == sketch(v1 + v2) up to fp32 rounding
    oracle.cs_update(v2, cs_a, 1.0)
    cs_b = np.zeros((n, w), np.float32)
    oracle.cs_update(v1 + v2, cs_b, 1.0)
    np.testing.assert_allclose(cs_a, cs_b, rtol=1e-4, atol=1e-5)


def test_exact_recovery_when_hash_is_injective(oracle):
    # pick columns whose buckets are all distinct; then unsketch(sketch(v)) == v exactly
    w = 4096
    bucket, _ = oracle.hash_table(600, w)
    d = 0
    seen = set()
    while bucket[d] not in seen:
        seen.add(int(bucket[d]))
        d += 1
    assert d >= 8
    rng = np.random.RandomState(5)
    v = rng.randn(2, d).astype(np.float32)
    cs = np.zeros((2, w), np.float32)
    oracle.cs_update(v, cs, 1.0)
    x = np.zeros_like(v)
    oracle.cs_query(x, cs, 1.0)
    np.testing.assert_array_equal(x, v)


def test_rows_share_one_hash_and_are_independent(oracle):
    rng = np.random.RandomState(11)
    n, d, w = 4, 90, 13
    v = rng.randn(n, d).astype(np.float32)
    cs = rng.randn(n, w).astype(np.float32)
    full = cs.copy()
    oracle.cs_update(v, full, 0.9)
    for r in range(n):
        one = cs[r:r + 1].copy()
        oracle.cs_update(v[r:r + 1].copy(), one, 0.9)
        np.testing.assert_array_equal(one[0], full[r])


def test_update_term_is_evaluated_in_double(oracle):
    # one column, one bucket: cs' = cs + fl32(s*(v - (1.-beta)*s*cs)) with the inner expression in
    # double.  Values chosen so fp32 evaluation of (1-beta)*cs rounds differently.
    beta = np.float32(0.9)
    v = np.array([[np.float32(1.0000001)]], np.float32)
    cs = np.array([[np.float32(3.3333333)]], np.float32)
    s = float(oracle.hash_table(1, 1)[1][0])
    want = np.float32(cs[0, 0]) + np.float32(s * (float(v[0, 0]) - (1.0 - float(beta)) * s * float(cs[0, 0])))
    oracle.cs_update(v, cs, beta)
    assert cs[0, 0] == np.float32(want)


def test_clean(oracle):
    cs = oracle.DenseCS(3, 20, 0.5)
    cs.cs[:] = 2.0
    cs.clean(0)
    assert (cs.cs == 0).all()
    assert cs.range == 10 and oracle.DenseCS(3, 1, 0.1).range == 1


# ------------------------------------------------------------ 3-hash sketch --

def test_hash3_against_dense_and_median(oracle):
    rng = np.random.RandomState(21)
    n, d, w = 2, 31, 6
    hs = [(994443, 609478, 2, 3, 3), (4113759, 2949676, 4, 5, 5), (9171025, 2171464, 8, 4, 7)]
    cs = [rng.randn(n, w).astype(np.float32) for _ in range(3)]
    x0 = rng.randn(n, d).astype(np.float32)
    alpha = np.float32(0.3)
    est = []
    for (a, b, da, db_u, db_q), c in zip(hs, cs):
        S = dense_selection(d, w, oracle, a, b, a + da, b + db_q)
        est.append(float(alpha) * c.astype(np.float64) @ S.T)
    want = x0 + np.median(np.stack(est), axis=0)
    x = x0.copy()
    oracle.cs3_query(x, *cs, alpha)
    np.testing.assert_allclose(x, want, rtol=2e-6, atol=1e-6)
    # update: u_k = -(1-beta) s_k aux_k[h_k]; m = median(u); mem_k[h_k] += s_k (m + v)
    beta = np.float32(0.9)
    v = rng.randn(n, d).astype(np.float32)
    want_cs = [c.astype(np.float64).copy() for c in cs]
    tabs = [oracle.hash_table(d, w, a, b, a + da, b + db_u) for (a, b, da, db_u, db_q) in hs]
    for r in range(n):
        for i in range(d):
            u = [-(1.0 - float(beta)) * tabs[k][1][i] * float(cs[k][r, tabs[k][0][i]]) for k in range(3)]
            m = sorted(u)[1]
            for k in range(3):
                want_cs[k][r, tabs[k][0][i]] += tabs[k][1][i] * (m + float(v[r, i]))
    got = [c.copy() for c in cs]
    oracle.cs3_update(v, *got, beta)
    for g, wnt in zip(got, want_cs):
        np.testing.assert_allclose(g, wnt, rtol=1e-5, atol=2e-6)
    # the reference's update/query disagreement on the third sign seed is kept
    _, s_u = oracle.hash_table(4000, 1000, 9171025, 2171464, 9171025 + 8, 2171464 + 4)
    _, s_q = oracle.hash_table(4000, 1000, 9171025, 2171464, 9171025 + 8, 2171464 + 7)
    assert (s_u != s_q).any()


def test_half_sketch_is_fp32_path_plus_round_trip(oracle):
    rng = np.random.RandomState(8)
    n, d = 3, 50
    h = oracle.HalfDenseCS(n, d, 0.2)
    f = oracle.DenseCS(n, d, 0.2)
    v = (rng.randn(n, d) * 1e-2).astype(np.float32)
    h.update(v.copy(), 0.9)
    f.update(v.copy(), 0.9)
    assert h.cs.dtype == np.float16
    np.testing.assert_array_equal(h.cs, f.cs.astype(np.float16))


# -------------------------------------------------------------- Gram-Schmidt --

@pytest.mark.parametrize("rows,cols,eps", [(50, 1, 0.0), (64, 4, 0.0), (300, 8, 0.0), (40, 3, 1e-8), (200, 32, 0.0)])
def test_gram_schmidt_vs_torch_library(oracle, rows, cols, eps):
    from torch.distributed.algorithms.ddp_comm_hooks.powerSGD_hook import _orthogonalize_gram_schmidt
    g = torch.Generator().manual_seed(rows + cols)
    a = torch.randn(rows, cols, generator=g)
    want = a.clone().unsqueeze(0)
    _orthogonalize_gram_schmidt(want, eps)       # library routine: batched form of the same procedure
    got = a.numpy().copy()
    oracle.gram_schmidt(got, eps)
    np.testing.assert_allclose(got, want[0].numpy(), rtol=2e-4, atol=2e-6)
    np.testing.assert_allclose(got.T.astype(np.float64) @ got.astype(np.float64), np.eye(cols), atol=5e-6)
    if eps == 0:
        q, r = torch.linalg.qr(a.double())
        q = q * torch.sign(torch.diagonal(r))
        np.testing.assert_allclose(got, q.numpy(), rtol=0, atol=5e-5)


def test_gram_schmidt_zero_column_gives_nan(oracle):
    a = np.zeros((8, 2), np.float32)
    a[:, 1] = 1.0
    oracle.gram_schmidt(a, 0.0)
    assert np.isnan(a[:, 0]).all()


# ------------------------------------------------------------ skinny products --

def test_products_vs_float64(oracle):
    rng = np.random.RandomState(2)
    n, m, r = 13, 29, 3          # all different: a transposed operand cannot pass
    M = rng.randn(n, m).astype(np.float32)
    Q = rng.randn(m, r).astype(np.float32)
    P = rng.randn(n, r).astype(np.float32)
    np.testing.assert_allclose(oracle.mq(M, Q), M.astype(np.float64) @ Q, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.mtp(M, P), M.T.astype(np.float64) @ P, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.pqt(P, Q), P.astype(np.float64) @ Q.T, rtol=1e-6, atol=1e-6)


# -------------------------------------------------------------- random block --

def test_numpy_randomstate_known_answers():
    r = np.random.RandomState(42)
    assert [int(r.choice(6_500_000)) for _ in range(4)] == [6413414, 6423388, 1692743, 4304572]
    r = np.random.RandomState(0)
    assert [int(r.randint(1_000_000_000)) for _ in range(3)] == [209652396, 398764591, 924231285]


def test_block_bounds(oracle):
    assert oracle.block_bounds(6_500_000, 0.1, 6413414) == (650000, 6_500_000, 563414)
    assert oracle.block_bounds(5, 0.1, 3) == (1, 4, 0)
    assert oracle.block_bounds(100, 0.25, 90) == (25, 100, 15)


@pytest.mark.parametrize("conef", [False, True])
def test_randomblock_partition_invariants(oracle, conef):
    rng = np.random.RandomState(4)
    shapes = [(6, 5, 3), (7,), (4, 9)]
    total = sum(int(np.prod(s)) for s in shapes)
    st = oracle.RandomBlockOracle(compression_ratio=0.3, use_error_compression=conef, sketch_size=0.5)
    for step in range(3):
        g = rng.randn(total).astype(np.float32)
        before = g.copy()
        old_err = [e.copy() if not conef else e.cs.copy() for e in st.error_dict.get(0, [])]
        payload = st.step(0, g, shapes).copy()
        outs = oracle.split_bucket(g, shapes)
        ins = oracle.split_bucket(before, shapes)
        np.testing.assert_array_equal(outs[1], ins[1])        # 1-D tensors pass through
        off = 0
        for k, ti in enumerate((0, 2)):
            numel = outs[ti].size
            block, end, rest = oracle.block_bounds(numel, 0.3, st.last_starts[k])
            mask = np.zeros(numel, bool)
            mask[st.last_starts[k]:end] = True
            mask[:rest] = True
            assert mask.sum() == block
            out = outs[ti].reshape(-1)
            assert (out[~mask] == 0).all()
            if not conef:
                x = ins[ti].reshape(-1) + (old_err[k].reshape(-1) if old_err else 0)
                x = x.astype(np.float32)
                err = st.error_dict[0][k].reshape(-1)
                # disjoint partition: output + residual == g + e bit for bit
                np.testing.assert_array_equal(out + err, x)
                assert (err[mask] == 0).all()
            else:
                # the composition of the sketched branch (RandomBlock_hook.py:190,231-243), through the
                # sketch class alone: the block holds g + (1 - beta) * unsketch(old sketch), and the new
                # sketch is ONE update, with beta, of that sum with the block zeroed
                n, m = ins[ti].shape[0], ins[ti].size // ins[ti].shape[0]
                twin = oracle.DenseCS(n, m, 0.5)
                if old_err:
                    twin.cs[...] = old_err[k]
                x = ins[ti].reshape(n, m).copy()
                twin.query(x, 1 - st.beta)
                np.testing.assert_array_equal(out[mask], x.reshape(-1)[mask])
                rest_of_x = np.where(mask, np.float32(0), x.reshape(-1)).reshape(n, m)
                twin.update(rest_of_x, st.beta)
                np.testing.assert_array_equal(st.error_dict[0][k].cs, twin.cs)
                # and the update really took the zeroed copy: with the block left in, the sketch differs
                other = oracle.DenseCS(n, m, 0.5)
                if old_err:
                    other.cs[...] = old_err[k]
                other.update(x, st.beta)
                assert not np.array_equal(other.cs, twin.cs)
            np.testing.assert_array_equal(np.concatenate([out[st.last_starts[k]:end], out[:rest]]),
                                          payload[off:off + block])
            off += block


def test_unbiased_block_scaling(oracle):
    rng = np.random.RandomState(9)
    shapes = [(10, 10), (3,)]
    st = oracle.UnbiasedRandomBlockOracle(compression_ratio=0.2)
    g = rng.randn(103).astype(np.float32)
    before = g.copy()
    payload = st.step(0, g, shapes)
    start = st.last_starts[0]
    prob = np.float32(20 / 100)
    sel = (np.arange(start, start + 20)) % 100
    np.testing.assert_array_equal(payload, before[:100][sel] / prob)
    np.testing.assert_array_equal(g[100:], before[100:])
    assert np.count_nonzero(g[:100]) <= 20


# ------------------------------------------------------------------- top-k --

def test_topk_vs_torch(oracle):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(37, 11, generator=g)       # distinct magnitudes with probability one
    k = max(1, int(0.5 * 0.4 * x.numel()))
    _, pos = torch.topk(x.view(-1).abs(), k, sorted=False)
    want = torch.zeros_like(x)
    want.view(-1)[pos] = x.view(-1)[pos]
    got = x.numpy().copy()
    assert oracle.topk_sparsify(got, 0.4) == k
    np.testing.assert_array_equal(got, want.numpy())
    tie = np.array([1.0, -1.0, 1.0, 0.5], np.float32)
    oracle.topk_sparsify(tie, 1.0)             # k = 2: lowest indices win the tie
    np.testing.assert_array_equal(tie, [1.0, -1.0, 0.0, 0.0])


# ------------------------------------------------------------ PowerSGD round --

def test_powersgd_projection_invariants(oracle):
    rng = np.random.RandomState(6)
    n, m, r = 24, 40, 3
    shapes = [(n, m), (m,)]
    st = oracle.PowerSGDOracle(matrix_approximation_rank=r, error_mode="ef")
    g = rng.randn(n * m + m).astype(np.float32)
    x = g.copy()
    st.step(0, g, shapes)
    M, Mhat = x[:n * m].reshape(n, m).astype(np.float64), g[:n * m].reshape(n, m).astype(np.float64)
    P = st.p_memory_dict[0][0].astype(np.float64)
    np.testing.assert_allclose(P.T @ P, np.eye(r), atol=1e-5)
    np.testing.assert_allclose(Mhat, P @ (P.T @ M), atol=1e-4)            # orthogonal projection onto span(P)
    assert np.linalg.matrix_rank(Mhat, tol=1e-4) <= r
    np.testing.assert_allclose(st.error_dict[0] + g, x, rtol=0, atol=5e-7)    # e' + M_hat == g + e up to one fp32 rounding
    np.testing.assert_array_equal(g[n * m:], x[n * m:])                   # the 1-D tensor is untouched
    assert st.last_seed == 209652396


def test_powersgd_exact_recovery_of_low_rank_input(oracle):
    rng = np.random.RandomState(12)
    n, m, r = 30, 50, 2
    M = (rng.randn(n, r) @ rng.randn(r, m)).astype(np.float32)
    st = oracle.PowerSGDOracle(matrix_approximation_rank=r, error_mode=None)
    g = M.reshape(-1).copy()
    st.step(0, g, [(n, m)])
    np.testing.assert_allclose(g.reshape(n, m), M, rtol=0, atol=2e-4)


def test_powersgd_vs_installed_torch_hook(oracle, tmp_path):
    """torch's own powerSGD_hook is the upstream of the reference file; for plain error feedback
    at rank <= 2 it orthogonalises with the same Gram-Schmidt, so it is an independent oracle."""
    import torch.distributed as dist
    from torch.distributed.algorithms.ddp_comm_hooks import powerSGD_hook as T

    if not dist.is_initialized():
        dist.init_process_group("gloo", init_method=f"file://{tmp_path}/pg", rank=0, world_size=1)

    class Bucket:
        def __init__(self, flat, shapes, idx=0):
            self._flat, self._shapes, self._idx = flat, shapes, idx

        def buffer(self):
            return self._flat

        def gradients(self):
            out, off = [], 0
            for s in self._shapes:
                c = int(np.prod(s))
                out.append(self._flat[off:off + c].view(*s))
                off += c
            return out

        def index(self):
            return self._idx

        def is_last(self):
            return True

    shapes = [(16, 27), (16,), (32, 20)]
    total = sum(int(np.prod(s)) for s in shapes)
    tstate = T.PowerSGDState(None, matrix_approximation_rank=2, start_powerSGD_iter=2, random_seed=0)
    tstate.iter = 5
    ostate = oracle.PowerSGDOracle(matrix_approximation_rank=2, error_mode="ef", random_seed=0)
    rng = np.random.RandomState(33)
    for step in range(3):
        g = (rng.randn(total) * 1e-3).astype(np.float32)
        tg = torch.from_numpy(g.copy())
        out = T.powerSGD_hook(tstate, Bucket(tg, shapes)).wait()
        og = g.copy()
        ostate.step(0, og, shapes)
        scale = np.abs(g).max()
        np.testing.assert_allclose(og, out.numpy(), rtol=0, atol=2e-5 * scale)
        np.testing.assert_allclose(ostate.error_dict[0], tstate.error_dict[0].numpy(), rtol=0, atol=2e-5 * scale)


def test_batched_powersgd_vs_installed_torch_hook(oracle, tmp_path, monkeypatch):
    """torch's batched_powerSGD_hook is the upstream of the reference's (powerSGD_hook.py:583-787);
    at rank <= 2 it orthogonalises with the same Gram-Schmidt.  The installed hook hands its 2-D
    P and Q to a routine that asserts a batch dimension, so for the duration of this test that
    routine is given the batch dimension (the library's own code does the work)."""
    import torch.distributed as dist
    from torch.distributed.algorithms.ddp_comm_hooks import powerSGD_hook as T

    if not dist.is_initialized():
        dist.init_process_group("gloo", init_method=f"file://{tmp_path}/pg", rank=0, world_size=1)
    library_orthogonalize = T._orthogonalize
    monkeypatch.setattr(T, "_orthogonalize",
                        lambda mat, epsilon=0: library_orthogonalize(mat.unsqueeze(0) if mat.dim() == 2 else mat, epsilon))

    class Bucket:
        def __init__(self, flat):
            self._flat = flat

        def buffer(self):
            return self._flat

        def index(self):
            return 0

        def is_last(self):
            return True

    for total, rank in [(5000, 1), (64 * 64, 2), (777, 2)]:
        tstate = T.PowerSGDState(None, matrix_approximation_rank=rank, start_powerSGD_iter=2, random_seed=0)
        tstate.iter = 5
        ostate = oracle.BatchedPowerSGDOracle(matrix_approximation_rank=rank, random_seed=0)
        rng = np.random.RandomState(34)
        for step in range(3):
            g = (rng.randn(total) * 1e-3).astype(np.float32)
            tg = torch.tensor(g)          # owns its storage: the hook resizes the buffer in place
            out = T.batched_powerSGD_hook(tstate, Bucket(tg)).wait()
            og = g.copy()
            ostate.step(0, og)
            scale = np.abs(g).max()
            assert out.shape[0] == total
            np.testing.assert_allclose(og, out.numpy(), rtol=0, atol=2e-5 * scale)
            np.testing.assert_allclose(ostate.error_dict[0], tstate.error_dict[0].numpy(), rtol=0, atol=2e-5 * scale)


def test_c2cs_v2_sketch_is_over_the_reviewed_memory(oracle):
    """C2CS_hook_v2 builds DenseCS(m, n) on matrix.view(m, n): with one [n,m] matrix and no
    compression loss to speak of, the sketch after a step equals a hand-made update of the
    residual re-viewed [m,n]; and for a square matrix v2 and the plain ConEF hook agree."""
    rng = np.random.RandomState(5)
    n, m, r = 12, 40, 2
    g = (rng.randn(n * m) * 1e-3).astype(np.float32)
    st = oracle.PowerSGDOracle(matrix_approximation_rank=r, error_mode="conef_v2", sketch_size=0.5, beta=0.9)
    work = g.copy()
    st.step(0, work, [(n, m)])
    cs = st.error_dict[0][0]
    assert (cs.N, cs.D, cs.range) == (m, n, max(int(n * 0.5), 1))
    hand = oracle.DenseCS(m, n, 0.5)
    hand.update((g - work).reshape(m, n), 0.9)       # first step: the queried sketch was zero
    np.testing.assert_array_equal(cs.cs, hand.cs)
    sq = (rng.randn(30 * 30) * 1e-3).astype(np.float32)
    a = oracle.PowerSGDOracle(matrix_approximation_rank=r, error_mode="conef_v2", sketch_size=0.5)
    b = oracle.PowerSGDOracle(matrix_approximation_rank=r, error_mode="conef", sketch_size=0.5)
    for _ in range(3):
        ga, gb = sq.copy(), sq.copy()
        a.step(0, ga, [(30, 30)])
        b.step(0, gb, [(30, 30)])
        np.testing.assert_array_equal(ga, gb)
