"""The benchmark configurations at their full shapes, checked through properties that do not need
the (scalar, slow) CPU oracle at this size:

* WideResNet-28-10 gradients (29 two-dimensional weights, 36.5 M elements, 25 MB buckets),
  PowerSGD rank 4 with a count-sketched error at 20 % memory;
* the 2-layer LSTM language model (vocabulary 33278, width 650) with a row-sparse embedding
  gradient, UnbiasedRandomBlock at 5 % and RandomBlock + count sketch on the same shapes;
* BERT-large (334 M elements), PowerSGD rank 8 and rank 32 with a count-sketched error at 10 %,
  and hPowerSGD (top-k error) on one bucket.

PowerSGD properties: the bucket holds P Q^T of the state's own factors; P has orthonormal
columns; the new sketch equals what the standalone compressor calls (query, subtract, update)
produce from the same inputs - the fused kernels and the separate ones add the same terms in the
same order, so that comparison is bit for bit; tensors that are not compressed pass through
untouched.  Small-shape parity with the oracle lives in test_gpu_hooks.py.
"""
import numpy as np
import pytest
import torch

from _helpers import FakeGradBucket, assert_close

pytestmark = pytest.mark.gpu

BUCKET_CAP = 25 * 1024 * 1024 // 4      # DDP's default 25 MiB in fp32 elements


def wrn_28_10_shapes():
    """examples/ImageClassification/models/wideresnet.py:44-87 (depth 28, widening 10), with the
    1-D batch-norm and bias tensors in between."""
    shapes = [(16, 3, 3, 3)]
    widths = [16, 160, 320, 640]
    for stage in range(3):
        cin, cout = widths[stage], widths[stage + 1]
        for block in range(4):
            a = cin if block == 0 else cout
            shapes += [(a,), (a,), (cout, a, 3, 3), (cout,), (cout,), (cout, cout, 3, 3)]
            if block == 0:
                shapes.append((cout, a, 1, 1))
    shapes += [(640,), (640,), (10, 640), (10,)]
    return shapes


def lstm_shapes():
    v, h = 33278, 650
    return [(v, h), (4 * h, h), (4 * h, h), (4 * h,), (4 * h,), (4 * h, h), (4 * h, h), (4 * h,), (4 * h,), (v, h),
            (v,)]


def bert_large_shapes():
    h, f, v = 1024, 4096, 30522
    shapes = [(v, h), (512, h), (2, h), (h,), (h,)]
    for _ in range(24):
        shapes += [(h, h), (h,)] * 4 + [(h,), (h,), (f, h), (f,), (h, f), (h,), (h,), (h,)]
    shapes += [(h, h), (h,), (h, h), (h,), (h,), (h,), (v,), (2, h), (2,)]
    return shapes


def numel(shape):
    return int(np.prod(shape))


def buckets_of(shapes):
    """Greedy packing in reverse parameter order, as DDP fills its buckets."""
    out, cur, size = [], [], 0
    for s in reversed(shapes):
        if cur and size + numel(s) > BUCKET_CAP:
            out.append(cur)
            cur, size = [], 0
        cur.append(s)
        size += numel(s)
    if cur:
        out.append(cur)
    return out


def test_shape_lists():
    two_d = [s for s in wrn_28_10_shapes() if len(s) > 1]
    assert len(two_d) == 29 and sum(numel(s) for s in two_d) == 36_461_232
    assert max(numel(s) for s in two_d) == 640 * 5760
    total = sum(numel(s) for s in bert_large_shapes())
    assert 330e6 < total < 340e6
    assert sum(numel(s) for s in lstm_shapes() if len(s) > 1) == 2 * 33278 * 650 + 4 * 2600 * 650


def views(flat, shapes):
    out, off = [], 0
    for s in shapes:
        out.append(flat[off:off + numel(s)].view(*s))
        off += numel(s)
    return out


def gram_schmidt_f64(a):
    """powerSGD_hook.py:12-44 in float64 on the device (epsilon 0)."""
    a = a.clone()
    for i in range(a.shape[1]):
        a[:, i] /= a[:, i].norm()
        if i + 1 < a.shape[1]:
            a[:, i + 1:] -= (a[:, i:i + 1] * a[:, i + 1:]).sum(0, keepdim=True) * a[:, i:i + 1]
    return a


def check_powersgd_conef_bucket(state, index, shapes, g_before, g_after, sketches_before, rank, ss, beta, q_before=None):
    from conef_amd.compressors.CountSketch import DenseCS
    from conef_amd.powerSGD_hook import _should_compress
    p_mem, q_mem = state.p_memory_dict[index], state.q_memory_dict[index]
    p_off = q_off = 0
    cnt = 0
    for before, after, s in zip(views(g_before, shapes), views(g_after, shapes), shapes):
        n = s[0]
        m = numel(s) // n
        r = min(n, m, rank)
        if not _should_compress(n, m, r, 2)[0]:
            assert torch.equal(before, after), "uncompressed tensor %s changed" % (s,)
            continue
        p = p_mem[p_off:p_off + n * r].view(n, r)
        q = q_mem[q_off:q_off + m * r].view(m, r)
        p_off += n * r
        q_off += m * r
        low = after.view(n, m)
        assert_close(low, (p.double() @ q.double().t()).float(), what="P Q^T of %s" % (s,))
        eye = (p.double().t() @ p.double()).cpu().numpy()
        np.testing.assert_allclose(eye, np.eye(r), atol=5e-5, err_msg="P^T P of %s" % (s,))
        # the sketch through the standalone compressor calls, from the same inputs
        ref = DenseCS(n, m, ss)
        if sketches_before is not None:
            ref.cs.copy_(sketches_before[cnt])
        x = before.reshape(n, m).clone()
        ref.query(x, 1 - beta)
        # The products themselves, against float64 on the device: what the round must leave is the
        # projection of X = gradient + unsketched error onto span(P), M^ = P (P^T X), and
        # Q = X^T P; and P must be the orthogonalised X Q' with Q' the orthogonalised factor the
        # round started from.  A wrong P = M Q or Q = M^T P at full shape fails here.
        x64, p64 = x.double(), p.double()
        assert_close(q, (x64.t() @ p64).float(), what="Q = X^T P of %s" % (s,))
        assert_close(low, (p64 @ (p64.t() @ x64)).float(), what="projection identity of %s" % (s,))
        if q_before is not None:
            q_start = gram_schmidt_f64(q_before[q_off - m * r:q_off].view(m, r).double())
            # Gram-Schmidt carries fp32 rounding from column to column: 5e-5 instead of 1e-5
            assert_close(p, gram_schmidt_f64(x64 @ q_start).float(), rel=5e-5, what="P = orth(X Q) of %s" % (s,))
        resid = x - low
        ref.update(resid, beta)
        got = state.error_dict[index][cnt].cs
        assert torch.equal(got, ref.cs), "sketch of %s: max diff %g" % (s, float((got - ref.cs).abs().max()))
        cnt += 1
    assert p_off == p_mem.numel() and q_off == q_mem.numel()


def run_powersgd_conef(shapes, rank, ss, sigma_of, steps, max_buckets=None, resume_at=None):
    """``resume_at``: before that step the state goes through state_dict -> torch.save -> a new
    state's load_state_dict, as a restarted job would restore it."""
    import io
    from conef_amd.powerSGD_hook import PowerSGDState, powerSGD_hook
    beta = 0.9

    def make():
        return PowerSGDState(None, matrix_approximation_rank=rank, start_powerSGD_iter=2, use_error_compression=True,
                             sketch_size=ss, beta=beta)

    state = make()
    state.iter = 2
    buckets = buckets_of(shapes)
    if max_buckets:
        buckets = buckets[:max_buckets]
    gen = torch.Generator(device="cuda").manual_seed(1234)
    for step in range(steps):
        if resume_at is not None and step == resume_at:
            buf = io.BytesIO()
            torch.save(state.state_dict(), buf)
            buf.seek(0)
            state = make()
            state.load_state_dict(torch.load(buf, weights_only=False))
            assert state.iter == 2 + step
        for index, bshapes in enumerate(buckets):
            total = sum(numel(s) for s in bshapes)
            g = torch.empty(total, device="cuda")
            for k, v in enumerate(views(g, bshapes)):
                v.copy_(torch.randn(v.shape, generator=gen, device="cuda") * sigma_of(index, k))
            before = g.clone()
            old = None
            if index in state.error_dict:
                old = {k: cs.cs.clone() for k, cs in state.error_dict[index].items()}
            q_before = state.q_memory_dict[index].clone() if index in state.q_memory_dict else None
            out = powerSGD_hook(state, FakeGradBucket(g, bshapes, index=index,
                                                      is_last=index == len(buckets) - 1)).wait()
            assert out.data_ptr() == g.data_ptr()
            assert torch.isfinite(g).all()
            check_powersgd_conef_bucket(state, index, bshapes, before, g, old, rank, ss, beta, q_before)
    assert state.iter == 2 + steps
    return state, buckets


def test_wideresnet_28_10_powersgd_rank4_sketch20():
    rs = np.random.RandomState(7)
    sigmas = {}

    def sigma_of(bucket, k):       # per-layer sigma, log-uniform in [1e-5, 1e-2], fixed across steps
        return sigmas.setdefault((bucket, k), float(10 ** rs.uniform(-5, -2)))

    state, buckets = run_powersgd_conef(wrn_28_10_shapes(), rank=4, ss=0.2, sigma_of=sigma_of, steps=3)
    assert len(buckets) >= 6
    rate, before, after = state.compression_stats()
    assert rate > 50          # rank 4 on [640,5760]-sized matrices


@pytest.mark.parametrize("rank", [8, 32])
def test_bert_large_powersgd_sketch10(rank):
    # the configuration's 10 steps, with a checkpoint restore in the middle
    state, buckets = run_powersgd_conef(bert_large_shapes(), rank=rank, ss=0.1, sigma_of=lambda b, k: 5e-4, steps=10,
                                        resume_at=5)
    assert len(buckets) >= 50
    # [2,1024] never passes the compression test at these ranks (powerSGD_hook.py:46-70)
    from conef_amd.powerSGD_hook import _should_compress
    assert not _should_compress(2, 1024, 2, 2)[0]


@pytest.mark.parametrize("rank", [8, 32])
def test_bert_large_hpowersgd_topk_one_bucket(rank):
    """hPowerSGD keeps a dense per-matrix error cut down to the int(0.5 * 0.4 * numel) largest
    magnitudes (hPowerSGD_hook.py:90-97,553-554): count and threshold property on a full bucket,
    and the products against float64 on the device (Q = X^T P, M^ = P (P^T X), P orthonormal),
    at the configuration's rank 8 and at its rank-32 variant."""
    from conef_amd.hPowerSGD_hook import _should_compress, hPowerSGDState, hpowerSGD_hook
    shapes = buckets_of(bert_large_shapes())[3]
    state = hPowerSGDState(None, matrix_approximation_rank=rank, start_powerSGD_iter=2, use_error_compression=True,
                           topk_ratio=0.4)
    state.iter = 2
    total = sum(numel(s) for s in shapes)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for step in range(2):
        g = torch.randn(total, generator=gen, device="cuda") * 5e-4
        before = g.clone()
        state.settle()
        old = {k: e.clone() for k, e in state.error_dict.get(0, {}).items()}
        hpowerSGD_hook(state, FakeGradBucket(g, shapes)).wait()
        state.settle()                      # the top-k of this step's errors may run on a side stream
        cnt = 0
        p_off = q_off = 0
        p_mem, q_mem = state.p_memory_dict[0], state.q_memory_dict[0]
        for b, a, s in zip(views(before, shapes), views(g, shapes), shapes):
            n, m = s[0], numel(s) // s[0]
            r = min(n, m, rank)
            if not _should_compress(n, m, r, 2)[0]:
                assert torch.equal(a, b)
                continue
            err = state.error_dict[0][cnt]
            k = max(1, int(0.5 * 0.4 * numel(s)))
            assert int((err != 0).sum()) == k
            x = (b + old[cnt] if cnt in old else b).reshape(n, m)    # gradient + remembered error
            full = x - a.reshape(n, m)                               # the residual before sparsification
            kept = err != 0
            assert torch.equal(err[kept], full[kept])
            assert float(full[~kept].abs().max()) <= float(err[kept].abs().min())
            p = p_mem[p_off:p_off + n * r].view(n, r)
            q = q_mem[q_off:q_off + m * r].view(m, r)
            p_off += n * r
            q_off += m * r
            x64, p64 = x.double(), p.double()
            np.testing.assert_allclose((p64.t() @ p64).cpu().numpy(), np.eye(r), atol=5e-5, err_msg="P^T P of %s" % (s,))
            assert_close(q, (x64.t() @ p64).float(), what="Q = X^T P of %s" % (s,))
            assert_close(a.reshape(n, m), (p64 @ (p64.t() @ x64)).float(), what="projection identity of %s" % (s,))
            cnt += 1
        assert p_off == p_mem.numel() and q_off == q_mem.numel()


def lstm_gradient(shapes, step):
    """Dense N(0, (1e-3)^2) gradients, except the embedding: non-zero only on the rows of the
    20 x 35 token ids of the step, drawn Zipf(1.1) and clipped to the vocabulary."""
    gen = torch.Generator(device="cuda").manual_seed(900 + step)
    total = sum(numel(s) for s in shapes)
    g = torch.randn(total, generator=gen, device="cuda") * 1e-3
    ids = np.minimum(np.random.RandomState(step).zipf(1.1, size=700), 33278) - 1
    emb = views(g, shapes)[0]
    mask = torch.zeros(33278, dtype=torch.bool, device="cuda")
    mask[torch.from_numpy(np.unique(ids)).cuda()] = True
    emb[~mask] = 0
    return g


def block_mask(numel_, start, block):
    sel = torch.zeros(numel_, dtype=torch.bool, device="cuda")
    end = min(start + block, numel_)
    sel[start:end] = True
    sel[:block - (end - start)] = True
    return sel


def test_lstm_unbiased_randomblock_5pct():
    from conef_amd.UnbiasedRandomBlock_hook import UnbiasedRandomBlock_hook, UnbiasedRandomBlockState
    shapes = lstm_shapes()
    state = UnbiasedRandomBlockState(None, compression_ratio=0.05, start_compression_iter=2)
    state.iter = 2
    rng = np.random.RandomState(42)
    for step in range(3):
        g = lstm_gradient(shapes, step)
        before = g.clone()
        UnbiasedRandomBlock_hook(state, FakeGradBucket(g, shapes)).wait()
        for b, a, s in zip(views(before, shapes), views(g, shapes), shapes):
            if len(s) < 2:
                assert torch.equal(a, b)
                continue
            n = numel(s)
            block = max(1, int(0.05 * n))
            assert block in (1_081_535, 84_500)
            start = int(rng.choice(n))
            sel = block_mask(n, start, block)
            # a true IEEE division by fl32(block / numel): dividing a GPU tensor by a Python scalar
            # multiplies by the reciprocal instead, so the divisor goes in as a tensor
            prob = torch.full((), float(np.float32(block / n)), device="cuda")
            want = torch.where(sel, b.reshape(-1) / prob, torch.zeros((), device="cuda"))
            assert torch.equal(a.reshape(-1), want)
    assert state.iter == 5


def test_lstm_randomblock_with_sketched_error():
    """The same shapes through RandomBlock with a count-sketched error (the reference's unbiased
    hook keeps no error state at all): output = block of (gradient + unsketched error), zeros
    elsewhere, and the new sketch equals query + zero-the-block + update through the standalone
    compressor calls, bit for bit."""
    from conef_amd.compressors.CountSketch import DenseCS
    from conef_amd.RandomBlock_hook import RandomBlock_hook, RandomBlockState
    shapes = lstm_shapes()
    state = RandomBlockState(None, compression_ratio=0.05, start_compression_iter=2, use_error_compression=True,
                             sketch_size=0.1, beta=0.9)
    state.iter = 2
    rng = np.random.RandomState(42)
    mirror = {}
    for step in range(3):
        g = lstm_gradient(shapes, step)
        before = g.clone()
        RandomBlock_hook(state, FakeGradBucket(g, shapes)).wait()
        cnt = 0
        for b, a, s in zip(views(before, shapes), views(g, shapes), shapes):
            if len(s) < 2:
                assert torch.equal(a, b)
                continue
            n, m = s[0], numel(s) // s[0]
            ref = mirror.setdefault(cnt, DenseCS(n, m, 0.1))
            x = b.reshape(n, m).clone()
            ref.query(x, 1 - 0.9)
            block = max(1, int(0.05 * n * m))
            sel = block_mask(n * m, int(rng.choice(n * m)), block).view(n, m)
            assert torch.equal(a.reshape(n, m), torch.where(sel, x, torch.zeros((), device="cuda")))
            ref.update(torch.where(sel, torch.zeros((), device="cuda"), x), 0.9)
            assert torch.equal(state.error_dict[0][cnt].cs, ref.cs)
            cnt += 1
