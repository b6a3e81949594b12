"""The headline configuration at full size: RandomBlock 10 % + count-sketch 10 % on a flat 6.5 M
element bucket viewed [5, 1_300_000], heavy-tailed gradients, error carried across steps.
Checked against the oracle over the configuration's 100 steps (bit for bit: the planned path adds
in the oracle's order) and through size-independent properties."""
import numpy as np
import pytest
import torch

from _helpers import FakeGradBucket, heavy_tail_gradient, to_np

pytestmark = pytest.mark.gpu

N, M = 5, 1_300_000
L = N * M


def test_headline_steps_match_oracle_bit_for_bit(oracle):
    from conef_amd.RandomBlock_hook import RandomBlock_hook, RandomBlockState
    st = RandomBlockState(None, compression_ratio=0.1, start_compression_iter=2, use_error_compression=True,
                          sketch_size=0.1, beta=0.9, random_seed=42)
    st.iter = 2
    ost = oracle.RandomBlockOracle(compression_ratio=0.1, use_error_compression=True, sketch_size=0.1, beta=0.9,
                                   random_seed=42)
    bases = [heavy_tail_gradient(L, seed=500 + k) for k in range(6)]
    for step in range(100):         # the configuration's own length, error carried from step to step
        g = bases[step % 6] if step < 6 else bases[step % 6].roll(step * 7919)
        gd = g.cuda()
        RandomBlock_hook(st, FakeGradBucket(gd, [(N, M)])).wait()
        og = g.numpy().copy()
        ost.step(0, og, [(N, M)])
        np.testing.assert_array_equal(to_np(gd), og)
        np.testing.assert_array_equal(to_np(st.compressed_tensor_memory[0]), ost.compressed_tensor_memory[0])
        np.testing.assert_array_equal(to_np(st.error_dict[0][0].cs), ost.error_dict[0][0].cs)
        if step == 2:
            assert ost.last_starts == [1692743]          # third draw of RandomState(42).choice(6.5 M)
    assert st.error_dict[0][0].range == 130_000 and st.compressed_tensor_memory[0].numel() == 650_000


def test_headline_properties_over_many_steps():
    from conef_amd.compressors.CountSketch import DenseCS
    from conef_amd.RandomBlock_hook import RandomBlock_hook, RandomBlockState
    st = RandomBlockState(None, compression_ratio=0.1, start_compression_iter=2, use_error_compression=True,
                          sketch_size=0.1, beta=0.9)
    st.iter = 2
    rng = np.random.RandomState(42)
    g0 = heavy_tail_gradient(L, seed=77).cuda()
    for step in range(20):
        g = g0.roll(step * 1001)
        before = g.clone()
        # what the step must add to the gradient: the unsketched error, from a separate query call
        want = before.clone().view(N, M)
        if 0 in st.error_dict:
            st.error_dict[0][0].query(want, 1 - 0.9)
        RandomBlock_hook(st, FakeGradBucket(g, [(N, M)])).wait()
        start = int(rng.choice(L))
        sel = torch.zeros(L, dtype=torch.bool, device="cuda")
        end = min(start + 650_000, L)
        sel[start:end] = True
        sel[:650_000 - (end - start)] = True
        assert int(sel.sum()) == 650_000
        assert torch.equal(g[sel], want.view(-1)[sel])            # block = gradient + unsketched error
        assert float(g[~sel].abs().max()) == 0.0                  # everything else zero
        payload = st.compressed_tensor_memory[0]
        assert torch.equal(payload, torch.cat([g[start:end], g[:650_000 - (end - start)]]))
        assert torch.isfinite(st.error_dict[0][0].cs).all()
    # linearity of the sketch in the sketched values at beta = 1 (pure linear sketch)
    a = DenseCS(N, M, 0.1)
    b = DenseCS(N, M, 0.1)
    c = DenseCS(N, M, 0.1)
    u = heavy_tail_gradient(L, seed=1).cuda().view(N, M)
    v = heavy_tail_gradient(L, seed=2).cuda().view(N, M)
    a.update(u, 1.0)
    b.update(v, 1.0)
    c.update(u + v, 1.0)
    diff = (a.cs + b.cs - c.cs).abs().max() / c.cs.abs().max()
    assert float(diff) < 1e-5
