"""The top-k entry point that allocates nothing (`conef_topk_sparsify_noalloc_f32`, selection state
in the library's own per-GPU scratch) against `conef_topk_sparsify_f32`, which takes a workspace.
Bar: bit-exact (integer select on magnitudes, values copied or zeroed)."""
import numpy as np
import pytest
import torch

from conef_amd import _lib

pytestmark = pytest.mark.gpu


def _gradient(numel, seed, repeats=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(numel, generator=g) * 1e-3
    if repeats:                       # many equal magnitudes: the tie rule (lowest indices stay) matters
        x = torch.round(x * 2e3) / 2e3
    return x.float()


def _with_workspace(lib, x, k):
    ws = torch.empty(lib.conef_topk_workspace_bytes(x.numel()), dtype=torch.uint8, device=x.device)
    rc = lib.conef_topk_sparsify_f32(x.data_ptr(), x.numel(), k, ws.data_ptr(), ws.numel(), _lib.stream_ptr(x))
    _lib.check(rc, "conef_topk_sparsify_f32")
    torch.cuda.synchronize()
    return x


def test_noalloc_topk_matches_workspace_entry_point_on_two_calls_in_a_row():
    lib = _lib.load()
    torch.cuda.set_device(0)
    # second call smaller than the first, then one with surplus ties on the threshold, then k >= numel
    cases = [(1_048_576, 209_715, False), (70_001, 14_000, False), (262_144, 40_000, True), (1000, 1000, False)]
    inputs = [(_gradient(n, 100 + i, rep).cuda(), k) for i, (n, k, rep) in enumerate(cases)]
    want = [_with_workspace(lib, x.clone(), k).cpu().numpy() for x, k in inputs]
    got = []
    # a first call on a throw-away input: whatever the runtime sets up lazily for the library's code
    # object (the symbol lookup of the scratch array included) is not what is being checked
    warm = _gradient(4096, 7).cuda()
    _lib.check(lib.conef_topk_sparsify_noalloc_f32(warm.data_ptr(), warm.numel(), 100, _lib.stream_ptr(warm)),
               "conef_topk_sparsify_noalloc_f32")
    torch.cuda.synchronize()
    # free bytes as the driver reports them: this sees a hipMalloc inside the library too, which
    # torch's own allocator statistics would not
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_allocated()
    for x, k in inputs:               # back to back on one stream, nothing waited for in between
        rc = lib.conef_topk_sparsify_noalloc_f32(x.data_ptr(), x.numel(), k, _lib.stream_ptr(x))
        _lib.check(rc, "conef_topk_sparsify_noalloc_f32")
        got.append(x)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for (n, k, _), g, w in zip(cases, got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w, err_msg="numel %d k %d" % (n, k))
        if k < n:
            assert int((g != 0).sum()) <= k


def test_noalloc_topk_rejects_what_it_cannot_take():
    lib = _lib.load()
    x = torch.ones(16, device="cuda")
    s = _lib.stream_ptr(x)
    assert lib.conef_topk_sparsify_noalloc_f32(x.data_ptr(), 1 << 32, 5, s) == -2      # beyond the stated maximum
    assert lib.conef_topk_sparsify_noalloc_f32(x.data_ptr(), 0, 5, s) == -1
    assert lib.conef_topk_sparsify_noalloc_f32(x.data_ptr(), 16, 0, s) == -1
    assert lib.conef_topk_sparsify_noalloc_f32(None, 16, 4, s) == -1
    with pytest.raises(ValueError, match="maximum"):
        _lib.check(-2, "conef_topk_sparsify_noalloc_f32")
    torch.cuda.synchronize()
    assert torch.equal(x.cpu(), torch.ones(16))
