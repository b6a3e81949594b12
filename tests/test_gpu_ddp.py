"""The hooks under a real DistributedDataParallel model on one GPU (world size 1): registration
through ``register_comm_hook``, the plain all-reduce warm-up iterations, DDP's bucket rebuild after
the first iteration, several buckets per step with ``is_last()`` closing the iteration, and the
Future handed back to the reducer.  The gradient a hook leaves in ``param.grad`` is compared with
the CPU oracle fed the gradient each bucket held when the reducer handed it to the hook."""
import copy
from argparse import Namespace

import numpy as np
import pytest
import torch
import torch.distributed as dist
import torch.nn as nn

from _helpers import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def process_group(tmp_path_factory):
    created = False
    if not dist.is_initialized():
        store = tmp_path_factory.mktemp("pg") / "store"
        dist.init_process_group("nccl", init_method="file://%s" % store, rank=0, world_size=1,
                                device_id=torch.device("cuda", 0))
        created = True
    yield
    if created:
        dist.destroy_process_group()


def make_model():
    torch.manual_seed(7)
    return nn.Sequential(nn.Conv2d(3, 16, 3, padding=1), nn.ReLU(), nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(),
                         nn.AdaptiveAvgPool2d(4), nn.Flatten(), nn.Linear(512, 768), nn.ReLU(), nn.Linear(768, 10))


ARGS = dict(start_compression_iter=3, compression_ratio=0.1, beta=0.9, sketch_size=0.2, matrix_approximation_rank=2,
            min_compression_rate=2, orthogonalization_epsilon=0)


def recording(hook, calls):
    """Wraps a hook: remembers (bucket index, per-parameter shapes, the gradient as it arrived,
    is_last, the state's iteration, the ids of the bucket's parameters)."""

    def recorded_hook(state, bucket):
        calls.append((bucket.index(), [tuple(g.shape) for g in bucket.gradients()],
                      bucket.buffer().detach().cpu().numpy().copy(), bucket.is_last(), state.iter,
                      [id(p) for p in bucket.parameters()]))
        return hook(state, bucket)

    return recorded_hook


@pytest.mark.parametrize("name,streams", [("conef_randomblock", 1), ("ef_randomblock", 1), ("unbiased_randomblock", 1),
                                          ("conef_powersgd", 1), ("ef_powersgd", 1), ("hefsgd_powersgd", 1),
                                          # the PowerSGD rounds of a step spread over side streams
                                          ("conef_powersgd", 3), ("hefsgd_powersgd", 2)])
def test_hook_under_ddp(process_group, oracle, name, streams):
    from torch.nn.parallel import DistributedDataParallel as DDP

    from conef_amd.get_comm_hooks import make_state
    model = make_model().cuda()
    # a small bucket cap so that the model spans several buckets
    ddp = DDP(copy.deepcopy(model), device_ids=[0], bucket_cap_mb=0.25)
    state, hook = make_state(Namespace(grad_reducer=name, **ARGS))
    if streams > 1:
        state.hook_streams = streams
    calls_log = []
    ddp.register_comm_hook(state, recording(hook, calls_log))

    if "randomblock" in name:
        if name == "unbiased_randomblock":
            ostate = oracle.UnbiasedRandomBlockOracle(compression_ratio=0.1)
        else:
            ostate = oracle.RandomBlockOracle(compression_ratio=0.1, use_error_compression=name.startswith("conef"),
                                              sketch_size=0.2, beta=0.9)
    else:
        mode = {"conef_powersgd": "conef", "ef_powersgd": "ef", "hefsgd_powersgd": "topk"}[name]
        ostate = oracle.PowerSGDOracle(matrix_approximation_rank=2, error_mode=mode, sketch_size=0.2, beta=0.9,
                                       topk_ratio=0.4)
    loss_fn = nn.CrossEntropyLoss()
    steps = 6
    for step in range(steps):
        gen = torch.Generator().manual_seed(100 + step)
        x = torch.randn(8, 3, 16, 16, generator=gen).cuda()
        y = torch.randint(0, 10, (8,), generator=gen).cuda()
        calls_log.clear()
        ddp.zero_grad(set_to_none=True)
        loss_fn(ddp(x), y).backward()
        torch.cuda.synchronize()
        calls = list(calls_log)
        # iteration 0 runs on one all-embracing bucket; the reducer rebuilds its buckets after it
        assert len(calls) >= (2 if step > 0 else 1), "the model should span several buckets"
        assert [c[3] for c in calls].count(True) == 1 and calls[-1][3]      # exactly one closes the iteration
        assert state.iter == step + 1
        got = {id(p): p.grad.detach().cpu().numpy().copy() for p in ddp.parameters()}
        if step < ARGS["start_compression_iter"]:
            # warm-up: plain all-reduce, the identity at world size 1 - what arrived is what stays
            for index, shapes, flat, _, _, param_ids in calls:
                off = 0
                for pid, shp in zip(param_ids, shapes):
                    cnt = int(np.prod(shp))
                    np.testing.assert_array_equal(got[pid].reshape(-1), flat[off:off + cnt])
                    off += cnt
            continue
        # compressed: replay every bucket, in the order the reducer delivered them, through the
        # oracle; DDP's gradient views alias the bucket buffers, so p.grad shows what the hook left
        for index, shapes, flat, _, _, param_ids in calls:
            want = flat.copy()
            ostate.step(index, want, shapes)
            off = 0
            for pid, shp in zip(param_ids, shapes):
                cnt = int(np.prod(shp))
                assert_close(got[pid].reshape(-1), want[off:off + cnt],
                             what="%s step %d bucket %d param %s" % (name, step, index, shp))
                off += cnt
            assert off == want.size


@pytest.mark.parametrize("name,rank", [("conef_powersgd", 4), ("hefsgd_powersgd", 4), ("conef_powersgd", 32)])
def test_streams_chosen_by_bucket_size_under_ddp(process_group, name, rank):
    """With ``hook_streams`` left alone, buckets of 2**20 elements or more alternate between the hook's
    stream and a side stream (rank <= 8) or are dealt over three streams (above): under the real reducer
    the parameters' gradients must come out bit for bit as with everything on one stream."""
    from torch.nn.parallel import DistributedDataParallel as DDP

    from conef_amd import _psgd_engine
    from conef_amd.get_comm_hooks import make_state

    def big_model():
        torch.manual_seed(11)
        return nn.Sequential(nn.Linear(1100, 1024), nn.ReLU(), nn.Linear(1024, 1200), nn.ReLU(), nn.Linear(1200, 1024),
                             nn.ReLU(), nn.Linear(1024, 10))

    results = []
    for streams in (None, 1):
        ddp = DDP(big_model().cuda(), device_ids=[0], bucket_cap_mb=4.5)
        args = dict(ARGS, matrix_approximation_rank=rank)
        state, hook = make_state(Namespace(grad_reducer=name, **args))
        if streams is not None:
            state.hook_streams = streams
        else:
            assert state.hook_streams == (3 if rank > 8 else 0)
        seen = []

        def watching(st, bucket, hook=hook, seen=seen):
            seen.append(_psgd_engine.streams_for(st, bucket.buffer()))
            return hook(st, bucket)

        ddp.register_comm_hook(state, watching)
        loss_fn = nn.CrossEntropyLoss()
        grads_per_step = []
        for step in range(7):
            gen = torch.Generator().manual_seed(300 + step)
            x = torch.randn(16, 1100, generator=gen).cuda()
            y = torch.randint(0, 10, (16,), generator=gen).cuda()
            ddp.zero_grad(set_to_none=True)
            loss_fn(ddp(x), y).backward()
            torch.cuda.synchronize()
            grads_per_step.append([p.grad.detach().cpu().numpy().copy() for p in ddp.parameters()])
        if streams is None:
            assert max(seen) == (3 if rank > 8 else 2), "the large buckets were expected to be dealt over streams"
        results.append(grads_per_step)
        del ddp
    for step, (a, b) in enumerate(zip(*results)):
        for ga, gb in zip(a, b):
            np.testing.assert_array_equal(ga, gb, err_msg="step %d" % step)
    assert _psgd_engine.gram_schmidt_give_ups() == 0
