"""The ``--grad_reducer`` factory (reference: examples/ImageClassification/get_comm_hooks.py:9-126):
every reducer name maps to the state class, hook and constructor keywords the reference passes."""
from argparse import Namespace

import pytest

ARGS = dict(start_compression_iter=10, compression_ratio=0.1, beta=0.9, sketch_size=0.2, matrix_approximation_rank=4,
            min_compression_rate=2, orthogonalization_epsilon=0)


class Net:
    def __init__(self):
        self.registered = []

    def register_comm_hook(self, state, hook):
        self.registered.append((state, hook))


def make(name, **over):
    from conef_amd.get_comm_hooks import get_comm_hooks
    net = Net()
    state = get_comm_hooks(Namespace(grad_reducer=name, **dict(ARGS, **over)), net, 0)
    return state, net


def test_allreduce_registers_nothing():
    state, net = make("allreduce")
    assert state is None and net.registered == []


def test_unknown_name_raises_like_the_reference():
    with pytest.raises(ValueError, match="Communication hook unsupported error."):
        make("topk")


def test_names_are_case_insensitive():
    state, net = make("ConEF_RandomBlock")
    assert type(state).__name__ == "RandomBlockState" and len(net.registered) == 1


@pytest.mark.parametrize("name,cls,hook,fields", [
    ("ef_randomblock", "RandomBlockState", "RandomBlock_hook",
     dict(compression_ratio=0.1, start_compression_iter=10, use_error_feedback=True, use_error_compression=False)),
    ("conef_randomblock", "RandomBlockState", "RandomBlock_hook",
     dict(compression_ratio=0.1, start_compression_iter=10, use_error_compression=True, sketch_size=0.2, beta=0.9)),
    ("unbiased_randomblock", "UnbiasedRandomBlockState", "UnbiasedRandomBlock_hook",
     dict(compression_ratio=0.1, start_compression_iter=10)),
    ("ef_powersgd", "PowerSGDState", "powerSGD_hook",
     dict(matrix_approximation_rank=4, start_powerSGD_iter=10, min_compression_rate=2, orthogonalization_epsilon=0,
          use_error_feedback=True, use_error_compression=False, warm_start=True)),
    ("hefsgd_powersgd", "hPowerSGDState", "hpowerSGD_hook",
     dict(matrix_approximation_rank=4, start_powerSGD_iter=10, use_error_compression=True, topk_ratio=0.4)),
    ("conef_powersgd", "PowerSGDState", "powerSGD_hook",
     dict(matrix_approximation_rank=4, start_powerSGD_iter=10, use_error_compression=True, sketch_size=0.2, beta=0.9)),
    ("unbiased_mtrx", "unbiasedMtrxState", "UnbiasedMtrx_hook",
     dict(matrix_approximation_rank=4, start_powerSGD_iter=10, min_compression_rate=2)),
])
def test_reducer_mapping(name, cls, hook, fields):
    state, net = make(name)
    assert type(state).__name__ == cls
    assert len(net.registered) == 1 and net.registered[0][0] is state and net.registered[0][1].__name__ == hook
    assert state.process_group is None and state.iter == 0
    for k, v in fields.items():
        assert getattr(state, k) == v, k


def test_state_constructor_errors_pass_through():
    with pytest.raises(ValueError, match="Expect `start_compression_iter` > 1"):
        make("conef_randomblock", start_compression_iter=1)
    with pytest.raises(ValueError, match="Expect `start_powerSGD_iter` > 1"):
        make("conef_powersgd", start_compression_iter=1)


def test_bert_driver_signature_without_gpu_argument():
    """examples/BertPretraining/get_comm_hooks.py:6 calls get_comm_hooks(args, model)."""
    from conef_amd.get_comm_hooks import get_comm_hooks
    net = Net()
    state = get_comm_hooks(Namespace(grad_reducer="ef_randomblock", **ARGS), net)
    assert type(state).__name__ == "RandomBlockState" and len(net.registered) == 1


def test_hooks_register_directly():
    """register_comm_hook checks the hook's annotations (bucket: GradBucket or none, return:
    Future[Tensor] or none): every hook of the package must pass as it is."""
    import inspect

    import torch
    import torch.distributed as dist

    from conef_amd import RandomBlock_hook, UnbiasedRandomBlock_hook, hPowerSGD_hook, powerSGD_hook, unbiasedMtrx_hook
    hooks = [RandomBlock_hook.RandomBlock_hook, UnbiasedRandomBlock_hook.UnbiasedRandomBlock_hook,
             hPowerSGD_hook.hpowerSGD_hook, powerSGD_hook.powerSGD_hook, powerSGD_hook.batched_powerSGD_hook,
             powerSGD_hook.C2CS_hook_v2, unbiasedMtrx_hook.UnbiasedMtrx_hook]
    for hook in hooks:
        sig = inspect.signature(hook)
        assert sig.parameters["bucket"].annotation in (inspect._empty, dist.GradBucket), hook.__name__
        assert sig.return_annotation in (inspect._empty, torch.futures.Future[torch.Tensor]), hook.__name__


def test_hook_streams_is_taken_from_the_namespace_when_present():
    """Not a flag of the reference's drivers.  Unless the namespace says otherwise: three streams above
    rank 8; up to rank 8 each bucket's size decides (0)."""
    import torch
    from conef_amd import _psgd_engine
    for name in ("ef_powersgd", "conef_powersgd", "hefsgd_powersgd"):
        assert make(name)[0].hook_streams == 0
        state = make(name)[0]
        assert _psgd_engine.streams_for(state, torch.empty(1 << 20)) == 2
        assert _psgd_engine.streams_for(state, torch.empty(1000)) == 1
        assert make(name, hook_streams=2)[0].hook_streams == 2
        assert make(name, matrix_approximation_rank=32)[0].hook_streams == 3
        assert make(name, matrix_approximation_rank=32, hook_streams=1)[0].hook_streams == 1
