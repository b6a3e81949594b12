"""Name -> (state, hook) factory for the ``--grad_reducer`` flag of the reference's training drivers.

Drop-in for examples/ImageClassification/get_comm_hooks.py:9-126 (the LanguageModeling and
MachineTranslation copies are identical; the BertPretraining one, :6-47, knows only the first four
names and takes no ``gpu`` argument, which is optional here).  ``args`` is the drivers' argparse
namespace (examples/ImageClassification/main.py:361-385): ``grad_reducer``,
``start_compression_iter`` and, depending on the reducer, ``compression_ratio``, ``beta``,
``sketch_size``, ``matrix_approximation_rank``, ``min_compression_rate``,
``orthogonalization_epsilon``.  Returns the state object, or None for plain all-reduce (no hook).
"""
from . import RandomBlock_hook as RandomBlock
from . import UnbiasedRandomBlock_hook as UnbiasedRandomBlock
from . import hPowerSGD_hook as hPowerSGD
from . import powerSGD_hook as powerSGD
from . import unbiasedMtrx_hook as UnbiasedMtrx


def _block(args):
    return dict(compression_ratio=args.compression_ratio, start_compression_iter=args.start_compression_iter)


def _lowrank(args):
    return dict(matrix_approximation_rank=args.matrix_approximation_rank,
                start_powerSGD_iter=args.start_compression_iter, min_compression_rate=args.min_compression_rate)


def _lowrank_eps(args):
    # hook_streams is not a flag of the reference's drivers: taken when the namespace has it
    return dict(_lowrank(args), orthogonalization_epsilon=args.orthogonalization_epsilon,
                hook_streams=getattr(args, "hook_streams", None))


def _sketch(args):
    return dict(use_error_compression=True, sketch_size=args.sketch_size, beta=args.beta)


# reducer name -> (state class, hook, [functions of args that supply constructor keywords])
REDUCERS = {
    "ef_randomblock": (RandomBlock.RandomBlockState, RandomBlock.RandomBlock_hook, [_block]),
    "conef_randomblock": (RandomBlock.RandomBlockState, RandomBlock.RandomBlock_hook, [_block, _sketch]),
    "unbiased_randomblock": (UnbiasedRandomBlock.UnbiasedRandomBlockState,
                             UnbiasedRandomBlock.UnbiasedRandomBlock_hook, [_block]),
    "ef_powersgd": (powerSGD.PowerSGDState, powerSGD.powerSGD_hook, [_lowrank_eps]),
    "hefsgd_powersgd": (hPowerSGD.hPowerSGDState, hPowerSGD.hpowerSGD_hook,
                        [_lowrank_eps, lambda args: dict(use_error_compression=True, topk_ratio=0.4)]),
    "conef_powersgd": (powerSGD.PowerSGDState, powerSGD.powerSGD_hook, [_lowrank_eps, _sketch]),
    "unbiased_mtrx": (UnbiasedMtrx.unbiasedMtrxState, UnbiasedMtrx.UnbiasedMtrx_hook, [_lowrank]),
}


def make_state(args):
    """(state, hook) for ``args.grad_reducer``; (None, None) for 'allreduce'."""
    name = args.grad_reducer.lower()
    if name == "allreduce":
        return None, None
    if name not in REDUCERS:
        raise ValueError("Communication hook unsupported error.")
    state_cls, hook, parts = REDUCERS[name]
    kwargs = {}
    for part in parts:
        kwargs.update(part(args))
    return state_cls(process_group=None, **kwargs), hook


def get_comm_hooks(args, net, gpu=None):
    """Registers the DDP communication hook ``args.grad_reducer`` names on ``net`` and returns
    its state (None for plain all-reduce)."""
    state, hook = make_state(args)
    if hook is not None:
        net.register_comm_hook(state, hook)
    return state
