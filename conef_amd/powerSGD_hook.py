"""PowerSGD low-rank gradient compression with dense or count-sketched error feedback as a DDP
communication hook.

Drop-in for the reference's communication/powerSGD_hook.py: ``PowerSGDState`` keeps the
constructor arguments, defaults, fields and the ValueError of :146-239; ``powerSGD_hook`` keeps
the contract of :280-580 (gradient bucket in, Future of the same buffer out, state carried
across iterations).  The per-bucket work runs as fused gfx950 streaming kernels, see _psgd_engine.
"""
import logging

import numpy as np
import torch

from . import _bucket
from ._checkpoint import Checkpointable
from ._psgd_engine import orthogonalize as _orthogonalize  # noqa: F401  (reference name, :12)
from ._psgd_engine import run_batched_round, run_round
from ._psgd_engine import should_compress as _should_compress  # noqa: F401  (reference name, :46)


class PowerSGDState(Checkpointable):
    """Hyper-parameters and cross-iteration state.

    ``matrix_approximation_rank`` is the rank r of the P [n,r] / Q [m,r] factors;
    ``start_powerSGD_iter`` iterations run a plain all-reduce first (must exceed 1 when error
    feedback or warm start is on, because DDP rebuilds its buckets after iteration 1);
    a tensor is compressed only if (n + m) * r * ``min_compression_rate`` < n * m;
    ``use_error_feedback`` keeps the compression residual and adds it to the next gradient;
    ``use_error_compression`` keeps that residual in a count sketch (``sketch_size`` buckets per
    column, decay ``beta``) instead of a dense tensor; ``warm_start`` reuses P and Q.
    """

    CHECKPOINT_FIELDS = ("iter", "rng", "error_dict", "p_memory_dict", "q_memory_dict", "total_numel_before_compression", "total_numel_after_compression")

    __slots__ = [
        "process_group",
        "matrix_approximation_rank",
        "start_powerSGD_iter",
        "min_compression_rate",
        "orthogonalization_epsilon",
        "use_error_compression",
        "beta",
        "sketch_size",
        "use_error_feedback",
        "warm_start",
        "rng",
        "error_dict",
        "p_memory_dict",
        "q_memory_dict",
        "iter",
        "total_numel_before_compression",
        "total_numel_after_compression",
        "compression_stats_logging_frequency",
        "next_stats_report",
        "round_cache",
        "batched_square_dict",
        "hook_streams",
    ]

    def __init__(
        self,
        process_group,
        matrix_approximation_rank=1,
        start_powerSGD_iter=1_000,
        min_compression_rate=2,
        use_error_compression=False,
        beta=0.9,
        sketch_size=0.5,
        use_error_feedback=True,
        warm_start=True,
        orthogonalization_epsilon=0,
        random_seed=0,
        compression_stats_logging_frequency=10_000,
        hook_streams=None,
    ):
        logging.info(
            "PowerSGD config: matrix_approximation_rank = {}; start_powerSGD_iter = {}; "
            "min_compression_rate = {}; orthogonalization_epsilon = {}; use_error_feedback = {}; warm_start = {}; "
            "random_seed = {}; compression_stats_logging_frequency = {}".format(
                matrix_approximation_rank, start_powerSGD_iter, min_compression_rate, orthogonalization_epsilon,
                use_error_feedback, warm_start, random_seed, compression_stats_logging_frequency))
        if (use_error_feedback or warm_start) and start_powerSGD_iter <= 1:
            raise ValueError(
                "Expect `start_powerSGD_iter` > 1 if `use_error_feedback` or `warm_start` is enabled, "
                "because PowerSGD can only be applied after the first two iterations in DDP."
            )
        self.process_group = process_group
        self.matrix_approximation_rank = matrix_approximation_rank
        self.start_powerSGD_iter = start_powerSGD_iter
        self.min_compression_rate = min_compression_rate
        self.use_error_feedback = use_error_feedback
        self.warm_start = warm_start
        self.orthogonalization_epsilon = orthogonalization_epsilon
        self.rng = np.random.RandomState(random_seed)
        self.error_dict = {}
        self.p_memory_dict = {}
        self.q_memory_dict = {}
        self.iter = 0
        self.total_numel_before_compression = 0
        self.total_numel_after_compression = 0
        self.compression_stats_logging_frequency = max(1, compression_stats_logging_frequency)
        self.next_stats_report = 0
        self.round_cache = {}            # per-bucket launch tables of the engine, rebuilt when a bucket changes
        # Not in the reference: with hook_streams > 1 bucket i runs on side stream i % hook_streams
        # of its device (the Future orders the consumer after it, as the reference's Futures order it
        # after the work of the communication stream), so the latency-bound launches of one bucket
        # overlap the streaming passes of the next; bucket i with i % hook_streams == 0 stays on
        # the hook's own stream.  None: three streams above rank 8, where a bucket's round is ten
        # launches (BERT-large rank 32: 4.0 ms a step against 6.0); up to rank 8 the choice is left
        # to each bucket's size (0: two streams for buckets of a million elements or more -
        # BERT-large rank 8: 2.5 ms a step against 3.2 - one for smaller ones).
        if hook_streams is None:
            hook_streams = 3 if matrix_approximation_rank > 8 else 0
        self.hook_streams = hook_streams
        self.use_error_compression = use_error_compression
        self.beta = beta
        self.sketch_size = sketch_size
        self.batched_square_dict = {}    # batched_powerSGD_hook: the zero-padded square copy of a bucket

    def maybe_increase_iter(self, bucket):
        if _bucket.is_last(bucket):
            self.iter += 1
        if self.iter == self.start_powerSGD_iter:
            logging.info("Start to apply PowerSGD after {} iterations.".format(self.iter))

    def compression_stats(self):
        """(rate, elements before compression, elements after compression) so far."""
        after = self.total_numel_after_compression
        rate = self.total_numel_before_compression / after if after > 0 else 0
        return (rate, self.total_numel_before_compression, after)

    def clean_error(self):
        """Scales every sketch by 0 (reference :273-277: only valid with error compression)."""
        if self.use_error_feedback:
            for per_bucket in self.error_dict.values():
                for cs in per_bucket.values():
                    cs.clean(0)


def _error_mode(state):
    if not state.use_error_feedback:
        return None
    return "conef" if state.use_error_compression else "ef"


def powerSGD_hook(state: PowerSGDState, bucket) -> torch.futures.Future[torch.Tensor]:
    return run_round(state, bucket, _error_mode(state))


def batched_powerSGD_hook(state: PowerSGDState, bucket) -> torch.futures.Future[torch.Tensor]:
    """The whole bucket as one zero-padded square matrix, dense error feedback (reference :583-787)."""
    return run_batched_round(state, bucket)


def C2CS_hook_v2(state: PowerSGDState, bucket) -> torch.futures.Future[torch.Tensor]:
    """powerSGD_hook whose count sketches are built over the [m,n] re-view of each [n,m] matrix's
    memory: DenseCS(m, n, sketch_size) on matrix.view(m, n) (reference :791-1092)."""
    mode = _error_mode(state)
    return run_round(state, bucket, "conef_v2" if mode == "conef" else mode)
