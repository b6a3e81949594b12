"""Unbiased random-matrix compressor as a DDP communication hook.

Drop-in for the reference's communication/unbiasedMtrx_hook.py (state :47-139, hook :143-309):
every gradient worth compressing is replaced by (M Q) Q^T with Q a fresh [m, r] standard-normal
matrix per step; no orthogonalisation, no error feedback, P and Q are dropped after every step.
The reference draws Q with ``torch.randn(..., device=device)`` after ``torch.manual_seed(seed)``
(:41-45), i.e. from the device's own generator; so does this hook, so the values are whatever
torch's generator gives on the device at hand.  The two products are the gfx950 streaming kernels
``conef_psgd_mq_f32`` and ``conef_psgd_pqt_f32``.
"""
import logging

import numpy as np
import torch

from . import _bucket
from . import _lib
from ._checkpoint import Checkpointable
from ._psgd_engine import _workspace
from ._psgd_engine import should_compress as _should_compress


def set_random(vector, state, device):
    """Fills ``vector`` with N(0,1) draws under a seed taken from ``state.rng`` (:41-45).  As in
    the reference only the host generator's state is put back afterwards."""
    cur_state = torch.get_rng_state()
    torch.manual_seed(state.rng.randint(1_000_000_000))
    vector.data[:] = torch.randn(*vector.shape, device=device)
    torch.set_rng_state(cur_state)


class unbiasedMtrxState(Checkpointable):
    CHECKPOINT_FIELDS = ("iter", "rng", "total_numel_before_compression", "total_numel_after_compression")

    __slots__ = [
        "process_group",
        "matrix_approximation_rank",
        "start_powerSGD_iter",
        "min_compression_rate",
        "orthogonalization_epsilon",
        "rng",
        "p_memory_dict",
        "q_memory_dict",
        "iter",
        "total_numel_before_compression",
        "total_numel_after_compression",
        "compression_stats_logging_frequency",
        "next_stats_report",
    ]

    def __init__(
        self,
        process_group,
        matrix_approximation_rank=1,
        start_powerSGD_iter=1_000,
        min_compression_rate=2,
        random_seed=421,
        compression_stats_logging_frequency=10_000,
    ):
        self.process_group = process_group
        self.matrix_approximation_rank = matrix_approximation_rank
        self.start_powerSGD_iter = start_powerSGD_iter
        self.min_compression_rate = min_compression_rate
        self.rng = np.random.RandomState(random_seed)
        self.p_memory_dict = {}
        self.q_memory_dict = {}
        self.iter = 0
        self.total_numel_before_compression = 0
        self.total_numel_after_compression = 0
        self.compression_stats_logging_frequency = max(1, compression_stats_logging_frequency)
        self.next_stats_report = 0

    def maybe_increase_iter(self, bucket):
        if _bucket.is_last(bucket):
            self.iter += 1
        if self.iter == self.start_powerSGD_iter:
            logging.info("Start to apply PowerSGD after {} iterations.".format(self.iter))

    def compression_stats(self):
        after = self.total_numel_after_compression
        rate = self.total_numel_before_compression / after if after > 0 else 0
        return (rate, self.total_numel_before_compression, after)


def UnbiasedMtrx_hook(state: unbiasedMtrxState, bucket) -> torch.futures.Future[torch.Tensor]:
    group, world_size = _bucket.group_and_size(state.process_group)
    input_tensor = _bucket.buffer(bucket)
    if state.iter < state.start_powerSGD_iter:
        state.maybe_increase_iter(bucket)
        return _bucket.allreduce_fut(group, input_tensor, world_size)
    if world_size != 1:
        raise NotImplementedError("the MI355X low-rank hooks run the whole round on one GPU; the P and Q "
                                  "all-reduces for %d ranks are not wired up" % world_size)
    _lib.require_device_f32(input_tensor, "bucket buffer")
    lib = _lib.load()
    stream = _lib.stream_ptr(input_tensor)
    device, dtype = input_tensor.device, input_tensor.dtype
    bucket_index = _bucket.index(bucket)

    work, total_ps, total_qs = [], 0, 0
    for tensor in _bucket.gradients(bucket):
        matrix = tensor.view(tensor.shape[0], -1)
        n, m = matrix.shape
        rank = min(n, m, state.matrix_approximation_rank)
        ok, before, after = _should_compress(n, m, rank, state.min_compression_rate)
        state.total_numel_before_compression += before
        state.total_numel_after_compression += after if ok else before
        if ok:
            work.append((matrix, n, m, rank))
            total_ps += n * rank
            total_qs += m * rank

    if bucket_index not in state.p_memory_dict:
        state.p_memory_dict[bucket_index] = torch.empty(total_ps, device=device, dtype=dtype)
        state.q_memory_dict[bucket_index] = torch.empty(total_qs, device=device, dtype=dtype)
    p_mem, q_mem = state.p_memory_dict[bucket_index], state.q_memory_dict[bucket_index]
    ws = _workspace(device, stream, max([lib.conef_psgd_workspace_bytes(n, m, min(rank, 32)) for _, n, m, rank in work] or [256]))
    p_idx = q_idx = 0
    for matrix, n, m, rank in work:
        p = p_mem[p_idx: p_idx + n * rank].view(n, rank)
        q = q_mem[q_idx: q_idx + m * rank].view(m, rank)
        p_idx += n * rank
        q_idx += m * rank
        set_random(q, state, device)                                                      # :231
        if rank > 32:
            # The kernels take ranks up to 32: a wider factor goes through them in column chunks,
            # P_c = M Q_c for every chunk first (M is read, not written), then M = sum of P_c Q_c^T,
            # the first chunk's product written into M and the others added to it in chunk order.
            from ._psgd_wide import chunk_widths
            chunks, o = [], 0
            for wd in chunk_widths(rank):
                pc, qc = torch.empty(n, wd, device=device, dtype=dtype), q[:, o:o + wd].contiguous()
                _lib.check(lib.conef_psgd_mq_f32(matrix.data_ptr(), qc.data_ptr(), pc.data_ptr(), n, m, wd, ws.data_ptr(),
                                                 ws.numel(), stream), "conef_psgd_mq_f32")
                p[:, o:o + wd].copy_(pc)
                chunks.append((pc, qc, wd))
                o += wd
            part = torch.empty(n, m, device=device, dtype=dtype)
            for c, (pc, qc, wd) in enumerate(chunks):
                out = matrix if c == 0 else part
                _lib.check(lib.conef_psgd_pqt_f32(out.data_ptr(), pc.data_ptr(), qc.data_ptr(), n, m, wd, stream),
                           "conef_psgd_pqt_f32")
                if c > 0:
                    _lib.check(lib.conef_ef_passthrough_f32(matrix.data_ptr(), part.data_ptr(), n * m, stream),
                               "conef_ef_passthrough_f32")
            continue
        _lib.check(lib.conef_psgd_mq_f32(matrix.data_ptr(), q.data_ptr(), p.data_ptr(), n, m, rank, ws.data_ptr(),
                                         ws.numel(), stream),
                   "conef_psgd_mq_f32")                                                   # :232
        _lib.check(lib.conef_psgd_pqt_f32(matrix.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank, stream),
                   "conef_psgd_pqt_f32")                                                  # :292
    state.p_memory_dict.clear()
    state.q_memory_dict.clear()
    state.maybe_increase_iter(bucket)
    return _bucket.completed_future(input_tensor)
