"""Unbiased random-block compressor as a DDP communication hook.

Drop-in for the reference's communication/UnbiasedRandomBlock_hook.py (state :12-95, hook :98-219):
the kept block is divided by block/numel so the compressed gradient is unbiased; there is no error
state.  One fused gfx950 kernel per >=2-D gradient writes the scaled payload and the decompressed
gradient (``conef_randblock_unbiased_step_f32``).
"""
import logging

import numpy as np
import torch
import torch.distributed as dist

from . import _bucket
from . import _lib
from ._checkpoint import Checkpointable


class UnbiasedRandomBlockState(Checkpointable):
    CHECKPOINT_FIELDS = ("iter", "rng")

    __slots__ = [
        "process_group",
        "compression_ratio",
        "start_compression_iter",
        "n_blocks",
        "rng",
        "iter",
        "compression_stats_logging_frequency",
        "next_stats_report",
        "compressed_tensor_memory",
    ]

    def __init__(
        self,
        process_group,
        compression_ratio=0.1,
        start_compression_iter=1_000,
        random_seed=42,
        compression_stats_logging_frequency=10_000,
    ):
        if start_compression_iter <= 1:
            raise ValueError(
                "Expect `start_compression_iter` > 1 if `use_error_feedback`, "
                "because gradient compression can only be applied after the first two iterations in DDP."
            )
        self.process_group = process_group
        self.compression_ratio = compression_ratio
        self.start_compression_iter = start_compression_iter
        self.rng = np.random.RandomState(random_seed)
        self.iter = 0
        self.compression_stats_logging_frequency = max(1, compression_stats_logging_frequency)
        self.next_stats_report = 0
        self.compressed_tensor_memory = {}

    def maybe_increase_iter(self, bucket):
        if _bucket.is_last(bucket):
            self.iter += 1
        if self.iter == self.start_compression_iter:
            logging.info("Start to apply PowerSGD after {} iterations.".format(self.iter))


def UnbiasedRandomBlock_hook(state: UnbiasedRandomBlockState, bucket) -> torch.futures.Future[torch.Tensor]:
    group, world_size = _bucket.group_and_size(state.process_group)
    input_tensor = _bucket.buffer(bucket)

    if state.iter < state.start_compression_iter:
        state.maybe_increase_iter(bucket)
        return _bucket.allreduce_fut(group, input_tensor, world_size)

    _lib.require_device_f32(input_tensor, "bucket buffer")
    lib = _lib.load()
    stream = _lib.stream_ptr(input_tensor)
    device = input_tensor.device
    bucket_index = _bucket.index(bucket)

    tensors, uncompressed = [], []
    for tensor in _bucket.gradients(bucket):
        (tensors if tensor.ndimension() > 1 else uncompressed).append(tensor)

    blocks = [max(1, int(state.compression_ratio * t.nelement())) for t in tensors]
    if bucket_index not in state.compressed_tensor_memory:
        state.compressed_tensor_memory[bucket_index] = torch.empty(sum(blocks), dtype=torch.float32,
                                                                   device=device)
    payload_all = state.compressed_tensor_memory[bucket_index]

    spans, idx = [], 0
    for tensor, block in zip(tensors, blocks):
        numel = tensor.nelement()
        prob = block / numel                                    # :155
        start = int(state.rng.choice(numel))                    # :157
        payload = payload_all[idx: idx + block]
        rc = lib.conef_randblock_unbiased_step_f32(tensor.data_ptr(), payload.data_ptr(), numel, start, block,
                                                   float(prob), stream)
        _lib.check(rc, "conef_randblock_unbiased_step_f32")
        spans.append((tensor, start, block, idx))
        idx += block

    if world_size == 1:
        state.maybe_increase_iter(bucket)
        return _bucket.completed_future(input_tensor)

    # More than one rank (not exercised on the single-GPU boxes this was developed on).
    flat_small = (torch.cat([t.view(-1) for t in uncompressed]) if uncompressed
                  else torch.tensor([], device=device, dtype=input_tensor.dtype))
    fut = dist.all_reduce(flat_small, group=group, async_op=True).get_future()

    def unpack_small_and_reduce_payload(f):
        small = f.value()[0].div_(world_size)
        off = 0
        for t in uncompressed:
            t.copy_(small[off: off + t.numel()].view_as(t))
            off += t.numel()
        return dist.all_reduce(payload_all, group=group, async_op=True).get_future().wait()[0]

    def decompress(f):
        reduced = f.value().div_(world_size)
        state.compressed_tensor_memory[bucket_index] = reduced
        s = _lib.stream_ptr(input_tensor)
        for tensor, start, block, off in spans:
            rc = lib.conef_randblock_scatter_f32(tensor.data_ptr(), reduced[off: off + block].data_ptr(),
                                                 tensor.nelement(), start, block, s)
            _lib.check(rc, "conef_randblock_scatter_f32")
        state.maybe_increase_iter(bucket)
        return input_tensor

    return fut.then(unpack_small_and_reduce_payload).then(decompress)
