"""Unbiased random-block compressor as a DDP communication hook.

Drop-in for the reference's communication/UnbiasedRandomBlock_hook.py (state :12-95, hook :98-219):
the kept block is divided by block/numel so the compressed gradient is unbiased; there is no error
state.  One fused gfx950 kernel writes the scaled payload and the decompressed gradient of every
>=2-D gradient of a bucket (``conef_randblock_step_batch_f32``, mode 0: one foreign call and one
launch per bucket, from a table built once).
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
        "round_cache",
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
        self.round_cache = {}     # bucket index -> launch table (derived data, never checkpointed)

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

    grads = _bucket.gradients(bucket)
    shapes = [g.shape for g in grads]
    payload_all = state.compressed_tensor_memory.get(bucket_index)
    key = (input_tensor.data_ptr(), input_tensor.numel(), state.compression_ratio,
           payload_all.data_ptr() if payload_all is not None else 0)
    table = state.round_cache.get(bucket_index)
    if table is None or table[0] != key or table[1] != shapes:
        # worked out once per bucket: the >= 2-D gradients, their block sizes and the item table
        tensors = [g for g in grads if g.ndimension() > 1]
        uncompressed = [g for g in grads if g.ndimension() <= 1]
        numels = [t.nelement() for t in tensors]
        blocks = [max(1, int(state.compression_ratio * n)) for n in numels]
        if payload_all is None:
            payload_all = torch.empty(sum(blocks), dtype=torch.float32, device=device)
            state.compressed_tensor_memory[bucket_index] = payload_all
        items = (_lib.RandBlockItem * max(len(tensors), 1))()
        offsets, idx = [], 0
        for it, tensor, numel, block in zip(items, tensors, numels, blocks):
            it.x, it.payload = tensor.data_ptr(), payload_all.data_ptr() + 4 * idx
            it.n, it.m, it.block = tensor.shape[0], numel // tensor.shape[0], block     # prob = block / numel is formed in the library (:155)
            offsets.append(idx)
            idx += block
        table = (key[:3] + (payload_all.data_ptr(),), shapes, tensors, uncompressed, numels, blocks, offsets, items)
        state.round_cache[bucket_index] = table
    _, _, tensors, uncompressed, numels, blocks, offsets, items = table
    payload_all = state.compressed_tensor_memory[bucket_index]

    starts = []
    randint = state.rng.randint     # RandomState.choice(n) of an int n draws randint(0, n): same stream (:157)
    for it, numel in zip(items, numels):
        start = int(randint(0, numel))                          # :157
        it.start = start
        starts.append(start)
    if tensors:
        rc = lib.conef_randblock_step_batch_f32(items, len(tensors), 0, 0.0, 0.0, 0, 0, stream)
        _lib.check(rc, "conef_randblock_step_batch_f32")

    if world_size == 1:
        state.maybe_increase_iter(bucket)
        return _bucket.completed_future(input_tensor)
    spans = list(zip(tensors, starts, blocks, offsets))

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
