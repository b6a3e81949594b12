"""Random contiguous-block compressor with (contractive) error feedback as a DDP communication hook.

Drop-in for the reference's communication/RandomBlock_hook.py: same ``RandomBlockState`` constructor
arguments, defaults, fields and error messages (:60-115), same ``RandomBlock_hook(state, bucket)``
contract (:138-295).  What differs is how a step executes: for each >=2-D gradient the reference
issues a query kernel, a clone, slice copies, memsets, an update kernel, a zero_ and copies back;
here one fused gfx950 kernel reads the gradient once and leaves payload, decompressed gradient and
new error state behind, and all tensors of a bucket go through it in ONE foreign call
(``conef_randblock_step_batch_f32``) from a table that is built once per bucket.
"""
import logging

import numpy as np
import torch
import torch.distributed as dist

from . import _bucket
from . import _lib
from . import _pools
from ._checkpoint import Checkpointable
from .compressors.CountSketch import HASH_A, HASH_B, DenseCS


class RandomBlockState(Checkpointable):
    """Hyper-parameters and per-bucket state (reference: RandomBlock_hook.py:16-135).

    ``compression_ratio`` is the fraction of entries of every >=2-D gradient that is kept;
    ``start_compression_iter`` (must exceed 1 because DDP rebuilds its buckets after the first
    iteration) is the number of leading iterations that use a plain all-reduce;
    ``use_error_compression`` stores the residual in a count sketch of ``sketch_size * columns``
    buckets per row with decay ``beta`` instead of a dense tensor.
    """

    CHECKPOINT_FIELDS = ("iter", "rng", "error_dict")

    __slots__ = [
        "process_group",
        "compression_ratio",
        "start_compression_iter",
        "n_blocks",
        "use_error_compression",
        "beta",
        "sketch_size",
        "use_error_feedback",
        "rng",
        "error_dict",
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
        use_error_compression=False,
        beta=0.9,
        sketch_size=0.5,
        use_error_feedback=True,
        random_seed=42,
        compression_stats_logging_frequency=10_000,
    ):
        if start_compression_iter <= 1:
            raise ValueError(
                "Expect `start_compression_iter` > 1 if `use_error_feedback`, "
                "because gradient compression can only be applied after the first two iterations in DDP."
            )
        if (not use_error_feedback) and use_error_compression:
            raise ValueError(
                "Expect `use_error_feedback` = True if `use_error_compression`, "
                "otherwise there is no need to use error compression."
            )
        self.process_group = process_group
        self.compression_ratio = compression_ratio
        self.start_compression_iter = start_compression_iter
        self.use_error_feedback = use_error_feedback
        self.use_error_compression = use_error_compression
        self.beta = beta
        self.sketch_size = sketch_size
        self.rng = np.random.RandomState(random_seed)
        self.error_dict = {}
        self.iter = 0
        self.compression_stats_logging_frequency = max(1, compression_stats_logging_frequency)
        self.next_stats_report = 0
        self.compressed_tensor_memory = {}
        self.round_cache = {}     # bucket index -> launch table (derived data, never checkpointed)

    def maybe_increase_iter(self, bucket):
        # the last bucket to be reduced closes an iteration
        if _bucket.is_last(bucket):
            self.iter += 1
        if self.iter == self.start_compression_iter:
            logging.info("Start to apply PowerSGD after {} iterations.".format(self.iter))

    def clean_error(self):
        """Zeroes the sketches (reference :129-135; only meaningful with error compression)."""
        if self.use_error_feedback and self.use_error_compression:
            for errors in self.error_dict.values():
                for cs in errors or ():
                    cs.clean(0)


def _block_size(state, numel):
    return max(1, int(state.compression_ratio * numel))      # RandomBlock_hook.py:207,216


class _BucketTable:
    """What a bucket's step needs, worked out once: the >= 2-D gradients as matrices, their block
    sizes, payload slices and the item table the batch entry point reads.  Rebuilt when the
    bucket's buffer or layout changes."""
    __slots__ = ("key", "shapes", "matrices", "uncompressed", "numels", "blocks", "offsets", "items", "count")


def _build_table(state, grads, shapes, key, device, bucket_index, errors):
    t = _BucketTable()
    t.key, t.shapes = key, shapes
    t.matrices = [g.view(g.shape[0], -1) for g in grads if g.ndimension() > 1]
    t.uncompressed = [g for g in grads if g.ndimension() <= 1]
    t.numels = [m.numel() for m in t.matrices]
    t.blocks = [_block_size(state, n) for n in t.numels]
    t.count = len(t.matrices)
    for cnt, matrix in enumerate(t.matrices):
        if len(errors) <= cnt:
            if state.use_error_compression:
                errors.append(DenseCS(matrix.shape[0], matrix.shape[1], state.sketch_size, device=device))
            else:
                errors.append(torch.zeros_like(matrix))
    if bucket_index not in state.compressed_tensor_memory:
        state.compressed_tensor_memory[bucket_index] = torch.empty(sum(t.blocks), dtype=torch.float32, device=device)
    payload_all = state.compressed_tensor_memory[bucket_index]
    t.items = (_lib.RandBlockItem * max(t.count, 1))()
    t.offsets, idx = [], 0
    for cnt, (matrix, block) in enumerate(zip(t.matrices, t.blocks)):
        it = t.items[cnt]
        it.x = matrix.data_ptr()
        it.payload = payload_all.data_ptr() + 4 * idx
        it.n, it.m, it.block = matrix.shape[0], matrix.shape[1], block
        t.offsets.append(idx)
        idx += block
    return t


def RandomBlock_hook(state: RandomBlockState, bucket) -> torch.futures.Future[torch.Tensor]:
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

    if not state.use_error_feedback:
        # the reference indexes error_dict[bucket_index] unconditionally (:215) although it only
        # creates the entry under use_error_feedback (:158-160); same failure, same exception type
        raise KeyError(bucket_index)
    errors = state.error_dict.setdefault(bucket_index, [])

    grads = _bucket.gradients(bucket)
    shapes = [g.shape for g in grads]
    payload_all = state.compressed_tensor_memory.get(bucket_index)
    key = (input_tensor.data_ptr(), input_tensor.numel(), bool(state.use_error_compression), state.compression_ratio,
           payload_all.data_ptr() if payload_all is not None else 0)
    table = state.round_cache.get(bucket_index)
    if table is None or table.key != key or table.shapes != shapes or len(errors) < table.count:
        table = _build_table(state, grads, shapes, key, device, bucket_index, errors)
        payload_all = state.compressed_tensor_memory[bucket_index]
        table.key = key[:4] + (payload_all.data_ptr(),)
        state.round_cache[bucket_index] = table
    items, count = table.items, table.count

    alpha = 1 - state.beta          # python double, rounded to fp32 at the boundary (reference :190)
    starts = []
    randint = state.rng.randint     # RandomState.choice(n) of an int n draws randint(0, n): same stream (:218)
    written = []
    staging = None
    if state.use_error_compression:
        # One staging buffer serves every binned sketch of the bucket (the launches run one after the
        # other on this stream): it is sized for the largest of them before any pointer is taken, since
        # the pool replaces its buffer when it has to grow.
        need = max((p.workspace_bytes for p in (errors[cnt].plan() for cnt in range(count))
                    if p is not None and not p.in_place), default=0)
        if need:
            staging = _pools.staging(device, stream, need).data_ptr()
    for cnt in range(count):
        it = items[cnt]
        start = int(randint(0, table.numels[cnt]))             # one draw per tensor, in bucket order (:218)
        it.start = start
        starts.append(start)
        error = errors[cnt]
        if state.use_error_compression:
            plan = error.plan()
            it.w = error.range
            it.cs_in = error.cs.data_ptr()
            if plan is not None:
                # the binned step reads the old sketch while it writes the new one
                out = error.cs if plan.in_place else error.spare_buffer()
                it.plan_host, it.plan_dev = plan.host_ptr, plan.device.data_ptr()
                it.staging = None if plan.in_place else staging
            else:
                out = error.next_buffer()
                it.plan_host = it.plan_dev = it.staging = None
            it.cs_out = out.data_ptr()
            written.append(out)
        else:
            it.err = error.data_ptr()
    if count:
        rc = lib.conef_randblock_step_batch_f32(items, count, 2 if state.use_error_compression else 1, float(alpha),
                                                float(state.beta), HASH_A, HASH_B, stream)
        _lib.check(rc, "conef_randblock_step_batch_f32")
    for error, out in zip(errors, written):
        error.commit(out)

    if world_size == 1:
        # every all-reduce is the identity: the fused kernels already left zeros + block in place
        state.maybe_increase_iter(bucket)
        return _bucket.completed_future(input_tensor)

    # More than one rank (not exercised on the single-GPU boxes this was developed on): average the
    # small tensors and the payload, then put the averaged block back.
    uncompressed = table.uncompressed
    spans = [(m, st, bl, off) for m, st, bl, off in zip(table.matrices, starts, table.blocks, table.offsets)]
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
        for matrix, start, block, off in spans:
            rc = lib.conef_randblock_scatter_f32(matrix.data_ptr(), reduced[off: off + block].data_ptr(),
                                                 matrix.numel(), start, block, s)
            _lib.check(rc, "conef_randblock_scatter_f32")
        state.maybe_increase_iter(bucket)
        return input_tensor

    return fut.then(unpack_small_and_reduce_payload).then(decompress)
