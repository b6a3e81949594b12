"""The per-bucket PowerSGD round shared by powerSGD_hook and hpowerSGD_hook.

Reference flow (communication/powerSGD_hook.py:338-580, hPowerSGD_hook.py:328-570):
split the bucket into matrices worth compressing and the rest; add the remembered error; P = M Q;
orthogonalise P; Q = M^T P; M = P Q^T; remember the new error.  The all-reduces that sit between
those stages in the reference are the identity at world size 1.  Here each matrix costs three
streaming passes over its memory: the error add is fused into the first product, the residual
(dense, or count-sketched) into the last.
"""
import logging

import torch
import torch.distributed as dist

from . import _bucket, _lib
from .compressors.CountSketch import DenseCS


def should_compress(num_rows, num_cols, matrix_approximation_rank, min_compression_rate):
    """(worth compressing?, uncompressed count, compressed count) - powerSGD_hook.py:46-70."""
    uncompressed_size = num_rows * num_cols
    compressed_size = (num_rows + num_cols) * matrix_approximation_rank
    return (compressed_size * min_compression_rate < uncompressed_size, uncompressed_size, compressed_size)


def orthogonalize(matrix, epsilon=0, workspace=None):
    """In-place Gram-Schmidt of a contiguous [rows, r] device matrix (powerSGD_hook.py:12-44)."""
    _lib.require_device_f32(matrix, "matrix")
    rows, r = matrix.shape
    lib = _lib.load()
    need = lib.conef_psgd_workspace_bytes(rows, 1, r)
    if workspace is None or workspace.numel() < need:
        workspace = _workspace(matrix.device, _lib.stream_ptr(matrix), need)
    rc = lib.conef_gram_schmidt_f32(matrix.data_ptr(), rows, r, float(epsilon), workspace.data_ptr(),
                                    workspace.numel(), _lib.stream_ptr(matrix))
    _lib.check(rc, "conef_gram_schmidt_f32")
    return workspace


def orthogonalize_all(matrices, epsilon, ws_ptr, ws_len, stream):
    """Gram-Schmidt of independent [rows, r] device matrices, side by side in as few launches as
    their shapes allow."""
    import ctypes
    count = len(matrices)
    if count == 0:
        return
    ptrs = (ctypes.c_void_p * count)(*[m.data_ptr() for m in matrices])
    rows = (ctypes.c_int64 * count)(*[m.shape[0] for m in matrices])
    ranks = (ctypes.c_int32 * count)(*[m.shape[1] for m in matrices])
    rc = _lib.load().conef_gram_schmidt_batch_f32(ptrs, rows, ranks, count, float(epsilon), ws_ptr, ws_len, stream)
    _lib.check(rc, "conef_gram_schmidt_batch_f32")


_WORKSPACES = {}


def _workspace(device, stream, nbytes):
    """Device scratch for sums that cross workgroups: one buffer per (device, stream), grown on
    demand.  Kernels that use it are ordered by that stream."""
    key = (device, stream)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


_SCRATCH = {}


def _scratch_f32(device, stream, numel):
    """fp32 scratch for a residual that only lives between two launches on ``stream``."""
    key = (device, stream)
    buf = _SCRATCH.get(key)
    if buf is None or buf.numel() < numel:
        buf = torch.empty(numel, dtype=torch.float32, device=device)
        _SCRATCH[key] = buf
    return buf


def topk_sparsify(err, topk_ratio, workspace=None):
    """Keeps the max(1, int(0.5 * ratio * numel)) largest magnitudes of ``err`` in place
    (hPowerSGD_hook.py:90-97); ties on the threshold keep the lowest flat indices."""
    _lib.require_device_f32(err, "err")
    lib = _lib.load()
    numel = err.numel()
    k = max(1, int(0.5 * topk_ratio * numel))
    need = lib.conef_topk_workspace_bytes(numel)
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=err.device)
    rc = lib.conef_topk_sparsify_f32(err.data_ptr(), numel, k, workspace.data_ptr(), workspace.numel(),
                                     _lib.stream_ptr(err))
    _lib.check(rc, "conef_topk_sparsify_f32")
    return workspace


def run_round(state, bucket, error_mode):
    """One hook call.  error_mode: None | 'ef' (dense, whole bucket) | 'conef' (count sketch per
    matrix) | 'conef_v2' (count sketch over the [m,n] re-view of each matrix's memory,
    powerSGD_hook.py:918-920,1074-1076) | 'topk' (dense per matrix, magnitude-sparsified)."""
    group, world_size = _bucket.group_and_size(state.process_group)
    input_tensor = _bucket.buffer(bucket)

    if state.iter < state.start_powerSGD_iter:
        state.maybe_increase_iter(bucket)
        return _bucket.allreduce_fut(group, input_tensor, world_size)

    if world_size != 1:
        raise NotImplementedError(
            "the MI355X PowerSGD hooks run the whole round on one GPU; with %d ranks the P and Q "
            "all-reduces between the passes are not wired up" % world_size)

    _lib.require_device_f32(input_tensor, "bucket buffer")
    lib = _lib.load()
    stream = _lib.stream_ptr(input_tensor)
    device, dtype = input_tensor.device, input_tensor.dtype
    bucket_index = _bucket.index(bucket)
    total_length = input_tensor.shape[0]

    dense_err = None
    if error_mode == "ef":
        if bucket_index not in state.error_dict:
            logging.info("A zero tensor of length {} that represents local error is created.".format(total_length))
            state.error_dict[bucket_index] = torch.zeros(total_length, device=device, dtype=dtype)
        dense_err = state.error_dict[bucket_index]
    elif error_mode in ("conef", "conef_v2", "topk"):
        state.error_dict.setdefault(bucket_index, {})

    # Step I: which tensors are worth compressing (:394-418)
    base_ptr = input_tensor.data_ptr()
    work, passthrough = [], []
    total_ps, total_qs = 0, 0
    for tensor in _bucket.gradients(bucket):
        matrix = tensor.view(tensor.shape[0], -1)
        n, m = matrix.shape
        rank = min(n, m, state.matrix_approximation_rank)
        ok, before, after = should_compress(n, m, rank, state.min_compression_rate)
        state.total_numel_before_compression += before
        if ok:
            work.append((matrix, n, m, rank))
            total_ps += n * rank
            total_qs += m * rank
            state.total_numel_after_compression += after
        else:
            passthrough.append(tensor)
            state.total_numel_after_compression += before

    # Step III: P and Q arenas, reused across iterations under warm start (:434-471)
    need_randomize_qs = (not state.warm_start) or bucket_index not in state.p_memory_dict
    if need_randomize_qs:
        if state.warm_start:
            logging.info("Allocating contiguous memory of length {} for Ps, and of length {} for Qs, "
                         "respectively.".format(total_ps, total_qs))
        state.p_memory_dict[bucket_index] = torch.empty(total_ps, device=device, dtype=dtype)
        state.q_memory_dict[bucket_index] = torch.empty(total_qs, device=device, dtype=dtype)
    p_mem, q_mem = state.p_memory_dict[bucket_index], state.q_memory_dict[bucket_index]
    ps, qs, p_idx, q_idx = [], [], 0, 0
    for matrix, n, m, rank in work:
        ps.append(p_mem[p_idx: p_idx + n * rank].view(n, rank))
        qs.append(q_mem[q_idx: q_idx + m * rank].view(m, rank))
        p_idx += n * rank
        q_idx += m * rank

    eps = float(state.orthogonalization_epsilon)
    ws_bytes = max([lib.conef_psgd_workspace_bytes(n, m, rank) for _, n, m, rank in work] or [256])
    ws = _workspace(device, stream, ws_bytes)
    ws_ptr, ws_len = ws.data_ptr(), ws.numel()
    if need_randomize_qs:
        # same seeded CPU draws as the reference so every replica starts from the same Q (:479-494)
        with torch.random.fork_rng(devices=[]):
            torch.manual_seed(state.rng.randint(1_000_000_000))
            host_q = [torch.randn(*q.shape, device="cpu", dtype=dtype) for q in qs]
        for q, hq in zip(qs, host_q):
            q.copy_(hq)
    orthogonalize_all(qs, eps, ws_ptr, ws_len, stream)

    alpha = 1 - state.beta if error_mode in ("conef", "conef_v2") else 0.0
    residual = None
    if work and (error_mode == "conef_v2" or (error_mode == "conef" and state.matrix_approximation_rank > 8)):
        residual = _scratch_f32(device, stream, max(n * m for _, n, m, _ in work))
    errs = state.error_dict.get(bucket_index)

    # pass 1: error add fused into P = M Q
    for cnt, ((matrix, n, m, rank), p, q) in enumerate(zip(work, ps, qs)):
        if error_mode == "ef":
            off = (matrix.data_ptr() - base_ptr) // 4
            e = dense_err[off: off + n * m]
            rc = lib.conef_psgd_mq_ef_f32(matrix.data_ptr(), e.data_ptr(), q.data_ptr(), p.data_ptr(), n, m, rank,
                                          ws_ptr, ws_len, stream)
        elif error_mode == "conef":
            if cnt not in errs:
                errs[cnt] = DenseCS(n, m, state.sketch_size, device=device)
            cs = errs[cnt]
            plan = cs.plan()
            if plan is not None:
                rc = lib.conef_psgd_mq_conef_planned_f32(matrix.data_ptr(), cs.cs.data_ptr(), q.data_ptr(),
                                                         p.data_ptr(), plan.host_ptr, plan.device.data_ptr(), n, m,
                                                         rank, cs.range, float(alpha), cs.a, cs.b, ws_ptr, ws_len,
                                                         stream)
            else:
                rc = lib.conef_psgd_mq_conef_f32(matrix.data_ptr(), cs.cs.data_ptr(), q.data_ptr(), p.data_ptr(), n,
                                                 m, rank, cs.range, float(alpha), cs.a, cs.b, ws_ptr, ws_len, stream)
        elif error_mode == "conef_v2":
            # the sketch sees the same memory as m rows of n columns, so its rows are not the
            # matrix rows: query as a pass of its own, then the plain product
            if cnt not in errs:
                errs[cnt] = DenseCS(m, n, state.sketch_size, device=device)
            errs[cnt].query(matrix.view(m, n), alpha)
            rc = lib.conef_psgd_mq_f32(matrix.data_ptr(), q.data_ptr(), p.data_ptr(), n, m, rank, ws_ptr, ws_len,
                                       stream)
        elif error_mode == "topk":
            if cnt not in errs:
                errs[cnt] = torch.zeros_like(matrix)
            rc = lib.conef_psgd_mq_ef_f32(matrix.data_ptr(), errs[cnt].data_ptr(), q.data_ptr(), p.data_ptr(), n, m,
                                          rank, ws_ptr, ws_len, stream)
        else:
            rc = lib.conef_psgd_mq_f32(matrix.data_ptr(), q.data_ptr(), p.data_ptr(), n, m, rank, ws_ptr, ws_len,
                                       stream)
        _lib.check(rc, "conef_psgd_mq")

    if error_mode == "ef":
        # tensors that are not compressed: g += e, and their new error is exactly zero (:361,:558)
        for tensor in passthrough:
            off = (tensor.data_ptr() - base_ptr) // 4
            cnt_el = tensor.numel()
            rc = lib.conef_ef_passthrough_f32(tensor.data_ptr(), dense_err[off: off + cnt_el].data_ptr(), cnt_el,
                                              stream)
            _lib.check(rc, "conef_ef_passthrough_f32")

    # pass 2: orthogonalise all P side by side, then Q = M^T P
    orthogonalize_all(ps, eps, ws_ptr, ws_len, stream)
    for (matrix, n, m, rank), p, q in zip(work, ps, qs):
        _lib.check(lib.conef_psgd_mtp_f32(matrix.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank, ws_ptr, ws_len,
                                          stream), "conef_psgd_mtp_f32")

    # pass 3: M = P Q^T with the residual fused
    topk_ws = None
    for cnt, ((matrix, n, m, rank), p, q) in enumerate(zip(work, ps, qs)):
        if error_mode == "ef":
            off = (matrix.data_ptr() - base_ptr) // 4
            e = dense_err[off: off + n * m]
            rc = lib.conef_psgd_pqt_ef_f32(matrix.data_ptr(), e.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank,
                                           stream)
        elif error_mode == "conef" and rank > 8:
            # at these ranks the low-rank product belongs on the matrix cores: M = P Q^T with the
            # residual written out (MFMA kernel), then the sketch update as a pass of its own
            res = residual[: n * m]
            rc = lib.conef_psgd_pqt_ef_f32(matrix.data_ptr(), res.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank,
                                           stream)
            _lib.check(rc, "conef_psgd_pqt_ef_f32")
            errs[cnt].update(res.view(n, m), state.beta)
            rc = 0
        elif error_mode == "conef":
            cs = errs[cnt]
            plan = cs.plan()
            if plan is not None and plan.in_place:
                rc = lib.conef_psgd_pqt_conef_planned_f32(matrix.data_ptr(), p.data_ptr(), q.data_ptr(),
                                                          cs.cs.data_ptr(), cs.cs.data_ptr(), plan.host_ptr,
                                                          plan.device.data_ptr(), n, m, rank, cs.range,
                                                          float(state.beta), cs.a, cs.b, stream)
            else:
                out = cs.next_buffer()
                rc = lib.conef_psgd_pqt_conef_f32(matrix.data_ptr(), p.data_ptr(), q.data_ptr(), cs.cs.data_ptr(),
                                                  out.data_ptr(), n, m, rank, cs.range, float(state.beta), cs.a,
                                                  cs.b, stream)
                cs.commit(out)
        elif error_mode == "conef_v2":
            res = residual[: n * m]
            rc = lib.conef_psgd_pqt_ef_f32(matrix.data_ptr(), res.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank,
                                           stream)
            _lib.check(rc, "conef_psgd_pqt_ef_f32")
            errs[cnt].update(res.view(m, n), state.beta)
            rc = 0
        elif error_mode == "topk":
            rc = lib.conef_psgd_pqt_ef_f32(matrix.data_ptr(), errs[cnt].data_ptr(), p.data_ptr(), q.data_ptr(), n, m,
                                           rank, stream)
            _lib.check(rc, "conef_psgd_pqt_ef_f32")
            topk_ws = topk_sparsify(errs[cnt], state.topk_ratio, topk_ws)
            rc = 0
        else:
            rc = lib.conef_psgd_pqt_f32(matrix.data_ptr(), p.data_ptr(), q.data_ptr(), n, m, rank, stream)
        _lib.check(rc, "conef_psgd_pqt")

    if not state.warm_start:
        state.p_memory_dict.clear()
        state.q_memory_dict.clear()

    state.maybe_increase_iter(bucket)
    return _bucket.completed_future(input_tensor)


def run_batched_round(state, bucket):
    """batched_powerSGD_hook (powerSGD_hook.py:583-787): the whole flat bucket, zero-padded to a
    square [s,s] with s = ceil(sqrt(length)), is one matrix; dense error feedback over the padded
    length; P and Q are [s, matrix_approximation_rank]."""
    import math

    group, world_size = _bucket.group_and_size(state.process_group)
    input_tensor = _bucket.buffer(bucket)
    if state.iter < state.start_powerSGD_iter:
        state.maybe_increase_iter(bucket)
        return _bucket.allreduce_fut(group, input_tensor, world_size)
    if world_size != 1:
        raise NotImplementedError(
            "the MI355X PowerSGD hooks run the whole round on one GPU; with %d ranks the P and Q "
            "all-reduces between the passes are not wired up" % world_size)
    _lib.require_device_f32(input_tensor, "bucket buffer")
    lib = _lib.load()
    stream = _lib.stream_ptr(input_tensor)
    device, dtype = input_tensor.device, input_tensor.dtype
    bucket_index = _bucket.index(bucket)
    total_length = input_tensor.shape[0]
    side = math.isqrt(total_length)
    if side * side < total_length:
        side += 1
    rank = state.matrix_approximation_rank
    state.total_numel_before_compression += total_length
    state.total_numel_after_compression += side * rank * 2
    padded = side * side
    if rank > side or rank > 32:
        raise ValueError("matrix_approximation_rank %d does not fit a %d x %d matrix (at most 32)" % (rank, side, side))

    # the bucket buffer cannot grow in place, so a padded bucket is worked on in a square buffer
    if padded == total_length:
        square = input_tensor
    else:
        square = state.batched_square_dict.get(bucket_index)
        if square is None or square.numel() != padded:
            square = torch.empty(padded, device=device, dtype=dtype)
            state.batched_square_dict[bucket_index] = square
        square[:total_length].copy_(input_tensor)
        square[total_length:].zero_()

    err = None
    if state.use_error_feedback:
        if bucket_index not in state.error_dict:
            logging.info("A zero tensor of length {} that represents local error is created.".format(padded))
            state.error_dict[bucket_index] = torch.zeros(padded, device=device, dtype=dtype)
        err = state.error_dict[bucket_index]

    if not state.warm_start or bucket_index not in state.p_memory_dict:
        if state.warm_start:
            logging.info("Initializing low-rank tensors P and Q, each of which has a shape of {} x {}.".format(
                side, rank))
        state.p_memory_dict[bucket_index] = torch.empty(side, rank, device=device, dtype=dtype)
        with torch.random.fork_rng(devices=[]):
            torch.manual_seed(state.rng.randint(1_000_000_000))
            host_q = torch.randn(side, rank, device="cpu", dtype=dtype)
        state.q_memory_dict[bucket_index] = host_q.to(device)
    p, q = state.p_memory_dict[bucket_index], state.q_memory_dict[bucket_index]

    eps = float(state.orthogonalization_epsilon)
    ws = _workspace(device, stream, lib.conef_psgd_workspace_bytes(side, side, rank))
    ws_ptr, ws_len = ws.data_ptr(), ws.numel()
    _lib.check(lib.conef_gram_schmidt_f32(q.data_ptr(), side, rank, eps, ws_ptr, ws_len, stream),
               "conef_gram_schmidt_f32")
    if err is not None:
        rc = lib.conef_psgd_mq_ef_f32(square.data_ptr(), err.data_ptr(), q.data_ptr(), p.data_ptr(), side, side, rank,
                                      ws_ptr, ws_len, stream)
    else:
        rc = lib.conef_psgd_mq_f32(square.data_ptr(), q.data_ptr(), p.data_ptr(), side, side, rank, ws_ptr, ws_len,
                                   stream)
    _lib.check(rc, "conef_psgd_mq")
    _lib.check(lib.conef_gram_schmidt_f32(p.data_ptr(), side, rank, eps, ws_ptr, ws_len, stream),
               "conef_gram_schmidt_f32")
    _lib.check(lib.conef_psgd_mtp_f32(square.data_ptr(), p.data_ptr(), q.data_ptr(), side, side, rank, ws_ptr, ws_len,
                                      stream), "conef_psgd_mtp_f32")
    if err is not None:
        rc = lib.conef_psgd_pqt_ef_f32(square.data_ptr(), err.data_ptr(), p.data_ptr(), q.data_ptr(), side, side, rank,
                                       stream)
    else:
        rc = lib.conef_psgd_pqt_f32(square.data_ptr(), p.data_ptr(), q.data_ptr(), side, side, rank, stream)
    _lib.check(rc, "conef_psgd_pqt")
    if square is not input_tensor:
        input_tensor.copy_(square[:total_length])
    if not state.warm_start:
        state.p_memory_dict.clear()
        state.q_memory_dict.clear()
    state.maybe_increase_iter(bucket)
    return _bucket.completed_future(input_tensor)
