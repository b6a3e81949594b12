"""The per-bucket PowerSGD round shared by powerSGD_hook and hpowerSGD_hook.

Reference flow (communication/powerSGD_hook.py:338-580, hPowerSGD_hook.py:328-570):
split the bucket into matrices worth compressing and the rest; add the remembered error; P = M Q;
orthogonalise P; Q = M^T P; M = P Q^T; remember the new error.  The all-reduces that sit between
those stages in the reference are the identity at world size 1.  Here each matrix costs three
streaming passes over its memory: the error add is fused into the first product, the residual
(dense, or count-sketched) into the last.
"""
import logging
import os

import torch
import torch.distributed as dist

from . import _bucket, _lib, _pools
from .compressors.CountSketch import HASH_A, HASH_B, DenseCS


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


def orthogonalize_all(matrices, epsilon, ws_ptr, ws_len, stream, table=None):
    """Gram-Schmidt of independent [rows, r] device matrices, side by side in as few launches as
    their shapes allow.  ``table``: what an earlier call over the same matrices returned (the host
    arrays are reused while the matrices stay where they are); returns the table."""
    import ctypes
    count = len(matrices)
    if count == 0:
        return None
    key = tuple(m.data_ptr() for m in matrices)
    if table is None or table[0] != key:
        ptrs = (ctypes.c_void_p * count)(*key)
        rows = (ctypes.c_int64 * count)(*[m.shape[0] for m in matrices])
        ranks = (ctypes.c_int32 * count)(*[m.shape[1] for m in matrices])
        table = (key, ptrs, rows, ranks)
    _, ptrs, rows, ranks = table
    rc = _lib.load().conef_gram_schmidt_batch_f32(ptrs, rows, ranks, count, float(epsilon), ws_ptr, ws_len, stream)
    _lib.check(rc, "conef_gram_schmidt_batch_f32")
    return table


def gram_schmidt_give_ups():
    """How many Gram-Schmidt workgroups on the current device have run out their bounded wait for a
    neighbouring workgroup since the library was loaded (each leaves NaN in its rows of the factor).
    The kernels that spread one factor over several workgroups rely on those workgroups being
    resident together; with several hook streams busy that is an assumption, and this is where its
    failure shows before the NaN reaches a gradient.  Waits for the device.  With CONEF_CHECK_GS=1
    every hook call ends with this check and raises."""
    import ctypes
    count = ctypes.c_int64(0)
    _lib.check(_lib.load().conef_gram_schmidt_give_ups(ctypes.byref(count)), "conef_gram_schmidt_give_ups")
    return count.value


# one buffer per (device, stream), grown on demand; held and released by conef_amd._pools
_workspace = _pools.workspace
_scratch_f32 = _pools.scratch_f32


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


def topk_sparsify_all(tensors, topk_ratio, table=None, stream=None):
    """``topk_sparsify`` of every tensor of a list (one stream, one device) with each pass a
    single launch over all of them.  ``table`` is what an earlier call over the same tensors
    returned: the host arrays and the workspace are reused while the tensors stay where they are.
    ``stream``: the raw stream to launch on (torch's current one if None)."""
    import ctypes
    count = len(tensors)
    if count == 0:
        return table
    key = tuple(t.data_ptr() for t in tensors)
    lib = _lib.load()
    if table is None or table[0] != key:
        for t in tensors:
            _lib.require_device_f32(t, "err")
        ptrs = (ctypes.c_void_p * count)(*key)
        numels = (ctypes.c_int64 * count)(*[t.numel() for t in tensors])
        ks = (ctypes.c_int64 * count)(*[max(1, int(0.5 * topk_ratio * t.numel())) for t in tensors])
        # zero-filled once: the table keeps this workspace with these tensors, and the passes clear the
        # selection state behind themselves (conef_topk_sparsify_batch_kept_f32)
        ws = torch.zeros(lib.conef_topk_batch_workspace_bytes(numels, count), dtype=torch.uint8, device=tensors[0].device)
        table = (key, ptrs, numels, ks, ws, topk_ratio)
    elif table[5] != topk_ratio:
        return topk_sparsify_all(tensors, topk_ratio, None, stream)
    _, ptrs, numels, ks, ws, _ = table
    rc = lib.conef_topk_sparsify_batch_kept_f32(ptrs, numels, ks, count, ws.data_ptr(), ws.numel(),
                                                _lib.stream_ptr(tensors[0]) if stream is None else stream)
    _lib.check(rc, "conef_topk_sparsify_batch_kept_f32")
    return table


class _RoundPlan:
    """What a bucket's round needs that does not change from step to step: which tensors are
    compressed, the table of matrices the batch entry points read, the views into the P / Q
    arenas.  Built on the first step of a bucket and reused while the bucket keeps its buffer
    and layout, so that a step costs a handful of foreign calls however many tensors it has."""
    __slots__ = ("small", "sig", "errs_sig", "cs_static", "env_ahead", "env_topk_side", "env_small", "key", "shapes", "work", "passthrough", "before", "after", "total_ps", "total_qs", "arena_key", "ps",
                 "qs", "items", "count", "sketches", "fused_sketch", "batched_update", "residual_offsets",
                 "topk_table", "q_next", "q_next_ptrs", "q_next_ready", "made", "q_next_views", "items_next", "q_next_event",
                 "topk_event", "ws_need", "handoff_event", "gs_table", "topk_number", "q_next_number", "is_wide", "wide")


def _layout_signature(grads):
    """What a step compares instead of every tensor's shape: a bucket keeps its buffer, its length
    (both part of the plan's key) and its parameters for as long as DDP keeps the bucket."""
    return (len(grads), grads[0].shape, grads[-1].shape) if grads else (0, None, None)


def _build_round(state, grads, shapes, key, error_mode):
    plan = _RoundPlan()
    plan.key, plan.shapes = key, shapes
    plan.sig = _layout_signature(grads)
    plan.errs_sig = None
    plan.cs_static = False
    # switches read when the plan is built (a bucket's plan lives as long as its buffer does)
    plan.env_ahead = os.environ.get("CONEF_ROUND_AHEAD", "1") != "0"
    plan.env_topk_side = os.environ.get("CONEF_TOPK_SIDE", "1") != "0"
    plan.env_small = os.environ.get("CONEF_ROUND_SMALL", "1") != "0"
    plan.work, plan.passthrough = [], []
    plan.before = plan.after = plan.total_ps = plan.total_qs = 0
    for tensor in grads:                                            # Step I (:394-418)
        matrix = tensor.view(tensor.shape[0], -1)
        n, m = matrix.shape
        rank = min(n, m, state.matrix_approximation_rank)
        ok, before, after = should_compress(n, m, rank, state.min_compression_rate)
        plan.before += before
        if ok:
            plan.work.append((matrix, n, m, rank))
            plan.total_ps += n * rank
            plan.total_qs += m * rank
            plan.after += after
        else:
            plan.passthrough.append(tensor)
            plan.after += before
    plan.count = len(plan.work)
    plan.items = (_lib.PsgdItem * max(plan.count, 1))()
    for cnt, (matrix, n, m, rank) in enumerate(plan.work):
        it = plan.items[cnt]
        it.x, it.n, it.m, it.r, it.w = matrix.data_ptr(), n, m, rank, 1
    plan.arena_key = None
    # a rank above 32 goes through column chunks of the factors (conef_amd/_psgd_wide.py)
    plan.is_wide = any(rank > 32 for _, _, _, rank in plan.work)
    plan.wide = None
    plan.small = None               # (mode1, mode3) -> whether the bucket's round runs as one launch (a bucket of small matrices)
    plan.sketches = []
    plan.fused_sketch = False
    plan.batched_update = False
    plan.topk_table = None
    plan.topk_event = None          # the side stream's top-k of this bucket's errors, to be waited for by its next round
    plan.topk_number = None         # the side stream's running number of that top-k (None: nothing to wait for)
    plan.q_next_number = None       # likewise for the Gram-Schmidt of the next round's Q factors
    plan.ws_need = None             # bytes of workspace the batch entry points ask for (a function of the table's shapes)
    plan.handoff_event = None       # recorded on the hook's stream where the side stream may start (one event, reused)
    plan.gs_table = None            # host arrays of the side stream's Gram-Schmidt call
    # Second buffer for the Q factors, orthogonalised at the end of a round for the bucket's next
    # round (conef_psgd_round_ahead_f32).  Derived data: q_memory_dict keeps what the reference
    # keeps, and the flag falls with the plan whenever the state is replaced.
    plan.q_next = plan.q_next_ptrs = None
    plan.q_next_ready = False
    plan.made = None
    plan.residual_offsets = []
    off = 0
    for _, n, m, _ in plan.work:
        plan.residual_offsets.append(off)
        off += n * m
    plan.residual_offsets.append(off)
    return plan


_side_stream = _pools.side_stream


def topk_table_is_stale(table, tensors, topk_ratio):
    """Whether ``topk_sparsify_all`` would build a new table (and allocate its workspace) for these tensors."""
    return table is None or table[0] != tuple(t.data_ptr() for t in tensors) or table[5] != topk_ratio


def plan_for(state, bucket_index, grads, key, error_mode, device, stream_now):
    """The bucket's cached round plan, rebuilt when its buffer or layout changed.  What the
    replaced plan's last round left running on the side stream works on tensors that outlive the
    plan (the error tensors in ``state.error_dict``, the Q arena): the pending top-k is handed on
    to the new plan, whose round waits for it before it touches the errors, and the stream the
    round is about to run on (``stream_now()``) is ordered after a pending copy of the Q arena
    here, since the new plan no longer knows of it."""
    plan = state.round_cache.get(bucket_index)
    if plan is None or plan.key != key or plan.sig != _layout_signature(grads):
        old = plan
        plan = _build_round(state, grads, [t.shape for t in grads], key, error_mode)
        if old is not None:
            plan.topk_number, plan.topk_event = old.topk_number, old.topk_event
            if old.q_next_number is not None:
                _pools.side_wait(device, stream_now(), old.q_next_number)
        state.round_cache[bucket_index] = plan
    return plan


def wait_for_side_topk(plan, device, stream_now):
    """Orders the stream a round is about to run on after the side stream's top-k of the bucket's
    error tensors from its previous round, if one may still be running."""
    if plan.topk_number is not None:
        _pools.side_wait(device, stream_now(), plan.topk_number)
        plan.topk_number = None


def settle(state):
    """Orders torch's current stream after whatever the rounds of ``state`` left running on a side
    stream that touches the state's own tensors (the top-k of the error tensors): to be called
    before those tensors are read or written from outside the hooks."""
    for plan in getattr(state, "round_cache", {}).values():
        event = getattr(plan, "topk_event", None)
        if event is not None:
            torch.cuda.current_stream().wait_event(event)


def run_round(state, bucket, error_mode):
    """One hook call.  error_mode: None | 'ef' (dense, whole bucket) | 'conef' (count sketch per
    matrix) | 'conef_v2' (count sketch over the [m,n] re-view of each matrix's memory,
    powerSGD_hook.py:918-920,1074-1076) | 'topk' (dense per matrix, magnitude-sparsified).

    With ``state.hook_streams`` = N > 1 the buckets of a step are dealt out over N streams: bucket
    i with i % N == 0 stays on the stream the hook was called on, the others go to one of N - 1 side
    streams.  A side stream first waits for the hook's stream (the gradients are ready there), and
    the returned Future carries the side stream's completion event, which is what DDP (or any caller
    of ``wait()``) orders its own stream after.  (Handing a bucket to another stream costs the host
    about 30 us, more than issuing its four launches: every N-th bucket is spared that.)"""
    input_tensor = _bucket.buffer(bucket)
    streams = streams_for(state, input_tensor)
    if streams <= 1 or not input_tensor.is_cuda or state.iter < state.start_powerSGD_iter:
        return _run_round(state, bucket, error_mode, 1)
    device = input_tensor.device
    index = _bucket.index(bucket)
    lane = index % streams
    if lane == 0:
        return _run_round(state, bucket, error_mode, streams)
    side = _side_stream(device, lane - 1, streams - 1)
    # the side stream starts where the hook's stream is now (one event per side stream, recorded again
    # for every bucket: a wait takes the event as it is when the wait is enqueued)
    event = _pools.side_event(device, lane - 1, streams - 1)
    event.record(_lib.current_stream(device))
    side.wait_event(event)
    input_tensor.record_stream(side)
    with _lib.on_stream(side):
        return _run_round(state, bucket, error_mode, streams)


AUTO_STREAMS_MIN_NUMEL = 1 << 20


def streams_for(state, input_tensor):
    """Streams the rounds of this state's buckets are dealt out over (the hook's own included).
    ``state.hook_streams`` 0 leaves it to the bucket's size: buckets of a million elements or more
    alternate between the hook's stream and a side stream (a bucket's launches that are mostly
    latency then overlap the neighbouring bucket's streaming passes), a smaller one stays on the
    hook's stream, where handing it over would cost more than it brings."""
    streams = int(getattr(state, "hook_streams", 1) or 0)
    if streams == 0:
        streams = 2 if input_tensor.numel() >= AUTO_STREAMS_MIN_NUMEL else 1
    return streams


def _run_round(state, bucket, error_mode, streams=1):
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
    base_ptr = input_tensor.data_ptr()

    dense_err = None
    if error_mode == "ef":
        if bucket_index not in state.error_dict:
            logging.info("A zero tensor of length {} that represents local error is created.".format(total_length))
            state.error_dict[bucket_index] = torch.zeros(total_length, device=device, dtype=dtype)
        dense_err = state.error_dict[bucket_index]
    elif error_mode in ("conef", "conef_v2", "topk"):
        state.error_dict.setdefault(bucket_index, {})
    errs = state.error_dict.get(bucket_index)

    grads = _bucket.gradients(bucket)
    key = (base_ptr, total_length, error_mode, state.matrix_approximation_rank, state.min_compression_rate,
           getattr(state, "sketch_size", None), dense_err.data_ptr() if dense_err is not None else 0)
    plan = plan_for(state, bucket_index, grads, key, error_mode, device, lambda: _lib.current_stream(device))
    work, items, count = plan.work, plan.items, plan.count
    state.total_numel_before_compression += plan.before
    state.total_numel_after_compression += plan.after

    # Step III: P and Q arenas, reused across iterations under warm start (:434-471)
    need_randomize_qs = (not state.warm_start) or bucket_index not in state.p_memory_dict
    if need_randomize_qs:
        if state.warm_start:
            logging.info("Allocating contiguous memory of length {} for Ps, and of length {} for Qs, "
                         "respectively.".format(plan.total_ps, plan.total_qs))
        state.p_memory_dict[bucket_index] = torch.empty(plan.total_ps, device=device, dtype=dtype)
        state.q_memory_dict[bucket_index] = torch.empty(plan.total_qs, device=device, dtype=dtype)
    p_mem, q_mem = state.p_memory_dict[bucket_index], state.q_memory_dict[bucket_index]
    if plan.arena_key != (p_mem.data_ptr(), q_mem.data_ptr()):
        plan.ps, plan.qs, p_idx, q_idx = [], [], 0, 0
        for cnt, (matrix, n, m, rank) in enumerate(work):
            plan.ps.append(p_mem[p_idx: p_idx + n * rank].view(n, rank))
            plan.qs.append(q_mem[q_idx: q_idx + m * rank].view(m, rank))
            items[cnt].p, items[cnt].q = plan.ps[-1].data_ptr(), plan.qs[-1].data_ptr()
            p_idx += n * rank
            q_idx += m * rank
        plan.arena_key = (p_mem.data_ptr(), q_mem.data_ptr())
        plan.q_next = None
        plan.q_next_ready = False
        if plan.is_wide and plan.wide is None:
            from ._psgd_wide import WideRound
            plan.wide = WideRound(work, plan.ps, plan.qs, device)
    if need_randomize_qs:
        plan.q_next_ready = False
    qs = plan.qs

    # error memory of every matrix in the table (created on first use; pointers that can move
    # between steps are refreshed)
    alpha = 1 - state.beta if error_mode in ("conef", "conef_v2") else 0.0
    if error_mode == "ef":
        if items[0].err is None and count:
            for cnt, (matrix, n, m, rank) in enumerate(work):
                items[cnt].err = dense_err.data_ptr() + (matrix.data_ptr() - base_ptr)
    elif error_mode == "topk":
        for cnt, (matrix, n, m, rank) in enumerate(work):
            if cnt not in errs:
                errs[cnt] = torch.zeros_like(matrix)
            items[cnt].err = errs[cnt].data_ptr()
    elif error_mode == "conef":
        # (the dict of a bucket's sketches is only ever replaced as a whole, with the round cache cleared:
        # load_state_dict; its identity and size stand for its entries)
        if plan.errs_sig != (id(errs), len(errs)) or len(plan.sketches) != count:
            plan.sketches = []
            for cnt, (matrix, n, m, rank) in enumerate(work):
                if cnt not in errs:
                    errs[cnt] = DenseCS(n, m, state.sketch_size, device=device)
                cs = errs[cnt]
                sk_plan = cs.plan()
                it = items[cnt]
                it.w = cs.range
                it.plan_host, it.plan_dev = (sk_plan.host_ptr, sk_plan.device.data_ptr()) if sk_plan is not None else (None, None)
                plan.sketches.append((cs, sk_plan))
            plan.batched_update = all(p is not None and p.batchable for _, p in plan.sketches)
            plan.fused_sketch = state.matrix_approximation_rank <= 8 and plan.batched_update
            plan.small = None
            plan.errs_sig = (id(errs), len(errs))
            # sketches on row lists are updated in place: their cells never move.  The others swap
            # two buffers, so their pointers are refreshed every step.
            plan.cs_static = all(p is not None and p.in_place for _, p in plan.sketches)
            for cnt, (cs, _) in enumerate(plan.sketches):
                items[cnt].cs = cs.cs.data_ptr()
        if not plan.cs_static:
            for cnt, (cs, _) in enumerate(plan.sketches):
                items[cnt].cs = cs.cs.data_ptr()
    elif error_mode == "conef_v2":
        for cnt, (matrix, n, m, rank) in enumerate(work):
            if cnt not in errs:
                errs[cnt] = DenseCS(m, n, state.sketch_size, device=device)

    # the errors this round adds to may still be being sparsified on the side stream
    wait_for_side_topk(plan, device, lambda: _lib.current_stream(device))
    eps = float(state.orthogonalization_epsilon)
    if plan.ws_need is None:
        plan.ws_need = plan.wide.ws_need if plan.is_wide else max(lib.conef_psgd_batch_workspace_bytes(items, count), 256)
    ws = _workspace(device, stream, plan.ws_need)
    ws_ptr, ws_len = ws.data_ptr(), ws.numel()
    if need_randomize_qs:
        # same seeded CPU draws as the reference so every replica starts from the same Q (:479-494)
        with torch.random.fork_rng(devices=[]):
            torch.manual_seed(state.rng.randint(1_000_000_000))
            host_q = [torch.randn(*q.shape, device="cpu", dtype=dtype) for q in qs]
        for q, hq in zip(qs, host_q):
            q.copy_(hq)
    if error_mode == "conef_v2":
        # the sketch sees the same memory as m rows of n columns, so its rows are not the matrix
        # rows: query as a pass of its own (P = M Q then runs without a fused error add)
        for cnt, (matrix, n, m, rank) in enumerate(work):
            errs[cnt].query(matrix.view(m, n), alpha)
    if error_mode == "ef":
        # tensors that are not compressed: g += e, and their new error is exactly zero (:361,:558)
        for tensor in plan.passthrough:
            off = (tensor.data_ptr() - base_ptr) // 4
            cnt_el = tensor.numel()
            rc = lib.conef_ef_passthrough_f32(tensor.data_ptr(), dense_err.data_ptr() + 4 * off, cnt_el, stream)
            _lib.check(rc, "conef_ef_passthrough_f32")

    # The round itself, one foreign call: orthogonalise all Q side by side; pass 1, the error add
    # fused into P = M Q; orthogonalise all P; pass 2, Q = M^T P; pass 3, M = P Q^T with the
    # residual fused.
    mode1 = {"ef": 1, "topk": 1, "conef": 2}.get(error_mode, 0)
    residual = None
    if error_mode in ("ef", "topk"):
        mode3 = 1
    elif error_mode == "conef" and plan.fused_sketch:
        mode3 = 2
    elif error_mode in ("conef", "conef_v2"):
        # The residual goes out dense and the sketches are updated from it afterwards: ranks above
        # 8 (the low-rank product belongs on the matrix cores), sketches whose plan is not a row
        # list, and the re-viewed sketches of C2CS_hook_v2.
        residual = _scratch_f32(device, stream, max(plan.residual_offsets[-1], 1))
        for cnt in range(count):
            items[cnt].err = residual.data_ptr() + 4 * plan.residual_offsets[cnt]
        # every sketch of the bucket from its matrix's residual in one more launch, when the plans allow
        mode3 = 3 if error_mode == "conef" and plan.batched_update else 1
    else:
        mode3 = 0
    if plan.is_wide:
        # A rank above 32: the error is added in passes of its own, the round runs on column chunks of
        # the factors, and the residual leaves the round dense (a sketch is updated from it below).
        plan.small = ((mode1, mode3), False)
        plan.q_next_ready = False
        if mode3 == 3:
            mode3 = 1
        for cnt, (matrix, n, m, rank) in enumerate(work):
            if mode1 == 1:
                _lib.check(lib.conef_ef_passthrough_f32(matrix.data_ptr(), items[cnt].err, n * m, stream), "conef_ef_passthrough_f32")
            elif mode1 == 2:
                errs[cnt].query(matrix, alpha)
        dest = [items[cnt].err if mode3 == 1 else None for cnt in range(count)]
        plan.wide.run(lib, plan.ps, plan.qs, dest, eps, ws_ptr, ws_len, stream)
    elif plan.small is None or plan.small[0] != (mode1, mode3):
        # a bucket of small matrices (every one fits a workgroup's LDS with its factors): the whole round in one launch
        fits = bool(count and mode3 in (0, 1, 2) and plan.env_small
                    and lib.conef_psgd_round_small_fits(items, count, mode1, mode3, HASH_A, HASH_B))
        plan.small = ((mode1, mode3), fits)
    if plan.is_wide:
        pass
    elif plan.small[1]:
        plan.q_next_ready = False
        rc = lib.conef_psgd_round_small_f32(items, count, mode1, mode3, float(alpha), float(state.beta) if mode3 == 2 else 0.0,
                                            eps, HASH_A, HASH_B, ws_ptr, ws_len, stream)
        _lib.check(rc, "conef_psgd_round_small_f32")
    elif (state.matrix_approximation_rank > 8 and state.warm_start and count
            and streams <= 1 and plan.env_ahead):
        # Ranks on the matrix cores: the round as its separate launches, with the Gram-Schmidt of the new
        # Q factors (which the reference runs at the start of the bucket's next round,
        # powerSGD_hook.py:496-497: 27-35 us of dependent steps on a few workgroups) on a side stream,
        # out of place, while this stream goes on with M = P Q^T and the sketch update.  The next round
        # of this bucket waits for it.  CONEF_ROUND_AHEAD=0 keeps everything on one stream; so does
        # hook_streams > 1, where buckets already run side by side (measured: the two together are slower).
        _round_with_q_on_the_side(state, plan, lib, items, count, mode1, mode3, alpha, eps, ws_ptr, ws_len, stream,
                                  device, q_mem, qs)
    elif (mode3 in (0, 1, 2) and state.matrix_approximation_rank <= 8 and state.warm_start and count and count <= 24
            and plan.env_ahead):
        # The bucket's next round starts by orthogonalising the Q factors this round leaves
        # (powerSGD_hook.py:496-497): a few workgroups and an idle machine.  Workgroups of this
        # round's last launch do it instead, into a second buffer, where the kernel allows
        # (CONEF_ROUND_AHEAD=0 keeps the reference's order, for comparisons).
        import ctypes
        if plan.q_next is None:
            plan.q_next = torch.empty_like(q_mem)
            offs, off = [], 0
            for _, n, m, rank in work:
                offs.append(off)
                off += m * rank
            plan.q_next_ptrs = (ctypes.c_void_p * count)(*[plan.q_next.data_ptr() + 4 * o for o in offs])
            plan.made = ctypes.c_int32(0)
            plan.q_next_ready = False
        flags = (1 if plan.q_next_ready else 0) | 2
        rc = lib.conef_psgd_round_ahead_f32(items, count, mode1, mode3, float(alpha), float(state.beta) if mode3 == 2 else 0.0, eps, HASH_A,
                                            HASH_B, plan.q_next_ptrs, flags, ctypes.byref(plan.made), ws_ptr, ws_len,
                                            stream)
        _lib.check(rc, "conef_psgd_round_ahead_f32")
        plan.q_next_ready = bool(plan.made.value)
    else:
        plan.q_next_ready = False
        rc = lib.conef_psgd_round_f32(items, count, mode1, mode3, float(alpha), float(state.beta) if mode3 in (2, 3) else 0.0,
                                      eps, HASH_A, HASH_B, ws_ptr, ws_len, stream)
        _lib.check(rc, "conef_psgd_round_f32")
    if error_mode == "topk":
        if count and streams <= 1 and plan.env_ahead and plan.env_topk_side:
            # The sparsification only touches the error tensors, which nobody reads before this bucket's
            # next round: it runs on a side stream while this stream goes on with the next bucket (five
            # streaming passes next to launches that are mostly latency).  Same kernels, same values.
            if plan.handoff_event is None:
                plan.handoff_event = torch.cuda.Event()
            plan.handoff_event.record(_lib.current_stream(device))
            side = _pools.side_stream(device, 0, 1)
            side.wait_event(plan.handoff_event)
            tensors = [errs[cnt] for cnt in range(count)]
            # a table that no longer fits (an error tensor was replaced, another ratio) is a new one: its
            # workspace has to be allocated and zero-filled on the stream whose kernels rely on the zeros
            if topk_table_is_stale(plan.topk_table, tensors, state.topk_ratio):
                with _lib.on_stream(side):
                    plan.topk_table = topk_sparsify_all(tensors, state.topk_ratio, None)
                # memory the side stream works on must not go back to the allocator under it
                for t in tensors:
                    t.record_stream(side)
                plan.topk_table[4].record_stream(side)
            else:
                plan.topk_table = topk_sparsify_all(tensors, state.topk_ratio, plan.topk_table, side.cuda_stream)
            if plan.topk_event is None:
                plan.topk_event = torch.cuda.Event()
            plan.topk_event.record(side)
            plan.topk_number = _pools.side_recorded(device, plan.topk_event)
        else:
            plan.topk_table = topk_sparsify_all([errs[cnt] for cnt in range(count)], state.topk_ratio, plan.topk_table)
    elif residual is not None and mode3 != 3:
        for cnt, (matrix, n, m, rank) in enumerate(work):
            res = residual[plan.residual_offsets[cnt]: plan.residual_offsets[cnt + 1]]
            errs[cnt].update(res.view(n, m) if error_mode == "conef" else res.view(m, n), state.beta)

    if not state.warm_start:
        state.p_memory_dict.clear()
        state.q_memory_dict.clear()

    if os.environ.get("CONEF_CHECK_GS", "0") == "1" and gram_schmidt_give_ups():
        raise RuntimeError("a Gram-Schmidt workgroup gave up waiting for its neighbours: the factors of bucket %d hold NaN"
                           % bucket_index)
    state.maybe_increase_iter(bucket)
    return _bucket.completed_future(input_tensor)


def _round_with_q_on_the_side(state, plan, lib, items, count, mode1, mode3, alpha, eps, ws_ptr, ws_len, stream, device,
                              q_mem, qs):
    import ctypes
    main = _lib.current_stream(device)
    fresh_q_next = plan.q_next is None
    if fresh_q_next:
        plan.q_next = torch.empty_like(q_mem)
        plan.q_next_views, off = [], 0
        for q in qs:
            plan.q_next_views.append(plan.q_next[off: off + q.numel()].view(q.shape))
            off += q.numel()
        plan.items_next = (type(items[0]) * count)()      # the same table with the first product reading the second buffer
        plan.q_next_event = torch.cuda.Event()
        plan.q_next_ready = False
    if plan.q_next_ready:
        for k in range(count):                              # pointers of the table can move between steps (err, cs)
            ctypes.memmove(ctypes.byref(plan.items_next[k]), ctypes.byref(items[k]), ctypes.sizeof(items[k]))
            plan.items_next[k].q = plan.q_next_views[k].data_ptr()
        _pools.side_wait(device, main, plan.q_next_number)
        first = plan.items_next
    else:
        orthogonalize_all(qs, eps, ws_ptr, ws_len, stream)
        first = None
    # P = M Q, P orthogonalised, Q = M^T P
    rc = lib.conef_psgd_products_f32(items, first, count, mode1, float(alpha), eps, HASH_A, HASH_B, ws_ptr, ws_len, stream)
    _lib.check(rc, "conef_psgd_products_f32")
    # the new Q is final: orthogonalise a copy of it on the side
    if plan.handoff_event is None:
        plan.handoff_event = torch.cuda.Event()
    plan.handoff_event.record(main)
    side = _pools.side_stream(device, 0, 1)
    side.wait_event(plan.handoff_event)
    if fresh_q_next:
        plan.q_next.record_stream(side)       # memory the side stream works on must not go back to the allocator under it
    with _lib.on_stream(side):
        plan.q_next.copy_(q_mem, non_blocking=True)
        side_ws = _workspace(device, side.cuda_stream, max(ws_len, 256))
    plan.gs_table = orthogonalize_all(plan.q_next_views, eps, side_ws.data_ptr(), side_ws.numel(), side.cuda_stream,
                                      plan.gs_table)
    plan.q_next_event.record(side)
    plan.q_next_number = _pools.side_recorded(device, plan.q_next_event)
    plan.q_next_ready = True
    beta = float(state.beta) if mode3 in (2, 3) else 0.0
    rc = lib.conef_psgd_pqt_batch_f32(items, count, 1 if mode3 == 3 else mode3, beta if mode3 == 2 else 0.0, HASH_A, HASH_B,
                                      stream)
    _lib.check(rc, "conef_psgd_pqt_batch_f32")
    if mode3 == 3:
        rc = lib.conef_psgd_sketch_update_batch_f32(items, count, beta, HASH_A, HASH_B, stream)
        _lib.check(rc, "conef_psgd_sketch_update_batch_f32")


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
    if rank > side:
        raise ValueError("matrix_approximation_rank %d does not fit a %d x %d matrix" % (rank, side, side))

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
    if rank > 32:
        # column chunks of the factors (conef_amd/_psgd_wide.py), built once per bucket and square buffer
        from ._psgd_wide import WideRound
        wide = state.round_cache.get(bucket_index)
        if wide is None or wide[0] != (square.data_ptr(), side, rank):
            wide = ((square.data_ptr(), side, rank), WideRound([(square.view(side, side), side, side, rank)], [p], [q], device))
            state.round_cache[bucket_index] = wide
        ws = _workspace(device, stream, wide[1].ws_need)
        if err is not None:
            _lib.check(lib.conef_ef_passthrough_f32(square.data_ptr(), err.data_ptr(), padded, stream), "conef_ef_passthrough_f32")
        wide[1].run(lib, [p], [q], [err.data_ptr() if err is not None else None], eps, ws.data_ptr(), ws.numel(), stream)
        if square is not input_tensor:
            input_tensor.copy_(square[:total_length])
        if not state.warm_start:
            state.p_memory_dict.clear()
            state.q_memory_dict.clear()
        state.maybe_increase_iter(bucket)
        return _bucket.completed_future(input_tensor)
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
