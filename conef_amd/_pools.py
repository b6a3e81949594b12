"""Process-wide device memory the hooks and compressors share, and its release.

Everything here is derived data or scratch, never state a checkpoint has to carry:

  * accumulation plans (``plan``): a plan is a fixed function of (n, d, w, hash seeds, tiling), so
    every sketch of that shape on a device reads the same tables;
  * staging (``staging``): the buffer the two binned passes of a long-row sketch update hand their
    records through is live only inside one call, so there is one per (device, stream);
  * workspaces and fp32 scratch of the PowerSGD rounds, one per (device, stream);
  * side streams of ``hook_streams`` > 1.

``release()`` waits for the devices involved and drops all of it; it also runs at interpreter
exit, registered when this module is first imported, i.e. before any tool that hooks the HIP
runtime later in the process's life registers its own exit handlers (handlers run last-in
first-out), so device memory held here is returned while the runtime is still intact.
"""
import atexit
import threading

import torch

_LOCK = threading.Lock()
_PLANS = {}
_STAGING = {}
_WORKSPACES = {}
_SCRATCH = {}
_SIDE_STREAMS = {}


def plan(key, build):
    """The shared plan for ``key`` (built by ``build()`` on first use).  A build that raises
    ValueError is remembered as "no plan for this shape"."""
    with _LOCK:
        hit = _PLANS.get(key, None)
    if hit is None:
        try:
            made = build()
        except ValueError:
            made = False
        with _LOCK:
            hit = _PLANS.setdefault(key, made)
    if hit is False:
        raise ValueError("no plan for %r" % (key,))
    return hit


def _grown(pool, key, numel, dtype, device):
    buf = pool.get(key)
    if buf is None or buf.numel() < numel:
        buf = torch.empty(max(int(numel), 64), dtype=dtype, device=device)
        pool[key] = buf
    return buf


def staging(device, stream, nbytes):
    """Staging buffer of the binned sketch update on ``stream`` (grown on demand)."""
    return _grown(_STAGING, (device, stream), nbytes, torch.uint8, device)


def workspace(device, stream, nbytes):
    """Device scratch for sums that cross workgroups: one buffer per (device, stream), grown on
    demand.  Kernels that use it are ordered by that stream."""
    return _grown(_WORKSPACES, (device, stream), max(nbytes, 256), torch.uint8, device)


def scratch_f32(device, stream, numel):
    """fp32 scratch for a residual that only lives between two launches on ``stream``."""
    return _grown(_SCRATCH, (device, stream), numel, torch.float32, device)


def side_stream(device, bucket_index, count):
    """Side stream ``bucket_index % count`` of ``device`` (default priority), created on first use.
    A bucket keeps its stream from step to step, so its state is only ever touched in order."""
    pool = _SIDE_STREAMS.get((device, count))
    if pool is None:
        pool = [torch.cuda.Stream(device=device) for _ in range(count)]
        _SIDE_STREAMS[(device, count)] = pool
    return pool[bucket_index % count]


_SIDE_EVENTS = {}


def side_event(device, bucket_index, count):
    """The event by which ``side_stream(device, bucket_index, count)`` is told where to start."""
    key = (device, count, bucket_index % count)
    event = _SIDE_EVENTS.get(key)
    if event is None:
        event = _SIDE_EVENTS[key] = torch.cuda.Event()
    return event


class _SideOrder:
    __slots__ = ("issued", "latest", "waited")

    def __init__(self):
        self.issued, self.latest, self.waited = 0, None, {}


_SIDE_ORDER = {}


def side_recorded(device, event):
    """Numbers a piece of work whose end ``event`` has just been recorded on ``side_stream(device, 0, 1)``.
    The stream runs its work in order, so whoever has waited for number n has waited for all before it."""
    order = _SIDE_ORDER.get(device)
    if order is None:
        order = _SIDE_ORDER[device] = _SideOrder()
    order.issued += 1
    order.latest = event
    return order.issued


def side_wait(device, stream, number):
    """Orders ``stream`` (a torch Stream of ``device``) after the side stream's work ``number``.  A
    stream that has already waited for a later piece of work is not made to wait again: with fifty
    buckets a step, the first wait of a step (on the newest event) covers the other forty-nine, and a
    wait costs the host 7 us."""
    order = _SIDE_ORDER.get(device)
    if order is None or number is None:
        return
    key = stream.cuda_stream
    if order.waited.get(key, 0) >= number:
        return
    stream.wait_event(order.latest)
    order.waited[key] = order.issued


def held_bytes():
    """Bytes of device memory the pools hold right now, by pool (diagnostics and tests)."""
    def total(pool):
        return sum(t.numel() * t.element_size() for t in pool.values())
    plans = sum(p.device.numel() for p in _PLANS.values() if p)
    return {"plans": plans, "staging": total(_STAGING), "workspaces": total(_WORKSPACES), "scratch": total(_SCRATCH)}


def release():
    """Waits for every device that has pooled memory, then drops plans, staging, workspaces,
    scratch and side streams.  Objects still referenced elsewhere (a sketch keeps its plan) stay
    valid; whatever is needed again is rebuilt on demand."""
    with _LOCK:
        devices = {k[-1] if isinstance(k[-1], torch.device) else None for k in _PLANS}
        devices |= {k[0] for pool in (_STAGING, _WORKSPACES, _SCRATCH, _SIDE_STREAMS) for k in pool}
        devices.discard(None)
        if devices and torch.cuda.is_available():
            for dev in devices:
                try:
                    torch.cuda.synchronize(dev)
                except Exception:      # a device that is already gone has nothing left to wait for
                    pass
        for pool in (_PLANS, _STAGING, _WORKSPACES, _SCRATCH, _SIDE_STREAMS, _SIDE_ORDER, _SIDE_EVENTS):
            pool.clear()


atexit.register(release)
