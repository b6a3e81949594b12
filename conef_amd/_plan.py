"""Host/device holder of an accumulation plan of a count sketch.

The plan (built once per sketch by ``conef_plan_build_host``) lists where every column goes, so
that the count-sketch update runs without atomics and adds each bucket's terms in ascending
column order: per-bucket column lists when a row fits LDS (``kind`` 1), the same lists cut into
column panels for longer rows of a tall matrix (``kind`` 2), two binned streaming passes through a
staging buffer for long rows of a matrix with few of them (``kind`` 0).
"""
import numpy as np
import torch

from . import _lib
from . import _pools


class SketchPlan:
    """plan bytes on the host (read for launch geometry) and the same bytes on the device.  Plans
    are immutable: ``SketchPlan.shared`` hands every sketch of one shape on a device the same
    object.  The staging buffer of a binned plan is not part of it (``workspace``)."""

    def __init__(self, n, d, w, a, b, device, chunk_cols=0, bin_buckets=0, sign_seeds=None):
        """``sign_seeds``: (sa, sb) of the sign hash; None means the single-hash sketch's (a + 2, b + 3)."""
        lib = _lib.load()
        nbytes = lib.conef_plan_bytes(n, d, w, chunk_cols, bin_buckets)
        if nbytes <= 0:
            raise ValueError("no plan for shape n=%d d=%d w=%d" % (n, d, w))
        self.host = np.zeros(nbytes, dtype=np.uint8)
        sa, sb = sign_seeds if sign_seeds is not None else (a + 2, b + 3)
        rc = lib.conef_plan_build_host_seeded(self.host.ctypes.data, nbytes, n, d, w, a, b, sa, sb, chunk_cols,
                                              bin_buckets)
        _lib.check(rc, "conef_plan_build_host_seeded")
        self.device = torch.from_numpy(self.host).to(device)
        self.workspace_bytes = int(lib.conef_plan_workspace_bytes(self.host.ctypes.data))
        self.kind = lib.conef_plan_kind(self.host.ctypes.data)
        self.key = (n, d, w, a, b)

    @classmethod
    def shared(cls, n, d, w, a, b, device, chunk_cols=0, bin_buckets=0, sign_seeds=None):
        """The process-wide plan for this shape, seeds, tiling and device (built on first use);
        raises ValueError when the shape has none."""
        device = torch.device(device)
        if device.type == "cuda" and device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        sa, sb = sign_seeds if sign_seeds is not None else (a + 2, b + 3)
        key = (int(n), int(d), int(w), int(a), int(b), int(sa), int(sb), int(chunk_cols), int(bin_buckets), device)
        return _pools.plan(key, lambda: cls(n, d, w, a, b, device, chunk_cols, bin_buckets, sign_seeds))

    @property
    def workspace(self):
        """Staging buffer of a binned plan for work on torch's current stream: one buffer per
        (device, stream), shared by every sketch, live only inside a call."""
        dev = self.device.device
        stream = (_lib._raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())
                  if _lib._raw_stream is not None else torch.cuda.current_stream(dev).cuda_stream)
        return _pools.staging(dev, stream, max(self.workspace_bytes, 16))

    @property
    def host_ptr(self):
        return self.host.ctypes.data

    BINNED, ROWLIST, PANELS = 0, 1, 2

    @property
    def in_place(self):
        """Whether the fused steps may write the sketch they read (row lists, whole or in panels) or
        need a second buffer and a staging buffer (binned)."""
        return self.kind in (self.ROWLIST, self.PANELS)

    @property
    def batchable(self):
        """Whether the PowerSGD batch entry points (all sketches of a bucket in one launch, the
        residual fused) take this plan: whole row lists only."""
        return self.kind == self.ROWLIST

    @staticmethod
    def applicable(n, d, w, chunk_cols=0, bin_buckets=0):
        return _lib.load().conef_plan_bytes(n, d, w, chunk_cols, bin_buckets) > 0

    def header(self):
        """Decoded header fields (for tests and diagnostics)."""
        h = self.host
        i32 = h[:128].view(np.int32)
        i64 = h[:136].view(np.int64)
        return {"n": int(i64[1]), "d": int(i64[2]), "w": int(i32[6]), "a": int(i32[7]), "b": int(i32[8]),
                "chunk_cols": int(i32[9]), "nchunks": int(i32[10]), "bin_buckets": int(i32[11]),
                "nbins": int(i32[12]), "max_bin_records": int(i32[13]), "off_pos": int(i64[7]),
                "off_seg": int(i64[8]), "off_csr": int(i64[9]), "off_ent": int(i64[10]), "off_pk": int(i64[11]),
                "total_bytes": int(i64[12]), "workspace_bytes": int(i64[13]), "kind": int(i64[14]),
                "off_order": int(i64[16])}
