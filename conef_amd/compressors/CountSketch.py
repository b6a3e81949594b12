"""Single-hash count sketch held in fp32 (reference: communication/compressors/CountSketch.py:102-182).

Same constructor, attributes (N, D, blk_size, range, cs, a, b) and methods as the reference class.
Differences a maintainer should know about:
  * the kernels are precompiled gfx950 code reached through libconef_hip.so, not CuPy/NVRTC;
  * alpha, beta, a, b travel by value, so ``a``/``b`` are Python ints, not 1-element device tensors;
  * updates run on a plan built once per sketch (no atomics, deterministic, the accumulation order
    of the reference's serial definition): per-bucket column lists when a row fits LDS, the same
    lists in column panels for longer rows of a tall matrix, two binned streaming passes (over
    groups of 8 rows) for long rows of a matrix with few of them.  The binned fused step writes
    into a second buffer and ``self.cs`` is rebound to it.  A shape no plan covers falls back to
    float atomics and says so in the log, once;
  * ``state_dict``/``load_state_dict`` round-trip (the reference's __setstate__ loses a, b).
"""
import logging
import os

import torch

from .. import _lib
from .._plan import SketchPlan

HASH_A = 994443   # CountSketch.py:112
HASH_B = 609478   # CountSketch.py:113

_WARNED = set()   # shapes that have been told about their fallback


def _warn_no_plan(n, d, w):
    """Once per shape: its updates run on float atomics (slower, and the order in which a cell
    receives its terms is no longer fixed)."""
    if (n, d, w) not in _WARNED:
        _WARNED.add((n, d, w))
        logging.warning("count sketch of a [%d, %d] tensor at width %d: no accumulation plan covers this shape, "
                        "its updates fall back to float atomics (slower; accumulation order not fixed)" % (n, d, w))


class DenseCS:
    def __init__(self, N, D, sketch_size, device=None):
        self.N = int(N)
        self.D = int(D)
        self.blk_size = 256
        self.range = max(int(D * sketch_size), 1)          # CountSketch.py:107
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.cs = torch.zeros(self.N, self.range, dtype=torch.float32, device=device)
        self.a = HASH_A
        self.b = HASH_B
        self._lib = _lib.load()
        self._inplace = bool(self._lib.conef_cs_update_inplace_ok(self.N, self.D, self.range))
        self._spare = None
        self._plan = None

    # -- persistence ---------------------------------------------------------------------------
    def state_dict(self):
        return {"N": self.N, "D": self.D, "blk_size": self.blk_size, "range": self.range,
                "cs": self.cs.detach().cpu().numpy(), "a": self.a, "b": self.b}

    def load_state_dict(self, d):
        if (d["N"], d["D"], d["range"]) != (self.N, self.D, self.range):
            raise ValueError("sketch shape mismatch: have (%d,%d,%d), state holds (%d,%d,%d)" % (
                self.N, self.D, self.range, d["N"], d["D"], d["range"]))
        self.cs.copy_(torch.from_numpy(d["cs"]).to(self.cs.device))
        self.a = int(d.get("a", HASH_A))
        self.b = int(d.get("b", HASH_B))

    @classmethod
    def from_state_dict(cls, d, device=None):
        """A sketch rebuilt from ``state_dict()`` output (width taken from the state, not recomputed)."""
        obj = cls(d["N"], d["D"], 0.0, device=device)
        obj.range = int(d["range"])
        obj.cs = torch.from_numpy(d["cs"]).to(obj.cs.device).contiguous()
        obj.a, obj.b = int(d.get("a", HASH_A)), int(d.get("b", HASH_B))
        obj._inplace = bool(obj._lib.conef_cs_update_inplace_ok(obj.N, obj.D, obj.range))
        return obj

    __getstate__ = state_dict

    def __setstate__(self, d):
        device = torch.device("cuda", torch.cuda.current_device())
        self.N, self.D, self.blk_size, self.range = d["N"], d["D"], d["blk_size"], d["range"]
        self.cs = torch.from_numpy(d["cs"]).to(device)
        self.a, self.b = int(d.get("a", HASH_A)), int(d.get("b", HASH_B))
        self._lib = _lib.load()
        self._inplace = bool(self._lib.conef_cs_update_inplace_ok(self.N, self.D, self.range))
        self._spare = None
        self._plan = None

    # -- kernels -------------------------------------------------------------------------------
    def _check(self, t, name):
        _lib.require_device_f32(t, name)
        if t.numel() != self.N * self.D:
            raise ValueError("%s has %d elements, the sketch was built for %d x %d" % (
                name, t.numel(), self.N, self.D))
        if t.device != self.cs.device:
            raise ValueError("%s is on %s, the sketch on %s" % (name, t.device, self.cs.device))

    def plan(self):
        """Accumulation plan (built on first use), or None when no kind of plan covers the shape.
        CONEF_PLAN_CHUNK / CONEF_PLAN_BIN ask for a binned plan with those tile sizes and
        CONEF_PLAN=0 disables the planned path (the kernels then accumulate with float atomics)."""
        if self._plan is None and os.environ.get("CONEF_PLAN", "1") != "0":
            chunk = int(os.environ.get("CONEF_PLAN_CHUNK", "0"))
            tbin = int(os.environ.get("CONEF_PLAN_BIN", "0"))
            if SketchPlan.applicable(self.N, self.D, self.range, chunk, tbin):
                try:
                    self._plan = SketchPlan.shared(self.N, self.D, self.range, self.a, self.b, self.cs.device, chunk, tbin)
                except ValueError:       # e.g. one bucket collects more columns than a bin image can hold
                    self._plan = False
            else:
                self._plan = False
            if self._plan is False:
                _warn_no_plan(self.N, self.D, self.range)
        if self._plan is False:
            return None
        if self._plan is not None and self._plan.key != (self.N, self.D, self.range, self.a, self.b):
            self._plan = None
            return self.plan()
        return self._plan

    def spare_buffer(self):
        if self._spare is None:
            self._spare = torch.empty_like(self.cs)
        return self._spare

    def next_buffer(self):
        """Buffer the next update writes into: ``cs`` itself when a row fits LDS, else a spare."""
        return self.cs if self._inplace else self.spare_buffer()

    def commit(self, written):
        """Makes the buffer an update wrote into the current sketch."""
        if written is not self.cs:
            self._spare, self.cs = self.cs, written

    def update(self, vec, beta):
        """cs <- cs + sketch-accumulate(vec) with the reference's per-element decay (CountSketch.py:27-67)."""
        self._check(vec, "vec")
        plan = self.plan()
        if plan is not None:
            rc = self._lib.conef_cs_update_planned_f32(vec.data_ptr(), self.cs.data_ptr(), self.cs.data_ptr(),
                                                       plan.host_ptr, plan.device.data_ptr(),
                                                       plan.workspace.data_ptr(), self.N, self.D, self.range,
                                                       float(beta), self.a, self.b, _lib.stream_ptr(vec))
            _lib.check(rc, "conef_cs_update_planned_f32")
            return
        out = self.next_buffer()
        rc = self._lib.conef_cs_update_f32(vec.data_ptr(), self.cs.data_ptr(), out.data_ptr(), self.N, self.D,
                                           self.range, float(beta), self.a, self.b, _lib.stream_ptr(vec))
        _lib.check(rc, "conef_cs_update_f32")
        self.commit(out)

    def randblock_step(self, x, payload, start, block, alpha, beta):
        """One fused RandomBlock + ConEF step on the [N,D] gradient ``x`` (in place): adds the
        unsketched error, moves the wrap-around block [start, start+block) to ``payload``, leaves
        zeros + block in ``x`` and sketches the rest."""
        self._check(x, "x")
        stream = _lib.stream_ptr(x)
        plan = self.plan()
        if plan is not None:
            # the binned step reads the old sketch while it writes the new one
            out = self.cs if plan.in_place else self.spare_buffer()
            rc = self._lib.conef_randblock_conef_step_planned_f32(
                x.data_ptr(), self.cs.data_ptr(), out.data_ptr(), payload.data_ptr(), plan.host_ptr,
                plan.device.data_ptr(), plan.workspace.data_ptr(), self.N, self.D, self.range, start, block,
                float(alpha), float(beta), self.a, self.b, stream)
            _lib.check(rc, "conef_randblock_conef_step_planned_f32")
            self.commit(out)
            return
        out = self.next_buffer()
        rc = self._lib.conef_randblock_conef_step_f32(
            x.data_ptr(), self.cs.data_ptr(), out.data_ptr(), payload.data_ptr(), self.N, self.D, self.range,
            start, block, float(alpha), float(beta), self.a, self.b, stream)
        _lib.check(rc, "conef_randblock_conef_step_f32")
        self.commit(out)

    def query(self, grad_plus_error, alpha):
        """grad_plus_error += alpha * unsketch(cs), in place (CountSketch.py:70-98)."""
        self._check(grad_plus_error, "grad_plus_error")
        plan = self.plan()
        if plan is not None:
            # buckets and signs from the plan's table instead of two hashes and modulos per column
            # (and, for a few long rows, the sketch interleaved into the plan's staging buffer first)
            staging = None if plan.in_place else plan.workspace.data_ptr()
            rc = self._lib.conef_cs_query_planned_f32(grad_plus_error.data_ptr(), self.cs.data_ptr(), plan.host_ptr,
                                                      plan.device.data_ptr(), staging, self.N, self.D, self.range,
                                                      float(alpha), self.a, self.b, _lib.stream_ptr(grad_plus_error))
            _lib.check(rc, "conef_cs_query_planned_f32")
            return
        rc = self._lib.conef_cs_query_f32(grad_plus_error.data_ptr(), self.cs.data_ptr(), self.N, self.D,
                                          self.range, float(alpha), self.a, self.b,
                                          _lib.stream_ptr(grad_plus_error))
        _lib.check(rc, "conef_cs_query_f32")

    def clean(self, alpha):
        """cs *= alpha (CountSketch.py:181-182)."""
        rc = self._lib.conef_scale_f32(self.cs.data_ptr(), self.cs.numel(), float(alpha),
                                       _lib.stream_ptr(self.cs))
        _lib.check(rc, "conef_scale_f32")
