"""Single-hash count sketch stored in fp16 (reference: communication/compressors/halfCountSketch.py:110-197).

The reference casts the whole sketch to fp32 before every kernel and back to fp16 after it.  Here
the kernels read fp16 cells, compute in fp32 and round once on the way out, which gives the same
values without the two extra passes.  ``update`` runs on a row-list plan (no atomics) when a row
fits LDS; longer rows go through an explicit fp32 staging copy.
"""
import os

import torch

from .. import _lib
from .._plan import SketchPlan
from .CountSketch import HASH_A, HASH_B


class DenseCS:
    def __init__(self, N, D, sketch_size, device=None):
        self.N = int(N)
        self.D = int(D)
        self.blk_size = 256
        self.range = max(int(D * sketch_size), 1)
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.cs = torch.zeros(self.N, self.range, dtype=torch.float16, device=device)
        self.a = HASH_A
        self.b = HASH_B
        self._lib = _lib.load()
        self._inplace = bool(self._lib.conef_cs_update_inplace_ok(self.N, self.D, self.range))
        self._plan = None

    def plan(self):
        """Row-list plan, whole or in column panels (built on first use), or None; CONEF_PLAN=0 disables it."""
        if self._plan is None and os.environ.get("CONEF_PLAN", "1") != "0":
            if SketchPlan.applicable(self.N, self.D, self.range):
                plan = SketchPlan.shared(self.N, self.D, self.range, self.a, self.b, self.cs.device)
                self._plan = plan if plan.kind in (SketchPlan.ROWLIST, SketchPlan.PANELS) else False
        return self._plan or None

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
        self._plan = None          # a plan belongs to its hash seeds

    @classmethod
    def from_state_dict(cls, d, device=None):
        obj = cls(d["N"], d["D"], 0.0, device=device)
        obj.range = int(d["range"])
        obj.cs = torch.from_numpy(d["cs"]).to(obj.cs.device).contiguous()
        obj.a, obj.b = int(d.get("a", HASH_A)), int(d.get("b", HASH_B))
        obj._inplace = bool(obj._lib.conef_cs_update_inplace_ok(obj.N, obj.D, obj.range))
        return obj

    # pickling carries the state, not the library handle (the reference class pickles too)
    __getstate__ = state_dict

    def __setstate__(self, d):
        device = torch.device("cuda", torch.cuda.current_device())
        self.N, self.D, self.blk_size, self.range = d["N"], d["D"], d["blk_size"], d["range"]
        self.cs = torch.from_numpy(d["cs"]).to(device)
        self.a, self.b = int(d.get("a", HASH_A)), int(d.get("b", HASH_B))
        self._lib = _lib.load()
        self._inplace = bool(self._lib.conef_cs_update_inplace_ok(self.N, self.D, self.range))
        self._plan = None

    def _check(self, t, name):
        _lib.require_device_f32(t, name)
        if t.numel() != self.N * self.D:
            raise ValueError("%s has %d elements, the sketch was built for %d x %d" % (
                name, t.numel(), self.N, self.D))

    def update(self, vec, beta):
        self._check(vec, "vec")
        s = _lib.stream_ptr(vec)
        plan = self.plan()
        if plan is not None:
            rc = self._lib.conef_cs_update_planned_f16(vec.data_ptr(), self.cs.data_ptr(), self.cs.data_ptr(),
                                                       plan.host_ptr, plan.device.data_ptr(), self.N, self.D,
                                                       self.range, float(beta), self.a, self.b, s)
            _lib.check(rc, "conef_cs_update_planned_f16")
            return
        if self._inplace:
            rc = self._lib.conef_cs_update_f16(vec.data_ptr(), self.cs.data_ptr(), self.cs.data_ptr(), self.N,
                                               self.D, self.range, float(beta), self.a, self.b, s)
            _lib.check(rc, "conef_cs_update_f16")
            return
        cells = self.cs.numel()
        wide_in = torch.empty(self.N, self.range, dtype=torch.float32, device=self.cs.device)
        wide_out = torch.empty_like(wide_in)
        _lib.check(self._lib.conef_convert_f16_to_f32(wide_in.data_ptr(), self.cs.data_ptr(), cells, s),
                   "conef_convert_f16_to_f32")
        _lib.check(self._lib.conef_cs_update_f32(vec.data_ptr(), wide_in.data_ptr(), wide_out.data_ptr(), self.N,
                                                 self.D, self.range, float(beta), self.a, self.b, s),
                   "conef_cs_update_f32")
        _lib.check(self._lib.conef_convert_f32_to_f16(self.cs.data_ptr(), wide_out.data_ptr(), cells, s),
                   "conef_convert_f32_to_f16")

    def query(self, grad_plus_error, alpha):
        self._check(grad_plus_error, "grad_plus_error")
        plan = self.plan()
        if plan is not None:
            rc = self._lib.conef_cs_query_planned_f16(grad_plus_error.data_ptr(), self.cs.data_ptr(), plan.host_ptr,
                                                      plan.device.data_ptr(), self.N, self.D, self.range, float(alpha),
                                                      self.a, self.b, _lib.stream_ptr(grad_plus_error))
            _lib.check(rc, "conef_cs_query_planned_f16")
            return
        rc = self._lib.conef_cs_query_f16(grad_plus_error.data_ptr(), self.cs.data_ptr(), self.N, self.D,
                                          self.range, float(alpha), self.a, self.b,
                                          _lib.stream_ptr(grad_plus_error))
        _lib.check(rc, "conef_cs_query_f16")

    def clean(self, alpha):
        rc = self._lib.conef_scale_f16(self.cs.data_ptr(), self.cs.numel(), float(alpha),
                                       _lib.stream_ptr(self.cs))
        _lib.check(rc, "conef_scale_f16")
