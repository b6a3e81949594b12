"""Three-hash count sketch with median-of-three estimates
(reference: communication/compressors/CountSketchHash3.py:152-238).  Kept for comparison, as in
the reference; the hash constants and the update/query disagreement on the third sign seed are
the reference's (:40-41,:85,:137)."""
import os

import torch

from .. import _lib
from .._plan import SketchPlan


class DenseCSHash3:
    def __init__(self, N, D, sketch_size, device=None):
        self.N = int(N)
        self.D = int(D)
        self.blk_size = 512
        self.range = max(int(D * sketch_size), 1)
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.cs0, self.cs1, self.cs2 = (torch.zeros(self.N, self.range, dtype=torch.float32, device=device)
                                        for _ in range(3))
        self._spare = None
        self._plans = None
        self._value = None
        self._lib = _lib.load()

    def state_dict(self):
        d = {"N": self.N, "D": self.D, "blk_size": self.blk_size, "range": self.range}
        for k in ("cs0", "cs1", "cs2"):
            d[k] = getattr(self, k).detach().cpu().numpy()
        return d

    def load_state_dict(self, d):
        if (d["N"], d["D"], d["range"]) != (self.N, self.D, self.range):
            raise ValueError("sketch shape mismatch: have (%d,%d,%d), state holds (%d,%d,%d)" % (
                self.N, self.D, self.range, d["N"], d["D"], d["range"]))
        for k in ("cs0", "cs1", "cs2"):
            getattr(self, k).copy_(torch.from_numpy(d[k]).to(self.cs0.device))

    @classmethod
    def from_state_dict(cls, d, device=None):
        obj = cls(d["N"], d["D"], 0.0, device=device)
        obj.range = int(d["range"])
        for k in ("cs0", "cs1", "cs2"):
            setattr(obj, k, torch.from_numpy(d[k]).to(obj.cs0.device).contiguous())
        return obj

    # pickling carries the state, not the library handle (the reference class pickles too)
    __getstate__ = state_dict

    def __setstate__(self, d):
        device = torch.device("cuda", torch.cuda.current_device())
        self.N, self.D, self.blk_size, self.range = d["N"], d["D"], d["blk_size"], d["range"]
        for k in ("cs0", "cs1", "cs2"):
            setattr(self, k, torch.from_numpy(d[k]).to(device))
        self._spare = self._plans = self._value = None
        self._lib = _lib.load()

    def _check(self, t, name):
        _lib.require_device_f32(t, name)
        if t.numel() != self.N * self.D:
            raise ValueError("%s has %d elements, the sketch was built for %d x %d" % (
                name, t.numel(), self.N, self.D))

    # (a, b) of the three bucket hashes and the seeds of their sign hashes in update
    # (CountSketchHash3.py:40-41,68,77,85)
    HASHES = ((994443, 609478, 994443 + 2, 609478 + 3), (4113759, 2949676, 4113759 + 4, 2949676 + 5),
              (9171025, 2171464, 9171025 + 8, 2171464 + 4))

    def plans(self):
        """One accumulation plan per sketch (built on first use), or None when the shape has none
        or CONEF_PLAN=0: the update then accumulates with float atomics."""
        if self._plans is None:
            self._plans = False
            if os.environ.get("CONEF_PLAN", "1") != "0" and SketchPlan.applicable(self.N, self.D, self.range):
                try:
                    self._plans = [SketchPlan.shared(self.N, self.D, self.range, a, b, self.cs0.device, sign_seeds=(sa, sb))
                                   for a, b, sa, sb in self.HASHES]
                except ValueError:
                    self._plans = False
        return self._plans or None

    def update(self, vec, beta):
        self._check(vec, "vec")
        plans = self.plans()
        if plans is not None:
            # t = median of the three decays + value, then every sketch adds sign * t (an update
            # with beta = 1) along its plan: no atomics, the serial definition's order
            s = _lib.stream_ptr(vec)
            if self._value is None:
                self._value = torch.empty(self.N, self.D, dtype=torch.float32, device=self.cs0.device)
            rc = self._lib.conef_cs3_value_f32(vec.data_ptr(), self.cs0.data_ptr(), self.cs1.data_ptr(),
                                               self.cs2.data_ptr(), self._value.data_ptr(), self.N, self.D, self.range,
                                               float(beta), s)
            _lib.check(rc, "conef_cs3_value_f32")
            for cs, plan, (a, b, _, _) in zip((self.cs0, self.cs1, self.cs2), plans, self.HASHES):
                rc = self._lib.conef_cs_update_planned_f32(self._value.data_ptr(), cs.data_ptr(), cs.data_ptr(),
                                                           plan.host_ptr, plan.device.data_ptr(),
                                                           plan.workspace.data_ptr(), self.N, self.D, self.range, 1.0,
                                                           a, b, s)
                _lib.check(rc, "conef_cs_update_planned_f32")
            return
        if self._spare is None:
            self._spare = [torch.empty_like(self.cs0) for _ in range(3)]
        o = self._spare
        rc = self._lib.conef_cs3_update_f32(vec.data_ptr(), self.cs0.data_ptr(), self.cs1.data_ptr(),
                                            self.cs2.data_ptr(), o[0].data_ptr(), o[1].data_ptr(), o[2].data_ptr(),
                                            self.N, self.D, self.range, float(beta), _lib.stream_ptr(vec))
        _lib.check(rc, "conef_cs3_update_f32")
        self._spare = [self.cs0, self.cs1, self.cs2]
        self.cs0, self.cs1, self.cs2 = o

    def query(self, grad_plus_error, alpha):
        self._check(grad_plus_error, "grad_plus_error")
        rc = self._lib.conef_cs3_query_f32(grad_plus_error.data_ptr(), self.cs0.data_ptr(), self.cs1.data_ptr(),
                                           self.cs2.data_ptr(), self.N, self.D, self.range, float(alpha),
                                           _lib.stream_ptr(grad_plus_error))
        _lib.check(rc, "conef_cs3_query_f32")

    def clean(self, alpha):
        for c in (self.cs0, self.cs1, self.cs2):
            _lib.check(self._lib.conef_scale_f32(c.data_ptr(), c.numel(), float(alpha), _lib.stream_ptr(c)),
                       "conef_scale_f32")
