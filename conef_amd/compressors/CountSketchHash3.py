"""Three-hash count sketch with median-of-three estimates
(reference: communication/compressors/CountSketchHash3.py:152-238).  Kept for comparison, as in
the reference; the hash constants and the update/query disagreement on the third sign seed are
the reference's (:40-41,:85,:137)."""
import torch

from .. import _lib


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
        self._lib = _lib.load()

    def state_dict(self):
        d = {"N": self.N, "D": self.D, "blk_size": self.blk_size, "range": self.range}
        for k in ("cs0", "cs1", "cs2"):
            d[k] = getattr(self, k).detach().cpu().numpy()
        return d

    def load_state_dict(self, d):
        if (d["N"], d["D"], d["range"]) != (self.N, self.D, self.range):
            raise ValueError("sketch shape mismatch")
        for k in ("cs0", "cs1", "cs2"):
            getattr(self, k).copy_(torch.from_numpy(d[k]).to(self.cs0.device))

    def _check(self, t, name):
        _lib.require_device_f32(t, name)
        if t.numel() != self.N * self.D:
            raise ValueError("%s has %d elements, the sketch was built for %d x %d" % (
                name, t.numel(), self.N, self.D))

    def update(self, vec, beta):
        self._check(vec, "vec")
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
