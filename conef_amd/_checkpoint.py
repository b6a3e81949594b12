"""Saving and restoring the cross-iteration state of the hooks.

The reference never checkpoints its compressor state (its DenseCS.__setstate__ drops the hash seeds,
communication/compressors/CountSketch.py:124-137, and the hook states have no serialisation at all),
so a resumed run starts with empty error memory.  Here every state class has ``state_dict()`` /
``load_state_dict()``: the iteration counter, the generators that pick block offsets and Q seeds,
the error memory (dense tensors or sketches), the warm-start P / Q arenas and the compression
statistics.  Hyper-parameters are not part of it: they are constructor arguments.

The packed form holds only Python scalars, lists, dicts and numpy arrays, so it can be written
with torch.save or numpy.savez as it is.
"""
import numpy as np
import torch

from .compressors import CountSketch, CountSketchHash3, halfCountSketch

SKETCH_CLASSES = {"DenseCS": CountSketch.DenseCS, "HalfDenseCS": halfCountSketch.DenseCS,
                  "DenseCSHash3": CountSketchHash3.DenseCSHash3}


def pack(obj):
    if isinstance(obj, torch.Tensor):
        return {"__kind__": "tensor", "value": obj.detach().cpu().numpy()}
    if isinstance(obj, np.random.RandomState):
        return {"__kind__": "rng", "value": obj.get_state()}
    for name, cls in SKETCH_CLASSES.items():
        if type(obj) is cls:
            return {"__kind__": "sketch", "class": name, "value": obj.state_dict()}
    if isinstance(obj, dict):
        return {"__kind__": "dict", "items": [(k, pack(v)) for k, v in obj.items()]}
    if isinstance(obj, (list, tuple)):
        return {"__kind__": "list", "items": [pack(v) for v in obj]}
    if obj is None or isinstance(obj, (bool, int, float, str)):
        return obj
    raise TypeError("cannot checkpoint a %s" % type(obj).__name__)


def unpack(obj, device):
    if not isinstance(obj, dict):
        return obj
    kind = obj["__kind__"]
    if kind == "tensor":
        return torch.from_numpy(np.ascontiguousarray(obj["value"])).to(device)
    if kind == "rng":
        rng = np.random.RandomState()
        rng.set_state(obj["value"])
        return rng
    if kind == "sketch":
        return SKETCH_CLASSES[obj["class"]].from_state_dict(obj["value"], device=device)
    if kind == "dict":
        return {k: unpack(v, device) for k, v in obj["items"]}
    if kind == "list":
        return [unpack(v, device) for v in obj["items"]]
    raise ValueError("unknown checkpoint entry %r" % kind)


class Checkpointable:
    """Mixin of the hook state classes.  ``CHECKPOINT_FIELDS`` names the slots that change from
    iteration to iteration."""
    __slots__ = ()
    CHECKPOINT_FIELDS = ()

    def settle(self):
        """Work the hooks left on a side stream that touches this state's tensors is ordered before
        the current stream's next operation (a no-op for the states that leave none)."""
        if hasattr(self, "round_cache"):
            from ._psgd_engine import settle
            settle(self)

    def state_dict(self):
        self.settle()
        return {"class": type(self).__name__, "fields": {f: pack(getattr(self, f)) for f in self.CHECKPOINT_FIELDS}}

    def load_state_dict(self, state, device=None):
        if state.get("class") != type(self).__name__:
            raise ValueError("checkpoint of a %s cannot be loaded into a %s" % (state.get("class"), type(self).__name__))
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        missing = [f for f in self.CHECKPOINT_FIELDS if f not in state["fields"]]
        if missing:
            raise ValueError("checkpoint lacks %s" % ", ".join(missing))
        for f in self.CHECKPOINT_FIELDS:
            setattr(self, f, unpack(state["fields"][f], device))
        if hasattr(self, "round_cache"):
            self.round_cache = {}        # launch tables hold pointers into the state just replaced
