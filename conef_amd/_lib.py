"""ctypes binding of libconef_hip.so - the one native boundary of the package.

This replaces what communication/compressors/cupy_kernel.py:10-45 does in the reference
(NVRTC-compile a CUDA string and launch it with raw pointers on torch's current stream): here the
kernels are precompiled for gfx950 and every entry point takes raw device pointers, sizes,
scalars by value and the stream.  There is no CPU implementation behind these calls: if the
library is missing the import of any op fails loudly.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBPATH = os.path.join(_HERE, "lib", "libconef_hip.so")

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_I32 = ctypes.c_int32
_F32 = ctypes.c_float

# name -> argtypes; every function returns int (0 = ok, >0 hipError_t, -1 invalid argument, -2 too large),
# except the *_bytes functions, which return a byte count as int64
SIGNATURES = {
    "conef_version": [],
    "conef_hash_table_i32": [_P, _P, _I64, _I32, _I32, _I32, _I32, _I32, _P],
    "conef_hash_table_host_i32": [_P, _P, _I64, _I32, _I32, _I32, _I32, _I32],
    "conef_cs_query_f32": [_P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_query_f16": [_P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_query_planned_f32": [_P, _P, _P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_query_planned_f16": [_P, _P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_update_inplace_ok": [_I64, _I64, _I32],
    "conef_cs_update_f32": [_P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_update_f16": [_P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs3_query_f32": [_P, _P, _P, _P, _I64, _I64, _I32, _F32, _P],
    "conef_cs3_update_f32": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I32, _F32, _P],
    "conef_scale_f32": [_P, _I64, _F32, _P],
    "conef_scale_f16": [_P, _I64, _F32, _P],
    "conef_convert_f16_to_f32": [_P, _P, _I64, _P],
    "conef_convert_f32_to_f16": [_P, _P, _I64, _P],
    "conef_randblock_conef_step_f32": [_P, _P, _P, _P, _I64, _I64, _I32, _I64, _I64, _F32, _F32, _I32, _I32, _P],
    "conef_randblock_ef_step_f32": [_P, _P, _P, _I64, _I64, _I64, _P],
    "conef_randblock_unbiased_step_f32": [_P, _P, _I64, _I64, _I64, _F32, _P],
    "conef_randblock_gather_f32": [_P, _P, _I64, _I64, _I64, _F32, _P],
    "conef_randblock_scatter_f32": [_P, _P, _I64, _I64, _I64, _P],
    "conef_psgd_mq_f32": [_P, _P, _P, _I64, _I64, _I32, _P, _I64, _P],
    "conef_psgd_mq_ef_f32": [_P, _P, _P, _P, _I64, _I64, _I32, _P, _I64, _P],
    "conef_psgd_mq_conef_f32": [_P, _P, _P, _P, _I64, _I64, _I32, _I32, _F32, _I32, _I32, _P, _I64, _P],
    "conef_psgd_mq_conef_planned_f32": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _F32, _I32, _I32, _P, _I64,
                                        _P],
    "conef_psgd_workspace_bytes": [_I64, _I64, _I32],
    "conef_psgd_batch_workspace_bytes": [_P, _I32],
    "conef_psgd_mq_batch_f32": [_P, _I32, _I32, _F32, _I32, _I32, _P, _I64, _P],
    "conef_psgd_products_f32": [_P, _P, _I32, _I32, _F32, _F32, _I32, _I32, _P, _I64, _P],
    "conef_psgd_mtp_batch_f32": [_P, _I32, _P, _I64, _P],
    "conef_psgd_pqt_batch_f32": [_P, _I32, _I32, _F32, _I32, _I32, _P],
    "conef_psgd_sketch_update_batch_f32": [_P, _I32, _F32, _I32, _I32, _P],
    "conef_psgd_round_f32": [_P, _I32, _I32, _I32, _F32, _F32, _F32, _I32, _I32, _P, _I64, _P],
    "conef_psgd_round_small_fits": [_P, _I32, _I32, _I32, _I32, _I32],
    "conef_psgd_round_small_workspace_bytes": [_P, _I32],
    "conef_psgd_round_small_f32": [_P, _I32, _I32, _I32, _F32, _F32, _F32, _I32, _I32, _P, _I64, _P],
    "conef_psgd_round_ahead_f32": [_P, _I32, _I32, _I32, _F32, _F32, _F32, _I32, _I32, _P, _I32, _P, _P, _I64, _P],
    "conef_psgd_mtp_f32": [_P, _P, _P, _I64, _I64, _I32, _P, _I64, _P],
    "conef_psgd_pqt_f32": [_P, _P, _P, _I64, _I64, _I32, _P],
    "conef_psgd_pqt_ef_f32": [_P, _P, _P, _P, _I64, _I64, _I32, _P],
    "conef_psgd_pqt_conef_f32": [_P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _F32, _I32, _I32, _P],
    "conef_psgd_pqt_conef_planned_f32": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _F32, _I32, _I32, _P],
    "conef_gram_schmidt_f32": [_P, _I64, _I32, _F32, _P, _I64, _P],
    "conef_gram_schmidt_batch_f32": [_P, _P, _P, _I32, _F32, _P, _I64, _P],
    "conef_gram_schmidt_give_ups": [_P],
    "conef_ef_passthrough_f32": [_P, _P, _I64, _P],
    "conef_plan_bytes": [_I64, _I64, _I32, _I32, _I32],
    "conef_plan_build_host": [_P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32],
    "conef_plan_build_host_seeded": [_P, _I64, _I64, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _I32],
    "conef_cs3_value_f32": [_P, _P, _P, _P, _P, _I64, _I64, _I32, _F32, _P],
    "conef_plan_workspace_bytes": [_P],
    "conef_plan_kind": [_P],
    "conef_cs_update_planned_f16": [_P, _P, _P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_cs_update_planned_f32": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I32, _F32, _I32, _I32, _P],
    "conef_randblock_conef_step_planned_f32": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I32, _I64, _I64, _F32, _F32,
                                               _I32, _I32, _P],
    "conef_topk_workspace_bytes": [_I64],
    "conef_topk_sparsify_f32": [_P, _I64, _I64, _P, _I64, _P],
    "conef_topk_batch_workspace_bytes": [_P, _I32],
    "conef_topk_sparsify_batch_f32": [_P, _P, _P, _I32, _P, _I64, _P],
    "conef_topk_sparsify_batch_kept_f32": [_P, _P, _P, _I32, _P, _I64, _P],
    "conef_topk_sparsify_noalloc_f32": [_P, _I64, _I64, _P],
    "conef_randblock_step_batch_f32": [_P, _I32, _I32, _F32, _F32, _I32, _I32, _P],
}

class PsgdItem(ctypes.Structure):
    """ConefPsgdItem of include/conef_hip.h: one matrix of a bucket for the batch entry points."""
    _fields_ = [("x", _P), ("err", _P), ("cs", _P), ("plan_host", _P), ("plan_dev", _P), ("p", _P), ("q", _P),
                ("n", _I64), ("m", _I64), ("r", _I32), ("w", _I32)]


class RandBlockItem(ctypes.Structure):
    """ConefRandBlockItem of include/conef_hip.h: one tensor of a bucket for conef_randblock_step_batch_f32."""
    _fields_ = [("x", _P), ("err", _P), ("cs_in", _P), ("cs_out", _P), ("payload", _P), ("plan_host", _P),
                ("plan_dev", _P), ("staging", _P), ("n", _I64), ("m", _I64), ("start", _I64), ("block", _I64),
                ("w", _I32), ("reserved", _I32)]


_RETURNS_I64 = ("conef_topk_workspace_bytes", "conef_topk_batch_workspace_bytes", "conef_plan_bytes",
                "conef_plan_workspace_bytes", "conef_psgd_workspace_bytes", "conef_psgd_batch_workspace_bytes",
                "conef_psgd_round_small_workspace_bytes")

_handle = None


class ConefLibraryError(RuntimeError):
    pass


def load():
    """Loads the shared library (once) and types every entry point.  Raises if it is not built."""
    global _handle
    if _handle is not None:
        return _handle
    if not os.path.exists(LIBPATH):
        raise ConefLibraryError(
            "libconef_hip.so is not built (expected at %s); run `python -m conef_amd.build`. "
            "There is no CPU fallback for the ConEF kernels." % LIBPATH)
    lib = ctypes.CDLL(LIBPATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError here means header and library disagree
        fn.argtypes = argtypes
        fn.restype = _I64 if name in _RETURNS_I64 else ctypes.c_int
    _handle = lib
    return lib


def check(code, what):
    if code != 0:
        if code == -1:
            raise ValueError("%s: invalid argument" % what)
        if code == -2:
            raise ValueError("%s: input larger than the entry point's stated maximum" % what)
        raise ConefLibraryError("%s: HIP error %d" % (what, code))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(tensor):
    """hipStream_t of torch's current stream on the tensor's device, as an integer."""
    if _raw_stream is not None:       # the handle without building a Stream object: a hook calls this per bucket
        return _raw_stream(tensor.get_device())
    return torch.cuda.current_stream(tensor.device).cuda_stream


_current_stream_ids = getattr(torch._C, "_cuda_getCurrentStream", None)
_set_stream_ids = getattr(torch._C, "_cuda_setStream", None)


def current_stream(device):
    """torch's current stream on ``device`` as a Stream object, without the device-index lookups of
    ``torch.cuda.current_stream`` (5 us a call: a hook that orders two streams makes several)."""
    if _current_stream_ids is not None:
        sid, idx, kind = _current_stream_ids(device.index if device.index is not None else torch.cuda.current_device())
        return torch.cuda.Stream(stream_id=sid, device_index=idx, device_type=kind)
    return torch.cuda.current_stream(device)


class on_stream:
    """``with torch.cuda.stream(s)`` for a stream of the current device, without the lookups."""
    __slots__ = ("stream", "back", "ctx")

    def __init__(self, stream):
        self.stream = stream

    def __enter__(self):
        if _current_stream_ids is None or _set_stream_ids is None:
            self.ctx = torch.cuda.stream(self.stream)
            return self.ctx.__enter__()
        self.ctx = None
        self.back = _current_stream_ids(self.stream.device_index)
        _set_stream_ids(stream_id=self.stream.stream_id, device_index=self.stream.device_index,
                        device_type=self.stream.device_type)

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        _set_stream_ids(stream_id=self.back[0], device_index=self.back[1], device_type=self.back[2])
        return False


def require_device_f32(t, name, dtype=torch.float32):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a tensor on the GPU; the ConEF kernels have no CPU path" % name)
    if t.dtype != dtype:
        raise ValueError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t
