"""ctypes binding of include/gufo_hip_model.h: a GGUF model file opened on the MI355X and
the reference's Projections calls on it.  Thin by design: it is the binding the tests and
the bench use, the product is the library."""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

import numpy as np

from . import capi

MODEL_LIBRARY_PATH = Path(__file__).resolve().parent / "lib" / "libgufo_hip_model.so"

(LINEAR_IN, ATTENTION_IN, MIXER_OUT, FFN_IN, FFN_DOWN, LM_HEAD, ROUTER, EXPERT_IN, EXPERT_DOWN,
 MTP_IN) = range(10)
STAGE_NAMES = ("linear_in", "attention_in", "mixer_out", "ffn_in", "ffn_down", "lm_head",
               "router", "expert_in", "expert_down", "mtp_in")


class Shape(C.Structure):
    """struct gufo_model_shape."""
    _fields_ = [("is_moe", C.c_int), ("layers", C.c_int), ("mtp_layers", C.c_int),
                ("hidden", C.c_int), ("ffn", C.c_int), ("vocab", C.c_int),
                ("rms_eps", C.c_float), ("full_attention_interval", C.c_int),
                ("heads", C.c_int), ("kv_heads", C.c_int), ("head_dim", C.c_int),
                ("rope_dim", C.c_int), ("rope_theta", C.c_float), ("conv_kernel", C.c_int),
                ("linear_key_heads", C.c_int), ("linear_value_heads", C.c_int),
                ("linear_head_dim", C.c_int), ("experts", C.c_int), ("experts_used", C.c_int),
                ("expert_ffn", C.c_int), ("shared_expert_ffn", C.c_int),
                ("tied_embeddings", C.c_int), ("has_mtp_layer", C.c_int), ("tensors", C.c_int)]

    def as_dict(self) -> dict:
        return {name: getattr(self, name) for name, _ in self._fields_}


class BorrowedMatrix(capi.Matrix):
    """A resident matrix that belongs to an open model: usable wherever a capi.Matrix is,
    never destroyed from here."""

    def __init__(self, handle):
        self.handle = handle
        self.type, self.rows, self.cols, self.nbytes = self.info()

    def destroy(self) -> None:
        self.handle = None

    def __del__(self):
        pass


_P = C.c_void_p
# name -> (restype, argtypes): every symbol include/gufo_hip_model.h declares.
SIGNATURES = {
    "gufo_model_last_error": (C.c_char_p, []),
    "gufo_model_inspect": (C.c_int, [C.c_char_p, C.POINTER(Shape)]),
    "gufo_model_open": (C.c_int, [C.c_char_p, C.c_int, C.POINTER(_P)]),
    "gufo_model_close": (C.c_int, [_P]),
    "gufo_model_get_shape": (C.c_int, [_P, C.POINTER(Shape)]),
    "gufo_model_weight_bytes": (C.c_uint64, [_P]),
    "gufo_model_stage_inputs": (C.c_size_t, [_P, C.c_int, C.c_int]),
    "gufo_model_stage_outputs": (C.c_size_t, [_P, C.c_int, C.c_int]),
    "gufo_model_stage_matrices": (C.c_int, [_P, C.c_int, C.c_int, _P, C.c_int,
                                            C.POINTER(C.c_int)]),
    "gufo_model_expert_matrices": (C.c_int, [_P, C.c_int, C.POINTER(_P), C.POINTER(_P),
                                             C.POINTER(_P)]),
    "gufo_model_apply": (C.c_int, [_P, C.c_int, C.c_int, _P, C.c_int, _P]),
    "gufo_model_apply_expert": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, _P, C.c_int, _P]),
    "gufo_model_norm_weight": (C.c_int, [_P, C.c_int, C.c_int, _P]),
}

_lib = None


def load_library(path: os.PathLike | None = None) -> C.CDLL:
    global _lib
    if _lib is not None and path is None:
        return _lib
    target = Path(path) if path is not None else MODEL_LIBRARY_PATH
    if not target.exists():
        raise ImportError(f"{target} is missing: build it first (python -c 'import "
                          "__graft_entry__ as g; g.build()')")
    lib = C.CDLL(str(target))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if path is None:
        _lib = lib
    return lib


def _check(code: int) -> None:
    if code == capi.OK:
        return
    message = load_library().gufo_model_last_error().decode("utf-8", "replace")
    raise capi._ERRORS.get(code, capi.GufoHipError)(code, message)


def inspect(path) -> dict:
    """Shape of the model in `path` after every check the loader makes; no device needed."""
    shape = Shape()
    _check(load_library().gufo_model_inspect(str(path).encode(), C.byref(shape)))
    return shape.as_dict()


class Model:
    """A model file with its projection weights in HBM."""

    def __init__(self, path, device: int = 0):
        self.handle = _P()
        _check(load_library().gufo_model_open(str(path).encode(), device, C.byref(self.handle)))
        shape = Shape()
        _check(load_library().gufo_model_get_shape(self.handle, C.byref(shape)))
        self.shape = shape.as_dict()

    @property
    def weight_bytes(self) -> int:
        return int(load_library().gufo_model_weight_bytes(self.handle))

    def stage_inputs(self, stage: int, layer: int) -> int:
        return int(load_library().gufo_model_stage_inputs(self.handle, stage, layer))

    def stage_outputs(self, stage: int, layer: int) -> int:
        return int(load_library().gufo_model_stage_outputs(self.handle, stage, layer))

    @staticmethod
    def _borrowed(handle) -> "BorrowedMatrix | None":
        return BorrowedMatrix(handle) if handle else None

    def stage_matrices(self, stage: int, layer: int) -> list:
        """The resident matrices of a stage (gufo_model_stage_matrices), usable with
        capi's device entry points for as long as the model is open."""
        count = C.c_int()
        _check(load_library().gufo_model_stage_matrices(self.handle, stage, layer, None, 0,
                                                        C.byref(count)))
        handles = (_P * max(count.value, 1))()
        _check(load_library().gufo_model_stage_matrices(self.handle, stage, layer, handles,
                                                        count.value, C.byref(count)))
        return [self._borrowed(handles[i]) for i in range(count.value)]

    def expert_matrices(self, layer: int):
        """gate, up, down expert tensors of a mixture layer (None each for a dense one)."""
        gate, up, down = _P(), _P(), _P()
        _check(load_library().gufo_model_expert_matrices(self.handle, layer, C.byref(gate),
                                                         C.byref(up), C.byref(down)))
        return tuple(self._borrowed(h.value) for h in (gate, up, down))

    def apply(self, stage: int, layer: int, x: np.ndarray, expert: int = -1) -> np.ndarray:
        """Projections::Apply (ApplyExpert with expert >= 0) on tokens x inputs rows."""
        x = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
        outputs = self.stage_outputs(stage, layer)
        y = np.empty((x.shape[0], outputs), dtype=np.float32)
        xp, yp = x.ctypes.data_as(_P), y.ctypes.data_as(_P)
        if expert < 0:
            _check(load_library().gufo_model_apply(self.handle, stage, layer, xp, x.shape[0], yp))
        else:
            _check(load_library().gufo_model_apply_expert(self.handle, stage, layer, expert, xp,
                                                          x.shape[0], yp))
        return y

    def norm_weight(self, which: int, layer: int = 0) -> np.ndarray:
        out = np.empty(self.shape["hidden"], dtype=np.float32)
        _check(load_library().gufo_model_norm_weight(self.handle, which, layer,
                                                     out.ctypes.data_as(_P)))
        return out

    def close(self) -> None:
        if self.handle:
            _check(load_library().gufo_model_close(self.handle))
            self.handle = _P()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
