"""ctypes binding of include/gufo_hip.h.

The tests, the smoke check and the bench drive the library through this module; it
adds nothing to the C-ABI except numpy marshalling and turning status codes into
exceptions (the same mapping the C++ adapter uses).  There is no fallback: if the
built library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path
from typing import Sequence

import numpy as np

PACKAGE_DIR = Path(__file__).resolve().parent
# GUFO_HIP_LIBRARY names another build of the same library (kernel experiments).
LIBRARY_PATH = Path(os.environ.get("GUFO_HIP_LIBRARY") or PACKAGE_DIR / "lib" / "libgufo_hip.so")

OK = 0
ERR_NO_DEVICE = 1
ERR_NOT_INITIALIZED = 2
ERR_INVALID_ARGUMENT = 3
ERR_SHAPE = 4
ERR_LOGIC = 5
ERR_OUT_OF_RANGE = 6
ERR_OUT_OF_MEMORY = 7
ERR_RUNTIME = 8


class GufoHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"gufo_hip status {code}: {message}")
        self.code = code
        self.message = message


class NoDeviceError(GufoHipError):
    """std::runtime_error of the reference's stub backend (src/npu/gemv_stub.cpp:8-10)."""


class InvalidArgumentError(GufoHipError, ValueError):
    """std::invalid_argument (src/core/quant.cpp:224,233)."""


class ShapeError(GufoHipError):
    """std::runtime_error for a shape mismatch (gguf_projections.cpp:43)."""


class LogicError(GufoHipError):
    """std::logic_error (gguf_projections.cpp:214,223,235)."""


class OutOfRangeError(GufoHipError, IndexError):
    """std::out_of_range."""


_ERRORS = {
    ERR_NO_DEVICE: NoDeviceError,
    ERR_INVALID_ARGUMENT: InvalidArgumentError,
    ERR_SHAPE: ShapeError,
    ERR_LOGIC: LogicError,
    ERR_OUT_OF_RANGE: OutOfRangeError,
}

# name -> (restype, argtypes): every symbol include/gufo_hip.h declares.
_P = C.c_void_p
_SZ = C.c_size_t
SIGNATURES = {
    "gufo_hip_init": (C.c_int, [C.c_int]),
    "gufo_hip_shutdown": (C.c_int, []),
    "gufo_hip_last_error": (C.c_char_p, []),
    "gufo_hip_device_info": (C.c_int, [C.c_char_p, _SZ, C.POINTER(C.c_int)]),
    "gufo_hip_block_bytes": (_SZ, [C.c_int]),
    "gufo_hip_row_bytes": (_SZ, [C.c_int, _SZ]),
    "gufo_hip_malloc": (C.c_int, [C.POINTER(_P), _SZ]),
    "gufo_hip_free": (C.c_int, [_P]),
    "gufo_hip_memcpy_h2d": (C.c_int, [_P, _P, _SZ]),
    "gufo_hip_memcpy_d2h": (C.c_int, [_P, _P, _SZ]),
    "gufo_hip_synchronize": (C.c_int, []),
    "gufo_hip_matrix_create": (C.c_int, [C.c_int, _P, _SZ, _SZ, C.POINTER(_P)]),
    "gufo_hip_matrix_destroy": (C.c_int, [_P]),
    "gufo_hip_matrix_info": (C.c_int, [_P, C.POINTER(C.c_int), C.POINTER(_SZ),
                                       C.POINTER(_SZ), C.POINTER(_SZ)]),
    "gufo_hip_gemv": (C.c_int, [C.POINTER(_P), C.POINTER(_SZ), C.POINTER(_SZ), C.c_int,
                                _P, C.c_int, _P]),
    "gufo_hip_gemv_dev": (C.c_int, [C.POINTER(_P), C.POINTER(_SZ), C.POINTER(_SZ), C.c_int,
                                    _P, C.c_int, _P]),
    "gufo_hip_gemv_fused_dev": (C.c_int, [C.POINTER(_P), C.POINTER(_SZ), C.POINTER(_SZ),
                                          C.c_int, _P, _P, C.c_int, _P]),
    "gufo_hip_gemv_argmax_dev": (C.c_int, [C.POINTER(_P), C.POINTER(_SZ), C.POINTER(_SZ),
                                           C.c_int, _P, _P, C.c_int, _P]),
    "gufo_hip_matrix_gather_rows": (C.c_int, [_P, _P, _SZ, C.POINTER(_P)]),
    "gufo_hip_matrix_prepare_prefill": (C.c_int, [_P]),
    "gufo_hip_argmax_dev": (C.c_int, [_P, _SZ, C.POINTER(C.c_int64)]),
    "gufo_hip_route_topk": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, _P, _P]),
    "gufo_hip_route_topk_dev": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, _P, _P]),
    "gufo_hip_moe_group": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, _P, _P, _P,
                                     C.POINTER(C.c_int)]),
    "gufo_hip_moe_ffn": (C.c_int, [_P, _P, _P, C.c_int, _P, C.c_int, _P, _P, C.c_int, _P]),
    "gufo_hip_moe_ffn_dev": (C.c_int, [_P, _P, _P, C.c_int, _P, C.c_int, _P, _P, C.c_int,
                                       _P]),
    "gufo_hip_moe_layer_dev": (C.c_int, [_P, C.c_int, _P, _P, _P, C.c_int, C.c_int, _P, C.c_int,
                                         _P, _P]),
    "gufo_hip_gemm_bf16": (C.c_int, [_P, _P, _SZ, _P]),
    "gufo_hip_gemm_bf16_dev": (C.c_int, [_P, _P, _SZ, _P]),
    "gufo_hip_gemm_bf16_parts_dev": (C.c_int, [_P, C.c_int, _P, _SZ, _P]),
    "gufo_hip_gemm_q4k_bf16": (C.c_int, [_P, _P, _SZ, _P]),
    "gufo_hip_gemm_q4k_bf16_dev": (C.c_int, [_P, _P, _SZ, _P]),
    "gufo_hip_capture_begin": (C.c_int, []),
    "gufo_hip_capture_end": (C.c_int, [C.POINTER(_P)]),
    "gufo_hip_graph_launch": (C.c_int, [_P]),
    "gufo_hip_graph_destroy": (C.c_int, [_P]),
    "gufo_hip_timer_begin": (C.c_int, []),
    "gufo_hip_timer_end": (C.c_int, [C.POINTER(C.c_float)]),
    "gufo_hip_read_probe_dev": (C.c_int, [_P, _SZ, _P]),
    "gufo_hip_write_probe_dev": (C.c_int, [_P, _SZ]),
}

_lib = None


def load_library(path: os.PathLike | None = None) -> C.CDLL:
    """dlopen the built library and bind every declared symbol."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    target = Path(path) if path is not None else LIBRARY_PATH
    if not target.exists():
        raise ImportError(
            f"{target} is missing: build it first (python -c 'import __graft_entry__ as g; "
            "g.build()'); this backend has no CPU fallback")
    lib = C.CDLL(str(target))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    if path is None:
        _lib = lib
    return lib


def _check(code: int) -> None:
    if code == OK:
        return
    message = load_library().gufo_hip_last_error().decode("utf-8", "replace")
    raise _ERRORS.get(code, GufoHipError)(code, message)


def init(device: int = 0) -> None:
    _check(load_library().gufo_hip_init(device))


def shutdown() -> None:
    _check(load_library().gufo_hip_shutdown())


def synchronize() -> None:
    _check(load_library().gufo_hip_synchronize())


def device_info() -> tuple[str, int]:
    name = C.create_string_buffer(256)
    cus = C.c_int(0)
    _check(load_library().gufo_hip_device_info(name, 256, C.byref(cus)))
    return name.value.decode(), cus.value


def block_bytes(ggml_type: int) -> int:
    return load_library().gufo_hip_block_bytes(ggml_type)


def row_bytes(ggml_type: int, cols: int) -> int:
    return load_library().gufo_hip_row_bytes(ggml_type, cols)


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


class DeviceBuffer:
    """A device allocation (npu::Buffer's role, src/npu/gemv.hpp:82-131)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        handle = C.c_void_p()
        _check(load_library().gufo_hip_malloc(C.byref(handle), self.nbytes))
        self.ptr = handle.value

    @classmethod
    def from_array(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(max(a.nbytes, 16))
        buf.upload(a)
        return buf

    def upload(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        if a.nbytes > self.nbytes:
            raise ValueError("array larger than the device buffer")
        _check(load_library().gufo_hip_memcpy_h2d(C.c_void_p(self.ptr), _ptr(a), a.nbytes))

    def download(self, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        if out.nbytes > self.nbytes:
            raise ValueError("array larger than the device buffer")
        _check(load_library().gufo_hip_memcpy_d2h(_ptr(out), C.c_void_p(self.ptr), out.nbytes))
        return out

    def free(self) -> None:
        if self.ptr:
            _check(load_library().gufo_hip_free(C.c_void_p(self.ptr)))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Matrix:
    """A K-quant matrix resident in HBM (gufo_hip_matrix)."""

    def __init__(self, ggml_type: int, blocks: np.ndarray, rows: int, cols: int):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        self.type, self.rows, self.cols = int(ggml_type), int(rows), int(cols)
        handle = C.c_void_p()
        _check(load_library().gufo_hip_matrix_create(self.type, _ptr(blocks), self.rows,
                                                     self.cols, C.byref(handle)))
        self.handle = handle.value
        self.nbytes = blocks.nbytes

    def info(self) -> tuple[int, int, int, int]:
        t, r, c, b = C.c_int(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        _check(load_library().gufo_hip_matrix_info(C.c_void_p(self.handle), C.byref(t),
                                                   C.byref(r), C.byref(c), C.byref(b)))
        return t.value, r.value, c.value, b.value

    def gather_rows(self, rows) -> "Matrix":
        """A new resident matrix of the given rows of this one, in that order."""
        ids = np.ascontiguousarray(rows, dtype=np.int64)
        handle = C.c_void_p()
        _check(load_library().gufo_hip_matrix_gather_rows(C.c_void_p(self.handle), _ptr(ids),
                                                          ids.size, C.byref(handle)))
        picked = Matrix.__new__(Matrix)
        picked.type, picked.rows, picked.cols = self.type, int(ids.size), self.cols
        picked.handle = handle.value
        picked.nbytes = self.nbytes // max(self.rows, 1) * int(ids.size)
        return picked

    def prepare_prefill(self) -> None:
        """Keeps the weights in the prefill product's own form beside the packed rows."""
        _check(load_library().gufo_hip_matrix_prepare_prefill(C.c_void_p(self.handle)))

    def destroy(self) -> None:
        if self.handle:
            _check(load_library().gufo_hip_matrix_destroy(C.c_void_p(self.handle)))
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


Part = tuple  # (Matrix, first_row, n_rows)


def _parts_arrays(parts: Sequence[Part]):
    n = len(parts)
    handles = (C.c_void_p * max(n, 1))(*[p[0].handle for p in parts])
    first = (C.c_size_t * max(n, 1))(*[int(p[1]) for p in parts])
    rows = (C.c_size_t * max(n, 1))(*[int(p[2]) for p in parts])
    return handles, first, rows, n


def whole(m: Matrix) -> Part:
    return (m, 0, m.rows)


def gemv(parts: Sequence[Part], x: np.ndarray, tokens: int | None = None) -> np.ndarray:
    """Host-pointer product: y[t] = [W_0 x[t] | W_1 x[t] | ...]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if tokens is None:
        tokens = x.shape[0] if x.ndim == 2 else 1
    stride = sum(int(p[2]) for p in parts)
    y = np.empty((max(tokens, 0), stride), dtype=np.float32)
    handles, first, rows, n = _parts_arrays(parts)
    _check(load_library().gufo_hip_gemv(handles, first, rows, n, _ptr(x), tokens, _ptr(y)))
    return y


def gemv_dev(parts: Sequence[Part], x: DeviceBuffer, tokens: int, y: DeviceBuffer) -> None:
    handles, first, rows, n = _parts_arrays(parts)
    _check(load_library().gufo_hip_gemv_dev(handles, first, rows, n, C.c_void_p(x.ptr),
                                            tokens, C.c_void_p(y.ptr)))


PROLOGUE_PLAIN, PROLOGUE_SWIGLU, PROLOGUE_RESNORM = 0, 1, 2


class Prologue(C.Structure):
    """struct gufo_hip_prologue: what a product does to its activation rows first."""
    _fields_ = [("kind", C.c_int), ("delta_dev", C.c_void_p), ("norm_weight_dev", C.c_void_p),
                ("eps", C.c_float), ("residual_out_dev", C.c_void_p),
                ("normed_out_dev", C.c_void_p)]


def _dev_ptr(buf: "DeviceBuffer | None"):
    return None if buf is None else C.c_void_p(buf.ptr)


def swiglu_prologue() -> Prologue:
    return Prologue(PROLOGUE_SWIGLU, None, None, 0.0, None, None)


def resnorm_prologue(norm_weight: DeviceBuffer, eps: float, delta: DeviceBuffer | None = None,
                     residual_out: DeviceBuffer | None = None,
                     normed_out: DeviceBuffer | None = None) -> Prologue:
    return Prologue(PROLOGUE_RESNORM, _dev_ptr(delta), _dev_ptr(norm_weight), eps,
                    _dev_ptr(residual_out), _dev_ptr(normed_out))


def gemv_fused_dev(parts: Sequence[Part], prologue: Prologue | None, x: DeviceBuffer,
                   tokens: int, y: DeviceBuffer) -> None:
    """gemv_dev with the elementwise step before the product taken into its kernel."""
    handles, first, rows, n = _parts_arrays(parts)
    _check(load_library().gufo_hip_gemv_fused_dev(
        handles, first, rows, n, None if prologue is None else C.byref(prologue),
        C.c_void_p(x.ptr), tokens, C.c_void_p(y.ptr)))


def gemv_argmax_dev(parts: Sequence[Part], prologue: Prologue | None, x: DeviceBuffer,
                    tokens: int, index: DeviceBuffer) -> None:
    """The product with the greedy pick inside: index[t] (int64, device) = position of the
    first maximum of y[t]; y is not stored."""
    handles, first, rows, n = _parts_arrays(parts)
    _check(load_library().gufo_hip_gemv_argmax_dev(
        handles, first, rows, n, None if prologue is None else C.byref(prologue),
        C.c_void_p(x.ptr), tokens, C.c_void_p(index.ptr)))


def argmax_dev(logits: DeviceBuffer, n: int) -> int:
    out = C.c_int64(-1)
    _check(load_library().gufo_hip_argmax_dev(C.c_void_p(logits.ptr), n, C.byref(out)))
    return out.value


def route_topk(logits: np.ndarray, k: int) -> tuple[np.ndarray, np.ndarray]:
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tokens, experts = logits.shape
    ids = np.empty((tokens, k), dtype=np.int32)
    weights = np.empty((tokens, k), dtype=np.float32)
    _check(load_library().gufo_hip_route_topk(_ptr(logits), tokens, experts, k, _ptr(ids),
                                              _ptr(weights)))
    return ids, weights


def moe_group(ids: np.ndarray, experts: int):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    tokens, k = ids.shape
    counts = np.empty(experts, dtype=np.int32)
    offsets = np.empty(experts + 1, dtype=np.int32)
    pairs = np.empty(tokens * k, dtype=np.int32)
    distinct = C.c_int(0)
    _check(load_library().gufo_hip_moe_group(_ptr(ids), tokens, k, experts, _ptr(counts),
                                             _ptr(offsets), _ptr(pairs), C.byref(distinct)))
    return counts, offsets, pairs, distinct.value


def moe_ffn(gate: Matrix, up: Matrix, down: Matrix, experts: int, x: np.ndarray,
            ids: np.ndarray, weights: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    tokens, k = ids.shape
    y = np.empty((tokens, x.shape[1]), dtype=np.float32)
    _check(load_library().gufo_hip_moe_ffn(C.c_void_p(gate.handle), C.c_void_p(up.handle),
                                           C.c_void_p(down.handle), experts, _ptr(x), tokens,
                                           _ptr(ids), _ptr(weights), k, _ptr(y)))
    return y


def moe_ffn_dev(gate: Matrix, up: Matrix, down: Matrix, experts: int, x: DeviceBuffer,
                tokens: int, ids: DeviceBuffer, weights: DeviceBuffer, k: int,
                y: DeviceBuffer) -> None:
    _check(load_library().gufo_hip_moe_ffn_dev(
        C.c_void_p(gate.handle), C.c_void_p(up.handle), C.c_void_p(down.handle), experts,
        C.c_void_p(x.ptr), tokens, C.c_void_p(ids.ptr), C.c_void_p(weights.ptr), k,
        C.c_void_p(y.ptr)))


def moe_layer_dev(router: "Matrix | Sequence[Matrix]", gate: Matrix, up: Matrix, down: Matrix,
                  experts: int, k: int, x: DeviceBuffer, tokens: int,
                  shared: "DeviceBuffer | None", y: DeviceBuffer) -> None:
    """Router, routing, routed experts and the scaled shared expert in one call
    (gufo_hip_moe_layer_dev).  `router`: the matrix, or the matrices, of the router stage."""
    parts = [router] if isinstance(router, Matrix) else list(router)
    handles = (C.c_void_p * len(parts))(*[m.handle for m in parts])
    _check(load_library().gufo_hip_moe_layer_dev(
        handles, len(parts), C.c_void_p(gate.handle), C.c_void_p(up.handle),
        C.c_void_p(down.handle), experts, k, C.c_void_p(x.ptr), tokens, _dev_ptr(shared),
        C.c_void_p(y.ptr)))


def route_topk_dev(logits: DeviceBuffer, tokens: int, experts: int, k: int,
                   ids: DeviceBuffer, weights: DeviceBuffer) -> None:
    _check(load_library().gufo_hip_route_topk_dev(C.c_void_p(logits.ptr), tokens, experts, k,
                                                  C.c_void_p(ids.ptr), C.c_void_p(weights.ptr)))


def gemm_bf16(w: Matrix, a_bf16: np.ndarray) -> np.ndarray:
    """The prefill product for rows of any quantized type (gufo_hip_gemm_bf16)."""
    a_bf16 = np.ascontiguousarray(a_bf16, dtype=np.uint16)
    m = a_bf16.shape[0]
    c = np.empty((m, w.rows), dtype=np.float32)
    _check(load_library().gufo_hip_gemm_bf16(C.c_void_p(w.handle), _ptr(a_bf16), m, _ptr(c)))
    return c


def gemm_bf16_parts_dev(parts: Sequence[Matrix], a: DeviceBuffer, m: int,
                        c: DeviceBuffer) -> None:
    """The prefill product of a stage's matrices, outputs side by side per token
    (gufo_hip_gemm_bf16_parts_dev)."""
    handles = (C.c_void_p * len(parts))(*[p.handle for p in parts])
    _check(load_library().gufo_hip_gemm_bf16_parts_dev(handles, len(parts), C.c_void_p(a.ptr), m,
                                                       C.c_void_p(c.ptr)))


def gemm_bf16_dev(w: Matrix, a: DeviceBuffer, m: int, c: DeviceBuffer) -> None:
    _check(load_library().gufo_hip_gemm_bf16_dev(C.c_void_p(w.handle), C.c_void_p(a.ptr), m,
                                                 C.c_void_p(c.ptr)))


def gemm_q4k_bf16(w: Matrix, a_bf16: np.ndarray) -> np.ndarray:
    a_bf16 = np.ascontiguousarray(a_bf16, dtype=np.uint16)
    m = a_bf16.shape[0]
    c = np.empty((m, w.rows), dtype=np.float32)
    _check(load_library().gufo_hip_gemm_q4k_bf16(C.c_void_p(w.handle), _ptr(a_bf16), m,
                                                 _ptr(c)))
    return c


def gemm_q4k_bf16_dev(w: Matrix, a: DeviceBuffer, m: int, c: DeviceBuffer) -> None:
    _check(load_library().gufo_hip_gemm_q4k_bf16_dev(C.c_void_p(w.handle), C.c_void_p(a.ptr),
                                                     m, C.c_void_p(c.ptr)))


class Graph:
    """A recorded sequence of _dev product calls (gufo_hip_graph)."""

    def __init__(self, handle):
        self.handle = handle

    def launch(self) -> None:
        _check(load_library().gufo_hip_graph_launch(C.c_void_p(self.handle)))

    def destroy(self) -> None:
        if self.handle:
            _check(load_library().gufo_hip_graph_destroy(C.c_void_p(self.handle)))
            self.handle = None


def capture_begin() -> None:
    _check(load_library().gufo_hip_capture_begin())


def capture_end() -> Graph:
    handle = C.c_void_p()
    _check(load_library().gufo_hip_capture_end(C.byref(handle)))
    return Graph(handle.value)


def timer_begin() -> None:
    _check(load_library().gufo_hip_timer_begin())


def timer_end() -> float:
    ms = C.c_float(0.0)
    _check(load_library().gufo_hip_timer_end(C.byref(ms)))
    return ms.value


def read_probe_dev_at(src: DeviceBuffer, offset: int, nbytes: int, sink: DeviceBuffer) -> None:
    """The read probe over src[offset : offset + nbytes] (offset a multiple of 16)."""
    if offset % 16 or offset + nbytes > src.nbytes:
        raise ValueError("probe window outside the buffer")
    _check(load_library().gufo_hip_read_probe_dev(C.c_void_p(src.ptr + offset), nbytes,
                                                  C.c_void_p(sink.ptr)))


def write_probe_dev(dst: DeviceBuffer, nbytes: int) -> None:
    if nbytes > dst.nbytes:
        raise ValueError("probe window outside the buffer")
    _check(load_library().gufo_hip_write_probe_dev(C.c_void_p(dst.ptr), nbytes))


def read_probe_dev(src: DeviceBuffer, nbytes: int, sink: DeviceBuffer) -> None:
    _check(load_library().gufo_hip_read_probe_dev(C.c_void_p(src.ptr), nbytes,
                                                  C.c_void_p(sink.ptr)))
