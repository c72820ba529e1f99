"""ctypes access to the CPU checker: the C restatement (libkquant_oracle.so) and,
where it was built, the compiled reference (_ref/libgufo_ref.so).

TEST INFRASTRUCTURE.  Only tests, the smoke check and the bench's cpu_baseline leg
import this module; the shipped library and its Python binding never do.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
ORACLE_LIB = ORACLE_DIR / "libkquant_oracle.so"
REF_LIB = ORACLE_DIR / "_ref" / "libgufo_ref.so"

F32, Q8_0, Q4_K, Q5_K, Q6_K = 0, 8, 12, 13, 14
_SZ = C.c_size_t
_P = C.c_void_p


def build(ref: bool = True) -> None:
    """make the checker libraries (the reference build is skipped where its sources
    are absent)."""
    targets = ["all"] + (["ref"] if ref else [])
    subprocess.run(["make", "-s", "-C", str(ORACLE_DIR), *targets], check=True)


_oracle = None
_ref = None


def lib() -> C.CDLL:
    global _oracle
    if _oracle is None:
        if not ORACLE_LIB.exists():
            build(ref=False)
        o = C.CDLL(str(ORACLE_LIB))
        o.gufo_oracle_half_to_float.restype = C.c_float
        o.gufo_oracle_half_to_float.argtypes = [C.c_uint16]
        o.gufo_oracle_block_bytes.restype = _SZ
        o.gufo_oracle_block_bytes.argtypes = [C.c_int]
        o.gufo_oracle_row_bytes.restype = _SZ
        o.gufo_oracle_row_bytes.argtypes = [C.c_int, _SZ]
        o.gufo_oracle_scale_min_k4.restype = None
        o.gufo_oracle_scale_min_k4.argtypes = [_SZ, _P, _P, _P]
        o.gufo_oracle_dequantize.restype = C.c_int
        o.gufo_oracle_dequantize.argtypes = [C.c_int, _P, _P, _SZ]
        for name in ("q4_k", "q5_k", "q6_k", "q8_0", "f32"):
            fn = getattr(o, f"gufo_oracle_dot_{name}")
            fn.restype = C.c_float
            fn.argtypes = [_P, _P, _SZ]
        o.gufo_oracle_dot_double.restype = C.c_double
        o.gufo_oracle_dot_double.argtypes = [C.c_int, _P, _P, _SZ]
        o.gufo_oracle_matmul.restype = C.c_int
        o.gufo_oracle_matmul.argtypes = [C.c_int, _P, _P, _P, _P, _SZ, _P, C.c_int, _P,
                                         C.c_int, C.c_int]
        o.gufo_oracle_route.restype = None
        o.gufo_oracle_route.argtypes = [_P, C.c_int, C.c_int, _P, _P]
        o.gufo_oracle_argmax.restype = C.c_int64
        o.gufo_oracle_argmax.argtypes = [_P, _SZ]
        o.gufo_oracle_moe_group.restype = C.c_int
        o.gufo_oracle_moe_group.argtypes = [_P, C.c_int, C.c_int, C.c_int, _P, _P, _P]
        o.gufo_oracle_moe_ffn.restype = C.c_int
        o.gufo_oracle_moe_ffn.argtypes = [_P, C.c_int, _P, C.c_int, _P, C.c_int, C.c_int,
                                          C.c_int, C.c_int, _P, _P, C.c_int, C.c_int, _P, _P,
                                          _P, C.c_int, C.c_int]
        o.gufo_oracle_silu.restype = C.c_float
        o.gufo_oracle_silu.argtypes = [C.c_float]
        o.gufo_oracle_rms_norm.restype = None
        o.gufo_oracle_rms_norm.argtypes = [_P, _P, _SZ, C.c_float, _P]
        o.gufo_oracle_res_norm.restype = None
        o.gufo_oracle_res_norm.argtypes = [_P, _P, _P, _SZ, C.c_float, _P, _P]
        o.gufo_oracle_swiglu.restype = None
        o.gufo_oracle_swiglu.argtypes = [_P, _SZ, _P]
        _oracle = o
    return _oracle


def ref_available() -> bool:
    return REF_LIB.exists()


def ref() -> C.CDLL:
    """The compiled reference; raises FileNotFoundError where it was not built."""
    global _ref
    if _ref is None:
        if not REF_LIB.exists():
            raise FileNotFoundError(f"{REF_LIB} was not built (reference sources absent)")
        r = C.CDLL(str(REF_LIB))
        r.ref_half_to_float.restype = C.c_float
        r.ref_half_to_float.argtypes = [C.c_uint16]
        r.ref_dequantize.restype = C.c_int
        r.ref_dequantize.argtypes = [C.c_int, _P, _P, _SZ]
        r.ref_dot.restype = C.c_float
        r.ref_dot.argtypes = [C.c_int, _P, _P, _SZ]
        r.ref_route.restype = None
        r.ref_route.argtypes = [_P, C.c_int, C.c_int, _P, _P]
        r.ref_silu.restype = C.c_float
        r.ref_silu.argtypes = [C.c_float]
        r.ref_last_error.restype = C.c_char_p
        r.ref_gguf_open.restype = _P
        r.ref_gguf_open.argtypes = [C.c_char_p]
        r.ref_gguf_close.restype = None
        r.ref_gguf_close.argtypes = [_P]
        r.ref_gguf_config.restype = None
        r.ref_gguf_config.argtypes = [_P, _P, _P]
        r.ref_gguf_apply.restype = C.c_int
        r.ref_gguf_apply.argtypes = [_P, C.c_int, C.c_int, C.c_int, _P, C.c_int, _P, C.c_int]
        r.ref_decoder_open.restype = _P
        r.ref_decoder_open.argtypes = [_P, C.c_int, _P, _P, _P]
        r.ref_decoder_close.restype = None
        r.ref_decoder_close.argtypes = [_P]
        r.ref_decoder_step.restype = C.c_int
        r.ref_decoder_step.argtypes = [_P, C.c_int, _P]
        r.ref_decoder_reset.restype = None
        r.ref_decoder_reset.argtypes = [_P]
        r.ref_decoder_foreign_calls.restype = C.c_long
        r.ref_decoder_foreign_calls.argtypes = [_P]
        r.ref_rms_norm.restype = None
        r.ref_rms_norm.argtypes = [_P, _P, C.c_int, C.c_float, _P]
        r.ref_shared_expert_scale.restype = C.c_float
        r.ref_shared_expert_scale.argtypes = [C.c_float]
        r.ref_default_threads.restype = C.c_int
        r.ref_usable_cpus.restype = C.c_int
        r.ref_matmul.restype = C.c_int
        r.ref_matmul.argtypes = [C.c_int, _P, _P, _P, _P, _SZ, _P, C.c_int, _P, C.c_int]
        _ref = r
    return _ref


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def half_to_float(bits: int) -> float:
    return lib().gufo_oracle_half_to_float(bits)


def scale_min_k4(j: int, packed: np.ndarray) -> tuple[int, int]:
    packed = _u8(packed)
    sc = np.zeros(1, np.uint8)
    m = np.zeros(1, np.uint8)
    lib().gufo_oracle_scale_min_k4(j, _p(packed), _p(sc), _p(m))
    return int(sc[0]), int(m[0])


def dequantize(ggml_type: int, blocks: np.ndarray, n: int, use_ref: bool = False) -> np.ndarray:
    blocks = _u8(blocks)
    out = np.empty(n, dtype=np.float32)
    fn = ref().ref_dequantize if use_ref else lib().gufo_oracle_dequantize
    if fn(ggml_type, _p(blocks), _p(out), n) != 0:
        raise ValueError("dequantize: unknown type or partial block")
    return out


def dot(ggml_type: int, row: np.ndarray, x: np.ndarray, use_ref: bool = False) -> float:
    row, x = _u8(row), _f32(x)
    if use_ref:
        return ref().ref_dot(ggml_type, _p(row), _p(x), x.size)
    name = {Q4_K: "q4_k", Q5_K: "q5_k", Q6_K: "q6_k", Q8_0: "q8_0", F32: "f32"}[ggml_type]
    return getattr(lib(), f"gufo_oracle_dot_{name}")(_p(row), _p(x), x.size)


def dot_double(ggml_type: int, row: np.ndarray, x: np.ndarray) -> float:
    row, x = _u8(row), _f32(x)
    return lib().gufo_oracle_dot_double(ggml_type, _p(row), _p(x), x.size)


def matmul(parts, x: np.ndarray, precision: str = "float", threads: int = 1,
           use_ref: bool = False) -> np.ndarray:
    """parts: sequence of (ggml_type, blocks[rows_total, row_bytes], first_row, n_rows).
    Returns y[tokens, sum(n_rows)].  precision "float" = fused fp32 dots, "double" =
    dequantize + double sum."""
    x = _f32(x)
    tokens, cols = x.shape
    n = len(parts)
    keep = [_u8(p[1]) for p in parts]
    data = (C.c_void_p * n)(*[k.ctypes.data for k in keep])
    types = (C.c_int * n)(*[int(p[0]) for p in parts])
    first = (C.c_size_t * n)(*[int(p[2]) for p in parts])
    rows = (C.c_size_t * n)(*[int(p[3]) for p in parts])
    y = np.empty((tokens, sum(int(p[3]) for p in parts)), dtype=np.float32)
    if use_ref:
        if precision != "float":
            raise ValueError("the reference driver runs the fused fp32 dots only")
        status = ref().ref_matmul(n, data, types, first, rows, cols, _p(x), tokens, _p(y),
                                  threads)
    else:
        status = lib().gufo_oracle_matmul(n, data, types, first, rows, cols, _p(x), tokens,
                                          _p(y), 1 if precision == "double" else 0, threads)
    if status != 0:
        raise ValueError("matmul: bad argument")
    return y


def route(logits: np.ndarray, k: int, use_ref: bool = False):
    logits = _f32(logits)
    tokens, experts = logits.shape
    ids = np.empty((tokens, k), dtype=np.int32)
    weights = np.empty((tokens, k), dtype=np.float32)
    fn = ref().ref_route if use_ref else lib().gufo_oracle_route
    for t in range(tokens):
        fn(_p(logits[t]), experts, k, _p(ids[t]), _p(weights[t]))
    return ids, weights


def argmax(v: np.ndarray) -> int:
    v = _f32(v)
    return lib().gufo_oracle_argmax(_p(v), v.size)


def moe_group(ids: np.ndarray, experts: int):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    tokens, k = ids.shape
    counts = np.empty(experts, np.int32)
    offsets = np.empty(experts + 1, np.int32)
    pairs = np.empty(tokens * k, np.int32)
    distinct = lib().gufo_oracle_moe_group(_p(ids), tokens, k, experts, _p(counts),
                                           _p(offsets), _p(pairs))
    return counts, offsets, pairs, distinct


def moe_ffn(gate, gate_type, up, up_type, down, down_type, experts, hidden, ffn, logits, x,
            k, precision: str = "float", threads: int = 1):
    gate, up, down = _u8(gate), _u8(up), _u8(down)
    logits, x = _f32(logits), _f32(x)
    tokens = x.shape[0]
    ids = np.empty((tokens, k), np.int32)
    weights = np.empty((tokens, k), np.float32)
    y = np.empty((tokens, hidden), np.float32)
    status = lib().gufo_oracle_moe_ffn(_p(gate), gate_type, _p(up), up_type, _p(down),
                                       down_type, experts, hidden, ffn, _p(logits), _p(x),
                                       tokens, k, _p(ids), _p(weights), _p(y),
                                       1 if precision == "double" else 0, threads)
    if status != 0:
        raise ValueError("moe_ffn: bad argument")
    return ids, weights, y


def silu(x: float) -> float:
    return lib().gufo_oracle_silu(x)


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float, use_ref: bool = False) -> np.ndarray:
    """RmsNorm of one row (core/vec.hpp:56-63)."""
    x = _f32(x)
    w = _f32(w)
    out = np.empty_like(x)
    if use_ref:
        ref().ref_rms_norm(_p(x), _p(w), x.size, eps, _p(out))
    else:
        lib().gufo_oracle_rms_norm(_p(x), _p(w), x.size, eps, _p(out))
    return out


def res_norm(x: np.ndarray, delta, w: np.ndarray, eps: float):
    """(residual, normed) of tokens x n rows: residual = x + delta, normed = RmsNorm(residual)
    (models/qwen35/decoder.cpp:504-509).  delta may be None."""
    x = np.atleast_2d(_f32(x))
    w = _f32(w)
    d = None if delta is None else np.atleast_2d(_f32(delta))
    residual = np.empty_like(x)
    normed = np.empty_like(x)
    for t in range(x.shape[0]):
        lib().gufo_oracle_res_norm(_p(x[t]), None if d is None else _p(d[t]), _p(w),
                                   x.shape[1], eps, _p(residual[t]), _p(normed[t]))
    return residual, normed


def swiglu(gate_up: np.ndarray) -> np.ndarray:
    """silu(gate) * up of tokens x 2f rows [gate | up] (models/qwen35/decoder.cpp:511-514)."""
    g = np.atleast_2d(_f32(gate_up))
    f = g.shape[1] // 2
    act = np.empty((g.shape[0], f), dtype=np.float32)
    for t in range(g.shape[0]):
        lib().gufo_oracle_swiglu(_p(g[t]), f, _p(act[t]))
    return act


def shared_expert_scale(logit, use_ref: bool = False) -> np.float32:
    """Sigmoid of the shared expert's gate logit, in double, rounded to fp32
    (models/qwen35/moe.cpp:44-47)."""
    if use_ref:
        return np.float32(ref().ref_shared_expert_scale(float(np.float32(logit))))
    return np.float32(1.0 / (1.0 + np.exp(-np.float64(np.float32(logit)))))


def moe_layer(router_type, router, gate, gate_type, up, up_type, down, down_type, experts,
              hidden, ffn, x, k, shared=None, threads: int = 1):
    """Decoder::MoeFfn (models/qwen35/decoder.cpp:530-558) for every token of x: the router
    product, Route over its first `experts` logits, the chosen experts, and - with
    `shared`, the shared expert's output rows - the start value shared * scale(logit
    `experts`).  Products and sums in double.  Returns ids, weights, y."""
    x = _f32(x)
    rows = router.shape[0]
    logits = matmul([(router_type, router, 0, rows)], x, precision="double", threads=threads)
    ids, weights, routed = moe_ffn(gate, gate_type, up, up_type, down, down_type, experts,
                                   hidden, ffn, np.ascontiguousarray(logits[:, :experts]), x, k,
                                   precision="double", threads=threads)
    y = routed.astype(np.float64)
    if shared is not None:
        scale = np.array([shared_expert_scale(l) for l in logits[:, experts]], np.float32)
        y = y + (_f32(shared) * scale[:, None]).astype(np.float64)
    return ids, weights, y.astype(np.float32)


CONFIG_FIELDS = ("layers", "mtp_layers", "hidden", "ffn", "vocab", "full_attention_interval",
                 "heads", "kv_heads", "head_dim", "rope_dim", "conv_kernel", "linear_key_heads",
                 "linear_value_heads", "linear_head_dim", "experts", "experts_used",
                 "expert_ffn", "shared_expert_ffn", "tied_embeddings", "has_mtp_layer")


class RefModel:
    """A GGUF file opened by the compiled reference: its reader, ReadConfig and
    GgufProjections (core/gguf.cpp, models/qwen35/config.cpp, gguf_projections.cpp)."""

    def __init__(self, path):
        self.handle = ref().ref_gguf_open(str(path).encode())
        if not self.handle:
            raise RuntimeError(ref().ref_last_error().decode())
        fields = np.zeros(len(CONFIG_FIELDS), dtype=np.int32)
        eps = np.zeros(1, dtype=np.float32)
        ref().ref_gguf_config(self.handle, _p(fields), _p(eps))
        self.config = dict(zip(CONFIG_FIELDS, (int(v) for v in fields)))
        self.config["rms_eps"] = float(eps[0])

    def apply(self, stage: int, layer: int, x: np.ndarray, outputs: int, expert: int = -1,
              exact: bool = False) -> np.ndarray:
        """Projections::Apply (ApplyExpert with expert >= 0) on tokens x inputs rows."""
        x = np.atleast_2d(_f32(x))
        y = np.empty((x.shape[0], outputs), dtype=np.float32)
        if ref().ref_gguf_apply(self.handle, stage, layer, expert, _p(x), x.shape[0], _p(y),
                                int(exact)) != 0:
            raise RuntimeError(ref().ref_last_error().decode())
        return y

    def close(self):
        if self.handle:
            ref().ref_gguf_close(self.handle)
            self.handle = None


class RefDecoder:
    """The reference's Decoder (models/qwen35/decoder.cpp) on a RefModel, over the
    reference's own GgufProjections ("float" / "double") or over foreign entry points with
    the signatures of gufo_model_apply / gufo_model_apply_expert: `foreign` is then
    (model handle, apply function, apply_expert function) as ctypes objects."""

    def __init__(self, model: RefModel, projections: str = "float", foreign=None):
        self.model = model
        which = {"float": 0, "double": 1, "foreign": 2}[projections]
        handle, apply, apply_expert = foreign if foreign is not None else (None, None, None)
        self.handle = ref().ref_decoder_open(
            model.handle, which, handle,
            None if apply is None else C.cast(apply, C.c_void_p),
            None if apply_expert is None else C.cast(apply_expert, C.c_void_p))
        if not self.handle:
            raise RuntimeError(ref().ref_last_error().decode())

    def step(self, token: int) -> np.ndarray:
        """Decoder::Step: the logits after `token` at the decoder's position."""
        logits = np.empty(self.model.config["vocab"], dtype=np.float32)
        if ref().ref_decoder_step(self.handle, int(token), _p(logits)) != 0:
            raise RuntimeError(ref().ref_last_error().decode())
        return logits

    def reset(self) -> None:
        ref().ref_decoder_reset(self.handle)

    @property
    def foreign_calls(self) -> int:
        return int(ref().ref_decoder_foreign_calls(self.handle))

    def close(self) -> None:
        if self.handle:
            ref().ref_decoder_close(self.handle)
            self.handle = None


# ---- which tensors make up which stage -------------------------------------------------
# Stage numbers of qwen35::Stage (models/qwen35/projections.hpp:14-39).
(STAGE_LINEAR_IN, STAGE_ATTENTION_IN, STAGE_MIXER_OUT, STAGE_FFN_IN, STAGE_FFN_DOWN,
 STAGE_LM_HEAD, STAGE_ROUTER, STAGE_EXPERT_IN, STAGE_EXPERT_DOWN, STAGE_MTP_IN) = range(10)


def stage_parts(config: dict, stage: int, layer: int, expert: int = -1):
    """The row ranges of one stage as (tensor name, first row, rows or None for all), in
    output order: the table the GgufProjections constructor builds and Apply /
    ApplyExpert read (models/qwen35/gguf_projections.cpp:100-237).  `config` holds the
    Config fields (CONFIG_FIELDS).  An empty list: the layer has no such stage."""
    c = config
    moe = c["experts"] > 0
    full = layer >= c["layers"] or (layer + 1) % c["full_attention_interval"] == 0
    p = f"blk.{layer}."
    tail = "_shexp.weight" if moe else ".weight"
    if stage == STAGE_LM_HEAD:
        return [("token_embd.weight" if c["tied_embeddings"] else "output.weight", 0, None)]
    if stage == STAGE_LINEAR_IN:
        names = [] if full else ["attn_qkv", "attn_gate", "ssm_alpha", "ssm_beta"]
        return [(p + n + ".weight", 0, None) for n in names]
    if stage == STAGE_ATTENTION_IN:
        names = ["attn_q", "attn_k", "attn_v"] if full else []
        return [(p + n + ".weight", 0, None) for n in names]
    if stage == STAGE_MIXER_OUT:
        return [(p + ("attn_output" if full else "ssm_out") + ".weight", 0, None)]
    if stage == STAGE_FFN_IN:
        return [(p + "ffn_gate" + tail, 0, None), (p + "ffn_up" + tail, 0, None)]
    if stage == STAGE_FFN_DOWN:
        return [(p + "ffn_down" + tail, 0, None)]
    if stage == STAGE_ROUTER:
        if not moe:
            return []
        return [(p + "ffn_gate_inp.weight", 0, None), (p + "ffn_gate_inp_shexp.weight", 0, None)]
    if stage == STAGE_MTP_IN:
        return [(p + "nextn.eh_proj.weight", 0, None)] if layer >= c["layers"] else []
    if stage == STAGE_EXPERT_IN and moe and 0 <= expert < c["experts"]:
        f = c["expert_ffn"]
        return [(p + "ffn_gate_exps.weight", expert * f, f),
                (p + "ffn_up_exps.weight", expert * f, f)]
    if stage == STAGE_EXPERT_DOWN and moe and 0 <= expert < c["experts"]:
        h = c["hidden"]
        return [(p + "ffn_down_exps.weight", expert * h, h)]
    return []


def _full_attention(c: dict, layer: int) -> bool:
    return layer >= c["layers"] or (layer + 1) % c["full_attention_interval"] == 0


def stage_inputs(c: dict, stage: int, layer: int) -> int:
    """StageInputs (models/qwen35/reference.cpp:609-624): values per token row read."""
    if stage == STAGE_MIXER_OUT:
        return (c["heads"] * c["head_dim"] if _full_attention(c, layer)
                else c["linear_value_heads"] * c["linear_head_dim"])
    if stage == STAGE_FFN_DOWN:
        return c["shared_expert_ffn"] if c["experts"] > 0 else c["ffn"]
    if stage == STAGE_EXPERT_DOWN:
        return c["expert_ffn"]
    if stage == STAGE_MTP_IN:
        return 2 * c["hidden"]
    return c["hidden"]


def stage_outputs(c: dict, stage: int, layer: int) -> int:
    """StageOutputs (models/qwen35/reference.cpp:626-648): values per token row written."""
    key_dim = c["linear_key_heads"] * c["linear_head_dim"]
    value_dim = c["linear_value_heads"] * c["linear_head_dim"]
    ffn = c["shared_expert_ffn"] if c["experts"] > 0 else c["ffn"]
    return {
        STAGE_LINEAR_IN: 2 * key_dim + 2 * value_dim + 2 * c["linear_value_heads"],
        STAGE_ATTENTION_IN: 2 * c["heads"] * c["head_dim"] + 2 * c["kv_heads"] * c["head_dim"],
        STAGE_MIXER_OUT: c["hidden"], STAGE_FFN_DOWN: c["hidden"],
        STAGE_EXPERT_DOWN: c["hidden"], STAGE_MTP_IN: c["hidden"],
        STAGE_FFN_IN: 2 * ffn, STAGE_LM_HEAD: c["vocab"], STAGE_ROUTER: c["experts"] + 1,
        STAGE_EXPERT_IN: 2 * c["expert_ffn"],
    }[stage]


def widen_16bit(ggml_type: int, data: np.ndarray) -> tuple[int, np.ndarray]:
    """F16 / BF16 rows as F32 rows (quant::Dequantize, core/quant.cpp:240-262): what the
    reference does with such tensors before it multiplies them."""
    raw = np.ascontiguousarray(data).view(np.uint8).reshape(data.shape[0], -1)
    if ggml_type == 1:
        wide = raw.view(np.float16).astype(np.float32)
    elif ggml_type == 30:
        wide = (raw.view(np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
    else:
        return ggml_type, raw
    return F32, np.ascontiguousarray(wide).view(np.uint8).reshape(data.shape[0], -1)


def stage_apply(config: dict, tensors: dict, stage: int, layer: int, x: np.ndarray,
                expert: int = -1, precision: str = "double", threads: int = 4) -> np.ndarray:
    """Projections::Apply / ApplyExpert by the checker.  tensors: name -> (ggml type,
    bytes[rows_total, row_bytes])."""
    parts = []
    for name, first, rows in stage_parts(config, stage, layer, expert):
        ggml_type, data = widen_16bit(*tensors[name])
        parts.append((ggml_type, data, first, data.shape[0] if rows is None else rows))
    if not parts:
        raise LookupError("qwen35: no weights for this stage and layer")
    return matmul(parts, np.atleast_2d(_f32(x)), precision=precision, threads=threads)


def rel_l2(got: np.ndarray, want: np.ndarray) -> float:
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300))
