"""Writes GGUF v3 images and builds small synthetic Qwen3.5-shaped models.

The backend reads real model files through its own GGUF reader
(gufo-npu_amd/host/gguf_model.cpp).  No model file exists where the tests run, so they
are handed synthetic ones: the same metadata keys and tensor names as a Qwen3.5 /
Qwen3.6 file (src/models/qwen35/config.cpp:18-72 and gguf_projections.cpp:100-175 of the
reference list them), a few layers, small widths, seeded weights.  The reference's own
tests build their GGUF images in memory the same way (tests/core/gguf_test.cpp:13-98).

Layout written (the GGUF v3 container): "GGUF", u32 version 3, u64 tensor count, u64
metadata count; metadata as (string key, u32 value type, value); tensor records as
(string name, u32 rank, u64 dims in ggml order - dims[0] is the contiguous one -, u32
ggml type, u64 offset into the data section); zero padding to `general.alignment`
(32); the tensors' bytes, each aligned.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field

import numpy as np

from . import synth

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 8, 12, 13, 14, 30

# Metadata value types of the container.
_U32, _F32, _BOOL, _STRING, _ARRAY, _U64 = 4, 6, 7, 8, 9, 10
ALIGNMENT = 32


def _string(text: str) -> bytes:
    raw = text.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", _BOOL, int(v))
    if isinstance(v, int):
        return struct.pack("<II", _U32, v) if v < 2 ** 32 else struct.pack("<IQ", _U64, v)
    if isinstance(v, float):
        return struct.pack("<If", _F32, v)
    if isinstance(v, str):
        return struct.pack("<I", _STRING) + _string(v)
    if isinstance(v, (list, tuple)):  # arrays of strings only
        return struct.pack("<IIQ", _ARRAY, _STRING, len(v)) + b"".join(_string(s) for s in v)
    raise TypeError(f"no GGUF value type for {type(v)}")


@dataclass
class TensorSpec:
    name: str
    ggml_type: int
    shape: tuple          # ggml order: (cols, rows[, experts])
    data: np.ndarray      # the bytes as stored, any shape, uint8


def _header(metadata: dict, tensors: list[TensorSpec]) -> bytes:
    """Everything before the data section, padding included."""
    head = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(metadata)))
    for key, v in metadata.items():
        head += _string(key) + _value(v)
    at = 0
    for t in tensors:
        head += _string(t.name) + struct.pack("<I", len(t.shape))
        head += b"".join(struct.pack("<Q", d) for d in t.shape)
        head += struct.pack("<IQ", t.ggml_type, at)
        at += (t.data.size + ALIGNMENT - 1) // ALIGNMENT * ALIGNMENT
    head += b"\0" * (-len(head) % ALIGNMENT)
    return bytes(head)


def write_file(path, metadata: dict, tensors: list[TensorSpec]) -> None:
    """A GGUF v3 file holding `metadata` and `tensors`, streamed tensor by tensor."""
    with open(path, "wb") as f:
        f.write(_header(metadata, tensors))
        for t in tensors:
            raw = np.ascontiguousarray(t.data).view(np.uint8).reshape(-1)
            f.write(raw.data)
            f.write(b"\0" * (-raw.size % ALIGNMENT))


def write_image(metadata: dict, tensors: list[TensorSpec]) -> bytes:
    """The same file as bytes in memory (for small models and for damaging on purpose)."""
    parts = [_header(metadata, tensors)]
    for t in tensors:
        raw = np.ascontiguousarray(t.data).view(np.uint8).reshape(-1)
        parts += [raw.tobytes(), b"\0" * (-raw.size % ALIGNMENT)]
    return b"".join(parts)


# ---- synthetic models ---------------------------------------------------------------

@dataclass
class ModelSpec:
    """Shape of a synthetic model, in the vocabulary of the reference's Config
    (src/models/qwen35/config.hpp:13-60)."""
    architecture: str = "qwen35"
    layers: int = 4
    mtp_layers: int = 0
    hidden: int = 512
    ffn: int = 768
    vocab: int = 1000
    rms_eps: float = 1e-6
    full_attention_interval: int = 4
    heads: int = 4
    kv_heads: int = 2
    head_dim: int = 128
    linear_key_heads: int = 2
    linear_value_heads: int = 4
    linear_head_dim: int = 128
    experts: int = 0
    experts_used: int = 0
    expert_ffn: int = 0
    shared_expert_ffn: int = 0
    tied_embeddings: bool = True
    seed: int = synth.BASE_SEED + 9000
    # Row type per tensor suffix; anything not named takes `default_type`.
    default_type: int = Q4_K
    types: dict = field(default_factory=dict)

    @property
    def is_moe(self) -> bool:
        return self.experts > 0

    @property
    def ffn_width(self) -> int:
        return self.shared_expert_ffn if self.is_moe else self.ffn

    def is_full_attention(self, layer: int) -> bool:
        return layer >= self.layers or (layer + 1) % self.full_attention_interval == 0

    @property
    def key_dim(self) -> int:
        return self.linear_key_heads * self.linear_head_dim

    @property
    def value_dim(self) -> int:
        return self.linear_value_heads * self.linear_head_dim


def _half_matrix(rows: int, cols: int, seed: int, bf16: bool) -> np.ndarray:
    w = synth.rng(seed).standard_normal((rows, cols), dtype=np.float32) * np.float32(0.05)
    if bf16:
        return synth.bf16_round(w).view(np.uint8).reshape(rows, cols * 2)
    return w.astype(np.float16).view(np.uint8).reshape(rows, cols * 2)


def tensor_bytes(ggml_type: int, rows: int, cols: int, seed: int) -> np.ndarray:
    if ggml_type in (F16, BF16):
        return _half_matrix(rows, cols, seed, ggml_type == BF16)
    return synth.matrix(ggml_type, rows, cols, seed)


def model_tensors(spec: ModelSpec) -> list[TensorSpec]:
    """Every tensor the reference's decoder and projections look up, in file order."""
    out: list[TensorSpec] = []
    counter = [0]

    def add(name: str, cols: int, rows: int, experts: int = 0, one_dim: bool = False):
        suffix = name.split(".", 2)[-1] if name.startswith("blk.") else name
        ggml_type = spec.types.get(suffix, spec.default_type)
        counter[0] += 1
        total_rows = rows * max(experts, 1)
        data = tensor_bytes(ggml_type, total_rows, cols, spec.seed + counter[0])
        shape = (cols,) if one_dim else (cols, rows, experts) if experts else (cols, rows)
        out.append(TensorSpec(name, ggml_type, shape, data))

    def norm(name: str, n: int):
        counter[0] += 1
        w = 1.0 + 0.1 * synth.rng(spec.seed + counter[0]).standard_normal(n, dtype=np.float32)
        out.append(TensorSpec(name, F32, (n,), w.astype(np.float32).view(np.uint8)))

    h = spec.hidden
    attn_dim, kv_dim = spec.heads * spec.head_dim, spec.kv_heads * spec.head_dim
    add("token_embd.weight", h, spec.vocab)
    if not spec.tied_embeddings:
        add("output.weight", h, spec.vocab)
    norm("output_norm.weight", h)
    for il in range(spec.layers + spec.mtp_layers):
        p = f"blk.{il}."
        norm(p + "attn_norm.weight", h)
        norm(p + "post_attention_norm.weight", h)
        if il >= spec.layers:
            add(p + "nextn.eh_proj.weight", 2 * h, h)
        if spec.is_full_attention(il):
            add(p + "attn_q.weight", h, 2 * attn_dim)
            add(p + "attn_k.weight", h, kv_dim)
            add(p + "attn_v.weight", h, kv_dim)
            add(p + "attn_output.weight", attn_dim, h)
        else:
            add(p + "attn_qkv.weight", h, 2 * spec.key_dim + spec.value_dim)
            add(p + "attn_gate.weight", h, spec.value_dim)
            add(p + "ssm_alpha.weight", h, spec.linear_value_heads)
            add(p + "ssm_beta.weight", h, spec.linear_value_heads)
            add(p + "ssm_out.weight", spec.value_dim, h)
        if spec.is_moe:
            add(p + "ffn_gate_inp.weight", h, spec.experts)
            add(p + "ffn_gate_inp_shexp.weight", h, 1, one_dim=True)
            add(p + "ffn_gate_exps.weight", h, spec.expert_ffn, spec.experts)
            add(p + "ffn_up_exps.weight", h, spec.expert_ffn, spec.experts)
            add(p + "ffn_down_exps.weight", spec.expert_ffn, h, spec.experts)
        tail = "_shexp.weight" if spec.is_moe else ".weight"
        add(p + "ffn_gate" + tail, h, spec.ffn_width)
        add(p + "ffn_up" + tail, h, spec.ffn_width)
        add(p + "ffn_down" + tail, spec.ffn_width, h)
    # The small fp32 tensors of the mixers (src/models/qwen35/decoder.cpp:72-87 of the
    # reference), so that the reference's own decoder can run on the file.  They are
    # seeded apart from the projections and do not enter any product of this backend.
    for il in range(spec.layers + spec.mtp_layers):
        p = f"blk.{il}."
        gen = synth.rng(spec.seed + 50_000 + il)

        def small(name, shape, values):
            out.append(TensorSpec(p + name, F32, shape,
                                  np.ascontiguousarray(values, dtype=np.float32).view(np.uint8)))

        if spec.is_full_attention(il):
            for name in ("attn_q_norm.weight", "attn_k_norm.weight"):
                small(name, (spec.head_dim,),
                      1.0 + 0.1 * gen.standard_normal(spec.head_dim, dtype=np.float32))
        else:
            channels = 2 * spec.key_dim + spec.value_dim
            small("ssm_conv1d.weight", (4, channels),
                  0.3 * gen.standard_normal((channels, 4), dtype=np.float32))
            # A decay rate: negative, so the recurrent state shrinks (decoder.cpp:227).
            small("ssm_a", (spec.linear_value_heads,),
                  -np.exp(0.5 * gen.standard_normal(spec.linear_value_heads, dtype=np.float32)))
            small("ssm_dt.bias", (spec.linear_value_heads,),
                  0.5 * gen.standard_normal(spec.linear_value_heads, dtype=np.float32))
            small("ssm_norm.weight", (spec.linear_head_dim,),
                  1.0 + 0.1 * gen.standard_normal(spec.linear_head_dim, dtype=np.float32))
    return out


def model_metadata(spec: ModelSpec) -> dict:
    a = spec.architecture + "."
    meta = {
        "general.architecture": spec.architecture,
        "general.name": "synthetic " + spec.architecture,
        "general.alignment": ALIGNMENT,
        a + "block_count": spec.layers + spec.mtp_layers,
        a + "embedding_length": spec.hidden,
        a + "attention.layer_norm_rms_epsilon": float(spec.rms_eps),
        a + "full_attention_interval": spec.full_attention_interval,
        a + "attention.head_count": spec.heads,
        a + "attention.head_count_kv": spec.kv_heads,
        a + "attention.key_length": spec.head_dim,
        a + "attention.value_length": spec.head_dim,
        a + "rope.dimension_count": spec.head_dim // 2,
        a + "rope.freq_base": 1e7,
        a + "ssm.conv_kernel": 4,
        a + "ssm.state_size": spec.linear_head_dim,
        a + "ssm.group_count": spec.linear_key_heads,
        a + "ssm.time_step_rank": spec.linear_value_heads,
        a + "ssm.inner_size": spec.value_dim,
        "tokenizer.ggml.tokens": ["<a>", "<b>", "<c>"],  # an array value to step over
    }
    if spec.mtp_layers:
        meta[a + "nextn_predict_layers"] = spec.mtp_layers
    if spec.is_moe:
        meta[a + "expert_count"] = spec.experts
        meta[a + "expert_used_count"] = spec.experts_used
        meta[a + "expert_feed_forward_length"] = spec.expert_ffn
        meta[a + "expert_shared_feed_forward_length"] = spec.shared_expert_ffn
    else:
        meta[a + "feed_forward_length"] = spec.ffn
    return meta


def model_image(spec: ModelSpec) -> bytes:
    return write_image(model_metadata(spec), model_tensors(spec))


def write_model(path, spec: ModelSpec) -> None:
    write_file(path, model_metadata(spec), model_tensors(spec))


# The row types of a real Unsloth "UD-Q4_K_XL" file, in miniature: K-quants for the large
# projections, Q8_0 here and there, fp32 for the router and the per-head gates, and a
# 16-bit tensor (which the reference converts to fp32 before multiplying,
# gguf_projections.cpp:56-60).
_MIXED_TYPES = {
    "token_embd.weight": Q6_K, "attn_q.weight": Q4_K, "attn_k.weight": Q5_K,
    "attn_v.weight": Q6_K, "attn_output.weight": Q4_K, "attn_qkv.weight": Q5_K,
    "attn_gate.weight": Q8_0, "ssm_alpha.weight": F32, "ssm_beta.weight": BF16,
    "ssm_out.weight": Q6_K, "ffn_gate.weight": Q4_K, "ffn_up.weight": Q4_K,
    "ffn_down.weight": Q6_K, "nextn.eh_proj.weight": Q8_0,
    "ffn_gate_inp.weight": F32, "ffn_gate_inp_shexp.weight": F32,
    "ffn_gate_exps.weight": Q4_K, "ffn_up_exps.weight": Q4_K, "ffn_down_exps.weight": Q5_K,
    "ffn_gate_shexp.weight": Q4_K, "ffn_up_shexp.weight": Q4_K, "ffn_down_shexp.weight": Q6_K,
    "output.weight": Q6_K,
}


def tiny_dense(seed: int = synth.BASE_SEED + 9000) -> ModelSpec:
    """Four layers (three linear-attention, one full-attention), tied embeddings, one
    MTP layer: the shape of Qwen3.5-2B at 1/4 width."""
    return ModelSpec(architecture="qwen35", layers=4, mtp_layers=1, seed=seed,
                     types=dict(_MIXED_TYPES))


def dense_2b_like(seed: int = synth.BASE_SEED + 9700) -> ModelSpec:
    """The widths of the 2B decode set at full size: hidden 2048, FFN 6144, 24 layers of
    which every fourth is full attention, a 151,936-row tied Q6_K head.  About 1.2 GB."""
    return ModelSpec(architecture="qwen35", layers=24, hidden=2048, ffn=6144, vocab=151936,
                     heads=8, kv_heads=4, head_dim=128, linear_key_heads=16,
                     linear_value_heads=16, linear_head_dim=128, seed=seed,
                     types=dict(_MIXED_TYPES))


def tiny_moe(seed: int = synth.BASE_SEED + 9500) -> ModelSpec:
    """Two layers of 16 experts (top 4) plus a shared expert, untied head: the shape of
    Qwen3.6-35B-A3B in miniature."""
    types = dict(_MIXED_TYPES)
    types["ssm_beta.weight"] = F16
    return ModelSpec(architecture="qwen35moe", layers=2, full_attention_interval=2, ffn=0,
                     experts=16, experts_used=4, expert_ffn=256, shared_expert_ffn=512,
                     tied_embeddings=False, seed=seed, types=types)
