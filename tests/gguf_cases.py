"""The synthetic model files of the GGUF tests: their specs, tensors by name, the list of
(stage, layer, expert) calls that exercise every row of the stage table, and seeded
inputs.  Shared by the CPU tests, the GPU tests and the golden-vector writer, so all
three see identical bytes."""
from __future__ import annotations

import numpy as np

from gufo_npu_amd import gguf_writer, synth

MODELS = {"tiny_dense": gguf_writer.tiny_dense, "tiny_moe": gguf_writer.tiny_moe}
TOKENS = 2  # rows per golden call


def config_of(spec: gguf_writer.ModelSpec) -> dict:
    """The reference's Config fields for `spec` (what ReadConfig must return)."""
    return {
        "layers": spec.layers, "mtp_layers": spec.mtp_layers, "hidden": spec.hidden,
        "ffn": spec.ffn, "vocab": spec.vocab,
        "full_attention_interval": spec.full_attention_interval, "heads": spec.heads,
        "kv_heads": spec.kv_heads, "head_dim": spec.head_dim, "rope_dim": spec.head_dim // 2,
        "conv_kernel": 4, "linear_key_heads": spec.linear_key_heads,
        "linear_value_heads": spec.linear_value_heads, "linear_head_dim": spec.linear_head_dim,
        "experts": spec.experts, "experts_used": spec.experts_used,
        "expert_ffn": spec.expert_ffn, "shared_expert_ffn": spec.shared_expert_ffn,
        "tied_embeddings": int(spec.tied_embeddings), "has_mtp_layer": int(spec.mtp_layers > 0),
    }


def tensors_by_name(spec: gguf_writer.ModelSpec) -> dict:
    """name -> (ggml type, bytes[rows_total, row_bytes]) for the 2-D and 3-D tensors."""
    out = {}
    for t in gguf_writer.model_tensors(spec):
        rows = 1
        for d in t.shape[1:]:
            rows *= d
        out[t.name] = (t.ggml_type, np.ascontiguousarray(t.data).view(np.uint8).reshape(rows, -1))
    return out


def calls(spec: gguf_writer.ModelSpec):
    """(stage, layer, expert) for every stage every loaded layer has, the head, and three
    experts of every mixture layer."""
    out = [(5, -1, -1)]  # lm_head
    for il in range(spec.layers + spec.mtp_layers):
        full = spec.is_full_attention(il)
        out.append((1 if full else 0, il, -1))
        out += [(2, il, -1), (3, il, -1), (4, il, -1)]
        if il >= spec.layers:
            out.append((9, il, -1))
        if spec.is_moe:
            out.append((6, il, -1))
            for expert in (0, spec.experts // 2 + 1, spec.experts - 1):
                out += [(7, il, expert), (8, il, expert)]
    return out


def call_key(stage: int, layer: int, expert: int) -> str:
    return f"s{stage}_l{layer}_e{expert}"


def call_input(oracle, config: dict, stage: int, layer: int, expert: int,
               tokens: int = TOKENS) -> np.ndarray:
    seed = synth.BASE_SEED + 9900 + 97 * stage + 13 * (layer + 1) + 5 * (expert + 1) + tokens
    return synth.activations(tokens, oracle.stage_inputs(config, stage, layer), seed)


def write_model(name: str, directory) -> tuple:
    """Writes MODELS[name] into `directory`; returns (path, spec)."""
    spec = MODELS[name]()
    path = directory / f"{name}.gguf"
    path.write_bytes(gguf_writer.model_image(spec))
    return path, spec
