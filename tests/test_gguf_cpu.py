"""The GGUF reader, the model shape and the stage table, without a GPU.

What is checked against what:
  * this backend's reader (gufo_model_inspect, host C++) reads the synthetic files back to
    the shape they were written with, and to the Config the reference's own reader and
    ReadConfig return for the same bytes (compiled reference, and its committed output);
  * the checker's stage table (oracle.stage_parts / stage_apply) gives, for every stage
    of every layer, what the reference's GgufProjections gives: bit for bit in its
    Precision::kDouble mode (both dequantize and add in double, in the same order),
    within 1e-5 of its AVX2 fp32 mode;
  * malformed and inconsistent files are refused by this backend's reader wherever the
    reference refuses them.
"""
import struct

import numpy as np
import pytest

import gguf_cases
from conftest import GOLDEN
from gufo_npu_amd import gguf_writer as gw
from gufo_npu_amd import model as hip_model


@pytest.fixture(scope="module", params=list(gguf_cases.MODELS))
def case(request, tmp_path_factory):
    path, spec = gguf_cases.write_model(request.param, tmp_path_factory.mktemp("gguf"))
    golden = np.load(GOLDEN / "gguf" / f"{request.param}.npz")
    return request.param, path, spec, golden


def test_library_exports_every_declared_symbol():
    lib = hip_model.load_library()
    header = (GOLDEN.parent.parent / "include" / "gufo_hip_model.h").read_text()
    import re
    declared = set(re.findall(r"\b(gufo_model_[a-z_]+)\(", header))
    assert declared == set(hip_model.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None


def test_reader_returns_the_shape_that_was_written(case):
    _, path, spec, _ = case
    shape = hip_model.inspect(path)
    want = gguf_cases.config_of(spec)
    for field, value in want.items():
        assert shape[field] == value, field
    assert shape["is_moe"] == int(spec.is_moe)
    assert shape["rms_eps"] == np.float32(spec.rms_eps)
    assert shape["rope_theta"] == np.float32(1e7)
    assert shape["tensors"] == len(gw.model_tensors(spec))


def test_reader_agrees_with_the_reference_config(case, oracle):
    # The Config the reference read from these very bytes, as committed with the golden
    # outputs ...
    _, path, _, golden = case
    shape = hip_model.inspect(path)
    for field, value in zip(oracle.CONFIG_FIELDS, golden["config_fields"]):
        assert shape[field] == int(value), field
    assert shape["rms_eps"] == golden["rms_eps"][0]


def test_reader_agrees_with_the_compiled_reference(case, ref_oracle):
    # ... and as the compiled reference reads them now.
    _, path, _, _ = case
    shape = hip_model.inspect(path)
    model = ref_oracle.RefModel(path)
    for field in ref_oracle.CONFIG_FIELDS:
        assert shape[field] == model.config[field], field
    assert shape["rms_eps"] == np.float32(model.config["rms_eps"])
    model.close()


def test_stage_table_matches_reference_outputs(case, oracle):
    name, _, spec, golden = case
    config = dict(zip(oracle.CONFIG_FIELDS, (int(v) for v in golden["config_fields"])))
    tensors = gguf_cases.tensors_by_name(spec)
    worst = 0.0
    for stage, layer, expert in gguf_cases.calls(spec):
        x = gguf_cases.call_input(oracle, config, stage, layer, expert)
        key = gguf_cases.call_key(stage, layer, expert)
        exact = oracle.stage_apply(config, tensors, stage, layer, x, expert, precision="double")
        assert exact.shape == golden[key + "_exact"].shape, key
        assert np.array_equal(exact, golden[key + "_exact"]), key
        fused = oracle.stage_apply(config, tensors, stage, layer, x, expert, precision="float")
        worst = max(worst, oracle.rel_l2(fused, golden[key + "_fused"]))
        assert oracle.stage_outputs(config, stage, layer) == exact.shape[1]
    assert worst <= 1e-5
    print(name, "fused fp32 orders differ by", worst)


def test_stage_table_matches_compiled_reference(case, ref_oracle):
    # The same through the compiled reference, on a token count the fixtures do not hold.
    _, path, spec, _ = case
    model = ref_oracle.RefModel(path)
    tensors = gguf_cases.tensors_by_name(spec)
    for stage, layer, expert in gguf_cases.calls(spec):
        x = gguf_cases.call_input(ref_oracle, model.config, stage, layer, expert, tokens=3)
        want = model.apply(stage, layer, x, ref_oracle.stage_outputs(model.config, stage, layer),
                           expert, exact=True)
        got = ref_oracle.stage_apply(model.config, tensors, stage, layer, x, expert)
        assert np.array_equal(got, want), (stage, layer, expert)
    model.close()


def test_stages_a_layer_does_not_have(case, oracle):
    _, _, spec, golden = case
    config = dict(zip(oracle.CONFIG_FIELDS, (int(v) for v in golden["config_fields"])))
    linear_layer, full_layer = 0, spec.full_attention_interval - 1
    assert oracle.stage_parts(config, oracle.STAGE_ATTENTION_IN, linear_layer) == []
    assert oracle.stage_parts(config, oracle.STAGE_LINEAR_IN, full_layer) == []
    assert oracle.stage_parts(config, oracle.STAGE_MTP_IN, 0) == []
    if not spec.is_moe:
        assert oracle.stage_parts(config, oracle.STAGE_ROUTER, 0) == []
        assert oracle.stage_parts(config, oracle.STAGE_EXPERT_IN, 0, 0) == []
    else:
        assert oracle.stage_parts(config, oracle.STAGE_EXPERT_IN, 0, spec.experts) == []


# ---- files the reader must refuse -----------------------------------------------------

def _dense_parts():
    spec = gw.tiny_dense()
    return spec, gw.model_metadata(spec), gw.model_tensors(spec)


def _refused(tmp_path, image: bytes, fragment: str, ref_oracle=None):
    path = tmp_path / "bad.gguf"
    path.write_bytes(image)
    with pytest.raises(hip_model.capi.GufoHipError) as caught:
        hip_model.inspect(path)
    assert fragment in str(caught.value), str(caught.value)
    return path


BAD_HEADERS = [
    ("bad magic", lambda b: b"GGUX" + b[4:], "bad magic"),
    ("version 2", lambda b: b[:4] + struct.pack("<I", 2) + b[8:], "unsupported version 2"),
    ("cut inside the metadata", lambda b: b[:200], "truncated header"),
    ("cut inside the tensor data", lambda b: b[:len(b) // 2], "runs past the end of the file"),
    ("empty", lambda b: b"", "cannot mmap"),
]


@pytest.mark.parametrize("label,damage,fragment", BAD_HEADERS, ids=[c[0] for c in BAD_HEADERS])
def test_damaged_container_is_refused(tmp_path, label, damage, fragment):
    spec = gw.tiny_dense()
    _refused(tmp_path, damage(gw.model_image(spec)), fragment)


def test_missing_file_is_refused(tmp_path):
    with pytest.raises(hip_model.capi.GufoHipError) as caught:
        hip_model.inspect(tmp_path / "none.gguf")
    assert "cannot open" in str(caught.value)


def _variants():
    """(label, metadata edit, tensor edit, message fragment) - each breaks one rule of
    ReadConfig (config.cpp:18-72) or of the stage table's shape checks
    (gguf_projections.cpp:25-46,100-175)."""
    def drop_key(key):
        return lambda meta: meta.pop("qwen35." + key)

    def set_key(key, value):
        return lambda meta: meta.__setitem__("qwen35." + key, value)

    def drop_tensor(name):
        return lambda ts: ts.remove(next(t for t in ts if t.name == name))

    def reshape(name, shape):
        def edit(ts):
            t = next(t for t in ts if t.name == name)
            t.shape = shape
        return edit

    return [
        ("another architecture", lambda m: m.__setitem__("general.architecture", "llama"), None,
         "not a Qwen3.5 GGUF: llama"),
        ("no block_count", drop_key("block_count"), None, "missing key qwen35.block_count"),
        ("no rms epsilon", drop_key("attention.layer_norm_rms_epsilon"), None,
         "missing float key"),
        ("block_count is a string", set_key("block_count", "five"), None,
         "is not an unsigned integer"),
        ("value heads do not match", set_key("attention.value_length", 64), None,
         "key and value head dims differ"),
        ("inner size does not match", set_key("ssm.inner_size", 100), None, "ssm.inner_size"),
        ("heads not a multiple of kv heads", set_key("attention.head_count_kv", 3), None,
         "inconsistent shape metadata"),
        ("dense model without an FFN width", drop_key("feed_forward_length"), None,
         "inconsistent FFN or expert metadata"),
        ("dense model with experts", set_key("expert_count", 4), None,
         "inconsistent FFN or expert metadata"),
        ("no embedding", None, drop_tensor("token_embd.weight"), "missing tensor token_embd.weight"),
        ("no ffn_up in layer 2", None, drop_tensor("blk.2.ffn_up.weight"),
         "missing tensor blk.2.ffn_up.weight"),
        ("attn_k of the wrong height", None, reshape("blk.3.attn_k.weight", (512, 128, 2)),
         "tensor blk.3.attn_k.weight has shape [512, 128, 2], expected [512, 256]"),
        ("ssm_out transposed", None, reshape("blk.0.ssm_out.weight", (256, 1024)),
         "tensor blk.0.ssm_out.weight has shape [256, 1024], expected [512, 512]"),
    ]


VARIANTS = _variants()


@pytest.mark.parametrize("label,meta_edit,tensor_edit,fragment", VARIANTS,
                         ids=[v[0] for v in VARIANTS])
def test_inconsistent_model_is_refused(tmp_path, label, meta_edit, tensor_edit, fragment):
    spec, meta, tensors = _dense_parts()
    if meta_edit is not None:
        meta_edit(meta)
    if tensor_edit is not None:
        tensor_edit(tensors)
    _refused(tmp_path, gw.write_image(meta, tensors), fragment)


@pytest.mark.parametrize("label,meta_edit,tensor_edit,fragment", VARIANTS,
                         ids=[v[0] for v in VARIANTS])
def test_reference_refuses_the_same_files(tmp_path, ref_oracle, label, meta_edit, tensor_edit,
                                          fragment):
    # The compiled reference rejects each of these files too, with the same message.
    spec, meta, tensors = _dense_parts()
    if meta_edit is not None:
        meta_edit(meta)
    if tensor_edit is not None:
        tensor_edit(tensors)
    path = tmp_path / "bad.gguf"
    path.write_bytes(gw.write_image(meta, tensors))
    with pytest.raises(RuntimeError) as caught:
        ref_oracle.RefModel(path)
    assert fragment in str(caught.value), str(caught.value)


def test_unknown_tensor_type_and_partial_block(tmp_path):
    spec, meta, tensors = _dense_parts()
    victim = next(t for t in tensors if t.name == "blk.1.ffn_down.weight")
    victim.ggml_type = 2  # Q4_0: not a type these models use
    _refused(tmp_path, gw.write_image(meta, tensors), "unsupported ggml type 2 for blk.1.ffn_down")
    spec, meta, tensors = _dense_parts()
    victim = next(t for t in tensors if t.name == "blk.1.ffn_down.weight")
    victim.shape = (700, 512)
    _refused(tmp_path, gw.write_image(meta, tensors), "is not a whole number of blocks")


def test_signed_and_wide_integers_are_read(tmp_path):
    # Writers differ in the integer type they pick for a count; GetUInt takes any
    # unsigned type and a signed one that is not negative (gguf.cpp:296-309).
    spec, meta, tensors = _dense_parts()
    image = bytearray(gw.write_image(meta, tensors))
    key = b"qwen35.embedding_length"
    at = image.index(key) + len(key)
    assert struct.unpack_from("<I", image, at)[0] == 4          # u32 ...
    struct.pack_into("<I", image, at, 5)                          # ... read as i32
    path = tmp_path / "signed.gguf"
    path.write_bytes(bytes(image))
    assert hip_model.inspect(path)["hidden"] == spec.hidden
    struct.pack_into("<i", image, at + 4, -512)
    path.write_bytes(bytes(image))
    with pytest.raises(hip_model.capi.GufoHipError) as caught:
        hip_model.inspect(path)
    assert "is not an unsigned integer" in str(caught.value)
