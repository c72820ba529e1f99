"""A model file through the whole backend: GGUF reader -> stage table -> weights in HBM ->
Projections::Apply / ApplyExpert on the MI355X, against what the reference's own
GgufProjections returned for the same file (tests/golden/gguf, written by
tests/golden/make_gguf_golden.py) and against the checker's stage table.

Bars: rel-L2 <= 1e-4 against the reference's Precision::kDouble outputs and against its
fp32 outputs; stage widths equal StageInputs / StageOutputs; the reference's exceptions
for stages and experts a model does not have."""
import numpy as np
import pytest

import gguf_cases
from conftest import GOLDEN
from gufo_npu_amd import model as hip_model

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-4


def say(*args):
    print(*args, flush=True)


@pytest.fixture(scope="module", params=list(gguf_cases.MODELS))
def opened(request, tmp_path_factory, hip):
    path, spec = gguf_cases.write_model(request.param, tmp_path_factory.mktemp("gguf"))
    golden = np.load(GOLDEN / "gguf" / f"{request.param}.npz")
    say("open", request.param)
    model = hip_model.Model(path)
    yield request.param, spec, golden, model
    model.close()


def test_shape_and_resident_bytes(opened, oracle):
    _, spec, golden, model = opened
    for field, value in zip(oracle.CONFIG_FIELDS, golden["config_fields"]):
        assert model.shape[field] == int(value), field
    # Every projection tensor is resident; 16-bit tensors count at their fp32 size.
    config = dict(zip(oracle.CONFIG_FIELDS, (int(v) for v in golden["config_fields"])))
    tensors = gguf_cases.tensors_by_name(spec)
    names = {oracle.stage_parts(config, oracle.STAGE_LM_HEAD, -1)[0][0]}
    for layer in range(spec.layers + spec.mtp_layers):
        for stage in range(10):
            names.update(part[0] for part in oracle.stage_parts(config, stage, layer, expert=0))
    want = 0
    for name in names:
        ggml_type, data = tensors[name]
        want += data.size * (2 if ggml_type in (1, 30) else 1)
    assert model.weight_bytes == want


def test_every_stage_matches_the_reference(opened, oracle):
    name, spec, golden, model = opened
    config = dict(zip(oracle.CONFIG_FIELDS, (int(v) for v in golden["config_fields"])))
    worst = 0.0
    for stage, layer, expert in gguf_cases.calls(spec):
        say(name, hip_model.STAGE_NAMES[stage], "layer", layer, "expert", expert)
        x = gguf_cases.call_input(oracle, config, stage, layer, expert)
        key = gguf_cases.call_key(stage, layer, expert)
        assert model.stage_inputs(stage, layer) == x.shape[1]
        assert model.stage_outputs(stage, layer) == oracle.stage_outputs(config, stage, layer)
        got = model.apply(stage, layer, x, expert)
        err = oracle.rel_l2(got, golden[key + "_exact"])
        worst = max(worst, err)
        assert err <= TOLERANCE, (key, err)
        assert oracle.rel_l2(got, golden[key + "_fused"]) <= TOLERANCE, key
    say(name, "worst rel-L2 against the reference", worst)


def test_token_counts_beyond_the_fixtures(opened, oracle):
    # 1, 3 and 5 rows (5 runs as two passes over the weights) against the checker's
    # stage table, which the CPU tests tie to the reference bit for bit.
    name, spec, golden, model = opened
    config = dict(zip(oracle.CONFIG_FIELDS, (int(v) for v in golden["config_fields"])))
    tensors = gguf_cases.tensors_by_name(spec)
    for stage, layer, expert in gguf_cases.calls(spec)[:12]:
        for tokens in (1, 3, 5):
            say(name, hip_model.STAGE_NAMES[stage], "layer", layer, "expert", expert, "N", tokens)
            x = gguf_cases.call_input(oracle, config, stage, layer, expert, tokens)
            want = oracle.stage_apply(config, tensors, stage, layer, x, expert)
            got = model.apply(stage, layer, x, expert)
            assert oracle.rel_l2(got, want) <= TOLERANCE


def test_norm_weights_are_the_files(opened):
    _, spec, _, model = opened
    tensors = gguf_cases.tensors_by_name(spec)
    layers = spec.layers + spec.mtp_layers
    for layer in (0, layers - 1):
        for which, tensor in ((0, "attn_norm"), (1, "post_attention_norm")):
            want = tensors[f"blk.{layer}.{tensor}.weight"][1].view(np.float32).reshape(-1)
            assert np.array_equal(model.norm_weight(which, layer), want)
    want = tensors["output_norm.weight"][1].view(np.float32).reshape(-1)
    assert np.array_equal(model.norm_weight(2), want)


def test_calls_the_reference_refuses(opened):
    _, spec, _, model = opened
    capi = hip_model.capi
    x = np.zeros((1, spec.hidden), dtype=np.float32)
    layers = spec.layers + spec.mtp_layers
    say("refused calls")
    with pytest.raises(capi.LogicError):      # a linear-attention layer has no attention_in
        model.apply(hip_model.ATTENTION_IN, 0, x)
    with pytest.raises(capi.LogicError):      # expert stages go through apply_expert
        model.apply(hip_model.EXPERT_IN, 0, x)
    with pytest.raises(capi.OutOfRangeError):  # std::vector::at in Apply
        model.apply(hip_model.FFN_IN, layers, x)
    if spec.is_moe:
        with pytest.raises(capi.LogicError):  # no such expert
            model.apply(hip_model.EXPERT_IN, 0, x, expert=spec.experts)
        with pytest.raises(capi.LogicError):  # ApplyExpert takes expert stages only
            model.apply(hip_model.FFN_IN, 0, x, expert=0)
    else:
        with pytest.raises(capi.LogicError):  # a dense model has no router and no experts
            model.apply(hip_model.ROUTER, 0, x)
        with pytest.raises(capi.LogicError):
            model.apply(hip_model.EXPERT_IN, 0, x, expert=0)
    with pytest.raises(capi.InvalidArgumentError):
        model.apply(42, 0, x)


def test_a_loaded_model_lends_its_matrices_to_the_device_entry_points(opened, hip, oracle):
    # gufo_model_stage_matrices / _expert_matrices: the matrices a model file was loaded
    # into, used with rows that stay on the device.  Apply through the handles equals
    # Apply through the model bit for bit; the stages with a prologue, the prefill product
    # and - on the mixture model - the whole mixture layer run on them.
    name, spec, golden, model = opened
    from gufo_npu_amd import synth
    hidden, tokens = model.shape["hidden"], 3
    x = synth.activations(tokens, hidden, 4242) * np.float32(0.1)
    dx = hip.DeviceBuffer.from_array(x)
    for stage in (hip_model.ATTENTION_IN, hip_model.FFN_IN, hip_model.LM_HEAD):
        layer = -1 if stage == hip_model.LM_HEAD else 0
        mats = model.stage_matrices(stage, layer)
        if not mats:  # a stage this layer does not have
            assert model.stage_outputs(stage, layer) == 0
            continue
        say(name, "borrowed", hip_model.STAGE_NAMES[stage], len(mats), "matrices")
        outputs = model.stage_outputs(stage, layer)
        assert sum(m.rows for m in mats) == outputs and all(m.cols == hidden for m in mats)
        dy = hip.DeviceBuffer(4 * tokens * outputs)
        hip.gemv_dev([hip.whole(m) for m in mats], dx, tokens, dy)
        hip.synchronize()
        got = dy.download((tokens, outputs), np.float32)
        want = model.apply(stage, layer, x)
        assert bool(np.array_equal(got.view(np.uint32), want.view(np.uint32)))
        if all(m.type in (synth.Q4_K, synth.Q5_K, synth.Q6_K, synth.Q8_0) for m in mats):
            bits = synth.bf16_round(x)
            da = hip.DeviceBuffer.from_array(bits)
            hip.gemm_bf16_parts_dev(mats, da, tokens, dy)
            hip.synchronize()
            prefill = dy.download((tokens, outputs), np.float32)
            assert oracle.rel_l2(prefill, model.apply(stage, layer, synth.bf16_to_float(bits))) <= 1e-3
    assert model.stage_matrices(hip_model.MTP_IN, 0) == [] or spec.mtp_layers > 0
    gate, up, down = model.expert_matrices(0)
    if not model.shape["is_moe"]:
        assert gate is None and up is None and down is None
        return
    experts, k = model.shape["experts"], model.shape["experts_used"]
    router = model.stage_matrices(hip_model.ROUTER, 0)
    say(name, "mixture layer on borrowed matrices:", len(router), "router tensors")
    shared = synth.activations(tokens, hidden, 4243)
    ds = hip.DeviceBuffer.from_array(shared)
    dy = hip.DeviceBuffer(4 * tokens * hidden)
    hip.moe_layer_dev(router, gate, up, down, experts, k, dx, tokens, ds, dy)
    hip.synchronize()
    got = dy.download((tokens, hidden), np.float32)
    # the same through the model's host-pointer calls, as Decoder::MoeFfn makes them
    logits = model.apply(hip_model.ROUTER, 0, x)
    assert logits.shape[1] == experts + 1
    ids, weights = hip.route_topk(np.ascontiguousarray(logits[:, :experts]), k)
    want = np.zeros((tokens, hidden), np.float64)
    for t in range(tokens):
        want[t] = shared[t] * oracle.shared_expert_scale(logits[t, experts])
        for slot in range(k):
            e = int(ids[t, slot])
            gu = model.apply(hip_model.EXPERT_IN, 0, x[t:t + 1], e)
            act = oracle.swiglu(gu)
            want[t] += np.float64(weights[t, slot]) * model.apply(hip_model.EXPERT_DOWN, 0, act, e)[0]
    assert oracle.rel_l2(got, want) <= 1e-5
