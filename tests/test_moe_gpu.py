"""Parity of the MoE path (routing, device-side grouping, expert products, combine)
with the CPU checker and the golden reference outputs, through the C-ABI.

Bars: routing indices bit-exact; grouping tables exact; weights and outputs to
rel-L2 <= 1e-4; the grouped batch equals the per-token result; repeats bit-identical."""
import numpy as np
import pytest

from conftest import GOLDEN
from gufo_npu_amd import configs as cfg
from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-4


def say(*args):
    print(*args, flush=True)


def same(a, b) -> bool:
    """Exact equality as a bool, so a failure prints no arrays."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.dtype == np.float32:
        a, b = a.view(np.uint32), b.view(np.uint32)
    return bool(np.array_equal(a, b))


def close(a, b, rtol=1e-6) -> bool:
    return bool(np.allclose(a, b, rtol=rtol, atol=0))


def engineered_logits():
    # The rows tests/golden/make_golden.py routes through the reference.
    logits = synth.router_logits(64, cfg.EXPERTS4, cfg.SEED + 180)
    logits[1, :] = 0.0
    logits[2, 40:60] = logits[2, 7]
    logits[3, ::2] = 1.5
    logits[4, 8:] = -900.0
    logits[5, 200] = logits[5, 3] = logits[5].max() + 1.0
    logits[6, :] = np.float32(1e-9) * np.arange(cfg.EXPERTS4, dtype=np.float32)
    return logits


def test_route_indices_bit_exact_against_reference_golden(hip, oracle):
    say("route golden")
    golden = np.load(GOLDEN / "config4_moe.npz")
    logits = engineered_logits()
    ids, weights = hip.route_topk(logits, cfg.TOPK4)
    assert same(ids, golden["route_ids"])
    assert close(weights, golden["route_weights"])
    want_ids, want_w = oracle.route(logits, cfg.TOPK4)
    assert same(ids, want_ids)
    assert close(weights, want_w)


@pytest.mark.parametrize("experts,k", [(8, 1), (8, 8), (60, 6), (64, 8), (256, 8), (1000, 17)])
def test_route_shapes_and_ties(hip, oracle, experts, k):
    say("route", experts, k)
    logits = synth.router_logits(37, experts, 500 + experts)
    logits[0, :] = -2.0                              # all tied: ids 0..k-1
    logits[1, experts // 2:] = logits[1, 0]           # long run of ties
    logits[2] = np.round(logits[2] * 2) / 2           # many duplicate values
    ids, weights = hip.route_topk(logits, k)
    want_ids, want_w = oracle.route(logits, k)
    assert same(ids, want_ids)
    assert list(ids[0]) == list(range(k))
    assert close(weights, want_w)
    assert np.allclose(weights.sum(axis=1), 1.0, atol=1e-5)


def test_group_tables_exact(hip, oracle):
    say("group")
    gen = synth.rng(31)
    for tokens, k, experts in ((1, 8, 256), (4, 8, 256), (5, 4, 16), (64, 8, 256), (7, 3, 5)):
        ids = np.stack([gen.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
        counts, offsets, pairs, distinct = hip.moe_group(ids, experts)
        w_counts, w_offsets, w_pairs, w_distinct = oracle.moe_group(ids, experts)
        assert same(counts, w_counts)
        assert same(offsets, w_offsets)
        assert same(pairs, w_pairs)
        assert distinct == w_distinct
    golden = np.load(GOLDEN / "config4_moe.npz")
    for b in (1, 4):
        counts, offsets, pairs, distinct = hip.moe_group(golden[f"ids_b{b}"], cfg.EXPERTS4)
        assert same(counts, golden[f"counts_b{b}"])
        assert same(offsets, golden[f"offsets_b{b}"])
        assert same(pairs, golden[f"pairs_b{b}"])
        assert distinct == int(golden[f"distinct_b{b}"])


def test_group_rejects_unknown_expert(hip):
    say("group bad id")
    ids = np.array([[0, 1, 99]], np.int32)
    with pytest.raises(hip.LogicError):
        hip.moe_group(ids, 16)


def test_moe_ffn_small_with_crowded_experts(hip, oracle):
    # 16 experts and 9 tokens x 4 slots: some experts serve more than four tokens, so
    # their token lists split into several segments.
    say("moe small")
    experts, hidden, ffn, k, tokens = 16, 512, 256, 4, 9
    gate = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 50)
    up = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 51)
    down = synth.kquant_matrix(synth.Q5_K, experts * hidden, ffn, 52)
    logits = synth.router_logits(tokens, experts, 53)
    logits[:, 3] += 4.0  # expert 3 is chosen by every token
    x = synth.activations(tokens, hidden, 54) * np.float32(0.05)
    mg = hip.Matrix(synth.Q4_K, gate, experts * ffn, hidden)
    mu = hip.Matrix(synth.Q4_K, up, experts * ffn, hidden)
    md = hip.Matrix(synth.Q5_K, down, experts * hidden, ffn)
    ids, weights = hip.route_topk(logits, k)
    want_ids, want_w, want_y = oracle.moe_ffn(gate, synth.Q4_K, up, synth.Q4_K, down,
                                              synth.Q5_K, experts, hidden, ffn, logits, x, k,
                                              precision="double")
    assert same(ids, want_ids)
    assert int(np.max(np.bincount(ids.reshape(-1), minlength=experts))) > 4
    y = hip.moe_ffn(mg, mu, md, experts, x, ids, weights)
    assert oracle.rel_l2(y, want_y) <= TOLERANCE
    # grouped batch == per-token calls, bit for bit; repeats too
    for t in range(tokens):
        single = hip.moe_ffn(mg, mu, md, experts, x[t:t + 1], ids[t:t + 1], weights[t:t + 1])
        assert same(single[0], y[t])
    assert same(y, hip.moe_ffn(mg, mu, md, experts, x, ids, weights))
    # a caller may name an expert twice in one token: both slots count, in slot order
    twice = ids.copy()
    twice[:, 1] = twice[:, 0]
    y_twice = hip.moe_ffn(mg, mu, md, experts, x, twice, weights)
    total = np.zeros(y_twice.shape, np.float64)
    for slots in ((0,), (1,), (2, 3)):  # the output is linear in the slot weights
        part = np.zeros_like(weights)
        part[:, slots] = weights[:, slots]
        total += hip.moe_ffn(mg, mu, md, experts, x, twice, part)
    assert oracle.rel_l2(y_twice, total) <= 1e-6
    for t in (0, tokens - 1):
        single = hip.moe_ffn(mg, mu, md, experts, x[t:t + 1], twice[t:t + 1], weights[t:t + 1])
        assert same(single[0], y_twice[t])
    with pytest.raises(hip.LogicError):
        bad = ids.copy()
        bad[0, 0] = experts
        hip.moe_ffn(mg, mu, md, experts, x, bad, weights)
    with pytest.raises(hip.ShapeError):
        hip.moe_ffn(mg, mu, mg, experts, x, ids, weights)
    for m in (mg, mu, md):
        m.destroy()


def test_config4_moe_expert_gemv(hip, oracle):
    # Config 4: 256 experts, hidden 2048, expert FFN 512, top-8; batch 1 and a ragged
    # batch of 4 tokens grouped by expert on the device.
    gate, up, down = (cfg.CONFIG4[n] for n in ("gate", "up", "down"))
    wg, wu, wd = gate.build(), up.build(), down.build()
    mg = hip.Matrix(gate.ggml_type, wg, gate.rows, gate.cols)
    mu = hip.Matrix(up.ggml_type, wu, up.rows, up.cols)
    md = hip.Matrix(down.ggml_type, wd, down.rows, down.cols)
    golden = np.load(GOLDEN / "config4_moe.npz")
    for tokens in (1, 4):
        say("config 4 batch", tokens)
        logits = synth.router_logits(tokens, cfg.EXPERTS4, cfg.CONFIG4_LOGIT_SEED + tokens)
        x = synth.activations(tokens, cfg.HIDDEN4, cfg.CONFIG4_X_SEED + tokens)
        x = x * np.float32(cfg.CONFIG4_X_SCALE)
        ids, weights = hip.route_topk(logits, cfg.TOPK4)
        assert same(ids, golden[f"ids_b{tokens}"])
        assert close(weights, golden[f"weights_b{tokens}"])
        y = hip.moe_ffn(mg, mu, md, cfg.EXPERTS4, x, ids, weights)
        assert oracle.rel_l2(y, golden[f"y_b{tokens}"]) <= TOLERANCE
        _, _, want = oracle.moe_ffn(wg, gate.ggml_type, wu, up.ggml_type, wd, down.ggml_type,
                                    cfg.EXPERTS4, cfg.HIDDEN4, cfg.FFN4, logits, x, cfg.TOPK4,
                                    precision="double", threads=8)
        assert oracle.rel_l2(y, want) <= TOLERANCE
        for t in range(tokens):
            single = hip.moe_ffn(mg, mu, md, cfg.EXPERTS4, x[t:t + 1], ids[t:t + 1],
                                 weights[t:t + 1])
            assert same(single[0], y[t])
    for m in (mg, mu, md):
        m.destroy()


@pytest.mark.parametrize("router_type", [synth.F32, synth.Q8_0])
@pytest.mark.parametrize("tokens", [1, 4, 9])
def test_moe_layer_in_one_call(hip, oracle, router_type, tokens):
    # Decoder::MoeFfn whole: router product, routing, routed experts, and the shared
    # expert's output scaled by the sigmoid of the router's extra logit.
    say("moe layer", synth.TYPE_NAMES[router_type], tokens)
    experts, hidden, ffn, k = 16, 512, 256, 4
    router = synth.matrix(router_type, experts + 1, hidden, 70)
    gate = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 71)
    up = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 72)
    down = synth.kquant_matrix(synth.Q5_K, experts * hidden, ffn, 73)
    x = synth.activations(tokens, hidden, 74 + tokens) * np.float32(0.05)
    # (the routed outputs are of the order 1e4 with these weights)
    shared = synth.activations(tokens, hidden, 75 + tokens) * np.float32(3000.0)
    mr = hip.Matrix(router_type, router, experts + 1, hidden)
    mg = hip.Matrix(synth.Q4_K, gate, experts * ffn, hidden)
    mu = hip.Matrix(synth.Q4_K, up, experts * ffn, hidden)
    md = hip.Matrix(synth.Q5_K, down, experts * hidden, ffn)
    dx = hip.DeviceBuffer.from_array(x)
    ds = hip.DeviceBuffer.from_array(shared)
    dy = hip.DeviceBuffer(4 * tokens * hidden)

    want_ids, want_w, want = oracle.moe_layer(router_type, router, gate, synth.Q4_K, up,
                                              synth.Q4_K, down, synth.Q5_K, experts, hidden, ffn,
                                              x, k, shared=shared, threads=4)
    hip.moe_layer_dev(mr, mg, mu, md, experts, k, dx, tokens, ds, dy)
    hip.synchronize()
    got = dy.download((tokens, hidden), np.float32)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    # the shared term is really there: a visible part of the output by construction
    _, _, routed_only = oracle.moe_layer(router_type, router, gate, synth.Q4_K, up, synth.Q4_K,
                                         down, synth.Q5_K, experts, hidden, ffn, x, k, threads=4)
    assert oracle.rel_l2(routed_only, want) > 0.02

    # The same from the separate entry points, bit for bit: router product, routing, the
    # expert call; then the scaled shared rows added in double.
    logits = hip.gemv([hip.whole(mr)], x, tokens)
    ids, weights = hip.route_topk(np.ascontiguousarray(logits[:, :experts]), k)
    assert same(ids, want_ids)
    assert close(weights, want_w, rtol=1e-5)
    routed = hip.moe_ffn(mg, mu, md, experts, x, ids, weights)
    hip.moe_layer_dev(mr, mg, mu, md, experts, k, dx, tokens, None, dy)
    hip.synchronize()
    assert same(dy.download((tokens, hidden), np.float32), routed)
    scale = np.array([oracle.shared_expert_scale(v) for v in logits[:, experts]], np.float32)
    composed = (routed.astype(np.float64) + (shared * scale[:, None]).astype(np.float64))
    assert oracle.rel_l2(got, composed) <= 1e-6

    # In place: the output over the shared expert's rows, as the reference's s.out.
    hip.moe_layer_dev(mr, mg, mu, md, experts, k, dx, tokens, ds, ds)
    hip.synchronize()
    assert same(ds.download((tokens, hidden), np.float32), got)

    # A router without the extra row cannot serve a shared expert.
    plain = hip.Matrix(router_type, router[:experts], experts, hidden)
    with pytest.raises(hip.ShapeError):
        hip.moe_layer_dev(plain, mg, mu, md, experts, k, dx, tokens, ds, dy)
    hip.moe_layer_dev(plain, mg, mu, md, experts, k, dx, tokens, None, dy)
    hip.synchronize()
    assert same(dy.download((tokens, hidden), np.float32), routed)
    # The router stage as a model file holds it: the experts' rows and the shared
    # expert's gate row as two tensors.
    gate_row = hip.Matrix(router_type, router[experts:], 1, hidden)
    ds.upload(shared)  # the call in place has overwritten it
    hip.moe_layer_dev([plain, gate_row], mg, mu, md, experts, k, dx, tokens, ds, dy)
    hip.synchronize()
    assert same(dy.download((tokens, hidden), np.float32), got)
    for m in (mr, mg, mu, md, plain, gate_row):
        m.destroy()
