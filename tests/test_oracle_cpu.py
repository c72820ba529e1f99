"""Pins the CPU checker (oracle/) before anything is compared with it: the
reference's own fixtures and known answers, the compiled reference where it was
built, closed forms and brute force.  No GPU."""
import math

import numpy as np
import pytest

from conftest import GOLDEN
from gufo_npu_amd import synth

TYPES = [synth.Q4_K, synth.Q5_K, synth.Q6_K]
NAMES = synth.TYPE_NAMES


# ---- fp16 ---------------------------------------------------------------------

def test_half_known_answers(oracle):
    # The table of the reference's tests/core/quant_test.cpp:56-61.
    table = {0x0000: 0.0, 0x3C00: 1.0, 0xC000: -2.0, 0x3555: 0.333251953125,
             0x0001: 5.96046448e-08, 0x7BFF: 65504.0}
    for bits, value in table.items():
        assert oracle.half_to_float(bits) == np.float32(value)


def test_half_exhaustive_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([oracle.half_to_float(int(b)) for b in bits], dtype=np.float32).view(np.uint32)
    nan = np.isnan(bits.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got.view(np.float32)[nan]))


# ---- block geometry and dequantization -----------------------------------------

def test_block_geometry(oracle):
    lib = oracle.lib()
    assert [lib.gufo_oracle_block_bytes(t) for t in TYPES] == [144, 176, 210]
    assert lib.gufo_oracle_block_bytes(2) == 0
    assert lib.gufo_oracle_row_bytes(synth.Q6_K, 2048) == 1680
    assert lib.gufo_oracle_row_bytes(synth.Q4_K, 2000) == 0  # partial block


@pytest.mark.parametrize("ggml_type", TYPES)
def test_dequantize_matches_gguf_py_fixture_bit_for_bit(oracle, ggml_type):
    raw = np.fromfile(GOLDEN / "quant" / f"{NAMES[ggml_type]}.bin", dtype=np.uint8)
    want = np.fromfile(GOLDEN / "quant" / f"{NAMES[ggml_type]}.f32", dtype=np.float32)
    assert raw.size == synth.row_bytes(ggml_type, want.size)
    got = oracle.dequantize(ggml_type, raw, want.size)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_rejects_partial_block(oracle):
    with pytest.raises(ValueError):
        oracle.dequantize(synth.Q4_K, np.zeros(144, np.uint8), 255)
    with pytest.raises(ValueError):
        oracle.dequantize(2, np.zeros(144, np.uint8), 256)


@pytest.mark.parametrize("ggml_type", TYPES)
def test_dequantize_matches_compiled_reference(ref_oracle, ggml_type):
    # Random bytes everywhere, the fp16 fields included (subnormals, either sign);
    # inf/nan scales are kept out as the models never store them.
    gen = synth.rng(11 + ggml_type)
    blocks = gen.integers(0, 256, size=(400, synth.BLOCK_BYTES[ggml_type]), dtype=np.uint8)
    for off in ((0, 2) if ggml_type != synth.Q6_K else (208,)):
        blocks[:, off + 1] &= 0x7B | 0x80  # exponent < 31
    n = 400 * 256
    got = ref_oracle.dequantize(ggml_type, blocks, n)
    want = ref_oracle.dequantize(ggml_type, blocks, n, use_ref=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_scale_min_round_trip(oracle):
    # Every 6-bit value in every one of the 8 positions survives pack -> unpack.
    gen = synth.rng(5)
    for _ in range(200):
        scales = gen.integers(0, 64, 8)
        mins = gen.integers(0, 64, 8)
        packed = synth.pack_scales_k4(scales, mins)
        for j in range(8):
            assert oracle.scale_min_k4(j, packed) == (scales[j], mins[j])
    for value in range(64):
        for j in range(8):
            scales = np.zeros(8, int)
            mins = np.zeros(8, int)
            scales[j] = value
            mins[j] = 63 - value
            packed = synth.pack_scales_k4(scales, mins)
            assert oracle.scale_min_k4(j, packed) == (value, 63 - value)


# ---- fused dots -----------------------------------------------------------------

def reference_style_row(ggml_type, n, gen):
    """Random codes, scales and mins; fp16 scales normal, either sign, magnitude
    2^-10..2^-1 (the rows of the reference's gguf_dot_test.cpp:25-72)."""
    block = synth.BLOCK_BYTES[ggml_type]
    row = gen.integers(0, 256, size=(n // 256, block), dtype=np.uint8)
    offsets = (208,) if ggml_type == synth.Q6_K else (0, 2)
    for off in offsets:
        sign = gen.integers(0, 2, n // 256).astype(np.uint16) << 15
        exponent = (5 + gen.integers(0, 10, n // 256)).astype(np.uint16) << 10
        mantissa = gen.integers(0, 1024, n // 256).astype(np.uint16)
        half = (sign | exponent | mantissa).astype(np.uint16)
        row[:, off:off + 2] = half.view(np.uint8).reshape(-1, 2)
    return row.reshape(-1)


@pytest.mark.parametrize("ggml_type", TYPES)
@pytest.mark.parametrize("n", [256, 512, 2048])
def test_fused_dot_against_dequantize_and_double_sum(oracle, ggml_type, n):
    # The closed form and limit of the reference's gguf_dot_test.cpp:98-116.
    gen = synth.rng(20261105 + ggml_type * 10 + n)
    worst = 0.0
    for _ in range(200):
        row = reference_style_row(ggml_type, n, gen)
        x = gen.standard_normal(n, dtype=np.float32)
        w = oracle.dequantize(ggml_type, row, n).astype(np.float64)
        want = float(np.dot(w, x.astype(np.float64)))
        magnitude = float(np.sum(np.abs(w * x)))
        got = oracle.dot(ggml_type, row, x)
        worst = max(worst, abs(got - want) / magnitude)
        assert abs(oracle.dot_double(ggml_type, row, x) - want) <= 1e-12 * magnitude
    assert worst < 2e-5, worst


@pytest.mark.parametrize("ggml_type", TYPES)
def test_fused_dot_against_compiled_reference(ref_oracle, ggml_type):
    # The reference's AVX2 bodies sum in another order: agreement to fp32 rounding.
    gen = synth.rng(77 + ggml_type)
    for n in (256, 512, 2048, 6144):
        for _ in range(50):
            row = reference_style_row(ggml_type, n, gen)
            x = gen.standard_normal(n, dtype=np.float32)
            w = ref_oracle.dequantize(ggml_type, row, n).astype(np.float64)
            magnitude = float(np.sum(np.abs(w * x)))
            got = ref_oracle.dot(ggml_type, row, x)
            want = ref_oracle.dot(ggml_type, row, x, use_ref=True)
            assert abs(got - want) < 2e-5 * magnitude


def q8_0_row(n, gen):
    """Q8_0 blocks as the reference's gguf_dot_test.cpp:25-72 builds them: random int8,
    fp16 scale normal, either sign, magnitude 2^-10..2^-1."""
    blocks = n // 32
    row = gen.integers(0, 256, size=(blocks, 34), dtype=np.uint8)
    sign = gen.integers(0, 2, blocks).astype(np.uint16) << 15
    exponent = (5 + gen.integers(0, 10, blocks)).astype(np.uint16) << 10
    half = (sign | exponent | gen.integers(0, 1024, blocks).astype(np.uint16)).astype(np.uint16)
    row[:, 0:2] = half.view(np.uint8).reshape(-1, 2)
    return row.reshape(-1)


def test_q8_0_and_f32_geometry(oracle):
    lib = oracle.lib()
    assert lib.gufo_oracle_block_bytes(synth.Q8_0) == 34
    assert lib.gufo_oracle_block_bytes(synth.F32) == 4
    assert lib.gufo_oracle_row_bytes(synth.Q8_0, 2048) == 2176
    assert lib.gufo_oracle_row_bytes(synth.Q8_0, 2040) == 0   # partial block
    assert lib.gufo_oracle_row_bytes(synth.F32, 7) == 28
    assert lib.gufo_oracle_block_bytes(1) == 0                 # F16 is not on this path


def test_q8_0_dequantize_matches_gguf_py_fixture_bit_for_bit(oracle):
    raw = np.fromfile(GOLDEN / "quant" / "Q8_0.bin", dtype=np.uint8)
    want = np.fromfile(GOLDEN / "quant" / "Q8_0.f32", dtype=np.float32)
    assert raw.size == want.size // 32 * 34
    got = oracle.dequantize(synth.Q8_0, raw, want.size)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q8_0_integer_special_case(oracle):
    # d = 1: the row is the int8 codes themselves and the dot an integer dot product.
    gen = synth.rng(5)
    row = gen.integers(0, 256, size=(8, 34), dtype=np.uint8)
    row[:, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    codes = row[:, 2:].reshape(-1).view(np.int8).astype(np.int64)
    x = gen.integers(-8, 9, 256).astype(np.float32)
    assert np.array_equal(oracle.dequantize(synth.Q8_0, row, 256), codes.astype(np.float32))
    assert oracle.dot(synth.Q8_0, row, x) == float(np.dot(codes, x.astype(np.int64)))


@pytest.mark.parametrize("n", [32, 256, 2048])
def test_q8_0_and_f32_dots_against_double_sum(oracle, n):
    gen = synth.rng(300 + n)
    worst = 0.0
    for _ in range(200):
        row = q8_0_row(n, gen)
        x = gen.standard_normal(n, dtype=np.float32)
        w = oracle.dequantize(synth.Q8_0, row, n).astype(np.float64)
        want, magnitude = float(np.dot(w, x.astype(np.float64))), float(np.sum(np.abs(w * x)))
        worst = max(worst, abs(oracle.dot(synth.Q8_0, row, x) - want) / magnitude)
        assert abs(oracle.dot_double(synth.Q8_0, row, x) - want) <= 1e-12 * magnitude
        wf = gen.standard_normal(n + 3, dtype=np.float32)   # a tail after the 8-wide part
        xf = gen.standard_normal(n + 3, dtype=np.float32)
        want = float(np.dot(wf.astype(np.float64), xf.astype(np.float64)))
        magnitude = float(np.sum(np.abs(wf.astype(np.float64) * xf)))
        worst = max(worst, abs(oracle.dot(synth.F32, wf.view(np.uint8), xf) - want) / magnitude)
        assert np.array_equal(oracle.dequantize(synth.F32, wf.view(np.uint8), n + 3), wf)
    assert worst < 2e-5, worst


def test_q8_0_and_f32_against_compiled_reference(ref_oracle):
    gen = synth.rng(401)
    for n in (256, 2048, 6144):
        for _ in range(50):
            row = q8_0_row(n, gen)
            x = gen.standard_normal(n, dtype=np.float32)
            got = ref_oracle.dequantize(synth.Q8_0, row, n)
            assert np.array_equal(got, ref_oracle.dequantize(synth.Q8_0, row, n, use_ref=True))
            magnitude = float(np.sum(np.abs(got.astype(np.float64) * x)))
            assert abs(ref_oracle.dot(synth.Q8_0, row, x) -
                       ref_oracle.dot(synth.Q8_0, row, x, use_ref=True)) < 2e-5 * magnitude
            w = gen.standard_normal(n, dtype=np.float32)
            magnitude = float(np.sum(np.abs(w.astype(np.float64) * x)))
            assert abs(ref_oracle.dot(synth.F32, w.view(np.uint8), x) -
                       ref_oracle.dot(synth.F32, w.view(np.uint8), x, use_ref=True)) \
                < 2e-5 * magnitude
    # the row loop over mixed parts, against the reference's pool
    cols = 512
    a, b = synth.q8_0_matrix(40, cols, 1), synth.f32_matrix(9, cols, 2)
    x = synth.activations(3, cols, 3)
    parts = [(synth.Q8_0, a, 3, 30), (synth.F32, b, 0, 9)]
    got = ref_oracle.matmul(parts, x, threads=3)
    want = ref_oracle.matmul(parts, x, threads=3, use_ref=True)
    assert ref_oracle.rel_l2(got, want) < 1e-6


def test_q4_k_integer_special_case(oracle):
    # d = 1, dmin = 0, every scale 1: the weights are the 4-bit codes, and with small
    # integer x the dot product is an integer that fp32 holds exactly.
    gen = synth.rng(3)
    n = 512
    codes = gen.integers(0, 16, n)
    x = gen.integers(-8, 9, n).astype(np.float32)
    row = np.zeros((n // 256, 144), np.uint8)
    one = np.array([1.0], np.float16).view(np.uint8)
    for b in range(n // 256):
        row[b, 0:2] = one
        row[b, 4:16] = synth.pack_scales_k4([1] * 8, [0] * 8)
        c = codes[256 * b:256 * (b + 1)].reshape(4, 2, 32)  # run, nibble, byte
        row[b, 16:144] = (c[:, 0, :] | (c[:, 1, :] << 4)).reshape(-1)
    assert oracle.dot(synth.Q4_K, row, x) == float(np.dot(codes, x))


def test_q6_k_integer_special_case(oracle):
    # d = 1, every scale 1: weights are code - 32.
    gen = synth.rng(4)
    codes = gen.integers(0, 64, 256)
    x = gen.integers(-4, 5, 256).astype(np.float32)
    row = np.zeros(210, np.uint8)
    for half in range(2):
        c = codes[128 * half:128 * half + 128].reshape(4, 32)  # k, l
        ql = row[64 * half:64 * half + 64]
        ql[0:32] = (c[0] & 15) | ((c[2] & 15) << 4)
        ql[32:64] = (c[1] & 15) | ((c[3] & 15) << 4)
        row[128 + 32 * half:128 + 32 * half + 32] = (
            (c[0] >> 4) | ((c[1] >> 4) << 2) | ((c[2] >> 4) << 4) | ((c[3] >> 4) << 6))
    row[192:208] = 1
    row[208:210] = np.array([1.0], np.float16).view(np.uint8)
    assert oracle.dot(synth.Q6_K, row, x) == float(np.dot(codes - 32, x))
    w = oracle.dequantize(synth.Q6_K, row, 256)
    assert np.array_equal(w, (codes - 32).astype(np.float32))


def test_q5_k_fifth_bit_special_case(oracle):
    # Only the high bits set: every weight is 16 * (bit j of qh[l]).
    gen = synth.rng(6)
    bits = gen.integers(0, 2, (8, 32))  # sub-block j, value l
    row = np.zeros(176, np.uint8)
    row[0:2] = np.array([1.0], np.float16).view(np.uint8)
    row[4:16] = synth.pack_scales_k4([1] * 8, [0] * 8)
    qh = np.zeros(32, np.uint8)
    for j in range(8):
        qh |= (bits[j].astype(np.uint8) << j)
    row[16:48] = qh
    w = oracle.dequantize(synth.Q5_K, row, 256)
    assert np.array_equal(w, (16 * bits).reshape(-1).astype(np.float32))


# ---- MatMul ------------------------------------------------------------------------

def test_matmul_layout_parts_tokens_threads(oracle):
    # Each output is one dot product at y[t*stride + offset + r]
    # (gguf_projections.cpp:239-286): check against single dots, any thread count.
    cols = 512
    a = synth.kquant_matrix(synth.Q4_K, 40, cols, 1)
    b = synth.kquant_matrix(synth.Q4_K, 24, cols, 2)
    c = synth.kquant_matrix(synth.Q6_K, 33, cols, 3)
    x = synth.activations(3, cols, 4)
    parts = [(synth.Q4_K, a, 3, 30), (synth.Q4_K, b, 0, 24), (synth.Q6_K, c, 16, 17)]
    y = oracle.matmul(parts, x)
    assert y.shape == (3, 71)
    for t in range(3):
        assert y[t, 0] == np.float32(oracle.dot(synth.Q4_K, a[3], x[t]))
        assert y[t, 29] == np.float32(oracle.dot(synth.Q4_K, a[32], x[t]))
        assert y[t, 30] == np.float32(oracle.dot(synth.Q4_K, b[0], x[t]))
        assert y[t, 54] == np.float32(oracle.dot(synth.Q6_K, c[16], x[t]))
        assert y[t, 70] == np.float32(oracle.dot(synth.Q6_K, c[32], x[t]))
    assert np.array_equal(y, oracle.matmul(parts, x, threads=4))
    # "results do not depend on ... how many tokens come together"
    assert np.array_equal(y[1:2], oracle.matmul(parts, x[1:2]))
    exact = oracle.matmul(parts, x, precision="double")
    assert exact[2, 70] == np.float32(oracle.dot_double(synth.Q6_K, c[32], x[2]))
    assert oracle.rel_l2(y, exact) < 1e-6


@pytest.mark.parametrize("ggml_type", TYPES)
def test_matmul_against_compiled_reference(ref_oracle, ggml_type):
    cols, rows = 2048, 150
    w = synth.kquant_matrix(ggml_type, rows, cols, 30 + ggml_type)
    x = synth.activations(4, cols, 40)
    parts = [(ggml_type, w, 10, 100), (ggml_type, w, 0, 37)]
    got = ref_oracle.matmul(parts, x, threads=2)
    want = ref_oracle.matmul(parts, x, threads=3, use_ref=True)
    assert got.shape == want.shape == (4, 137)
    assert ref_oracle.rel_l2(got, want) < 1e-6
    exact = ref_oracle.matmul(parts, x, precision="double")
    assert ref_oracle.rel_l2(want, exact) < 1e-6


# ---- routing -----------------------------------------------------------------------

def brute_route(logits, k):
    """Softmax in double, stable sort by (-p, index), renormalise with the floor."""
    p = [math.exp(float(v) - float(max(logits))) for v in logits]
    total = 0.0
    for v in p:
        total += v
    order = sorted(range(len(p)), key=lambda e: (-p[e], e))[:k]
    top = 0.0
    for e in order:
        top += p[e] / total
    top = max(top, 6.103515625e-5)
    return order, [np.float32(p[e] / total / top) for e in order]


def test_route_brute_force_and_ties(oracle):
    gen = synth.rng(9)
    cases = [gen.standard_normal(e).astype(np.float32) for e in (8, 16, 64, 256) for _ in range(20)]
    tie = np.zeros(16, np.float32)          # all equal: lowest indices win, in order
    cases.append(tie)
    tie2 = np.array([1, 3, 3, 2, 3, 0, 2, 2], np.float32)  # ties inside and at the cut
    cases.append(tie2)
    far = np.array([0, -800, -900, -1000, 5], np.float32)  # underflow to p = 0: index order
    cases.append(far)
    for logits in cases:
        for k in (1, 2, min(8, logits.size)):
            ids, weights = oracle.route(logits[None, :], k)
            want_ids, want_w = brute_route(logits, k)
            assert list(ids[0]) == want_ids
            assert np.array_equal(weights[0], np.array(want_w, np.float32))
    ids, _ = oracle.route(tie[None, :], 4)
    assert list(ids[0]) == [0, 1, 2, 3]
    ids, _ = oracle.route(tie2[None, :], 5)
    assert list(ids[0]) == [1, 2, 4, 3, 6]
    ids, _ = oracle.route(far[None, :], 4)
    assert list(ids[0]) == [4, 0, 1, 2]


def test_route_weight_floor(oracle):
    # 20,000 equal logits, k = 1: p/total = 5e-5 is below the floor 2^-14.
    logits = np.zeros((1, 20000), np.float32)
    ids, weights = oracle.route(logits, 1)
    assert ids[0, 0] == 0
    assert weights[0, 0] == np.float32((1.0 / 20000) / 6.103515625e-5)


def test_route_against_compiled_reference(ref_oracle):
    logits = synth.router_logits(64, 256, 21)
    logits[3, 10:20] = logits[3, 5]          # engineered ties
    logits[4, :] = 0.25
    logits[5, 100:] = -1000.0
    ids, weights = ref_oracle.route(logits, 8)
    want_ids, want_w = ref_oracle.route(logits, 8, use_ref=True)
    assert np.array_equal(ids, want_ids)
    assert np.array_equal(weights.view(np.uint32), want_w.view(np.uint32))
    zeros = np.zeros((1, 20000), np.float32)
    assert np.array_equal(ref_oracle.route(zeros, 1)[1], ref_oracle.route(zeros, 1, use_ref=True)[1])


def test_argmax_first_maximum(oracle):
    v = np.array([1, 5, 3, 5, 5, -2], np.float32)
    assert oracle.argmax(v) == 1
    assert oracle.argmax(np.full(7, -3.0, np.float32)) == 0
    gen = synth.rng(2)
    w = gen.standard_normal(10000).astype(np.float32)
    assert oracle.argmax(w) == int(np.argmax(w))


# ---- expert grouping and the routed FFN ----------------------------------------------

def test_moe_group_tables(oracle):
    ids = np.array([[3, 1, 7], [1, 3, 0], [7, 7, 2]], np.int32)  # tokens x k
    counts, offsets, pairs, distinct = oracle.moe_group(ids, 8)
    assert list(counts) == [1, 2, 1, 2, 0, 0, 0, 3]
    assert list(offsets) == [0, 1, 3, 4, 6, 6, 6, 6, 9]
    assert list(pairs) == [5, 1, 3, 8, 0, 4, 2, 6, 7]
    assert distinct == 5


def test_moe_ffn_equals_per_token_result(oracle):
    experts, hidden, ffn, k, tokens = 16, 512, 256, 4, 5
    gate = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 50)
    up = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 51)
    down = synth.kquant_matrix(synth.Q5_K, experts * hidden, ffn, 52)
    logits = synth.router_logits(tokens, experts, 53)
    x = synth.activations(tokens, hidden, 54) * np.float32(0.05)
    ids, weights, y = oracle.moe_ffn(gate, synth.Q4_K, up, synth.Q4_K, down, synth.Q5_K,
                                     experts, hidden, ffn, logits, x, k)
    want_ids, want_w = oracle.route(logits, k)
    assert np.array_equal(ids, want_ids) and np.array_equal(weights, want_w)
    silu = np.vectorize(lambda v: oracle.silu(float(v)), otypes=[np.float32])
    for t in range(tokens):
        acc = np.zeros(hidden, np.float64)
        for slot in range(k):
            e = int(ids[t, slot])
            gu = oracle.matmul([(synth.Q4_K, gate, e * ffn, ffn), (synth.Q4_K, up, e * ffn, ffn)],
                               x[t:t + 1])[0]
            act = (silu(gu[:ffn]) * gu[ffn:]).astype(np.float32)
            out = oracle.matmul([(synth.Q5_K, down, e * hidden, hidden)], act[None, :])[0]
            acc += np.float64(weights[t, slot]) * out.astype(np.float64)
        assert np.array_equal(y[t], acc.astype(np.float32))


def test_shared_expert_scale_is_the_sigmoid(oracle):
    # Closed forms: 1/2 at 0, s(v) + s(-v) = 1, saturation, and the textbook value at 1.
    assert oracle.shared_expert_scale(0.0) == np.float32(0.5)
    assert oracle.shared_expert_scale(1.0) == np.float32(1.0 / (1.0 + math.exp(-1.0)))
    assert oracle.shared_expert_scale(200.0) == np.float32(1.0)
    assert oracle.shared_expert_scale(-200.0) == np.float32(0.0)
    for v in synth.router_logits(1, 64, 77)[0] * np.float32(4.0):
        total = np.float64(oracle.shared_expert_scale(v)) + np.float64(oracle.shared_expert_scale(-v))
        assert abs(total - 1.0) <= 2.0 ** -24


def test_shared_expert_scale_equals_the_compiled_reference(ref_oracle):
    for v in np.concatenate([synth.router_logits(1, 256, 78)[0] * np.float32(6.0),
                             np.array([0.0, -0.0, 88.0, -88.0, 1e-30], np.float32)]):
        assert ref_oracle.shared_expert_scale(v) == ref_oracle.shared_expert_scale(v, use_ref=True)


def test_moe_layer_is_router_plus_routed_experts_plus_scaled_shared_expert(oracle):
    experts, hidden, ffn, k, tokens = 8, 256, 256, 2, 3
    router = synth.f32_matrix(experts + 1, hidden, 60)
    gate = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 61)
    up = synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, 62)
    down = synth.kquant_matrix(synth.Q6_K, experts * hidden, ffn, 63)
    x = synth.activations(tokens, hidden, 64) * np.float32(0.05)
    shared = synth.activations(tokens, hidden, 65)
    ids, weights, y = oracle.moe_layer(synth.F32, router, gate, synth.Q4_K, up, synth.Q4_K, down,
                                       synth.Q6_K, experts, hidden, ffn, x, k, shared=shared)
    w = router.view(np.float32).reshape(experts + 1, hidden).astype(np.float64)
    logits = (x.astype(np.float64) @ w.T).astype(np.float32)
    want_ids, want_w = oracle.route(np.ascontiguousarray(logits[:, :experts]), k)
    assert np.array_equal(ids, want_ids) and np.allclose(weights, want_w, rtol=1e-6)
    _, _, routed = oracle.moe_ffn(gate, synth.Q4_K, up, synth.Q4_K, down, synth.Q6_K, experts,
                                  hidden, ffn, np.ascontiguousarray(logits[:, :experts]), x, k,
                                  precision="double")
    _, _, without = oracle.moe_layer(synth.F32, router, gate, synth.Q4_K, up, synth.Q4_K, down,
                                     synth.Q6_K, experts, hidden, ffn, x, k)
    assert oracle.rel_l2(without, routed) <= 1e-7
    for t in range(tokens):
        scale = 1.0 / (1.0 + math.exp(-float(logits[t, experts])))
        assert oracle.rel_l2(y[t], routed[t].astype(np.float64) + scale * shared[t]) <= 1e-6
