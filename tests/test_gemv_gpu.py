"""Parity of the HIP matrix-vector kernels with the CPU checker, through the C-ABI.

Bars: rel-L2 <= 1e-4 against dequantize + double sum (the reference's oracle
arithmetic, GgufProjections Precision::kDouble); bit-exact dequantization against the
gguf-py fixtures; identical lm_head argmax; column t of an N-column call bit-identical
to the one-column call; repeats bit-identical."""
import numpy as np
import pytest

from conftest import GOLDEN
from gufo_npu_amd import configs as cfg
from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu

TYPES = [synth.Q4_K, synth.Q5_K, synth.Q6_K]     # the formats that have a fixture pair
ROW_TYPES = TYPES + [synth.Q8_0, synth.F32]      # every row type GgufProjections multiplies
NAMES = synth.TYPE_NAMES
TOLERANCE = 1e-4  # rel-L2, fp32 accumulation


def say(*args):
    print(*args, flush=True)


def same_bits(a, b) -> bool:
    """Bit-for-bit equality, reported as a bool so a failure prints no arrays."""
    return bool(np.array_equal(np.ascontiguousarray(a).view(np.uint32),
                               np.ascontiguousarray(b).view(np.uint32)))


@pytest.mark.parametrize("ggml_type", TYPES + [synth.Q8_0])
def test_decode_matches_gguf_py_fixture_bit_for_bit(hip, ggml_type):
    # One row of the fixture's 512 values times the 512 unit vectors returns the
    # dequantized weights themselves: every code, scale and position is checked bit
    # for bit against gguf-py's output, as the reference checks its Dequantize.
    say("fixture", NAMES[ggml_type])
    raw = np.fromfile(GOLDEN / "quant" / f"{NAMES[ggml_type]}.bin", dtype=np.uint8)
    want = np.fromfile(GOLDEN / "quant" / f"{NAMES[ggml_type]}.f32", dtype=np.float32)
    m = hip.Matrix(ggml_type, raw, 1, want.size)
    y = hip.gemv([hip.whole(m)], np.eye(want.size, dtype=np.float32), want.size)
    m.destroy()
    got = np.ascontiguousarray(y[:, 0])
    # A dot product cannot return -0 (it adds to +0), which gguf-py gives for a zero
    # code under a negative scale: zeros are compared by value, the rest bit for bit.
    nonzero = want != 0
    assert int(np.count_nonzero(nonzero)) > 400
    assert same_bits(got[nonzero], want[nonzero])
    assert bool(np.all(got[~nonzero] == 0))


SHAPES = [
    # rows, cols: one block, odd block counts, ragged row counts, the config widths
    (64, 512), (7, 256), (33, 768), (100, 2048), (130, 2560), (61, 6144), (19, 9216),
    (257, 1024), (1, 2048),
]


@pytest.mark.parametrize("ggml_type", ROW_TYPES)
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_gemv_parity(hip, oracle, ggml_type, rows, cols):
    seed = synth.BASE_SEED + ggml_type * 1000 + rows + cols
    w = synth.matrix(ggml_type, rows, cols, seed)
    m = hip.Matrix(ggml_type, w, rows, cols)
    for tokens in (1, 2, 3, 4):
        say("gemv", NAMES[ggml_type], rows, cols, "N", tokens)
        x = synth.activations(tokens, cols, seed + tokens)
        got = hip.gemv([hip.whole(m)], x, tokens)
        exact = oracle.matmul([(ggml_type, w, 0, rows)], x, precision="double", threads=4)
        fused = oracle.matmul([(ggml_type, w, 0, rows)], x, precision="float", threads=4)
        assert got.shape == exact.shape
        assert oracle.rel_l2(got, exact) <= TOLERANCE
        assert oracle.rel_l2(got, fused) <= TOLERANCE
        # column t equals the one-column call, bit for bit
        for t in range(tokens):
            single = hip.gemv([hip.whole(m)], x[t:t + 1], 1)
            assert same_bits(single[0], got[t])
    m.destroy()


def test_gemv_parts_row_ranges_and_mixed_types(hip, oracle):
    # [q | k | v]-style concatenation with first_row offsets and two types in one
    # call: the layout y[t*stride + offset + r] of GgufProjections::MatMul.
    say("gemv parts")
    cols = 2048
    a = synth.kquant_matrix(synth.Q4_K, 300, cols, 1)
    b = synth.kquant_matrix(synth.Q4_K, 64, cols, 2)
    c = synth.kquant_matrix(synth.Q6_K, 90, cols, 3)
    d = synth.kquant_matrix(synth.Q5_K, 50, cols, 4)
    ma, mb = hip.Matrix(synth.Q4_K, a, 300, cols), hip.Matrix(synth.Q4_K, b, 64, cols)
    mc, md = hip.Matrix(synth.Q6_K, c, 90, cols), hip.Matrix(synth.Q5_K, d, 50, cols)
    x = synth.activations(3, cols, 5)
    parts = [(ma, 17, 256), (mb, 0, 64), (mc, 40, 50), (md, 1, 33), (ma, 0, 5)]
    got = hip.gemv(parts, x, 3)
    want = oracle.matmul([(synth.Q4_K, a, 17, 256), (synth.Q4_K, b, 0, 64),
                          (synth.Q6_K, c, 40, 50), (synth.Q5_K, d, 1, 33),
                          (synth.Q4_K, a, 0, 5)], x, precision="double")
    assert got.shape == (3, 408)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    for t in range(3):
        for lo, hi in ((0, 256), (256, 320), (320, 370), (370, 403), (403, 408)):
            assert oracle.rel_l2(got[t, lo:hi], want[t, lo:hi]) <= TOLERANCE
    for m in (ma, mb, mc, md):
        m.destroy()


def test_linear_in_style_stage_with_f32_and_q8_0_parts(hip, oracle):
    # The linear-attention input stage of a real file: [qkv | z | alpha | beta] with the
    # two small projections stored in fp32 and one matrix in Q8_0
    # (Stage::kLinearIn, src/models/qwen35/projections.hpp:15-17 of the reference).
    say("gemv mixed row types")
    cols = 2048
    specs = [(synth.Q5_K, 384), (synth.Q8_0, 256), (synth.F32, 16), (synth.F32, 16),
             (synth.Q4_K, 64)]
    blocks = [synth.matrix(t, rows, cols, 70 + i) for i, (t, rows) in enumerate(specs)]
    mats = [hip.Matrix(t, b, rows, cols) for (t, rows), b in zip(specs, blocks)]
    for tokens in (1, 3):
        x = synth.activations(tokens, cols, 80 + tokens)
        got = hip.gemv([hip.whole(m) for m in mats], x, tokens)
        want = oracle.matmul([(t, b, 0, rows) for (t, rows), b in zip(specs, blocks)], x,
                             precision="double")
        assert got.shape == want.shape == (tokens, 736)
        lo = 0
        for (t, rows) in specs:
            assert oracle.rel_l2(got[:, lo:lo + rows], want[:, lo:lo + rows]) <= TOLERANCE
            lo += rows
    for m in mats:
        m.destroy()


def test_f32_rows_return_themselves_for_unit_activations(hip):
    say("f32 identity")
    rows, cols = 9, 512
    w = synth.f32_matrix(rows, cols, 91)
    m = hip.Matrix(synth.F32, w, rows, cols)
    y = hip.gemv([hip.whole(m)], np.eye(cols, dtype=np.float32), cols)
    m.destroy()
    assert same_bits(np.ascontiguousarray(y.T), w.view(np.float32).reshape(rows, cols))


def test_gemv_many_tokens_and_empty(hip, oracle):
    say("gemv tokens 0 and 11")
    w = synth.kquant_matrix(synth.Q4_K, 48, 512, 8)
    m = hip.Matrix(synth.Q4_K, w, 48, 512)
    x = synth.activations(11, 512, 9)
    got = hip.gemv([hip.whole(m)], x, 11)
    want = oracle.matmul([(synth.Q4_K, w, 0, 48)], x, precision="double")
    assert oracle.rel_l2(got, want) <= TOLERANCE
    assert hip.gemv([hip.whole(m)], x[:0], 0).shape == (0, 48)
    assert hip.gemv([(m, 5, 0)], x[:1], 1).shape == (1, 0)
    m.destroy()


def test_repeats_are_bit_identical(hip):
    say("gemv repeats")
    w = synth.kquant_matrix(synth.Q6_K, 512, 2048, 12)
    m = hip.Matrix(synth.Q6_K, w, 512, 2048)
    x = synth.activations(4, 2048, 13)
    first = hip.gemv([hip.whole(m)], x, 4)
    for _ in range(5):
        assert same_bits(first, hip.gemv([hip.whole(m)], x, 4))
    m.destroy()


def test_config1_single_q4k_gemv(hip, oracle):
    # Config 1: W 6144x2048 Q4_K, x N(0,1), N = 1.
    say("config 1")
    spec = cfg.CONFIG1
    w = spec.build()
    x = synth.activations(1, spec.cols, cfg.CONFIG1_X_SEED)
    m = hip.Matrix(spec.ggml_type, w, spec.rows, spec.cols)
    got = hip.gemv([hip.whole(m)], x, 1)
    want = oracle.matmul([(spec.ggml_type, w, 0, spec.rows)], x, precision="double", threads=4)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    golden = np.load(GOLDEN / "config1_q4k_6144x2048.npz")
    assert oracle.rel_l2(got, golden["y_reference_avx2"]) <= TOLERANCE
    assert oracle.rel_l2(got, golden["y_reference_double"]) <= TOLERANCE
    m.destroy()


def test_config3_mtp_verify_shapes(hip, oracle):
    # Config 3: gate/up 9216x2560 Q4_K and down 2560x9216 Q6_K, N = 2, 3, 4.
    gate, up, down = (cfg.CONFIG3[n] for n in ("gate", "up", "down"))
    wg, wu, wd = gate.build(), up.build(), down.build()
    mg = hip.Matrix(gate.ggml_type, wg, gate.rows, gate.cols)
    mu = hip.Matrix(up.ggml_type, wu, up.rows, up.cols)
    md = hip.Matrix(down.ggml_type, wd, down.rows, down.cols)
    golden = np.load(GOLDEN / "config3_mtp_verify.npz")
    for tokens in (2, 3, 4):
        say("config 3 N", tokens)
        x = synth.activations(tokens, cfg.HIDDEN3, cfg.CONFIG3_X_SEED + tokens)
        a = synth.activations(tokens, cfg.FFN3, cfg.CONFIG3_ACT_SEED + tokens)
        gu = hip.gemv([hip.whole(mg), hip.whole(mu)], x, tokens)
        dn = hip.gemv([hip.whole(md)], a, tokens)
        want_gu = oracle.matmul([(gate.ggml_type, wg, 0, gate.rows),
                                 (up.ggml_type, wu, 0, up.rows)], x, precision="double",
                                threads=8)
        want_dn = oracle.matmul([(down.ggml_type, wd, 0, down.rows)], a, precision="double",
                                threads=8)
        assert oracle.rel_l2(gu, want_gu) <= TOLERANCE
        assert oracle.rel_l2(dn, want_dn) <= TOLERANCE
        assert oracle.rel_l2(gu[:, ::16], golden[f"gate_up_n{tokens}_every16"]) <= TOLERANCE
        assert oracle.rel_l2(dn, golden[f"down_n{tokens}"]) <= TOLERANCE
        for t in range(tokens):  # the verify pass must equal plain decoding
            single = hip.gemv([hip.whole(md)], a[t:t + 1], 1)
            assert same_bits(single[0], dn[t])
            single = hip.gemv([hip.whole(mg), hip.whole(mu)], x[t:t + 1], 1)
            assert same_bits(single[0], gu[t])
    for m in (mg, mu, md):
        m.destroy()


def test_config2_decode_set_and_lm_head_argmax(hip, oracle):
    # Config 2: the Qwen3.5-2B-like decode set at N = 1; the lm_head's argmax must
    # be the CPU's (first maximum wins).
    golden = np.load(GOLDEN / "config2_decode_set.npz")
    x = synth.activations(1, cfg.HIDDEN2, cfg.CONFIG2_X_SEED)
    act = synth.activations(1, cfg.FFN2, cfg.CONFIG2_ACT_SEED)
    for stage, names in cfg.CONFIG2_STAGES.items():
        if stage == "lm_head":
            continue
        say("config 2", stage)
        specs = [cfg.CONFIG2[n] for n in names]
        host = [s.build() for s in specs]
        dev = [hip.Matrix(s.ggml_type, w, s.rows, s.cols) for s, w in zip(specs, host)]
        inp = act if stage == "ffn_down" else x
        got = hip.gemv([hip.whole(m) for m in dev], inp, 1)
        want = oracle.matmul([(s.ggml_type, w, 0, s.rows) for s, w in zip(specs, host)], inp,
                             precision="double", threads=8)
        assert oracle.rel_l2(got, want) <= TOLERANCE
        assert oracle.rel_l2(got, golden[stage]) <= TOLERANCE
        for m in dev:
            m.destroy()

    say("config 2 lm_head")
    spec = cfg.CONFIG2["lm_head"]
    head = spec.build()
    mh = hip.Matrix(spec.ggml_type, head, spec.rows, spec.cols)
    xd = hip.DeviceBuffer.from_array(x)
    yd = hip.DeviceBuffer(spec.rows * 4)
    hip.gemv_dev([hip.whole(mh)], xd, 1, yd)
    pick = hip.argmax_dev(yd, spec.rows)
    logits = yd.download((spec.rows,), np.float32)
    want = oracle.matmul([(spec.ggml_type, head, 0, spec.rows)], x, precision="double",
                         threads=8)[0]
    assert oracle.rel_l2(logits, want) <= TOLERANCE
    assert pick == oracle.argmax(want) == oracle.argmax(logits)
    assert pick == int(golden["lm_head_argmax"]) == int(golden["lm_head_argmax_double"])
    top = golden["lm_head_top8_index"]
    assert oracle.rel_l2(logits[top], golden["lm_head_top8_value"]) <= TOLERANCE
    assert oracle.rel_l2(logits[::64], golden["lm_head_every64"]) <= TOLERANCE
    assert abs(float(np.sum(logits, dtype=np.float64)) - float(golden["lm_head_sum"])) <= \
        TOLERANCE * float(golden["lm_head_abs_sum"])
    mh.destroy()
    xd.free()
    yd.free()


def test_argmax_first_maximum(hip, oracle):
    say("argmax")
    gen = synth.rng(77)
    for n in (1, 5, 1000, 151936, 300001):
        v = gen.standard_normal(n).astype(np.float32)
        if n > 10:
            v[n // 2] = v[n // 3] = v[n - 1] = 9.5  # the first of equal maxima wins
        buf = hip.DeviceBuffer.from_array(v)
        assert hip.argmax_dev(buf, n) == oracle.argmax(v) == int(np.argmax(v))
        buf.free()


def test_error_codes(hip):
    say("errors")
    w = synth.kquant_matrix(synth.Q4_K, 8, 512, 1)
    with pytest.raises(hip.InvalidArgumentError):  # partial block
        hip.Matrix(synth.Q4_K, w, 8, 500)
    with pytest.raises(hip.InvalidArgumentError):  # a type GgufProjections does not take: F16
        hip.Matrix(1, w, 8, 512)
    with pytest.raises(hip.InvalidArgumentError):  # Q8_0 rows are multiples of 256 values here
        hip.Matrix(synth.Q8_0, synth.q8_0_matrix(4, 288, 1), 4, 288)
    a = hip.Matrix(synth.Q4_K, w, 8, 512)
    b = hip.Matrix(synth.Q4_K, synth.kquant_matrix(synth.Q4_K, 8, 256, 2), 8, 256)
    x = synth.activations(1, 512, 3)
    with pytest.raises(hip.ShapeError):  # parts of one product share their input
        hip.gemv([hip.whole(a), hip.whole(b)], x, 1)
    with pytest.raises(hip.OutOfRangeError):
        hip.gemv([(a, 4, 5)], x, 1)
    with pytest.raises(hip.LogicError):  # no weights for this stage
        hip.gemv([], x, 1)
    with pytest.raises(hip.InvalidArgumentError):
        hip.gemv([hip.whole(a)], x, -1)
    # the library still works after the failures
    assert hip.gemv([hip.whole(a)], x, 1).shape == (1, 8)
    a.destroy()
    b.destroy()
