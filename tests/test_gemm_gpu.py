"""Parity of the prefill GEMM (Q4_K weights x bf16 activations on the matrix cores)
with the CPU checker and the golden reference slice, through the C-ABI.

Bar: rel-L2 <= 1e-3 against dequantize + double sum over the same bf16 activation
values (the bar stated for this kernel).  The kernel rounds each dequantized weight to
fp16 once (relative 2^-12 at most) and accumulates in fp32, which lands near 1.5e-4."""
import numpy as np
import pytest

from conftest import GOLDEN
from gufo_npu_amd import configs as cfg
from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-3
VS_GEMV = 5e-4     # the GEMV kernels are ~1e-7 from the truth, so this bounds the GEMM alone


def say(*args):
    print(*args, flush=True)


def bf16_activations(tokens, cols, seed):
    bits = synth.bf16_round(synth.activations(tokens, cols, seed))
    return bits, synth.bf16_to_float(bits)


@pytest.mark.parametrize("tokens,rows,cols", [(128, 128, 256), (1, 32, 512), (77, 200, 512),
                                              (300, 129, 2048), (130, 257, 768)])
def test_gemm_parity_small_and_ragged(hip, oracle, tokens, rows, cols):
    say("gemm", tokens, rows, cols)
    seed = 7000 + tokens + rows + cols
    w = synth.kquant_matrix(synth.Q4_K, rows, cols, seed)
    bits, a = bf16_activations(tokens, cols, seed + 1)
    m = hip.Matrix(synth.Q4_K, w, rows, cols)
    got = hip.gemm_q4k_bf16(m, bits)
    want = oracle.matmul([(synth.Q4_K, w, 0, rows)], a, precision="double", threads=8)
    assert got.shape == want.shape == (tokens, rows)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    # every row of C is the matrix-vector product of that token
    for t in sorted({0, tokens // 2, tokens - 1}):
        single = hip.gemv([hip.whole(m)], a[t:t + 1], 1)
        assert oracle.rel_l2(got[t], single[0]) <= VS_GEMV
    m.destroy()


def test_gemm_unit_activations_return_the_weights(hip, oracle):
    # a = unit vectors (exact in bf16): C[t] is column t of the dequantized matrix, each
    # weight rounded to fp16 once: off by at most half an fp16 ulp, 2^-11 relative (the
    # weights here are far above the fp16 subnormal range, where the bound is absolute).
    say("gemm identity")
    rows, cols = 64, 512
    w = synth.kquant_matrix(synth.Q4_K, rows, cols, 99)
    m = hip.Matrix(synth.Q4_K, w, rows, cols)
    bits = synth.bf16_round(np.eye(cols, dtype=np.float32))
    got = hip.gemm_q4k_bf16(m, bits)
    want = np.stack([oracle.dequantize(synth.Q4_K, w[r], cols) for r in range(rows)], axis=1)
    assert got.shape == want.shape
    # plus the offset 1024 d sc + dmin m rounded to fp32: below 1e-4 of the row's largest
    slack = 1e-4 * np.abs(want).max(axis=0, keepdims=True)
    bound = np.maximum(np.abs(want) * 2.0 ** -11, 2.0 ** -25) + slack
    assert bool(np.all(np.abs(got.astype(np.float64) - want) <= bound))
    assert oracle.rel_l2(got, want) <= 3e-4
    m.destroy()


def test_gemm_full_size_is_independent_of_token_order(hip):
    # Config-5 size, every one of the 4096 x 6144 outputs: a token's row of C is computed
    # from that token's activations alone, in an order that does not depend on where the
    # token sits, so reversing the token order must reverse C bit for bit.  Any mix-up of
    # tiles, stages of the LDS ring or store addresses breaks this.
    say("gemm token order, full size")
    spec = cfg.CONFIG5
    w = spec.build()
    bits, _ = bf16_activations(cfg.CONFIG5_TOKENS, spec.cols, cfg.CONFIG5_A_SEED)
    m = hip.Matrix(spec.ggml_type, w, spec.rows, spec.cols)
    forward = hip.gemm_q4k_bf16(m, bits)
    backward = hip.gemm_q4k_bf16(m, np.ascontiguousarray(bits[::-1]))
    assert bool(np.array_equal(forward.view(np.uint32), backward[::-1].view(np.uint32)))
    # and a second run repeats the first
    again = hip.gemm_q4k_bf16(m, bits)
    assert bool(np.array_equal(forward.view(np.uint32), again.view(np.uint32)))
    m.destroy()


def test_gemm_rejects_other_types(hip):
    say("gemm type check")
    w = synth.kquant_matrix(synth.Q6_K, 32, 256, 1)
    m = hip.Matrix(synth.Q6_K, w, 32, 256)
    with pytest.raises(hip.InvalidArgumentError):
        hip.gemm_q4k_bf16(m, np.zeros((4, 256), np.uint16))
    m.destroy()
    f = hip.Matrix(synth.F32, synth.matrix(synth.F32, 32, 256, 2), 32, 256)
    with pytest.raises(hip.InvalidArgumentError):
        hip.gemm_bf16(f, np.zeros((4, 256), np.uint16))
    f.destroy()


OTHER_TYPES = [synth.Q5_K, synth.Q6_K, synth.Q8_0]


@pytest.mark.parametrize("ggml_type", OTHER_TYPES)
@pytest.mark.parametrize("tokens,rows,cols", [(128, 256, 256), (77, 200, 512), (300, 129, 2048),
                                              (5, 33, 2304)])
def test_gemm_parity_other_row_types(hip, oracle, ggml_type, tokens, rows, cols):
    # The prefill product for the other row types a stage can hold: the same product
    # kernel behind a pre-pass that dequantizes that type.
    say("gemm", synth.TYPE_NAMES[ggml_type], tokens, rows, cols)
    seed = 7100 + 31 * ggml_type + tokens + rows + cols
    w = synth.matrix(ggml_type, rows, cols, seed)
    bits, a = bf16_activations(tokens, cols, seed + 1)
    m = hip.Matrix(ggml_type, w, rows, cols)
    got = hip.gemm_bf16(m, bits)
    want = oracle.matmul([(ggml_type, w, 0, rows)], a, precision="double", threads=8)
    assert got.shape == want.shape == (tokens, rows)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    for t in sorted({0, tokens // 2, tokens - 1}):
        single = hip.gemv([hip.whole(m)], a[t:t + 1], 1)
        assert oracle.rel_l2(got[t], single[0]) <= VS_GEMV
    m.destroy()


@pytest.mark.parametrize("ggml_type", [synth.Q5_K, synth.Q6_K])
def test_gemm_unit_activations_return_the_weights_other_types(hip, oracle, ggml_type):
    # Every weight of the matrix, one by one, as the pre-pass dequantized it: within half
    # an fp16 ulp of the checker's dequantization (pinned by the reference's fixtures).
    # A wrong bit of a code, a wrong scale index or a wrong position shows here.
    say("gemm identity", synth.TYPE_NAMES[ggml_type])
    rows, cols = 64, 512
    w = synth.kquant_matrix(ggml_type, rows, cols, 98)
    m = hip.Matrix(ggml_type, w, rows, cols)
    bits = synth.bf16_round(np.eye(cols, dtype=np.float32))
    got = hip.gemm_bf16(m, bits)
    want = np.stack([oracle.dequantize(ggml_type, w[r], cols) for r in range(rows)], axis=1)
    bound = np.maximum(np.abs(want) * 2.0 ** -11, 2.0 ** -25)
    if ggml_type == synth.Q5_K:  # d sc q - dmin m is rounded once more, in fp32
        bound = bound + 2.0 ** -23 * np.abs(want).max(axis=0, keepdims=True)
    assert bool(np.all(np.abs(got.astype(np.float64) - want) <= bound))
    m.destroy()


@pytest.mark.parametrize("ggml_type", [synth.Q4_K, synth.Q6_K])
def test_gemm_with_prepared_weights_gives_the_same_bits(hip, ggml_type):
    # gufo_hip_matrix_prepare_prefill keeps the converted weights with the matrix: every
    # later product skips that half of the pre-pass and must not change by a bit, whatever
    # the token count, and a row subset taken from a prepared matrix stands on its own.
    say("gemm prepared", synth.TYPE_NAMES[ggml_type])
    rows, cols = 300, 768
    w = synth.matrix(ggml_type, rows, cols, 7300 + ggml_type)
    m = hip.Matrix(ggml_type, w, rows, cols)
    inputs = [bf16_activations(tokens, cols, 7310 + tokens)[0] for tokens in (1, 130, 257)]
    before = [hip.gemm_bf16(m, bits) for bits in inputs]
    m.prepare_prefill()
    m.prepare_prefill()  # a second call changes nothing
    for bits, want in zip(inputs, before):
        assert bool(np.array_equal(hip.gemm_bf16(m, bits).view(np.uint32), want.view(np.uint32)))
    picked = m.gather_rows(np.arange(10, 74))
    got = hip.gemm_bf16(picked, inputs[1])
    assert bool(np.array_equal(got.view(np.uint32), before[1][:, 10:74].view(np.uint32)))
    picked.destroy()
    # the GEMV entry points are untouched by it
    x = synth.activations(2, cols, 5)
    y = hip.gemv([hip.whole(m)], x, 2)
    m.destroy()
    again = hip.Matrix(ggml_type, w, rows, cols)
    assert bool(np.array_equal(hip.gemv([hip.whole(again)], x, 2).view(np.uint32), y.view(np.uint32)))
    again.destroy()
    f = hip.Matrix(synth.F32, synth.matrix(synth.F32, 32, 256, 2), 32, 256)
    with pytest.raises(hip.InvalidArgumentError):
        f.prepare_prefill()
    f.destroy()


def test_gemm_of_a_stage_lays_its_parts_side_by_side(hip, oracle):
    # [q | k | v]-like: three matrices of two types sharing their input, one of them with
    # prepared weights; c[t] = [part 0 | part 1 | part 2], each column block bit for bit
    # the matrix's own product, ragged row counts included.
    say("gemm parts")
    cols, tokens = 512, 150
    shapes = [(synth.Q4_K, 200), (synth.Q6_K, 33), (synth.Q4_K, 64)]
    blocks = [synth.matrix(t, rows, cols, 7400 + i) for i, (t, rows) in enumerate(shapes)]
    mats = [hip.Matrix(t, b, rows, cols) for (t, rows), b in zip(shapes, blocks)]
    mats[2].prepare_prefill()
    bits, a = bf16_activations(tokens, cols, 7410)
    stride = sum(rows for _, rows in shapes)
    da = hip.DeviceBuffer.from_array(bits)
    dc = hip.DeviceBuffer(4 * tokens * stride)
    hip.gemm_bf16_parts_dev(mats, da, tokens, dc)
    hip.synchronize()
    got = dc.download((tokens, stride), np.float32)
    offset = 0
    for m, (_, rows) in zip(mats, shapes):
        alone = hip.gemm_bf16(m, bits)
        assert bool(np.array_equal(got[:, offset:offset + rows].view(np.uint32),
                                   alone.view(np.uint32)))
        offset += rows
    want = oracle.matmul([(t, b, 0, rows) for (t, rows), b in zip(shapes, blocks)], a,
                         precision="double", threads=8)
    assert oracle.rel_l2(got, want) <= TOLERANCE
    other = hip.Matrix(synth.Q4_K, synth.matrix(synth.Q4_K, 32, 256, 1), 32, 256)
    with pytest.raises(hip.ShapeError):
        hip.gemm_bf16_parts_dev([mats[0], other], da, tokens, dc)
    for m in mats + [other]:
        m.destroy()


def test_gemm_q4k_entry_point_equals_the_general_one(hip):
    w = synth.kquant_matrix(synth.Q4_K, 96, 512, 5)
    m = hip.Matrix(synth.Q4_K, w, 96, 512)
    bits, _ = bf16_activations(40, 512, 6)
    assert bool(np.array_equal(hip.gemm_q4k_bf16(m, bits).view(np.uint32),
                               hip.gemm_bf16(m, bits).view(np.uint32)))
    m.destroy()


def test_config5_prefill_projection(hip, oracle):
    # Config 5: activations 4096 x 2048 bf16 times Q4_K 6144 x 2048.
    say("config 5")
    spec = cfg.CONFIG5
    w = spec.build()
    bits, a = bf16_activations(cfg.CONFIG5_TOKENS, spec.cols, cfg.CONFIG5_A_SEED)
    m = hip.Matrix(spec.ggml_type, w, spec.rows, spec.cols)
    got = hip.gemm_q4k_bf16(m, bits)
    golden = np.load(GOLDEN / "config5_prefill_slice.npz")
    tokens = golden["tokens"]
    assert oracle.rel_l2(got[tokens][:, ::8], golden["c_double_every8"]) <= TOLERANCE
    # other token rows against the CPU checker, and against the GEMV kernel
    pick = np.array([1, 777, 2049, 4095])
    want = oracle.matmul([(spec.ggml_type, w, 0, spec.rows)], a[pick], precision="double",
                         threads=8)
    assert oracle.rel_l2(got[pick], want) <= TOLERANCE
    single = hip.gemv([hip.whole(m)], a[pick], len(pick))
    assert oracle.rel_l2(got[pick], single) <= VS_GEMV
    say("config 5 rel-L2 vs double", oracle.rel_l2(got[pick], want))
    m.destroy()
