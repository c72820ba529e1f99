"""Parity of the products that take the decoder's elementwise steps into their own
kernel (gufo_hip_gemv_fused_dev) with the CPU checker, through the C-ABI.

The checker runs the steps the way Decoder::Step does, one after the other: residual
add, RmsNorm, product; SwiGLU, product.  Bars: rel-L2 <= 1e-4 on the products; the stored
residual row bit-exact (one fp32 add); the stored normalized row within 4 ulp-sized
steps of the checker's (the sum of squares is added in another order); a token's
outputs bit-identical in whichever column of whichever call it travels."""
import numpy as np
import pytest

from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu

NAMES = synth.TYPE_NAMES
TOLERANCE = 1e-4
EPS = 1e-6  # Config::rms_eps of the Qwen3.5 files
QUANT_TYPES = [synth.Q4_K, synth.Q5_K, synth.Q6_K, synth.Q8_0]


def say(*args):
    print(*args, flush=True)


def same_bits(a, b) -> bool:
    return bool(np.array_equal(np.ascontiguousarray(a).view(np.uint32),
                               np.ascontiguousarray(b).view(np.uint32)))


def norm_weight(cols, seed):
    # GGUF norm weights already hold Qwen's +1: values around 1.
    rng = np.random.default_rng(seed)
    return (1.0 + 0.1 * rng.standard_normal(cols)).astype(np.float32)


class ResNormCall:
    """Device operands of one resnorm product, freed together."""

    def __init__(self, hip, m, x, delta, w, keep=True):
        self.hip = hip
        tokens, cols = x.shape
        self.tokens = tokens
        self.x = hip.DeviceBuffer.from_array(x)
        self.delta = None if delta is None else hip.DeviceBuffer.from_array(delta)
        self.w = hip.DeviceBuffer.from_array(w)
        self.residual = hip.DeviceBuffer(4 * tokens * cols) if keep else None
        self.normed = hip.DeviceBuffer(4 * tokens * cols) if keep else None
        self.y = hip.DeviceBuffer(4 * tokens * m.rows)
        self.m = m
        self.cols = cols

    def run(self):
        hip = self.hip
        prologue = hip.resnorm_prologue(self.w, EPS, self.delta, self.residual, self.normed)
        hip.gemv_fused_dev([hip.whole(self.m)], prologue, self.x, self.tokens, self.y)
        hip.synchronize()
        y = self.y.download((self.tokens, self.m.rows), np.float32)
        if self.residual is None:
            return y, None, None
        return (y, self.residual.download((self.tokens, self.cols), np.float32),
                self.normed.download((self.tokens, self.cols), np.float32))

    def free(self):
        for b in (self.x, self.delta, self.w, self.residual, self.normed, self.y):
            if b is not None:
                b.free()


RESNORM_SHAPES = [(96, 2048), (130, 2560), (33, 256), (40, 768), (64, 512), (17, 6144)]


@pytest.mark.parametrize("ggml_type", QUANT_TYPES)
@pytest.mark.parametrize("rows,cols", RESNORM_SHAPES)
def test_resnorm_product_parity(hip, oracle, ggml_type, rows, cols):
    seed = synth.BASE_SEED + 7000 + ggml_type * 100 + rows + cols
    w_rows = synth.matrix(ggml_type, rows, cols, seed)
    m = hip.Matrix(ggml_type, w_rows, rows, cols)
    w = norm_weight(cols, seed + 1)
    for tokens in (1, 2, 3, 4):
        say("resnorm", NAMES[ggml_type], rows, cols, "N", tokens)
        x = synth.activations(tokens, cols, seed + 10 + tokens)
        delta = 0.5 * synth.activations(tokens, cols, seed + 20 + tokens)
        want_residual, want_normed = oracle.res_norm(x, delta, w, EPS)
        exact = oracle.matmul([(ggml_type, w_rows, 0, rows)], want_normed, precision="double",
                              threads=4)
        call = ResNormCall(hip, m, x, delta, w)
        y, residual, normed = call.run()
        call.free()
        assert same_bits(residual, want_residual)
        # The checker adds the squares in eight long fp32 chains (the reference's
        # order), the kernel in a tree: against the checker the rows agree to the
        # chains' rounding (1e-6 relative), against the norm in double to a few units
        # in the last place.
        assert bool(np.all(np.abs(normed - want_normed) <= 2e-6 * np.abs(want_normed)))
        r64 = want_residual.astype(np.float64)
        closed = r64 / np.sqrt(np.mean(r64 * r64, axis=1, keepdims=True) + EPS) * w
        step = np.spacing(np.abs(closed).astype(np.float32))
        assert bool(np.all(np.abs(normed - closed) <= 4 * step))
        assert oracle.rel_l2(y, exact) <= TOLERANCE
        # The product of the stored normalized row is the fused product, bit for bit.
        plain = hip.gemv([hip.whole(m)], normed, tokens)
        assert same_bits(plain, y)
    m.destroy()


def test_resnorm_without_delta_or_outputs(hip, oracle):
    rows, cols = 64, 2048
    seed = synth.BASE_SEED + 7100
    w_rows = synth.matrix(synth.Q4_K, rows, cols, seed)
    m = hip.Matrix(synth.Q4_K, w_rows, rows, cols)
    w = norm_weight(cols, seed + 1)
    x = synth.activations(2, cols, seed + 2)
    _, want_normed = oracle.res_norm(x, None, w, EPS)
    exact = oracle.matmul([(synth.Q4_K, w_rows, 0, rows)], want_normed, precision="double")
    say("resnorm, no delta, outputs kept")
    kept = ResNormCall(hip, m, x, None, w)
    y_kept, residual, _ = kept.run()
    kept.free()
    say("resnorm, no delta, no outputs")
    bare = ResNormCall(hip, m, x, None, w, keep=False)
    y_bare, _, _ = bare.run()
    bare.free()
    m.destroy()
    assert oracle.rel_l2(y_kept, exact) <= TOLERANCE
    assert same_bits(y_kept, y_bare)
    assert same_bits(residual, x)


@pytest.mark.parametrize("ggml_type", [synth.Q4_K, synth.Q6_K])
@pytest.mark.parametrize("cols", [2048, 2560])
def test_resnorm_token_travels_unchanged(hip, ggml_type, cols):
    # The verify step relies on a token's result not depending on its column or on the
    # number of columns of the call (tests/models/qwen35_2b/npu_decode_test.cpp:136-148
    # of the reference): here through the norm as well.
    rows = 48
    seed = synth.BASE_SEED + 7200 + ggml_type + cols
    m = hip.Matrix(ggml_type, synth.matrix(ggml_type, rows, cols, seed), rows, cols)
    w = norm_weight(cols, seed + 1)
    x = synth.activations(4, cols, seed + 2)
    delta = synth.activations(4, cols, seed + 3)
    say("resnorm columns", NAMES[ggml_type], cols)
    call = ResNormCall(hip, m, x, delta, w)
    y4, _, normed4 = call.run()
    call.free()
    for t in range(4):
        say("  token", t, "alone")
        one = ResNormCall(hip, m, x[t:t + 1], delta[t:t + 1], w)
        y1, _, normed1 = one.run()
        one.free()
        assert same_bits(y1[0], y4[t])
        assert same_bits(normed1[0], normed4[t])
    # The same token in every column gives the same column four times.
    say("  one token in four columns")
    rep = ResNormCall(hip, m, np.repeat(x[1:2], 4, axis=0), np.repeat(delta[1:2], 4, axis=0), w)
    y_rep, _, _ = rep.run()
    rep.free()
    m.destroy()
    for t in range(4):
        assert same_bits(y_rep[t], y4[1])


def test_resnorm_constant_row_closed_form(hip):
    # RmsNorm of a constant row c with unit weights is sign(c) / sqrt(1 + eps / c^2) in
    # every position, whatever the row length; an identity-like matrix returns it.
    cols = 2048
    c = np.float32(-3.0)
    # fp32 rows take no prologue, so the identity is a Q8_0 matrix: d = 1, code 1 on the
    # diagonal - exactly representable.
    blocks = np.zeros((cols, cols // 32, 34), dtype=np.uint8)
    blocks[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    r = np.arange(cols)
    blocks[r, r // 32, 2 + r % 32] = 1
    ident = hip.Matrix(synth.Q8_0, blocks.reshape(-1), cols, cols)
    x = np.full((1, cols), c, dtype=np.float32)
    ones = np.ones(cols, dtype=np.float32)
    say("resnorm constant row")
    call = ResNormCall(hip, ident, x, None, ones)
    y, _, normed = call.run()
    call.free()
    ident.destroy()
    want = np.sign(np.float64(c)) / np.sqrt(1.0 + np.float64(EPS) / np.float64(c) ** 2)
    assert bool(np.all(np.abs(normed.astype(np.float64) - want) <= 2e-7))
    # The product quantizes the activations to 21 bits per scale group: 1e-6 relative.
    assert bool(np.all(np.abs(y.astype(np.float64) - want) <= 2e-6))


SWIGLU_SHAPES = [(64, 512), (96, 6144), (33, 256), (130, 9216), (50, 768)]


@pytest.mark.parametrize("ggml_type", QUANT_TYPES)
@pytest.mark.parametrize("rows,f", SWIGLU_SHAPES)
def test_swiglu_product_parity(hip, oracle, ggml_type, rows, f):
    seed = synth.BASE_SEED + 7300 + ggml_type * 100 + rows + f
    w_rows = synth.matrix(ggml_type, rows, f, seed)
    m = hip.Matrix(ggml_type, w_rows, rows, f)
    for tokens in (1, 2, 3, 4):
        say("swiglu", NAMES[ggml_type], rows, f, "N", tokens)
        gate_up = synth.activations(tokens, 2 * f, seed + tokens)
        act = oracle.swiglu(gate_up)
        exact = oracle.matmul([(ggml_type, w_rows, 0, rows)], act, precision="double", threads=4)
        x = hip.DeviceBuffer.from_array(gate_up)
        y = hip.DeviceBuffer(4 * tokens * rows)
        hip.gemv_fused_dev([hip.whole(m)], hip.swiglu_prologue(), x, tokens, y)
        hip.synchronize()
        got = y.download((tokens, rows), np.float32)
        assert oracle.rel_l2(got, exact) <= TOLERANCE
        for t in range(tokens):
            x1 = hip.DeviceBuffer.from_array(gate_up[t:t + 1])
            y1 = hip.DeviceBuffer(4 * rows)
            hip.gemv_fused_dev([hip.whole(m)], hip.swiglu_prologue(), x1, 1, y1)
            hip.synchronize()
            assert same_bits(y1.download((rows,), np.float32), got[t])
            x1.free()
            y1.free()
        x.free()
        y.free()
    m.destroy()


def test_decoder_layer_chain(hip, oracle):
    # The products of one dense layer as Decoder::Step orders them
    # (src/models/qwen35/decoder.cpp:491-521 of the reference), with a stand-in for the
    # mixer (it is not on this path): four launches, nothing between them, against the
    # same steps run one by one on the host.
    hidden, ffn = 2048, 6144  # the decode set's layer widths
    seed = synth.BASE_SEED + 7400
    q = synth.matrix(synth.Q4_K, hidden, hidden, seed)
    o = synth.matrix(synth.Q4_K, hidden, hidden, seed + 1)
    gate = synth.matrix(synth.Q4_K, ffn, hidden, seed + 2)
    up = synth.matrix(synth.Q4_K, ffn, hidden, seed + 3)
    down = synth.matrix(synth.Q6_K, hidden, ffn, seed + 4)
    mats = {n: hip.Matrix(t, w, r, k) for n, (t, w, r, k) in {
        "q": (synth.Q4_K, q, hidden, hidden), "o": (synth.Q4_K, o, hidden, hidden),
        "gate": (synth.Q4_K, gate, ffn, hidden), "up": (synth.Q4_K, up, ffn, hidden),
        "down": (synth.Q6_K, down, hidden, ffn)}.items()}
    attn_norm = norm_weight(hidden, seed + 5)
    post_norm = norm_weight(hidden, seed + 6)
    # Weights as synthesized are not zero-mean (products of 1e2): scale the stand-in
    # outputs back so the residual stream stays of order one, as in a trained model.
    shrink = np.float32(1.0 / 256)
    for tokens in (1, 2):
        say("layer chain, N", tokens)
        h = synth.activations(tokens, hidden, seed + 10 + tokens)
        prev = 0.25 * synth.activations(tokens, hidden, seed + 20 + tokens)

        # Host, step by step.
        h1, normed = oracle.res_norm(h, prev, attn_norm, EPS)
        mixed = oracle.matmul([(synth.Q4_K, q, 0, hidden)], normed, precision="double")
        mixed = (mixed * shrink).astype(np.float32)
        out = oracle.matmul([(synth.Q4_K, o, 0, hidden)], mixed, precision="double")
        out = (out * shrink).astype(np.float32)
        h2, normed2 = oracle.res_norm(h1, out, post_norm, EPS)
        gu = oracle.matmul([(synth.Q4_K, gate, 0, ffn), (synth.Q4_K, up, 0, ffn)], normed2,
                           precision="double")
        gu = (gu * shrink).astype(np.float32)
        want = oracle.matmul([(synth.Q6_K, down, 0, hidden)], oracle.swiglu(gu),
                             precision="double")

        # Device: the mixer stand-in and the scaling run on the host between launches.
        d = {k: hip.DeviceBuffer.from_array(v) for k, v in {
            "h": h, "prev": prev, "attn_norm": attn_norm, "post_norm": post_norm}.items()}
        for name, floats in {"h1": hidden, "h2": hidden, "in": hidden, "mixed": hidden,
                             "out": hidden, "gu": 2 * ffn, "y": hidden}.items():
            d[name] = hip.DeviceBuffer(4 * tokens * floats)
        hip.gemv_fused_dev([hip.whole(mats["q"])],
                           hip.resnorm_prologue(d["attn_norm"], EPS, d["prev"], d["h1"]),
                           d["h"], tokens, d["in"])
        hip.synchronize()
        d["mixed"].upload(d["in"].download((tokens, hidden), np.float32) * shrink)
        hip.gemv_dev([hip.whole(mats["o"])], d["mixed"], tokens, d["out"])
        hip.synchronize()
        d["out"].upload(d["out"].download((tokens, hidden), np.float32) * shrink)
        hip.gemv_fused_dev([hip.whole(mats["gate"]), hip.whole(mats["up"])],
                           hip.resnorm_prologue(d["post_norm"], EPS, d["out"], d["h2"]),
                           d["h1"], tokens, d["gu"])
        hip.synchronize()
        d["gu"].upload(d["gu"].download((tokens, 2 * ffn), np.float32) * shrink)
        hip.gemv_fused_dev([hip.whole(mats["down"])], hip.swiglu_prologue(), d["gu"], tokens,
                           d["y"])
        hip.synchronize()
        got = d["y"].download((tokens, hidden), np.float32)
        got_h2 = d["h2"].download((tokens, hidden), np.float32)
        for b in d.values():
            b.free()
        assert oracle.rel_l2(got_h2, h2) <= 1e-5
        assert oracle.rel_l2(got, want) <= 3 * TOLERANCE  # four products deep
    for m in mats.values():
        m.destroy()


def test_prologue_argument_errors(hip):
    rows, cols = 32, 512
    m = hip.Matrix(synth.Q4_K, synth.matrix(synth.Q4_K, rows, cols, 5), rows, cols)
    f = hip.Matrix(synth.F32, synth.matrix(synth.F32, rows, cols, 6), rows, cols)
    x = hip.DeviceBuffer(4 * 2 * cols)
    w = hip.DeviceBuffer(4 * cols)
    y = hip.DeviceBuffer(4 * 2 * rows)
    say("prologue errors")
    with pytest.raises(hip.InvalidArgumentError):   # unknown kind
        hip.gemv_fused_dev([hip.whole(m)], hip.Prologue(9, None, None, 0.0, None, None), x, 1, y)
    with pytest.raises(hip.InvalidArgumentError):   # no norm weight
        hip.gemv_fused_dev([hip.whole(m)], hip.Prologue(2, None, None, EPS, None, None), x, 1, y)
    with pytest.raises(hip.InvalidArgumentError):   # the residual row would overwrite x
        hip.gemv_fused_dev([hip.whole(m)], hip.resnorm_prologue(w, EPS, None, x), x, 1, y)
    with pytest.raises(hip.InvalidArgumentError):   # outputs overlap each other
        hip.gemv_fused_dev([hip.whole(m)], hip.resnorm_prologue(w, EPS, None, y, y), x, 1, y)
    with pytest.raises(hip.InvalidArgumentError):   # fp32 rows take no prologue
        hip.gemv_fused_dev([hip.whole(f)], hip.swiglu_prologue(), x, 1, y)
    # A null prologue is the plain product.
    hip.gemv_fused_dev([hip.whole(m)], None, x, 1, y)
    hip.synchronize()
    for b in (x, w, y):
        b.free()
    m.destroy()
    f.destroy()
