"""What pins the checker's RmsNorm, residual add and SwiGLU (no GPU needed): closed forms
in double, special cases a wrong term would break, and the compiled reference."""
import numpy as np
import pytest

EPS = 1e-6


def rows(n, seed, scale=1.0):
    return (scale * np.random.default_rng(seed).standard_normal(n)).astype(np.float32)


@pytest.mark.parametrize("n", [8, 256, 2048, 2560, 4099])
def test_rms_norm_matches_closed_form(oracle, n):
    x, w = rows(n, n), rows(n, n + 1)
    got = oracle.rms_norm(x, w, EPS)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt(np.mean(x64 * x64) + EPS) * w
    # fp32 throughout: a few rounding steps per value, no more.
    assert np.all(np.abs(got - want) <= 4 * np.spacing(np.abs(want).astype(np.float32)))


def test_rms_norm_constant_row(oracle):
    # Every position of a constant row c normalizes to sign(c) / sqrt(1 + eps / c^2):
    # a mean taken over the wrong count, or eps added outside the root, changes it.
    for c, eps in ((2.0, 1e-6), (-3.0, 0.5), (0.125, 4.0)):
        n = 1000
        got = oracle.rms_norm(np.full(n, c, np.float32), np.ones(n, np.float32), eps)
        want = np.sign(c) / np.sqrt(1.0 + eps / (c * c))
        assert np.all(np.abs(got.astype(np.float64) - want) <= 2e-7)


def test_rms_norm_scale_invariance_and_weight(oracle):
    # With eps = 0 scaling the row by a power of two changes nothing, bit for bit; the
    # weight multiplies position by position.
    n = 768
    x, w = rows(n, 3), rows(n, 4)
    base = oracle.rms_norm(x, w, 0.0)
    assert np.array_equal(oracle.rms_norm(x * np.float32(64.0), w, 0.0), base)
    unit = oracle.rms_norm(x, np.ones(n, np.float32), 0.0)
    assert np.array_equal(base, unit * w)
    # The mean of the squares of a normalized row is one.
    assert abs(float(np.mean(unit.astype(np.float64) ** 2)) - 1.0) <= 1e-6
    # Zero row: eps keeps it finite and zero.
    assert np.array_equal(oracle.rms_norm(np.zeros(n, np.float32), w, EPS),
                          np.zeros(n, np.float32))


def test_rms_norm_in_place(oracle):
    import ctypes as C
    n = 512
    x, w = rows(n, 5), rows(n, 6)
    want = oracle.rms_norm(x, w, EPS)
    buf = x.copy()
    p = buf.ctypes.data_as(C.c_void_p)
    oracle.lib().gufo_oracle_rms_norm(p, w.ctypes.data_as(C.c_void_p), n, EPS, p)
    assert np.array_equal(buf, want)


@pytest.mark.parametrize("n", [256, 2048, 2560, 9216])
def test_rms_norm_matches_compiled_reference(ref_oracle, n):
    # vec::RmsNorm as the reference builds it adds the squares in its AVX2 order: the
    # inverse may differ in its last place, so each value by a couple of steps.
    x, w = rows(n, 7 + n), rows(n, 8 + n)
    ours = ref_oracle.rms_norm(x, w, EPS)
    theirs = ref_oracle.rms_norm(x, w, EPS, use_ref=True)
    assert bool(np.all(np.abs(ours - theirs) <= 4 * np.spacing(np.abs(theirs))))


def test_res_norm_is_add_then_norm(oracle):
    n = 2048
    x = np.stack([rows(n, 10), rows(n, 11)])
    d = np.stack([rows(n, 12, 0.5), rows(n, 13, 0.5)])
    w = rows(n, 14)
    residual, normed = oracle.res_norm(x, d, w, EPS)
    assert np.array_equal(residual, x + d)
    for t in range(2):
        assert np.array_equal(normed[t], oracle.rms_norm(x[t] + d[t], w, EPS))
    # No addend: the residual row is the input.
    residual, normed = oracle.res_norm(x, None, w, EPS)
    assert np.array_equal(residual, x)
    assert np.array_equal(normed[1], oracle.rms_norm(x[1], w, EPS))


def test_swiglu_closed_form_and_special_values(oracle):
    f = 1000
    gu = np.random.default_rng(20).standard_normal((3, 2 * f)).astype(np.float32) * 4
    got = oracle.swiglu(gu)
    g = gu[:, :f].astype(np.float64)
    want = g / (1.0 + np.exp(-g)) * gu[:, f:]
    assert np.all(np.abs(got - want) <= 4 * np.spacing(np.abs(want).astype(np.float32)) + 1e-30)
    # silu(0) = 0; silu(x) -> x for large x; silu(-x) = silu(x) - x; the up half scales.
    special = np.array([[0.0, 40.0, -40.0, 1.5, -1.5, 2.0, 2.0, 2.0, 1.0, 1.0]], np.float32)
    out = oracle.swiglu(special)[0]
    assert out[0] == 0.0
    assert out[1] == 80.0
    assert abs(out[2]) < 1e-15
    silu = lambda v: v / (1.0 + np.exp(-v))  # noqa: E731
    assert abs(out[3] - silu(1.5)) <= 1e-7
    assert abs((out[3] - out[4]) - 1.5) <= 2e-7
    # Gate and up halves are not interchangeable: swapping them changes the result.
    swapped = np.concatenate([gu[:, f:], gu[:, :f]], axis=1)
    assert not np.allclose(oracle.swiglu(swapped), got)
