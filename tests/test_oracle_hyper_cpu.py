"""Pins of the oracle's hyper-connection (oracle/qw_oracle.c: qwo_hyper_gg) that do not come from retyping it: cases the
mathematics fixes, one-hot matrices that show which operand is transposed, an element-by-element loop on a tiny shape,
and the float64 matrix statement (the form of the reference's tools/hc_ref.py:60-70, which reads model dumps that do
not exist here)."""
import numpy as np
import pytest

HC, LR = 4, 320
ONE = 0x3F80  # bfloat16 1.0


def bf16(a):
    """float -> bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf2f(u):
    return (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def draw(rng, nb, D, hc=HC, lr=LR):
    h = rng.standard_normal((nb, hc, D)).astype(np.float32)
    out = (0.5 * rng.standard_normal((nb, D))).astype(np.float16)
    inj = rng.standard_normal((nb, hc, hc)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(hc * D)).astype(np.float32)
    Wd = bf16(rng.standard_normal((lr, hc * D)) / np.sqrt(hc * D))
    Wi = bf16(rng.standard_normal((hc, hc * D)) / np.sqrt(D))
    Wu = bf16(rng.standard_normal((hc * D, lr)) / np.sqrt(lr))
    return h, out, inj, w, Wd, Wi, Wu


def sig(v):
    return 1 / (1 + np.exp(-v))


def statement(h, out, inj, w, Wd, Wi, Wu, apply):
    nb, hc, D = h.shape
    h1 = h.astype(np.float64)
    if apply:
        h1 = h1 + out.astype(np.float64)[:, None, :] * (2 * sig(inj.astype(np.float64).sum(1) / hc))[:, :, None]
    r = 1 / np.sqrt((h1 ** 2).mean(2) + 1e-6)
    y = (h1 * r[:, :, None]).reshape(nb, hc * D) * w.astype(np.float64)
    d = y @ bf2f(Wd).T
    u = ((d / hc) * sig(d / hc)) @ bf2f(Wu).T
    x = (sig(u) * y).reshape(nb, hc, D).mean(1)
    io = None if Wi is None else np.einsum("tsi,qsi->tsq", y.reshape(nb, hc, D), bf2f(Wi).reshape(hc, hc, D))
    return h1, x, io, y.reshape(nb, hc, D)


@pytest.mark.parametrize("apply", [0, 1])
def test_matrix_statement(oracle, apply):
    a = draw(np.random.default_rng(1), 3, 256)
    h1, x, io = oracle.hyper_gg(*a, apply)
    rh, rx, rio, _ = statement(*a, apply)
    assert np.abs(h1 - rh).max() < 1e-12 and np.abs(x - rx).max() < 1e-12 and np.abs(io - rio).max() < 1e-11


def test_element_by_element_on_a_tiny_shape(oracle):
    rng = np.random.default_rng(2)
    hc, D, lr, nb = 2, 8, 3, 2
    h, out, inj, w, Wd, Wi, Wu = draw(rng, nb, D, hc, lr)
    h1, x, io = oracle.hyper_gg(h, out, inj, w, Wd, Wi, Wu, 1)
    fd, fi, fu = bf2f(Wd), bf2f(Wi), bf2f(Wu)
    for t in range(nb):
        y = np.zeros((hc, D))
        for s in range(hc):
            js = 2 / (1 + np.exp(-sum(float(inj[t, q, s]) for q in range(hc)) / hc))
            row = [float(h[t, s, j]) + float(out[t, j]) * js for j in range(D)]
            r = 1 / np.sqrt(sum(v * v for v in row) / D + 1e-6)
            for j in range(D):
                assert abs(h1[t, s, j] - row[j]) < 1e-14
                y[s, j] = row[j] * r * float(w[s * D + j])
        sx = []
        for r_ in range(lr):
            d = sum(fd[r_, s * D + j] * y[s, j] for s in range(hc) for j in range(D)) / hc
            sx.append(d / (1 + np.exp(-d)))
        for j in range(D):
            m = 0.0
            for s in range(hc):
                u = sum(fu[s * D + j, r_] * sx[r_] for r_ in range(lr))
                m += y[s, j] / (1 + np.exp(-u))
            assert abs(x[t, j] - m / hc) < 1e-13
        for s in range(hc):
            for q in range(hc):
                assert abs(io[t, s, q] - sum(fi[q, s * D + j] * y[s, j] for j in range(D))) < 1e-13


def test_zero_mix_up_halves_the_normalised_mean(oracle):
    h, out, inj, w, Wd, Wi, Wu = draw(np.random.default_rng(3), 2, 256)
    h1, x, _ = oracle.hyper_gg(h, out, inj, w, Wd, Wi, np.zeros_like(Wu), 0)
    hd = h.astype(np.float64)
    y = hd / np.sqrt((hd ** 2).mean(2, keepdims=True) + 1e-6) * w.astype(np.float64).reshape(1, HC, -1)
    assert np.array_equal(h1, hd)  # not applied: the streams come back as they were, whatever inj holds
    assert np.abs(x - 0.5 * y.mean(1)).max() < 1e-13


def test_zero_inject_sums_give_coefficient_one(oracle):
    h, out, inj, w, Wd, Wi, Wu = draw(np.random.default_rng(4), 2, 256)
    h1, _, _ = oracle.hyper_gg(h, out, np.zeros_like(inj), w, Wd, Wi, Wu, 1)
    assert np.abs(h1 - (h.astype(np.float64) + out.astype(np.float64)[:, None, :])).max() < 1e-15
    # and a column of large sums saturates one stream's coefficient at 2 while a column of very negative ones gives 0
    inj2 = np.zeros_like(inj)
    inj2[:, :, 1] = 200
    inj2[:, :, 2] = -200
    h2, _, _ = oracle.hyper_gg(h, out, inj2, w, Wd, Wi, Wu, 1)
    o = out.astype(np.float64)
    assert np.abs(h2[:, 1] - (h[:, 1] + 2 * o)).max() < 1e-12 and np.abs(h2[:, 2] - h[:, 2]).max() < 1e-12 and np.abs(h2[:, 0] - (h[:, 0] + o)).max() < 1e-15


def test_scaling_the_streams_changes_nothing_but_h(oracle):
    h, out, inj, w, Wd, Wi, Wu = draw(np.random.default_rng(5), 2, 256)
    _, x1, i1 = oracle.hyper_gg(h, out, inj, w, Wd, Wi, Wu, 0)
    _, x2, i2 = oracle.hyper_gg(h * np.float32(8), out, inj, w, Wd, Wi, Wu, 0)
    assert np.abs(x1 - x2).max() / np.abs(x1).max() < 2e-6 and np.abs(i1 - i2).max() / np.abs(i1).max() < 2e-6  # only through the 1e-6 under the root


def test_one_hot_rows_show_the_orientation(oracle):
    rng = np.random.default_rng(6)
    D = 256
    h, out, inj, w, _, _, _ = draw(rng, 1, D)
    _, _, _, y = statement(h, out, inj, w, np.zeros((LR, HC * D), np.uint16), None, np.zeros((HC * D, LR), np.uint16), 0)
    r0, s0, j0, s1, j1, q0 = 7, 2, 33, 1, 190, 3
    Wd = np.zeros((LR, HC * D), np.uint16)
    Wd[r0, s0 * D + j0] = ONE            # d[r0] = y[s0][j0]
    Wu = np.zeros((HC * D, LR), np.uint16)
    Wu[s1 * D + j1, r0] = ONE            # u[s1 D + j1] = silu(d[r0] / HC)
    Wi = np.zeros((HC, HC * D), np.uint16)
    Wi[q0, s0 * D + j0] = ONE            # inject sum [s0][q0] = y[s0][j0]
    _, x, io = oracle.hyper_gg(h, out, inj, w, Wd, Wi, Wu, 0)
    d = y[0, s0, j0] / HC
    u = d * sig(d)
    want = 0.5 * y[0].mean(0)
    want[j1] = (0.5 * (y[0, :, j1].sum() - y[0, s1, j1]) + sig(u) * y[0, s1, j1]) / HC
    assert np.abs(x[0] - want).max() < 1e-14
    wi = np.zeros((HC, HC))
    wi[s0, q0] = y[0, s0, j0]
    assert np.abs(io[0] - wi).max() < 1e-14
