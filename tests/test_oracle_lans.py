"""Pins the NumPy LANS oracle: hand-computable cases, special cases fixed by the
formula, and an independent fp64 derivation written from the LANS paper
(arXiv 2006.13484, Algorithm 2) rather than from the kernel."""
import numpy as np
import pytest

from oracle import lans_oracle as lo


def paper_lans_fp64(g, x, m, v, t, lr, b1, b2, eps, lam):
    """Algorithm 2 of the paper (block = tensor, phi = identity), with the eps
    placement of the implementation the reference descends from."""
    g, x, m, v = (a.astype(np.float64) for a in (g, x, m, v))
    gt = g / (np.linalg.norm(g) + eps)
    m = b1 * m + (1 - b1) * gt
    v = b2 * v + (1 - b2) * gt * gt
    mh = m / (1 - b1 ** t)
    vh = v / (1 - b2 ** t)
    r = mh / (np.sqrt(vh) + eps) + lam * x
    c = gt / (np.sqrt(vh) + eps) + lam * x
    xn = np.linalg.norm(x)
    x = x - lr * b1 * xn / np.linalg.norm(r) * r - lr * (1 - b1) * xn / np.linalg.norm(c) * c
    return x, m, v


def test_against_paper_fp64_ten_steps():
    rng = np.random.default_rng(0)
    shapes = [(17,), (8, 9), (3, 5, 7), (1,), (64, 33)]
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    p64 = [a.astype(np.float64) for a in p]
    m64 = [a.astype(np.float64) for a in m]
    v64 = [a.astype(np.float64) for a in v]
    for step in range(1, 11):
        g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
        lo.lans_step(g, p, m, v, step)
        for i in range(len(shapes)):
            p64[i], m64[i], v64[i] = paper_lans_fp64(g[i], p64[i], m64[i], v64[i], step,
                                                     1e-3, np.float64(np.float32(0.9)),
                                                     np.float64(np.float32(0.999)),
                                                     np.float64(np.float32(1e-6)),
                                                     np.float64(np.float32(0.01)))
    for i in range(len(shapes)):
        np.testing.assert_allclose(p[i], p64[i], rtol=2e-5, atol=1e-9)
        np.testing.assert_allclose(m[i], m64[i], rtol=2e-5, atol=1e-9)
        np.testing.assert_allclose(v[i], v64[i], rtol=2e-5, atol=1e-12)


def test_single_element_closed_form():
    """For a 1-element tensor ratio*u = lr*|p|*sign(u): p' = p - lr*|p| (both terms
    have the sign of u, and beta1 + beta3 = 1)."""
    g, p = [np.array([2.0], np.float32)], [np.array([3.0], np.float32)]
    m, v = [np.zeros(1, np.float32)], [np.zeros(1, np.float32)]
    norms = lo.lans_step(g, p, m, v, 1)
    np.testing.assert_allclose(p[0], 3.0 - 1e-3 * 3.0, rtol=3e-7)
    ghat = 2.0 / (2.0 + 1e-6)
    np.testing.assert_allclose(m[0], 0.1 * ghat, rtol=1e-6)
    np.testing.assert_allclose(v[0], (1.0 - float(np.float32(0.999))) * ghat * ghat, rtol=1e-6)  # (1-beta2) is taken in fp32
    assert norms[0][0] == np.float32(2.0) and norms[0][1] == np.float32(3.0)
    # u_m = ghat/(ghat+eps) + 0.01*3
    np.testing.assert_allclose(norms[0][2], ghat / (ghat + 1e-6) + 0.03, rtol=1e-6)


def test_zero_grad_tensor():
    """g = 0: no normalisation (norm == 0), m = v = 0, u = wd*p, ratio = lr/wd,
    so p' = p*(1 - lr)."""
    p0 = np.array([0.5, -1.0, 2.0, 4.0], np.float32)
    g, p = [np.zeros(4, np.float32)], [p0.copy()]
    m, v = [np.zeros(4, np.float32)], [np.zeros(4, np.float32)]
    lo.lans_step(g, p, m, v, 3)
    np.testing.assert_allclose(p[0], p0 * (1 - 1e-3), rtol=3e-7)
    assert not m[0].any() and not v[0].any()


def test_zero_param_tensor_uses_plain_lr():
    """||p|| == 0 -> both ratios fall back to lr (multi_tensor_lans.cu:349-350)."""
    rng = np.random.default_rng(3)
    g0 = rng.normal(0, 1, 6).astype(np.float32)
    g, p = [g0.copy()], [np.zeros(6, np.float32)]
    m, v = [np.zeros(6, np.float32)], [np.zeros(6, np.float32)]
    lo.lans_step(g, p, m, v, 1, weight_decay=0.0, bias_correction=1)
    gh = g0.astype(np.float64) / (np.linalg.norm(g0.astype(np.float64)) + 1e-6)
    u = gh / (np.abs(gh) + 1e-6)           # step 1: mhat = ghat, sqrt(vhat) = |ghat|
    np.testing.assert_allclose(p[0], -1e-3 * (0.9 * u + 0.1 * u), rtol=1e-4)


def test_mode0_equals_mode1_without_weight_decay_and_scale_invariance():
    rng = np.random.default_rng(4)
    g0 = rng.normal(0, 1e-3, (7, 5)).astype(np.float32)
    p0 = rng.normal(0, 0.02, (7, 5)).astype(np.float32)
    outs = []
    for mode, scale in [(0, 1.0), (1, 1.0), (1, 64.0)]:
        g, p = [g0 * np.float32(scale)], [p0.copy()]
        m, v = [np.zeros_like(p0)], [np.zeros_like(p0)]
        for step in (1, 2, 3):
            lo.lans_step(g, p, m, v, step, weight_decay=0.0, mode=mode)
        outs.append(p[0])
    np.testing.assert_array_equal(outs[0], outs[1])
    np.testing.assert_allclose(outs[1], outs[2], rtol=1e-5)


@pytest.mark.parametrize("bias_correction,grad_averaging", [(0, 1), (1, 0), (0, 0)])
def test_flags(bias_correction, grad_averaging):
    g, p = [np.array([1.0, -1.0], np.float32)], [np.array([1.0, 1.0], np.float32)]
    m, v = [np.zeros(2, np.float32)], [np.zeros(2, np.float32)]
    lo.lans_step(g, p, m, v, 5, bias_correction=bias_correction, grad_averaging=grad_averaging,
                 normalize_grad=False, weight_decay=0.0)
    beta3 = 0.1 if grad_averaging else 1.0
    np.testing.assert_allclose(m[0], beta3 * np.array([1.0, -1.0]), rtol=1e-6)
    np.testing.assert_allclose(v[0], (1.0 - float(np.float32(0.999))) * np.ones(2), rtol=1e-6)
    bc1, bc2 = lo.bias_corrections(5, 0.9, 0.999, bias_correction)
    if bias_correction:
        np.testing.assert_allclose([bc1, bc2], [1 - 0.9 ** 5, 1 - 0.999 ** 5], rtol=1e-4)
    else:
        assert bc1 == 1 and bc2 == 1


def test_mode0_weight_decay_two_elements_by_hand():
    """Mode 0 adds weight_decay * p to the scaled gradient BEFORE the moments
    (multi_tensor_lans.cu:287-297); mode 1 adds it to the two updates after them (:299-306).  With two
    elements the placement shows in p, m and v.  Numbers worked out by hand for g = (0.3, -0.4),
    p = (2, 1), m = v = 0, lr 0.1, beta1 = beta2 = 0.5, eps 0, no bias correction, wd 0.25:
    ||g|| = 0.5, g/||g|| = (0.6, -0.8), + wd*p = (1.1, -0.55); m' = 0.5 * that, v' = 0.5 * that^2;
    u_m = m'/sqrt(v') = (1, -1)/sqrt(2), u_g = (1, -1)*sqrt(2); ||u_m|| = 1, ||u_g|| = 2, ||p|| = sqrt(5);
    p' = p - (0.1*sqrt(5)/1*0.5)*u_m - (0.1*sqrt(5)/2*0.5)*u_g = p -/+ 0.1*sqrt(5)/sqrt(2)."""
    kw = dict(lr=0.1, beta1=0.5, beta2=0.5, eps=0.0, bias_correction=0, weight_decay=0.25, grad_averaging=1,
              normalize_grad=True)
    g = [np.array([0.3, -0.4], np.float32)]
    p, m, v = [np.array([2.0, 1.0], np.float32)], [np.zeros(2, np.float32)], [np.zeros(2, np.float32)]
    lo.lans_step(g, p, m, v, 1, mode=0, **kw)
    np.testing.assert_allclose(m[0], [0.55, -0.275], rtol=1e-6)
    np.testing.assert_allclose(v[0], [0.605, 0.15125], rtol=1e-6)
    np.testing.assert_allclose(p[0], [2.0 - 0.15811388300841897, 1.0 + 0.15811388300841897], rtol=1e-6)
    # the same input in mode 1: the moments see the bare scaled gradient, the updates get wd*p:
    # m' = (0.3, -0.4), v' = (0.18, 0.32); u_m = (1/sqrt(2) + 0.5, -1/sqrt(2) + 0.25),
    # u_g = (sqrt(2) + 0.5, -sqrt(2) + 0.25): a different step
    p1, m1, v1 = [np.array([2.0, 1.0], np.float32)], [np.zeros(2, np.float32)], [np.zeros(2, np.float32)]
    lo.lans_step(g, p1, m1, v1, 1, mode=1, **kw)
    np.testing.assert_allclose(m1[0], [0.3, -0.4], rtol=1e-6)
    np.testing.assert_allclose(v1[0], [0.18, 0.32], rtol=1e-6)
    um = np.array([0.7071067811865476 + 0.5, -0.7071067811865476 + 0.25])
    ug = np.array([1.4142135623730951 + 0.5, -1.4142135623730951 + 0.25])
    rm = 0.1 * 2.23606797749979 / np.sqrt((um * um).sum()) * 0.5
    rg = 0.1 * 2.23606797749979 / np.sqrt((ug * ug).sum()) * 0.5
    np.testing.assert_allclose(p1[0], np.array([2.0, 1.0]) - rm * um - rg * ug, rtol=1e-6)
    assert abs(p1[0][0] - p[0][0]) > 1e-3
