"""Pins the oracle to what the mathematics fixes, independently of its own source:
float64 brute force on tiny inputs, torch's convolution and autograd, numpy matmul,
central differences, closed forms. A dropped term, a wrong sign, a transposed operand or
a wrong padding offset fails at least one of these. CPU only."""
import numpy as np
import pytest
import torch

from conftest import assert_close, rel_err


def brute_conv(x, w, b, in_c, in_h, in_w, k, out_c, same, stride):
    """Definition: zero-pad k//2 before the data for padding::same, cross-correlate."""
    batch = x.shape[0]
    x = x.reshape(batch, in_c, in_h, in_w).astype(np.float64)
    w = w.reshape(out_c, in_c, k, k).astype(np.float64)
    if same:
        xp = np.zeros((batch, in_c, in_h + k - 1, in_w + k - 1))
        xp[:, :, k // 2:k // 2 + in_h, k // 2:k // 2 + in_w] = x
        oh, ow = -(-in_h // stride), -(-in_w // stride)
    else:
        xp = x
        oh, ow = -(-(in_h - k + 1) // stride), -(-(in_w - k + 1) // stride)
    y = np.zeros((batch, out_c, oh, ow))
    for n in range(batch):
        for o in range(out_c):
            for yy in range(oh):
                for xx in range(ow):
                    win = xp[n, :, yy * stride:yy * stride + k, xx * stride:xx * stride + k]
                    y[n, o, yy, xx] = np.sum(win * w[o]) + b[o]
    return y, xp


def brute_conv_bwd(xp, w, dy, in_c, in_h, in_w, k, out_c, same, stride):
    batch, _, oh, ow = dy.shape
    w = w.reshape(out_c, in_c, k, k).astype(np.float64)
    dxp = np.zeros_like(xp)
    dw = np.zeros_like(w)
    for n in range(batch):
        for o in range(out_c):
            for yy in range(oh):
                for xx in range(ow):
                    g = dy[n, o, yy, xx]
                    sl = (n, slice(None), slice(yy * stride, yy * stride + k),
                          slice(xx * stride, xx * stride + k))
                    dxp[sl] += g * w[o]
                    dw[o] += g * xp[sl]
    off = k // 2 if same else 0
    dx = dxp[:, :, off:off + in_h, off:off + in_w]
    return dx, dw, dy.sum(axis=(0, 2, 3))


@pytest.mark.parametrize("cfg", [(6, 5, 2, 3, 3, True, 1, 2), (7, 7, 1, 3, 2, False, 2, 2),
                                 (6, 6, 2, 5, 2, True, 1, 1), (7, 6, 2, 3, 2, True, 2, 2)])
def test_conv_against_brute_force(O, cfg):
    in_w, in_h, in_c, k, out_c, same, stride, batch = cfg
    rng = np.random.default_rng(7)
    d = O.conv_desc(in_w, in_h, in_c, k, k, out_c, pad_same=same, w_stride=stride, h_stride=stride)
    ow, oh = O.conv_out_shape(d)
    x = rng.standard_normal((batch, in_c * in_h * in_w)).astype(np.float32)
    w = rng.standard_normal(out_c * in_c * k * k).astype(np.float32)
    b = rng.standard_normal(out_c).astype(np.float32)
    dy = rng.standard_normal((batch, out_c * oh * ow)).astype(np.float32)
    y_ref, xp = brute_conv(x, w, b, in_c, in_h, in_w, k, out_c, same, stride)
    assert y_ref.shape == (batch, out_c, oh, ow)
    assert_close(O.conv2d_fwd(d, x, w, b), y_ref.reshape(batch, -1), 1e-5, "forward")
    dx_ref, dw_ref, db_ref = brute_conv_bwd(xp, w, dy.reshape(batch, out_c, oh, ow).astype(np.float64),
                                            in_c, in_h, in_w, k, out_c, same, stride)
    dx, dw, db = O.conv2d_bwd(d, x, w, dy)
    assert_close(dx, dx_ref.reshape(batch, -1), 1e-5, "dx")
    assert_close(dw, dw_ref.ravel(), 1e-5, "dw")
    assert_close(db, db_ref, 1e-5, "db")


@pytest.mark.parametrize("cfg", [(16, 16, 8, 5, 12, True, 1, 3), (14, 14, 6, 5, 16, False, 1, 2),
                                 (20, 18, 4, 3, 8, True, 1, 2), (15, 15, 3, 3, 5, False, 2, 2)])
def test_conv_against_torch_autograd(O, cfg):
    """Textbook cross-correlation, OIHW weights: torch.nn.functional.conv2d and its autograd."""
    in_w, in_h, in_c, k, out_c, same, stride, batch = cfg
    rng = np.random.default_rng(11)
    d = O.conv_desc(in_w, in_h, in_c, k, k, out_c, pad_same=same, w_stride=stride, h_stride=stride)
    ow, oh = O.conv_out_shape(d)
    x = rng.standard_normal((batch, in_c * in_h * in_w)).astype(np.float32)
    w = rng.standard_normal(out_c * in_c * k * k).astype(np.float32)
    b = rng.standard_normal(out_c).astype(np.float32)
    dy = rng.standard_normal((batch, out_c * oh * ow)).astype(np.float32)
    tx = torch.tensor(x.reshape(batch, in_c, in_h, in_w), dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(w.reshape(out_c, in_c, k, k), dtype=torch.float64, requires_grad=True)
    tb = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    ty = torch.nn.functional.conv2d(tx, tw, tb, stride=stride, padding=k // 2 if same else 0)
    assert tuple(ty.shape) == (batch, out_c, oh, ow)
    ty.backward(torch.tensor(dy.reshape(batch, out_c, oh, ow), dtype=torch.float64))
    assert_close(O.conv2d_fwd(d, x, w, b), ty.detach().numpy().reshape(batch, -1), 1e-5)
    dx, dw, db = O.conv2d_bwd(d, x, w, dy)
    assert_close(dx, tx.grad.numpy().reshape(batch, -1), 1e-5, "dx")
    assert_close(dw, tw.grad.numpy().ravel(), 1e-5, "dw")
    assert_close(db, tb.grad.numpy(), 1e-5, "db")


def test_conv_connection_table_equals_masked_weights(O):
    rng = np.random.default_rng(3)
    tbl = rng.integers(0, 2, (4, 6)).astype(np.uint8)  # [in_c][out_c]
    d_t = O.conv_desc(9, 9, 4, 3, 3, 6, tbl=tbl)
    d_f = O.conv_desc(9, 9, 4, 3, 3, 6)
    x = rng.standard_normal((2, 4 * 81)).astype(np.float32)
    w = rng.standard_normal(6 * 4 * 9).astype(np.float32)
    b = rng.standard_normal(6).astype(np.float32)
    dy = rng.standard_normal((2, 6 * 49)).astype(np.float32)
    mask = np.repeat(tbl.T.reshape(6, 4, 1), 9, axis=2).ravel().astype(np.float32)  # OIHW
    assert_close(O.conv2d_fwd(d_t, x, w, b), O.conv2d_fwd(d_f, x, w * mask, b), 1e-6)
    dx_t, dw_t, db_t = O.conv2d_bwd(d_t, x, w, dy)
    dx_f, dw_f, db_f = O.conv2d_bwd(d_f, x, w * mask, dy)
    assert_close(dx_t, dx_f, 1e-6)
    assert_close(dw_t, dw_f * mask, 1e-6)
    assert np.array_equal(db_t, db_f)


def test_fc_against_numpy(O):
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (9, 53)).astype(np.float32)
    w = rng.uniform(-1, 1, 53 * 31).astype(np.float32)
    b = rng.uniform(-1, 1, 31).astype(np.float32)
    dy = rng.standard_normal((9, 31)).astype(np.float32)
    W2 = w.reshape(53, 31).astype(np.float64)  # [in][out]
    assert_close(O.fc_fwd(x, w, b), x.astype(np.float64) @ W2 + b, 1e-5)
    dx, dw, db = O.fc_bwd(x, w, dy)
    assert_close(dx, dy.astype(np.float64) @ W2.T, 1e-5, "dx")
    assert_close(dw, (x.astype(np.float64).T @ dy).ravel(), 1e-5, "dw = sum over samples, unscaled")
    assert_close(db, dy.astype(np.float64).sum(0), 1e-5, "db")
    dx2, dw2, db2 = O.fc_bwd(x, w, dy, has_bias=False)
    assert db2 is None and np.array_equal(dx, dx2) and np.array_equal(dw, dw2)


def test_maxpool_tie_nan_and_argmax_rules(O):
    d = O.pool_desc(4, 2, 1, 2)
    x = np.array([[5, 5, np.nan, 1,
                   5, 9, np.nan, np.nan]], np.float32)
    y, am = O.maxpool_fwd(d, x)
    assert am[0, 0] == 5 and y[0, 0] == 9           # plain maximum
    assert am[0, 1] == 3 and y[0, 1] == 1           # NaN never wins the strict '>' scan
    x2 = np.array([[7, 7, np.nan, np.nan, 7, 7, np.nan, np.nan]], np.float32)
    y2, am2 = O.maxpool_fwd(d, x2)
    assert am2[0, 0] == 0                            # first of equal maxima (row-major scan)
    assert am2[0, 1] == 0 and y2[0, 1] == np.finfo(np.float32).min   # all-NaN: index 0, lowest()


def test_maxpool_backward_routes_to_argmax_only(O):
    rng = np.random.default_rng(2)
    d = O.pool_desc(8, 6, 3, 2)
    x = rng.standard_normal((4, 3 * 48)).astype(np.float32)
    dy = rng.standard_normal((4, 3 * 12)).astype(np.float32)
    y, am = O.maxpool_fwd(d, x)
    dx = O.maxpool_bwd(d, dy, am)
    want = np.zeros_like(x)
    for s in range(4):
        want[s, am[s]] = dy[s]
    assert np.array_equal(dx, want)
    assert np.array_equal(np.take_along_axis(x, am, 1), y)


def test_avepool_closed_form_and_numeric_gradient(O):
    rng = np.random.default_rng(9)
    c, h, w_, p = 3, 6, 8, 2
    d = O.pool_desc(w_, h, c, p)
    x = rng.standard_normal((2, c * h * w_)).astype(np.float32)
    wt = rng.standard_normal(c).astype(np.float32)
    b = rng.standard_normal(c).astype(np.float32)
    y = O.avepool_fwd(d, x, wt, b)
    x4 = x.reshape(2, c, h // p, p, w_ // p, p).astype(np.float64)
    want = x4.mean(axis=(3, 5)) * wt[None, :, None, None] + b[None, :, None, None]
    assert_close(y, want.reshape(2, -1), 1e-5, "W[c]*mean(window)+b[c]")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx, dw, db = O.avepool_bwd(d, x, wt, dy)
    dy4 = dy.reshape(2, c, h // p, w_ // p).astype(np.float64)
    want_dx = np.repeat(np.repeat(dy4, p, 2), p, 3) * wt[None, :, None, None] / (p * p)
    assert_close(dx, want_dx.reshape(2, -1), 1e-5, "dx")
    assert_close(dw, (x4.mean(axis=(3, 5)) * dy4).sum(axis=(0, 2, 3)), 1e-5, "dw")
    assert_close(db, dy4.sum(axis=(0, 2, 3)), 1e-5, "db")
    # central differences of L = <y, dy> w.r.t. one weight and one input element
    def loss(xx, ww):
        return float((O.avepool_fwd(d, xx, ww, b).astype(np.float64) * dy).sum())
    hstep = 1e-2
    wp, wm = wt.copy(), wt.copy(); wp[1] += hstep; wm[1] -= hstep
    assert abs((loss(x, wp) - loss(x, wm)) / (2 * hstep) - dw[1]) < 1e-2 * max(1, abs(dw[1]))
    xp_, xm_ = x.copy(), x.copy(); xp_[1, 17] += hstep; xm_[1, 17] -= hstep
    assert abs((loss(xp_, wt) - loss(xm_, wt)) / (2 * hstep) - dx[1, 17]) < 1e-2


@pytest.mark.parametrize("kind", ["tanh", "relu", "sigmoid", "softmax"])
def test_activation_closed_forms(O, kind):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((5, 12)).astype(np.float32)
    dy = rng.standard_normal((5, 12)).astype(np.float32)
    x64 = x.astype(np.float64)
    if kind == "tanh":
        y = np.tanh(x64); dx = dy * (1 - y * y)
    elif kind == "relu":
        y = np.maximum(x64, 0); dx = dy * (y > 0)
    elif kind == "sigmoid":
        y = 1 / (1 + np.exp(-x64)); dx = dy * y * (1 - y)
    else:
        e = np.exp(x64 - x64.max(1, keepdims=True)); y = e / e.sum(1, keepdims=True)
        # J^T dy with J_jk = y_j (delta_jk - y_k)
        dx = y * (dy - (dy * y).sum(1, keepdims=True))
    got_y = O.act_fwd(kind, x)
    assert_close(got_y, y, 1e-6, "forward")
    assert_close(O.act_bwd(kind, x, got_y, dy), dx, 1e-5, "backward")


ACT_FORMS = {
    # kind: (params, y(x), dy/dx as a function of (x, y)) in float64; formulas are the textbook ones
    "leaky_relu": ((0.2,), lambda x: np.where(x > 0, x, 0.2 * x), lambda x, y: np.where(x > 0, 1.0, 0.2)),
    "elu": ((0.5,), lambda x: np.where(x < 0, 0.5 * np.expm1(x), x), lambda x, y: np.where(x > 0, 1.0, 0.5 * np.exp(x))),
    "selu": (None, lambda x: 1.05070 * np.where(x > 0, x, 1.67326 * np.expm1(x)),
             lambda x, y: 1.05070 * np.where(x > 0, 1.0, 1.67326 * np.exp(x))),
    "softplus": ((2.0, 5.0), lambda x: np.where(2 * x > 5, x, np.log1p(np.exp(2 * x)) / 2),
                 lambda x, y: np.where(2 * y > 5, 1.0, -np.expm1(-2 * y))),
    "softsign": (None, lambda x: x / (1 + np.abs(x)), lambda x, y: 1 / (1 + np.abs(x)) ** 2),
    "asinh": (None, np.arcsinh, lambda x, y: 1 / np.sqrt(1 + x * x)),
    "tanh_p1m2": (None, lambda x: (np.tanh(x) + 1) / 2, lambda x, y: (1 - np.tanh(x) ** 2) / 2),
}


@pytest.mark.parametrize("kind", sorted(ACT_FORMS))
def test_more_activation_closed_forms(O, kind):
    """Each layer against its textbook definition and derivative in float64 (the derivative as a
    function of x, where the layers compute it from y: a dropped term or wrong sign shows)."""
    prm, f, df = ACT_FORMS[kind]
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((4, 50)) * 2).astype(np.float32)
    x[np.abs(x) < 1e-3] = 0.5
    dy = rng.standard_normal((4, 50)).astype(np.float32)
    x64 = x.astype(np.float64)
    y = O.act_fwd(kind, x, prm)
    assert_close(y, f(x64), 2e-6, "forward")
    assert_close(O.act_bwd(kind, x, y, dy, prm), dy * df(x64, f(x64)), 2e-5, "backward")


def test_activation_layers_match_reference_outputs(O, act_golden):
    """The committed outputs of the compiled reference (tests/golden/make_fixtures.py): bit for bit."""
    g = act_golden
    names = sorted({f.rsplit(".", 1)[0] for f in g.files if "." in f})
    assert len(names) == 14
    for name in names:
        kind, prm = name.split(".", 1)[1], tuple(g[name + ".p"])
        y = O.act_fwd(kind, g["x"], prm)
        assert np.array_equal(y, g[name + ".y"]), name
        assert np.array_equal(O.act_bwd(kind, g["x"], y, g["dy"], prm), g[name + ".dx"]), name


def test_loss_gradients_and_softmax_xent_identity(O):
    rng = np.random.default_rng(6)
    z = rng.standard_normal((7, 10)).astype(np.float32)
    y = O.act_fwd("softmax", z)
    t = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 7)]
    assert_close(O.loss_grad("mse", y, t), 2.0 / 10 * (y.astype(np.float64) - t), 1e-6)
    assert_close(O.loss_grad("ce", y, t), (y.astype(np.float64) - t) / (y * (1.0 - y)), 1e-5)
    dy = O.loss_grad("ce_multiclass", y, t)
    assert_close(dy, -t / y.astype(np.float64), 1e-6)
    dz = O.act_bwd("softmax", z, y, dy)
    assert_close(dz, y.astype(np.float64) - t, 1e-5, "softmax o CE-multiclass = y - t")
    assert np.all(np.abs(dz.sum(1)) < 1e-5)


def test_optimizer_closed_forms_and_adam_per_call_powers(O):
    g = np.array([0.5, -2.0, 3.0], np.float32)
    w0 = np.array([1.0, -1.0, 0.25], np.float32)
    # SGD
    o = O.opt_desc("sgd", alpha=0.1, lambda_=0.5); w = w0.copy()
    O.opt_update(o, g, w)
    assert_close(w, w0 - 0.1 * (g + 0.5 * w0), 1e-6)
    # momentum, two steps
    o = O.opt_desc("momentum", alpha=0.1, mu=0.9); w = w0.copy(); v = np.zeros_like(w)
    O.opt_update(o, g, w, v); O.opt_update(o, g, w, v)
    assert_close(w, w0 - 0.1 * g + (0.9 * (-0.1 * g) - 0.1 * g), 1e-6)
    # Adam: eps inside the square root, bias-correction powers advance once per update() call
    o = O.opt_desc("adam"); w = w0.copy(); m = np.zeros_like(w); s = np.zeros_like(w)
    O.opt_update(o, g, w, m, s)
    g64 = g.astype(np.float64)
    want = w0 - 1e-3 * g64 / np.sqrt(g64 * g64 + 1e-8)
    assert_close(w, want, 1e-6, "first call: m/(1-b1) = g, v/(1-b2) = g^2")
    assert abs(o.b1_t - 0.81) < 1e-7 and abs(o.b2_t - 0.998001) < 1e-7
    # a second TENSOR updated in the same training step sees the advanced powers
    w2 = w0.copy(); m2 = np.zeros_like(w); s2 = np.zeros_like(w)
    O.opt_update(o, g, w2, m2, s2)
    want2 = w0 - 1e-3 * (0.1 * g64 / (1 - 0.81)) / np.sqrt(0.001 * g64 * g64 / (1 - 0.998001) + 1e-8)
    assert_close(w2, want2, 1e-5, "second call uses b1^2, b2^2")
    assert rel_err(w2, want) > 1e-5   # and differs from the textbook per-step schedule


def test_update_weight_feeds_the_sum_not_the_mean(O):
    """layer::update_weight scales by 1/size(weight edge data) = 1 (pinned end to end by the
    compiled-reference fixtures in test_oracle_kats.py); here: the arithmetic of the call."""
    o = O.opt_desc("sgd", alpha=0.5)
    merged = np.array([2.0, -4.0], np.float32)
    w = np.zeros(2, np.float32)
    O.update_weight(o, 1, merged, w)
    assert np.array_equal(w, -0.5 * merged)


# ---------------------------------------------------------------- batch normalization, dropout
def test_mt19937_known_answer(O):
    """std::mt19937 is specified by its 10000th output for the default seed 5489: 4123659995
    (ISO C++ [rand.predef]). The mask generator's engine must reproduce it."""
    lib = O.oracle_lib()
    import ctypes as C
    st = np.zeros(625, np.uint32)
    lib.tdo_mt_seed(st.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_uint32(5489))
    # tdo_dropout_mask draws one word per element: rate 1 accepts every draw, so only the state moves
    mask = np.zeros(9999, np.uint8)
    lib.tdo_dropout_mask(st.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_float(1.0), C.c_size_t(9999),
                         mask.ctypes.data_as(C.POINTER(C.c_uint8)))
    assert mask.all()
    # the 10000th word decides one more element against a threshold just below / above it
    want = np.float32(4123659995) / np.float32(4294967296.0)
    for rate, expect in ((np.nextafter(want, np.float32(0)), 0), (want, 1)):
        s2 = st.copy()
        one = np.zeros(1, np.uint8)
        lib.tdo_dropout_mask(s2.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_float(rate), C.c_size_t(1),
                             one.ctypes.data_as(C.POINTER(C.c_uint8)))
        assert one[0] == expect


def test_batchnorm_closed_forms(O):
    rng = np.random.default_rng(5)
    c, s, b = 6, 40, 10
    x = (rng.standard_normal((b, c * s)) * 3 + 1).astype(np.float32)
    y, mean, var, sd = O.batchnorm_fwd(c, s, x, eps=1e-5)
    xs = x.reshape(b, c, s).astype(np.float64)
    # moments: plain mean, variance over n-1 (util/math_functions.h:57-60)
    np.testing.assert_allclose(mean, xs.mean(axis=(0, 2)), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var, xs.var(axis=(0, 2), ddof=1), rtol=1e-5)
    np.testing.assert_allclose(sd, np.sqrt(var.astype(np.float64) + 1e-5), rtol=1e-6)
    ys = y.reshape(b, c, s).astype(np.float64)
    assert np.abs(ys.mean(axis=(0, 2))).max() < 1e-5
    np.testing.assert_allclose(ys.var(axis=(0, 2), ddof=1), var / (var + 1e-5), rtol=1e-4)
    # backward: a gradient that is constant per channel, or proportional to y, is annihilated
    const = np.repeat(rng.standard_normal(c).astype(np.float32), s)[None].repeat(b, 0)
    assert np.abs(O.batchnorm_bwd(c, s, y, const, sd)).max() < 1e-5
    dy = rng.standard_normal((b, c * s)).astype(np.float32)
    dx = O.batchnorm_bwd(c, s, y, dy, sd).reshape(b, c, s).astype(np.float64)
    assert np.abs(dx.sum(axis=(0, 2))).max() < 1e-3                  # sum of dx is zero
    want = (dy.reshape(b, c, s) - dy.reshape(b, c, s).mean(axis=(0, 2), keepdims=True)
            - (dy.reshape(b, c, s) * ys).mean(axis=(0, 2), keepdims=True) * ys) / sd[None, :, None]
    np.testing.assert_allclose(dx, want, rtol=1e-4, atol=1e-5)
    # one element per channel: variance over max(1, n-1) = 1 is zero, y = 0
    y1, m1, v1, sd1 = O.batchnorm_fwd(3, 1, np.array([[1.0, -2.0, 3.0]], np.float32))
    assert np.array_equal(m1, [1.0, -2.0, 3.0]) and not v1.any() and not y1.any()


def test_dropout_quirks(O):
    """dropout_layer keeps an element when bernoulli(rate) is TRUE, scales the kept ones by
    1/(1-rate) on the way forward and by nothing on the way back (dropout_layer.h:62-113)."""
    x = np.arange(1, 9, dtype=np.float32)[None]
    mask = np.array([[1, 0, 1, 1, 0, 0, 1, 0]], np.uint8)
    y = O.dropout_fwd(mask, x, rate=0.75)
    assert np.array_equal(y, mask * np.float32(4.0) * x)
    assert np.array_equal(O.dropout_fwd(mask, x, rate=0.75, train=False), x)
    assert np.array_equal(O.dropout_bwd(mask, x), mask * x)
    m = O.dropout_mask(1, 0.2, 50, 400)
    assert abs(m.mean() - 0.2) < 0.01          # kept with probability `rate`
    assert np.array_equal(m, O.dropout_mask(1, 0.2, 50, 400)) and not np.array_equal(m, O.dropout_mask(2, 0.2, 50, 400))


def test_norm_layers_match_reference_outputs(O, norm_golden):
    g = norm_golden
    i = 0
    while f"bn{i}.x" in g:
        x, dy = g[f"bn{i}.x"], g[f"bn{i}.dy"]
        c = g[f"bn{i}.mean"].size
        s = x.shape[1] // c
        y, mean, var, sd = O.batchnorm_fwd(c, s, x)
        assert np.array_equal(y, g[f"bn{i}.y"]) and np.array_equal(mean, g[f"bn{i}.mean"])
        assert np.array_equal(var, g[f"bn{i}.var"])
        assert np.array_equal(O.batchnorm_bwd(c, s, y, dy, sd), g[f"bn{i}.dx"])
        yt, _, _, _ = O.batchnorm_fwd(c, s, x, train=False, mean=g[f"bn{i}.m0"], variance=g[f"bn{i}.v0"])
        assert np.array_equal(yt, g[f"bn{i}.y_test"])
        m1, v1 = O.batchnorm_update_moving(0.9, mean, var, g[f"bn{i}.m0"], g[f"bn{i}.v0"])
        # the reference prints the moving averages with 8 significant digits
        np.testing.assert_allclose(m1, g[f"bn{i}.m1"], rtol=2e-7, atol=1e-9)
        np.testing.assert_allclose(v1, g[f"bn{i}.v1"], rtol=2e-7, atol=1e-9)
        i += 1
    assert i == 4
    from tests.golden.make_fixtures import DROPOUT_CASES
    for k, (seed, rate) in enumerate(DROPOUT_CASES):
        mask = O.dropout_mask(seed, rate, *g["do.x"].shape)
        assert np.array_equal(mask, g[f"do{k}.mask"])
        assert np.array_equal(O.dropout_fwd(mask, g["do.x"], rate), g[f"do{k}.y"])
        assert np.array_equal(O.dropout_bwd(mask, g["do.dy"]), g[f"do{k}.dx"])


def test_oracle_refuses_same_padding_with_dilation(O):
    """The reference pads by the undilated window, so its forward loop reads past the padded
    rows when a dilation is set: the oracle restates no result for that case."""
    d = O.conv_desc(8, 8, 2, 3, 3, 4, pad_same=True, w_dilation=2, h_dilation=2)
    x = np.zeros((1, 128), np.float32)
    w = np.zeros(72, np.float32)
    with pytest.raises(RuntimeError, match="code -2"):
        O.conv2d_fwd(d, x, w)
