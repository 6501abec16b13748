"""Live comparison of the oracle with the compiled reference (oracle/_ref, built from the
unmodified tiny-dnn headers). Bit-for-bit against the scalar build; within the path's
tolerance against the OpenMP+AVX build. Skipped where the reference is not built."""
import numpy as np
import pytest

from conftest import assert_close


@pytest.fixture(scope="module")
def ref(O):
    if O.ref_lib("scalar") is None:
        pytest.skip("oracle/_ref not built (the tiny-dnn tree is not on this machine)")
    return O


CONV = [(5, 5, 1, 3, 1, False, 2, 1), (12, 10, 3, 3, 4, True, 1, 3), (9, 9, 2, 5, 3, True, 2, 2),
        (32, 32, 1, 5, 6, False, 1, 4), (16, 16, 8, 5, 8, True, 1, 2), (11, 7, 3, 3, 5, True, 1, 5)]


@pytest.mark.parametrize("cfg", CONV)
def test_conv_bit_exact(ref, cfg):
    O = ref
    iw, ih, ic, k, oc, same, st, bs = cfg
    rng = np.random.default_rng(hash(cfg) % 2**31)
    d = O.conv_desc(iw, ih, ic, k, k, oc, pad_same=same, w_stride=st, h_stride=st)
    ow, oh = O.conv_out_shape(d)
    x = rng.standard_normal((bs, ic * ih * iw)).astype(np.float32)
    w = rng.standard_normal(oc * ic * k * k).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    dy = rng.standard_normal((bs, oc * oh * ow)).astype(np.float32)
    assert np.array_equal(O.conv2d_fwd(d, x, w, b), O.ref_conv2d_fwd(d, x, w, b))
    for got, want in zip(O.conv2d_bwd(d, x, w, dy), O.ref_conv2d_bwd(d, x, w, dy)):
        assert np.array_equal(got, want)
    if O.ref_lib("avx") is not None:
        for got, want in zip(O.conv2d_bwd(d, x, w, dy), O.ref_conv2d_bwd(d, x, w, dy, "avx", 1)):
            assert_close(got, want, what="vs AVX engine")


def test_conv_connection_table_bit_exact(ref):
    O = ref
    rng = np.random.default_rng(8)
    tbl = rng.integers(0, 2, (6, 16)).astype(np.uint8)
    d = O.conv_desc(14, 14, 6, 5, 5, 16, tbl=tbl)
    x = rng.standard_normal((3, 6 * 196)).astype(np.float32)
    w = rng.standard_normal(16 * 6 * 25).astype(np.float32)
    b = rng.standard_normal(16).astype(np.float32)
    dy = rng.standard_normal((3, 16 * 100)).astype(np.float32)
    assert np.array_equal(O.conv2d_fwd(d, x, w, b), O.ref_conv2d_fwd(d, x, w, b))
    for got, want in zip(O.conv2d_bwd(d, x, w, dy), O.ref_conv2d_bwd(d, x, w, dy)):
        assert np.array_equal(got, want)


def test_fc_pool_act_loss_opt_bit_exact(ref):
    O = ref
    rng = np.random.default_rng(12)
    x = rng.standard_normal((5, 37)).astype(np.float32)
    w = rng.standard_normal(37 * 19).astype(np.float32)
    b = rng.standard_normal(19).astype(np.float32)
    dy = rng.standard_normal((5, 19)).astype(np.float32)
    assert np.array_equal(O.fc_fwd(x, w, b), O.ref_fc_fwd(x, w, b))
    for got, want in zip(O.fc_bwd(x, w, dy), O.ref_fc_bwd(x, w, dy)):
        assert np.array_equal(got, want)
    for cfg in [(4, 4, 1, 2, 2, 2, 2, 0, 0), (7, 7, 2, 2, 2, 2, 2, 0, 1), (4, 4, 1, 2, 2, 1, 1, 1, 0),
                (9, 8, 3, 3, 3, 2, 2, 0, 0), (6, 6, 2, 2, 2, 3, 3, 0, 0)]:
        d = O.pool_desc(*cfg)
        ow, oh = O.pool_out_shape(d)
        xi = rng.integers(-3, 4, (3, cfg[2] * cfg[1] * cfg[0])).astype(np.float32)
        g = rng.standard_normal((3, cfg[2] * oh * ow)).astype(np.float32)
        y, am = O.maxpool_fwd(d, xi)
        yr, dxr = O.ref_maxpool_fwd_bwd(d, xi, g)
        assert np.array_equal(y, yr) and np.array_equal(O.maxpool_bwd(d, g, am), dxr)
    for kind in ("tanh", "relu", "softmax", "sigmoid"):
        xa = rng.standard_normal((4, 10)).astype(np.float32)
        g = rng.standard_normal((4, 10)).astype(np.float32)
        y = O.act_fwd(kind, xa)
        yr, dxr = O.ref_act(kind, xa, g)
        assert np.array_equal(y, yr) and np.array_equal(O.act_bwd(kind, xa, y, g), dxr)
    for kind, prm in (("leaky_relu", None), ("leaky_relu", (0.3,)), ("elu", (0.7,)), ("selu", None),
                      ("selu", (1.2, 0.9)), ("softplus", None), ("softplus", (3.0, 4.0)),
                      ("softsign", None), ("asinh", None), ("tanh_p1m2", None)):
        xa = (rng.standard_normal((4, 33)) * 3).astype(np.float32)
        g = rng.standard_normal((4, 33)).astype(np.float32)
        y = O.act_fwd(kind, xa, prm)
        yr, dxr = O.ref_act(kind, xa, g, params=prm)
        assert np.array_equal(y, yr) and np.array_equal(O.act_bwd(kind, xa, y, g, prm), dxr), kind
    y = O.act_fwd("softmax", rng.standard_normal((4, 10)).astype(np.float32))
    t = np.eye(10, dtype=np.float32)[[1, 3, 5, 7]]
    for kind in ("mse", "ce_multiclass", "ce"):
        assert np.array_equal(O.loss_grad(kind, y, t), O.ref_loss_grad(kind, y, t))
    for kind in O.OPT:
        o, o2 = O.opt_desc(kind), O.opt_desc(kind)
        w0 = rng.standard_normal(17).astype(np.float32)
        g = rng.standard_normal(17).astype(np.float32)
        want = O.ref_opt_updates(o2, g, w0, 3)
        w1, s0, s1 = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
        for _ in range(3):
            O.opt_update(o, g, w1, s0, s1)
        assert np.array_equal(w1, want), kind


def test_vgg_style_step_bit_exact(ref, W):
    """A shrunken VGG stack (16x16 input, batch 2): one momentum SGD step through fit().
    (A second step already overflows in the reference itself: its update uses the gradient
    summed over the batch, and softmax outputs that underflow to 0 turn -t/y into NaN.)"""
    O = ref
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("vgg_stack_b64", batch=2, size=16)
    net = O.OracleNet(W.build_layers(O, spec), batch)
    rn = O.RefNet(W.build_layers(O, spec), "scalar", 0)
    for (i, which, a) in params:
        (net.weight(i) if which == 0 else net.bias(i))[:] = a
        rn.set_param(i, which, a)
    o, o2 = O.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
    net.train_step(o, loss, x, t)
    rn.fit(o2, loss, x, t, 1)
    for (i, which, a) in params:
        got = net.weight(i) if which == 0 else net.bias(i)
        assert np.all(np.isfinite(got))
        assert np.array_equal(got, rn.get_param(i, which)[:a.size]), (i, which)


@pytest.mark.parametrize("shape", [(5, 7, 4), (3, 100, 9), (16, 64, 32), (4, 1, 1), (2, 3, 1)])
def test_batchnorm_bit_exact(ref, shape):
    O = ref
    c, s, b = shape
    rng = np.random.default_rng(c * 1000 + s)
    x = (rng.standard_normal((b, c * s)) * 2 + 0.5).astype(np.float32)
    dy = rng.standard_normal((b, c * s)).astype(np.float32)
    y, mean, var, sd = O.batchnorm_fwd(c, s, x)
    ry, rmean, rvar, rdx = O.ref_batchnorm(c, s, x, dy)
    assert np.array_equal(y, ry) and np.array_equal(mean, rmean) and np.array_equal(var, rvar)
    assert np.array_equal(O.batchnorm_bwd(c, s, y, dy, sd), rdx)
    m0, v0 = rng.standard_normal(c).astype(np.float32), rng.uniform(0.5, 2, c).astype(np.float32)
    yt = O.batchnorm_fwd(c, s, x, train=False, mean=m0, variance=v0)[0]
    assert np.array_equal(yt, O.ref_batchnorm(c, s, x, train=False, mean=m0, variance=v0)[0])
    m1, v1 = O.batchnorm_update_moving(0.9, mean, var, m0, v0)
    rm1, rv1 = O.ref_batchnorm_post_update(c, s, x, m0, v0, momentum=0.9)
    np.testing.assert_allclose(m1, rm1, rtol=2e-7, atol=1e-9)   # read back through the text format
    np.testing.assert_allclose(v1, rv1, rtol=2e-7, atol=1e-9)


@pytest.mark.parametrize("seed,rate", [(1, 0.3), (7, 0.5), (3, 0.9), (11, 0.0)])
def test_dropout_bit_exact(ref, seed, rate):
    O = ref
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((9, 333)).astype(np.float32)
    dy = rng.standard_normal((9, 333)).astype(np.float32)
    mask = O.dropout_mask(seed, rate, 9, 333)
    rmask, ry, rdx = O.ref_dropout(x, dy, rate, seed)
    assert np.array_equal(mask, rmask)
    assert np.array_equal(O.dropout_fwd(mask, x, rate), ry)
    assert np.array_equal(O.dropout_bwd(mask, dy), rdx)


@pytest.mark.parametrize("name,batch,steps", [("lenet5_mnist_b16", 16, 2), ("cifar10_cnn_b128", 128, 2)])
def test_example_nets_fit_bit_exact(ref, W, name, batch, steps):
    """The MNIST example's LeNet-5 (C3 with its connection table, adagrad) and the CIFAR-10 net
    at the batch it is benchmarked at: the oracle's steps equal network<sequential>::fit bit
    for bit."""
    O = ref
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
    net = O.OracleNet(W.build_layers(O, spec), batch)
    rn = O.RefNet(W.build_layers(O, spec), "scalar", 0)
    for (i, which, a) in params:
        (net.weight(i) if which == 0 else net.bias(i))[:] = a
        rn.set_param(i, which, a)
    o, o2 = O.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
    for _ in range(steps):
        net.train_step(o, loss, x, t)
    rn.fit(o2, loss, x, t, steps)
    for (i, which, a) in params:
        got = net.weight(i) if which == 0 else net.bias(i)
        assert not np.array_equal(got, a) or which == 1
        assert np.array_equal(got, rn.get_param(i, which)[:a.size]), (i, which)


def test_net_with_batchnorm_and_dropout_fit_bit_exact(ref, W):
    """conv -> batch-norm -> relu -> pool -> fc -> tanh -> dropout -> fc -> softmax: three Adam
    steps of network<sequential>::fit after set_random_seed (the dropout masks are drawn from
    the reference's generator in forward order) against the oracle's net, which is handed the
    masks drawn by the restated generator; weights and the batch-norm running averages."""
    O = ref
    params, x, t = W.bn_dropout_case()
    batch, steps, seed = x.shape[0], 3, 5
    net = O.OracleNet(W.build_layers(O, W.BN_DROPOUT_NET), batch)
    rn = O.RefNet(W.build_layers(O, W.BN_DROPOUT_NET), "scalar", 0)
    for (i, which, a) in params:
        (net.weight(i) if which == 0 else net.bias(i))[:] = a
        rn.set_param(i, which, a)
    o, o2 = O.opt_desc("adam"), O.opt_desc("adam")
    state = np.zeros(625, np.uint32)
    O.mt_seed(state, seed)
    for _ in range(steps):
        net.set_dropout_mask(6, O.dropout_mask(seed, 0.4, batch, 20, state))
        net.train_step(o, "ce_multiclass", x, t)
    rn.set_random_seed(seed)
    rn.fit(o2, "ce_multiclass", x, t, steps)
    for (i, which, a) in params:
        got = net.weight(i) if which == 0 else net.bias(i)
        assert np.array_equal(got, rn.get_param(i, which)[:a.size]), (i, which)
    for which in (0, 1):   # read back through the reference's text format: 8 significant digits
        np.testing.assert_allclose(net.bn_stat(1, which), rn.bn_stat(1, which, 6), rtol=2e-7, atol=1e-9)
