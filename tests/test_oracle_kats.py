"""The oracle against the known-answer vectors of tiny-dnn's own unit tests
(tests/golden/reference_kats.json) and against the outputs the compiled reference produced
for seeded inputs (tests/golden/*.npz). CPU only."""
import numpy as np
import pytest

from conftest import assert_close, input_checksum


def test_conv_fprop_kat(O, kats):
    k = kats["conv_fprop"]
    d = O.conv_desc(5, 5, 1, 3, 3, 2)
    y = O.conv2d_fwd(d, np.array([k["x"]], np.float32), np.array(k["w"], np.float32),
                     np.zeros(2, np.float32))
    np.testing.assert_allclose(y[0, :9], k["y_first9"], atol=k["tol"])


def test_conv_with_stride_kat(O, kats):
    k = kats["conv_with_stride"]
    d = O.conv_desc(5, 5, 1, 3, 3, 1, w_stride=2, h_stride=2)
    x, w, b = (np.array([k["x"]], np.float32), np.array(k["w"], np.float32),
               np.array(k["b"], np.float32))
    assert np.array_equal(O.conv2d_fwd(d, x, w, b)[0], np.array(k["y"], np.float32))
    dx, dw, db = O.conv2d_bwd(d, x, w, np.array([k["dy"]], np.float32))
    assert np.array_equal(dx[0], np.array(k["dx"], np.float32))
    assert np.array_equal(dw, np.array(k["dw"], np.float32))
    assert np.array_equal(db, np.array(k["db"], np.float32))


def test_conv_with_dilation_kat(O, kats):
    k = kats["conv_with_dilation"]
    d = O.conv_desc(7, 7, 1, 3, 3, 1, w_dilation=2, h_dilation=2)
    x = np.arange(k["x_is_arange"], dtype=np.float32)[None]
    y = O.conv2d_fwd(d, x, np.array(k["w"], np.float32), np.zeros(1, np.float32))
    np.testing.assert_allclose(y[0], k["y"], atol=k["tol"])


def test_fc_forward_kats(O, kats):
    k = kats["fc_forward"]
    w = np.full(k["in"] * k["out"], k["w_const"], np.float32)
    b = np.full(k["out"], k["b_const"], np.float32)
    assert np.array_equal(O.fc_fwd(np.array([k["x"]], np.float32), w, b)[0],
                          np.array(k["y"], np.float32))
    k = kats["fc_forward_nobias"]
    assert np.array_equal(O.fc_fwd(np.array([k["x"]], np.float32), w, None)[0],
                          np.array(k["y"], np.float32))


def test_maxpool_forward_kats(O, kats):
    x = np.array([kats["pool_input_4x4"]], np.float32)
    for k in kats["maxpool_forward"]:
        d = O.pool_desc(4, 4, 1, k["pool"][0], k["pool"][1], k["stride"][0], k["stride"][1],
                        pad_same=k["pad_same"])
        if "out_wh" in k:
            assert list(O.pool_out_shape(d)) == k["out_wh"], k["source"]
        y, _ = O.maxpool_fwd(d, x)
        assert np.array_equal(y[0], np.array(k["y"], np.float32)), k["source"]


def test_maxpool_backward_kat(O, kats):
    k = kats["maxpool_backward"]
    d = O.pool_desc(4, 4, 1, 2)
    _, am = O.maxpool_fwd(d, np.array([kats["pool_input_4x4"]], np.float32))
    dx = O.maxpool_bwd(d, np.array([k["dy"]], np.float32), am)
    assert np.array_equal(dx[0], np.array(k["dx"], np.float32))


def test_avepool_forward_kats(O, kats):
    x = np.array([kats["pool_input_4x4"]], np.float32)
    for k in kats["avepool_forward"]:
        d = O.pool_desc(4, 4, 1, k["pool"], k["pool"], k["stride"], k["stride"])
        y = O.avepool_fwd(d, x, np.ones(1, np.float32), np.zeros(1, np.float32))
        np.testing.assert_allclose(y[0], k["y"], rtol=1.2e-5), k["source"]


def test_optimizer_two_step_kats(O, kats):
    for c in kats["optimizers"]["cases"]:
        o = O.opt_desc(c["kind"])
        w = np.array(c["w"], np.float32)
        g = np.array(c["g"], np.float32)
        s0, s1 = np.zeros_like(w), np.zeros_like(w)
        O.opt_update(o, g, w, s0, s1)
        np.testing.assert_allclose(w, c["first"], atol=kats["optimizers"]["tol"], err_msg=c["kind"])
        O.opt_update(o, g, w, s0, s1)
        np.testing.assert_allclose(w, c["second"], atol=kats["optimizers"]["tol"], err_msg=c["kind"])


# ---- outputs of the compiled reference on seeded inputs (bit-for-bit for the scalar engine)

CONV_CASES = ["conv5x5_same", "conv3x3_same", "conv5x5_valid", "conv3x3_stride2"]


@pytest.mark.parametrize("name", CONV_CASES)
def test_conv_matches_reference_outputs(O, layer_grads, name):
    g = layer_grads
    iw, ih, ic, k, oc, same, stride, batch = [int(v) for v in g[f"{name}.cfg"]]
    d = O.conv_desc(iw, ih, ic, k, k, oc, pad_same=bool(same), w_stride=stride, h_stride=stride)
    x, w, b, dy = g[f"{name}.x"], g[f"{name}.w"], g[f"{name}.b"], g[f"{name}.dy"]
    assert np.array_equal(O.conv2d_fwd(d, x, w, b), g[f"{name}.y"])
    dx, dw, db = O.conv2d_bwd(d, x, w, dy)
    assert np.array_equal(dx, g[f"{name}.internal.dx"])
    assert np.array_equal(dw, g[f"{name}.internal.dw"])
    assert np.array_equal(db, g[f"{name}.internal.db"])
    # the AVX engine sums in another order: same result within the path's tolerance
    assert_close(dx, g[f"{name}.avx.dx"], what="dx vs avx engine")
    assert_close(dw, g[f"{name}.avx.dw"], what="dw vs avx engine")
    assert_close(db, g[f"{name}.avx.db"], what="db vs avx engine")


def test_fc_matches_reference_outputs(O, layer_grads):
    g = layer_grads
    assert np.array_equal(O.fc_fwd(g["fc.x"], g["fc.w"], g["fc.b"]), g["fc.y"])
    dx, dw, db = O.fc_bwd(g["fc.x"], g["fc.w"], g["fc.dy"])
    assert np.array_equal(dx, g["fc.internal.dx"])
    assert np.array_equal(dw, g["fc.internal.dw"])
    assert np.array_equal(db, g["fc.internal.db"])
    assert_close(dx, g["fc.avx.dx"])
    assert_close(dw, g["fc.avx.dw"])


@pytest.mark.parametrize("name", ["maxpool2x2", "maxpool3x3s2", "maxpool_same_s1", "maxpool_ceil",
                                  "maxpool_gap"])
def test_maxpool_matches_reference_outputs(O, layer_grads, name):
    g = layer_grads
    d = O.pool_desc(*[int(v) for v in g[f"{name}.cfg"]])
    y, am = O.maxpool_fwd(d, g[f"{name}.x"])
    assert np.array_equal(y, g[f"{name}.y"])
    assert np.array_equal(O.maxpool_bwd(d, g[f"{name}.dy"], am), g[f"{name}.dx"])


@pytest.mark.parametrize("name", ["avepool2", "avepool2s1", "avepool3"])
def test_avepool_matches_reference_outputs(O, layer_grads, name):
    g = layer_grads
    iw, ih, c, p, s = [int(v) for v in g[f"{name}.cfg"]]
    d = O.pool_desc(iw, ih, c, p, p, s, s)
    assert np.array_equal(O.avepool_fwd(d, g[f"{name}.x"], g[f"{name}.w"], g[f"{name}.b"]),
                          g[f"{name}.y"])
    dx, dw, db = O.avepool_bwd(d, g[f"{name}.x"], g[f"{name}.w"], g[f"{name}.dy"])
    assert np.array_equal(dx, g[f"{name}.dx"])
    assert np.array_equal(dw, g[f"{name}.dw"])
    assert np.array_equal(db, g[f"{name}.db"])


@pytest.mark.parametrize("key", ["lenet5_b16", "cifar10_cnn_b128", "cifar10_cnn_b128@128", "lenet5_mnist_b16"])
def test_net_steps_match_reference_fit(O, W, net_steps, key):
    """Parameters after network<sequential>::fit steps of the compiled reference."""
    g = net_steps
    name, key_full = key.split("@")[0], key
    g = {k.replace(key_full + ".", name + ".", 1): g[k] for k in g.files if k.startswith(key_full + ".")}
    batch, steps, stride = int(g[f"{name}.batch"]), int(g[f"{name}.steps"]), int(g[f"{name}.stride"])
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
    assert input_checksum(x, t, params) == float(g[f"{name}.input_checksum"]), \
        "seeded inputs drifted from the ones the fixture was made with"
    net = O.OracleNet(W.build_layers(O, spec), batch)
    for (i, which, a) in params:
        (net.weight(i) if which == 0 else net.bias(i))[:] = a
    opt = O.opt_desc(opt_kind, **opt_kw)
    for _ in range(steps):
        net.train_step(opt, loss, x, t)
    for (i, which, a) in params:
        got = net.weight(i) if which == 0 else net.bias(i)
        assert np.array_equal(got[::stride], g[f"{name}.p{i}.{which}"]), (name, i, which)
        assert float(got.astype(np.float64).sum()) == float(g[f"{name}.p{i}.{which}.sum"])
