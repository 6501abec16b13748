"""Parity of every operator of the hot path, called through the C ABI on the MI355X, with
the CPU oracle on identical seeded inputs, and with the outputs tiny-dnn itself produced
(tests/golden/layer_grads.npz). Floating point: max relative error 1e-4 (conftest.rel_err);
max-pool argmax indices and routed gradients: bit-exact."""
import ctypes as C

import numpy as np
import pytest

from conftest import assert_close, REL_TOL

pytestmark = pytest.mark.gpu


def run_conv(T, d, x, w, b, dy, accumulate=False, dw0=None):
    bs = x.shape[0]
    ow, oh = T.conv_out_shape(d)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    bd = T.to_device(b) if b is not None else None
    y = T.DevBuf((bs, d.out_c * oh * ow))
    dx = T.DevBuf(x.shape)
    dw = T.to_device(dw0) if dw0 is not None else T.DevBuf(w.shape)
    db = T.DevBuf((d.out_c,), zero=True)
    T.conv2d_fwd(d, bs, xd, wd, bd, y)
    T.conv2d_bwd(d, bs, xd, wd, dyd, dx, dw, db if d.has_bias else None, accumulate)
    return y.numpy(), dx.numpy(), dw.numpy(), db.numpy()


CONV = [
    # in_w, in_h, in_c, k, out_c, same, stride, batch
    (5, 5, 1, 3, 1, False, 2, 1), (12, 10, 3, 3, 4, True, 1, 3), (9, 9, 2, 5, 3, True, 2, 2),
    (32, 32, 1, 5, 6, False, 1, 16), (14, 14, 6, 5, 16, False, 1, 16), (5, 5, 16, 5, 120, False, 1, 16),
    (32, 32, 3, 5, 32, True, 1, 8), (16, 16, 32, 5, 32, True, 1, 8), (8, 8, 32, 5, 64, True, 1, 8),
    (24, 24, 32, 3, 64, True, 1, 4), (17, 13, 5, 3, 7, True, 1, 3), (11, 11, 4, 3, 6, False, 3, 2),
    (33, 31, 3, 3, 130, True, 1, 2), (16, 16, 64, 3, 128, True, 1, 2), (7, 7, 3, 7, 5, False, 1, 1),
    # LDS-staged dW kernel: ragged widths, partial channel blocks, valid padding, column tiles
    (13, 11, 16, 3, 40, True, 1, 3), (18, 18, 20, 5, 24, False, 1, 2), (70, 9, 33, 3, 65, True, 1, 2),
    (12, 12, 48, 5, 16, True, 1, 5), (40, 6, 16, 3, 16, False, 1, 1),
    # 5x5 windows split by filter row: stacked small images with a ragged last chunk, row chunks
    (10, 10, 16, 5, 40, True, 1, 7), (36, 36, 16, 5, 16, False, 1, 2), (8, 8, 32, 5, 64, True, 1, 11),
    # 5x5 windows on 8x8 images, all filter rows in one workgroup (four tap groups, four images a
    # chunk): a last chunk of two images, several channel blocks either way, several chunks a slice
    (8, 8, 64, 5, 96, True, 1, 6), (8, 8, 64, 5, 96, True, 1, 130), (8, 8, 32, 5, 32, True, 1, 4),
    # stride-1 MFMA kernel with scalar loads: rows or channel counts that are not multiples of 4,
    # a last chunk of reduction channels that is not full
    (26, 26, 16, 3, 32, True, 1, 32), (14, 14, 16, 5, 32, True, 1, 64), (16, 16, 16, 3, 30, True, 1, 64),
    # direct small-Cin forward kernel: ragged tiles, one and two channel blocks
    (20, 17, 3, 3, 40, True, 1, 3), (23, 22, 1, 5, 33, False, 1, 2), (37, 9, 3, 5, 64, True, 1, 2),
    # small-Cin dW + db kernel: strides, several bands with a ragged last one, partial and
    # several output-channel tiles, one to three column tiles
    (16, 16, 3, 3, 8, True, 2, 4), (19, 14, 2, 5, 33, False, 2, 3), (64, 64, 3, 5, 16, True, 1, 2),
    (32, 37, 3, 3, 70, True, 1, 5), (32, 32, 3, 5, 32, True, 1, 128), (28, 28, 2, 5, 6, True, 1, 40),
    # first-layer dX on the matrix cores (output rows of 16, 32 or 64): a ragged last band, one
    # to four input channels, one output channel and two chunks of them, valid padding, and an
    # image with fewer rows than a band (the vector-ALU kernel takes that one)
    (16, 19, 4, 3, 40, True, 1, 3), (36, 20, 3, 5, 33, False, 1, 2), (64, 9, 2, 3, 1, True, 1, 2),
    (18, 7, 1, 3, 70, False, 1, 4), (64, 3, 3, 3, 8, True, 1, 2), (20, 12, 2, 5, 6, False, 1, 5),
]


@pytest.mark.parametrize("cfg", CONV)
def test_conv_fwd_bwd_matches_oracle(T, O, cfg):
    iw, ih, ic, k, oc, same, st, bs = cfg
    rng = np.random.default_rng(abs(hash(cfg)) % 2**31)
    d = T.conv_desc(iw, ih, ic, k, k, oc, pad_same=same, w_stride=st, h_stride=st)
    do = O.conv_desc(iw, ih, ic, k, k, oc, pad_same=same, w_stride=st, h_stride=st)
    ow, oh = T.conv_out_shape(d)
    assert (ow, oh) == O.conv_out_shape(do)
    x = rng.standard_normal((bs, ic * ih * iw)).astype(np.float32)
    w = rng.uniform(-0.3, 0.3, oc * ic * k * k).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    dy = rng.standard_normal((bs, oc * oh * ow)).astype(np.float32)
    y, dx, dw, db = run_conv(T, d, x, w, b, dy)
    assert_close(y, O.conv2d_fwd(do, x, w, b), what="y")
    rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
    assert_close(dx, rdx, what="dx")
    assert_close(dw, rdw, what="dw")
    assert_close(db, rdb, what="db")


def test_conv_reference_kat_with_stride(T, kats):
    k = kats["conv_with_stride"]
    d = T.conv_desc(5, 5, 1, 3, 3, 1, w_stride=2, h_stride=2)
    y, dx, dw, db = run_conv(T, d, np.array([k["x"]], np.float32), np.array(k["w"], np.float32),
                             np.array(k["b"], np.float32), np.array([k["dy"]], np.float32))
    assert np.array_equal(y[0], np.array(k["y"], np.float32))
    assert np.array_equal(dx[0], np.array(k["dx"], np.float32))
    assert np.array_equal(dw, np.array(k["dw"], np.float32))
    assert np.array_equal(db, np.array(k["db"], np.float32))


def test_conv_reference_kats_forward(T, kats):
    k = kats["conv_fprop"]
    d = T.conv_desc(5, 5, 1, 3, 3, 2, has_bias=False)
    y = T.DevBuf((1, 18))
    T.conv2d_fwd(d, 1, T.to_device(np.array([k["x"]], np.float32)),
                 T.to_device(np.array(k["w"], np.float32)), None, y)
    np.testing.assert_allclose(y.numpy()[0, :9], k["y_first9"], atol=k["tol"])
    k = kats["conv_with_dilation"]
    d = T.conv_desc(7, 7, 1, 3, 3, 1, has_bias=False, w_dilation=2, h_dilation=2)
    y = T.DevBuf((1, 9))
    T.conv2d_fwd(d, 1, T.to_device(np.arange(49, dtype=np.float32)[None]),
                 T.to_device(np.array(k["w"], np.float32)), None, y)
    np.testing.assert_allclose(y.numpy()[0], k["y"], atol=1e-3)


@pytest.mark.parametrize("name", ["conv5x5_same", "conv3x3_same", "conv5x5_valid", "conv3x3_stride2"])
def test_conv_matches_reference_outputs(T, layer_grads, name):
    g = layer_grads
    iw, ih, ic, k, oc, same, stride, batch = [int(v) for v in g[f"{name}.cfg"]]
    d = T.conv_desc(iw, ih, ic, k, k, oc, pad_same=bool(same), w_stride=stride, h_stride=stride)
    y, dx, dw, db = run_conv(T, d, g[f"{name}.x"], g[f"{name}.w"], g[f"{name}.b"], g[f"{name}.dy"])
    assert_close(y, g[f"{name}.y"], what="y")
    for eng in ("internal", "avx"):
        assert_close(dx, g[f"{name}.{eng}.dx"], what=f"dx vs {eng}")
        assert_close(dw, g[f"{name}.{eng}.dw"], what=f"dw vs {eng}")
        assert_close(db, g[f"{name}.{eng}.db"], what=f"db vs {eng}")


def test_conv_connection_table(T, O):
    rng = np.random.default_rng(21)
    tbl = rng.integers(0, 2, (6, 16)).astype(np.uint8)
    d, do = T.conv_desc(14, 14, 6, 5, 5, 16, tbl=tbl), O.conv_desc(14, 14, 6, 5, 5, 16, tbl=tbl)
    x = rng.standard_normal((4, 6 * 196)).astype(np.float32)
    w = rng.uniform(-0.3, 0.3, 16 * 6 * 25).astype(np.float32)
    b = rng.standard_normal(16).astype(np.float32)
    dy = rng.standard_normal((4, 1600)).astype(np.float32)
    y, dx, dw, db = run_conv(T, d, x, w, b, dy)
    assert_close(y, O.conv2d_fwd(do, x, w, b))
    rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
    assert_close(dx, rdx); assert_close(dw, rdw); assert_close(db, rdb)
    # unconnected pairs get exactly zero gradient
    mask = np.repeat(tbl.T.reshape(16, 6, 1), 25, axis=2).ravel()
    assert np.all(dw[mask == 0] == 0.0)


def test_conv_accumulate_and_skipped_outputs(T, O):
    """dW/db are added to when accumulate=1 (the reference's += between clear_grads calls);
    NULL outputs are skipped; dX is always overwritten."""
    rng = np.random.default_rng(22)
    d, do = T.conv_desc(10, 10, 3, 3, 3, 5, pad_same=True), O.conv_desc(10, 10, 3, 3, 3, 5, pad_same=True)
    x = rng.standard_normal((3, 300)).astype(np.float32)
    w = rng.standard_normal(135).astype(np.float32)
    dy = rng.standard_normal((3, 500)).astype(np.float32)
    dw0 = rng.standard_normal(135).astype(np.float32)
    _, dx, dw, db = run_conv(T, d, x, w, np.zeros(5, np.float32), dy, accumulate=True, dw0=dw0)
    rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
    assert_close(dw, rdw + dw0); assert_close(dx, rdx); assert_close(db, rdb)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    dxb = T.to_device(np.full((3, 300), 7.0, np.float32))
    T.conv2d_bwd(d, 3, xd, wd, dyd, dxb, None, None)
    assert_close(dxb.numpy(), rdx)
    dwb = T.DevBuf((135,))
    T.conv2d_bwd(d, 3, xd, wd, dyd, None, dwb, None)
    assert_close(dwb.numpy(), rdw)


@pytest.mark.parametrize("hw,bs,ic,oc", [(8, 9, 32, 64), (16, 97, 32, 32), (16, 128, 64, 32)])
def test_conv_weight_gradient_of_whole_images_options(T, O, hw, bs, ic, oc):
    """The dW kernel that stages whole 8x8 or 16x16 images (the latter from batch 96 on): added to
    a previous value, without a bias gradient, without dX, twice with equal bits; tensors that
    are not 16-byte aligned take the general kernel."""
    rng = np.random.default_rng(88 + hw + bs)
    d, do = T.conv_desc(hw, hw, ic, 5, 5, oc, pad_same=True), O.conv_desc(hw, hw, ic, 5, 5, oc, pad_same=True)
    x = rng.standard_normal((bs, ic * hw * hw)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, oc * ic * 25).astype(np.float32)
    dy = rng.standard_normal((bs, oc * hw * hw)).astype(np.float32)
    dw0 = rng.standard_normal(w.size).astype(np.float32)
    rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    dw, db = T.to_device(dw0), T.DevBuf((oc,), zero=True)
    T.conv2d_bwd(d, bs, xd, wd, dyd, None, dw, db, True)
    assert_close(dw.numpy(), rdw + dw0, what="dw added to a previous value")
    assert_close(db.numpy(), rdb, what="db")
    first = T.DevBuf(w.shape)
    T.conv2d_bwd(d, bs, xd, wd, dyd, None, first, None)
    assert_close(first.numpy(), rdw, what="dw alone")
    again = T.to_device(np.full(w.shape, np.nan, np.float32))
    T.conv2d_bwd(d, bs, xd, wd, dyd, None, again, None)
    assert np.array_equal(first.numpy(), again.numpy())
    # the same tensors one float further on in memory
    xs, dys = T.DevBuf((x.size + 4,)), T.DevBuf((dy.size + 4,))
    xs.upload(np.concatenate([np.zeros(1, np.float32), x.ravel(), np.zeros(3, np.float32)]))
    dys.upload(np.concatenate([np.zeros(1, np.float32), dy.ravel(), np.zeros(3, np.float32)]))
    xo = T.DevBuf.view(xs.ptr.value + 4, x.shape)
    dyo = T.DevBuf.view(dys.ptr.value + 4, dy.shape)
    shifted, dbs = T.DevBuf(w.shape), T.DevBuf((oc,))
    T.conv2d_bwd(d, bs, xo, wd, dyo, None, shifted, dbs)
    assert_close(shifted.numpy(), rdw, what="dw of unaligned tensors")
    assert_close(dbs.numpy(), rdb, what="db of unaligned tensors")


@pytest.mark.parametrize("w_,h_,c_,k_,oc_,same,batch", [
    (32, 32, 3, 5, 32, True, 128),    # the CIFAR net's first layer
    (32, 32, 3, 5, 20, True, 80),     # 20 of 32 output channels, a batch that is no multiple of anything
    (36, 36, 3, 5, 32, False, 64),    # no padding: 32 x 32 outputs under 36 input rows, five bands
    (32, 20, 3, 3, 16, True, 96),     # 3x3, a last band of four rows
    (16, 16, 1, 5, 8, True, 256),     # one input channel, rows of 16, one band an image
])
def test_first_conv_gradients_from_one_launch(T, O, w_, h_, c_, k_, oc_, same, batch):
    """dX, dW and db of a first convolution (few input channels, at most 32 output channels, a
    workgroup for every compute unit) leave one launch when they are asked for together: each
    against the oracle, the same bits as the three asked for one by one, and dW / db added to a
    previous value."""
    rng = np.random.default_rng(w_ * 7 + h_ + c_ + k_ + oc_)
    d, do = T.conv_desc(w_, h_, c_, k_, k_, oc_, pad_same=same), O.conv_desc(w_, h_, c_, k_, k_, oc_, pad_same=same)
    ow, oh = (w_, h_) if same else (w_ - k_ + 1, h_ - k_ + 1)
    x = rng.standard_normal((batch, c_ * w_ * h_)).astype(np.float32)
    w = rng.uniform(-0.2, 0.2, oc_ * c_ * k_ * k_).astype(np.float32)
    dy = rng.standard_normal((batch, oc_ * ow * oh)).astype(np.float32)
    rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    dx, dw, db = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc_,))
    T.conv2d_bwd(d, batch, xd, wd, dyd, dx, dw, db)
    assert_close(dx.numpy(), rdx, what="dX"); assert_close(dw.numpy(), rdw, what="dW"); assert_close(db.numpy(), rdb, what="db")
    dx1, dw1, db1 = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc_,))
    T.conv2d_bwd(d, batch, xd, wd, dyd, dx1, None, None)
    T.conv2d_bwd(d, batch, xd, wd, dyd, None, dw1, db1)
    assert np.array_equal(dx.numpy(), dx1.numpy()), "dX alone"
    assert np.array_equal(dw.numpy(), dw1.numpy()), "dW without dX"
    assert np.array_equal(db.numpy(), db1.numpy()), "db without dX"
    dw0 = rng.standard_normal(w.size).astype(np.float32)
    dw2, dx2 = T.to_device(dw0), T.to_device(np.full(x.shape, np.nan, np.float32))
    T.conv2d_bwd(d, batch, xd, wd, dyd, dx2, dw2, None, True)     # no bias gradient, added to dw0
    assert_close(dw2.numpy(), rdw + dw0, what="dW added to a previous value")
    assert np.array_equal(dx2.numpy(), dx.numpy())


def test_conv_errors_and_empty_batch(T):
    d = T.conv_desc(8, 8, 2, 3, 3, 4, w_dilation=2, h_dilation=2)
    buf = T.DevBuf((16,))
    with pytest.raises(T.TdhError, match="dilation"):
        T.conv2d_bwd(d, 1, buf, buf, buf, buf, buf, buf)
    same_dilated = T.conv_desc(8, 8, 2, 3, 3, 4, pad_same=True, w_dilation=2, h_dilation=2)
    with pytest.raises(T.TdhError, match="padding::same and dilation"):
        T.conv2d_fwd(same_dilated, 1, buf, buf, buf, buf)
    bad = T.conv_desc(2, 2, 1, 3, 3, 1)
    with pytest.raises(T.TdhError, match="window larger"):
        T.conv2d_fwd(bad, 1, buf, buf, buf, buf)
    ok = T.conv_desc(8, 8, 2, 3, 3, 4)
    T.conv2d_fwd(ok, 0, None, None, None, None)          # empty batch: nothing to do
    with pytest.raises(T.TdhError, match="null"):
        T.conv2d_fwd(ok, 1, None, buf, buf, buf)


FC = [(1, 4, 2, True), (5, 37, 19, True), (16, 120, 10, True), (128, 1024, 64, True),
      (64, 300, 257, False), (256, 512, 384, True), (3, 2048, 40, True), (130, 70, 1000, True)]


@pytest.mark.parametrize("cfg", FC)
def test_fc_fwd_bwd_matches_oracle(T, O, cfg):
    bs, ni, no, bias = cfg
    rng = np.random.default_rng(abs(hash(cfg)) % 2**31)
    x = rng.uniform(-1, 1, (bs, ni)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, ni * no).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, no).astype(np.float32)
    dy = rng.standard_normal((bs, no)).astype(np.float32)
    xd, wd, bd, dyd = T.to_device(x), T.to_device(w), T.to_device(b), T.to_device(dy)
    y, dx, dw, db = T.DevBuf((bs, no)), T.DevBuf((bs, ni)), T.DevBuf((ni * no,)), T.DevBuf((no,))
    T.fc_fwd(ni, no, bias, bs, xd, wd, bd if bias else None, y)
    assert_close(y.numpy(), O.fc_fwd(x, w, b if bias else None), what="y")
    T.fc_bwd(ni, no, bias, bs, xd, wd, dyd, dx, dw, db if bias else None)
    rdx, rdw, rdb = O.fc_bwd(x, w, dy, bias)
    assert_close(dx.numpy(), rdx, what="dx")
    assert_close(dw.numpy(), rdw, what="dw")
    if bias:
        assert_close(db.numpy(), rdb, what="db")


def test_fc_reference_kats_and_outputs(T, kats, layer_grads):
    k = kats["fc_forward"]
    y = T.DevBuf((1, 2))
    T.fc_fwd(4, 2, True, 1, T.to_device(np.array([k["x"]], np.float32)),
             T.to_device(np.full(8, 1.0, np.float32)), T.to_device(np.full(2, 0.5, np.float32)), y)
    assert np.array_equal(y.numpy()[0], np.array(k["y"], np.float32))
    T.fc_fwd(4, 2, False, 1, T.to_device(np.array([k["x"]], np.float32)),
             T.to_device(np.full(8, 1.0, np.float32)), None, y)
    assert np.array_equal(y.numpy()[0], np.array(kats["fc_forward_nobias"]["y"], np.float32))
    g = layer_grads
    xd, wd, dyd = T.to_device(g["fc.x"]), T.to_device(g["fc.w"]), T.to_device(g["fc.dy"])
    dx, dw, db = T.DevBuf((6, 37)), T.DevBuf((37 * 19,)), T.DevBuf((19,))
    T.fc_bwd(37, 19, True, 6, xd, wd, dyd, dx, dw, db)
    for eng in ("internal", "avx"):
        assert_close(dx.numpy(), g[f"fc.{eng}.dx"]); assert_close(dw.numpy(), g[f"fc.{eng}.dw"])
        assert_close(db.numpy(), g[f"fc.{eng}.db"])


POOL = [(4, 4, 1, 2, 2, 2, 2, 0, 0), (7, 7, 2, 2, 2, 2, 2, 0, 1), (4, 4, 1, 2, 2, 1, 1, 1, 0),
        (9, 8, 3, 3, 3, 2, 2, 0, 0), (6, 6, 2, 2, 2, 3, 3, 0, 0), (32, 32, 32, 2, 2, 2, 2, 0, 0),
        (4, 4, 1, 2, 1, 2, 1, 0, 0), (4, 4, 1, 1, 2, 1, 2, 0, 0), (13, 9, 5, 3, 2, 2, 1, 1, 1),
        # 2x2 stride-2 windows over rows of whole 16-byte words (two outputs a thread), and not
        (8, 6, 3, 2, 2, 2, 2, 0, 0), (12, 4, 5, 2, 2, 2, 2, 0, 0), (6, 6, 2, 2, 2, 2, 2, 0, 0),
        (16, 16, 7, 2, 2, 2, 2, 1, 0)]


@pytest.mark.parametrize("cfg", POOL)
def test_maxpool_bit_exact(T, O, cfg):
    iw, ih, c = cfg[:3]
    rng = np.random.default_rng(abs(hash(cfg)) % 2**31)
    d, do = T.pool_desc(*cfg), O.pool_desc(*cfg)
    ow, oh = T.pool_out_shape(d)
    assert (ow, oh) == O.pool_out_shape(do)
    bs = 5
    x = rng.integers(-3, 4, (bs, c * ih * iw)).astype(np.float32)     # many ties
    dy = rng.standard_normal((bs, c * oh * ow)).astype(np.float32)
    y, am, dx = T.DevBuf((bs, c * oh * ow)), T.DevBuf((bs, c * oh * ow), np.int32), T.DevBuf(x.shape)
    T.maxpool_fwd(d, bs, T.to_device(x), y, am)
    T.maxpool_bwd(d, bs, T.to_device(dy), am, dx)
    ry, ram = O.maxpool_fwd(do, x)
    assert np.array_equal(y.numpy(), ry)
    assert np.array_equal(am.numpy().astype(np.int64), ram), "argmax indices must be bit-exact"
    assert np.array_equal(dx.numpy(), O.maxpool_bwd(do, dy, ram))


def test_maxpool_nan_and_reference_outputs(T, O, kats, layer_grads):
    d, do = T.pool_desc(4, 2, 1, 2), O.pool_desc(4, 2, 1, 2)
    x = np.array([[5, 5, np.nan, 1, 5, 9, np.nan, np.nan],
                  [7, 7, np.nan, np.nan, 7, 7, np.nan, np.nan]], np.float32)
    y, am = T.DevBuf((2, 2)), T.DevBuf((2, 2), np.int32)
    T.maxpool_fwd(d, 2, T.to_device(x), y, am)
    ry, ram = O.maxpool_fwd(do, x)
    assert np.array_equal(am.numpy().astype(np.int64), ram) and np.array_equal(y.numpy(), ry)
    k = kats["maxpool_backward"]
    d = T.pool_desc(4, 4, 1, 2)
    y, am, dx = T.DevBuf((1, 4)), T.DevBuf((1, 4), np.int32), T.DevBuf((1, 16))
    T.maxpool_fwd(d, 1, T.to_device(np.array([kats["pool_input_4x4"]], np.float32)), y, am)
    T.maxpool_bwd(d, 1, T.to_device(np.array([k["dy"]], np.float32)), am, dx)
    assert np.array_equal(dx.numpy()[0], np.array(k["dx"], np.float32))
    g = layer_grads
    for name in ("maxpool2x2", "maxpool3x3s2", "maxpool_same_s1", "maxpool_ceil", "maxpool_gap"):
        cfg = [int(v) for v in g[f"{name}.cfg"]]
        d = T.pool_desc(*cfg)
        x, dy = g[f"{name}.x"], g[f"{name}.dy"]
        y, am, dx = T.DevBuf(g[f"{name}.y"].shape), T.DevBuf(g[f"{name}.y"].shape, np.int32), T.DevBuf(x.shape)
        T.maxpool_fwd(d, x.shape[0], T.to_device(x), y, am)
        T.maxpool_bwd(d, x.shape[0], T.to_device(dy), am, dx)
        assert np.array_equal(y.numpy(), g[f"{name}.y"]), name
        assert np.array_equal(dx.numpy(), g[f"{name}.dx"]), name


@pytest.mark.parametrize("cfg", [(4, 4, 1, 2, 2), (4, 4, 2, 2, 1), (28, 28, 6, 2, 2), (6, 6, 3, 3, 3),
                                 (10, 10, 16, 2, 2), (64, 64, 8, 2, 2)])
def test_avepool_matches_oracle(T, O, cfg):
    iw, ih, c, p, s = cfg
    rng = np.random.default_rng(abs(hash(cfg)) % 2**31)
    d, do = T.pool_desc(iw, ih, c, p, p, s, s), O.pool_desc(iw, ih, c, p, p, s, s)
    ow, oh = T.pool_out_shape(d)
    bs = 5
    x = rng.standard_normal((bs, c * ih * iw)).astype(np.float32)
    w = rng.standard_normal(c).astype(np.float32)
    b = rng.standard_normal(c).astype(np.float32)
    dy = rng.standard_normal((bs, c * oh * ow)).astype(np.float32)
    xd, wd = T.to_device(x), T.to_device(w)
    y, dx, dw, db = T.DevBuf(dy.shape), T.DevBuf(x.shape), T.DevBuf((c,)), T.DevBuf((c,))
    T.avepool_fwd(d, bs, xd, wd, T.to_device(b), y)
    assert_close(y.numpy(), O.avepool_fwd(do, x, w, b), what="y")
    T.avepool_bwd(d, bs, xd, wd, T.to_device(dy), dx, dw, db)
    rdx, rdw, rdb = O.avepool_bwd(do, x, w, dy)
    assert_close(dx.numpy(), rdx, what="dx"); assert_close(dw.numpy(), rdw, what="dw")
    assert_close(db.numpy(), rdb, what="db")


def test_avepool_reference_outputs_and_errors(T, kats, layer_grads):
    g = layer_grads
    for name in ("avepool2", "avepool2s1", "avepool3"):
        iw, ih, c, p, s = [int(v) for v in g[f"{name}.cfg"]]
        d = T.pool_desc(iw, ih, c, p, p, s, s)
        x, dy = g[f"{name}.x"], g[f"{name}.dy"]
        xd, wd = T.to_device(x), T.to_device(g[f"{name}.w"])
        y, dx, dw, db = T.DevBuf(dy.shape), T.DevBuf(x.shape), T.DevBuf((c,)), T.DevBuf((c,))
        T.avepool_fwd(d, 3, xd, wd, T.to_device(g[f"{name}.b"]), y)
        T.avepool_bwd(d, 3, xd, wd, T.to_device(dy), dx, dw, db)
        assert_close(y.numpy(), g[f"{name}.y"]); assert_close(dx.numpy(), g[f"{name}.dx"])
        assert_close(dw.numpy(), g[f"{name}.dw"]); assert_close(db.numpy(), g[f"{name}.db"])
    x = np.array([kats["pool_input_4x4"]], np.float32)
    for k in kats["avepool_forward"]:
        d = T.pool_desc(4, 4, 1, k["pool"], k["pool"], k["stride"], k["stride"])
        y = T.DevBuf((1, len(k["y"])))
        T.avepool_fwd(d, 1, T.to_device(x), T.to_device(np.ones(1, np.float32)),
                      T.to_device(np.zeros(1, np.float32)), y)
        np.testing.assert_allclose(y.numpy()[0], k["y"], rtol=1.2e-5)
    buf = T.DevBuf((64,))
    with pytest.raises(T.TdhError, match="multiple of the window"):   # reference ctor throws too
        T.avepool_fwd(T.pool_desc(5, 5, 1, 2), 1, buf, buf, buf, buf)


def test_activation_layers_match_reference_outputs(T, act_golden):
    """Every activation layer against what the compiled reference produced for the same input."""
    g = act_golden
    x, dy = g["x"], g["dy"]
    xd, dyd = T.to_device(x), T.to_device(dy)
    names = sorted({f.rsplit(".", 1)[0] for f in g.files if "." in f})
    assert len(names) == 14
    for name in names:
        kind, prm = name.split(".", 1)[1], tuple(float(v) for v in g[name + ".p"])
        y, dx = T.DevBuf(x.shape), T.DevBuf(x.shape)
        T.act_fwd(kind, x.shape[0], x.shape[1], xd, y, params=prm)
        assert_close(y.numpy(), g[name + ".y"], REL_TOL, name + " forward")
        T.act_bwd(kind, x.shape[0], x.shape[1], T.to_device(g[name + ".y"]), dyd, dx, x=xd, params=prm)
        assert_close(dx.numpy(), g[name + ".dx"], REL_TOL, name + " backward")
    # the gradients of selu and softsign read the layer input: refused without it
    with pytest.raises(T.TdhError, match="reads the layer input"):
        T.act_bwd("selu", x.shape[0], x.shape[1], xd, dyd, T.DevBuf(x.shape))


@pytest.mark.parametrize("kind", ["tanh", "relu", "sigmoid", "softmax"])
@pytest.mark.parametrize("shape", [(4, 10), (3, 1000), (7, 77), (1, 1), (64, 4099)])
def test_activations_match_oracle(T, O, kind, shape):
    rng = np.random.default_rng(shape[1])
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    y, dx = T.DevBuf(shape), T.DevBuf(shape)
    T.act_fwd(kind, shape[0], shape[1], T.to_device(x), y)
    ry = O.act_fwd(kind, x)
    assert_close(y.numpy(), ry, 1e-5, "forward")
    T.act_bwd(kind, shape[0], shape[1], T.to_device(ry), T.to_device(dy), dx)
    assert_close(dx.numpy(), O.act_bwd(kind, x, ry, dy), 1e-5, "backward")


@pytest.mark.parametrize("shape,scale", [((1, 255), 20.0), ((3, 10), 50.0), ((16, 1000), 8.0)])
def test_softmax_backward_of_saturated_rows_matches_oracle(T, O, shape, scale):
    """Rows whose largest output is next to 1: every term of the reference's Jacobian row is
    small there, and y*(dy - <dy, y>) in float would lose the element of the largest output."""
    rng = np.random.default_rng(int(scale))
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    x[np.arange(shape[0]), rng.integers(0, shape[1], shape[0])] += 5 * scale
    dy = rng.standard_normal(shape).astype(np.float32)
    ry = O.act_fwd("softmax", x)
    assert ry.max(axis=1).min() > 0.9
    dx = T.DevBuf(shape)
    T.act_bwd("softmax", shape[0], shape[1], T.to_device(ry), T.to_device(dy), dx)
    want = O.act_bwd("softmax", x, ry, dy)
    got = dx.numpy()
    for r in range(shape[0]):   # row by row: a saturated row's gradient is tiny beside the others'
        assert_close(got[r], want[r], REL_TOL, f"row {r}")


def test_unaligned_views_take_the_scalar_path(T, O):
    """Sub-tensors that are not 16-byte aligned still give the same results."""
    rng = np.random.default_rng(5)
    n = 1001
    y = rng.standard_normal((1, n + 1)).astype(np.float32)
    dy = rng.standard_normal((1, n + 1)).astype(np.float32)
    yd, dyd, out = T.to_device(y), T.to_device(dy), T.DevBuf((1, n + 1), zero=True)
    off = lambda b: T.DevBuf.view(b.ptr.value + 4, (1, n))
    T.act_bwd("tanh", 1, n, off(yd), off(dyd), off(out))
    want = O.act_bwd("tanh", y[:, 1:], y[:, 1:], dy[:, 1:])
    got = out.numpy()
    assert got[0, 0] == 0.0
    assert_close(got[:, 1:], want, 1e-6)


def test_losses_match_oracle(T, O):
    rng = np.random.default_rng(6)
    y = O.act_fwd("softmax", rng.standard_normal((33, 10)).astype(np.float32))
    t = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 33)]
    yd, td, g = T.to_device(y), T.to_device(t), T.DevBuf((33, 10))
    for kind in ("mse", "ce_multiclass", "ce"):
        T.loss_grad(kind, 33, 10, yd, td, g)
        assert_close(g.numpy(), O.loss_grad(kind, y, t), 1e-6, kind)
    T.softmax_xent_grad(33, 10, yd, td, g)
    want = O.act_bwd("softmax", y, y, O.loss_grad("ce_multiclass", y, t))
    assert_close(g.numpy(), want, 1e-5, "fused softmax + cross-entropy gradient")
    # soft targets: y*sum(t) - t
    t2 = rng.uniform(0, 1, (33, 10)).astype(np.float32)
    T.softmax_xent_grad(33, 10, yd, T.to_device(t2), g)
    assert_close(g.numpy(), O.act_bwd("softmax", y, y, O.loss_grad("ce_multiclass", y, t2)), 1e-5)


@pytest.mark.parametrize("kind", ["sgd", "momentum", "adam", "adagrad", "rmsprop", "adamax", "nesterov"])
def test_optimizers_match_oracle_and_reference_kats(T, O, kats, kind):
    rng = np.random.default_rng(17)
    n = 4099
    o, ro = T.opt_desc(kind), O.opt_desc(kind)
    w = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    wd, gd = T.to_device(w), T.to_device(g)
    s0, s1 = T.DevBuf((n,), zero=True), T.DevBuf((n,), zero=True)
    rw, r0, r1 = w.copy(), np.zeros_like(w), np.zeros_like(w)
    for _ in range(3):
        T.opt_update(o, n, gd, wd, s0, s1)
        O.opt_update(ro, g, rw, r0, r1)
    assert_close(wd.numpy(), rw, 1e-6, "weights after 3 updates")
    assert o.b1_t == ro.b1_t and o.b2_t == ro.b2_t, "per-call bias-correction powers"
    for c in kats["optimizers"]["cases"]:
        if c["kind"] != kind:
            continue
        o = T.opt_desc(kind)
        wd, gd = T.to_device(np.array(c["w"], np.float32)), T.to_device(np.array(c["g"], np.float32))
        s0, s1 = T.DevBuf((5,), zero=True), T.DevBuf((5,), zero=True)
        T.opt_update(o, 5, gd, wd, s0, s1)
        np.testing.assert_allclose(wd.numpy(), c["first"], atol=1e-3)
        T.opt_update(o, 5, gd, wd, s0, s1)
        np.testing.assert_allclose(wd.numpy(), c["second"], atol=1e-3)


def test_optimizer_grad_scale_and_state_checks(T, O):
    o = T.opt_desc("sgd", alpha=0.5)
    w = T.to_device(np.zeros(3, np.float32))
    T.opt_update(o, 3, T.to_device(np.array([2, -4, 8], np.float32)), w, grad_scale=0.25)
    assert np.array_equal(w.numpy(), np.array([-0.25, 0.5, -1.0], np.float32))
    with pytest.raises(T.TdhError, match="state"):
        T.opt_update(T.opt_desc("adam"), 3, w, w, None, None)


@pytest.mark.parametrize("n,dst_off,src_off", [(1, 0, 0), (1023, 0, 0), (4096, 4, 8), (100003, 12, 0),
                                               (1 << 20, 0, 4)])
def test_device_copy_is_exact(T, n, dst_off, src_off):
    """tdh_memcpy_d2d (a copy kernel): every word arrives, nothing outside the range is written."""
    rng = np.random.default_rng(n)
    src = rng.integers(0, 2**32, n + 8, dtype=np.uint32)
    dst0 = rng.integers(0, 2**32, n + 8, dtype=np.uint32)
    s, d = T.to_device(src, np.uint32), T.to_device(dst0, np.uint32)
    T.copy_d2d(d, s, nbytes=4 * n, dst_offset=dst_off, src_offset=src_off)
    got = d.numpy()
    want = dst0.copy()
    want[dst_off // 4: dst_off // 4 + n] = src[src_off // 4: src_off // 4 + n]
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- batch normalization, dropout
@pytest.mark.parametrize("shape", [(5, 7, 4), (3, 100, 9), (64, 256, 128), (4, 1, 1), (130, 33, 70)])
def test_batchnorm_matches_oracle(T, O, shape):
    c, s, b = shape
    rng = np.random.default_rng(c + s)
    x = (rng.standard_normal((b, c * s)) * 2 + 0.5).astype(np.float32)
    dy = rng.standard_normal((b, c * s)).astype(np.float32)
    xd, dyd = T.to_device(x), T.to_device(dy)
    y, dx = T.DevBuf(x.shape), T.DevBuf(x.shape)
    mean, var, sd = T.DevBuf((c,)), T.DevBuf((c,)), T.DevBuf((c,))
    T.batchnorm_fwd(c, s, b, xd, mean, var, sd, y)
    ry, rmean, rvar, rsd = O.batchnorm_fwd(c, s, x)
    assert_close(mean.numpy(), rmean, 1e-5, "mean")
    assert_close(var.numpy(), rvar, 1e-5, "variance")
    assert_close(sd.numpy(), rsd, 1e-5, "stddev")
    assert_close(y.numpy(), ry, REL_TOL, "y")
    T.batchnorm_bwd(c, s, b, T.to_device(ry), dyd, T.to_device(rsd), dx)
    assert_close(dx.numpy(), O.batchnorm_bwd(c, s, ry, dy, rsd), REL_TOL, "dx")
    # test phase: the given moving averages are read, not written
    m0, v0 = rng.standard_normal(c).astype(np.float32), rng.uniform(0.5, 2, c).astype(np.float32)
    md, vd = T.to_device(m0), T.to_device(v0)
    T.batchnorm_fwd(c, s, b, xd, md, vd, sd, y, train=False)
    assert_close(y.numpy(), O.batchnorm_fwd(c, s, x, train=False, mean=m0, variance=v0)[0], REL_TOL, "test phase")
    assert np.array_equal(md.numpy(), m0) and np.array_equal(vd.numpy(), v0)
    T.batchnorm_update_moving(c, 0.9, mean, var, md, vd)
    rm1, rv1 = O.batchnorm_update_moving(0.9, rmean, rvar, m0, v0)
    assert_close(md.numpy(), rm1, 1e-5, "moving mean")
    assert_close(vd.numpy(), rv1, 1e-5, "moving variance")


def test_norm_layers_match_reference_outputs(T, norm_golden):
    """Against outputs of the compiled reference itself (tests/golden/norm.npz)."""
    g = norm_golden
    i = 0
    while f"bn{i}.x" in g:
        x, dy = g[f"bn{i}.x"], g[f"bn{i}.dy"]
        c = g[f"bn{i}.mean"].size
        s, b = x.shape[1] // c, x.shape[0]
        y, dx = T.DevBuf(x.shape), T.DevBuf(x.shape)
        mean, var, sd = T.DevBuf((c,)), T.DevBuf((c,)), T.DevBuf((c,))
        T.batchnorm_fwd(c, s, b, T.to_device(x), mean, var, sd, y)
        assert_close(y.numpy(), g[f"bn{i}.y"], REL_TOL, "y")
        assert_close(var.numpy(), g[f"bn{i}.var"], 1e-5, "variance")
        T.batchnorm_bwd(c, s, b, T.to_device(g[f"bn{i}.y"]), T.to_device(dy), sd, dx)
        assert_close(dx.numpy(), g[f"bn{i}.dx"], REL_TOL, "dx")
        i += 1
    from tests.golden.make_fixtures import DROPOUT_CASES
    x, dy = g["do.x"], g["do.dy"]
    for k, (seed, rate) in enumerate(DROPOUT_CASES):
        mask = T.dropout_mask(T.Mt19937(seed), rate, *x.shape)
        assert np.array_equal(mask, g[f"do{k}.mask"])           # host-side draw, bit for bit
        md = T.to_device(mask, np.uint8)
        y, dx = T.DevBuf(x.shape), T.DevBuf(x.shape)
        T.dropout_fwd(x.shape[0], x.shape[1], md, T.to_device(x), y, rate=rate)
        assert np.array_equal(y.numpy(), g[f"do{k}.y"])
        T.dropout_bwd(x.shape[0], x.shape[1], md, T.to_device(dy), dx)
        assert np.array_equal(dx.numpy(), g[f"do{k}.dx"])
    T.dropout_fwd(x.shape[0], x.shape[1], None, T.to_device(x), y, train=False)
    assert np.array_equal(y.numpy(), x)


def test_norm_argument_errors(T):
    buf = T.DevBuf((4,))
    with pytest.raises(T.TdhError, match="null tensor"):
        T.batchnorm_fwd(2, 2, 1, None, buf, buf, buf, buf)
    with pytest.raises(T.TdhError, match="null tensor"):
        T.dropout_fwd(1, 4, None, buf, buf, train=True)
    T.batchnorm_fwd(0, 2, 1, None, None, None, None, None)      # empty tensors: nothing to do
    T.dropout_bwd(0, 4, None, None, None)


@pytest.mark.parametrize("seed", [11, 12])
def test_randomized_conv_shapes_match_oracle(T, O, seed):
    """A seeded sweep over window, channel counts, image sizes, padding, stride, dilation
    (forward only, as in the reference) and batch: whichever kernel the shape selects, forward
    and all three gradients agree with the oracle."""
    rng = np.random.default_rng(seed)
    done = 0
    while done < 60:
        k = int(rng.choice([3, 5]))
        ic = int(rng.choice([1, 2, 3, 4, 8, 16, 20, 32, 48]))
        oc = int(rng.choice([1, 5, 16, 32, 33, 40, 64, 70]))
        iw, ih = int(rng.integers(k, 44)), int(rng.integers(k, 30))
        same = bool(rng.integers(0, 2))
        st = int(rng.choice([1, 1, 1, 2, 3]))
        dil = 1 if same else int(rng.choice([1, 1, 1, 2]))
        bs = int(rng.choice([1, 2, 3, 5, 8, 17]))
        if not same and (iw < dil * (k - 1) + 1 or ih < dil * (k - 1) + 1):
            continue
        kw = dict(pad_same=same, w_stride=st, h_stride=st, w_dilation=dil, h_dilation=dil)
        d, do = T.conv_desc(iw, ih, ic, k, k, oc, **kw), O.conv_desc(iw, ih, ic, k, k, oc, **kw)
        ow, oh = T.conv_out_shape(d)
        if ow < 1 or oh < 1:
            continue
        what = f"{(iw, ih, ic, k, oc, same, st, dil, bs)}"
        x = rng.standard_normal((bs, ic * ih * iw)).astype(np.float32)
        w = rng.uniform(-0.3, 0.3, oc * ic * k * k).astype(np.float32)
        b = rng.standard_normal(oc).astype(np.float32)
        dy = rng.standard_normal((bs, oc * oh * ow)).astype(np.float32)
        xd, wd, bd, dyd = T.to_device(x), T.to_device(w), T.to_device(b), T.to_device(dy)
        y = T.DevBuf((bs, oc * oh * ow))
        T.conv2d_fwd(d, bs, xd, wd, bd, y)
        assert_close(y.numpy(), O.conv2d_fwd(do, x, w, b), what=what + " y")
        if dil == 1:
            dx, dw, db = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,), zero=True)
            T.conv2d_bwd(d, bs, xd, wd, dyd, dx, dw, db, 0)
            rdx, rdw, rdb = O.conv2d_bwd(do, x, w, dy)
            assert_close(dx.numpy(), rdx, what=what + " dx")
            assert_close(dw.numpy(), rdw, what=what + " dw")
            assert_close(db.numpy(), rdb, what=what + " db")
        done += 1


def test_randomized_conv_and_fc_options_match_oracle(T, O):
    """A seeded sweep over what a caller may leave out or ask for: no bias, any subset of the
    three gradients (NULL outputs are skipped), accumulation onto prior dW/db, windows that are
    not square (1x1 up to 7x7), different strides along the two axes; on shapes that pick the
    few-channel kernels as well as the tiled ones."""
    rng = np.random.default_rng(31)
    done = 0
    while done < 70:
        kw = int(rng.choice([1, 2, 3, 3, 5, 5, 7]))
        kh = kw if rng.random() < 0.6 else int(rng.choice([1, 2, 3, 5]))
        big = rng.random() < 0.5
        ic = int(rng.choice([16, 32, 48, 64] if big else [1, 2, 3, 4, 6, 8, 20]))
        oc = int(rng.choice([16, 32, 64, 96] if big else [1, 3, 6, 16, 33]))
        iw, ih = int(rng.integers(max(kw, 4), 36)), int(rng.integers(max(kh, 4), 28))
        if big and rng.random() < 0.6:
            iw, ih = int(rng.choice([8, 12, 16, 24, 32])), int(rng.choice([8, 16, 24, 32]))
        same = bool(rng.integers(0, 2))
        sw = int(rng.choice([1, 1, 1, 2]))
        sh = sw if rng.random() < 0.7 else int(rng.choice([1, 2, 3]))
        bias, acc = bool(rng.random() < 0.7), bool(rng.integers(0, 2))
        want = [bool(v) for v in rng.integers(0, 2, 3)]   # dx, dw, db
        if not any(want):
            want[1] = True
        want[2] = want[2] and bias
        bs = int(rng.choice([1, 2, 4, 7, 16]))
        if iw < kw or ih < kh:
            continue
        opts = dict(pad_same=same, has_bias=bias, w_stride=sw, h_stride=sh)
        d, do = T.conv_desc(iw, ih, ic, kw, kh, oc, **opts), O.conv_desc(iw, ih, ic, kw, kh, oc, **opts)
        ow, oh = T.conv_out_shape(d)
        if ow < 1 or oh < 1:
            continue
        what = f"conv {(iw, ih, ic, kw, kh, oc, same, sw, sh, bias, acc, want, bs)}"
        x = rng.standard_normal((bs, ic * ih * iw)).astype(np.float32)
        w = rng.uniform(-0.3, 0.3, oc * ic * kh * kw).astype(np.float32)
        b = rng.standard_normal(oc).astype(np.float32)
        dy = rng.standard_normal((bs, oc * oh * ow)).astype(np.float32)
        prior = [rng.standard_normal(n).astype(np.float32) for n in (x.shape, w.shape, (oc,))]
        xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
        y = T.DevBuf((bs, oc * oh * ow))
        T.conv2d_fwd(d, bs, xd, wd, T.to_device(b) if bias else None, y)
        assert_close(y.numpy(), O.conv2d_fwd(do, x, w, b if bias else None), what=what + " y")
        out = [T.to_device(p0) if wanted else None for p0, wanted in zip(prior, want)]
        T.conv2d_bwd(d, bs, xd, wd, dyd, out[0], out[1], out[2], acc)
        ref = O.conv2d_bwd(do, x, w, dy)
        for k, name in enumerate(("dx", "dw", "db")):
            if want[k]:
                base = prior[k] if acc and k > 0 else 0.0     # dX is always overwritten
                assert_close(out[k].numpy(), ref[k] + base, what=f"{what} {name}")
        done += 1
    for _ in range(40):
        ni = int(rng.choice([1, 7, 64, 120, 256, 512, 1000, 2048]))
        no = int(rng.choice([1, 10, 33, 64, 256, 1024]))
        bs = int(rng.choice([1, 2, 16, 17, 128]))
        bias, acc = bool(rng.random() < 0.7), bool(rng.integers(0, 2))
        want = [bool(v) for v in rng.integers(0, 2, 3)]
        if not any(want):
            want[0] = True
        want[2] = want[2] and bias
        what = f"fc {(ni, no, bs, bias, acc, want)}"
        x = rng.standard_normal((bs, ni)).astype(np.float32)
        w = rng.uniform(-0.2, 0.2, ni * no).astype(np.float32)
        b = rng.standard_normal(no).astype(np.float32)
        dy = rng.standard_normal((bs, no)).astype(np.float32)
        prior = [rng.standard_normal(n).astype(np.float32) for n in (x.shape, w.shape, (no,))]
        xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
        y = T.DevBuf((bs, no))
        T.fc_fwd(ni, no, bias, bs, xd, wd, T.to_device(b) if bias else None, y)
        assert_close(y.numpy(), O.fc_fwd(x, w, b if bias else None), what=what + " y")
        out = [T.to_device(p0) if wanted else None for p0, wanted in zip(prior, want)]
        T.fc_bwd(ni, no, bias, bs, xd, wd, dyd, out[0], out[1], out[2], acc)
        ref = O.fc_bwd(x, w, dy)
        for k, name in enumerate(("dx", "dw", "db")):
            if want[k]:
                base = prior[k] if acc and k > 0 else 0.0
                assert_close(out[k].numpy(), ref[k] + base, what=f"{what} {name}")


def test_randomized_fc_and_maxpool_shapes_match_oracle(T, O):
    """Seeded sweeps: fully-connected layers across the small / tiled / split products, and
    max-pool windows, strides, padding modes with tied values (outputs, argmax and routed
    gradients bit-exact)."""
    rng = np.random.default_rng(21)
    for _ in range(30):
        ni = int(rng.choice([1, 7, 10, 64, 100, 120, 256, 300, 512, 1000, 1024, 2048]))
        no = int(rng.choice([1, 2, 10, 33, 64, 100, 256, 500]))
        bs = int(rng.choice([1, 2, 5, 16, 17, 64, 128]))
        what = f"fc {(ni, no, bs)}"
        x = rng.standard_normal((bs, ni)).astype(np.float32)
        w = rng.uniform(-0.2, 0.2, ni * no).astype(np.float32)
        b = rng.standard_normal(no).astype(np.float32)
        dy = rng.standard_normal((bs, no)).astype(np.float32)
        xd, wd, bd, dyd = T.to_device(x), T.to_device(w), T.to_device(b), T.to_device(dy)
        y, dx, dw, db = T.DevBuf((bs, no)), T.DevBuf((bs, ni)), T.DevBuf((ni * no,)), T.DevBuf((no,))
        T.fc_fwd(ni, no, True, bs, xd, wd, bd, y)
        T.fc_bwd(ni, no, True, bs, xd, wd, dyd, dx, dw, db)
        rdx, rdw, rdb = O.fc_bwd(x, w, dy)
        assert_close(y.numpy(), O.fc_fwd(x, w, b), what=what + " y")
        assert_close(dx.numpy(), rdx, what=what + " dx")
        assert_close(dw.numpy(), rdw, what=what + " dw")
        assert_close(db.numpy(), rdb, what=what + " db")
    done = 0
    while done < 40:
        c = int(rng.choice([1, 3, 8, 33]))
        iw, ih = int(rng.integers(2, 40)), int(rng.integers(2, 30))
        pw, ph = int(rng.choice([2, 2, 3])), int(rng.choice([2, 2, 3]))
        sw, sh = int(rng.choice([1, 2, 2, 3])), int(rng.choice([1, 2, 2, 3]))
        same, ceil = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        bs = int(rng.choice([1, 3, 8]))
        if not same and (iw < pw or ih < ph):
            continue
        kw = dict(pad_same=same, ceil_mode=ceil)
        d, do = T.pool_desc(iw, ih, c, pw, ph, sw, sh, **kw), O.pool_desc(iw, ih, c, pw, ph, sw, sh, **kw)
        ow, oh = T.pool_out_shape(d)
        if ow < 1 or oh < 1:
            continue
        what = f"maxpool {(iw, ih, c, pw, ph, sw, sh, same, ceil, bs)}"
        x = rng.standard_normal((bs, c * ih * iw)).astype(np.float32)
        x[rng.random(x.shape) < 0.2] = 0.5  # ties
        dy = rng.standard_normal((bs, c * oh * ow)).astype(np.float32)
        ry, ram = O.maxpool_fwd(do, x)
        y, am, dx = T.DevBuf((bs, c * oh * ow)), T.DevBuf((bs, c * oh * ow), np.int32), T.DevBuf(x.shape)
        T.maxpool_fwd(d, bs, T.to_device(x), y, am)
        T.maxpool_bwd(d, bs, T.to_device(dy), am, dx)
        assert np.array_equal(y.numpy(), ry), what
        assert np.array_equal(am.numpy().astype(np.int64), ram), what
        assert np.array_equal(dx.numpy(), O.maxpool_bwd(do, dy, ram)), what
        done += 1
