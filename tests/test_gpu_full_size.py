"""The five benchmark configurations at their full sizes on the MI355X, checked through
size-independent properties and float64 spot checks (the scalar oracle would need minutes
at these sizes): exact float64 dot products for sampled gradient entries, db against a host
sum, linearity of the backward pass in dY, and whole fully-connected gradients against
numpy's float64 matmul."""
import numpy as np
import pytest

from conftest import assert_close, rel_err

pytestmark = pytest.mark.gpu


def test_config2_conv_backward_full_size(T, W):
    """configs[1]: batch 64, 32x64x64 -> 64 channels, 3x3, pad same, stride 1."""
    (hw, _, c, k, oc), x, w, dy = W.conv_bwd_case()
    bs = x.shape[0]
    d = T.conv_desc(hw, hw, c, k, k, oc, pad_same=True)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    dx, dw, db = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,))
    T.conv2d_bwd(d, bs, xd, wd, dyd, dx, dw, db)
    dxh, dwh, dbh = dx.numpy(), dw.numpy().reshape(oc, c, k, k), db.numpy()
    x4 = x.reshape(bs, c, hw, hw)
    dy4 = dy.reshape(bs, oc, hw, hw)
    w4 = w.reshape(oc, c, k, k)
    # db: exact sum on the host
    assert_close(dbh, dy4.astype(np.float64).sum(axis=(0, 2, 3)), what="db")
    # dW: float64 dot products over the whole batch for sampled taps
    rng = np.random.default_rng(0)
    xp = np.zeros((bs, c, hw + 2, hw + 2), np.float64)
    xp[:, :, 1:-1, 1:-1] = x4
    dw_scale = np.sqrt(np.mean(dwh.astype(np.float64) ** 2))
    for _ in range(40):
        o, i, ky, kx = rng.integers(oc), rng.integers(c), rng.integers(k), rng.integers(k)
        want = np.sum(xp[:, i, ky:ky + hw, kx:kx + hw] * dy4[:, o])
        assert abs(dwh[o, i, ky, kx] - want) <= 1e-4 * max(abs(want), dw_scale), (o, i, ky, kx)
    # dX: float64 correlation with the flipped filter at sampled positions
    dyp = np.zeros((oc, hw + 2, hw + 2), np.float64)
    dx4 = dxh.reshape(bs, c, hw, hw)
    dx_scale = np.sqrt(np.mean(dx4.astype(np.float64) ** 2))
    for _ in range(8):
        n = rng.integers(bs)
        dyp[:, 1:-1, 1:-1] = dy4[n]
        for _ in range(6):
            i, yy, xx = rng.integers(c), rng.integers(hw), rng.integers(hw)
            # dX[i,yy,xx] = sum_{o,ky,kx} W[o,i,ky,kx] * dY[o, yy+1-ky, xx+1-kx]
            win = dyp[:, yy:yy + 3, xx:xx + 3][:, ::-1, ::-1]
            want = np.sum(w4[:, i].astype(np.float64) * win)
            assert abs(dx4[n, i, yy, xx] - want) <= 1e-4 * max(abs(want), dx_scale)
    # linearity in dY: backward(2*dy) == 2*backward(dy), bit for bit (scaling by 2 is exact)
    dx2, dw2, db2 = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,))
    T.conv2d_bwd(d, bs, xd, wd, T.to_device(dy * 2), dx2, dw2, db2)
    assert np.array_equal(dx2.numpy(), 2 * dxh)
    assert np.array_equal(dw2.numpy().reshape(dwh.shape), 2 * dwh)
    assert np.array_equal(db2.numpy(), 2 * dbh)


@pytest.mark.parametrize("bs,ni,no", [
    (37, 4100, 2050),    # no tile of the kernel is whole in either direction; odd batch
    (8, 4096, 2048),     # exactly 256 workgroups; one group of loads
    (130, 2052, 4098),   # a tail of two samples behind eight full groups
])
def test_large_fc_weight_gradient_from_memory_fragments(T, bs, ni, no):
    """dW of a fully-connected layer with at least eight million weights runs on a kernel that
    feeds the matrix cores from memory (no LDS): against float64, stored and accumulated on top
    of a previous value, with dX and db of the same call."""
    rng = np.random.default_rng(bs * 7 + ni)
    x = rng.uniform(-1, 1, (bs, ni)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, ni * no).astype(np.float32)
    dy = rng.standard_normal((bs, no)).astype(np.float32)
    before = rng.standard_normal(ni * no).astype(np.float32)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    dx, dw, db = T.DevBuf((bs, ni)), T.DevBuf((ni * no,)), T.DevBuf((no,))
    T.fc_bwd(ni, no, True, bs, xd, wd, dyd, dx, dw, db)
    want = x.astype(np.float64).T @ dy.astype(np.float64)
    assert_close(dw.numpy().reshape(ni, no), want, what="dw")
    assert_close(dx.numpy(), dy.astype(np.float64) @ w.reshape(ni, no).astype(np.float64).T, what="dx")
    assert_close(db.numpy(), dy.astype(np.float64).sum(0), what="db")
    dw2, db2 = T.to_device(before), T.DevBuf((no,), zero=True)
    T.fc_bwd(ni, no, True, bs, xd, wd, dyd, dx, dw2, db2, accumulate=True)
    # (bit for bit: the same sums, added to the previous value at the end)
    assert np.array_equal(dw2.numpy(), before + dw.numpy())


@pytest.mark.parametrize("bs,ni,no", [
    (250, 3100, 1100),   # ragged in both directions, a last chunk of 76 outputs, idle workgroups at the grid's end
    (256, 4096, 1028),   # nearly the shortest reduction the kernel takes, a last chunk of one 16-byte word
    (200, 4160, 2048),   # whole chunks; a last column tile of its own
])
def test_large_fc_input_gradient_from_untransposed_tiles(T, bs, ni, no):
    """dX of a fully-connected layer with a 64 x 64 tile for (nearly) every compute unit and a
    long reduction runs on a kernel of its own (operands staged untransposed, no split reduction):
    against float64, twice with equal bits, and linear in dY bit for bit."""
    rng = np.random.default_rng(bs + ni + no)
    x = rng.uniform(-1, 1, (bs, ni)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, ni * no).astype(np.float32)
    dy = rng.standard_normal((bs, no)).astype(np.float32)
    xd, wd = T.to_device(x), T.to_device(w)
    dx, dw, db = T.DevBuf((bs, ni)), T.DevBuf((ni * no,)), T.DevBuf((no,))
    T.fc_bwd(ni, no, True, bs, xd, wd, T.to_device(dy), dx, dw, db)
    got = dx.numpy().copy()
    assert_close(got, dy.astype(np.float64) @ w.reshape(ni, no).astype(np.float64).T, what="dx")
    dx.upload(np.full((bs, ni), np.nan, np.float32))
    T.fc_bwd(ni, no, True, bs, xd, wd, T.to_device(dy), dx, dw, db)
    assert np.array_equal(dx.numpy(), got)
    T.fc_bwd(ni, no, True, bs, xd, wd, T.to_device(dy * 2), dx, dw, db)
    assert np.array_equal(dx.numpy(), 2 * got)


def test_config3_fc_backward_adam_full_size(T, O, W):
    """configs[2]: batch 256, 4096 -> 4096, tanh, Adam on W and b."""
    x, w, b, dy = W.fc_bwd_case()
    bs, n = x.shape[0], 4096
    xd, wd, bd = T.to_device(x), T.to_device(w), T.to_device(b)
    z, y = T.DevBuf((bs, n)), T.DevBuf((bs, n))
    T.fc_fwd(n, n, True, bs, xd, wd, bd, z)
    T.act_fwd("tanh", bs, n, z, y)
    W64 = w.reshape(n, n).astype(np.float64)
    z_ref = x.astype(np.float64) @ W64 + b
    assert_close(z.numpy(), z_ref, what="forward")
    y_ref = np.tanh(z_ref)
    assert_close(y.numpy(), y_ref, 1e-5, what="tanh")
    dz, dx, dw, db = T.DevBuf((bs, n)), T.DevBuf((bs, n)), T.DevBuf((n * n,)), T.DevBuf((n,))
    T.act_bwd("tanh", bs, n, y, T.to_device(dy), dz)
    yh = y.numpy().astype(np.float64)
    dz_ref = dy * (1 - yh * yh)
    assert_close(dz.numpy(), dz_ref, 1e-5, what="tanh gradient")
    T.fc_bwd(n, n, True, bs, xd, wd, dz, dx, dw, db)
    dzh = dz.numpy().astype(np.float64)
    assert_close(dx.numpy(), dzh @ W64.T, what="dx")
    dw_ref = x.astype(np.float64).T @ dzh
    assert_close(dw.numpy().reshape(n, n), dw_ref, what="dw (summed over the batch)")
    assert_close(db.numpy(), dzh.sum(0), what="db")
    # Adam on W then on b with one optimizer object: b sees the advanced powers
    opt, ropt = T.opt_desc("adam"), O.opt_desc("adam")
    s = [T.DevBuf((n * n,), zero=True), T.DevBuf((n * n,), zero=True), T.DevBuf((n,), zero=True),
         T.DevBuf((n,), zero=True)]
    dwh, dbh = dw.numpy(), db.numpy()
    T.opt_update(opt, n * n, dw, wd, s[0], s[1])
    T.opt_update(opt, n, db, bd, s[2], s[3])
    rw, rb = w.copy(), b.copy()
    O.opt_update(ropt, dwh, rw, np.zeros_like(rw), np.zeros_like(rw))
    O.opt_update(ropt, dbh, rb, np.zeros_like(rb), np.zeros_like(rb))
    assert_close(wd.numpy(), rw, 1e-6, what="W after Adam")
    assert_close(bd.numpy(), rb, 1e-6, what="b after Adam")
    assert opt.b1_t == ropt.b1_t


def test_config4_full_batch_step_properties(T, W):
    """configs[3] at batch 128: a step changes every parameter, stays finite, and the loss
    gradient rows sum to zero (softmax + cross-entropy)."""
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("cifar10_cnn_b128")
    net = T.Net(W.build_layers(T, spec), batch, 1)
    for (i, which, a) in params:
        net.set_param(i, which, a)
    xd, td = T.to_device(x), T.to_device(t)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    n = len(spec)
    dz = net.layer_dx(n - 1, batch)           # gradient w.r.t. the logits
    y = net.layer_out(n - 1, batch)
    assert_close(dz, y.astype(np.float64) - t, 1e-5, what="dz = y - t")
    assert np.all(np.abs(dz.sum(1)) < 1e-5)
    # bias gradient of the last fc layer is the column sum of dz
    assert_close(net.layer_grad(n - 2, 1), dz.astype(np.float64).sum(0), what="db of fc2")
    # weight gradient of the last fc layer is relu_out^T dz
    a = net.layer_out(n - 3, batch).astype(np.float64)
    assert_close(net.layer_grad(n - 2, 0), (a.T @ dz).ravel(), what="dW of fc2")
    opt = T.opt_desc(opt_kind, **opt_kw)
    net.train_step(opt, loss, batch, xd, td)
    for (i, which, a0) in params:
        got = net.get_param(i, which)
        assert np.all(np.isfinite(got))
        assert not np.array_equal(got, a0)
    net.close()


def test_config5_vgg_full_size_one_step(T, W):
    """configs[4] at its full size (batch 64, 3x128x128): one momentum step; spot-check the
    big fully-connected gradient (131072 x 256) against float64 and the first conv's bias
    gradient against a host sum."""
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("vgg_stack_b64")
    net = T.Net(W.build_layers(T, spec), batch, 1)
    for (i, which, a) in params:
        net.set_param(i, which, a)
    xd, td = T.to_device(x), T.to_device(t)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    n = len(spec)
    fc1 = n - 4
    a = net.layer_out(fc1 - 1, batch).astype(np.float64)      # pooled features [64][131072]
    dz1 = net.layer_dx(fc1 + 1, batch).astype(np.float64)     # grad w.r.t. fc1 output
    dw = net.layer_grad(fc1, 0).reshape(-1, 256)
    rng = np.random.default_rng(1)
    rows = rng.integers(0, dw.shape[0], 64)
    want = a[:, rows].T @ dz1
    scale = np.sqrt(np.mean(dw.astype(np.float64) ** 2))
    assert np.max(np.abs(dw[rows] - want) / np.maximum(np.abs(want), scale)) <= 1e-4
    assert_close(net.layer_grad(fc1, 1), dz1.sum(0), what="db of fc1")
    # first conv: db = sum of its output gradient over batch and pixels
    g0 = net.layer_dx(1, batch).astype(np.float64).reshape(batch, 64, -1)
    assert_close(net.layer_grad(0, 1), g0.sum(axis=(0, 2)), what="db of conv1")
    for (i, which, a0) in params:
        assert np.all(np.isfinite(net.layer_grad(i, which)))
    net.close()


def _sampled_conv_grads_match_float64(x4, w4, dy4, dw4, dx4, rng, what, taps=40, positions=48):
    """dW taps and dX positions of a 3x3 / pad same / stride 1 convolution against float64 dot
    products over the whole batch (the definition: conv2d_op_internal.h:91-169)."""
    bs, c, hw, _ = x4.shape
    oc = dy4.shape[1]
    dw_scale = np.sqrt(np.mean(dw4.astype(np.float64) ** 2))
    dx_scale = np.sqrt(np.mean(dx4.astype(np.float64) ** 2))
    worst_w = worst_x = 0.0
    for _ in range(taps):
        o, i, ky, kx = rng.integers(oc), rng.integers(c), rng.integers(3), rng.integers(3)
        # dW[o,i,ky,kx] = sum_{n,y,x} X[n,i,y+ky-1,x+kx-1] * dY[n,o,y,x] with zero padding
        y0, y1 = max(0, 1 - ky), min(hw, hw + 1 - ky)
        x0, x1 = max(0, 1 - kx), min(hw, hw + 1 - kx)
        a = x4[:, i, y0 + ky - 1:y1 + ky - 1, x0 + kx - 1:x1 + kx - 1].astype(np.float64)
        want = np.sum(a * dy4[:, o, y0:y1, x0:x1])
        worst_w = max(worst_w, abs(dw4[o, i, ky, kx] - want) / max(abs(want), dw_scale))
    for _ in range(positions):
        n, i, yy, xx = rng.integers(bs), rng.integers(c), rng.integers(hw), rng.integers(hw)
        # dX[n,i,yy,xx] = sum_{o,ky,kx} W[o,i,ky,kx] * dY[n,o,yy+1-ky,xx+1-kx]
        want = 0.0
        for ky in range(3):
            for kx in range(3):
                y, x = yy + 1 - ky, xx + 1 - kx
                if 0 <= y < hw and 0 <= x < hw:
                    want += np.dot(w4[:, i, ky, kx].astype(np.float64), dy4[n, :, y, x].astype(np.float64))
        worst_x = max(worst_x, abs(dx4[n, i, yy, xx] - want) / max(abs(want), dx_scale))
    assert worst_w <= 1e-4, f"{what}: sampled dW taps off by {worst_w:.2e}"
    assert worst_x <= 1e-4, f"{what}: sampled dX positions off by {worst_x:.2e}"
    return worst_w, worst_x


def _pool2x2_scan(x4):
    """Pooled values and the flat CHW index of the winner of every 2x2 window, scanning the
    window rows then columns and keeping the first strictly greater element
    (maxpool_op_internal.h:16-40)."""
    bs, c, h, w = x4.shape
    cand = np.stack([x4[:, :, dy::2, dx::2] for dy in (0, 1) for dx in (0, 1)], axis=-1)
    k = np.argmax(cand, axis=-1)          # the first of equal maxima, like "strictly greater"
    oy, ox = np.meshgrid(np.arange(h // 2), np.arange(w // 2), indexing="ij")
    ch = np.arange(c)[None, :, None, None]
    idx = (ch * h + (2 * oy + k // 2)) * w + 2 * ox + k % 2
    return np.take_along_axis(cand, k[..., None], axis=-1)[..., 0], idx


def test_config5_vgg_batch64_every_conv_layer_and_both_execution_modes(T, W):
    """configs[4] as it is benchmarked (batch 64, 3x128x128). Unfused (flags 0), where every
    tensor of the step is in memory: sampled dW taps and dX positions of all four convolutions
    against float64 dot products over the whole batch, every bias gradient against a float64
    sum, both max-pools against a numpy scan (indices exact). Then one momentum step fused and
    graph-replayed (the benchmark's flags): its updated parameters are those of the unfused step."""
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("vgg_stack_b64")
    xd, td = T.to_device(x), T.to_device(t)
    plain = T.Net(W.build_layers(T, spec), batch, 0)
    for (i, which, a) in params:
        plain.set_param(i, which, a)
    plain.train_step(None, loss, batch, xd, td, do_update=False)
    rng = np.random.default_rng(5)
    convs = [i for i, l in enumerate(spec) if l[0] == "conv"]
    assert len(convs) == 4
    for li in convs:
        _, hw, _, c, k, oc, _ = spec[li][:7]
        src = x if li == 0 else plain.layer_out(li - 1, batch)
        x4 = src.reshape(batch, c, hw, hw)
        dy4 = plain.layer_dx(li + 1, batch).reshape(batch, oc, hw, hw)
        dx4 = plain.layer_dx(li, batch).reshape(batch, c, hw, hw)
        w4 = plain.get_param(li, 0).reshape(oc, c, k, k)
        dw4 = plain.layer_grad(li, 0).reshape(oc, c, k, k)
        ew, ex = _sampled_conv_grads_match_float64(x4, w4, dy4, dw4, dx4, rng, f"conv layer {li}")
        assert_close(plain.layer_grad(li, 1), dy4.sum(axis=(0, 2, 3), dtype=np.float64), what=f"db of conv layer {li}")
        print(f"conv layer {li}: {c}->{oc} at {hw}x{hw}: dW taps {ew:.1e}, dX positions {ex:.1e}", flush=True)
        del x4, dy4, dx4, src
    for li in [i for i, l in enumerate(spec) if l[0] == "maxpool"]:
        _, hw, _, c, _ = spec[li]
        x4 = plain.layer_out(li - 1, batch).reshape(batch, c, hw, hw)
        want, idx = _pool2x2_scan(x4)
        assert np.array_equal(plain.layer_out(li, batch).reshape(want.shape), want), f"pool layer {li}: values"
        assert np.array_equal(plain.layer_argmax(li, batch).reshape(idx.shape), idx), f"pool layer {li}: argmax"
        # backward: the gradient goes to the winner of each window, zero elsewhere
        dy = plain.layer_dx(li + 1, batch).reshape(batch, -1)
        dx = plain.layer_dx(li, batch)
        routed = np.zeros_like(dx)
        np.put_along_axis(routed, idx.reshape(batch, -1), dy, axis=1)
        assert np.array_equal(dx, routed), f"pool layer {li}: routed gradient"
        del x4, want, idx, dy, dx, routed
    # one momentum step, unfused and as benchmarked
    opt = T.opt_desc(opt_kind, **opt_kw)
    plain.train_step(opt, loss, batch, xd, td)     # (the gradients of the pass above were kept: clear first)
    plain.close()
    results = {}
    for flags in (0, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH):
        net = T.Net(W.build_layers(T, spec), batch, flags)
        for (i, which, a) in params:
            net.set_param(i, which, a)
        net.train_step(T.opt_desc(opt_kind, **opt_kw), loss, batch, xd, td)
        results[flags] = [net.get_param(i, which) for (i, which, _) in params]
        net.close()
    for (i, which, a), p0, p3 in zip(params, results[0], results[3]):
        assert np.all(np.isfinite(p3))
        assert not np.array_equal(p0, a), f"parameter {i}.{which} did not move"
        # the two modes run the same products; what differs (activation gradients folded into
        # epilogues, split sums added by the optimizer kernel) is exact or a re-association
        assert_close(p3, p0, tol=1e-6, what=f"parameter {i}.{which} after one step, fused+graph against unfused")


def test_config5_vgg_batch64_step_matches_reference_fit(T, W):
    """One momentum step of the VGG-style stack at batch 64, fused and graph-replayed as in the
    benchmark, against what tiny-dnn's network<sequential>::fit itself computed for the same
    seeded batch and the float64 value of the same step (tests/golden/vgg_b64_step.npz: about
    4096 evenly spaced elements of every parameter tensor)."""
    import os
    from conftest import GOLDEN, input_checksum
    path = os.path.join(GOLDEN, "vgg_b64_step.npz")
    if not os.path.exists(path):
        pytest.skip("tests/golden/vgg_b64_step.npz has not been generated")
    g = np.load(path)
    key = "vgg_stack_b64@64"
    batch, steps, stride = int(g[f"{key}.batch"]), int(g[f"{key}.steps"]), int(g[f"{key}.stride"])
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("vgg_stack_b64", batch=batch)
    assert input_checksum(x, t, params) == float(g[f"{key}.input_checksum"])
    net = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
    for (i, which, a) in params:
        net.set_param(i, which, a)
    opt = T.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    for _ in range(steps):
        net.train_step(opt, loss, batch, xd, td)
    # What can be asked of this comparison. Every operator of the step is within 1e-6 of float64
    # on the tensors it is actually handed at this size, and every relu / max-pool decision is
    # exact for the values it sees (the test above and the operator tests). But the step takes
    # 130 million such decisions, and a handful of them sit within fp32 rounding of their
    # threshold: there two correct fp32 implementations (and float64) decide differently, and one
    # flipped element of a convolution's output gradient moves the 9 * Cin weight-gradient
    # entries it feeds by about 1 / sqrt(batch * pixels) of their size, 2e-3 for the last
    # convolution. tiny-dnn's own result shows the same against float64 (up to 4e-4 at the 99th
    # percentile in the first three convolutions). So: the layers behind the last such decision
    # (the two fully-connected layers) must agree with tiny-dnn to 1e-4 as everywhere else; for
    # the convolutions the error against float64 is bounded as a distribution (rms no more than
    # five times tiny-dnn's own or 5e-4, 99th percentile 3e-3, no element beyond 2e-2: a few
    # flips, not a wrong kernel, which would move every entry), and the figures are printed.
    for (i, which, a) in params:
        step = int(g[f"{key}.p{i}.{which}.stride"])
        got, ref = net.get_param(i, which)[::step].astype(np.float64), g[f"{key}.p{i}.{which}"].astype(np.float64)
        truth = g[f"{key}.p{i}.{which}.f64"]
        scale = np.maximum(np.abs(truth), np.sqrt(np.mean(truth * truth)))
        eg, eo = np.abs(got - truth) / scale, np.abs(ref - truth) / scale
        rms = lambda e: float(np.sqrt(np.mean(e * e)))
        print(f"{key} parameter {i}.{which} ({truth.size} elements) against float64: GPU rms {rms(eg):.2e} "
              f"p99 {np.quantile(eg, 0.99):.2e} max {eg.max():.2e}; tiny-dnn rms {rms(eo):.2e} "
              f"p99 {np.quantile(eo, 0.99):.2e} max {eo.max():.2e}", flush=True)
        if spec[i][0] == "fc":
            assert_close(got, ref, what=f"{key} parameter {i}.{which}")
        else:
            assert rms(eg) <= max(5 * rms(eo), 5e-4), f"{key} parameter {i}.{which}: rms error {rms(eg):.2e}"
            assert np.quantile(eg, 0.99) <= 3e-3 and eg.max() <= 2e-2, f"{key} parameter {i}.{which}"
    net.close()
