"""TDH_NET_SAMPLE_STEP: a small net trains with one workgroup per sample (forward, loss gradient
and the input gradients in one launch out of LDS), a launch for every sample's weight and bias
gradients, and the optimizer launch that adds them up (a step without an update adds them in
sample order with a launch of its own). Against the oracle (every layer output, input gradient,
max-pool record, weight and bias gradient; updated weights over several steps), against the
layer-by-layer step of the same library, against tiny-dnn's own fit (tests/golden/net_steps.npz),
and replayed from a captured graph bit for bit."""
import numpy as np
import pytest

from conftest import assert_close, input_checksum, REL_TOL
from f64_truth import assert_within_propagated_tolerance, f64_net_steps

pytestmark = pytest.mark.gpu

SAMPLE, FUSE, GRAPH = 4, 1, 2

# nets that the per-sample kernel takes: every layer kind it knows, a connection table, sizes
# that leave a column outside every pool window, each loss
NETS = {
    "lenet5": ("workload", "lenet5_b16"),
    "lenet5_c3_table": ("workload", "lenet5_mnist_b16"),
    "maxpool_relu_softmax_xent": ([("conv", 12, 12, 2, 3, 8, True), ("maxpool", 12, 12, 8, 2), ("act", "relu"),
                                   ("conv", 6, 6, 8, 3, 12, False), ("act", "leaky_relu", (0.1, 0.0)),
                                   ("fc", 12 * 16, 24), ("act", "sigmoid"), ("fc", 24, 10), ("act", "softmax")],
                                  "ce_multiclass", "adam"),
    "odd_sizes_uncovered_column_ce": ([("conv", 15, 11, 3, 5, 6, True), ("act", "tanh"), ("maxpool", 15, 11, 6, 2),
                                      ("fc", 6 * 5 * 7, 6), ("act", "sigmoid")], "ce", "momentum"),
    "fc_only_mse": ([("fc", 40, 30), ("act", "tanh"), ("fc", 30, 7)], "mse", "adagrad"),
    # unpadded stride-1 convolutions with eight or more output channels run their forward products
    # on the matrix cores: as the first layer with more pixel tiles than waves, as the layer whose
    # filters travel in registers, and with a connection table
    "valid_convs_on_matrix_cores": ([("conv", 22, 20, 3, 5, 12, False), ("act", "relu"), ("maxpool", 18, 16, 12, 2),
                                     ("conv", 9, 8, 12, 3, 16, False), ("act", "tanh"),
                                     ("conv", 7, 6, 16, 3, 8, False, [[(ci + co) % 3 != 0 for co in range(8)] for ci in range(16)]),
                                     ("act", "sigmoid"), ("fc", 8 * 5 * 4, 10), ("act", "softmax")], "ce_multiclass", "adam"),
}


def build(T, O, W, name, batch, flags, seed=3, nets=None):
    spec = (nets or NETS)[name]
    if spec[0] == "workload":
        spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(spec[1], batch=batch)
    else:
        spec, loss, opt_kind = spec
        opt_kw = {}
        rng = np.random.default_rng(seed)
        params = W.init_params(spec, "xavier", rng)
        params = [(i, which, a if which == 0 else rng.uniform(-0.1, 0.1, a.size).astype(np.float32))
                  for (i, which, a) in params]
        first = spec[0]
        n_in = first[1] * first[2] * first[3] if first[0] in ("conv", "maxpool", "avepool") else first[1]
        n_out = [l for l in spec if l[0] == "fc"][-1][2]
        x = rng.standard_normal((batch, n_in)).astype(np.float32)
        if loss == "ce":
            t = rng.uniform(0.05, 0.95, (batch, n_out)).astype(np.float32)
        elif loss == "ce_multiclass":
            t = np.eye(n_out, dtype=np.float32)[rng.integers(0, n_out, batch)]
        else:
            t = rng.uniform(-0.8, 0.8, (batch, n_out)).astype(np.float32)
    net = T.Net(W.build_layers(T, spec), batch, flags)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for (i, which, a) in params:
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    return spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref


@pytest.mark.parametrize("name", list(NETS))
@pytest.mark.parametrize("batch", [16, 5])
def test_every_tensor_of_a_sample_step_matches_oracle(T, O, W, name, batch):
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = build(T, O, W, name, batch, SAMPLE | FUSE)
    xd, td = T.to_device(x), T.to_device(t)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
    for i, l in enumerate(spec):
        assert net.out_written(i)      # the kernel writes every layer's output to memory as well
        assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), what=f"{name} layer {i} output")
        if l[0] == "maxpool":
            assert np.array_equal(net.layer_argmax(i, batch).astype(np.int64), ref.layer_argmax(i, batch)), f"{name} layer {i} argmax"
        if net.param_size(i, 0):
            assert_close(net.layer_grad(i, 0), ref.layer_dw(i), what=f"{name} layer {i} dW")
            assert_close(net.layer_grad(i, 1), ref.layer_db(i), what=f"{name} layer {i} db")
        assert net.dx_written(i)
        assert_close(net.layer_dx(i, batch), ref.layer_dx(i, batch), what=f"{name} layer {i} dX")
    # a second backward pass adds to the weight gradients (layer.h:680 clears them at the update)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    for (i, which, _) in params:
        want = 2.0 * (ref.layer_dw(i) if which == 0 else ref.layer_db(i))
        assert_close(net.layer_grad(i, which), want, what=f"{name} gradient {i}.{which} after two passes")
    net.close()


@pytest.mark.parametrize("name", list(NETS))
def test_updated_weights_of_sample_steps_match_oracle_and_the_layered_step(T, O, W, name):
    """Three optimizer steps: against the oracle, and the captured replay (flags 7) bit for bit
    against eager launches (flags 5); a short last batch goes through the same kernels."""
    batch, steps = 16, 3
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = build(T, O, W, name, batch, SAMPLE | FUSE)
    *_, replay, _ = build(T, O, W, name, batch, SAMPLE | FUSE | GRAPH)
    *_, layered, _ = build(T, O, W, name, batch, FUSE)
    opts = [T.opt_desc(opt_kind, **opt_kw) for _ in range(3)]
    ropt = O.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    sizes = [batch, batch, 7] if opt_kind != "adagrad" else [batch] * steps   # (the float64 helper steps whole batches)
    for n in sizes:
        for k, m in enumerate((net, replay, layered)):
            m.train_step(opts[k], loss, n, xd, td)
        ref.train_step(ropt, loss, x[:n], t[:n])
    truth = None
    if opt_kind == "adagrad":      # see test_updated_weights_match_oracle in test_gpu_nets.py
        o64 = {"kind": "adagrad", "alpha": opts[0].alpha}
        truth, trace = f64_net_steps(spec, params, x, t, loss, steps, o64, want_trace=True)
    for (i, which, a) in params:
        got, want = net.get_param(i, which), (ref.weight(i) if which == 0 else ref.bias(i))
        assert np.array_equal(got, replay.get_param(i, which)), f"{name} parameter {i}.{which}: replay differs from eager"
        if truth is not None:
            assert_within_propagated_tolerance(got, want, truth[(i, which)], o64, trace[(i, which)],
                                               f"{name} updated parameter {i}.{which}")
        else:
            assert_close(got, want, what=f"{name} updated parameter {i}.{which}")
            assert_close(got, layered.get_param(i, which), what=f"{name} parameter {i}.{which} against the layered step")
        assert not net.layer_grad(i, which).any()
    assert opts[0].b1_t == ropt.b1_t == opts[1].b1_t and opts[0].b2_t == ropt.b2_t
    for m in (net, replay, layered):
        m.close()


@pytest.mark.parametrize("key", ["lenet5_b16", "lenet5_mnist_b16"])
def test_sample_steps_match_reference_fit(T, W, net_steps, key):
    """Against what tiny-dnn's network<sequential>::fit itself produced, replayed from a graph."""
    g = net_steps
    batch, steps, stride = int(g[f"{key}.batch"]), int(g[f"{key}.steps"]), int(g[f"{key}.stride"])
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(key, batch=batch)
    assert input_checksum(x, t, params) == float(g[f"{key}.input_checksum"])
    net = T.Net(W.build_layers(T, spec), batch, SAMPLE | FUSE | GRAPH)
    for (i, which, a) in params:
        net.set_param(i, which, a)
    opt = T.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    for _ in range(steps):
        net.train_step(opt, loss, batch, xd, td)
    truth = None
    if opt_kind == "adagrad":
        o64 = {"kind": "adagrad", "alpha": opt.alpha}
        truth, trace = f64_net_steps(spec, params, x, t, loss, steps, o64, want_trace=True)
    for (i, which, a) in params:
        got = net.get_param(i, which)
        if truth is not None:
            assert_within_propagated_tolerance(got, g[f"{key}.p{i}.{which}"], truth[(i, which)], o64,
                                               trace[(i, which)], f"{key} parameter {i}.{which}")
        else:
            assert_close(got[::stride], g[f"{key}.p{i}.{which}"], what=f"{key} parameter {i}.{which}")
    net.close()


def test_nets_that_do_not_qualify_ignore_the_flag(T, O, W):
    """Batch normalization, or more arithmetic per sample than the kernel is meant for: the flag
    changes nothing, the layer-by-layer step runs (same bits as without the flag)."""
    for spec, batch in (([("fc", 12, 8), ("batchnorm", 8, 1), ("act", "relu"), ("fc", 8, 4)], 6),
                        (W.cifar10_cnn(), 4)):
        rng = np.random.default_rng(8)
        params = W.init_params([l for l in spec], "xavier", rng)
        first = spec[0]
        n_in = first[1] * first[2] * first[3] if first[0] == "conv" else first[1]
        n_out = [l for l in spec if l[0] == "fc"][-1][2]
        x = rng.standard_normal((batch, n_in)).astype(np.float32)
        t = np.eye(n_out, dtype=np.float32)[rng.integers(0, n_out, batch)]
        loss = "ce_multiclass" if spec[-1][0] == "act" else "mse"
        got = []
        for flags in (FUSE, FUSE | SAMPLE):
            net = T.Net(W.build_layers(T, spec), batch, flags)
            for (i, which, a) in params:
                net.set_param(i, which, a)
            net.train_step(T.opt_desc("sgd"), loss, batch, T.to_device(x), T.to_device(t))
            got.append([net.get_param(i, which) for (i, which, _) in params])
            net.close()
        for a, b in zip(*got):
            assert np.array_equal(a, b)


def _random_small_net(rng):
    """A random net that the per-sample kernel takes: one to three convolutions (3x3 or 5x5, with
    and without padding, 1 to 12 channels), pools that leave rows or columns uncovered, every
    activation it knows, one or two fully-connected layers, each loss."""
    def act():
        a = str(rng.choice(["relu", "tanh", "sigmoid", "leaky_relu"]))
        return ("act", a, (0.1, 0.0)) if a == "leaky_relu" else ("act", a)
    w, h, c = int(rng.choice([6, 8, 10, 12, 14, 16])), int(rng.choice([6, 8, 10, 12, 13])), int(rng.choice([1, 2, 3, 6]))
    spec = []
    for _ in range(int(rng.integers(1, 4))):
        k, oc, same = int(rng.choice([3, 5])), int(rng.choice([1, 3, 4, 5, 6, 8, 12])), bool(rng.integers(0, 2))
        same = same or w < k or h < k
        spec.append(("conv", w, h, c, k, oc, same))
        if not same:
            w, h = w - k + 1, h - k + 1
        c = oc
        order = int(rng.integers(0, 4))
        if order in (1, 3):
            spec.append(act())
        if w >= 4 and h >= 4 and rng.random() < 0.7:
            if rng.random() < 0.5:
                spec.append(("maxpool", w, h, c, 2))
                w, h = w // 2, h // 2
            elif w % 2 == 0 and h % 2 == 0:
                spec.append(("avepool", w, h, c, 2))
                w, h = w // 2, h // 2
            if order in (2, 3):
                spec.append(act())
    if rng.random() < 0.6:
        hid = int(rng.choice([7, 10, 24]))
        spec += [("fc", c * w * h, hid), act(), ("fc", hid, 10)]
    else:
        spec.append(("fc", c * w * h, 10))
    r = rng.random()
    if r < 0.4:
        return spec + [("act", "softmax")], "ce_multiclass"
    if r < 0.6:
        return spec + [("act", "sigmoid")], "ce"
    return spec, "mse"


def test_random_small_nets_match_oracle(T, O, W):
    """A seeded sweep: every layer output, input gradient, weight and bias gradient of one
    backward pass, then the weights after three steps, eager or replayed."""
    rng = np.random.default_rng(20)
    for case in range(40):
        spec, loss = _random_small_net(rng)
        batch = int(rng.choice([1, 3, 5, 16, 33]))
        flags = int(rng.choice([SAMPLE | FUSE, SAMPLE | FUSE | GRAPH]))
        tag = f"case {case} (batch {batch}, flags {flags}, {loss}, {spec})"
        params = []
        for i, l in enumerate(spec):
            nw, nb, fan_in, _ = W.layer_fans(l)
            if nw:
                wv = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
                if l[0] == "avepool":
                    wv = rng.uniform(0.5, 1.5, nw).astype(np.float32)
                params += [(i, 0, wv), (i, 1, rng.uniform(-0.2, 0.2, nb).astype(np.float32))]
        first = spec[0]
        x = rng.standard_normal((batch, first[1] * first[2] * first[3])).astype(np.float32)
        t = (np.eye(10, dtype=np.float32)[rng.integers(0, 10, batch)] if loss == "ce_multiclass"
             else rng.uniform(0.1, 0.9, (batch, 10)).astype(np.float32))
        xd, td = T.to_device(x), T.to_device(t)
        kind = str(rng.choice(["momentum", "sgd"]))

        def pair():
            net, ref = T.Net(W.build_layers(T, spec), batch, flags), O.OracleNet(W.build_layers(O, spec), batch)
            for (i, which, a) in params:
                net.set_param(i, which, a)
                (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
            return net, ref
        net, ref = pair()
        net.train_step(None, loss, batch, xd, td, do_update=False)
        ref.train_step(O.opt_desc(kind), loss, x, t, do_update=False)
        for i, l in enumerate(spec):
            assert net.out_written(i) and net.dx_written(i), f"{tag}: the per-sample kernel did not run"
            assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), what=f"{tag} layer {i} output")
            assert_close(net.layer_dx(i, batch), ref.layer_dx(i, batch), what=f"{tag} layer {i} dX")
            if l[0] == "maxpool":
                got, want = net.layer_argmax(i, batch).astype(np.int64), ref.layer_argmax(i, batch)
                if not np.array_equal(got, want):   # (another winner only where both hold the same value to rounding)
                    pin, rows = ref.layer_out(i - 1, batch), np.arange(batch)[:, None]
                    tol = 1e-5 * np.maximum(np.abs(pin[rows, want]), np.sqrt(np.mean(pin * pin)))
                    assert np.all(np.abs(pin[rows, got] - pin[rows, want]) <= tol), f"{tag} layer {i} argmax"
            if W.layer_fans(l)[0]:
                assert_close(net.layer_grad(i, 0), ref.layer_dw(i), what=f"{tag} layer {i} dW")
                assert_close(net.layer_grad(i, 1), ref.layer_db(i), what=f"{tag} layer {i} db")
        net.close()
        net, ref = pair()
        # (a rate at which three steps on summed gradients stay finite for every loss)
        opt, ropt = T.opt_desc(kind, alpha=1e-3), O.opt_desc(kind, alpha=1e-3)
        for _ in range(3):
            net.train_step(opt, loss, batch, xd, td)
            ref.train_step(ropt, loss, x, t)
        for (i, which, _) in params:
            want = ref.weight(i) if which == 0 else ref.bias(i)
            assert np.isfinite(want).all(), f"{tag}: the oracle's step diverged"
            assert_close(net.get_param(i, which), want, 2e-4, what=f"{tag} parameter {i}.{which} after three steps")
        net.close()


NO_INPUT_GRAD = 8
INPUT_GRAD_NETS = dict(NETS, cifar10=("workload", "cifar10_cnn_b128"),
                       fc_first_large=([("fc", 300, 200), ("act", "relu"), ("fc", 200, 10), ("act", "softmax")],
                                       "ce_multiclass", "adam"),
                       valid_conv_first=([("conv", 13, 13, 2, 3, 5, False), ("act", "tanh"), ("fc", 5 * 121, 4)],
                                         "mse", "sgd"))


@pytest.mark.parametrize("flags", [0, FUSE, FUSE | GRAPH, SAMPLE | FUSE, SAMPLE | FUSE | GRAPH])
@pytest.mark.parametrize("name", list(INPUT_GRAD_NETS))
def test_step_without_the_input_gradient_changes_nothing_else(T, O, W, name, flags):
    """TDH_NET_NO_INPUT_GRAD leaves out the first layer's input gradient (layer.h:557-575 computes
    it, training never reads it): that gradient is reported as not written, every other tensor
    of a pass and the weights after three updates are bit for bit those of the net without the flag."""
    batch = 16
    spec, params, x, t, batch, loss, opt_kind, opt_kw, full, ref = build(T, O, W, name, batch, flags, nets=INPUT_GRAD_NETS)
    *_, lean, _ = build(T, O, W, name, batch, flags | NO_INPUT_GRAD, nets=INPUT_GRAD_NETS)
    xd, td = T.to_device(x), T.to_device(t)
    for m in (full, lean):
        m.train_step(None, loss, batch, xd, td, do_update=False)
    ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
    assert full.dx_written(0) and not lean.dx_written(0)
    assert_close(full.layer_dx(0, batch), ref.layer_dx(0, batch), what=f"{name} input gradient")
    for i, l in enumerate(spec):
        assert full.out_written(i) == lean.out_written(i)
        if full.out_written(i):
            assert np.array_equal(full.layer_out(i, batch), lean.layer_out(i, batch)), f"{name} layer {i} output"
        if i:
            assert full.dx_written(i) == lean.dx_written(i)
            if full.dx_written(i):
                assert np.array_equal(full.layer_dx(i, batch), lean.layer_dx(i, batch)), f"{name} layer {i} dX"
        for which in (0, 1):
            if full.param_size(i, which):
                assert np.array_equal(full.layer_grad(i, which), lean.layer_grad(i, which)), f"{name} gradient {i}.{which}"
                want = ref.layer_dw(i) if which == 0 else ref.layer_db(i)
                assert_close(lean.layer_grad(i, which), want, what=f"{name} gradient {i}.{which}")
    opts = [T.opt_desc(opt_kind, **opt_kw) for _ in range(2)]
    for m in (full, lean):
        m.clear_grads()
    for n in (batch, batch, 7):
        for m, o in zip((full, lean), opts):
            m.train_step(o, loss, n, xd, td)
    for (i, which, _) in params:
        assert np.array_equal(full.get_param(i, which), lean.get_param(i, which)), f"{name} parameter {i}.{which}"
    assert not lean.dx_written(0)
    full.close()
    lean.close()


def test_first_layers_of_other_kinds_ignore_the_input_gradient_flag(T, O, W):
    nets = {"pool_first": ([("maxpool", 8, 8, 3, 2), ("fc", 48, 5)], "mse", "sgd")}
    for flags in (0, FUSE | GRAPH, SAMPLE | FUSE):
        spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = build(T, O, W, "pool_first", 6, flags | NO_INPUT_GRAD, nets=nets)
        net.train_step(None, loss, batch, T.to_device(x), T.to_device(t), do_update=False)
        ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
        assert net.dx_written(0)
        assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), what="input gradient of a net that starts with a pool")
        net.close()
