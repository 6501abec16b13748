"""Whole train steps (fprop, loss gradient, bprop, update) on the MI355X against the oracle
and against the parameters tiny-dnn's own network<sequential>::fit produced
(tests/golden/net_steps.npz). All through the C ABI (tdh_net_*)."""
import numpy as np
import pytest

from conftest import assert_close, input_checksum, REL_TOL
from f64_truth import assert_within_propagated_tolerance, f64_net_steps

pytestmark = pytest.mark.gpu


def make_pair(T, O, W, name, batch, flags, size=None):
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch, size=size)
    net = T.Net(W.build_layers(T, spec), batch, flags)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for (i, which, a) in params:
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    return spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref


CASES = [("lenet5_b16", 16, None), ("cifar10_cnn_b128", 8, None), ("vgg_stack_b64", 2, 16),
         ("lenet5_mnist_b16", 16, None)]   # the last one: C3 with LeNet-5's connection table


@pytest.mark.parametrize("name,batch,size", CASES)
@pytest.mark.parametrize("flags", [0, 1])
def test_gradients_of_every_layer_match_oracle(T, O, W, name, batch, size, flags):
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = make_pair(T, O, W, name, batch, flags, size)
    xd, td = T.to_device(x), T.to_device(t)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
    for i, l in enumerate(spec):
        if net.out_written(i):
            assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), what=f"{name} layer {i} output")
        if l[0] == "maxpool":
            assert np.array_equal(net.layer_argmax(i, batch).astype(np.int64),
                                  ref.layer_argmax(i, batch)), f"{name} layer {i} argmax"
        if net.param_size(i, 0):
            assert_close(net.layer_grad(i, 0), ref.layer_dw(i), what=f"{name} layer {i} dW")
            assert_close(net.layer_grad(i, 1), ref.layer_db(i), what=f"{name} layer {i} db")
    assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), what=f"{name} input gradient")
    net.close()


@pytest.mark.parametrize("name,batch,size,steps", [("lenet5_b16", 16, None, 3), ("cifar10_cnn_b128", 8, None, 3),
                                                   ("vgg_stack_b64", 2, 16, 1), ("lenet5_mnist_b16", 16, None, 3)])
@pytest.mark.parametrize("flags", [0, 1])
def test_updated_weights_match_oracle(T, O, W, name, batch, size, steps, flags):
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = make_pair(T, O, W, name, batch, flags, size)
    opt, ropt = T.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    for _ in range(steps):
        net.train_step(opt, loss, batch, xd, td)
        ref.train_step(ropt, loss, x, t)
    # adagrad divides every gradient element by its own accumulated magnitude, so the elements
    # of dW that nearly cancel carry their relative rounding error into the weight at full size
    # (1.9e-3 between GPU and oracle for a few of the 48 000 weights of C5 after three steps,
    # the oracle itself 5e-4 from float64): there the bound is the one the gradient tolerance
    # implies, against the float64 step
    truth = None
    if opt_kind == "adagrad":
        o64 = {"kind": "adagrad", "alpha": opt.alpha}
        truth, trace = f64_net_steps(spec, params, x, t, loss, steps, o64, want_trace=True)
    for (i, which, a) in params:
        want = ref.weight(i) if which == 0 else ref.bias(i)
        if truth is not None:
            assert_within_propagated_tolerance(net.get_param(i, which), want, truth[(i, which)], o64,
                                               trace[(i, which)], f"{name} updated parameter {i}.{which}")
        else:
            assert_close(net.get_param(i, which), want, what=f"{name} updated parameter {i}.{which}")
    assert opt.b1_t == ropt.b1_t and opt.b2_t == ropt.b2_t
    # gradients are cleared after the update (layer.h:680)
    for (i, which, a) in params:
        assert not net.layer_grad(i, which).any()
    net.close()


@pytest.mark.parametrize("key,flags", [("lenet5_b16", 1), ("cifar10_cnn_b128", 1), ("cifar10_cnn_b128@128", 3),
                                       ("lenet5_mnist_b16", 1), ("lenet5_mnist_b16", 3)])
def test_updated_weights_match_reference_fit(T, W, net_steps, key, flags):
    """Against what tiny-dnn's network<sequential>::fit itself produced; "@128" is the CIFAR-10
    net at the batch it is benchmarked at, stepped the way the benchmark steps it (folded
    activation gradients, captured graph, weight-gradient branches on side streams)."""
    g = net_steps
    name = key.split("@")[0]
    batch, steps, stride = int(g[f"{key}.batch"]), int(g[f"{key}.steps"]), int(g[f"{key}.stride"])
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
    assert input_checksum(x, t, params) == float(g[f"{key}.input_checksum"])
    net = T.Net(W.build_layers(T, spec), batch, flags)
    for (i, which, a) in params:
        net.set_param(i, which, a)
    opt = T.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    for _ in range(steps):
        net.train_step(opt, loss, batch, xd, td)
    truth = None
    if opt_kind == "adagrad":   # see test_updated_weights_match_oracle
        o64 = {"kind": "adagrad", "alpha": opt.alpha}
        truth, trace = f64_net_steps(spec, params, x, t, loss, steps, o64, want_trace=True)
    for (i, which, a) in params:
        got = net.get_param(i, which)
        if truth is not None:
            assert stride == 1
            assert_within_propagated_tolerance(got, g[f"{key}.p{i}.{which}"], truth[(i, which)], o64,
                                               trace[(i, which)], f"{key} parameter {i}.{which}")
        else:
            assert_close(got[::stride], g[f"{key}.p{i}.{which}"], what=f"{key} parameter {i}.{which}")
    net.close()


def relu_sign_flips(net, ref, spec, batch):
    """The last relu layer at which the GPU and the oracle disagree about the sign of an element
    (-1: none). relu' jumps at zero, so a pre-activation that both sides compute as zero to
    rounding (checked here: within 1e-5 of the tensor's rms) can come out positive on one side
    and negative on the other; every gradient in front of that layer then legitimately differs
    at the positions the element feeds. With millions of activations this happens (VGG stack at
    128x128, batch 2: one element of 6 million, -1.7e-6 against +2.2e-7 at an rms of 2.5)."""
    last = -1
    for i, l in enumerate(spec):
        if l[0] == "act" and l[1] == "relu":
            yg, yr = net.layer_out(i, batch), ref.layer_out(i, batch)
            flips = (yg > 0) != (yr > 0)
            if flips.any():
                if spec[i - 1][0] in ("conv", "fc"):     # the layer in front holds the pre-activation
                    pre_r = ref.layer_out(i - 1, batch)
                    # (a train step may have kept the convolution's own output in registers: the
                    # relu output is the pre-activation wherever it is positive)
                    pre_g = net.layer_out(i - 1, batch) if net.out_written(i - 1) else yg
                    rms = np.sqrt(np.mean(pre_r.astype(np.float64) ** 2))
                    assert np.all(np.abs(pre_g[flips]) < 1e-5 * rms) and np.all(np.abs(pre_r[flips]) < 1e-5 * rms), \
                        f"layer {i}: relu outputs differ in sign away from zero"
                assert flips.sum() <= 1e-5 * flips.size + 1
                last = i
    return last


def check_every_layer(net, ref, spec, batch, name, fused, passes=1, cancelling_db=()):
    flipped = relu_sign_flips(net, ref, spec, batch)
    for i, l in enumerate(spec):
        if net.out_written(i):
            assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), what=f"{name} layer {i} output")
        if l[0] == "maxpool":
            assert np.array_equal(net.layer_argmax(i, batch).astype(np.int64),
                                  ref.layer_argmax(i, batch)), f"{name} layer {i} argmax"
        if i <= flipped:
            continue      # gradients in front of a flipped relu element: see relu_sign_flips
        if net.param_size(i, 0):
            # weight gradients add up over backward passes until an update clears them
            # (layer.h:680); the oracle's net holds one pass
            assert_close(net.layer_grad(i, 0), passes * ref.layer_dw(i), what=f"{name} layer {i} dW")
            if i in cancelling_db:
                # the bias of a convolution in front of a batch normalization has no effect on the
                # loss: its gradient is a sum that cancels to rounding, so it is measured
                # against the sum of the magnitudes that were added up
                c = net.param_size(i, 1)
                mag = np.abs(ref.layer_dx(i + 1, batch).astype(np.float64)).reshape(batch, c, -1).sum(axis=(0, 2))
                err = np.abs(net.layer_grad(i, 1).astype(np.float64) - passes * ref.layer_db(i))
                assert np.all(err <= 1e-5 * mag), f"{name} layer {i} db: {err.max():.3e} of {mag.min():.3e}"
            else:
                assert_close(net.layer_grad(i, 1), passes * ref.layer_db(i), what=f"{name} layer {i} db")
        # the gradient with respect to a layer's input. A fusing net leaves two kinds unwritten:
        # the gradient of a folded activation's OUTPUT (it only ever exists in registers), and
        # the input gradient of a max-pool behind a first convolution whose backward kernels read
        # the pooled gradient and the argmax records themselves
        if net.dx_written(i):
            assert_close(net.layer_dx(i, batch), ref.layer_dx(i, batch), what=f"{name} layer {i} dX")
        else:
            assert fused and i >= 1 and (
                (spec[i - 1][0] == "act" and spec[i - 1][1] in ("tanh", "relu", "sigmoid")) or
                (l[0] == "maxpool" and spec[i - 1][0] == "conv")), f"{name} layer {i} dX is missing"
    return flipped


def test_cifar_net_at_the_benchmarked_batch_and_flags_matches_oracle(T, O, W):
    """configs[3] exactly as bench.py runs it: batch 128, folded activation gradients, the step
    captured into a graph (at this batch one chain of launches: the first layer's three gradients
    from one launch, every weight gradient's split sums left to the optimizer kernel). Every
    layer's output, argmax, dW, db and dX, then the parameters after each of two Adam steps."""
    name = "cifar10_cnn_b128"
    flags = T.NET_FUSE_ACT_GRAD | T.NET_GRAPH
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = make_pair(T, O, W, name, None, flags)
    assert batch == 128
    xd, td = T.to_device(x), T.to_device(t)
    ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
    for rep in range(2):       # the second pass replays the captured gradient-only step
        net.train_step(None, loss, batch, xd, td, do_update=False)
        check_every_layer(net, ref, spec, batch, f"{name} pass {rep}", True, passes=rep + 1)
    net.train_step(T.opt_desc("sgd", alpha=0.0), loss, batch, xd, td)   # clears the gradients
    opt, ropt = T.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
    for step in range(2):
        net.train_step(opt, loss, batch, xd, td)
        ref.train_step(ropt, loss, x, t)
        for (i, which, a) in params:
            want = ref.weight(i) if which == 0 else ref.bias(i)
            assert_close(net.get_param(i, which), want, what=f"{name} step {step} parameter {i}.{which}")
    assert opt.b1_t == ropt.b1_t and opt.b2_t == ropt.b2_t
    net.close()


@pytest.mark.parametrize("flags", [1, 3])
def test_vgg_layers_at_full_image_size_match_oracle(T, O, W, flags):
    """configs[4] at its real 3x128x128 input (every convolution at the tile plans of the full
    workload's image size), batch 2. The net as a whole: every output and argmax, and every
    gradient behind the last relu element whose sign differs (see relu_sign_flips). Then every
    convolution, max-pool and fully-connected layer's backward pass on its own, fed with the
    ORACLE's tensors of that layer, so that all of them are checked whatever flipped."""
    name = "vgg_stack_b64"
    spec, params, x, t, batch, loss, opt_kind, opt_kw, net, ref = make_pair(T, O, W, name, 2, flags, 128)
    xd, td = T.to_device(x), T.to_device(t)
    net.train_step(None, loss, batch, xd, td, do_update=False)
    ref.train_step(O.opt_desc(opt_kind), loss, x, t, do_update=False)
    flipped = check_every_layer(net, ref, spec, batch, name, True)
    print(f"last relu layer with a sign flip: {flipped}")
    for i, l in enumerate(spec):
        xin = x if i == 0 else ref.layer_out(i - 1, batch)
        dy = ref.layer_dx(i + 1, batch) if i + 1 < len(spec) else None
        if l[0] == "conv":
            _, w_, h_, c_, k_, oc_, same = l[:7]
            d = T.conv_desc(w_, h_, c_, k_, k_, oc_, pad_same=same)
            dx, dw, db = T.DevBuf(xin.shape), T.DevBuf((ref.weight(i).size,)), T.DevBuf((oc_,))
            T.conv2d_bwd(d, batch, T.to_device(xin), T.to_device(ref.weight(i)), T.to_device(dy), dx, dw, db)
            assert_close(dx.numpy(), ref.layer_dx(i, batch), what=f"conv layer {i} dX on its own")
            assert_close(dw.numpy(), ref.layer_dw(i), what=f"conv layer {i} dW on its own")
            assert_close(db.numpy(), ref.layer_db(i), what=f"conv layer {i} db on its own")
        elif l[0] == "fc":
            dx, dw, db = T.DevBuf(xin.shape), T.DevBuf((l[1] * l[2],)), T.DevBuf((l[2],))
            T.fc_bwd(l[1], l[2], True, batch, T.to_device(xin), T.to_device(ref.weight(i)), T.to_device(dy),
                     dx, dw, db)
            assert_close(dx.numpy(), ref.layer_dx(i, batch), what=f"fc layer {i} dX on its own")
            assert_close(dw.numpy(), ref.layer_dw(i), what=f"fc layer {i} dW on its own")
            assert_close(db.numpy(), ref.layer_db(i), what=f"fc layer {i} db on its own")
        elif l[0] == "maxpool":
            d = T.pool_desc(l[1], l[2], l[3], l[4])
            dx = T.DevBuf(xin.shape)
            T.maxpool_bwd(d, batch, T.to_device(dy), T.to_device(ref.layer_argmax(i, batch), np.int32), dx)
            assert np.array_equal(dx.numpy(), ref.layer_dx(i, batch)), f"max-pool layer {i} dX on its own"
        elif l[1] == "relu":
            dx = T.DevBuf(xin.shape)
            T.act_bwd("relu", batch, xin.shape[1], T.to_device(ref.layer_out(i, batch)), T.to_device(dy), dx)
            assert np.array_equal(dx.numpy(), ref.layer_dx(i, batch)), f"relu layer {i} dX on its own"
    if flipped < 0:    # one momentum step of the whole net
        opt, ropt = T.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
        net.train_step(opt, loss, batch, xd, td)
        ref.train_step(ropt, loss, x, t)
        for (i, which, a) in params:
            want = ref.weight(i) if which == 0 else ref.bias(i)
            assert_close(net.get_param(i, which), want, what=f"{name} parameter {i}.{which}")
    net.close()


def test_step_is_reproducible_bit_for_bit(T, W):
    """Fixed-order reductions: the same inputs give the same bits, run after run."""
    outs = []
    for _ in range(3):
        spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("cifar10_cnn_b128", batch=32)
        net = T.Net(W.build_layers(T, spec), batch, 1)
        for (i, which, a) in params:
            net.set_param(i, which, a)
        opt = T.opt_desc(opt_kind, **opt_kw)
        xd, td = T.to_device(x), T.to_device(t)
        for _ in range(2):
            net.train_step(opt, loss, batch, xd, td)
        outs.append([net.get_param(i, which) for (i, which, a) in params])
        net.close()
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert np.array_equal(a, b)


def test_smaller_batch_than_max_and_forward_only(T, O, W):
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch("cifar10_cnn_b128", batch=5)
    net = T.Net(W.build_layers(T, spec), 16, 0)            # max_batch 16, run 5
    ref = O.OracleNet(W.build_layers(O, spec), 5)
    for (i, which, a) in params:
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    net.forward(5, T.to_device(x))
    assert_close(net.layer_out(len(spec) - 1, 5), ref.forward(x))
    with pytest.raises(T.TdhError):
        net.forward(17, T.to_device(np.zeros((17, x.shape[1]), np.float32)))
    net.close()


@pytest.mark.parametrize("name,batch,flags", [("cifar10_cnn_b128", 16, 3), ("cifar10_cnn_b128", 16, 1),
                                              ("lenet5_b16", 16, 7), ("lenet5_b16", 16, 3), ("lenet5_mnist_b16", 8, 0),
                                              ("cifar10_cnn_b128", 16, 3 | 8), ("lenet5_b16", 5, 7 | 8)])
def test_several_steps_in_one_call_equal_single_steps(T, W, name, batch, flags):
    """tdh_net_train_steps: up to eight steps a call (one captured graph with TDH_NET_GRAPH), on
    batches that change from step to step, leave bit for bit the weights of as many single steps;
    adam's powers keep taking turns between their two buffers across calls of odd length."""
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
    nets = [T.Net(W.build_layers(T, spec), batch, flags) for _ in range(2)]
    for net in nets:
        for (i, which, a) in params:
            net.set_param(i, which, a)
    opts = [T.opt_desc(opt_kind, **opt_kw) for _ in range(2)]
    rng = np.random.default_rng(17)
    batches = []
    for k in range(3):   # three mini-batches that take turns
        p = rng.permutation(batch)
        batches.append((T.to_device(np.ascontiguousarray(x[p] * np.float32(1.0 - 0.1 * k))), T.to_device(np.ascontiguousarray(t[p]))))
    at = 0
    for n in (3, 2, 5, 1, 8, 3):
        use = [batches[(at + s) % 3] for s in range(n)]
        at += n
        nets[0].train_steps(opts[0], loss, batch, [b[0] for b in use], [b[1] for b in use])
        for (xb, tb) in use:
            nets[1].train_step(opts[1], loss, batch, xb, tb)
        for (i, which, _) in params:
            assert np.array_equal(nets[0].get_param(i, which), nets[1].get_param(i, which)), \
                f"{name} flags {flags}: parameter {i}.{which} after a call of {n} steps"
        assert opts[0].b1_t == opts[1].b1_t and opts[0].b2_t == opts[1].b2_t
    with pytest.raises(T.TdhError, match="steps a call"):
        nets[0].train_steps(opts[0], loss, batch, [batches[0][0]] * 9, [batches[0][1]] * 9)
    for net in nets:
        net.close()


def test_net_rejects_inconsistent_layers(T):
    with pytest.raises(T.TdhError, match="expects"):
        T.Net([T.L_fc(10, 5), T.L_fc(6, 2)], 4)
    with pytest.raises(T.TdhError, match="first layer"):
        T.Net([T.L_act("relu"), T.L_fc(6, 2)], 4)
    # a net is trained, and the reference's backward pass has no defined result with a dilation
    dilated = T.L_conv(8, 8, 2, 3, 4)
    dilated.conv.w_dilation = dilated.conv.h_dilation = 2
    with pytest.raises(T.TdhError, match="dilation"):
        T.Net([dilated, T.L_fc(4 * 4 * 4, 2)], 4)


# (the CIFAR net branches at batch 16 and runs as one chain, its first layer's gradients from one
# launch, at batch 128)
@pytest.mark.parametrize("name,batch", [("cifar10_cnn_b128", 16), ("cifar10_cnn_b128", 128), ("lenet5_b16", 16)])
def test_graph_replay_matches_eager_on_every_step(T, W, name, batch):
    """TDH_NET_GRAPH: the captured step is replayed five times with eager work, readbacks and
    synchronisations in between; after every replay all parameters equal the eager net's bit
    for bit (same kernels, same order), including Adam's per-tensor bias-correction powers."""
    spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
    eager = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD)
    graph = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
    for (i, which, a) in params:
        eager.set_param(i, which, a)
        graph.set_param(i, which, a)
    o1, o2 = T.opt_desc(opt_kind, **opt_kw), T.opt_desc(opt_kind, **opt_kw)
    xd, td = T.to_device(x), T.to_device(t)
    side_in = T.to_device(np.linspace(-2, 2, 4096, dtype=np.float32)[None])
    side_out = T.DevBuf((1, 4096))
    for step in range(5):
        eager.train_step(o1, loss, batch, xd, td)
        graph.train_step(o2, loss, batch, xd, td)
        T.act_fwd("tanh", 1, 4096, side_in, side_out)      # unrelated eager work in between
        T.sync()
        assert side_out.numpy()[0, 0] == np.float32(np.tanh(np.float32(-2.0)))
        for (i, which, a) in params:
            assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (step, i, which)
        assert o1.b1_t == o2.b1_t and o1.b2_t == o2.b2_t
    # a changed optimizer object (new hyper-parameter, reset powers) is honoured
    o1.alpha = o2.alpha = 0.5 * o1.alpha
    o1.b1_t = o2.b1_t = 0.9
    eager.train_step(o1, loss, batch, xd, td)
    graph.train_step(o2, loss, batch, xd, td)
    for (i, which, a) in params:
        assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (i, which)
    # another batch size re-captures
    eager.train_step(o1, loss, batch // 2, xd, td)
    graph.train_step(o2, loss, batch // 2, xd, td)
    for (i, which, a) in params:
        assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (i, which)
    # gradients without update through the graph path as well
    eager.train_step(None, loss, batch, xd, td, do_update=False)
    graph.train_step(None, loss, batch, xd, td, do_update=False)
    for (i, which, a) in params:
        assert np.array_equal(eager.layer_grad(i, which), graph.layer_grad(i, which))
    # what a step keeps out of memory is reported the same way after a replay; a forward pass
    # writes every output, and the next replay reports its own state again
    n = len(spec)
    kept_out = [graph.out_written(i) for i in range(n)]
    assert kept_out == [eager.out_written(i) for i in range(n)]
    assert [graph.dx_written(i) for i in range(n)] == [eager.dx_written(i) for i in range(n)]
    graph.forward(batch, xd)
    eager.forward(batch, xd)
    assert all(graph.out_written(i) for i in range(n))
    for i in range(n):
        assert np.array_equal(graph.layer_out(i, batch), eager.layer_out(i, batch)), i
    eager.train_step(o1, loss, batch, xd, td)
    graph.train_step(o2, loss, batch, xd, td)
    assert [graph.out_written(i) for i in range(n)] == [eager.out_written(i) for i in range(n)]
    for (i, which, a) in params:
        assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (i, which)
    eager.close(); graph.close()


@pytest.mark.parametrize("opt_kind", ["sgd", "momentum", "nesterov", "adagrad", "rmsprop", "adamax"])
def test_branching_replay_matches_eager_for_every_optimizer(T, W, opt_kind):
    """The replayed step of a net that branches leaves the weight gradients' split sums to the
    optimizer kernel and keeps the bias-correction powers in two device buffers that take turns:
    four steps of every optimizer kind give bit for bit the weights (and host-side powers) of
    eager steps, which run the reductions as launches of their own."""
    spec, params, x, t, _, loss, _, _ = W.make_batch("cifar10_cnn_b128", batch=16)
    batch = 16
    eager = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD)
    graph = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
    for (i, which, a) in params:
        eager.set_param(i, which, a)
        graph.set_param(i, which, a)
    o1, o2 = T.opt_desc(opt_kind), T.opt_desc(opt_kind)
    xd, td = T.to_device(x), T.to_device(t)
    for step in range(4):
        eager.train_step(o1, loss, batch, xd, td)
        graph.train_step(o2, loss, batch, xd, td)
        for (i, which, a) in params:
            assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (step, i, which)
        assert o1.b1_t == o2.b1_t and o1.b2_t == o2.b2_t
    eager.close(); graph.close()


def test_branching_replay_with_ragged_gradient_tensors_matches_eager_and_oracle(T, O, W):
    """Weight tensors whose element counts are no multiples of four (33 x 75, 35 x 297) and odd
    bias lengths: the optimizer kernel adds their split sums element by element. Three Adam
    steps of the replayed, branching step against eager steps (bit for bit) and the oracle."""
    spec = [("conv", 16, 16, 3, 5, 33, True), ("maxpool", 16, 16, 33, 2), ("act", "relu"),
            ("conv", 8, 8, 33, 3, 35, True), ("act", "tanh"), ("fc", 8 * 8 * 35, 10), ("act", "softmax")]
    batch = 64
    rng = np.random.default_rng(321)
    eager = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD)
    graph = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    params = []
    for i, l in enumerate(spec):
        nw, nb, fan_in, _ = W.layer_fans(l)
        if nw:
            w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
            b = rng.uniform(-0.2, 0.2, nb).astype(np.float32)
            for n in (eager, graph):
                n.set_param(i, 0, w); n.set_param(i, 1, b)
            ref.weight(i)[:] = w; ref.bias(i)[:] = b
            params += [(i, 0), (i, 1)]
    x = rng.standard_normal((batch, 3 * 16 * 16)).astype(np.float32)
    t = np.eye(10, dtype=np.float32)[rng.integers(0, 10, batch)]
    xd, td = T.to_device(x), T.to_device(t)
    o1, o2, ro = T.opt_desc("adam"), T.opt_desc("adam"), O.opt_desc("adam")
    for step in range(3):
        eager.train_step(o1, "ce_multiclass", batch, xd, td)
        graph.train_step(o2, "ce_multiclass", batch, xd, td)
        ref.train_step(ro, "ce_multiclass", x, t)
        for (i, which) in params:
            assert np.array_equal(eager.get_param(i, which), graph.get_param(i, which)), (step, i, which)
    # (Adam divides by the gradient's own size: the weights are compared at the looser bound that
    # the float64 tests justify; the bit-for-bit agreement above is the point here)
    for (i, which) in params:
        want = ref.weight(i) if which == 0 else ref.bias(i)
        assert_close(graph.get_param(i, which), want, 10 * REL_TOL, f"parameter {i}.{which}")
    eager.close(); graph.close()


def test_net_with_every_other_activation_matches_oracle(T, O, W):
    """A small net that chains the parameterised and remaining activation layers: two Adam
    steps, every layer output, gradient and updated weight against the oracle."""
    spec = [("conv", 10, 10, 2, 3, 4, True), ("act", "leaky_relu", (0.1,)), ("conv", 10, 10, 4, 3, 4, False),
            ("act", "elu", (0.7,)), ("avepool", 8, 8, 4, 2), ("act", "selu"), ("fc", 64, 24), ("act", "softplus"),
            ("fc", 24, 20), ("act", "softsign"), ("fc", 20, 16), ("act", "asinh"), ("fc", 16, 10),
            ("act", "tanh_p1m2")]
    batch = 6
    rng = np.random.default_rng(5)
    for flags in (0, T.NET_FUSE_ACT_GRAD):
        net = T.Net(W.build_layers(T, spec), batch, flags)
        ref = O.OracleNet(W.build_layers(O, spec), batch)
        for i, l in enumerate(spec):
            nw, nb, fan_in, _ = W.layer_fans(l)
            if nw:
                w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
                b = rng.uniform(-0.1, 0.1, nb).astype(np.float32)
                net.set_param(i, 0, w); net.set_param(i, 1, b)
                ref.weight(i)[:] = w; ref.bias(i)[:] = b
        x = rng.standard_normal((batch, 200)).astype(np.float32)
        t = rng.uniform(0.1, 0.9, (batch, 10)).astype(np.float32)
        xd, td = T.to_device(x), T.to_device(t)
        opt, ropt = T.opt_desc("adam"), O.opt_desc("adam")
        for step in range(2):
            net.train_step(opt, "mse", batch, xd, td)
            ref.train_step(ropt, "mse", x, t)
            for i, l in enumerate(spec):
                if net.out_written(i):
                    assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"step {step} out {i}")
                if W.layer_fans(l)[0]:
                    assert_close(net.get_param(i, 0), ref.weight(i), REL_TOL, f"step {step} w {i}")
                    assert_close(net.get_param(i, 1), ref.bias(i), REL_TOL, f"step {step} b {i}")


@pytest.mark.parametrize("spec", [
    # conv -> pool -> act, ragged width of the 32-column tiles, partial channel tile
    [("conv", 40, 12, 3, 5, 20, True), ("maxpool", 40, 12, 20, 2), ("act", "tanh"), ("fc", 20 * 20 * 6, 10)],
    # conv -> act -> pool (the pool reads the activation), two channel tiles, valid padding
    [("conv", 14, 18, 2, 3, 40, False), ("act", "relu"), ("maxpool", 12, 16, 40, 2), ("fc", 40 * 6 * 8, 10)],
    # conv -> pool without any activation, one input channel
    [("conv", 36, 8, 1, 5, 6, True), ("maxpool", 36, 8, 6, 2), ("fc", 6 * 18 * 4, 10)],
    # conv -> act -> pool -> act
    [("conv", 16, 16, 3, 3, 33, True), ("act", "sigmoid"), ("maxpool", 16, 16, 33, 2), ("act", "relu"),
     ("fc", 33 * 64, 10)],
])
def test_first_conv_with_pool_in_its_kernel_matches_oracle(T, O, W, spec):
    """The first convolution of a fusing net also computes the 2x2 max-pool (and the activations)
    behind it: every layer output, the argmax records (bit-exact) and all gradients against the
    oracle, and the same net without fusion gives the same outputs."""
    check_fusing_and_plain_net(T, O, W, spec, 5)


@pytest.mark.parametrize("spec,batch", [
    # rows of 16 pixels, one accumulator block a wave; relu behind the pool leaves the kernel too
    ([("conv", 16, 16, 16, 3, 32, True), ("maxpool", 16, 16, 32, 2), ("act", "relu"), ("fc", 32 * 64, 10)], 64),
    # rows of 8 pixels, two images a tile, 5x5 window, an activation between convolution and pool
    ([("conv", 8, 8, 16, 5, 32, True), ("act", "tanh"), ("maxpool", 8, 8, 32, 2), ("fc", 32 * 16, 10)], 256),
    # two channel blocks a wave; the sigmoid behind the pool stays a kernel of its own
    ([("conv", 16, 16, 32, 3, 64, True), ("maxpool", 16, 16, 64, 2), ("act", "sigmoid"), ("fc", 64 * 64, 10)], 128),
    # two pixel blocks a wave
    ([("conv", 16, 16, 16, 5, 32, True), ("maxpool", 16, 16, 32, 2), ("fc", 32 * 64, 10)], 256),
    # ragged tiles: 10 rows in tiles of 8, 12 columns in rows of 16; 40 of 64 channels
    ([("conv", 12, 10, 16, 3, 40, True), ("maxpool", 12, 10, 40, 2), ("act", "relu"), ("fc", 40 * 30, 10)], 128),
    # no padding: 18x18 -> 16x16
    ([("conv", 18, 18, 16, 3, 32, False), ("act", "relu"), ("maxpool", 16, 16, 32, 2), ("act", "relu"),
      ("fc", 32 * 64, 10)], 64),
])
def test_stride1_conv_with_pool_in_its_kernel_matches_oracle(T, O, W, spec, batch):
    """A stride-1 convolution with many input channels whose 32-pixel accumulator blocks hold
    whole pool windows also computes the 2x2 max-pool behind it (and a relu behind that): every
    layer output, the argmax records (bit-exact) and all gradients against the oracle, the same
    outputs as the net without fusion, and the convolution's own output is left out of a train
    step only."""
    check_fusing_and_plain_net(T, O, W, spec, batch)


@pytest.mark.parametrize("spec", [
    # 2x2 pools behind and in front of the second convolution: they add up its split reductions
    [("conv", 16, 16, 3, 5, 32, True), ("maxpool", 16, 16, 32, 2), ("act", "relu"),
     ("conv", 8, 8, 32, 5, 64, True), ("maxpool", 8, 8, 64, 2), ("act", "relu"), ("fc", 1024, 10)],
    # the same without activations: the pool in front reads dX directly
    [("conv", 16, 16, 3, 5, 32, True), ("maxpool", 16, 16, 32, 2),
     ("conv", 8, 8, 32, 5, 64, True), ("maxpool", 8, 8, 64, 2), ("fc", 1024, 10)],
    # 4x4 pools: not the kernel that can take the sums, the reductions run on their own
    [("conv", 32, 32, 3, 5, 32, True), ("maxpool", 32, 32, 32, 4), ("act", "tanh"),
     ("conv", 8, 8, 32, 5, 64, True), ("maxpool", 8, 8, 64, 4), ("act", "relu"), ("fc", 256, 10)],
    # an activation between convolution and pool: the reduction applies it, nothing is left
    [("conv", 16, 16, 3, 5, 32, True), ("maxpool", 16, 16, 32, 2), ("act", "relu"),
     ("conv", 8, 8, 32, 5, 64, True), ("act", "sigmoid"), ("maxpool", 8, 8, 64, 2), ("fc", 1024, 10)],
])
def test_split_convolution_sums_taken_by_the_pools_match_oracle(T, O, W, spec):
    """A stride-1 convolution too small to fill the chip splits its reduction; in a fusing net the
    2x2 max-pool kernel that reads the result (forward: behind it; backward: in front of it) adds
    the partial sums up instead of a reduction launch. Same checks as above, at a batch where the
    second convolution runs on the stride-1 kernel and splits four ways."""
    check_fusing_and_plain_net(T, O, W, spec, 64)


def check_fusing_and_plain_net(T, O, W, spec, batch):
    rng = np.random.default_rng(len(spec) * 131 + spec[0][1])
    nets = [T.Net(W.build_layers(T, spec), batch, f) for f in (0, T.NET_FUSE_ACT_GRAD)]
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for i, l in enumerate(spec):
        nw, nb, fan_in, _ = W.layer_fans(l)
        if nw:
            w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
            b = rng.uniform(-0.5, 0.5, nb).astype(np.float32)
            for net in nets:
                net.set_param(i, 0, w); net.set_param(i, 1, b)
            ref.weight(i)[:] = w; ref.bias(i)[:] = b
    first = spec[0]
    x = rng.standard_normal((batch, first[1] * first[2] * first[3])).astype(np.float32)
    t = rng.uniform(0.1, 0.9, (batch, 10)).astype(np.float32)
    xd, td = T.to_device(x), T.to_device(t)
    ref.train_step(O.opt_desc("sgd"), "mse", x, t, do_update=False)
    for net in nets:
        net.train_step(None, "mse", batch, xd, td, do_update=False)
        for i, l in enumerate(spec):
            if net.out_written(i):
                assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"layer {i} output")
            if l[0] == "maxpool":
                assert np.array_equal(net.layer_argmax(i, batch).astype(np.int64), ref.layer_argmax(i, batch))
                if i >= 1 and spec[i - 1][0] == "conv" and net.dx_written(i):
                    # the gradient routed through the pool (by the pool's kernel, or by the dX
                    # epilogue of the fully-connected layer behind it; not written at all where
                    # the convolution in front reads the pooled gradient itself)
                    assert_close(net.layer_dx(i, batch), ref.layer_dx(i, batch), REL_TOL, f"layer {i} dX")
            if net.param_size(i, 0):
                assert_close(net.layer_grad(i, 0), ref.layer_dw(i), REL_TOL, f"layer {i} dW")
                assert_close(net.layer_grad(i, 1), ref.layer_db(i), REL_TOL, f"layer {i} db")
        assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), REL_TOL, "input gradient")
    for i in range(len(spec)):
        if nets[0].out_written(i) and nets[1].out_written(i):
            assert np.array_equal(nets[0].layer_out(i, batch), nets[1].layer_out(i, batch)), f"layer {i} fused vs not"
    # a train step may keep a convolution's own output in registers when its kernel also computes
    # the pool behind it; the forward pass of its own writes every layer
    for net in nets:
        net.forward(batch, xd)
        for i in range(len(spec)):
            assert net.out_written(i)
            assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"forward pass, layer {i} output")
    for i in range(len(spec)):
        assert np.array_equal(nets[0].layer_out(i, batch), nets[1].layer_out(i, batch)), f"layer {i} fused vs not"
    for net in nets:
        net.close()


@pytest.mark.parametrize("flags", [1, 3])
@pytest.mark.parametrize("spec,batch,pool_dx_written", [
    # the CIFAR net's first layers at a small batch; 5x5 window, a second convolution's dX
    # (relu folded) produces the pooled gradient
    ([("conv", 32, 32, 3, 5, 32, True), ("maxpool", 32, 32, 32, 2), ("act", "relu"),
      ("conv", 16, 16, 32, 5, 8, True), ("act", "tanh"), ("fc", 2048, 10)], 12, False),
    # one input channel, no padding (24x24 outputs), 6 of 32 output channels in use; a
    # fully-connected layer's dX (tanh folded) produces the pooled gradient
    ([("conv", 28, 28, 1, 5, 6, False), ("maxpool", 24, 24, 6, 2), ("act", "tanh"), ("fc", 864, 10)], 7, False),
    # 40 output channels: a second, partial tile of them in dW and a ragged last chunk in dX;
    # four input channels, 3x3 window
    ([("conv", 16, 8, 4, 3, 40, True), ("maxpool", 16, 8, 40, 2), ("act", "sigmoid"), ("fc", 1280, 10)], 5, False),
    # a window without compile-time loops (4x4, no padding: 13x13 outputs would be odd, so 16+3)
    ([("conv", 19, 11, 2, 4, 9, False), ("maxpool", 16, 8, 9, 2), ("fc", 288, 10)], 3, False),
    # output width 18 is not a multiple of four: the kernels read a gradient the pool has written
    ([("conv", 20, 12, 2, 3, 8, False), ("maxpool", 18, 10, 8, 2), ("act", "relu"), ("fc", 360, 10)], 6, True),
    # an activation between convolution and pool: the pool's kernel runs and folds its gradient
    # (so that it is the activation's output gradient that stays in registers)
    ([("conv", 16, 16, 3, 3, 8, True), ("act", "relu"), ("maxpool", 16, 16, 8, 2), ("fc", 512, 10)], 6, False),
])
def test_first_conv_reading_its_gradient_through_the_pool_matches_oracle(T, O, W, spec, batch, pool_dx_written, flags):
    """The backward kernels of a fusing net's first convolution (few input channels, stride 1)
    with a 2x2 max-pool directly behind it take the pooled gradient and the argmax records and
    rebuild their operand on the way to LDS; the pool's backward kernel does not run and its
    input gradient is reported as not written. Two passes without update (gradients add up),
    then two SGD steps: gradients, input gradient and weights against the oracle."""
    rng = np.random.default_rng(len(spec) * 17 + batch)
    net = T.Net(W.build_layers(T, spec), batch, flags)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for i, l in enumerate(spec):
        nw, nb, fan_in, _ = W.layer_fans(l)
        if nw:
            w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
            b = rng.uniform(-0.5, 0.5, nb).astype(np.float32)
            net.set_param(i, 0, w); net.set_param(i, 1, b)
            ref.weight(i)[:] = w; ref.bias(i)[:] = b
    first = spec[0]
    x = rng.standard_normal((batch, first[1] * first[2] * first[3])).astype(np.float32)
    t = rng.uniform(0.1, 0.9, (batch, 10)).astype(np.float32)
    xd, td = T.to_device(x), T.to_device(t)
    pool = [i for i, l in enumerate(spec) if l[0] == "maxpool"][0]
    ref.train_step(O.opt_desc("sgd"), "mse", x, t, do_update=False)
    for passes in (1, 2):
        net.train_step(None, "mse", batch, xd, td, do_update=False)
        assert net.dx_written(pool) == pool_dx_written
        assert np.array_equal(net.layer_argmax(pool, batch).astype(np.int64), ref.layer_argmax(pool, batch))
        for i, l in enumerate(spec):
            if net.param_size(i, 0):
                assert_close(net.layer_grad(i, 0), passes * ref.layer_dw(i), REL_TOL, f"pass {passes} layer {i} dW")
                assert_close(net.layer_grad(i, 1), passes * ref.layer_db(i), REL_TOL, f"pass {passes} layer {i} db")
        assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), REL_TOL, f"pass {passes} input gradient")
    net.clear_grads()
    opt, ropt = T.opt_desc("sgd"), O.opt_desc("sgd")
    for step in range(2):
        net.train_step(opt, "mse", batch, xd, td, do_update=True)
        ref.train_step(ropt, "mse", x, t, do_update=True)
        for i, l in enumerate(spec):
            if net.param_size(i, 0):
                assert_close(net.get_param(i, 0), ref.weight(i), REL_TOL, f"step {step} layer {i} weights")
                assert_close(net.get_param(i, 1), ref.bias(i), REL_TOL, f"step {step} layer {i} bias")
    net.close()


@pytest.mark.parametrize("spec,batch", [
    # both limits of the one-launch kernel (128 inputs, 64 outputs), relu folded, ragged batch
    ([("fc", 100, 128), ("act", "relu"), ("fc", 128, 64), ("act", "softmax")], 37),
    # the fully-connected layer is the first layer: its dX is the net's input gradient
    ([("fc", 30, 10), ("act", "softmax")], 5),
    # 70 inputs: a second, partial block of dX columns; tanh folded
    ([("fc", 50, 70), ("act", "tanh"), ("fc", 70, 3), ("act", "softmax")], 16),
    # a pool in front: nothing to fold (five input channels: the convolution's backward kernels
    # are not those that read the pooled gradient themselves, so that the dX epilogue scatters)
    ([("conv", 8, 8, 5, 3, 4, True), ("maxpool", 8, 8, 4, 2), ("fc", 64, 10), ("act", "softmax")], 9),
    # the same with two: the convolution's kernels read the pooled gradient this layer writes
    ([("conv", 8, 8, 2, 3, 4, True), ("maxpool", 8, 8, 4, 2), ("fc", 64, 10), ("act", "softmax")], 9),
    # too wide for the one-launch kernel: the three separate launches
    ([("fc", 20, 200), ("act", "relu"), ("fc", 200, 10), ("act", "softmax")], 8),
    # nets that end in the fully-connected layer, trained with mse: the same kernel without softmax
    ([("fc", 50, 70), ("act", "tanh"), ("fc", 70, 3)], 16),
    ([("fc", 30, 10)], 5),
    ([("conv", 8, 8, 5, 3, 4, True), ("maxpool", 8, 8, 4, 2), ("act", "sigmoid"), ("fc", 64, 64)], 19),
])
@pytest.mark.parametrize("targets", ["one_hot", "soft"])
def test_last_fc_softmax_xent_in_one_launch_matches_oracle(T, O, W, spec, batch, targets):
    """A fusing net trained with cross_entropy_multiclass (or, ending in a fully-connected layer,
    with mse) runs its last fully-connected layer, the softmax, the loss gradient and that
    layer's dX as one kernel: outputs and gradients
    against the oracle, and bit for bit against the same net without fusion (same terms, same
    order), for one-hot and for soft targets."""
    rng = np.random.default_rng(len(spec) * 17 + batch)
    nets = [T.Net(W.build_layers(T, spec), batch, f) for f in (0, T.NET_FUSE_ACT_GRAD)]
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for i, l in enumerate(spec):
        nw, nb, fan_in, _ = W.layer_fans(l)
        if nw:
            w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
            b = rng.uniform(-0.5, 0.5, nb).astype(np.float32)
            for net in nets:
                net.set_param(i, 0, w); net.set_param(i, 1, b)
            ref.weight(i)[:] = w; ref.bias(i)[:] = b
    softmax = spec[-1] == ("act", "softmax")
    loss = "ce_multiclass" if softmax else "mse"
    last_fc = len(spec) - (2 if softmax else 1)
    first, classes = spec[0], spec[last_fc][2]
    n_in = first[1] if first[0] == "fc" else first[1] * first[2] * first[3]
    x = rng.standard_normal((batch, n_in)).astype(np.float32)
    one_hot = np.eye(classes, dtype=np.float32)[rng.integers(0, classes, batch)]
    soft = rng.uniform(0.0, 1.0, (batch, classes)).astype(np.float32)
    xd = T.to_device(x)
    for t in ((one_hot,) if targets == "one_hot" else (soft,)):
        td = T.to_device(t)
        ref.train_step(O.opt_desc("sgd"), loss, x, t, do_update=False)
        for net in nets:
            net.train_step(None, loss, batch, xd, td, do_update=False)
            for i, l in enumerate(spec):
                if net.out_written(i):
                    assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"layer {i} output")
                if net.param_size(i, 0):
                    assert_close(net.layer_grad(i, 0), ref.layer_dw(i), REL_TOL, f"layer {i} dW")
                    assert_close(net.layer_grad(i, 1), ref.layer_db(i), REL_TOL, f"layer {i} db")
            assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), REL_TOL, "input gradient")
        for i in range(len(spec)):
            if nets[0].out_written(i) and nets[1].out_written(i):
                assert np.array_equal(nets[0].layer_out(i, batch), nets[1].layer_out(i, batch)), f"layer {i} fused vs not"
        # (a folded activation gradient rounds differently from the activation layer's own kernel,
        # so the layers in front agree to rounding only)
        for which in (0, 1):
            assert np.array_equal(nets[0].layer_grad(last_fc, which), nets[1].layer_grad(last_fc, which)), \
                f"last layer's gradient {which} fused vs not"
        if last_fc == 0:
            assert np.array_equal(nets[0].layer_dx(0, batch), nets[1].layer_dx(0, batch)), "input gradient fused vs not"
    for net in nets:
        net.close()


@pytest.mark.parametrize("spec,batch", [
    # the benchmarked net's classifier: eight 128-deep slices, a pool in front, ragged batch
    ([("conv", 16, 16, 3, 5, 16, True), ("maxpool", 16, 16, 16, 2), ("act", "relu"), ("fc", 1024, 64),
      ("act", "relu"), ("fc", 64, 10), ("act", "softmax")], 37),
    # the pool in front reads an activation: its own kernel routes the gradient
    ([("conv", 16, 16, 3, 5, 16, True), ("act", "relu"), ("maxpool", 16, 16, 16, 2), ("fc", 1024, 64),
      ("act", "relu"), ("fc", 64, 10), ("act", "softmax")], 37),
    # the first layer of the net (its dX is the input gradient); 300 inputs: a short last slice;
    # 40 hidden units
    ([("fc", 300, 40), ("act", "tanh"), ("fc", 40, 10), ("act", "softmax")], 16),
    # mse on the second layer, both at the 64-unit limit
    ([("fc", 200, 64), ("act", "sigmoid"), ("fc", 64, 64)], 5),
    # an activation in front whose gradient the dX epilogue applies; 132 inputs: one full slice and
    # four more; 130 inputs: not a multiple of four, the separate launches
    ([("fc", 50, 132), ("act", "tanh"), ("fc", 132, 24), ("act", "relu"), ("fc", 24, 3), ("act", "softmax")], 20),
    ([("fc", 50, 130), ("act", "tanh"), ("fc", 130, 24), ("act", "relu"), ("fc", 24, 3), ("act", "softmax")], 20),
    # pool and a folded activation in front
    ([("conv", 8, 8, 5, 3, 4, True), ("maxpool", 8, 8, 4, 2), ("act", "sigmoid"), ("fc", 64, 12), ("act", "relu"),
      ("fc", 12, 10), ("act", "softmax")], 19),
    # 36 hidden units are fine, 35 are not (rows of the first layer's filters are read four at a time)
    ([("fc", 260, 36), ("act", "relu"), ("fc", 36, 10), ("act", "softmax")], 33),
    ([("fc", 260, 35), ("act", "relu"), ("fc", 35, 10), ("act", "softmax")], 33),
])
@pytest.mark.parametrize("flags", [1, 3])
def test_two_closing_fc_layers_in_one_launch_match_oracle(T, O, W, spec, batch, flags):
    """A fusing net whose classifier is fc -> pointwise activation -> fc [-> softmax] runs both
    layers' forward passes, the loss gradient and the second layer's input gradient as one kernel
    (the first layer's product split over workgroups, the last to finish carries on), and the
    second layer's weight and bias gradients beside the first layer's in its backward launch.
    Three SGD steps: every layer output, every gradient and every updated weight against the
    oracle, and the outputs against the same net without fusion. Replayed steps (flags 3) also
    show that the kernel leaves its tickets ready for the next launch."""
    rng = np.random.default_rng(len(spec) * 29 + batch)
    net, plain = T.Net(W.build_layers(T, spec), batch, flags), T.Net(W.build_layers(T, spec), batch, 0)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for i, l in enumerate(spec):
        nw, nb, fan_in, _ = W.layer_fans(l)
        if nw:
            w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
            b = rng.uniform(-0.5, 0.5, nb).astype(np.float32)
            for n in (net, plain):
                n.set_param(i, 0, w); n.set_param(i, 1, b)
            ref.weight(i)[:] = w; ref.bias(i)[:] = b
    softmax = spec[-1] == ("act", "softmax")
    loss = "ce_multiclass" if softmax else "mse"
    first, classes = spec[0], spec[-2 if softmax else -1][2]
    n_in = first[1] if first[0] == "fc" else first[1] * first[2] * first[3]
    x = rng.standard_normal((batch, n_in)).astype(np.float32)
    t = np.eye(classes, dtype=np.float32)[rng.integers(0, classes, batch)]
    xd, td = T.to_device(x), T.to_device(t)
    opt, ropt = T.opt_desc("sgd"), O.opt_desc("sgd")
    # gradients first (an update clears them), then three steps with updates
    ref.train_step(ropt, loss, x, t, do_update=False)
    for n in (net, plain):
        n.train_step(None, loss, batch, xd, td, do_update=False)
    for i, l in enumerate(spec):
        if net.out_written(i):
            assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"layer {i} output")
            assert_close(net.layer_out(i, batch), plain.layer_out(i, batch), REL_TOL, f"layer {i} output, fused vs not")
        if l[0] == "maxpool" and spec[i - 1][0] == "conv":
            for n_ in (net, plain):
                if n_.dx_written(i):
                    assert_close(n_.layer_dx(i, batch), ref.layer_dx(i, batch), REL_TOL, f"layer {i} dX (through the pool)")
            assert plain.dx_written(i)
        if net.param_size(i, 0):
            assert_close(net.layer_grad(i, 0), ref.layer_dw(i), REL_TOL, f"layer {i} dW")
            assert_close(net.layer_grad(i, 1), ref.layer_db(i), REL_TOL, f"layer {i} db")
    assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), REL_TOL, "input gradient")
    net.train_step(T.opt_desc("sgd", alpha=0.0), loss, batch, xd, td)   # clears the gradients
    for step in range(3):
        net.train_step(opt, loss, batch, xd, td)
        ref.train_step(ropt, loss, x, t)
        for i, l in enumerate(spec):
            if net.out_written(i):
                assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"step {step} layer {i} output")
            if net.param_size(i, 0):
                assert_close(net.get_param(i, 0), ref.weight(i), REL_TOL, f"step {step} layer {i} weights")
                assert_close(net.get_param(i, 1), ref.bias(i), REL_TOL, f"step {step} layer {i} bias")
    net.close(); plain.close()


def test_layers_without_bias_through_the_one_launch_kernels(T, O):
    """No layer has a bias: the last layer's one-launch kernel, the fully-connected backward that
    routes dX through the pool in front, and the convolution kernels against the oracle."""
    def layers(api):
        return [api.L_conv(8, 8, 5, 3, 4, pad_same=True, has_bias=False), api.L_maxpool(8, 8, 4, 2),
                api.L_act("relu"), api.L_fc(64, 24, has_bias=False), api.L_act("tanh"),
                api.L_fc(24, 10, has_bias=False), api.L_act("softmax")]
    batch = 9
    rng = np.random.default_rng(77)
    nets = [T.Net(layers(T), batch, f) for f in (0, T.NET_FUSE_ACT_GRAD)]
    ref = O.OracleNet(layers(O), batch)
    for i, (nw, fan_in) in {0: (180, 45), 3: (64 * 24, 64), 5: (240, 24)}.items():
        w = rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(np.sqrt(3.0 / fan_in))
        for net in nets:
            assert net.param_size(i, 1) == 0
            net.set_param(i, 0, w)
        ref.weight(i)[:] = w
    x = rng.standard_normal((batch, 320)).astype(np.float32)
    t = np.eye(10, dtype=np.float32)[rng.integers(0, 10, batch)]
    ref.train_step(O.opt_desc("sgd"), "ce_multiclass", x, t, do_update=False)
    for net in nets:
        net.train_step(None, "ce_multiclass", batch, T.to_device(x), T.to_device(t), do_update=False)
        for i in range(7):
            if net.out_written(i):
                assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), REL_TOL, f"layer {i} output")
        for i in (0, 3, 5):
            assert_close(net.layer_grad(i, 0), ref.layer_dw(i), REL_TOL, f"layer {i} dW")
        assert_close(net.layer_dx(1, batch), ref.layer_dx(1, batch), REL_TOL, "gradient routed through the pool")
        assert_close(net.layer_dx(0, batch), ref.layer_dx(0, batch), REL_TOL, "input gradient")
        net.close()


@pytest.mark.parametrize("ahead", [1, 2])
def test_feeder_batches_staged_ahead_match_oracle(T, O, W, ahead):
    """tdh_feeder_*: different host batches every step, a short last batch, graph replay from
    the three device slots in turn, staged one and two batches ahead of the step; updated weights
    against the oracle after every step. A third outstanding batch and an acquire with nothing
    staged are refused."""
    spec, params, _, _, _, loss, opt_kind, opt_kw = W.make_batch("cifar10_cnn_b128", batch=8)
    batch = 8
    net = T.Net(W.build_layers(T, spec), batch, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for (i, which, a) in params:
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    rng = np.random.default_rng(9)
    sizes = [8, 8, 8, 3, 8, 8, 8, 3]   # two "epochs" with a short last batch
    xs = [rng.standard_normal((n, 3072)).astype(np.float32) for n in sizes]
    ts = [np.eye(10, dtype=np.float32)[rng.integers(0, 10, n)] for n in sizes]
    opt, ropt = T.opt_desc(opt_kind, **opt_kw), O.opt_desc(opt_kind, **opt_kw)
    feed = T.Feeder(3072, 10, batch)
    for k in range(ahead):
        feed.stage(xs[k], ts[k])
    for k in range(len(sizes)):
        xd, td, n = feed.acquire()
        assert n == sizes[k]
        if k + ahead < len(sizes):
            feed.stage(xs[k + ahead], ts[k + ahead])
        net.train_step(opt, loss, n, xd, td)
        if k == 2:    # as many staged as the feeder takes (two), or nothing staged at the end
            extra = 2 - ahead
            for _ in range(extra):
                feed.stage(xs[k], ts[k])
            with pytest.raises(T.TdhError, match="batches are staged and have not been acquired"):
                feed.stage(xs[k], ts[k])
            for _ in range(extra):   # drop what this check staged: acquire it and move on
                feed.acquire()
            if extra:                # the order of the real batches is restored
                feed.close()
                feed = T.Feeder(3072, 10, batch)
                for j in range(k + 1, min(k + 1 + ahead, len(sizes))):
                    feed.stage(xs[j], ts[j])
        ref.train_step(ropt, loss, xs[k], ts[k])
        for (i, which, _) in params:
            want = ref.weight(i) if which == 0 else ref.bias(i)
            assert_close(net.get_param(i, which), want, REL_TOL, f"step {k} layer {i}.{which}")
    with pytest.raises(T.TdhError, match="nothing has been staged"):
        feed.acquire()
    feed.close()


def test_weight_files_round_trip_with_the_reference(T, tmp_path):
    """A weight file written by the reference's network::save loads into the device network,
    and the file the device network writes is byte for byte the reference's."""
    import importlib, os
    io = importlib.import_module("tiny-cnn_amd.io")
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "io.npz"))
    nets = {"weights_avepool": [T.L_conv(8, 8, 2, 3, 3, pad_same=True), T.L_act("tanh"),
                                T.L_avepool(8, 8, 3, 2), T.L_fc(48, 5)],
            "weights_plain": [T.L_conv(6, 6, 1, 3, 4), T.L_act("relu"), T.L_fc(64, 3)]}
    for name, layers in nets.items():
        path = str(tmp_path / (name + ".txt"))
        g[name + ".text"].tofile(path)
        net = T.Net(layers, 2)
        io.load_weights(net, path)
        for k, (i, which, n) in enumerate(net.params()):
            want = g[f"{name}.param{k}"]
            assert np.allclose(net.get_param(i, which), want, rtol=1e-7, atol=0), (name, k)
        out = str(tmp_path / (name + ".out.txt"))
        io.save_weights(net, out)
        assert open(out).read() == open(path).read(), name
    with pytest.raises(ValueError, match="fewer weights"):
        io.load_weights(T.Net(nets["weights_avepool"], 2), str(tmp_path / "weights_plain.txt"))


def test_weight_archives_round_trip_with_the_reference(T, W, tmp_path):
    """The cereal archives that the reference's network::save(file, content_type::weights, ...)
    wrote (tests/golden/archives.npz) load into the device network bit for bit, and what the
    device network writes is byte for byte the reference's file, in both binary formats."""
    import importlib, os
    io = importlib.import_module("tiny-cnn_amd.io")
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "archives.npz"))
    specs = {"avepool": [("conv", 8, 8, 2, 3, 3, True), ("act", "tanh"), ("avepool", 8, 8, 3, 2),
                         ("act", "leaky_relu", (0.05, 0.0)), ("fc", 48, 5), ("act", "softmax")],
             "lenet5_mnist": W.lenet5_mnist(), "cifar10_cnn": W.cifar10_cnn(),
             "bn_dropout": [("fc", 12, 8), ("batchnorm", 8, 1), ("act", "relu"), ("dropout", 0.3), ("fc", 8, 4),
                            ("act", "tanh_p1m2")]}
    for name, spec in specs.items():
        for fmt in ("binary", "portable_binary"):
            path = str(tmp_path / f"{name}.{fmt}")
            g[f"{name}.{fmt}"].tofile(path)
            net = T.Net(W.build_layers(T, spec), 2, T.NET_FUSE_ACT_GRAD | T.NET_GRAPH)
            io.load_weights_archive(net, path, fmt)
            for k, (i, which, n) in enumerate(net.params()):
                assert np.array_equal(net.get_param(i, which), g[f"{name}.param{k}"]), (name, fmt, k)
            out = path + ".out"
            io.save_weights_archive(net, out, fmt)
            assert open(out, "rb").read() == open(path, "rb").read(), (name, fmt)
            net.close()
    with pytest.raises(ValueError, match="holds|ends inside"):
        io.load_weights_archive(T.Net(W.build_layers(T, specs["avepool"]), 2), str(tmp_path / "bn_dropout.binary"))


@pytest.mark.parametrize("flags", [0, 1, 3])
def test_net_with_batchnorm_and_dropout_matches_oracle_and_reference_fit(T, O, W, net_steps, flags):
    """batch_normalization_layer and dropout_layer as layer kinds of the device-resident step:
    conv -> batch-norm -> relu -> pool -> fc -> tanh -> dropout -> fc -> softmax, masks drawn on
    the host with the reference's generator and handed over before every step. Every layer
    against the oracle after a gradient-only pass, then three Adam steps against the oracle and
    against what network<sequential>::fit produced after set_random_seed (running averages
    included), then a test-phase forward pass (running averages, no mask)."""
    g = net_steps
    spec = W.BN_DROPOUT_NET
    params, x, t = W.bn_dropout_case()
    assert input_checksum(x, t, params) == float(g["bn_dropout.input_checksum"])
    batch, steps, seed = x.shape[0], int(g["bn_dropout.steps"]), int(g["bn_dropout.seed"])
    net = T.Net(W.build_layers(T, spec), batch, flags)
    ref = O.OracleNet(W.build_layers(O, spec), batch)
    for (i, which, a) in params:
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    xd, td = T.to_device(x), T.to_device(t)
    rng = T.Mt19937(seed)                       # set_random_seed(seed)
    probe = T.dropout_mask(T.Mt19937(99), 0.4, batch, 20)
    net.set_dropout_mask(6, probe); ref.set_dropout_mask(6, probe)
    net.train_step(None, "ce_multiclass", batch, xd, td, do_update=False)
    ref.train_step(O.opt_desc("adam"), "ce_multiclass", x, t, do_update=False)
    check_every_layer(net, ref, spec, batch, "bn/dropout net", bool(flags & 1), cancelling_db=(0,))
    net.clear_grads()
    assert not net.layer_grad(0, 0).any()
    opt, ropt = T.opt_desc("adam"), O.opt_desc("adam")
    for step in range(steps):
        mask = T.dropout_mask(rng, 0.4, batch, 20)
        net.set_dropout_mask(6, mask); ref.set_dropout_mask(6, mask)
        net.train_step(opt, "ce_multiclass", batch, xd, td)
        ref.train_step(ropt, "ce_multiclass", x, t)
    for (i, which, a) in params:
        got = net.get_param(i, which)
        if (i, which) == (0, 1):
            # the bias in front of the batch normalization has no effect on the loss: its gradient
            # is rounding noise, which adam turns into steps of +-alpha on either side
            assert np.all(np.abs(got - ref.bias(0)) <= 2 * steps * opt.alpha)
            assert np.all(np.abs(got - g["bn_dropout.p0.1"]) <= 2 * steps * opt.alpha)
            continue
        assert_close(got, ref.weight(i) if which == 0 else ref.bias(i), what=f"parameter {i}.{which} vs oracle")
        assert_close(got, g[f"bn_dropout.p{i}.{which}"], what=f"parameter {i}.{which} vs network::fit")
    for which in (0, 1):
        assert net.param_size(1, 2 + which) == 6
        got = net.get_param(1, 2 + which)
        if which == 0:
            # the running mean carries the convolution's free bias with it: (1 - momentum) of that
            # bias's wandering per step on top of the usual bound
            slack = (1.0 - 0.999) * steps * (2 * steps * opt.alpha)
            for want in (ref.bn_stat(1, 0), g["bn_dropout.stat0"]):
                scale = np.maximum(np.abs(want), np.sqrt(np.mean(np.square(want))))
                assert np.all(np.abs(got - want) <= REL_TOL * scale + slack), "running mean"
            continue
        assert_close(got, ref.bn_stat(1, which), what=f"running average {which} vs oracle")
        assert_close(got, g[f"bn_dropout.stat{which}"], what=f"running average {which} vs network::fit")
    # net_phase::test: running averages instead of batch moments, dropout is the identity
    net.set_phase(False); ref.set_phase(False)
    net.forward(batch, xd)
    want = ref.forward(x)
    for i in range(len(spec)):
        assert_close(net.layer_out(i, batch), ref.layer_out(i, batch), what=f"test phase, layer {i}")
    assert np.array_equal(net.layer_out(6, batch), net.layer_out(5, batch))
    net.set_phase(True)
    net.forward(batch, xd)
    assert not np.array_equal(net.layer_out(6, batch), net.layer_out(5, batch))
    with pytest.raises(T.TdhError):
        net.set_dropout_mask(5, probe)     # not a dropout layer
    net.close()


@pytest.mark.parametrize("flags", [0, 3, 7])
def test_decisions_that_hang_on_summation_order_are_legitimate_and_the_gradients_follow_them(T, O, flags):
    """The one class of difference from the oracle that no tolerance covers: a relu whose
    pre-activation, or a max-pool whose two best candidates, differ by less than fp32 rounding
    of the sums behind them. Which way such a decision falls depends on the order of the
    additions, and everything behind it changes by whole gradient values.

    conv 3x3 (1 -> 3 channels, 6x6, pad same) -> relu -> max-pool 2x2 -> fc 27 -> 3 -> softmax,
    with an input built so that (i) channel 0 at pixel (2,2) is 1 + 3e-8 - 1: exactly 0 when
    added in tap order (the oracle: relu closed), 3e-8 in another order (relu open); (ii) channel
    1 has 0.25 at (0,4) and 1 + 0.25 + 3e-8 - 1 at (0,5): a tie that the first candidate wins in
    tap order, a win of the second candidate in another; (iii) channel 2 has an exact tie 1 / 1
    at (4,0) / (4,1), which the first candidate must win on both sides. Checked: every decision
    the GPU took is one that fp32 arithmetic allows (the float64 value lies within rounding of
    the threshold), the exact tie goes to the first candidate, and all gradients equal the
    float64 gradients of the net with the GPU's own decisions imposed. Where the oracle took the
    same decisions, the two are also compared directly."""
    e = np.float32(3e-8)
    X = np.zeros((6, 6), np.float32)
    X[1, 1] = X[2, 2] = X[3, 3] = 1.0; X[4, 4] = 2.0                                  # (i)
    X[0, 3] = X[0, 4] = X[0, 5] = X[1, 4] = X[1, 5] = X[2, 4] = 1.0; X[2, 5] = 2.0     # (ii)
    X[4, 0] = X[4, 1] = 2.0                                                           # (iii)
    w = np.zeros((3, 1, 3, 3), np.float32)
    w[0, 0, 0, 0], w[0, 0, 1, 1], w[0, 0, 2, 2] = 1.0, e, -1.0
    w[1, 0, 1, 0], w[1, 0, 1, 1], w[1, 0, 2, 0], w[1, 0, 2, 1] = 1.0, 0.25, e, -1.0
    w[2, 0, 1, 1] = 0.5
    x = np.zeros((2, 36), np.float32)
    x[0] = X.ravel()
    x[1] = np.linspace(-1.0, 1.0, 36, dtype=np.float32)     # an ordinary second sample
    b = np.zeros(3, np.float32)
    wf = np.random.default_rng(12).uniform(-0.5, 0.5, 27 * 3).astype(np.float32)
    bf = np.zeros(3, np.float32)
    t = np.zeros((2, 3), np.float32)
    t[0, 1] = t[1, 2] = 1.0
    layers = lambda api: [api.L_conv(6, 6, 1, 3, 3, pad_same=True), api.L_act("relu"), api.L_maxpool(6, 6, 3, 2),
                          api.L_fc(27, 3), api.L_act("softmax")]
    net, ref = T.Net(layers(T), 2, flags), O.OracleNet(layers(O), 2)
    for i, which, a in ((0, 0, w.ravel()), (0, 1, b), (3, 0, wf), (3, 1, bf)):
        net.set_param(i, which, a)
        (ref.weight(i) if which == 0 else ref.bias(i))[:] = a
    net.train_step(None, "ce_multiclass", 2, T.to_device(x), T.to_device(t), do_update=False)
    ref.train_step(O.opt_desc("sgd"), "ce_multiclass", x, t, do_update=False)

    # float64 pre-activations and the magnitude of the sums behind them
    xp = np.zeros((2, 8, 8)); xp[:, 1:7, 1:7] = x.reshape(2, 6, 6)
    z = np.zeros((2, 3, 6, 6)); mag = np.zeros_like(z)
    for ky in range(3):
        for kx in range(3):
            for c in range(3):
                term = np.float64(w[c, 0, ky, kx]) * xp[:, ky:ky + 6, kx:kx + 6]
                z[:, c] += term; mag[:, c] += np.abs(term)
    slack = 4 * np.finfo(np.float32).eps * mag       # what fp32 additions in any order can move a sum by
    # the construction is what the docstring says
    assert 0 < z[0, 0, 2, 2] < 1e-7 and z[0, 0, 2:4, 2:4].max() == z[0, 0, 2, 2]
    assert z[0, 1, 0, 4] == 0.25 and 0 < z[0, 1, 0, 5] - 0.25 < 1e-7 and z[0, 1, 1, 4:6].max() < 0
    assert z[0, 2, 4, 0] == z[0, 2, 4, 1] == 1.0 and z[0, 2, 5, 0:2].max() < 1.0

    def decisions(relu_out, pooled, argmax):
        arg = argmax.reshape(2, 27).astype(np.int64)
        if relu_out is not None:
            mask = relu_out.reshape(2, 3, 6, 6) > 0
        else:
            # a fused step keeps the relu's output out of memory: its decision is visible where it
            # matters, at the winners of the pool windows (no gradient reaches the other elements)
            mask = (z > 0).reshape(2, -1)
            np.put_along_axis(mask, arg, pooled.reshape(2, 27) > 0, axis=1)
            mask = mask.reshape(2, 3, 6, 6)
        wrong = mask != (z > 0)
        assert np.all(np.abs(z[wrong]) <= slack[wrong]), "a relu decision that fp32 rounding does not explain"
        a = np.where(mask, z, 0.0).reshape(2, -1)
        win = np.take_along_axis(a, arg, axis=1).reshape(2, 3, 3, 3)
        best = a.reshape(2, 3, 3, 2, 3, 2).max(axis=(3, 5))
        sl = slack.reshape(2, 3, 3, 2, 3, 2).max(axis=(3, 5))
        assert np.all(win >= best - sl), "a max-pool winner that fp32 rounding does not explain"
        return mask, arg

    mask, arg = decisions(net.layer_out(1, 2) if net.out_written(1) else None, net.layer_out(2, 2),
                          net.layer_argmax(2, 2))
    omask, oarg = decisions(ref.layer_out(1, 2), ref.layer_out(2, 2), ref.layer_argmax(2, 2))
    # the oracle adds in tap order: (i) gives exactly 0 (relu closed), (ii) a tie (first wins)
    assert not omask[0, 0, 2, 2] and oarg[0, 9 + 2] == 36 + 4
    # (iii) exact tie: the first candidate on both sides, whatever the order
    assert arg[0, 18 + 6] == oarg[0, 18 + 6] == 72 + 4 * 6
    same = np.array_equal(mask, omask) and np.array_equal(arg, oarg)
    print(f"flags {flags}: GPU relu at (i) {'open' if mask[0, 0, 2, 2] else 'closed'}, pool winner at (ii) "
          f"column {int(arg[0, 11]) - 36}; same decisions as the oracle: {same}", flush=True)

    # float64 gradients with the GPU's decisions imposed
    a = np.where(mask, z, 0.0).reshape(2, -1)
    p = np.take_along_axis(a, arg, axis=1)
    wf64 = wf.astype(np.float64).reshape(27, 3)
    logits = p @ wf64 + bf
    y = np.exp(logits - logits.max(1, keepdims=True)); y /= y.sum(1, keepdims=True)
    dlog = y * t.sum(1, keepdims=True) - t
    dwf, dbf = p.T @ dlog, dlog.sum(0)
    dp = dlog @ wf64.T
    da = np.zeros_like(a); np.put_along_axis(da, arg, dp, axis=1)
    dz = da.reshape(2, 3, 6, 6) * mask
    dw = np.zeros((3, 1, 3, 3)); dx = np.zeros((2, 8, 8))
    for ky in range(3):
        for kx in range(3):
            for c in range(3):
                dw[c, 0, ky, kx] = np.sum(xp[:, ky:ky + 6, kx:kx + 6] * dz[:, c])
                dx[:, ky:ky + 6, kx:kx + 6] += np.float64(w[c, 0, ky, kx]) * dz[:, c]
    want = {(0, 0): dw.ravel(), (0, 1): dz.sum(axis=(0, 2, 3)), (3, 0): dwf.ravel(), (3, 1): dbf}
    for (i, which), v in want.items():
        assert_close(net.layer_grad(i, which), v, what=f"flags {flags}: gradient {i}.{which} under the GPU's decisions")
    if net.dx_written(0):
        assert_close(net.layer_dx(0, 2), dx[:, 1:7, 1:7].reshape(2, 36), what=f"flags {flags}: input gradient")
    if same:
        for (i, which) in want:
            assert_close(net.layer_grad(i, which), ref.layer_dw(i) if which == 0 else ref.layer_db(i),
                         what=f"flags {flags}: gradient {i}.{which} vs oracle")
    net.close()
