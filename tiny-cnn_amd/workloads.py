"""The five workloads the path is measured and parity-tested on, as plain data.

A workload is a list of layer tuples plus seeded synthetic inputs. ``build_layers(api, spec)``
turns the tuples into the layer descriptors of whichever binding is passed as ``api`` (the
product binding or the test oracle expose the same ``L_conv``/``L_fc``/... constructors), so
the same spec drives the GPU path and its checker without either importing the other.

Weights are drawn here (numpy, seeded) and handed to both sides; tiny-dnn's own
``weight_init`` draws from libstdc++ distributions, which are not reproduced. The shapes of
the distributions follow the reference: xavier = U(+-sqrt(6/(fan_in+fan_out)))
(tiny_dnn/util/weight_init.h:37-47), he = N(0, sqrt(2/fan_in)) (:96-108), constant-0 biases,
with fan sizes from convolutional_layer.h:269-277, fully_connected_layer.h:51-53 and
partial_connected_layer.h:46-48.
"""
import math

import numpy as np


def lenet5():
    """LeNet-5-style net, 1x32x32 input (configs[0])."""
    return [("conv", 32, 32, 1, 5, 6, False), ("act", "tanh"), ("avepool", 28, 28, 6, 2),
            ("conv", 14, 14, 6, 5, 16, False), ("act", "tanh"), ("avepool", 10, 10, 16, 2),
            ("conv", 5, 5, 16, 5, 120, False), ("act", "tanh"), ("fc", 120, 10)]


# connection table of LeNet-5's C3 layer [LeCun 1998, table 1], [in_c = 6][out_c = 16]
# (examples/mnist/train.cpp:17-24)
LENET_C3_TABLE = [[c == "O" for c in row] for row in (
    "OXXXOOOXXOOOOXOO", "OOXXXOOOXXOOOOXO", "OOOXXXOOOXXOXOOO",
    "XOOOXXOOOOXXOXOO", "XXOOOXXOOOOXOOXO", "XXXOOOXXOOOOXOOO")]


def lenet5_mnist():
    """The LeNet-5 of examples/mnist/train.cpp:44-62: C3 with its connection table, a tanh
    behind every layer (also behind the pools and the last fully-connected layer)."""
    return [("conv", 32, 32, 1, 5, 6, False), ("act", "tanh"), ("avepool", 28, 28, 6, 2), ("act", "tanh"),
            ("conv", 14, 14, 6, 5, 16, False, LENET_C3_TABLE), ("act", "tanh"),
            ("avepool", 10, 10, 16, 2), ("act", "tanh"),
            ("conv", 5, 5, 16, 5, 120, False), ("act", "tanh"), ("fc", 120, 10), ("act", "tanh")]


def cifar10_cnn():
    """CIFAR-10-shape CNN of examples/cifar10/train.cpp:26-42 (configs[3])."""
    return [("conv", 32, 32, 3, 5, 32, True), ("maxpool", 32, 32, 32, 2), ("act", "relu"),
            ("conv", 16, 16, 32, 5, 32, True), ("maxpool", 16, 16, 32, 2), ("act", "relu"),
            ("conv", 8, 8, 32, 5, 64, True), ("maxpool", 8, 8, 64, 2), ("act", "relu"),
            ("fc", 1024, 64), ("act", "relu"), ("fc", 64, 10), ("act", "softmax")]


def vgg_stack(size=128):
    """VGG-style block stack, 3 x size x size input (configs[4] at size=128)."""
    h = size // 2
    q = size // 4
    return [("conv", size, size, 3, 3, 64, True), ("act", "relu"),
            ("conv", size, size, 64, 3, 64, True), ("act", "relu"), ("maxpool", size, size, 64, 2),
            ("conv", h, h, 64, 3, 128, True), ("act", "relu"),
            ("conv", h, h, 128, 3, 128, True), ("act", "relu"), ("maxpool", h, h, 128, 2),
            ("fc", 128 * q * q, 256), ("act", "relu"), ("fc", 256, 10), ("act", "softmax")]


WORKLOADS = {
    # name: (spec builder, batch, loss, optimizer kind, optimizer kwargs, init, input dist, seed)
    "lenet5_b16": (lenet5, 16, "mse", "sgd", {"alpha": 0.01}, "xavier", "uniform", 1234),
    # not one of the five benchmark configurations: the reference's own MNIST example net
    "lenet5_mnist_b16": (lenet5_mnist, 16, "mse", "adagrad", {}, "xavier", "uniform", 1239),
    "cifar10_cnn_b128": (cifar10_cnn, 128, "ce_multiclass", "adam", {}, "xavier", "normal", 1237),
    "vgg_stack_b64": (vgg_stack, 64, "ce_multiclass", "momentum", {"alpha": 0.01, "mu": 0.9},
                      "he", "normal", 1238),
}


def build_layers(api, spec):
    out = []
    for l in spec:
        kind = l[0]
        if kind == "conv":
            _, w, h, c, k, oc, same = l[:7]
            out.append(api.L_conv(w, h, c, k, oc, pad_same=same, tbl=l[7] if len(l) > 7 else None))
        elif kind == "fc":
            out.append(api.L_fc(l[1], l[2]))
        elif kind == "maxpool":
            out.append(api.L_maxpool(l[1], l[2], l[3], l[4]))
        elif kind == "avepool":
            out.append(api.L_avepool(l[1], l[2], l[3], l[4]))
        elif kind == "act":
            out.append(api.L_act(l[1], l[2] if len(l) > 2 else None))
        elif kind == "batchnorm":   # (channels, spatial[, eps, momentum])
            out.append(api.L_batchnorm(*l[1:]))
        elif kind == "dropout":     # (rate,)
            out.append(api.L_dropout(l[1]))
        else:
            raise ValueError(kind)
    return out


def layer_fans(l):
    """(weight count, bias count, fan_in, fan_out) of a layer tuple."""
    kind = l[0]
    if kind == "conv":
        _, w, h, c, k, oc, same = l[:7]
        return k * k * c * oc, oc, k * k * c, k * k * oc
    if kind == "fc":
        return l[1] * l[2], l[2], l[1], l[2]
    if kind == "avepool":
        return l[3], l[3], l[4] * l[4], 1
    return 0, 0, 0, 0


def init_params(spec, init, rng):
    """[(layer index, which, array)] in update order; biases are zero."""
    params = []
    for i, l in enumerate(spec):
        nw, nb, fan_in, fan_out = layer_fans(l)
        if nw == 0:
            continue
        if init == "xavier":
            bound = math.sqrt(6.0 / (fan_in + fan_out))
            w = rng.uniform(-bound, bound, nw).astype(np.float32)
        elif init == "he":
            w = (rng.standard_normal(nw) * math.sqrt(2.0 / fan_in)).astype(np.float32)
        else:
            raise ValueError(init)
        params.append((i, 0, w))
        params.append((i, 1, np.zeros(nb, np.float32)))
    return params


def spec_sizes(spec):
    """(input floats per sample, output floats per sample)."""
    first, last_out = spec[0], None
    in_size = first[1] * first[2] * first[3] if first[0] in ("conv", "maxpool", "avepool") else first[1]
    cur = in_size
    for l in spec:
        if l[0] == "conv":
            _, w, h, c, k, oc, same = l[:7]
            ow, oh = (w, h) if same else (w - k + 1, h - k + 1)
            cur = ow * oh * oc
        elif l[0] == "fc":
            cur = l[2]
        elif l[0] in ("maxpool", "avepool"):
            cur = (l[1] // l[4]) * (l[2] // l[4]) * l[3]
    last_out = cur
    return in_size, last_out


def make_batch(name, batch=None, size=None):
    """Seeded (spec, params, x, t, batch, loss, opt kind, opt kwargs) for a named workload.

    ``size`` shrinks the VGG stack's input edge for CPU-sized parity cases.
    """
    builder, b0, loss, opt_kind, opt_kw, init, dist, seed = WORKLOADS[name]
    batch = b0 if batch is None else batch
    spec = builder(size) if (size is not None and builder is vgg_stack) else builder()
    rng = np.random.Generator(np.random.Philox(seed))
    params = init_params(spec, init, rng)
    in_size, out_size = spec_sizes(spec)
    if dist == "uniform":
        x = rng.uniform(-1.0, 1.0, (batch, in_size)).astype(np.float32)
    else:
        x = rng.standard_normal((batch, in_size)).astype(np.float32)
    labels = rng.integers(0, out_size, batch)
    if loss == "mse":
        # one-hot targets scaled to tanh's range (tanh_layer::scale, tanh_layer.h:40-42)
        t = np.full((batch, out_size), -0.8, np.float32)
        t[np.arange(batch), labels] = 0.8
    else:
        t = np.zeros((batch, out_size), np.float32)
        t[np.arange(batch), labels] = 1.0
    return spec, params, x, t, batch, loss, opt_kind, opt_kw


def conv_bwd_case(batch=64, c=32, hw=64, oc=64, k=3, seed=1235):
    """configs[1]: single conv2d backward, pad same, stride 1. Returns (dims, x, w, dy)."""
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((batch, c * hw * hw)).astype(np.float32)
    dy = rng.standard_normal((batch, oc * hw * hw)).astype(np.float32)
    bound = math.sqrt(6.0 / (k * k * c + k * k * oc))
    w = rng.uniform(-bound, bound, oc * c * k * k).astype(np.float32)
    return (hw, hw, c, k, oc), x, w, dy


def fc_bwd_case(batch=256, n_in=4096, n_out=4096, seed=1236):
    """configs[2]: FC backward + Adam. Returns (x, w, b, dy); the layer is followed by tanh."""
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.uniform(-1.0, 1.0, (batch, n_in)).astype(np.float32)
    bound = math.sqrt(6.0 / (n_in + n_out))
    w = rng.uniform(-bound, bound, n_in * n_out).astype(np.float32)
    b = np.zeros(n_out, np.float32)
    dy = (rng.standard_normal((batch, n_out)) * 0.1).astype(np.float32)
    return x, w, b, dy


def flops_per_sample(spec):
    """2*MACs of the forward pass per sample for conv/fc layers; a train step is ~3x."""
    total = 0
    for l in spec:
        if l[0] == "conv":
            _, w, h, c, k, oc, same = l[:7]
            ow, oh = (w, h) if same else (w - k + 1, h - k + 1)
            total += 2 * ow * oh * oc * c * k * k
        elif l[0] == "fc":
            total += 2 * l[1] * l[2]
    return total


# not a benchmark configuration: a small net with the two layers whose backward pass needs more
# than the layer's own output gradient, for parity tests of the device-resident step
BN_DROPOUT_NET = [("conv", 10, 10, 2, 3, 6, True), ("batchnorm", 6, 100), ("act", "relu"),
                  ("maxpool", 10, 10, 6, 2), ("fc", 150, 20), ("act", "tanh"), ("dropout", 0.4),
                  ("fc", 20, 10), ("act", "softmax")]


def bn_dropout_case(batch=7, seed=21):
    """Seeded (params, x, one-hot t) for BN_DROPOUT_NET."""
    rng = np.random.default_rng(seed)
    params = []
    for i, l in enumerate(BN_DROPOUT_NET):
        nw, nb, fan_in, _ = layer_fans(l)
        if nw:
            params += [(i, 0, rng.uniform(-1, 1, nw).astype(np.float32) * np.float32(math.sqrt(3.0 / fan_in))),
                       (i, 1, rng.uniform(-.2, .2, nb).astype(np.float32))]
    x = rng.standard_normal((batch, 200)).astype(np.float32)
    t = np.eye(10, dtype=np.float32)[rng.integers(0, 10, batch)]
    return params, x, t
