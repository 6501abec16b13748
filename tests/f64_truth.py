"""Float64 re-statements used by the GPU tests where fp32 summation order alone decides whether
a result is within 1e-4 of the oracle: the value both are measured against."""
import numpy as np

from conftest import REL_TOL, elementwise_rel_err, rel_err


def assert_not_worse_than_oracle(gpu, oracle, truth, what, tol=REL_TOL):
    eg, eo = rel_err(gpu, truth), rel_err(oracle, truth)
    print(f"{what}: gpu-f64 {eg:.3e} (element-wise {elementwise_rel_err(gpu, truth):.3e}), "
          f"oracle-f64 {eo:.3e} (element-wise {elementwise_rel_err(oracle, truth):.3e}), "
          f"gpu-oracle {rel_err(gpu, oracle):.3e}")
    assert eg <= eo + tol, f"{what}: GPU is {eg:.3e} from float64, the oracle {eo:.3e}"


def f64_net_steps(spec, params, x, t, loss, steps, opt, want_trace=False):
    """The reference's train step in float64: torch CPU autograd for the layers (cross-correlation
    with OIHW filters and the connection table as a 0/1 mask, [in][out] fully-connected weights,
    average pooling with its trainable per-channel scale and bias, gradients SUMMED over the
    batch as layer::update_weight hands them to the optimizer) and tiny-dnn's optimizers in
    numpy (optimizer.h): adam with eps inside the square root and the bias-correction powers
    advanced once per tensor (:112-127), adagrad (:57-71), momentum (:201-218), sgd (:182-192).
    `opt` = {"kind", "alpha", ...}. Returns {(layer, which): updated parameter} and, with
    want_trace, {(layer, which): [(gradient, b1_t, b2_t) per step]}."""
    import torch
    import torch.nn.functional as F
    P = {(i, which): torch.tensor(np.asarray(a, np.float64), requires_grad=True) for (i, which, a) in params}
    state = {k: [np.zeros(p.numel()), np.zeros(p.numel())] for k, p in P.items()}
    trace = {k: [] for k in P}
    b1_t, b2_t = opt.get("b1", 0.0), opt.get("b2", 0.0)
    X, Tt = torch.tensor(x.astype(np.float64)), torch.tensor(t.astype(np.float64))
    for _ in range(steps):
        a = X
        for i, l in enumerate(spec):
            if l[0] == "conv":
                _, w, h, c, k, oc, same = l[:7]
                wt = P[(i, 0)].reshape(oc, c, k, k)
                if len(l) > 7 and l[7] is not None:
                    mask = torch.tensor(np.asarray(l[7], np.float64).reshape(c, oc).T.copy())
                    wt = wt * mask[:, :, None, None]
                a = F.conv2d(a.reshape(-1, c, h, w), wt, P[(i, 1)], padding=k // 2 if same else 0)
            elif l[0] == "fc":
                a = a.reshape(a.shape[0], -1) @ P[(i, 0)].reshape(l[1], l[2]) + P[(i, 1)]
            elif l[0] == "maxpool":
                a = F.max_pool2d(a.reshape(-1, l[3], l[2], l[1]), l[4])
            elif l[0] == "avepool":   # W[c] * scale * sum(window) + b[c] (average_pooling_layer.h:34-51)
                a = (F.avg_pool2d(a.reshape(-1, l[3], l[2], l[1]), l[4]) * P[(i, 0)][None, :, None, None]
                     + P[(i, 1)][None, :, None, None])
            elif l[0] == "act":
                flat = a.reshape(a.shape[0], -1)
                a = {"relu": torch.relu, "tanh": torch.tanh, "sigmoid": torch.sigmoid,
                     "softmax": lambda z: torch.softmax(z, 1)}[l[1]](flat)
            else:
                raise ValueError(l)
        y = a.reshape(a.shape[0], -1)
        if loss == "mse":      # sum over samples of mse::f; df = 2/n (y - t) (loss_function.h:28-36)
            L = ((y - Tt) ** 2).sum() / y.shape[1]
        else:                  # cross_entropy_multiclass: -sum t log y (loss_function.h:132-150)
            L = -(Tt * torch.log(y)).sum()
        for p in P.values():
            p.grad = None
        L.backward()
        with torch.no_grad():
            for key in sorted(P):       # layer by layer, weight before bias
                g = P[key].grad.numpy().ravel().copy()
                w = P[key].detach().numpy().reshape(-1)      # a view: updated in place
                trace[key].append((g, b1_t, b2_t))
                w += opt_delta(opt, state[key], g, w, b1_t, b2_t)
                if opt["kind"] == "adam":
                    b1_t *= opt["b1"]
                    b2_t *= opt["b2"]
    params_out = {k: p.detach().numpy().ravel().copy() for k, p in P.items()}
    return (params_out, trace) if want_trace else params_out


def opt_delta(opt, st, g, w, b1_t=0.0, b2_t=0.0):
    """One optimizer::update in float64, element-wise: returns the change of w and advances the
    state vectors st = [s0, s1] (tiny_dnn/optimizers/optimizer.h)."""
    kind = opt["kind"]
    if kind == "adam":       # :112-127, eps inside the square root
        st[0] = opt["b1"] * st[0] + (1 - opt["b1"]) * g
        st[1] = opt["b2"] * st[1] + (1 - opt["b2"]) * g * g
        return -opt["alpha"] * (st[0] / (1 - b1_t)) / np.sqrt(st[1] / (1 - b2_t) + opt["eps"])
    if kind == "adagrad":    # :57-71
        st[0] = st[0] + g * g
        return -opt["alpha"] * g / (np.sqrt(st[0]) + opt.get("eps", 1e-8))
    if kind == "momentum":   # :201-218
        st[0] = opt["mu"] * st[0] - opt["alpha"] * (g + opt.get("lambda", 0.0) * w)
        return st[0]
    if kind == "sgd":        # :182-192
        return -opt["alpha"] * (g + opt.get("lambda", 0.0) * w)
    raise ValueError(kind)


def propagated_gradient_tolerance(opt, trace, rel=REL_TOL):
    """What the parity bound ON GRADIENTS allows the updated weights to differ by, element by
    element, to first order: a gradient may be off by rel * rms(gradient) (the bound every
    gradient test uses); this replays one tensor's optimizer steps on its float64 gradients
    g_1..g_K with one step's gradient moved by that much, up and down, and adds up how far the
    total update moves. For sgd/momentum that is alpha * rel * rms(g): nothing. adam, adagrad,
    RMSprop and adamax divide an element by its own accumulated magnitude, so for an element
    whose gradient nearly cancelled (|g| << rms) the same absolute error moves the update by up
    to its full size, alpha."""
    assert opt.get("lambda", 0.0) == 0.0

    def total(grads):
        st = [np.zeros_like(grads[0]), np.zeros_like(grads[0])]
        out = np.zeros_like(grads[0])
        for (g, (_, b1_t, b2_t)) in zip(grads, trace):
            out += opt_delta(opt, st, g, 0.0, b1_t, b2_t)
        return out

    base = [g for (g, _, _) in trace]
    u0 = total(base)
    tol = np.zeros_like(u0)
    for k, g in enumerate(base):
        d = rel * np.sqrt(np.mean(g * g))
        moved = [np.abs(total(base[:k] + [g + sgn * d] + base[k + 1:]) - u0) for sgn in (1.0, -1.0)]
        tol += np.maximum(*moved)
    return tol


def assert_within_propagated_tolerance(gpu, oracle, truth, opt, trace, what, tol=REL_TOL):
    """Updated weights after steps of a normalising optimizer: every element within
    tol * max(|w|, rms(w)) plus what the gradient bound allows (propagated_gradient_tolerance),
    and the bulk (99th percentile of the error against float64) no worse than 2x the oracle's."""
    gpu, oracle, truth = (np.asarray(a, np.float64).ravel() for a in (gpu, oracle, truth))
    scale = np.maximum(np.abs(truth), np.sqrt(np.mean(truth * truth)) + 1e-30)
    allowed = tol * scale + propagated_gradient_tolerance(opt, trace, tol)
    eg, eo = np.abs(gpu - truth), np.abs(oracle - truth)
    qg, qo = np.quantile(eg / scale, 0.99), np.quantile(eo / scale, 0.99)
    worst = int(np.argmax(eg / allowed))
    print(f"{what}: gpu-f64 max {np.max(eg / scale):.3e} p99 {qg:.3e}; oracle-f64 max {np.max(eo / scale):.3e} "
          f"p99 {qo:.3e}; gpu-oracle max {rel_err(gpu, oracle):.3e}; worst element uses "
          f"{eg[worst] / allowed[worst]:.2f} of its allowance ({allowed[worst] / scale[worst]:.2e} relative)")
    assert np.all(eg <= allowed), f"{what}: element {worst} is {eg[worst]:.3e} off, allowed {allowed[worst]:.3e}"
    # (slack 3e-6: for a tensor of 16 biases the 99th percentile is the largest error, and two
    # fp32 summation orders differ by a few 1e-6 there whichever is nearer to float64)
    assert qg <= 2 * qo + 3e-6, f"{what}: 99th percentile of the error {qg:.3e}, the oracle's {qo:.3e}"
