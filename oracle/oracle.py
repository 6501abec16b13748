"""ctypes front-end for the CPU oracle (oracle/td_oracle.c) and, when built, the
compiled reference (oracle/_ref/*.so, see oracle/ref_shim.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py — never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libtd_oracle.so")
REF_SCALAR_SO = os.path.join(HERE, "_ref", "libtd_ref_scalar.so")
REF_AVX_SO = os.path.join(HERE, "_ref", "libtd_ref_avx.so")
REF_SER_SO = os.path.join(HERE, "_ref", "libtd_ref_ser.so")  # scalar build with serialization on

ACT = {"tanh": 0, "relu": 1, "softmax": 2, "sigmoid": 3, "leaky_relu": 4, "elu": 5, "selu": 6,
       "softplus": 7, "softsign": 8, "asinh": 9, "tanh_p1m2": 10}
# constructor defaults of the parameterised activation layers (leaky_relu_layer.h:25,
# elu_layer.h:18, selu_layer.h:26-27, softplus_layer.h:26-27)
ACT_DEFAULTS = {"leaky_relu": (0.01, 0.0), "elu": (1.0, 0.0), "selu": (1.05070, 1.67326),
                "softplus": (1.0, 20.0)}


def act_params(kind, params=None):
    p = list(params) if params is not None else list(ACT_DEFAULTS.get(kind, (0.0, 0.0)))
    p += [0.0] * (2 - len(p))
    return (C.c_float * 2)(*p)
LOSS = {"mse": 0, "ce_multiclass": 1, "ce": 2}
OPT = {"sgd": 0, "momentum": 1, "adam": 2, "adagrad": 3, "rmsprop": 4, "adamax": 5, "nesterov": 6}
L_CONV, L_FC, L_MAXPOOL, L_AVEPOOL, L_ACT, L_BATCHNORM, L_DROPOUT = range(7)

f32p = C.POINTER(C.c_float)
i64p = C.POINTER(C.c_int64)


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "in_c", "k_w", "k_h", "out_c", "w_stride", "h_stride",
        "w_dilation", "h_dilation", "pad_same", "has_bias")] + [("tbl", C.c_void_p)]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "in_c", "pool_w", "pool_h", "stride_w", "stride_h", "pad_same", "ceil_mode")]


class OptDesc(C.Structure):
    _fields_ = [("kind", C.c_int32)] + [(n, C.c_float) for n in (
        "alpha", "lam", "mu", "b1", "b2", "eps", "b1_t", "b2_t")]


class LayerDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("act", C.c_int32), ("conv", ConvDesc), ("pool", PoolDesc),
                ("fc_in", C.c_int32), ("fc_out", C.c_int32), ("fc_bias", C.c_int32),
                ("act_p", C.c_float * 2), ("bn_channels", C.c_int32), ("bn_spatial", C.c_int32),
                ("bn_eps", C.c_float), ("bn_momentum", C.c_float), ("dropout_rate", C.c_float)]


def conv_desc(in_w, in_h, in_c, k_w, k_h, out_c, pad_same=False, has_bias=True, w_stride=1,
              h_stride=1, w_dilation=1, h_dilation=1, tbl=None):
    """tbl: optional bool array [in_c][out_c] (rows = in channels, as the reference's
    connection_table(ar, rows, cols))."""
    d = ConvDesc(in_w, in_h, in_c, k_w, k_h, out_c, w_stride, h_stride, w_dilation, h_dilation,
                 int(pad_same), int(has_bias), None)
    if tbl is not None:
        keep = np.ascontiguousarray(np.asarray(tbl, dtype=np.uint8).reshape(in_c, out_c))
        d._keep = keep  # keep the buffer alive as long as the descriptor
        d.tbl = keep.ctypes.data
    return d


def pool_desc(in_w, in_h, in_c, pool_w, pool_h=None, stride_w=None, stride_h=None,
              pad_same=False, ceil_mode=False):
    pool_h = pool_w if pool_h is None else pool_h
    stride_w = pool_w if stride_w is None else stride_w
    stride_h = pool_h if stride_h is None else stride_h
    return PoolDesc(in_w, in_h, in_c, pool_w, pool_h, stride_w, stride_h, int(pad_same),
                    int(ceil_mode))


def opt_desc(kind, **kw):
    lib = oracle_lib()
    o = OptDesc()
    lib.tdo_opt_default(C.byref(o), OPT[kind] if isinstance(kind, str) else kind)
    for k, v in kw.items():
        setattr(o, "lam" if k == "lambda_" else k, v)
    return o


def build(force=False):
    """Compile libtd_oracle.so (and oracle/_ref when the reference tree exists)."""
    if force:
        subprocess.run(["make", "-C", HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)


_oracle = None
_ref = {}


def oracle_lib():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            build()
        lib = C.CDLL(ORACLE_SO)
        lib.tdo_loss_value.restype = C.c_float
        for name in ("tdo_net_create",):
            getattr(lib, name).restype = C.c_void_p
        for name in ("tdo_net_in_size", "tdo_net_out_size", "tdo_net_weight_size",
                     "tdo_net_bias_size", "tdo_net_layer_out_size"):
            getattr(lib, name).restype = C.c_size_t
        for name in ("tdo_net_weight", "tdo_net_bias", "tdo_net_layer_out", "tdo_net_layer_dx",
                     "tdo_net_layer_dw", "tdo_net_layer_db"):
            getattr(lib, name).restype = f32p
        lib.tdo_net_layer_argmax.restype = i64p
        _oracle = lib
    return _oracle


def ref_lib(kind="scalar"):
    """The compiled reference ('scalar', 'avx', or 'ser': the scalar build with the
    reference's cereal serialization compiled in), or None when it is not built."""
    if kind not in _ref:
        path = {"scalar": REF_SCALAR_SO, "avx": REF_AVX_SO, "ser": REF_SER_SO}[kind]
        if not os.path.exists(path):
            _ref[kind] = None
        else:
            lib = C.CDLL(path)
            lib.tdr_conv2d_bwd.restype = C.c_double
            lib.tdr_fc_bwd.restype = C.c_double
            lib.tdr_net_fit.restype = C.c_double
            lib.tdr_net_create.restype = C.c_void_p
            lib.tdr_net_param_size.restype = C.c_size_t
            _ref[kind] = lib
    return _ref[kind]


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(f32p)


def _chk(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def conv_out_shape(d):
    lib = oracle_lib()
    return lib.tdo_conv_out_w(C.byref(d)), lib.tdo_conv_out_h(C.byref(d))


def pool_out_shape(d):
    lib = oracle_lib()
    return lib.tdo_pool_out_w(C.byref(d)), lib.tdo_pool_out_h(C.byref(d))


# ------------------------------------------------------------------ oracle ops

def conv2d_fwd(d, x, w, b=None):
    lib = oracle_lib()
    batch = x.shape[0]
    ow, oh = conv_out_shape(d)
    x, xp = _f(x); w, wp = _f(w)
    b = np.zeros(d.out_c, np.float32) if b is None else b
    b, bp = _f(b)
    y = np.empty((batch, d.out_c * oh * ow), np.float32)
    _chk(lib.tdo_conv2d_fwd(C.byref(d), batch, xp, wp, bp, y.ctypes.data_as(f32p)), "conv2d_fwd")
    return y


def conv2d_bwd(d, x, w, dy):
    lib = oracle_lib()
    batch = x.shape[0]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    dw = np.empty(w.size, np.float32)
    db = np.zeros(d.out_c, np.float32)
    _chk(lib.tdo_conv2d_bwd(C.byref(d), batch, xp, wp, dyp, dx.ctypes.data_as(f32p),
                            dw.ctypes.data_as(f32p), db.ctypes.data_as(f32p)), "conv2d_bwd")
    return dx, dw, (db if d.has_bias else None)


def fc_fwd(x, w, b=None):
    lib = oracle_lib()
    batch, n_in = x.shape
    n_out = w.size // n_in
    x, xp = _f(x); w, wp = _f(w)
    bb, bp = _f(np.zeros(n_out, np.float32) if b is None else b)
    y = np.empty((batch, n_out), np.float32)
    _chk(lib.tdo_fc_fwd(n_in, n_out, int(b is not None), batch, xp, wp, bp,
                        y.ctypes.data_as(f32p)), "fc_fwd")
    return y


def fc_bwd(x, w, dy, has_bias=True):
    lib = oracle_lib()
    batch, n_in = x.shape
    n_out = dy.shape[1]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, n_in), np.float32)
    dw = np.empty(n_in * n_out, np.float32)
    db = np.zeros(n_out, np.float32)
    _chk(lib.tdo_fc_bwd(n_in, n_out, int(has_bias), batch, xp, wp, dyp, dx.ctypes.data_as(f32p),
                        dw.ctypes.data_as(f32p), db.ctypes.data_as(f32p)), "fc_bwd")
    return dx, dw, (db if has_bias else None)


def maxpool_fwd(d, x):
    lib = oracle_lib()
    batch = x.shape[0]
    ow, oh = pool_out_shape(d)
    x, xp = _f(x)
    y = np.empty((batch, d.in_c * oh * ow), np.float32)
    am = np.empty((batch, d.in_c * oh * ow), np.int64)
    _chk(lib.tdo_maxpool_fwd(C.byref(d), batch, xp, y.ctypes.data_as(f32p),
                             am.ctypes.data_as(i64p)), "maxpool_fwd")
    return y, am


def maxpool_bwd(d, dy, argmax):
    lib = oracle_lib()
    batch = dy.shape[0]
    dy, dyp = _f(dy)
    am = np.ascontiguousarray(argmax, dtype=np.int64)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    _chk(lib.tdo_maxpool_bwd(C.byref(d), batch, dyp, am.ctypes.data_as(i64p),
                             dx.ctypes.data_as(f32p)), "maxpool_bwd")
    return dx


def avepool_fwd(d, x, w, b):
    lib = oracle_lib()
    batch = x.shape[0]
    ow, oh = pool_out_shape(d)
    x, xp = _f(x); w, wp = _f(w); b, bp = _f(b)
    y = np.empty((batch, d.in_c * oh * ow), np.float32)
    _chk(lib.tdo_avepool_fwd(C.byref(d), batch, xp, wp, bp, y.ctypes.data_as(f32p)), "avepool_fwd")
    return y


def avepool_bwd(d, x, w, dy):
    lib = oracle_lib()
    batch = x.shape[0]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    dw = np.empty(d.in_c, np.float32)
    db = np.empty(d.in_c, np.float32)
    _chk(lib.tdo_avepool_bwd(C.byref(d), batch, xp, wp, dyp, dx.ctypes.data_as(f32p),
                             dw.ctypes.data_as(f32p), db.ctypes.data_as(f32p)), "avepool_bwd")
    return dx, dw, db


def act_fwd(kind, x, params=None):
    lib = oracle_lib()
    x, xp = _f(x)
    y = np.empty_like(x)
    _chk(lib.tdo_act_fwd_p(ACT[kind], act_params(kind, params), x.shape[0], x.shape[1], xp,
                           y.ctypes.data_as(f32p)), "act_fwd")
    return y


def act_bwd(kind, x, y, dy, params=None):
    lib = oracle_lib()
    x, xp = _f(x); y, yp = _f(y); dy, dyp = _f(dy)
    dx = np.empty_like(x)
    _chk(lib.tdo_act_bwd_p(ACT[kind], act_params(kind, params), x.shape[0], x.shape[1], xp, yp, dyp,
                           dx.ctypes.data_as(f32p)), "act_bwd")
    return dx


def batchnorm_fwd(channels, spatial, x, eps=1e-5, train=True, mean=None, variance=None):
    """Returns (y, mean, variance, stddev); train=False reads mean/variance."""
    lib = oracle_lib()
    x, xp = _f(x)
    mean = np.zeros(channels, np.float32) if mean is None else np.array(mean, np.float32)
    variance = np.zeros(channels, np.float32) if variance is None else np.array(variance, np.float32)
    stddev = np.zeros(channels, np.float32)
    y = np.empty_like(x)
    _chk(lib.tdo_batchnorm_fwd(channels, spatial, x.shape[0], C.c_float(eps), int(bool(train)), xp,
                               mean.ctypes.data_as(f32p), variance.ctypes.data_as(f32p),
                               stddev.ctypes.data_as(f32p), y.ctypes.data_as(f32p)), "batchnorm_fwd")
    return y, mean, variance, stddev


def batchnorm_bwd(channels, spatial, y, dy, stddev):
    lib = oracle_lib()
    y, yp = _f(y); dy, dyp = _f(dy); stddev, sp = _f(stddev)
    dx = np.empty_like(y)
    _chk(lib.tdo_batchnorm_bwd(channels, spatial, y.shape[0], yp, dyp, sp, dx.ctypes.data_as(f32p)),
         "batchnorm_bwd")
    return dx


def batchnorm_update_moving(momentum, mean_cur, var_cur, mean, variance):
    lib = oracle_lib()
    mean = np.array(mean, np.float32); variance = np.array(variance, np.float32)
    mc, mcp = _f(mean_cur); vc, vcp = _f(var_cur)
    lib.tdo_batchnorm_update_moving(mean.size, C.c_float(momentum), mcp, vcp,
                                    mean.ctypes.data_as(f32p), variance.ctypes.data_as(f32p))
    return mean, variance


def mt_seed(state, seed):
    """Seeds a 625-word generator state (np.uint32) like set_random_seed(seed)."""
    oracle_lib().tdo_mt_seed(state.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_uint32(seed))
    return state


def dropout_mask(seed, rate, batch, length, state=None):
    """The mask dropout_layer draws after set_random_seed(seed) (one worker thread)."""
    lib = oracle_lib()
    st = np.zeros(625, np.uint32) if state is None else state
    if state is None:
        lib.tdo_mt_seed(st.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_uint32(seed))
    mask = np.zeros((batch, length), np.uint8)
    lib.tdo_dropout_mask(st.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_float(rate),
                         C.c_size_t(batch * length), mask.ctypes.data_as(C.POINTER(C.c_uint8)))
    return mask


def dropout_fwd(mask, x, rate=0.5, train=True):
    lib = oracle_lib()
    x, xp = _f(x)
    mask = np.ascontiguousarray(mask, np.uint8)
    y = np.empty_like(x)
    scale = np.float32(1) / (np.float32(1) - np.float32(rate))
    _chk(lib.tdo_dropout_fwd(x.shape[0], x.shape[1], int(bool(train)), C.c_float(scale),
                             mask.ctypes.data_as(C.POINTER(C.c_uint8)), xp, y.ctypes.data_as(f32p)),
         "dropout_fwd")
    return y


def dropout_bwd(mask, dy):
    lib = oracle_lib()
    dy, dyp = _f(dy)
    mask = np.ascontiguousarray(mask, np.uint8)
    dx = np.empty_like(dy)
    _chk(lib.tdo_dropout_bwd(dy.shape[0], dy.shape[1], mask.ctypes.data_as(C.POINTER(C.c_uint8)), dyp,
                             dx.ctypes.data_as(f32p)), "dropout_bwd")
    return dx


def loss_grad(kind, y, t):
    lib = oracle_lib()
    y, yp = _f(y); t, tp = _f(t)
    dy = np.empty_like(y)
    _chk(lib.tdo_loss_grad(LOSS[kind], y.shape[0], y.shape[1], yp, tp, dy.ctypes.data_as(f32p)),
         "loss_grad")
    return dy


def opt_update(o, g, w, s0=None, s1=None):
    """In-place optimizer::update; o (OptDesc) carries b1_t/b2_t across calls."""
    lib = oracle_lib()
    g, gp = _f(g)
    assert w.dtype == np.float32 and w.flags.c_contiguous
    s0p = s0.ctypes.data_as(f32p) if s0 is not None else None
    s1p = s1.ctypes.data_as(f32p) if s1 is not None else None
    _chk(lib.tdo_opt_update(C.byref(o), C.c_size_t(w.size), gp, w.ctypes.data_as(f32p), s0p, s1p),
         "opt_update")


def update_weight(o, weight_edge_samples, merged, w, s0=None, s1=None):
    lib = oracle_lib()
    g, gp = _f(merged)
    assert w.dtype == np.float32 and w.flags.c_contiguous
    s0p = s0.ctypes.data_as(f32p) if s0 is not None else None
    s1p = s1.ctypes.data_as(f32p) if s1 is not None else None
    _chk(lib.tdo_update_weight(C.byref(o), C.c_size_t(w.size), weight_edge_samples, gp, w.ctypes.data_as(f32p),
                               s0p, s1p), "update_weight")


# ------------------------------------------------------------ network specs

def L_conv(in_w, in_h, in_c, k, out_c, pad_same=False, has_bias=True, stride=1, tbl=None):
    l = LayerDesc()
    l.kind = L_CONV
    d = conv_desc(in_w, in_h, in_c, k, k, out_c, pad_same, has_bias, stride, stride, tbl=tbl)
    l.conv = d                           # copies the struct: the table's array must outlive it
    l._keep = getattr(d, "_keep", None)
    return l


def L_fc(n_in, n_out, has_bias=True):
    l = LayerDesc()
    l.kind, l.fc_in, l.fc_out, l.fc_bias = L_FC, n_in, n_out, int(has_bias)
    return l


def L_maxpool(in_w, in_h, in_c, pool, stride=None):
    l = LayerDesc()
    l.kind = L_MAXPOOL
    l.pool = pool_desc(in_w, in_h, in_c, pool, stride_w=stride)
    return l


def L_avepool(in_w, in_h, in_c, pool, stride=None):
    l = LayerDesc()
    l.kind = L_AVEPOOL
    l.pool = pool_desc(in_w, in_h, in_c, pool, stride_w=stride)
    return l


def L_batchnorm(channels, spatial, eps=1e-5, momentum=0.999):
    """batch_normalization_layer(in_spatial_size, in_channels, epsilon, momentum)"""
    l = LayerDesc()
    l.kind, l.bn_channels, l.bn_spatial, l.bn_eps, l.bn_momentum = L_BATCHNORM, channels, spatial, eps, momentum
    return l


def L_dropout(rate):
    """dropout_layer(in_dim, dropout_rate); the shape is the previous layer's"""
    l = LayerDesc()
    l.kind, l.dropout_rate = L_DROPOUT, rate
    return l


def L_act(kind, params=None):
    l = LayerDesc()
    l.kind, l.act = L_ACT, ACT[kind]
    l.act_p = act_params(kind, params)
    return l


def layer_array(layers):
    arr = (LayerDesc * len(layers))()
    for i, l in enumerate(layers):
        arr[i] = l
    arr._keep = layers
    return arr


class OracleNet:
    """Sequential network stepped by the oracle (tdo_net_*)."""

    def __init__(self, layers, max_batch):
        self.lib = oracle_lib()
        self.layers = layers
        self.arr = layer_array(layers)
        self.h = C.c_void_p(self.lib.tdo_net_create(self.arr, len(layers), max_batch))
        if not self.h:
            raise RuntimeError("tdo_net_create failed (inconsistent layer shapes?)")
        self.n = len(layers)
        self.max_batch = max_batch

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.tdo_net_destroy(self.h)
            self.h = None

    def _view(self, ptr, n):
        return np.ctypeslib.as_array(ptr, shape=(n,)) if n else np.zeros(0, np.float32)

    def weight(self, i):
        return self._view(self.lib.tdo_net_weight(self.h, i), self.lib.tdo_net_weight_size(self.h, i))

    def bias(self, i):
        return self._view(self.lib.tdo_net_bias(self.h, i), self.lib.tdo_net_bias_size(self.h, i))

    def params(self):
        """[(layer, which, view)] in the reference's update order (weight then bias)."""
        out = []
        for i in range(self.n):
            if self.lib.tdo_net_weight_size(self.h, i):
                out.append((i, 0, self.weight(i)))
            if self.lib.tdo_net_bias_size(self.h, i):
                out.append((i, 1, self.bias(i)))
        return out

    def in_size(self):
        return self.lib.tdo_net_in_size(self.h)

    def out_size(self):
        return self.lib.tdo_net_out_size(self.h)

    def layer_out(self, i, batch):
        n = self.lib.tdo_net_layer_out_size(self.h, i)
        return self._view(self.lib.tdo_net_layer_out(self.h, i), n * batch).reshape(batch, n).copy()

    def layer_dw(self, i):
        return self._view(self.lib.tdo_net_layer_dw(self.h, i),
                          self.lib.tdo_net_weight_size(self.h, i)).copy()

    def layer_db(self, i):
        return self._view(self.lib.tdo_net_layer_db(self.h, i),
                          self.lib.tdo_net_bias_size(self.h, i)).copy()

    def layer_dx(self, i, batch):
        n = self.lib.tdo_net_in_size(self.h) if i == 0 else self.lib.tdo_net_layer_out_size(self.h, i - 1)
        return self._view(self.lib.tdo_net_layer_dx(self.h, i), n * batch).reshape(batch, n).copy()

    def layer_argmax(self, i, batch):
        n = self.lib.tdo_net_layer_out_size(self.h, i)
        p = self.lib.tdo_net_layer_argmax(self.h, i)
        return np.ctypeslib.as_array(p, shape=(n * batch,)).reshape(batch, n).copy()

    def set_phase(self, train):
        self.lib.tdo_net_set_phase(self.h, int(bool(train)))

    def set_dropout_mask(self, i, mask):
        """mask: uint8 [batch][len] that the next passes of dropout layer i apply"""
        mask = np.ascontiguousarray(mask, np.uint8)
        self.lib.tdo_net_dropout_mask.restype = C.POINTER(C.c_uint8)
        dst = np.ctypeslib.as_array(self.lib.tdo_net_dropout_mask(self.h, i), shape=(mask.size,))
        dst[:] = mask.ravel()

    def bn_stat(self, i, which):
        """moving mean (0) / variance (1) of batch-norm layer i (a view)"""
        self.lib.tdo_net_bn_stat.restype = f32p
        return np.ctypeslib.as_array(self.lib.tdo_net_bn_stat(self.h, i, which),
                                     shape=(self.layers[i].bn_channels,))

    def forward(self, x):
        x, xp = _f(x)
        _chk(self.lib.tdo_net_forward(self.h, x.shape[0], xp), "net_forward")
        return self.layer_out(self.n - 1, x.shape[0])

    def train_step(self, opt, loss, x, t, do_update=True):
        x, xp = _f(x); t, tp = _f(t)
        _chk(self.lib.tdo_net_train_step(self.h, C.byref(opt), LOSS[loss], x.shape[0], xp, tp,
                                         int(do_update)), "net_train_step")


class RefNet:
    """The same network built from real tiny-dnn layers (oracle/_ref)."""

    def __init__(self, layers, kind="scalar", engine=0):
        self.lib = ref_lib(kind)
        if self.lib is None:
            raise RuntimeError("compiled reference not built")
        self.arr = layer_array(layers)
        self.h = C.c_void_p(self.lib.tdr_net_create(self.arr, len(layers), engine))
        if not self.h:
            raise RuntimeError("tdr_net_create failed")
        self.n = len(layers)

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.tdr_net_destroy(self.h)
            self.h = None

    def param_size(self, layer, which):
        return self.lib.tdr_net_param_size(self.h, layer, which)

    def set_param(self, layer, which, a):
        n = self.param_size(layer, which)
        a = np.asarray(a, dtype=np.float32).ravel()
        if a.size < n:  # ave-pool weight vectors are longer than their used prefix
            a = np.concatenate([a, np.zeros(n - a.size, np.float32)])
        a, ap = _f(a)
        assert a.size == n
        _chk(self.lib.tdr_net_set_param(self.h, layer, which, ap), "set_param")

    def get_param(self, layer, which):
        a = np.empty(self.param_size(layer, which), np.float32)
        _chk(self.lib.tdr_net_get_param(self.h, layer, which, a.ctypes.data_as(f32p)), "get_param")
        return a

    def save_weights(self, path):
        _chk(self.lib.tdr_net_save_weights(self.h, str(path).encode()), "save_weights")

    def load_weights(self, path):
        _chk(self.lib.tdr_net_load_weights(self.h, str(path).encode()), "load_weights")

    # network::save / load with cereal archives (kind "ser" only): what 0 weights, 1 model,
    # 2 weights_and_model; fmt 0 binary, 1 portable_binary, 2 json
    def save_archive(self, path, what=0, fmt=0):
        _chk(self.lib.tdr_net_save_archive(self.h, str(path).encode(), what, fmt), "save_archive")

    def load_archive(self, path, what=0, fmt=0):
        _chk(self.lib.tdr_net_load_archive(self.h, str(path).encode(), what, fmt), "load_archive")

    def set_random_seed(self, seed):
        """set_random_seed of the reference: its dropout layers draw from this generator"""
        self.lib.tdr_set_random_seed(C.c_uint(seed))

    def bn_stat(self, layer, which, channels):
        a = np.empty(channels, np.float32)
        _chk(self.lib.tdr_net_get_bn_stat(self.h, layer, which, a.ctypes.data_as(f32p), channels), "bn_stat")
        return a

    def fit(self, opt, loss, x, t, steps=1):
        x, xp = _f(x); t, tp = _f(t)
        sec = self.lib.tdr_net_fit(self.h, C.byref(opt), LOSS[loss], x.shape[0], xp,
                                   C.c_size_t(x.shape[1]), tp, C.c_size_t(t.shape[1]), steps)
        if sec < 0:
            raise RuntimeError("tdr_net_fit failed")
        return sec

    def predict(self, x, out_len):
        x, xp = _f(x)
        y = np.empty((x.shape[0], out_len), np.float32)
        _chk(self.lib.tdr_net_predict(self.h, x.shape[0], xp, C.c_size_t(x.shape[1]),
                                      y.ctypes.data_as(f32p), C.c_size_t(out_len)), "predict")
        return y


# ----------------------------------------------------- compiled reference ops

def ref_conv2d_fwd(d, x, w, b=None, kind="scalar", engine=0):
    lib = ref_lib(kind)
    batch = x.shape[0]
    ow, oh = conv_out_shape(d)
    x, xp = _f(x); w, wp = _f(w)
    b, bp = _f(np.zeros(d.out_c, np.float32) if b is None else b)
    y = np.empty((batch, d.out_c * oh * ow), np.float32)
    _chk(lib.tdr_conv2d_fwd(C.byref(d), engine, batch, xp, wp, bp, y.ctypes.data_as(f32p)),
         "ref conv2d_fwd")
    return y


def ref_conv2d_bwd(d, x, w, dy, kind="scalar", engine=0, repeat=1, want_time=False):
    lib = ref_lib(kind)
    batch = x.shape[0]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    dw = np.empty(w.size, np.float32)
    db = np.zeros(d.out_c, np.float32)
    sec = lib.tdr_conv2d_bwd(C.byref(d), engine, batch, xp, wp, dyp, dx.ctypes.data_as(f32p),
                             dw.ctypes.data_as(f32p), db.ctypes.data_as(f32p), repeat)
    if sec < 0:
        raise RuntimeError("ref conv2d_bwd failed")
    out = (dx, dw, (db if d.has_bias else None))
    return out + (sec,) if want_time else out


def ref_fc_fwd(x, w, b=None, kind="scalar", engine=0):
    lib = ref_lib(kind)
    batch, n_in = x.shape
    n_out = w.size // n_in
    x, xp = _f(x); w, wp = _f(w)
    bb, bp = _f(np.zeros(n_out, np.float32) if b is None else b)
    y = np.empty((batch, n_out), np.float32)
    _chk(lib.tdr_fc_fwd(n_in, n_out, int(b is not None), engine, batch, xp, wp, bp,
                        y.ctypes.data_as(f32p)), "ref fc_fwd")
    return y


def ref_fc_bwd(x, w, dy, has_bias=True, kind="scalar", engine=0, repeat=1, want_time=False):
    lib = ref_lib(kind)
    batch, n_in = x.shape
    n_out = dy.shape[1]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, n_in), np.float32)
    dw = np.empty(n_in * n_out, np.float32)
    db = np.zeros(n_out, np.float32)
    sec = lib.tdr_fc_bwd(n_in, n_out, int(has_bias), engine, batch, xp, wp, dyp,
                         dx.ctypes.data_as(f32p), dw.ctypes.data_as(f32p),
                         db.ctypes.data_as(f32p), repeat)
    if sec < 0:
        raise RuntimeError("ref fc_bwd failed")
    out = (dx, dw, (db if has_bias else None))
    return out + (sec,) if want_time else out


def ref_maxpool_fwd_bwd(d, x, dy, kind="scalar", engine=0):
    lib = ref_lib(kind)
    batch = x.shape[0]
    ow, oh = pool_out_shape(d)
    x, xp = _f(x); dy, dyp = _f(dy)
    y = np.empty((batch, d.in_c * oh * ow), np.float32)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    _chk(lib.tdr_maxpool_fwd_bwd(C.byref(d), engine, batch, xp, y.ctypes.data_as(f32p), dyp,
                                 dx.ctypes.data_as(f32p)), "ref maxpool")
    return y, dx


def ref_avepool_fwd(d, x, w, b, kind="scalar"):
    lib = ref_lib(kind)
    batch = x.shape[0]
    ow, oh = pool_out_shape(d)
    x, xp = _f(x); w, wp = _f(w); b, bp = _f(b)
    y = np.empty((batch, d.in_c * oh * ow), np.float32)
    _chk(lib.tdr_avepool_fwd(C.byref(d), batch, xp, wp, bp, y.ctypes.data_as(f32p)),
         "ref avepool_fwd")
    return y


def ref_avepool_bwd(d, x, w, dy, kind="scalar"):
    lib = ref_lib(kind)
    batch = x.shape[0]
    x, xp = _f(x); w, wp = _f(w); dy, dyp = _f(dy)
    dx = np.empty((batch, d.in_c * d.in_h * d.in_w), np.float32)
    dw = np.empty(d.in_c, np.float32)
    db = np.empty(d.in_c, np.float32)
    _chk(lib.tdr_avepool_bwd(C.byref(d), batch, xp, wp, dyp, dx.ctypes.data_as(f32p),
                             dw.ctypes.data_as(f32p), db.ctypes.data_as(f32p)), "ref avepool_bwd")
    return dx, dw, db


def ref_act(kind_name, x, dy=None, kind="scalar", params=None):
    lib = ref_lib(kind)
    x, xp = _f(x)
    y = np.empty_like(x)
    prm = act_params(kind_name, params)
    if dy is None:
        _chk(lib.tdr_act_p(ACT[kind_name], prm, x.shape[0], x.shape[1], xp, y.ctypes.data_as(f32p),
                           None, None), "ref act")
        return y
    dy, dyp = _f(dy)
    dx = np.empty_like(x)
    _chk(lib.tdr_act_p(ACT[kind_name], prm, x.shape[0], x.shape[1], xp, y.ctypes.data_as(f32p), dyp,
                       dx.ctypes.data_as(f32p)), "ref act")
    return y, dx


def ref_batchnorm(channels, spatial, x, dy=None, eps=1e-5, train=True, mean=None, variance=None,
                  kind="scalar"):
    """The compiled reference's batch_normalization_layer: (y, mean, variance[, dx])."""
    lib = ref_lib(kind)
    x, xp = _f(x)
    mean = np.zeros(channels, np.float32) if mean is None else np.array(mean, np.float32)
    variance = np.zeros(channels, np.float32) if variance is None else np.array(variance, np.float32)
    y = np.empty_like(x)
    dx = np.empty_like(x) if dy is not None else None
    dyp = _f(dy)[1] if dy is not None else None
    _chk(lib.tdr_batchnorm(channels, spatial, x.shape[0], C.c_float(eps), int(bool(train)), xp,
                           mean.ctypes.data_as(f32p), variance.ctypes.data_as(f32p),
                           y.ctypes.data_as(f32p), dyp,
                           dx.ctypes.data_as(f32p) if dx is not None else None), "ref batchnorm")
    return (y, mean, variance) if dy is None else (y, mean, variance, dx)


def ref_batchnorm_post_update(channels, spatial, x, mean, variance, eps=1e-5, momentum=0.999,
                              kind="scalar"):
    lib = ref_lib(kind)
    x, xp = _f(x)
    mean = np.array(mean, np.float32); variance = np.array(variance, np.float32)
    _chk(lib.tdr_batchnorm_post_update(channels, spatial, x.shape[0], C.c_float(eps),
                                       C.c_float(momentum), xp, mean.ctypes.data_as(f32p),
                                       variance.ctypes.data_as(f32p)), "ref batchnorm post_update")
    return mean, variance


def ref_dropout(x, dy, rate, seed, kind="scalar"):
    """The compiled reference's dropout_layer after set_random_seed(seed): (mask, y, dx)."""
    lib = ref_lib(kind)
    x, xp = _f(x); dy, dyp = _f(dy)
    mask = np.zeros(x.shape, np.uint8)
    y = np.empty_like(x); dx = np.empty_like(x)
    _chk(lib.tdr_dropout(x.shape[1], x.shape[0], C.c_float(rate), C.c_uint32(seed), xp,
                         mask.ctypes.data_as(C.POINTER(C.c_uint8)), y.ctypes.data_as(f32p), dyp,
                         dx.ctypes.data_as(f32p)), "ref dropout")
    return mask, y, dx


def ref_loss_grad(kind_name, y, t, kind="scalar"):
    lib = ref_lib(kind)
    y, yp = _f(y); t, tp = _f(t)
    dy = np.empty_like(y)
    _chk(lib.tdr_loss_grad(LOSS[kind_name], y.shape[0], y.shape[1], yp, tp,
                           dy.ctypes.data_as(f32p)), "ref loss_grad")
    return dy


def ref_opt_updates(o, g, w, steps, kind="scalar"):
    lib = ref_lib(kind)
    g, gp = _f(g)
    w = np.array(w, dtype=np.float32)
    _chk(lib.tdr_opt_updates(C.byref(o), C.c_size_t(w.size), gp, w.ctypes.data_as(f32p), steps),
         "ref opt_updates")
    return w


# ---- the reference's dataset readers (io/mnist_parser.h, io/cifar10_parser.h)
def ref_parse_mnist_images(path, scale_min, scale_max, x_pad, y_pad, kind="scalar"):
    lib = ref_lib(kind)
    lib.tdr_parse_mnist_images.restype = C.c_long
    n_len = C.c_size_t()
    args = (str(path).encode(), C.c_float(scale_min), C.c_float(scale_max), x_pad, y_pad)
    n = lib.tdr_parse_mnist_images(*args, None, C.byref(n_len))
    if n < 0:
        raise ValueError("reference parser raised nn_error")
    out = np.empty((n, n_len.value), np.float32)
    lib.tdr_parse_mnist_images(*args, out.ctypes.data_as(f32p), None)
    return out


def ref_parse_mnist_labels(path, kind="scalar"):
    lib = ref_lib(kind)
    lib.tdr_parse_mnist_labels.restype = C.c_long
    n = lib.tdr_parse_mnist_labels(str(path).encode(), None)
    if n < 0:
        raise ValueError("reference parser raised nn_error")
    out = np.empty(n, np.int64)
    lib.tdr_parse_mnist_labels(str(path).encode(), out.ctypes.data_as(i64p))
    return out


def ref_parse_cifar10(path, scale_min, scale_max, x_pad, y_pad, kind="scalar"):
    lib = ref_lib(kind)
    lib.tdr_parse_cifar10.restype = C.c_long
    n_len = C.c_size_t()
    args = (str(path).encode(), C.c_float(scale_min), C.c_float(scale_max), x_pad, y_pad)
    n = lib.tdr_parse_cifar10(*args, None, None, C.byref(n_len))
    if n < 0:
        raise ValueError("reference parser raised nn_error")
    img, lab = np.empty((n, n_len.value), np.float32), np.empty(n, np.int64)
    lib.tdr_parse_cifar10(*args, img.ctypes.data_as(f32p), lab.ctypes.data_as(i64p), None)
    return img, lab
