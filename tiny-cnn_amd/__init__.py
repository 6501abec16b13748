"""tiny-cnn_amd — tiny-dnn's training hot path on one MI355X.

This module is the Python face of ``libtdh.so`` (hand-written HIP for gfx950, C ABI in
``include/tdh.h``). It only marshals numpy arrays to device buffers and calls the library;
there is no CPU fallback: importing works without a GPU (so the ABI can be inspected),
but every compute entry point needs the built library and a device, and raises otherwise.

The directory name carries a hyphen, so load it with ``importlib`` (see ``load()`` in
``__graft_entry__.py``) or put this directory's parent on ``sys.path`` and use
``importlib.import_module("tiny-cnn_amd")``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libtdh.so")
CSRC = os.path.join(HERE, "csrc")
HEADER = os.path.join(os.path.dirname(HERE), "include", "tdh.h")

ACT = {"tanh": 0, "relu": 1, "softmax": 2, "sigmoid": 3, "leaky_relu": 4, "elu": 5, "selu": 6,
       "softplus": 7, "softsign": 8, "asinh": 9, "tanh_p1m2": 10}
LOSS = {"mse": 0, "ce_multiclass": 1, "ce": 2}
OPT = {"sgd": 0, "momentum": 1, "adam": 2, "adagrad": 3, "rmsprop": 4, "adamax": 5, "nesterov": 6}
L_CONV, L_FC, L_MAXPOOL, L_AVEPOOL, L_ACT, L_BATCHNORM, L_DROPOUT = range(7)
NET_FUSE_ACT_GRAD, NET_GRAPH, NET_SAMPLE_STEP, NET_NO_INPUT_GRAD = 1, 2, 4, 8

f32p = C.POINTER(C.c_float)


class TdhError(RuntimeError):
    """A libtdh call failed (the reference raises nn_error in the same places)."""


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "in_c", "k_w", "k_h", "out_c", "w_stride", "h_stride",
        "w_dilation", "h_dilation", "pad_same", "has_bias")] + [("tbl", C.c_void_p)]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "in_c", "pool_w", "pool_h", "stride_w", "stride_h", "pad_same",
        "ceil_mode")]


class OptDesc(C.Structure):
    _fields_ = [("kind", C.c_int32)] + [(n, C.c_float) for n in (
        "alpha", "lam", "mu", "b1", "b2", "eps", "b1_t", "b2_t")]


class LayerDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("act", C.c_int32), ("conv", ConvDesc), ("pool", PoolDesc),
                ("fc_in", C.c_int32), ("fc_out", C.c_int32), ("fc_bias", C.c_int32),
                ("act_p", C.c_float * 2), ("bn_channels", C.c_int32), ("bn_spatial", C.c_int32),
                ("bn_eps", C.c_float), ("bn_momentum", C.c_float), ("dropout_rate", C.c_float)]


def build(verbose=False):
    """Compile libtdh.so for gfx950 (hipcc cross-compiles; no GPU needed)."""
    r = subprocess.run(["make", "-C", CSRC, "-j8"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:])
        print(r.stderr[-4000:])
    if r.returncode != 0:
        raise TdhError("building libtdh.so failed")
    return LIB_PATH


_lib = None


def lib():
    """The loaded library. Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TdhError(f"{LIB_PATH} is missing: run build() (make -C tiny-cnn_amd/csrc) first")
        l = C.CDLL(LIB_PATH)
        l.tdh_last_error.restype = C.c_char_p
        l.tdh_version.restype = C.c_char_p
        for n in ("tdh_net_in_size", "tdh_net_out_size", "tdh_net_layer_out_size",
                  "tdh_net_param_size"):
            getattr(l, n).restype = C.c_size_t
        for n in ("tdh_net_param", "tdh_net_layer_out", "tdh_net_layer_dx", "tdh_net_layer_grad",
                  "tdh_net_layer_argmax"):
            getattr(l, n).restype = C.c_void_p
        l.tdh_opt_default.restype = None
        l.tdh_act_default_params.restype = None
        _lib = l
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise TdhError(f"{what}: [{rc}] {lib().tdh_last_error().decode()}")


_inited = False


def init(device=0):
    global _inited
    check(lib().tdh_init(device), "tdh_init")
    _inited = True


def device_info():
    name = C.create_string_buffer(256)
    cus = C.c_int32()
    mem = C.c_size_t()
    check(lib().tdh_device_info(name, 256, C.byref(cus), C.byref(mem)), "tdh_device_info")
    return name.value.decode(), cus.value, mem.value


def sync():
    check(lib().tdh_sync(), "tdh_sync")


class DevBuf:
    """A device allocation with the shape/dtype of the numpy array it mirrors."""

    def __init__(self, shape, dtype=np.float32, zero=False):
        self.shape = tuple(shape) if not np.isscalar(shape) else (int(shape),)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().tdh_malloc(C.byref(p), C.c_size_t(self.nbytes)), "tdh_malloc")
        self.ptr = p
        self.owned = True
        if zero and self.nbytes:
            check(lib().tdh_fill_zero(self.ptr, C.c_size_t(self.nbytes)), "tdh_fill_zero")

    @classmethod
    def view(cls, ptr, shape, dtype=np.float32):
        self = cls.__new__(cls)
        self.shape = tuple(shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self.ptr = C.c_void_p(ptr)
        self.owned = False
        return self

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.shape, self.shape)
        check(lib().tdh_memcpy_h2d(self.ptr, a.ctypes.data_as(C.c_void_p), C.c_size_t(self.nbytes)),
              "tdh_memcpy_h2d")
        return self

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        check(lib().tdh_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self.ptr,
                                   C.c_size_t(self.nbytes)), "tdh_memcpy_d2h")
        return out

    def free(self):
        if getattr(self, "owned", False) and self.ptr:
            lib().tdh_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def copy_d2d(dst, src, nbytes=None, dst_offset=0, src_offset=0):
    """Device-to-device copy on the library's stream (a copy kernel for 4-byte-aligned sizes)."""
    n = src.nbytes if nbytes is None else int(nbytes)
    if n + dst_offset > dst.nbytes or n + src_offset > src.nbytes:
        raise ValueError("copy_d2d: range exceeds a buffer")
    check(lib().tdh_memcpy_d2d(C.c_void_p(dst.ptr.value + dst_offset),
                               C.c_void_p(src.ptr.value + src_offset), C.c_size_t(n)),
          "tdh_memcpy_d2d")


class Feeder:
    """Pipelined upload of host batches (tdh_feeder_*): stage(x, t) hands a batch to the
    feeder's worker thread (pinned copy + upload while earlier steps run; up to two batches
    ahead), acquire() returns device views of the oldest staged batch."""

    def __init__(self, x_len, t_len, max_batch):
        self.x_len, self.t_len, self.max_batch = int(x_len), int(t_len), int(max_batch)
        self.h = C.c_void_p()
        self._staged = []  # host arrays the worker thread may still read
        check(lib().tdh_feeder_create(C.c_size_t(self.x_len), C.c_size_t(self.t_len), self.max_batch,
                                      C.byref(self.h)), "tdh_feeder_create")

    def stage(self, x, t):
        x = np.ascontiguousarray(x, np.float32)
        t = np.ascontiguousarray(t, np.float32)
        batch = x.shape[0]
        assert x.size == batch * self.x_len and t.size == batch * self.t_len
        check(lib().tdh_feeder_stage(self.h, batch, x.ctypes.data_as(C.c_void_p),
                                     t.ctypes.data_as(C.c_void_p)), "tdh_feeder_stage")
        self._staged.append((x, t))  # the worker thread reads them until their acquire() returns

    def acquire(self):
        xp, tp, b = C.c_void_p(), C.c_void_p(), C.c_int()
        check(lib().tdh_feeder_acquire(self.h, C.byref(xp), C.byref(tp), C.byref(b)),
              "tdh_feeder_acquire")
        self._staged.pop(0)
        return (DevBuf.view(xp.value, (b.value, self.x_len)), DevBuf.view(tp.value, (b.value, self.t_len)),
                b.value)

    def close(self):
        if self.h:
            check(lib().tdh_feeder_destroy(self.h), "tdh_feeder_destroy")
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def to_device(a, dtype=np.float32):
    a = np.ascontiguousarray(a, dtype=dtype)
    return DevBuf(a.shape, dtype).upload(a)


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(lib().tdh_event_create(C.byref(p)), "tdh_event_create")
        self.ptr = p

    def record(self):
        check(lib().tdh_event_record(self.ptr), "tdh_event_record")

    def elapsed_ms_since(self, start):
        ms = C.c_float()
        check(lib().tdh_event_elapsed_ms(start.ptr, self.ptr, C.byref(ms)), "tdh_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().tdh_event_destroy(self.ptr)
        except Exception:
            pass


def profile_begin():
    """Start per-kernel timing (every launch gets a pair of events on the library stream)."""
    check(lib().tdh_profile_begin(), "tdh_profile_begin")


def profile_end():
    """Stop per-kernel timing. Returns [dict(tag, launches, total_ms, avg_us, work, unit)]
    sorted by total time; ``work`` is the algorithmic FLOP or bytes of one launch."""
    n = C.c_int32()
    check(lib().tdh_profile_end(C.byref(n)), "tdh_profile_end")
    out = []
    for i in range(n.value):
        tag = C.create_string_buffer(128)
        launches = C.c_int64()
        total = C.c_double()
        work = C.c_double()
        unit = C.c_int32()
        check(lib().tdh_profile_entry(i, tag, 128, C.byref(launches), C.byref(total),
                                      C.byref(work), C.byref(unit)), "tdh_profile_entry")
        out.append({"tag": tag.value.decode(), "launches": launches.value,
                    "total_ms": total.value,
                    "avg_us": 1e3 * total.value / max(1, launches.value),
                    "work": work.value, "unit": "flop" if unit.value == 0 else "byte"})
    return out


def profile_launches():
    """Tags of the kernel launches between the last profile_begin / profile_end, in dispatch order."""
    out, tag, i = [], C.create_string_buffer(160), 0
    while lib().tdh_profile_launch(i, tag, 160) == 0:
        out.append(tag.value.decode())
        i += 1
    return out


def profile_mark(buf):
    """Three launches of the fill kernel on `buf`, booked under the tag "profile_mark"."""
    check(lib().tdh_profile_mark(buf.ptr, C.c_size_t(buf.nbytes)), "tdh_profile_mark")


def fill_zero(buf):
    check(lib().tdh_fill_zero(buf.ptr, C.c_size_t(buf.nbytes)), "tdh_fill_zero")


# ------------------------------------------------------------------ descriptors

def conv_desc(in_w, in_h, in_c, k_w, k_h, out_c, pad_same=False, has_bias=True, w_stride=1,
              h_stride=1, w_dilation=1, h_dilation=1, tbl=None):
    d = ConvDesc(in_w, in_h, in_c, k_w, k_h, out_c, w_stride, h_stride, w_dilation, h_dilation,
                 int(pad_same), int(has_bias), None)
    if tbl is not None:
        keep = np.ascontiguousarray(np.asarray(tbl, dtype=np.uint8).reshape(in_c, out_c))
        d._keep = keep
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
    o = OptDesc()
    lib().tdh_opt_default(C.byref(o), OPT[kind] if isinstance(kind, str) else kind)
    for k, v in kw.items():
        setattr(o, "lam" if k == "lambda_" else k, v)
    return o


def conv_out_shape(d):
    return lib().tdh_conv_out_w(C.byref(d)), lib().tdh_conv_out_h(C.byref(d))


def pool_out_shape(d):
    return lib().tdh_pool_out_w(C.byref(d)), lib().tdh_pool_out_h(C.byref(d))


# ------------------------------------------------- operators on device buffers

def _p(buf):
    return buf.ptr if buf is not None else None


def conv2d_fwd(d, batch, x, w, b, y):
    check(lib().tdh_conv2d_fwd(C.byref(d), batch, _p(x), _p(w), _p(b), _p(y)), "tdh_conv2d_fwd")


def conv2d_bwd(d, batch, x, w, dy, dx, dw, db, accumulate=False):
    check(lib().tdh_conv2d_bwd(C.byref(d), batch, _p(x), _p(w), _p(dy), _p(dx), _p(dw), _p(db),
                               int(accumulate)), "tdh_conv2d_bwd")


def conv2d_bwd_static(d, batch, x, w, dy, dx, dw, db, accumulate=False):
    """tdh_conv2d_bwd with its scratch in the library's static device array (allocates nothing)."""
    check(lib().tdh_conv2d_bwd_static(C.byref(d), batch, _p(x), _p(w), _p(dy), _p(dx), _p(dw), _p(db),
                                      int(accumulate)), "tdh_conv2d_bwd_static")


def fc_fwd(n_in, n_out, has_bias, batch, x, w, b, y):
    check(lib().tdh_fc_fwd(n_in, n_out, int(has_bias), batch, _p(x), _p(w), _p(b), _p(y)),
          "tdh_fc_fwd")


def fc_bwd(n_in, n_out, has_bias, batch, x, w, dy, dx, dw, db, accumulate=False):
    check(lib().tdh_fc_bwd(n_in, n_out, int(has_bias), batch, _p(x), _p(w), _p(dy), _p(dx), _p(dw),
                           _p(db), int(accumulate)), "tdh_fc_bwd")


def maxpool_fwd(d, batch, x, y, argmax):
    check(lib().tdh_maxpool_fwd(C.byref(d), batch, _p(x), _p(y), _p(argmax)), "tdh_maxpool_fwd")


def maxpool_bwd(d, batch, dy, argmax, dx):
    check(lib().tdh_maxpool_bwd(C.byref(d), batch, _p(dy), _p(argmax), _p(dx)), "tdh_maxpool_bwd")


def avepool_fwd(d, batch, x, w, b, y):
    check(lib().tdh_avepool_fwd(C.byref(d), batch, _p(x), _p(w), _p(b), _p(y)), "tdh_avepool_fwd")


def avepool_bwd(d, batch, x, w, dy, dx, dw, db, accumulate=False):
    check(lib().tdh_avepool_bwd(C.byref(d), batch, _p(x), _p(w), _p(dy), _p(dx), _p(dw), _p(db),
                                int(accumulate)), "tdh_avepool_bwd")


def act_params(kind, params=None):
    """The two constructor parameters of an activation layer (the reference's defaults when
    `params` is None): leaky_relu (epsilon,), elu (alpha,), selu (lambda, alpha), softplus
    (beta, threshold)."""
    p = (C.c_float * 2)()
    lib().tdh_act_default_params(ACT[kind], p)
    for i, v in enumerate(params or ()):
        p[i] = v
    return p


def act_fwd(kind, batch, length, x, y, params=None):
    check(lib().tdh_act_fwd_p(ACT[kind], act_params(kind, params), batch, length, _p(x), _p(y)),
          "tdh_act_fwd_p")


def act_bwd(kind, batch, length, y, dy, dx, x=None, params=None):
    check(lib().tdh_act_bwd_p(ACT[kind], act_params(kind, params), batch, length, _p(x), _p(y),
                              _p(dy), _p(dx)), "tdh_act_bwd_p")


def batchnorm_fwd(channels, spatial, batch, x, mean, variance, stddev, y, eps=1e-5, train=True):
    """batch_normalization_layer::forward_propagation; train: mean/variance are written."""
    check(lib().tdh_batchnorm_fwd(channels, spatial, batch, C.c_float(eps), int(bool(train)), _p(x),
                                  _p(mean), _p(variance), _p(stddev), _p(y)), "tdh_batchnorm_fwd")


def batchnorm_bwd(channels, spatial, batch, y, dy, stddev, dx):
    check(lib().tdh_batchnorm_bwd(channels, spatial, batch, _p(y), _p(dy), _p(stddev), _p(dx)),
          "tdh_batchnorm_bwd")


def batchnorm_update_moving(channels, momentum, mean_cur, var_cur, mean, variance):
    check(lib().tdh_batchnorm_update_moving(channels, C.c_float(momentum), _p(mean_cur), _p(var_cur),
                                            _p(mean), _p(variance)), "tdh_batchnorm_update_moving")


def dropout_fwd(batch, length, mask, x, y, rate=0.5, train=True):
    """dropout_layer::forward_propagation; mask: device bytes [batch][length] (see dropout_mask)."""
    scale = np.float32(1) / (np.float32(1) - np.float32(rate))
    check(lib().tdh_dropout_fwd(batch, length, int(bool(train)), C.c_float(scale), _p(mask), _p(x),
                                _p(y)), "tdh_dropout_fwd")


def dropout_bwd(batch, length, mask, dy, dx):
    check(lib().tdh_dropout_bwd(batch, length, _p(mask), _p(dy), _p(dx)), "tdh_dropout_bwd")


class Mt19937:
    """The reference's random generator (tiny_dnn/util/random.h:19-37): one std::mt19937, seed 1
    unless set_random_seed is called. Draws 32-bit words like std::mt19937 does."""

    def __init__(self, seed=1):
        self._rs = np.random.RandomState()
        mt = np.empty(624, dtype=np.uint32)
        mt[0] = seed
        for i in range(1, 624):
            mt[i] = (1812433253 * (int(mt[i - 1]) ^ (int(mt[i - 1]) >> 30)) + i) & 0xFFFFFFFF
        self._rs.set_state(("MT19937", mt, 624))

    def words(self, n):
        return self._rs.randint(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)


def dropout_mask(rng, rate, batch, length):
    """mask[s][i] = bernoulli(rate) (tiny_dnn/util/random.h:67-69, dropout_layer.h:99-102): one draw
    of uniform_real_distribution<float>(0,1) per element, sample after sample; 1 where u <= rate."""
    u = rng.words(batch * length).astype(np.float32) / np.float32(4294967296.0)
    u = np.minimum(u, np.nextafter(np.float32(1), np.float32(0)))
    return (u <= np.float32(rate)).astype(np.uint8).reshape(batch, length)


def loss_grad(kind, batch, length, y, t, dy):
    check(lib().tdh_loss_grad(LOSS[kind], batch, length, _p(y), _p(t), _p(dy)), "tdh_loss_grad")


def softmax_xent_grad(batch, length, y, t, dz):
    check(lib().tdh_softmax_xent_grad(batch, length, _p(y), _p(t), _p(dz)),
          "tdh_softmax_xent_grad")


def opt_update(o, n, merged_grad, w, s0=None, s1=None, grad_scale=1.0):
    check(lib().tdh_opt_update(C.byref(o), C.c_size_t(n), _p(merged_grad), C.c_float(grad_scale),
                               _p(w), _p(s0), _p(s1)), "tdh_opt_update")


# ------------------------------------------------------------ sequential net

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


class Net:
    """network<sequential> with device-resident tensors (tdh_net_*)."""

    def __init__(self, layers, max_batch, flags=0):
        self.layers = list(layers)
        arr = (LayerDesc * len(layers))()
        for i, l in enumerate(layers):
            arr[i] = l
        self._arr = arr
        h = C.c_void_p()
        check(lib().tdh_net_create(arr, len(layers), max_batch, flags, C.byref(h)),
              "tdh_net_create")
        self.h = h
        self.n = len(layers)
        self.max_batch = max_batch

    def close(self):
        if getattr(self, "h", None):
            lib().tdh_net_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def in_size(self):
        return lib().tdh_net_in_size(self.h)

    def out_size(self):
        return lib().tdh_net_out_size(self.h)

    def layer_out_size(self, i):
        return lib().tdh_net_layer_out_size(self.h, i)

    def param_size(self, i, which):
        return lib().tdh_net_param_size(self.h, i, which)

    def params(self):
        """[(layer, which, size)] in update order (weight before bias, front to back)."""
        return [(i, k, self.param_size(i, k)) for i in range(self.n) for k in (0, 1)
                if self.param_size(i, k)]

    def set_param(self, i, which, a):
        a = np.ascontiguousarray(a, dtype=np.float32).ravel()
        assert a.size == self.param_size(i, which)
        check(lib().tdh_net_set_param(self.h, i, which, a.ctypes.data_as(f32p)),
              "tdh_net_set_param")

    def get_param(self, i, which):
        a = np.empty(self.param_size(i, which), np.float32)
        check(lib().tdh_net_get_param(self.h, i, which, a.ctypes.data_as(f32p)),
              "tdh_net_get_param")
        return a

    def out_written(self, i):
        """False when the last pass never wrote layer i's output: in a train step of a fusing
        net a convolution kernel that also writes the activation or computes the max-pool
        behind the convolution keeps the convolution's own output in registers."""
        return bool(lib().tdh_net_layer_out(self.h, i))

    def layer_out(self, i, batch):
        n = self.layer_out_size(i)
        p = lib().tdh_net_layer_out(self.h, i)
        if not p:
            raise RuntimeError(f"layer {i}: the last pass did not write this output to memory")
        return DevBuf.view(p, (batch, n)).numpy()

    def dx_written(self, i):
        """False when the last step never wrote the gradient with respect to layer i's input:
        a fusing net folds an activation gradient into the kernel behind it, and lets a first
        convolution read its output gradient through the max-pool behind it."""
        return bool(lib().tdh_net_layer_dx(self.h, i))

    def layer_dx(self, i, batch):
        n = self.in_size() if i == 0 else self.layer_out_size(i - 1)
        p = lib().tdh_net_layer_dx(self.h, i)
        if not p:
            raise RuntimeError(f"layer {i}: the last step did not write this gradient to memory")
        return DevBuf.view(p, (batch, n)).numpy()

    def layer_grad(self, i, which):
        n = self.param_size(i, which)
        return DevBuf.view(lib().tdh_net_layer_grad(self.h, i, which), (n,)).numpy()

    def layer_argmax(self, i, batch):
        n = self.layer_out_size(i)
        return DevBuf.view(lib().tdh_net_layer_argmax(self.h, i), (batch, n), np.int32).numpy()

    def set_phase(self, train):
        """network::set_netphase: train (default) or test; batch-norm and dropout follow it"""
        check(lib().tdh_net_set_phase(self.h, int(bool(train))), "tdh_net_set_phase")

    def set_dropout_mask(self, i, mask):
        """mask: uint8 [batch][len] drawn by the caller (dropout_mask) for dropout layer i"""
        mask = np.ascontiguousarray(mask, np.uint8)
        check(lib().tdh_net_set_dropout_mask(self.h, i, mask.shape[0], mask.ctypes.data_as(C.c_void_p)),
              "tdh_net_set_dropout_mask")

    def update_weights(self, opt):
        check(lib().tdh_net_update_weights(self.h, C.byref(opt)), "tdh_net_update_weights")

    def clear_grads(self):
        check(lib().tdh_net_clear_grads(self.h), "tdh_net_clear_grads")

    def forward(self, batch, x):
        check(lib().tdh_net_forward(self.h, batch, _p(x)), "tdh_net_forward")

    def train_step(self, opt, loss, batch, x, t, do_update=True):
        check(lib().tdh_net_train_step(self.h, C.byref(opt) if opt is not None else None,
                                       LOSS[loss], batch, _p(x), _p(t), int(do_update)),
              "tdh_net_train_step")

    def train_steps(self, opt, loss, batch, xs, ts):
        """len(xs) consecutive train steps with update, step s on (xs[s], ts[s]); with NET_GRAPH one
        captured graph holds them all (tdh_net_train_steps)."""
        n = len(xs)
        px = (C.c_void_p * n)(*[x.ptr.value for x in xs])
        pt = (C.c_void_p * n)(*[t.ptr.value for t in ts])
        check(lib().tdh_net_train_steps(self.h, C.byref(opt), LOSS[loss], batch, n, px, pt), "tdh_net_train_steps")
