"""tdh_conv2d_bwd_static: the convolution backward pass with its scratch in the library's static
device array, for callers that cannot allocate. Through the C ABI against tdh_conv2d_bwd (same
kernels, so the results must be bit for bit the same) and against the oracle, on calls in a row
that share the array: a larger shape first, then smaller ones whose scratch lies inside what the
first call left behind."""
import numpy as np
import pytest

from conftest import assert_close

pytestmark = pytest.mark.gpu


def run_both(T, O, cfg, seed, check_oracle):
    iw, ih, ic, k, oc, same, bs = cfg
    d, do = T.conv_desc(iw, ih, ic, k, k, oc, pad_same=same), O.conv_desc(iw, ih, ic, k, k, oc, pad_same=same)
    ow, oh = T.conv_out_shape(d)
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((bs, ic * ih * iw)).astype(np.float32)
    w = rng.uniform(-0.3, 0.3, oc * ic * k * k).astype(np.float32)
    dy = rng.standard_normal((bs, oc * oh * ow)).astype(np.float32)
    xd, wd, dyd = T.to_device(x), T.to_device(w), T.to_device(dy)
    got = [T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,))]
    want = [T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,))]
    T.conv2d_bwd_static(d, bs, xd, wd, dyd, *got)
    T.conv2d_bwd(d, bs, xd, wd, dyd, *want)
    for g, r, name in zip(got, want, ("dX", "dW", "db")):
        assert np.array_equal(g.numpy(), r.numpy()), f"{cfg}: {name} differs from tdh_conv2d_bwd"
    if check_oracle:
        for g, r, name in zip(got, O.conv2d_bwd(do, x, w, dy), ("dX", "dW", "db")):
            assert_close(g.numpy().ravel(), r.ravel(), what=f"{cfg}: {name} against the oracle")
    # accumulate = 1 adds to what is there, as the existing entry point does
    T.conv2d_bwd_static(d, bs, xd, wd, dyd, None, got[1], got[2], accumulate=True)
    T.conv2d_bwd(d, bs, xd, wd, dyd, None, want[1], want[2], accumulate=True)
    assert np.array_equal(got[1].numpy(), want[1].numpy()) and np.array_equal(got[2].numpy(), want[2].numpy())


def test_static_scratch_calls_in_a_row_match_the_allocating_entry_point(T, O):
    # (in_w, in_h, in_c, k, out_c, pad_same, batch); every one splits a reduction through scratch
    run_both(T, O, (16, 16, 32, 5, 32, True, 128), 1, False)   # CIFAR conv2: 5x5 dW slices + db partials
    run_both(T, O, (8, 8, 32, 5, 64, True, 16), 2, True)       # smaller: inside the first call's leftovers
    run_both(T, O, (12, 10, 3, 3, 8, False, 5), 3, True)       # first-layer kernels, tiny
    run_both(T, O, (64, 64, 32, 3, 64, True, 8), 4, False)     # 3x3 halo kernels, larger again
    run_both(T, O, (9, 7, 2, 3, 5, True, 3), 5, True)          # generic GEMM path, ragged


def device_free_bytes():
    """hipMemGetInfo of the current device, straight from the HIP runtime the library is linked to."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_scratch_calls_leave_device_memory_as_it_was(T):
    """Nothing is allocated or freed by the call: the free memory of the device is the same before
    and after, also for a first call of a shape (no scratch of the allocating kind has ever been
    grown for it in this test) and for a smaller one behind it."""
    shapes = [(16, 16, 32, 5, 48, True, 96), (8, 8, 16, 3, 24, True, 7)]
    held = []
    for (iw, ih, ic, k, oc, same, bs) in shapes:
        d = T.conv_desc(iw, ih, ic, k, k, oc, pad_same=same)
        ow, oh = T.conv_out_shape(d)
        rng = np.random.default_rng(bs)
        x = T.to_device(rng.standard_normal((bs, ic * ih * iw)).astype(np.float32))
        w = T.to_device(rng.uniform(-0.3, 0.3, oc * ic * k * k).astype(np.float32))
        dy = T.to_device(rng.standard_normal((bs, oc * oh * ow)).astype(np.float32))
        held.append((d, bs, x, w, dy, T.DevBuf((bs, ic * ih * iw)), T.DevBuf((oc * ic * k * k,)), T.DevBuf((oc,))))
    T.sync()
    before = device_free_bytes()
    for _ in range(2):
        for (d, bs, x, w, dy, dx, dw, db) in held:
            T.conv2d_bwd_static(d, bs, x, w, dy, dx, dw, db)
    T.sync()
    assert device_free_bytes() == before, "tdh_conv2d_bwd_static changed the device's free memory"
    for (d, bs, x, w, dy, dx, dw, db) in held:   # and the results are those of the allocating call
        want = [T.DevBuf(dx.shape), T.DevBuf(dw.shape), T.DevBuf(db.shape)]
        T.conv2d_bwd(d, bs, x, w, dy, *want)
        for g, r in zip((dx, dw, db), want):
            assert np.array_equal(g.numpy(), r.numpy())


def test_static_scratch_refuses_a_connection_table(T):
    # the table would be staged through a host copy that the call has to wait for
    tbl = np.ones((4, 6), np.uint8)
    tbl[1, 2] = 0
    d = T.conv_desc(8, 8, 4, 3, 3, 6, pad_same=True, tbl=tbl)
    x, dy = T.DevBuf((2, 4 * 64), zero=True), T.DevBuf((2, 6 * 64), zero=True)
    w = T.DevBuf((6 * 4 * 9,), zero=True)
    dx, dw, db = T.DevBuf((2, 4 * 64)), T.DevBuf((6 * 4 * 9,)), T.DevBuf((6,))
    with pytest.raises(T.TdhError, match="connection table"):
        T.conv2d_bwd_static(d, 2, x, w, dy, dx, dw, db)
    T.conv2d_bwd(d, 2, x, w, dy, dx, dw, db)       # the allocating entry point serves it


def test_static_scratch_refuses_what_does_not_fit(T):
    # 768 -> 768 channels, 3x3 on 8x8 images, batch 32: 21 MB of filters whose gradient is summed
    # from several partial slices, about 120 MiB of scratch. The tensors have their real sizes,
    # so the call would be harmless if it were accepted.
    iw = ih = 8
    ic = oc = 768
    bs = 32
    d = T.conv_desc(iw, ih, ic, 3, 3, oc, pad_same=True)
    x, dy = T.DevBuf((bs, ic * ih * iw), zero=True), T.DevBuf((bs, oc * ih * iw), zero=True)
    w = T.DevBuf((oc * ic * 9,), zero=True)
    dx, dw, db = T.DevBuf((bs, ic * ih * iw)), T.DevBuf((oc * ic * 9,)), T.DevBuf((oc,))
    with pytest.raises(T.TdhError, match=r"needs \d+ bytes of scratch, the static buffer holds 67108864"):
        T.conv2d_bwd_static(d, bs, x, w, dy, dx, dw, db)
    T.conv2d_bwd(d, bs, x, w, dy, dx, dw, db)      # the allocating entry point takes it
    assert not dw.numpy().any()
    # and the static entry point still works afterwards
    d2 = T.conv_desc(8, 8, 4, 3, 3, 4, pad_same=True)
    one = np.ones((2, 256), np.float32)
    dx2, dw2, db2 = T.DevBuf((2, 256)), T.DevBuf((144,)), T.DevBuf((4,))
    T.conv2d_bwd_static(d2, 2, T.to_device(one), T.to_device(np.zeros(144, np.float32)), T.to_device(one), dx2, dw2, db2)
    assert np.array_equal(db2.numpy(), np.full(4, 128.0, np.float32))
