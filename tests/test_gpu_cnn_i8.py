"""The int8 CNN chain (quantise, conv stages with folded BatchNorm + Relu, global average pool, Gemm) through the
C-ABI against the CPU chain: the int8 feature maps bit-exact, the fp32 tail to 1e-5."""
import ctypes as C

import numpy as np
import pytest

from sofie_amd.session import Int8CNNSession
from tests.refmodels import make_int8_cnn, int8_cnn_oracle

pytestmark = pytest.mark.gpu


def session(rt, m, pool_in_conv=True):
    return Int8CNNSession(rt, m["batch"], m["in_shape"], m["in_scale"], m["convs"], m["last_scale"], m["fc_w"], m["fc_b"], pool_in_conv)


# pooled: whether the last convolution can add its planes up in its store (planes of a multiple of 256 pixels)
@pytest.mark.parametrize("batch,hw,channels,pooled", [(3, 8, (3, 16, 32), False), (2, 12, (3, 64, 128, 256, 256), False), (5, 16, (3, 64, 128), True),
                                                      (2, 32, (3, 64, 128, 256), True), (3, 16, (3, 24), True)])
@pytest.mark.parametrize("pool_in_conv", [False, True])
def test_cnn_chain_matches_cpu_chain(rt, batch, hw, channels, pooled, pool_in_conv):
    from sofie_amd import Runtime
    m = make_int8_cnn(batch, hw, channels)
    print("cnn_i8", batch, hw, channels, pool_in_conv, flush=True)
    rt = Runtime(0)   # a Session owns its context's arena: one context per Session
    try:
        _check(rt, m, batch, pool_in_conv, pooled)
    finally:
        rt.close()


def _check(rt, m, batch, pool_in_conv, pooled):
    s = session(rt, m, pool_in_conv)
    assert s.pool_in_conv == (pool_in_conv and pooled)
    got = s.infer(m["x"])
    want = int8_cnn_oracle(m, m["x"])
    # the last feature map, int8 NHWC on the device, bit-exact
    from oracle import binding as ob
    h = ob.quantize_linear(m["x"], m["in_scale"])
    for cv in m["convs"]:
        h = ob.conv_i8(h, cv["W"], cv["bias"], cv["scale"], pads=cv["pads"], strides=cv["strides"], dils=cv["dils"], relu=1, out=2, omp=True)
    c, oh, ow = s.out_shape
    if s.pool_in_conv:
        # the last map is never stored: its plane sums are what the device holds
        sums = np.empty((batch, c), dtype=np.int32)
        rt.call("sofie_hip_download", sums.ctypes.data_as(C.c_void_p), s.p(s.off_sums), C.c_size_t(sums.nbytes))
        rt.sync()
        assert np.array_equal(sums, h.astype(np.int64).sum(axis=(2, 3)).astype(np.int32))
    else:
        fm = np.empty((batch, oh, ow, c), dtype=np.int8)
        rt.call("sofie_hip_download", fm.ctypes.data_as(C.c_void_p), s.p(s.off_last), C.c_size_t(fm.nbytes))
        rt.sync()
        assert np.array_equal(fm.transpose(0, 3, 1, 2), h)
    assert h.any() and (h > 0).mean() > 0.05          # the maps are not degenerate
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    # a second inference on the same session reuses every buffer and gives the same bits
    assert np.array_equal(s.infer(m["x"]).view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("pool_in_conv", [False, True])
def test_full_size_batch_256_on_sampled_images(pool_in_conv):
    """benchmark configuration 5 at its real size (batch 256, 64 x 64 images, 3 -> 64 -> 128 -> 256 -> 256): the kernels the
    heuristics pick for a million GEMM rows.  The images of a batch are independent, so the CPU chain runs on a sample of
    them: the last int8 feature map (or its plane sums, when the last convolution adds them up in its store) bit-exact, the
    fp32 outputs to 1e-5."""
    from oracle import binding as ob
    from sofie_amd import Runtime
    batch = 256
    m = make_int8_cnn(batch, 64)
    sample = [0, 1, 127, 255]
    rt = Runtime(0)
    try:
        s = session(rt, m, pool_in_conv)
        assert s.pool_in_conv == pool_in_conv
        print("cnn_i8 full size, pool_in_conv =", pool_in_conv, flush=True)
        got = s.infer(m["x"])
        xs = np.ascontiguousarray(m["x"][sample])
        want = int8_cnn_oracle(m, xs)
        h = ob.quantize_linear(xs, m["in_scale"])
        for cv in m["convs"]:
            h = ob.conv_i8(h, cv["W"], cv["bias"], cv["scale"], pads=cv["pads"], strides=cv["strides"], dils=cv["dils"], relu=1, out=2, omp=True)
        c, oh, ow = s.out_shape
        if s.pool_in_conv:
            sums = np.empty((batch, c), dtype=np.int32)
            rt.call("sofie_hip_download", sums.ctypes.data_as(C.c_void_p), s.p(s.off_sums), C.c_size_t(sums.nbytes))
            rt.sync()
            assert np.array_equal(sums[sample], h.astype(np.int64).sum(axis=(2, 3)).astype(np.int32))
        else:
            for k, img in enumerate(sample):
                fm = np.empty((oh, ow, c), dtype=np.int8)
                rt.call("sofie_hip_download", fm.ctypes.data_as(C.c_void_p), s.p(s.off_last + img * fm.nbytes), C.c_size_t(fm.nbytes))
                rt.sync()
                assert np.array_equal(fm.transpose(2, 0, 1), h[k]), "image %d" % img
        assert (h > 0).mean() > 0.05
        assert np.abs(got[sample] - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
        assert np.isfinite(got).all() and got.std() > 1e-3
    finally:
        rt.close()
