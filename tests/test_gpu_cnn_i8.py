"""The int8 CNN chain (quantise, conv stages with folded BatchNorm + Relu, global average pool, Gemm) through the
C-ABI against the CPU chain: the int8 feature maps bit-exact, the fp32 tail to 1e-5."""
import ctypes as C

import numpy as np
import pytest

from sofie_amd.session import Int8CNNSession
from tests.refmodels import make_int8_cnn, int8_cnn_oracle

pytestmark = pytest.mark.gpu


def session(rt, m):
    return Int8CNNSession(rt, m["batch"], m["in_shape"], m["in_scale"], m["convs"], m["last_scale"], m["fc_w"], m["fc_b"])


@pytest.mark.parametrize("batch,hw,channels", [(3, 8, (3, 16, 32)), (2, 12, (3, 64, 128, 256, 256)), (5, 16, (3, 64, 128))])
def test_cnn_chain_matches_cpu_chain(rt, batch, hw, channels):
    from sofie_amd import Runtime
    m = make_int8_cnn(batch, hw, channels)
    print("cnn_i8", batch, hw, channels, flush=True)
    rt = Runtime(0)   # a Session owns its context's arena: one context per Session
    try:
        _check(rt, m, batch)
    finally:
        rt.close()


def _check(rt, m, batch):
    s = session(rt, m)
    got = s.infer(m["x"])
    want = int8_cnn_oracle(m, m["x"])
    # the last feature map, int8 NHWC on the device, bit-exact
    from oracle import binding as ob
    h = ob.quantize_linear(m["x"], m["in_scale"])
    for cv in m["convs"]:
        h = ob.conv_i8(h, cv["W"], cv["bias"], cv["scale"], pads=cv["pads"], strides=cv["strides"], dils=cv["dils"], relu=1, out=2, omp=True)
    c, oh, ow = s.out_shape
    fm = np.empty((batch, oh, ow, c), dtype=np.int8)
    rt.call("sofie_hip_download", fm.ctypes.data_as(C.c_void_p), s.p(s.off_last), C.c_size_t(fm.nbytes))
    rt.sync()
    assert np.array_equal(fm.transpose(0, 3, 1, 2), h)
    assert h.any() and (h > 0).mean() > 0.05          # the maps are not degenerate
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    # a second inference on the same session reuses every buffer and gives the same bits
    assert np.array_equal(s.infer(m["x"]).view(np.uint32), got.view(np.uint32))
