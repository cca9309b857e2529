"""int8 convolution (GEMM over the whole batch) through the C-ABI: bit-exact against the direct 7-loop oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import util
from tests.test_gpu_f32 import conv_desc

pytestmark = pytest.mark.gpu

CASES = [
    # N, C, H, W, Cout, kh, kw, pads, strides, dils, group
    (1, 1, 5, 5, 1, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),
    (2, 3, 9, 7, 5, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1), 1),
    (2, 4, 8, 8, 6, 3, 2, (1, 0, 2, 1), (2, 1), (1, 1), 2),
    (1, 2, 10, 10, 4, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2), 1),
    (3, 32, 6, 6, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1), 2),
    (4, 3, 16, 16, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),
    (2, 64, 12, 12, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),
    (2, 16, 9, 9, 32, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1), 1),
]


def run_conv(rt, X, Wt, bias, scale, case, relu, out, x_layout, y_layout, packed, ws_images=None, column_matrix=False):
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    d = conv_desc(N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group)
    Xd = X if x_layout == R.LAYOUT_NCHW else np.ascontiguousarray(X.transpose(0, 2, 3, 1))
    dX, dW = util.to_dev(Xd), util.to_dev(Wt)
    db = None if bias is None else util.to_dev(bias)
    ds = None if scale is None else util.to_dev(scale)
    odt = {0: np.int32, 1: np.float32, 2: np.int8}[out]
    yshape = (N, Cout, d.OH, d.OW) if y_layout == R.LAYOUT_NCHW else (N, d.OH, d.OW, Cout)
    dY = util.dev_empty(yshape, odt)
    a = R.ConvI8Args()
    a.X, a.W, a.bias, a.scale, a.Y = util.ptr(dX), util.ptr(dW), util.ptr(db), util.ptr(ds), util.ptr(dY)
    a.relu, a.out, a.x_layout, a.y_layout = relu, out, x_layout, y_layout
    keep = []
    if packed:
        nb = rt.lib.sofie_hip_conv_weight_i8_packed_bytes(C.byref(d))
        dWp = util.dev_empty((nb,), np.int8)
        rt.call("sofie_hip_pack_conv_weight_i8", C.byref(d), util.ptr(dWp), util.ptr(dW))
        a.W, a.w_is_packed = util.ptr(dWp), 1
        keep.append(dWp)
    need = rt.lib.sofie_hip_conv_i8_workspace(C.byref(d), C.byref(a))
    if ws_images:
        need = need * ws_images
    if column_matrix:  # room for what the "conv_explicit" option needs on top of the minimum
        need += rt.lib.sofie_hip_conv_i8_column_matrix_bytes(C.byref(d)) * (ws_images or 1)
    ws = util.dev_empty((need + 256,), np.int8)
    a.workspace, a.workspace_bytes = util.ptr(ws), need
    import torch
    torch.cuda.synchronize()
    print("conv_i8", case, relu, out, x_layout, y_layout, packed, flush=True)
    rt.call("sofie_hip_conv_i8", C.byref(d), C.byref(a))
    rt.sync()
    y = util.to_host(dY)
    return y if y_layout == R.LAYOUT_NCHW else np.ascontiguousarray(y.transpose(0, 3, 1, 2))


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("x_layout,y_layout,packed", [(0, 0, 0), (1, 1, 1), (0, 1, 0), (1, 0, 1)])
@pytest.mark.parametrize("column_matrix", [0, 1])
def test_conv_i8_requant_bit_exact(rt, case, x_layout, y_layout, packed, column_matrix, opt):
    # column_matrix = 1 forces the explicit int8 im2col + GEMM; 0 lets the runtime choose: reductions of at most 64 bytes
    # (the first six cases) are gathered inside the GEMM kernel, 64-channel NHWC input takes the implicit GEMM
    if column_matrix:
        opt("conv_explicit", 1)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.int8_sym(50, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(51, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(52, Cout, -2000, 2000)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(53, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    got = run_conv(rt, X, Wt, bias, scale, case, 1, R.I8OUT_I8, x_layout, y_layout, packed, ws_images=2, column_matrix=bool(column_matrix))
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=1, out=2, omp=True)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("out,relu", [(R.I8OUT_I32, 0), (R.I8OUT_I32, 1), (R.I8OUT_F32, 0), (R.I8OUT_F32, 1), (R.I8OUT_I8, 0)])
def test_conv_i8_output_kinds(rt, out, relu):
    case = (3, 8, 7, 9, 12, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.int8_sym(60, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(61, Cout * Cc * kh * kw).reshape(Cout, Cc, kh, kw)
    scale = ((0.5 + util.uniform01(63, Cout)) / np.float32(127.0 * 8.5)).astype(np.float32)
    got = run_conv(rt, X, Wt, None, scale, case, relu, out, 0, 0, 0)
    want = ob.conv_i8(X, Wt, None, scale, pads=pads, strides=strides, dils=dils, group=group, relu=relu, out=out)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("N,Cc,H,W", [(3, 20, 5, 7), (3, 48, 5, 7), (2, 272, 4, 4), (4, 256, 9, 9), (1, 80, 33, 3)])
def test_global_avg_pool_i8_both_layouts(rt, N, Cc, H, W):
    X = util.int8_sym(70, N * Cc * H * W).reshape(N, Cc, H, W)
    want = ob.global_avg_pool_i8(X, np.float32(0.031))
    for layout in (0, 1):
        Xd = X if layout == 0 else np.ascontiguousarray(X.transpose(0, 2, 3, 1))
        dX = util.to_dev(Xd)
        dY = util.dev_empty((N, Cc), np.float32)
        rt.call("sofie_hip_global_avg_pool_i8", util.ptr(dY), util.ptr(dX), N, Cc, H * W, layout, C.c_float(0.031))
        rt.sync()
        assert np.array_equal(util.to_host(dY).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("tile", [256, 257, 258, 128, 64])
@pytest.mark.parametrize("case", [
    (2, 128, 12, 12, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),      # paired-slab kernels (channels % 128 == 0)
    (3, 64, 11, 9, 96, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),         # 64-byte slabs, ragged Cout
    (2, 128, 10, 10, 64, 3, 2, (2, 0, 1, 1), (2, 1), (1, 2), 2),       # groups, stride, dilation, asymmetric pads
    (1, 64, 7, 7, 32, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1), 1),          # 1x1
])
def test_conv_i8_implicit_gemm_every_tile(rt, case, tile, opt):
    """NHWC input with a power-of-two channel count >= 64 takes the implicit-GEMM kernels (no column matrix)."""
    opt("i8_tile", tile)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.int8_sym(80, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(81, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(82, Cout, -2000, 2000)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(83, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=1, out=2, omp=True)
    got = run_conv(rt, X, Wt, bias, scale, case, 1, R.I8OUT_I8, R.LAYOUT_NHWC, R.LAYOUT_NHWC, 1)
    assert np.array_equal(got, want)
    # and the explicit column-matrix path gives the same bits
    opt("conv_explicit", 1)
    opt("i8_tile", 0)
    got2 = run_conv(rt, X, Wt, bias, scale, case, 1, R.I8OUT_I8, R.LAYOUT_NHWC, R.LAYOUT_NCHW, 1, column_matrix=True)
    assert np.array_equal(got2, want)


@pytest.mark.parametrize("case", [
    (4, 128, 16, 16, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),       # 4 tiles, K = 1152
    (2, 256, 16, 32, 512, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),       # 8 tiles in two columns, K = 2304
    (2, 256, 15, 17, 512, 3, 2, (2, 0, 1, 1), (2, 1), (1, 2), 2),       # groups, stride, dilation, asymmetric pads: one tile per group
    (257, 128, 16, 16, 256, 1, 3, (0, 1, 0, 1), (1, 1), (1, 1), 1),     # 257 tiles: more than one per workgroup
])
@pytest.mark.parametrize("forced", [False, True])
def test_conv_i8_persistent_kernel(rt, case, forced, opt):
    """Convolutions whose GEMM divides into whole 256 x 256 tiles (rows = batch x output pixels, columns = output channels per
    group) take the persistent kernel: the rows of A are gathered from the NHWC activations tap by tap, taps outside the image
    read zeros, and the loads run on into the workgroup's next tile."""
    if forced:
        opt("i8_tile", 512)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.int8_sym(84, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(85, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(86, Cout, -2000, 2000)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(87, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    print("conv_i8 persistent", case, forced, flush=True)
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=1, out=2, omp=True)
    got = run_conv(rt, X, Wt, bias, scale, case, 1, R.I8OUT_I8, R.LAYOUT_NHWC, R.LAYOUT_NHWC, 1)
    assert np.array_equal(got, want)
    assert (want != 0).mean() > 0.2 and np.abs(want).max() > 60  # neither all zero nor saturated


@pytest.mark.parametrize("case", [
    (3, 64, 16, 16, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),        # 16 x 16: 18 x 18 patches, one tile per image
    (2, 64, 32, 32, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),        # 32 x 32: tiles of 8 rows, 4 per image
    (5, 64, 64, 64, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),        # the benchmark's second layer: 80 tiles
    (2, 64, 34, 66, 128, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1), 1),        # no padding: 32 x 64 outputs from 34 x 66 inputs
    (2, 64, 17, 31, 128, 3, 3, (0, 2, 1, 1), (1, 1), (1, 1), 1),        # unequal pads: 16 x 32 outputs
    (2, 128, 16, 32, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 2),       # two groups of 64 -> 128 channels
    (70, 64, 32, 32, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),       # 280 tiles: more than one per workgroup
])
@pytest.mark.parametrize("out,relu", [(R.I8OUT_I8, 1), (R.I8OUT_I8, 0), (R.I8OUT_I32, 1), (R.I8OUT_F32, 0)])
def test_conv_i8_small_layer_with_resident_weights(rt, case, out, relu, opt):
    """3 x 3, stride 1, 64 input and 128 output channels per group: the kernel that keeps the weights in LDS and loads each
    tile's pixels once with their halo (asked for by force: tile 576; by the heuristic's own choice when there are at least 256
    tiles).  Bit-exact against the oracle, edges (zeros outside the image) and image boundaries between tiles included."""
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    if N * 0 == 0 and (out != R.I8OUT_I8 or relu == 0) and N > 5:
        pytest.skip("the long case runs with the benchmark's store only")
    opt("i8_tile", 576)
    X = util.int8_sym(184, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(185, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(186, Cout, -2000, 2000)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(187, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=relu, out=out, omp=True)
    got = run_conv(rt, X, Wt, bias, scale, case, relu, out, R.LAYOUT_NHWC, R.LAYOUT_NHWC, 1)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    if out == R.I8OUT_I8:
        assert (want != 0).mean() > 0.2 and np.abs(want).max() > 60


@pytest.mark.parametrize("case", [
    (4, 3, 16, 16, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),      # RGB 3 x 3: the benchmark's first layer in small
    (2, 3, 64, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),      # the benchmark's image size: a group of 64 pixels is one row
    (4, 1, 16, 16, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),      # one channel; rows of 16: the last load of a row starts at byte 8 for five pixels
    (8, 4, 11, 20, 64, 4, 4, (0, 0, 0, 0), (1, 1), (1, 1), 1),      # 4 x 4 over 4 channels: all 16 pairs, no padding, 8 x 17 outputs
    (16, 3, 20, 16, 64, 5, 3, (2, 3, 2, 0), (1, 1), (1, 1), 1),     # 5 rows of taps, three columns of padding on the left, none on the right: 20 x 17 outputs
    (8, 2, 17, 16, 64, 3, 2, (1, 0, 1, 1), (2, 1), (2, 1), 1),      # stride 2 and dilation 2 in y, two columns of taps
    (4, 6, 16, 16, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 2),     # two groups of 3 -> 64 channels
    (70, 3, 32, 32, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),     # 1120 groups of pixels: more than one per wave
])
@pytest.mark.parametrize("out,relu", [(R.I8OUT_I8, 1), (R.I8OUT_I8, 0), (R.I8OUT_I32, 1), (R.I8OUT_F32, 0)])
def test_conv_i8_few_input_channels_read_as_windows(rt, case, out, relu, opt):
    """NCHW input with few channels, 64 output channels, stride and dilation 1 in x: the kernel that reads each (channel, row of
    taps) as one four-byte window cut from an aligned load (asked for by force: tile 27; it is also the heuristic's choice).
    Bit-exact against the oracle: zeros left, right, above and below the image, images and rows that change inside a group of
    64 pixels."""
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    if N > 16 and (out != R.I8OUT_I8 or relu == 0):
        pytest.skip("the long cases run with the benchmark's store only")
    opt("i8_tile", 27)
    X = util.int8_sym(194, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(195, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(196, Cout, -500, 500)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(197, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=relu, out=out, omp=True)
    got = run_conv(rt, X, Wt, bias, scale, case, relu, out, R.LAYOUT_NCHW, R.LAYOUT_NHWC, 1)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    if out == R.I8OUT_I8:
        assert (want != 0).mean() > 0.2 and np.abs(want).max() > 60


def test_first_layer_of_an_image_network_needs_no_workspace(rt):
    """3 input channels, 3x3: K = 27 fits one slab, the rows are gathered in the kernel (NCHW in, NHWC out, a ragged last tile)."""
    case = (3, 3, 21, 19, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    d = conv_desc(N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group)
    a = R.ConvI8Args()
    a.x_layout, a.y_layout, a.w_is_packed = R.LAYOUT_NCHW, R.LAYOUT_NHWC, 1
    assert rt.lib.sofie_hip_conv_i8_workspace(C.byref(d), C.byref(a)) == 0
    X = util.int8_sym(90, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(91, Cout * Cc * 9).reshape(Cout, Cc, 3, 3)
    bias = util.int32_range(92, Cout, -500, 500)
    scale = ((0.5 + util.uniform01(93, Cout)) / np.float32(127.0 * np.sqrt(27))).astype(np.float32)
    want = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=1, out=2, omp=True)
    got = run_conv(rt, X, Wt, bias, scale, case, 1, R.I8OUT_I8, R.LAYOUT_NCHW, R.LAYOUT_NHWC, 1, ws_images=0)
    assert np.array_equal(got, want) and (want > 0).any()


def run_conv_plane_sums(rt, X, Wt, bias, scale, case, relu, x_layout):
    """sofie_hip_conv_i8 with SOFIE_I8OUT_I8_PLANE_SUMS into a cleared int32 [N, Cout], then the average."""
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    d = conv_desc(N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group)
    Xd = X if x_layout == R.LAYOUT_NCHW else np.ascontiguousarray(X.transpose(0, 2, 3, 1))
    dX, dW, db, ds = util.to_dev(Xd), util.to_dev(Wt), util.to_dev(bias), util.to_dev(scale)
    dS = util.to_dev(np.full((N, Cout), 123456, np.int32))     # stale contents: the caller's clear is part of the contract
    dY = util.dev_empty((N, Cout), np.float32)
    nb = rt.lib.sofie_hip_conv_weight_i8_packed_bytes(C.byref(d))
    dWp = util.dev_empty((nb,), np.int8)
    rt.call("sofie_hip_pack_conv_weight_i8", C.byref(d), util.ptr(dWp), util.ptr(dW))
    a = R.ConvI8Args()
    a.X, a.W, a.bias, a.scale, a.Y = util.ptr(dX), util.ptr(dWp), util.ptr(db), util.ptr(ds), util.ptr(dS)
    a.relu, a.out, a.x_layout, a.y_layout, a.w_is_packed = relu, R.I8OUT_I8_PLANE_SUMS, x_layout, x_layout, 1
    assert rt.lib.sofie_hip_conv_i8_workspace(C.byref(d), C.byref(a)) == 0
    import torch
    torch.cuda.synchronize()
    print("conv_i8 plane sums", case, relu, x_layout, flush=True)
    rt.call("sofie_hip_fill_zero", util.ptr(dS), C.c_size_t(N * Cout * 4))
    rt.call("sofie_hip_conv_i8", C.byref(d), C.byref(a))
    rt.call("sofie_hip_plane_sums_to_average", util.ptr(dY), util.ptr(dS), N * Cout, d.OH * d.OW, C.c_float(0.037))
    rt.sync()
    return util.to_host(dS), util.to_host(dY)


PLANE_SUM_CASES = [
    # implicit GEMM (NHWC, 64 or 128 channels per group), planes of 256 and 1024 pixels
    ((3, 64, 16, 16, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1), R.LAYOUT_NHWC),
    ((2, 128, 32, 32, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1), R.LAYOUT_NHWC),
    ((2, 128, 32, 32, 96, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1), 2), R.LAYOUT_NHWC),     # grouped, 48 columns per group
    ((5, 64, 33, 33, 64, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1), 1), R.LAYOUT_NHWC),      # stride 2: 17 x 17 = 289 -> refused below
    # rows gathered in the kernel (3 channels), either input layout
    ((4, 3, 16, 32, 40, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1), R.LAYOUT_NCHW),
    ((4, 3, 16, 32, 40, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1), R.LAYOUT_NHWC),
]


@pytest.mark.parametrize("case,x_layout", PLANE_SUM_CASES)
@pytest.mark.parametrize("relu", [0, 1])
@pytest.mark.parametrize("tile", [0, 64, 128, 256, 258, 512])
def test_conv_i8_plane_sums_equal_the_sums_of_the_stored_map(rt, case, x_layout, relu, tile, opt):
    """The int8 feature map is never stored: the sums the kernel adds up in its store must be the sums of the map the
    oracle computes, and the average the bits of the oracle's DequantizeLinear + GlobalAveragePool on that map."""
    if tile:
        opt("i8_tile", tile)
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.int8_sym(70, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(71, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    bias = util.int32_range(72, Cout, -2000, 2000)
    K = (Cc // group) * kh * kw
    scale = ((0.5 + util.uniform01(73, Cout)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    OH = (H + pads[0] + pads[2] - dils[0] * (kh - 1) - 1) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - dils[1] * (kw - 1) - 1) // strides[1] + 1
    if (OH * OW) % 256:
        with pytest.raises(R.SofieHipError, match="multiple of 256"):
            run_conv_plane_sums(rt, X, Wt, bias, scale, case, relu, x_layout)
        return
    sums, avg = run_conv_plane_sums(rt, X, Wt, bias, scale, case, relu, x_layout)
    fmap = ob.conv_i8(X, Wt, bias, scale, pads=pads, strides=strides, dils=dils, group=group, relu=relu, out=2, omp=True)
    want_sums = fmap.astype(np.int64).sum(axis=(2, 3))
    assert np.array_equal(sums, want_sums.astype(np.int32))
    assert np.abs(want_sums).max() > 100          # the case does exercise the sums
    want_avg = ob.global_avg_pool_i8(fmap, 0.037)
    assert np.array_equal(avg.view(np.uint32), want_avg.view(np.uint32))


def test_plane_sums_take_average_gives_the_same_average_and_clears_the_sums(rt):
    """sofie_hip_plane_sums_take_average: the bits of sofie_hip_plane_sums_to_average, and the sums are zero afterwards, so that a
    convolution can add the next inference's planes up in the same buffer without a clearing launch (twice in a row here)."""
    nc, hw = 5 * 77, 1024
    sums = util.int32_range(311, nc, -120000, 130000)
    d1, d2 = util.to_dev(sums), util.to_dev(sums)
    y1, y2 = util.dev_empty((nc,), np.float32), util.dev_empty((nc,), np.float32)
    rt.call("sofie_hip_plane_sums_to_average", util.ptr(y1), util.ptr(d1), nc, hw, C.c_float(0.037))
    for again in range(2):
        if again:
            d2.copy_(util.to_dev(sums))
        rt.call("sofie_hip_plane_sums_take_average", util.ptr(y2), util.ptr(d2), nc, hw, C.c_float(0.037))
        rt.sync()
        assert np.array_equal(util.to_host(y1).view(np.uint32), util.to_host(y2).view(np.uint32))
        assert not util.to_host(d2).any() and np.array_equal(util.to_host(d1), sums)
    want = (sums.astype(np.float32) * np.float32(0.037)) / np.float32(hw)
    assert np.array_equal(util.to_host(y2).view(np.uint32), want.view(np.uint32))


def test_conv_i8_plane_sums_refuse_a_column_matrix_shape(rt):
    case = (2, 16, 16, 16, 32, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1)     # 144-byte reduction over NCHW input: needs a column matrix
    N, Cc, H, W, Cout, kh, kw, *_ = case
    X = util.int8_sym(74, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(75, Cout * Cc * kh * kw).reshape(Cout, Cc, kh, kw)
    with pytest.raises((R.SofieHipError, AssertionError)):
        run_conv_plane_sums(rt, X, Wt, np.zeros(Cout, np.int32), np.ones(Cout, np.float32), case, 0, R.LAYOUT_NCHW)
