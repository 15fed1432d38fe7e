"""conv2d on the device against the CPU checker.

Bars: bit-exact for integers; fp32/fp64 within 1e-5 relative plus K*eps*max|x||w|
for summation order; fp16/bf16 (fp32 accumulation on both sides) rel 2e-3 / abs 1e-3.
"""
import ctypes as C

import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import abi, ops

pytestmark = pytest.mark.gpu
SEED = 17
CONV_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] == "conv2d"]

# x shape, w shape, stride, padding: scaled-down relatives of the ResNet-50 layers plus odd cases
CASES = {
    "stem_k7_s2_p3": ((2, 3, 40, 40), (16, 3, 7, 7), (2, 2), (3, 3)),
    "body_k3_s1_p1": ((2, 16, 14, 14), (16, 16, 3, 3), (1, 1), (1, 1)),
    "body_k3_64ch": ((1, 64, 12, 12), (64, 64, 3, 3), (1, 1), (1, 1)),
    "down_k1_s2": ((2, 32, 14, 14), (48, 32, 1, 1), (2, 2), (0, 0)),
    "rect_kernel_rect_stride": ((1, 5, 13, 9), (7, 5, 3, 2), (2, 1), (0, 2)),
    "one_pixel_out": ((3, 4, 3, 3), (5, 4, 3, 3), (1, 1), (0, 0)),
    "wide_padding": ((1, 2, 4, 4), (3, 2, 3, 3), (1, 1), (2, 2)),
    # channel counts that are multiples of 32 with rows of 8n columns: the LDS-patch kernel
    "patch_k3_s1_p1": ((2, 32, 8, 8), (16, 32, 3, 3), (1, 1), (1, 1)),
    "patch_k3_64ch_rows": ((1, 64, 24, 56), (64, 64, 3, 3), (1, 1), (1, 1)),
    "patch_k1_s2": ((2, 64, 16, 16), (96, 64, 1, 1), (2, 2), (0, 0)),
    "patch_k5_s2_p2": ((1, 32, 24, 16), (40, 32, 5, 5), (2, 2), (2, 2)),
    "patch_many_out_channels": ((1, 96, 8, 24), (200, 96, 3, 3), (1, 1), (1, 1)),
    "patch_rect_stride": ((2, 32, 9, 16), (8, 32, 2, 3), (1, 2), (1, 0)),
    # 3x3 kernels over 32-channel chunks: stride 2, no padding with four chunks, a tall tile, rectangular stride
    "k3_s2_p1": ((2, 64, 16, 16), (64, 64, 3, 3), (2, 2), (1, 1)),
    "k3_p0_128ch": ((1, 128, 10, 16), (32, 128, 3, 3), (1, 1), (0, 0)),
    "k3_tall_tile": ((1, 32, 40, 16), (70, 32, 3, 3), (1, 1), (1, 1)),
    # few channels: rows of 8 consecutive columns as contraction slots (even horizontal stride), and shapes next to those
    "stem_c1_k5": ((2, 1, 20, 19), (10, 1, 5, 5), (1, 1), (2, 2)),
    "stem_c3_k3_two_tiles": ((1, 3, 12, 16), (70, 3, 3, 3), (1, 1), (1, 1)),
    "stem_c1_k5_s2": ((2, 1, 20, 24), (10, 1, 5, 5), (2, 2), (2, 2)),
    "stem_c3_k3_s1x2_p1": ((1, 3, 12, 16), (70, 3, 3, 3), (1, 2), (1, 1)),
    "stem_c4_k5x8_s3x2": ((1, 4, 17, 32), (8, 4, 5, 8), (3, 2), (0, 4)),
    "stem_c2_k7_s2_tall": ((1, 2, 64, 16), (5, 2, 7, 7), (2, 2), (3, 3)),
    "k3_rect_stride_pad": ((1, 96, 13, 24), (64, 96, 3, 3), (2, 1), (0, 2)),
    # more than four chunks: two LDS stages per block (up to four chunks a block has one stage and shares its compute unit)
    "k3_two_stages_160ch": ((1, 160, 12, 16), (64, 160, 3, 3), (1, 1), (1, 1)),
    "k3_two_stages_256ch_s2": ((2, 256, 16, 16), (40, 256, 3, 3), (2, 2), (1, 1)),
    "k3_one_stage_ragged_rows": ((2, 64, 19, 56), (64, 64, 3, 3), (1, 1), (1, 1)),
    # 5x5 kernels over 32-channel chunks (one LDS stage, one block per compute unit): padding 2, stride 2, no padding with a
    # ragged last row block, more output channels than a block holds
    "k5_s1_p2": ((2, 32, 12, 16), (64, 32, 5, 5), (1, 1), (2, 2)),
    "k5_s2_p2_96ch": ((1, 96, 17, 24), (40, 96, 5, 5), (2, 2), (2, 2)),
    "k5_p0_two_co_tiles": ((1, 64, 11, 32), (130, 64, 5, 5), (1, 1), (0, 0)),
    "k5_rect_stride_pad": ((2, 32, 13, 16), (16, 32, 5, 5), (2, 1), (1, 3)),
    # 1x1 kernels with the weights resident in registers: 64..256 channels in, multiples of 256 out, stride 1 and 2,
    # pixel counts that end inside a 64-pixel tile, several images per worker
    "k1_s2_256ch": ((2, 256, 24, 24), (256, 256, 1, 1), (2, 2), (0, 0)),
    "k1_s2_64ch_two_groups": ((1, 64, 16, 16), (512, 64, 1, 1), (2, 2), (0, 0)),
    "k1_s1_128ch_short_tile": ((3, 128, 5, 8), (256, 128, 1, 1), (1, 1), (0, 0)),
    "k1_s1_192ch": ((1, 192, 10, 16), (256, 192, 1, 1), (1, 1), (0, 0)),
    "k1_s2_odd_rows": ((1, 64, 15, 24), (256, 64, 1, 1), (2, 2), (0, 0)),
    "k1_s2_many_images": ((40, 64, 8, 8), (256, 64, 1, 1), (2, 2), (0, 0)),
    # window sizes on both sides of 31 and 63 taps (the fp32 kernel keeps a per-pixel map of the taps inside the image in
    # one or two words, or tests every tap), and windows that lie wholly in the padding
    "k1x31_one_word": ((1, 2, 4, 40), (5, 2, 1, 31), (1, 1), (0, 15)),
    "k4x8_two_words": ((1, 3, 9, 20), (6, 3, 4, 8), (1, 2), (2, 3)),
    "k7x9_last_bit": ((1, 2, 12, 14), (4, 2, 7, 9), (1, 1), (3, 4)),
    "k8x8_every_tap_tested": ((1, 2, 12, 12), (4, 2, 8, 8), (2, 1), (4, 3)),
    "window_in_the_padding": ((1, 2, 5, 5), (3, 2, 2, 2), (1, 1), (3, 3)),
    # 32-channel chunks with rows that are not a multiple of 8 wide (28, 14, 7 ... as deeper in a ResNet): the patch's
    # rows are staged as one run of the channel plane, cut into pieces of eight wherever they fall
    "k3_w28_128ch": ((2, 128, 28, 28), (64, 128, 3, 3), (1, 1), (1, 1)),
    "k3_w14_256ch_two_stages": ((2, 256, 14, 14), (64, 256, 3, 3), (1, 1), (1, 1)),
    "k3_w7_64ch": ((3, 64, 7, 7), (64, 64, 3, 3), (1, 1), (1, 1)),
    "k3_w14_s2": ((2, 64, 14, 14), (40, 64, 3, 3), (2, 2), (1, 1)),
    "k3_w12_p0": ((1, 32, 9, 12), (16, 32, 3, 3), (1, 1), (0, 0)),
    "k3_w9_rect_stride": ((2, 32, 11, 9), (70, 32, 3, 3), (2, 1), (1, 0)),
    "k3_w5_two_rows_a_piece": ((2, 32, 6, 5), (16, 32, 3, 3), (1, 1), (1, 1)),
    "k3_w4_three_rows_a_piece": ((1, 32, 4, 4), (8, 32, 3, 3), (1, 1), (1, 1)),
    "k3_w30_tall": ((1, 32, 40, 30), (64, 32, 3, 3), (1, 1), (1, 1)),
    "k5_w14": ((1, 64, 14, 14), (32, 64, 5, 5), (1, 1), (2, 2)),
    "k5_w7_s2": ((2, 32, 7, 7), (16, 32, 5, 5), (2, 2), (2, 2)),
    # 1x1 kernels over pixel counts that are not a multiple of 16 bytes (196, 49, 45, 55): the product per image runs on
    # rows of a rounded-up pitch
    "k1_14x14_c512": ((2, 512, 14, 14), (64, 512, 1, 1), (1, 1), (0, 0)),
    "k1_7x7_c256": ((3, 256, 7, 7), (40, 256, 1, 1), (1, 1), (0, 0)),
    "k1_s2_14_to_7": ((2, 128, 14, 14), (72, 128, 1, 1), (2, 2), (0, 0)),
    "k1_5x9": ((2, 64, 5, 9), (24, 64, 1, 1), (1, 1), (0, 0)),
    "k1_s2x1_to_5x11": ((1, 64, 9, 11), (16, 64, 1, 1), (2, 1), (0, 0)),
    # ... and, without a stride, reads the images where they lie: one pixel, fewer pixels than a piece holds, a group that
    # straddles tiles of 128 columns (200 per image), many output channels, one output channel, a short K
    "k1_one_pixel": ((9, 64, 1, 1), (24, 64, 1, 1), (1, 1), (0, 0)),
    "k1_3x1": ((4, 128, 3, 1), (200, 128, 1, 1), (1, 1), (0, 0)),
    "k1_14x14_many_images": ((7, 64, 14, 14), (136, 64, 1, 1), (1, 1), (0, 0)),
    "k1_7x7_one_channel_out": ((5, 72, 7, 7), (1, 72, 1, 1), (1, 1), (0, 0)),
    "k1_13x13_c8": ((3, 8, 13, 13), (520, 8, 1, 1), (1, 1), (0, 0)),
    # channel counts that are not a multiple of 16 bytes over aligned pixel counts: the product per image with rows of weights
    # that start anywhere
    "k1_c100_28x28": ((3, 100, 28, 28), (200, 100, 1, 1), (1, 1), (0, 0)),
    "k1_c7_8x8": ((5, 7, 8, 8), (33, 7, 1, 1), (1, 1), (0, 0)),
    # few output pixels per image under a long K: the whole batch unfolded side by side, one product
    "unfolded_k3_7x7": ((5, 128, 7, 7), (40, 128, 3, 3), (1, 1), (1, 1)),
    "unfolded_k3_s2_14_to_7": ((6, 64, 14, 14), (48, 64, 3, 3), (2, 2), (1, 1)),
    "unfolded_k5_9x9": ((8, 32, 9, 9), (16, 32, 5, 5), (1, 1), (2, 2)),
    "unfolded_k3x2_100_pixels": ((3, 96, 10, 11), (24, 96, 3, 2), (1, 1), (1, 0)),
    # ... and as the last resort before the general tiles, for channel counts that no patch kernel takes (K >= 320)
    "unfolded_any_k7_48ch": ((2, 48, 20, 20), (48, 48, 7, 7), (1, 1), (3, 3)),
    "unfolded_any_k3_72ch": ((4, 72, 17, 17), (100, 72, 3, 3), (1, 1), (1, 1)),
    "unfolded_any_k3_40ch_s2": ((3, 40, 21, 19), (24, 40, 3, 3), (2, 2), (1, 1)),
    # ... more pixels per image but few in the whole batch, signals one row high (conv1d's shape), and one image under a
    # K beyond the general tiles' table (fewer columns than a tile is wide)
    "unfolded_few_pixels_in_batch": ((2, 96, 14, 14), (24, 96, 3, 3), (1, 1), (1, 1)),
    "unfolded_one_row_high": ((4, 128, 1, 200), (40, 128, 1, 7), (1, 2), (0, 3)),
    "unfolded_any_one_image_long_k": ((1, 160, 12, 12), (8, 160, 7, 7), (1, 1), (3, 3)),
    # ... a K that no 16 bytes divide (the rows of the weights start anywhere: the product's tiles for misaligned operands),
    # and few output channels over few results (float64: the unfolded product instead of one thread per result)
    "unfolded_odd_k_few_pixels": ((3, 116, 8, 8), (40, 116, 5, 5), (2, 2), (2, 2)),
    "unfolded_any_odd_k": ((4, 77, 20, 20), (24, 77, 3, 3), (1, 1), (1, 1)),
    "unfolded_three_channels_out_long_k": ((4, 50, 8, 8), (3, 50, 7, 7), (2, 2), (0, 0)),
    # ... a handful of pixels in all (the product: a workgroup per 4 x 4 results), one pixel, a K padded with zeros to whole
    # 16 bytes under many pixels (fp32: beyond the gathering tiles' table)
    "unfolded_one_image_few_pixels": ((1, 96, 8, 8), (8, 96, 4, 4), (1, 1), (0, 0)),
    "unfolded_one_pixel_an_image": ((2, 64, 3, 3), (43, 64, 3, 3), (3, 3), (1, 1)),
    "unfolded_padded_k_many_pixels": ((1, 405, 30, 30), (8, 405, 5, 3), (1, 1), (2, 1)),
    # ... in runs of images when the whole batch unfolded would be large (13 images and 1; one image at a time), with a
    # K beyond what the general tiles keep a table of
    "unfolded_any_runs_of_images": ((14, 128, 40, 40), (4, 128, 7, 7), (1, 1), (3, 3)),
    "unfolded_any_one_image_a_run": ((2, 256, 112, 112), (2, 256, 7, 7), (1, 1), (3, 3)),
}


@pytest.mark.parametrize("case", CONV_GOLDEN, ids=lambda c: c["name"])
def test_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    support.assert_close(got, golden_cases.expected_of(case), 1e-5, 1e-8, case["name"])


def operands(dtype, name, device, bias):
    xs, ws, stride, pad = CASES[name]
    fan_in = ws[1] * ws[2] * ws[3]
    hx, dx = support.both(support.values_for(dtype, SEED, 1, xs, -2, 2), dtype, device)
    lim = 100 if dtype.is_integral else 2 * (2.0 / fan_in) ** 0.5
    hw, dw = support.both(support.values_for(dtype, SEED, 2, ws, -lim, lim), dtype, device)
    hb, db = support.both(support.values_for(dtype, SEED, 3, (ws[0],), -2, 2), dtype, device) if bias else (None, None)
    return (hx, hw, hb), (dx, dw, db), stride, pad, fan_in


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("dtype", [ta.float32, ta.float64], ids=str)
def test_float_conv(device, dtype, name, bias):
    host, dev, stride, pad, k = operands(dtype, name, device, bias)
    want, got = ops.convolve2d(*host, stride, pad), ops.convolve2d(*dev, stride, pad)
    assert got.shape == want.shape
    eps = 2.0 ** -24 if dtype is ta.float32 else 2.0 ** -53
    support.assert_close(got.numpy(), want.numpy(), 1e-5 if dtype is ta.float32 else 1e-13, k * eps * 4, f"conv {dtype} {name}")


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_16bit_conv_fp32_accumulate(device, dtype, name, bias):
    host, dev, stride, pad, _ = operands(dtype, name, device, bias)
    want, got = ops.convolve2d(*host, stride, pad), ops.convolve2d(*dev, stride, pad)
    rtol = 2e-3 if dtype is ta.float16 else 2.0 ** -7
    support.assert_close(got.numpy(), want.numpy(), rtol, 1e-3, f"conv {dtype} {name}")


@pytest.mark.parametrize("name", ["body_k3_s1_p1", "rect_kernel_rect_stride", "wide_padding"])
@pytest.mark.parametrize("dtype", [ta.int8, ta.int32, ta.int64], ids=str)
def test_integer_conv_bit_exact(device, dtype, name):
    host, dev, stride, pad, _ = operands(dtype, name, device, True)
    support.assert_bit_exact(ops.convolve2d(*dev, stride, pad).storage(), ops.convolve2d(*host, stride, pad).storage(), f"conv {dtype} {name}")


def test_strided_signal_view(device):
    hx, dx = support.both(support.values_for(ta.float32, SEED, 4, (2, 9, 10, 6)), ta.float32, device)
    hw, dw = support.both(support.values_for(ta.float32, SEED, 5, (8, 6, 3, 3)), ta.float32, device)
    want = ops.convolve2d(hx.permute(0, 3, 1, 2), hw, None, 1, 1).numpy()
    got = ops.convolve2d(dx.permute(0, 3, 1, 2), dw, None, 1, 1).numpy()
    support.assert_close(got, want, 1e-5, 54 * 2.0 ** -24 * 16, "NHWC view")


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_channel_slice_of_a_larger_signal(device, dtype):
    """Channels 3..34 of a [2, 40, 14, 14] signal: planes that start at odd multiples of 196 elements, images 40 planes apart;
    and the same from a width of 16 (aligned rows, but the slice starts in the middle of nothing aligned to 16 bytes)."""
    for width in (14, 16):
        hx, dx = support.both(support.values_for(dtype, SEED, 6, (2, 40, 14, width), -2, 2), dtype, device)
        hw, dw = support.both(support.values_for(dtype, SEED, 7, (24, 32, 3, 3), -0.2, 0.2), dtype, device)
        want = ops.convolve2d(hx[:, 3:35], hw, None, 1, 1).numpy()
        got = ops.convolve2d(dx[:, 3:35], dw, None, 1, 1).numpy()
        support.assert_close(got, want, 2e-3 if dtype is ta.float16 else 2.0 ** -7, 1e-3, f"channel slice, width {width}")


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32], ids=str)
def test_pointwise_over_a_channel_slice_with_odd_pixel_counts(device, dtype):
    """A 1x1 kernel over channels 5..68 of a [3, 80, 7, 7] signal with a bias: every plane starts at an odd multiple of 49
    elements and an image is 80 planes long, so no row of the product starts at a multiple of 16 bytes."""
    hx, dx = support.both(support.values_for(dtype, SEED, 8, (3, 80, 7, 7), -2, 2), dtype, device)
    hw, dw = support.both(support.values_for(dtype, SEED, 9, (40, 64, 1, 1), -0.2, 0.2), dtype, device)
    hb, db = support.both(support.values_for(dtype, SEED, 10, (40,), -1, 1), dtype, device)
    want = ops.convolve2d(hx[:, 5:69], hw, hb, 1, 0).numpy()
    got = ops.convolve2d(dx[:, 5:69], dw, db, 1, 0).numpy()
    if dtype is ta.float32: support.assert_close(got, want, 1e-5, 64 * 2.0 ** -24 * 4, "pointwise over a channel slice")
    else: support.assert_close(got, want, 2e-3 if dtype is ta.float16 else 2.0 ** -7, 1e-3, "pointwise over a channel slice")


def test_status_codes(device):
    lib = ta.library()
    dvc = device.structure()
    x = ta.Tensor(ta.float32, (1, 3, 5, 5)).initialize(device)
    w = ta.Tensor(ta.float32, (2, 4, 3, 3)).initialize(device)
    w_ok = ta.Tensor(ta.float32, (2, 3, 3, 3)).initialize(device)
    wi = ta.Tensor(ta.int32, (2, 3, 3, 3)).initialize(device)
    y = ta.Tensor(ta.float32, (1, 2, 3, 3)).initialize(device)
    y_bad = ta.Tensor(ta.float32, (1, 2, 4, 3)).initialize(device)
    r3 = ta.Tensor(ta.float32, (3, 5, 5)).initialize(device)
    stream = lib.pop_stream(C.byref(dvc))
    try:
        f = lib.kernels["conv2d"]
        d = {k: v.descriptor() for k, v in dict(x=x, w=w, w_ok=w_ok, wi=wi, y=y, y_bad=y_bad, r3=r3).items()}
        pad, stride = abi.SIZE2(0, 0), abi.SIZE2(1, 1)
        assert f(C.byref(d["x"]), C.byref(d["w"]), C.byref(d["y"]), stream, pad, stride) == abi.ERROR       # channel mismatch
        assert f(C.byref(d["x"]), C.byref(d["w_ok"]), C.byref(d["y_bad"]), stream, pad, stride) == abi.ERROR  # wrong output shape
        assert f(C.byref(d["r3"]), C.byref(d["w_ok"]), C.byref(d["y"]), stream, pad, stride) == abi.ERROR     # rank
        assert f(C.byref(d["x"]), C.byref(d["wi"]), C.byref(d["y"]), stream, pad, stride) == abi.UNSUPPORTED_DTYPE
        assert f(C.byref(d["x"]), C.byref(d["w_ok"]), C.byref(d["y"]), stream, pad, stride) == abi.SUCCESS
    finally:
        lib.put_stream(C.byref(dvc), stream)


def test_conv1x1_equals_gemm_on_device(device):
    x = support.values_for(ta.float16, SEED, 6, (2, 32, 6, 6), -1, 1)
    w = support.values_for(ta.float16, SEED, 7, (24, 32, 1, 1), -1, 1)
    _, dx = support.both(x, ta.float16, device)
    _, dw = support.both(w, ta.float16, device)
    conv = ops.convolve2d(dx, dw).numpy()
    _, pixels = support.both(np.ascontiguousarray(x.transpose(0, 2, 3, 1)).reshape(72, 32), ta.float16, device)
    _, weights = support.both(w.reshape(24, 32), ta.float16, device)
    gemm = ops.matmul(pixels, weights.transpose()).numpy().reshape(2, 6, 6, 24).transpose(0, 3, 1, 2)
    support.assert_close(conv, gemm, 2e-3, 1e-3, "1x1 conv vs gemm")


# ---- conv1d: the one-row case of the same kernels -------------------------------------------------------------------
CONV1D_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] == "conv1d"]
CASES_1D = {
    "plain": ((2, 3, 17), (4, 3, 5), 1, 0),
    "stride_pad": ((1, 2, 20), (3, 2, 4), 3, 2),
    "few_channels_even_stride": ((2, 3, 64), (20, 3, 7), 2, 3),
    "pointwise": ((2, 64, 40), (48, 64, 1), 1, 0),
    "many_channels": ((1, 96, 24), (40, 96, 3), 1, 1),
}


@pytest.mark.parametrize("case", CONV1D_GOLDEN, ids=lambda c: c["name"])
def test_conv1d_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    support.assert_close(got, golden_cases.expected_of(case), 1e-5, 1e-8, case["name"])


@pytest.mark.parametrize("name", list(CASES_1D))
@pytest.mark.parametrize("dtype", [ta.float32, ta.float64, ta.float16, ta.bfloat16, ta.int32, ta.int8], ids=str)
def test_conv1d(device, dtype, name):
    xs, ws, stride, pad = CASES_1D[name]
    fan_in = ws[1] * ws[2]
    hx, dx = support.both(support.values_for(dtype, SEED, 11, xs, -2, 2), dtype, device)
    lim = 100 if dtype.is_integral else 2 * (2.0 / fan_in) ** 0.5
    hw, dw = support.both(support.values_for(dtype, SEED, 12, ws, -lim, lim), dtype, device)
    want, got = ops.convolve1d(hx, hw, stride, pad), ops.convolve1d(dx, dw, stride, pad)
    assert got.shape == want.shape
    if dtype.is_integral:
        support.assert_bit_exact(got.storage(), want.storage(), f"conv1d {dtype} {name}")
    elif dtype in (ta.float16, ta.bfloat16):
        support.assert_close(got.numpy(), want.numpy(), 2e-3 if dtype is ta.float16 else 2.0 ** -7, 1e-3, f"conv1d {dtype} {name}")
    else:
        eps = 2.0 ** -24 if dtype is ta.float32 else 2.0 ** -53
        support.assert_close(got.numpy(), want.numpy(), 1e-5 if dtype is ta.float32 else 1e-13, fan_in * eps * 4, f"conv1d {dtype} {name}")


@pytest.mark.parametrize("dtype", [ta.float32, ta.float16, ta.int32], ids=str)
@pytest.mark.parametrize("kernel", [1, 3], ids=lambda k: f"k{k}")
def test_bias_and_kernel_seen_through_views(device, oracle, dtype, kernel):
    """A column of a matrix is a valid bias and every other output channel of a kernel tensor a valid kernel: both are
    read through their strides by every kernel path (the reference reads the bias as b[co], src/cpu/conv2d.cpp:86).
    Small integers, so every type is exact and numpy decides."""
    rng = np.random.default_rng(17)
    x = rng.integers(-2, 3, (2, 8, 10, 16)).astype(np.float64)
    w = rng.integers(-2, 3, (12, 8, kernel, kernel)).astype(np.float64)
    table = rng.integers(-2, 3, (6, 5)).astype(np.float64)
    pad = kernel // 2
    padded = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    want = np.zeros((2, 6, 10, 16))
    for kh in range(kernel):
        for kw in range(kernel):
            want += np.einsum("nchw,oc->nohw", padded[:, :, kh:kh + 10, kw:kw + 16], w[::2, :, kh, kw])
    want += table[:, 3].reshape(1, 6, 1, 1)
    for make in (lambda a: support.both(a, dtype, device)[1], lambda a: support.host_tensor(a, dtype)):
        tx, tw, tb = make(x), make(w), make(table)
        got = ops.convolve2d(tx, tw[::2], tb[:, 3], 1, pad).numpy().astype(np.float64)
        np.testing.assert_array_equal(got, want)
