"""Pins the CPU oracle (oracle/fyn_oracle.c) against evidence that does not come from the oracle:
the reference tests' known-answer patterns and fp64 library routines (torch.nn.functional) /
brute force.  Runs without a GPU."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fyusenet_amd import prng
from oracle import oracle as O
from util import conv_block, rel_l2

RELU = (O.ACT_RELU, 0.0, 0.0, 0.0)


def _w_from_block(block, cout, k, cin):
    """[o][ky][kx][i] -> torch [o][i][ky][kx]"""
    w = np.asarray(block[cout:cout + cout * k * k * cin], dtype=np.float64).reshape(cout, k, k, cin)
    return torch.from_numpy(w.transpose(0, 3, 1, 2).copy())


# ---- reference known-answer patterns ---------------------------------------------------------
@pytest.mark.parametrize("k,cin,cout,size", [(3, 4, 8, 32), (5, 16, 8, 24), (7, 8, 4, 20)])
def test_pattern_antisymmetric_kernel_on_ones(k, cin, cout, size):
    # unit_tests/convlayertests.cpp:242-261,281-304,355-376: all-ones input, kernel -1 above the centre row,
    # 0 on it, +1 below => interior outputs 0, border rows != 0 because the halo is zero
    r = k // 2
    w = np.zeros((cout, k, k, cin), np.float32)
    w[:, :r] = -1.0
    w[:, r + 1:] = 1.0
    block = np.concatenate([np.zeros(cout, np.float32), w.ravel()])
    x = np.ones((cin, size, size), np.float32)
    y = O.conv2d(O.pad_chw(x, r), r, block, cout, k)
    assert np.all(y[:, r:size - r, :] == 0.0)
    assert np.all(y[:, 0, r:size - r] == cin * k * r)        # top row misses the -1 rows: +k*r*cin
    assert np.all(y[:, size - 1, r:size - r] == -cin * k * r)


def test_pattern_1x1_ones():
    # convlayertests.cpp:165-182,319-336: 1x1 all-ones weights on all-ones input => every output = Cin
    cin, cout = 12, 8
    block = np.concatenate([np.zeros(cout, np.float32), np.ones(cout * cin, np.float32)])
    y = O.conv2d(np.ones((cin, 16, 16), np.float32), 0, block, cout, 1)
    assert np.all(y == cin)


def test_pattern_shallow_edge_clamp_zero_sum():
    # unit_tests/networktests.cpp:85-97,173-186: unpadded shallow 3x3 conv 4->8 @32x32, zero-sum kernel on ones
    # => exactly 0 everywhere including the borders (edge clamp)
    cin, cout = 4, 8
    w = np.zeros((cout, 3, 3, cin), np.float32)
    w[:, 0] = -1.0
    w[:, 2] = 1.0
    block = np.concatenate([np.zeros(cout, np.float32), w.ravel()])
    y = O.conv2d(np.ones((cin, 32, 32), np.float32), 0, block, cout, 3, border=1)
    assert np.all(y == 0.0)
    # the same with the zero-halo rule is NOT zero on the border: the rule matters
    y0 = O.conv2d(np.ones((cin, 32, 32), np.float32), 0, block, cout, 3, border=0)
    assert np.any(y0 != 0.0)


def test_pattern_gemm_alternating_rows():
    # unit_tests/misctests.cpp:238-265: 512 -> 256, rows of alternating +-1 on ones => 0
    cin, cout = 512, 256
    w = np.tile(np.array([1.0, -1.0], np.float32), cin // 2)
    block = np.concatenate([np.zeros(cout, np.float32), np.tile(w, cout)])
    assert np.all(O.gemm(np.ones(cin, np.float32), block, cout) == 0.0)


# ---- library-routine cross checks --------------------------------------------------------------
@pytest.mark.parametrize("k,stride,dil,cin,cout,h,w,relu", [
    (3, 1, 1, 5, 7, 11, 13, False), (3, 2, 1, 12, 8, 16, 12, True), (5, 1, 1, 3, 4, 9, 10, True),
    (1, 2, 1, 6, 5, 8, 8, False), (3, 1, 2, 4, 6, 12, 12, True), (7, 2, 1, 3, 8, 20, 18, False), (9, 1, 1, 3, 2, 12, 14, True)])
def test_conv_matches_torch(k, stride, dil, cin, cout, h, w, relu):
    r = (k - 1) // 2 * dil
    x = prng.uniform(11, (cin, h, w), -1, 1)
    block = conv_block(20, cout, k, cin)
    y = O.conv2d(O.pad_chw(x, r), r, block, cout, k, dil, stride, RELU if relu else None)
    xt = torch.from_numpy(x.astype(np.float64))[None]
    if relu:
        xt = xt.clamp(min=0)
    ref = F.conv2d(xt, _w_from_block(block, cout, k, cin), torch.from_numpy(block[:cout].astype(np.float64)),
                   stride=stride, padding=r, dilation=dil)[0].numpy()
    ref = ref[:, :h // stride, :w // stride]
    assert y.shape == ref.shape
    assert rel_l2(y, ref) < 1e-6


def test_conv_with_halo_narrower_than_the_kernel_radius_reads_zero():
    # the reference's ResNet-50 stem: 7x7 stride 2 on a tensor stored with a halo of 1
    # (samples/samplenetworks/resnet50.cpp:211-212); what lies beyond the stored frame is zero, so the result
    # equals an ordinary padding-3 convolution
    k, cin, cout, h, w, stride, pad = 7, 3, 8, 20, 18, 2, 1
    x = prng.uniform(12, (cin, h, w), -1, 1)
    block = conv_block(21, cout, k, cin)
    y = O.conv2d(O.pad_chw(x, pad), pad, block, cout, k, 1, stride, None)
    ref = F.conv2d(torch.from_numpy(x.astype(np.float64))[None], _w_from_block(block, cout, k, cin),
                   torch.from_numpy(block[:cout].astype(np.float64)), stride=stride, padding=3)[0].numpy()
    ref = ref[:, :h // stride, :w // stride]
    assert y.shape == ref.shape
    assert rel_l2(y, ref) < 1e-6


def test_conv_bn_residual_epilogue():
    # order: acc*scale + (bias*scale + bnBias) + relu(res)*scale  (batchnorm.inc / residual.inc)
    cin, cout, k, h, w = 6, 5, 3, 8, 9
    x = prng.uniform(1, (cin, h, w), -1, 1)
    res = prng.uniform(2, (cout, h, w), -1, 1)
    block = conv_block(3, cout, k, cin, bn=True)
    flags = O.POST_BATCHNORM | O.RESIDUAL_INPUT | O.RELU_ON_RESIDUAL | O.BATCHNORM_ON_RESIDUAL
    y = O.conv2d(O.pad_chw(x, 1), 1, block, cout, k, act=RELU, flags=flags, residual=res)
    nw = cout * k * k * cin
    bias, scale, bnb = block[:cout].astype(np.float64), block[cout + nw:cout + nw + cout].astype(np.float64), block[cout + nw + cout:].astype(np.float64)
    acc = F.conv2d(torch.from_numpy(x.astype(np.float64))[None].clamp(min=0), _w_from_block(block, cout, k, cin), None, padding=1)[0].numpy()
    ref = acc * scale[:, None, None] + (bias * scale + bnb)[:, None, None] + np.maximum(res, 0) * scale[:, None, None]
    assert rel_l2(y, ref) < 1e-6
    # invariants: zero residual == no residual; zero weights => bias' + residual path only
    y0 = O.conv2d(O.pad_chw(x, 1), 1, block, cout, k, act=RELU, flags=flags, residual=np.zeros_like(res))
    y1 = O.conv2d(O.pad_chw(x, 1), 1, block, cout, k, act=RELU, flags=O.POST_BATCHNORM)
    assert np.array_equal(y0, y1)


@pytest.mark.parametrize("stride,dil,c,h,w", [(1, 1, 8, 10, 12), (2, 1, 24, 16, 16), (1, 2, 5, 9, 9)])
def test_dwconv_matches_grouped_conv(stride, dil, c, h, w):
    x = prng.uniform(5, (c, h, w), -1, 1)
    block = conv_block(6, c, 3, c, depthwise=True)
    clip = (O.ACT_CLIP, 0.0, 0.0, 6.0)
    y = O.dwconv(O.pad_chw(x * 8, dil), dil, block, 1, 3, dil, stride, clip)
    wt = torch.from_numpy(block[c:c + 9 * c].astype(np.float64).reshape(c, 1, 3, 3))
    ref = F.conv2d(torch.from_numpy((x * 8).astype(np.float64))[None].clamp(0, 6), wt, torch.from_numpy(block[:c].astype(np.float64)),
                   stride=stride, padding=dil, dilation=dil, groups=c)[0].numpy()[:, :h // stride, :w // stride]
    assert rel_l2(y, ref) < 1e-6


@pytest.mark.parametrize("k,crop,cin,cout,h,w", [(3, 0, 4, 6, 5, 7), (3, 1, 8, 3, 6, 6), (2, 0, 5, 4, 4, 9)])
def test_transconv_matches_conv_transpose(k, crop, cin, cout, h, w):
    x = prng.uniform(7, (cin, h, w), -1, 1)
    block = conv_block(8, cout, k, cin)
    y = O.transconv(x, 0, block, cout, k, crop, RELU)
    wt = _w_from_block(block, cout, k, cin).permute(1, 0, 2, 3)  # [i][o][ky][kx]
    ref = F.conv_transpose2d(torch.from_numpy(x.astype(np.float64))[None].clamp(min=0), wt,
                             torch.from_numpy(block[:cout].astype(np.float64)), stride=2)[0].numpy()
    ho, wo = 2 * h + k - 2 - crop, 2 * w + k - 2 - crop
    assert y.shape == (cout, ho, wo)
    assert rel_l2(y, ref[:, :ho, :wo]) < 1e-6


def test_transconv_brute_force_tiny():
    # out[2y+ky, 2x+kx] += w[ky,kx]*in[y,x] on a 2x2 single-channel input, by hand
    x = np.array([[[1.0, 2.0], [3.0, 4.0]]], np.float32)
    w = np.arange(1, 10, dtype=np.float32)  # [ky][kx]
    block = np.concatenate([np.array([0.5], np.float32), w])
    y = O.transconv(x, 0, block, 1, 3)[0]
    ref = np.zeros((5, 5))
    for yy in range(2):
        for xx in range(2):
            ref[2 * yy:2 * yy + 3, 2 * xx:2 * xx + 3] += x[0, yy, xx] * w.reshape(3, 3)
    assert np.allclose(y, ref + 0.5)


@pytest.mark.parametrize("pool", [2, 4])
def test_pool_equals_stride_matches_torch(pool):
    # the case PoolLayerTest::computeMaxPool/computeAvgPool cover (pool == stride, no padding)
    x = prng.uniform(9, (12, 16, 24), -100, 100)
    xt = torch.from_numpy(x.astype(np.float64))[None]
    assert np.array_equal(O.maxpool(x, 0, pool, pool), F.max_pool2d(xt, pool)[0].numpy().astype(np.float32))
    assert rel_l2(O.avgpool(x, 0, pool, pool), F.avg_pool2d(xt, pool)[0].numpy()) < 1e-6


def test_maxpool_3x3_s2_pad1_relu_equals_neg_inf_padding():
    # deep rule: window starts input_padding before the stride origin; with ReLU on fetch the zero halo is
    # equivalent to -inf padding (ResNet stem pool)
    x = prng.normal(10, (8, 14, 14))
    y = O.maxpool(O.pad_chw(x, 1), 1, 3, 2, RELU)
    ref = F.max_pool2d(torch.from_numpy(x.astype(np.float64))[None].clamp(min=0), 3, 2, padding=1)[0].numpy()
    assert np.array_equal(y, ref.astype(np.float32))


def test_avgpool_3_window_is_centred():
    x = prng.uniform(12, (4, 9, 9), -1, 1)
    y = O.avgpool(O.pad_chw(x, 1), 1, 3, 1)
    ref = F.avg_pool2d(torch.from_numpy(x.astype(np.float64))[None], 3, 1, padding=1, count_include_pad=True)[0].numpy()
    assert rel_l2(y, ref) < 1e-6


def test_global_pool_bn_argmax_concat_closed_forms():
    x = prng.uniform(13, (23, 7, 5), -3, 3)
    assert rel_l2(O.global_pool(x, 0, False, RELU).ravel(), np.maximum(x, 0).astype(np.float64).mean(axis=(1, 2))) < 1e-6
    assert np.array_equal(O.global_pool(x, 0, True).ravel(), x.max(axis=(1, 2)))
    sb = np.concatenate([prng.uniform(14, (23,), 0.5, 1.5), prng.normal(15, (23,))])
    assert rel_l2(O.batchnorm(x, 0, sb), x * sb[:23, None, None] + sb[23:, None, None]) < 1e-6
    idx, val = O.argmax(x)
    assert np.array_equal(idx, np.argmax(x, axis=0)) and np.array_equal(val, x.max(axis=0))
    tie = np.zeros((5, 2, 2), np.float32)  # all equal: lowest index wins (strict '>' scan)
    assert np.all(O.argmax(tie)[0] == 0)
    a, b = x[:7], x[7:]
    assert np.array_equal(O.concat([a, b]), x)


def test_round_fp16_is_ieee_rn():
    x = np.concatenate([prng.normal(16, (4096,)) * 10.0 ** prng.uniform(17, (4096,), -8, 5), [0.0, 65504.0, 65520.0, 1e-8, -5.96e-8]]).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(O.round_fp16(x), x.astype(np.float16).astype(np.float32))


def test_deep_tiling_and_layout_round_trips():
    assert O.deep_tiling(4) == (1, 1) and O.deep_tiling(8) == (2, 1) and O.deep_tiling(16) == (2, 2)
    assert O.deep_tiling(64) == (4, 4) and O.deep_tiling(12) == (2, 2) and O.deep_tiling(2048) == (27, 19) and O.deep_tiling(80) == (5, 4)  # by hand: 27*19=513: cost 8+1
    x = prng.uniform(18, (23, 6, 5), -1, 1)
    for pad in (0, 1):
        d = O.chw_to_deep(x, pad)
        assert np.array_equal(O.deep_to_chw(d, 23, 6, 5, pad), x)
    assert np.array_equal(O.shallow_to_chw(O.chw_to_shallow(x[:3], 4), 3), x[:3])


def test_shallow_layout_is_the_pixel_major_transposition():
    # GPU_SHALLOW host buffers are pixel-major with 3 or 4 components per pixel (RGB triplets in, RGBA out:
    # cpu/cpubuffer.cpp:121-158 walks them as src[(y*width + x)*packing + c]); channels beyond the tensor's read as zero.
    for c, pc in ((3, 3), (3, 4), (4, 4), (1, 4), (2, 3)):
        x = prng.uniform(19 + c + pc, (c, 5, 7), -1, 1)
        hwc = O.chw_to_shallow(x, pc)
        assert hwc.shape == (5, 7, pc)
        assert np.array_equal(hwc[..., :c], x.transpose(1, 2, 0))
        assert not hwc[..., c:].any()
        back = O.shallow_to_chw(np.ascontiguousarray(hwc), c)
        assert np.array_equal(back, x)
        # a pixel-major array of our own making, read back channel by channel (a converter that walked rows or
        # components in another order would return something else)
        own = prng.uniform(31 + c + pc, (5, 7, pc), -1, 1)
        assert np.array_equal(O.shallow_to_chw(own, c), own[..., :c].transpose(2, 0, 1))


# ---- leaky ReLU, batch-norm layer with residual, GPU_DEEP layout ----------------------------------
@pytest.mark.parametrize("leak", [0.1, 0.25, 1.5])
def test_leaky_relu_on_fetch(leak):
    # shaders/activation.inc:6-8: sg = step(0, x); out = (sg + leak*(1 - sg)) * x, i.e. x for x >= 0 (step(0,0) = 1)
    # and leak*x below.  Checked through three oracle entry points that apply the activation while reading.
    cin, cout, k, h, w = 5, 4, 3, 7, 6
    x = prng.uniform(40, (cin, h, w), -2, 2)
    x[0, 0, :3] = (0.0, -0.0, 1e-30)
    act = (O.ACT_LEAKY, leak, 0.0, 0.0)
    x64 = x.astype(np.float64)
    sg = (x64 >= 0).astype(np.float64)
    shader = (sg + leak * (1.0 - sg)) * x64
    lib = F.leaky_relu(torch.from_numpy(x64), leak).numpy()
    assert np.allclose(shader, lib, rtol=0, atol=0)
    # (1) identity function layer: act(x) itself, to fp32 rounding of leak*x
    y = O.unary(x, O.FN_COPY, act=act)
    # (2) batch-norm layer with scale 1, bias 0 is act(x)
    sb = np.concatenate([np.ones(cin, np.float32), np.zeros(cin, np.float32)])
    yb = O.batchnorm(x, 0, sb, act=act)
    assert rel_l2(yb, shader) < 1e-7
    assert np.array_equal(yb[x >= 0], x[x >= 0])          # the positive side passes unchanged, -0.0 and 0.0 included
    assert np.all(yb[x < 0] == (np.float32(leak) * x[x < 0]))
    assert np.array_equal(y, yb)
    # (3) convolution reading a leaky input == library convolution of the library's leaky_relu
    block = conv_block(41, cout, k, cin)
    yc = O.conv2d(O.pad_chw(x, 1), 1, block, cout, k, act=act)
    ref = F.conv2d(torch.from_numpy(lib)[None], _w_from_block(block, cout, k, cin),
                   torch.from_numpy(block[:cout].astype(np.float64)), padding=1)[0].numpy()
    assert rel_l2(yc, ref) < 1e-6
    # a sign error or a swapped branch would give relu or leak*x everywhere: both differ
    assert rel_l2(yb, np.maximum(x64, 0)) > 1e-2 and rel_l2(yb, leak * x64) > 1e-2


@pytest.mark.parametrize("flags_names", [("RESIDUAL_INPUT",), ("RESIDUAL_INPUT", "RELU_ON_RESIDUAL"),
                                         ("RESIDUAL_INPUT", "BATCHNORM_ON_RESIDUAL"),
                                         ("RESIDUAL_INPUT", "RELU_ON_RESIDUAL", "BATCHNORM_ON_RESIDUAL")])
def test_batchnorm_layer_residual_variants(flags_names):
    # shaders/deep/deepbatchnorm.frag:26-35: out = act(in)*s + b; r = res; RELU_ON_RESIDUAL: r = max(0, r);
    # BATCHNORM_ON_RESIDUAL: r = r*s + b (scale AND bias, unlike the convolution's applyBNNB); out += r
    c, h, w = 7, 5, 6
    x = prng.uniform(42, (c, h, w), -2, 2)
    res = prng.uniform(43, (c, h, w), -2, 2)
    sb = np.concatenate([prng.uniform(44, (c,), 0.5, 1.5), prng.normal(45, (c,))]).astype(np.float32)
    s, b = sb[:c].astype(np.float64)[:, None, None], sb[c:].astype(np.float64)[:, None, None]
    flags = 0
    for n in flags_names:
        flags |= getattr(O, n)
    y = O.batchnorm(O.pad_chw(x, 1), 1, sb, act=RELU, flags=flags, residual=res)
    r = res.astype(np.float64)
    if "RELU_ON_RESIDUAL" in flags_names:
        r = np.maximum(r, 0.0)
    if "BATCHNORM_ON_RESIDUAL" in flags_names:
        r = r * s + b
    ref = np.maximum(x.astype(np.float64), 0.0) * s + b + r
    assert rel_l2(y, ref) < 1e-6
    # each flag changes the result (a dropped term would pass one of the other parametrisations unchanged)
    plain = np.maximum(x.astype(np.float64), 0.0) * s + b
    assert rel_l2(y, plain) > 1e-2
    if "BATCHNORM_ON_RESIDUAL" in flags_names:
        assert rel_l2(y, plain + (np.maximum(res, 0) if "RELU_ON_RESIDUAL" in flags_names else res) * s) > 1e-2  # bias is included
    # the residual flag without a residual tensor and a zero residual without BN-on-residual are the plain layer
    assert np.array_equal(O.batchnorm(O.pad_chw(x, 1), 1, sb, act=RELU, flags=O.RESIDUAL_INPUT, residual=np.zeros_like(res)),
                          O.batchnorm(O.pad_chw(x, 1), 1, sb, act=RELU))


def _deep_by_tiler(x, pad):
    """GPU_DEEP buffer written pixel by pixel from the output-tile arithmetic of DeepTiler
    (gpu/deep/deeptiler.cpp:73-76 viewport, :97-110: tiles in y-outer / x-inner order, tile (x, y) at image
    coordinates x*(w+pad)+pad, y*(h+pad)+pad), four channels per pixel."""
    c, h, w = x.shape
    tiles = (c + 3) // 4
    tx, ty = O.deep_tiling(c)
    vw, vh = tx * (w + pad) + pad, ty * (h + pad) + pad
    buf = np.zeros((vh, vw, 4), np.float32)
    tilenum = 0
    for y in range(ty):
        for xx in range(tx):
            if tilenum >= tiles:
                break
            ox, oy = xx * (w + pad) + pad, y * (h + pad) + pad
            for l in range(min(4, c - 4 * tilenum)):
                buf[oy:oy + h, ox:ox + w, l] = x[4 * tilenum + l]
            tilenum += 1
    return buf


def _chw_by_cpubuffer(src, c, th, tw, tx, ty):
    """CPUBuffer::deepToChannelWise at padding 0 (cpu/cpubuffer.cpp:424-437) restated index by index: tile
    (tx, ty) starts at row ty*tileHeight, column tx*tileWidth of a buffer that is shape.width_ = tx_count*tileWidth
    pixels wide; channels count up over ty-outer / tx-inner tiles.  (The reference multiplies the row index by
    PIXEL_PACKING twice, `(y*srcstride+x)*PIXEL_PACKING` with srcstride already in elements; the row stride used
    here is the buffer's actual one, width_*PIXEL_PACKING elements.)"""
    width = tx * tw
    flat = src.reshape(-1)
    out = np.zeros((c, th, tw), np.float32)
    ch = 0
    for tyi in range(ty):
        for txi in range(tx):
            rem = min(4, c - ch)
            base = (tyi * th) * width * 4 + (txi * tw) * 4
            for l in range(max(rem, 0)):
                for y in range(th):
                    for xx in range(tw):
                        out[ch, y, xx] = flat[base + (y * width + xx) * 4 + l]
                ch += 1
    return out


@pytest.mark.parametrize("c,h,w", [(23, 6, 5), (8, 3, 7), (36, 4, 4), (80, 2, 3), (5, 5, 2)])
def test_deep_layout_against_tiler_and_cpubuffer_arithmetic(c, h, w):
    x = prng.uniform(46, (c, h, w), -1, 1)
    x += np.arange(c, dtype=np.float32)[:, None, None]  # every channel distinct: a swapped tile row/column cannot pass
    tx, ty = O.deep_tiling(c)
    for pad in (0, 1):
        d = O.chw_to_deep(x, pad)
        ref = _deep_by_tiler(x, pad)
        assert d.shape == ref.shape == (ty * (h + pad) + pad, tx * (w + pad) + pad, 4)
        assert np.array_equal(d, ref)
    # padding 0: the reference's CPU-side reader gives back the tensor from the oracle's buffer, and the oracle's
    # own reader agrees with it
    d0 = O.chw_to_deep(x, 0)
    assert np.array_equal(_chw_by_cpubuffer(d0, c, h, w, tx, ty), x)
    assert np.array_equal(O.deep_to_chw(d0, c, h, w, 0), x)
    assert np.array_equal(O.deep_to_chw(_deep_by_tiler(x, 1), c, h, w, 1), x)
