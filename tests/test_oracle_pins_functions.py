"""Pins the oracle's function-type layers (scale, sigmoid, tanh, singleton arithmetic, cast, transpose, image-patch
extraction, non-maximum suppression, blur, RGB<->BGR) against evidence that does not come from the oracle: the
reference tests' known answers, numpy/scipy/torch routines in fp64 and brute force.  Runs without a GPU."""
import numpy as np
import pytest
import scipy.ndimage
import scipy.special
import torch
import torch.nn.functional as F

from fyusenet_amd import prng
from oracle import oracle as O

RELU = (O.ACT_RELU, 0.0, 0.0, 0.0)


# ---- reference known answers ------------------------------------------------------------------
# unit_tests/arithtests.cpp:205-234: constant tensor (op) scalar; (operand1, operand2, w, h, channels)
ARITH_CASES = [(3.0, 30.0, 400, 300, 4), (-2.0, 1.0, 200, 200, 5), (10.0, -10.0, 16, 16, 40), (-100.0, 23.0, 55, 57, 30),
               (15.0, -16.0, 99, 52, 47)]


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("a,b,w,h,c", ARITH_CASES)
def test_singleton_arithmetic_reference_patterns(op, a, b, w, h, c):
    x = np.full((c, h, w), a, np.float32)
    y = O.unary(x, O.FN_ARITH, op, b)
    expect = [a + b, a - b, a * b, a / b][op]
    assert y.shape == x.shape
    assert np.all(y == np.float32(expect))        # the reference accepts |diff| < 0.5 (arithtests.cpp:131)


# unit_tests/arithtests.cpp:236-248: constant (op) constant for the two-input add/sub layer
@pytest.mark.parametrize("sub", [False, True])
@pytest.mark.parametrize("a,b,w,h,c", ARITH_CASES)
def test_addsub_reference_patterns(sub, a, b, w, h, c):
    y = O.addsub(np.full((c, h, w), a, np.float32), np.full((c, h, w), b, np.float32), sub)
    assert np.all(y == np.float32(a - b if sub else a + b))


# ---- library routines / closed forms ----------------------------------------------------------
def test_sigmoid_and_tanh_against_scipy_numpy():
    x = prng.normal(11, (5, 17, 13), 0.0, 3.0)
    assert np.allclose(O.unary(x, O.FN_SIGMOID), scipy.special.expit(x.astype(np.float64)), rtol=0, atol=1e-7)
    assert np.allclose(O.unary(x, O.FN_TANH), np.tanh(x.astype(np.float64)), rtol=0, atol=1e-7)
    # the shader's spelling of tanh, 2*(e^{2x}/(1+e^{2x}))-1 (deeptanh.frag:21), where it does not overflow
    xd = x.astype(np.float64)
    assert np.allclose(O.unary(x, O.FN_TANH), 2.0 * (np.exp(2 * xd) / (1.0 + np.exp(2 * xd))) - 1.0, rtol=0, atol=1e-7)
    # activation on fetch comes first
    assert np.allclose(O.unary(x, O.FN_SIGMOID, act=RELU), scipy.special.expit(np.maximum(x, 0).astype(np.float64)), atol=1e-7)
    assert np.array_equal(O.unary(x, O.FN_COPY, act=RELU), np.maximum(x, 0))


@pytest.mark.parametrize("target,lo,hi", [(0, -2147483648.0, 2147483647.0), (1, -32768, 32767), (2, -128, 127),
                                          (3, 0, 4294967295.0), (4, 0, 65535), (5, 0, 255)])
def test_cast_integer_targets(target, lo, hi):
    x = np.concatenate([prng.uniform(5, (4000,), -400.0, 400.0), prng.uniform(6, (2000,), -7e4, 7e4),
                        np.array([0.49, -0.49, 1.51, -1.51, 254.6, 255.4, 1e12, -1e12], np.float32)]).reshape(1, 1, -1)
    x = x[np.abs(x - np.floor(x) - 0.5) > 1e-3].reshape(1, 1, -1)       # away from exact halves
    expect = np.clip(np.rint(x.astype(np.float64)), lo, hi).astype(np.float32)
    assert np.array_equal(O.unary(x, O.FN_CAST, target), expect)


def test_cast_float_targets():
    x = prng.normal(8, (3, 9, 9), 0.0, 100.0)
    assert np.array_equal(O.unary(x, O.FN_CAST, 7), x)
    assert np.array_equal(O.unary(x, O.FN_CAST, 6), x.astype(np.float16).astype(np.float32))


def test_transpose_is_numpy_transpose_and_involution():
    x = prng.normal(21, (6, 11, 7))
    y = O.transpose(x)
    assert np.array_equal(y, x.transpose(0, 2, 1))
    assert np.array_equal(O.transpose(y), x)
    assert np.array_equal(O.transpose(x, RELU), np.maximum(x, 0).transpose(0, 2, 1))


@pytest.mark.parametrize("cin,window", [(4, 2), (8, 2), (12, 3), (8, 4)])
def test_imgextract_is_space_to_depth(cin, window):
    h, w = 6 * window, 5 * window
    x = prng.normal(31, (cin, h, w))
    y = O.imgextract(x, window, cin * window * window)
    # out[(ypix*n + xpix)*C + c, y, x] = in[c, y*n + ypix, x*n + xpix]
    ref = x.reshape(cin, h // window, window, w // window, window).transpose(2, 4, 0, 1, 3).reshape(-1, h // window, w // window)
    assert np.array_equal(y, ref)


def test_imgextract_partial_group_brute_force():
    # 6 input channels occupy two texel groups (the second half empty): its output groups keep that gap
    cin, n, h, w = 6, 2, 4, 6
    x = prng.normal(32, (cin, h, w))
    cout = 8 * n * n
    y = O.imgextract(x, n, cout)
    for o in range(cout):
        g, j = divmod(o, 4)
        b, it = divmod(g, 2)
        c = it * 4 + j
        xp, yp = b % n, b // n
        ref = x[c, yp::n, xp::n] if c < cin else np.zeros((h // n, w // n), np.float32)
        assert np.array_equal(y[o], ref), o


def test_nonmax_against_maximum_filter():
    x = prng.uniform(41, (3, 20, 23), 0.0, 1.0)
    cross = np.array([[0, 1, 0], [1, 1, 1], [0, 1, 0]], bool)
    for pad in (0, 1):
        stored = O.pad_chw(x, pad)
        y = O.nonmax(stored, pad)
        ref = np.empty_like(x)
        for c in range(x.shape[0]):
            # unpadded texture: the edge repeats; padded: the zero halo takes part
            m = scipy.ndimage.maximum_filter(stored[c], footprint=cross, mode="nearest")
            m = m[pad:pad + x.shape[1], pad:pad + x.shape[2]]
            ref[c] = np.where((x[c] >= m) & (x[c] > np.float32(0.1)), x[c], 0.0)
        assert np.array_equal(y, ref)
        assert 0 < np.count_nonzero(y) < y.size // 3


def test_blur_coefficients():
    assert np.allclose(O.blur_coeffs(3, False), 1.0 / 9.0)
    g = O.blur_coeffs(5, True).astype(np.float64)
    g1 = np.exp(-np.arange(-2, 3, dtype=np.float64) ** 2)
    ref = np.outer(g1, g1)
    assert np.allclose(g, ref / ref.sum(), atol=1e-7)
    assert abs(g.sum() - 1.0) < 1e-6


@pytest.mark.parametrize("gaussian", [False, True])
def test_blur_3x3_against_correlate(gaussian):
    x = prng.normal(51, (2, 15, 18))
    k = O.blur_coeffs(3, gaussian).astype(np.float64)
    for pad in (0, 1):
        stored = O.pad_chw(x, pad)
        y = O.blur(stored, pad, 3, gaussian)
        for c in range(2):
            ref = scipy.ndimage.correlate(stored[c].astype(np.float64), k, mode="nearest")
            ref = ref[pad:pad + 15, pad:pad + 18]
            assert np.allclose(y[c], ref, atol=1e-6)


def test_blur_larger_kernels_follow_the_shader_loop():
    # generickernel.frag:98-104: offsets -(k-1)/2 .. (k-1)/2-1, coefficients in running order
    k, pad = 5, 2
    x = prng.normal(52, (1, 9, 10))
    stored = O.pad_chw(x, pad).astype(np.float64)
    coef = O.blur_coeffs(k, True).ravel().astype(np.float64)
    y = O.blur(O.pad_chw(x, pad), pad, k, True)
    ref = np.zeros((9, 10))
    i = 0
    for oy in range(-2, 2):
        for ox in range(-2, 2):
            ref += coef[i] * stored[0, pad + oy:pad + oy + 9, pad + ox:pad + ox + 10]
            i += 1
    assert np.allclose(y[0], ref, atol=1e-6)


def test_rgb2bgr_swaps_first_and_third_of_each_group():
    x = prng.normal(61, (8, 5, 6))
    y = O.rgb2bgr(x)
    assert np.array_equal(y, x[[2, 1, 0, 3, 6, 5, 4, 7]])
    x3 = x[:3]
    assert np.array_equal(O.rgb2bgr(x3), x3[::-1])
    assert np.array_equal(O.rgb2bgr(O.rgb2bgr(x)), x)


# ---- scale layer ----------------------------------------------------------------------------------
@pytest.mark.parametrize("up", [2, 3, 4])
def test_scale_nearest_upsampling_repeats_pixels(up):
    x = prng.normal(71, (3, 7, 9))
    for deep in (True, False):
        y = O.scale(x, 0, (up, up), (1, 1), False, deep)
        assert np.array_equal(y, np.repeat(np.repeat(x, up, axis=1), up, axis=2))
    y = O.scale(O.pad_chw(x, 1), 1, (up, 1), (1, 1), False, True, RELU)       # anisotropic, padded, activated
    assert np.array_equal(y, np.maximum(np.repeat(x, up, axis=2), 0))


@pytest.mark.parametrize("down", [2, 3, 4])
def test_scale_downsampling_sample_positions(down):
    x = prng.normal(72, (2, 24, 36))
    # deep: the quad starts (d-1)/2 texels early, samples sit on texel centres x*d (deeptiler.cpp:97-110)
    for linear in (False, True):
        assert np.array_equal(O.scale(x, 0, (1, 1), (down, down), linear, True), x[:, ::down, ::down])
    # shallow: position (x+1/2)*d; nearest takes the texel that contains it
    assert np.array_equal(O.scale(x, 0, (1, 1), (down, down), False, False), x[:, down // 2::down, down // 2::down])


def _torch_bilinear(stored, size):
    t = torch.from_numpy(stored.astype(np.float64))[None]
    return F.interpolate(t, size=size, mode="bilinear", align_corners=False)[0].numpy()


@pytest.mark.parametrize("up", [2, 3])
@pytest.mark.parametrize("pad", [0, 1])
def test_scale_linear_upsampling_against_interpolate(up, pad):
    # GL_LINEAR at position (x+1/2)/u is bilinear interpolation with half-pixel centres; on the stored (padded)
    # texture with clamp-to-edge that is torch's align_corners=False on the stored array, cropped
    x = prng.normal(73, (2, 8, 11))
    stored = O.pad_chw(x, pad)
    ref = _torch_bilinear(stored, (stored.shape[1] * up, stored.shape[2] * up))
    ref = ref[:, pad * up:pad * up + 8 * up, pad * up:pad * up + 11 * up]
    for deep in (True, False):
        y = O.scale(stored, pad, (up, up), (1, 1), True, deep)
        assert np.allclose(y, ref, atol=1e-6)
    # activation acts on the interpolated value
    y = O.scale(stored, pad, (up, up), (1, 1), True, True, RELU)
    assert np.allclose(y, np.maximum(ref, 0), atol=1e-6)


def test_scale_linear_shallow_downsampling_is_box_average():
    x = prng.normal(74, (2, 12, 16))
    y = O.scale(x, 0, (1, 1), (2, 2), True, False)
    ref = F.avg_pool2d(torch.from_numpy(x.astype(np.float64))[None], 2)[0].numpy()
    assert np.allclose(y, ref, atol=1e-6)
    assert np.allclose(y, _torch_bilinear(x, (6, 8)), atol=1e-6)


def test_scale_factor_one_is_a_copy_with_activation():
    x = prng.normal(75, (5, 6, 7))
    assert np.array_equal(O.scale(O.pad_chw(x, 2), 2, (1, 1), (1, 1), False, True), x)
    assert np.array_equal(O.scale(x, 0, (1, 1), (1, 1), True, False, (O.ACT_CLIP, 0.0, -0.5, 0.5)), np.clip(x, -0.5, 0.5))


# ---- fractional-step convolution ---------------------------------------------------------------
def _conv_block(seed, cout, k, cin, bn=False):
    parts = [prng.normal(seed, (cout,), 0, 0.3), prng.normal(seed + 1, (cout, k, k, cin), 0, 0.5).ravel()]
    if bn:
        parts += [prng.uniform(seed + 2, (cout,), 0.5, 1.5), prng.normal(seed + 3, (cout,), 0, 0.2)]
    return np.concatenate(parts).astype(np.float32)


@pytest.mark.parametrize("border", [0, 1])
@pytest.mark.parametrize("k,inv,stride,pad", [(5, 2, 1, 2), (9, 2, 1, 3), (7, 4, 2, 2), (5, 2, 2, 1), (9, 4, 1, 2), (5, 1, 1, 2), (7, 2, 1, 0),
                                              (5, 4, 2, 0), (3, 2, 1, 1), (3, 2, 2, 1), (3, 4, 2, 1), (3, 2, 1, 0), (3, 4, 2, 0)])
def test_fracconv_is_a_convolution_of_the_repeated_input(k, inv, stride, pad, border):
    """Sampling at floor((stride*x + t + 1/2) / inv) reads, from the input whose every stored pixel is repeated
    inv x inv times (numpy.repeat), the pixel stride*x + t: the layer equals the ordinary strided convolution (pinned
    elsewhere against torch and the reference's patterns) of that image.  The 3x3 shader's taps sit one step to the
    left (fraconv3x3.frag:14-19): there the comparison image is shifted right by one column."""
    cin, cout, h, w = 3, 4, 6, 8
    x = prng.uniform(71 + k, (cin, h, w), -1, 1)
    xs = np.pad(x, ((0, 0), (pad, pad), (pad, pad)))
    blk = _conv_block(900 + k, cout, k, cin, bn=True)
    res = prng.uniform(5, (cout, h * inv // stride, w * inv // stride), -1, 1)
    flags = O.POST_BATCHNORM | O.RESIDUAL_INPUT | O.RELU_ON_RESIDUAL
    got = O.fracconv(xs, pad, blk, cout, k, stride, inv, RELU, flags, res, border)
    up = np.repeat(np.repeat(xs, inv, axis=1), inv, axis=2)
    if k == 3:
        first = up[:, :, :1] if border else np.zeros_like(up[:, :, :1])     # what lies left of the stored image
        up = np.concatenate([first, up[:, :, :-1]], axis=2)
    want = O.conv2d(up, pad * inv, blk, cout, k, 1, stride, RELU, flags, res, border)
    assert got.shape == want.shape == (cout, h * inv // stride, w * inv // stride)
    if k == 3:      # the shifted comparison image has lost its last column, which the last output column reads
        got, want = got[:, :, :-1], want[:, :, :-1]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("k,step,stride,pad", [(3, 0.5, 1, 0), (3, 0.5, 2, 0), (3, 0.25, 2, 0), (5, 0.5, 1, 1), (9, 0.5, 1, 0), (7, 0.25, 2, 2)])
def test_fracconv_against_the_proxy_polygon_arithmetic(k, step, stride, pad):
    """Brute force from the geometry the reference renders with (gpu/vanilla/convlayerbase_vanilla.cpp:361-371,
    fractionalconvlayerNxN_vanilla.cpp:47-48,91): normalised texture coordinates of the polygon of row pass ky,
    interpolated at the fragment centre, the shader's horizontal offsets in units of texStep, nearest filtering
    (floor of coordinate x texture size) with clamping to the texture's edge.  Floats as in the reference."""
    f = np.float32
    cin, cout, h, w = 2, 3, 4, 8
    x = prng.uniform(31 + k, (cin, h, w), -1, 1)
    xs = np.pad(x, ((0, 0), (pad, pad), (pad, pad)))
    blk = _conv_block(700 + k, cout, k, cin)
    bias, wts = blk[:cout], blk[cout:].reshape(cout, k, k, cin)
    tw, th = int(f(w) / (f(step) * f(stride))), int(f(h) / (f(step) * f(stride)))
    texstep = f(step) / f(w + 2 * pad)
    hoffs = {3: [-2, -1, 0]}.get(k, list(range(-(k // 2), k // 2 + 1)))
    want = np.zeros((cout, th, tw))
    for ky in range(k):
        thspan, tvspan = f(w) / f(w + 2 * pad), f(h) / f(h + 2 * pad)
        tleft = f(pad) / f(w + 2 * pad)
        ttop = (f(pad) + f(step) * f(ky - (k - 1) // 2)) / f(h + 2 * pad)
        if stride > 1:
            tleft = tleft - f(step) * f(0.5) * f(stride - 1) / f(w + 2 * pad)
            ttop = ttop - f(step) * f(0.5) * f(stride - 1) / f(h + 2 * pad)
        for yo in range(th):
            v = float(ttop) + (yo + 0.5) / th * float(tvspan)
            sy = min(max(int(np.floor(v * (h + 2 * pad))), 0), h + 2 * pad - 1)
            for xo in range(tw):
                u0 = float(tleft) + (xo + 0.5) / tw * float(thspan)
                for kx in range(k):
                    u = u0 + hoffs[kx] * float(texstep)
                    sx = min(max(int(np.floor(u * (w + 2 * pad))), 0), w + 2 * pad - 1)
                    want[:, yo, xo] += wts[:, ky, kx, :].astype(np.float64) @ xs[:, sy, sx].astype(np.float64)
    want += bias[:, None, None]
    got = O.fracconv(xs, pad, blk, cout, k, stride, int(round(1 / step)), None, 0, None, 1)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
