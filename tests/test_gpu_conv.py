"""Parity of the HIP convolution family against the CPU oracle, through the C ABI (ctypes).

Tolerances (the north-star's): rel-L2 <= 1e-4 for fp32 storage, <= 2e-3 for fp16 storage.  For fp16
storage the oracle emulates the storage format (inputs, weights and outputs rounded to binary16)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import prng
from util import combos, conv_block, oracle_single, rel_l2, run_single

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}
A = fa.ActType
# axes of the generated combinations: (values, id function)
STORAGE_AXIS = ([fa.STORAGE_F32, fa.STORAGE_F16], lambda s: "f32" if s == fa.STORAGE_F32 else "f16")
SHALLOW_AXIS = ([False, True], lambda sh: "shallow_edge_clamp" if sh else "deep")
ACT3_AXIS = ([A.RELU, A.LEAKY_RELU, A.NONE], lambda a: {A.RELU: "relu", A.LEAKY_RELU: "leaky", A.NONE: "none"}[a])


def conv_builder(k, cout, h, w, cin, stride=1, dil=1, act=A.NONE, deep=True, pad_in=None, pad_out=0, bn=False, residual=None,
                 leak=0.0, clip=None, number=1):
    b = fa.ConvLayerBuilder(k, "conv").type(fa.LayerType.CONVOLUTION2D).number(number).shape(cout, h, w, cin)
    b.downsample(stride).dilation(dil).prefixAct(act).outputPadding(pad_out)
    b.inputPadding((k - 1) // 2 * dil if pad_in is None else pad_in)
    if deep:
        b.deep()
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    if residual is not None:
        b.residual(*residual).residualPadding(pad_out)
    if leak:
        b.leakyReLU(leak)
    if clip:
        b.clip(*clip)
    return b


CASES = [
    # k, cout, h, w, cin, stride, dil, act, kwargs
    (3, 64, 64, 64, 64, 1, 1, A.RELU, {}),
    (1, 16, 48, 40, 12, 1, 1, A.NONE, {}),
    (1, 64, 28, 28, 256, 2, 1, A.RELU, {}),
    (3, 8, 128, 256, 12, 2, 1, A.RELU, {}),        # unit_tests/convlayertests.cpp:380 DeepConv3x3 shape
    (5, 16, 40, 36, 16, 1, 1, A.NONE, {}),
    (7, 64, 64, 64, 3, 2, 1, A.NONE, {}),           # ResNet stem
    (9, 32, 40, 56, 3, 1, 1, A.NONE, {}),           # style net first layer (row-run path)
    (9, 3, 40, 56, 32, 1, 1, A.RELU, {"pad_out": 0}),
    (3, 128, 39, 47, 128, 1, 1, A.RELU, {"bn": True, "residual": (A.NONE, False), "pad_out": 1}),
    (3, 32, 20, 20, 24, 1, 2, A.RELU, {}),          # dilation
    (3, 40, 17, 23, 40, 1, 1, A.LEAKY_RELU, {"leak": 0.1}),
    (1, 96, 14, 14, 24, 1, 1, A.CLIP, {"clip": (0.0, 6.0)}),
    (3, 256, 14, 14, 256, 1, 1, A.RELU, {"bn": True, "residual": (A.RELU, True)}),
    (1, 2048, 7, 7, 512, 1, 1, A.RELU, {"bn": True}),
    (3, 64, 30, 30, 64, 1, 1, A.RELU, {"pad_in": 2, "pad_out": 4}),   # wider halo than needed
    # degenerate and ragged shapes
    (3, 1, 1, 1, 1, 1, 1, A.NONE, {}),              # one pixel, one channel
    (1, 1, 5, 7, 1, 1, 1, A.RELU, {}),
    (3, 5, 2, 3, 7, 1, 1, A.RELU, {"bn": True}),
    (3, 33, 9, 11, 33, 1, 1, A.RELU, {"residual": (A.NONE, False)}),   # channel counts one past a multiple of 32
    (5, 1000, 3, 3, 17, 1, 1, A.NONE, {}),
    (11, 8, 24, 24, 8, 1, 1, A.NONE, {}),           # largest kernel of the reference's shader set is 9x9; 11x11 still fits the step table
    (3, 16, 31, 29, 16, 2, 1, A.RELU, {}),          # odd size with stride 2 (output = floor(size / 2))
    (9, 3, 5, 6, 32, 1, 1, A.RELU, {}),             # wide-kernel path on images narrower than the kernel
    (9, 3, 12, 3, 32, 1, 1, A.NONE, {}),
    (7, 2, 3, 40, 16, 1, 1, A.RELU, {"bn": True}),
    (5, 64, 9, 9, 3, 2, 2, A.NONE, {}),             # stride and dilation together on a 3-channel input
    # strided pointwise layers (staged from the sub-sampled frame): odd sizes, stride 3, few channels, padded input, shallow
    (1, 24, 31, 29, 16, 2, 1, A.RELU, {}),
    (1, 8, 17, 23, 3, 2, 1, A.NONE, {}),
    (1, 40, 20, 21, 64, 3, 1, A.RELU, {"bn": True}),
    (1, 128, 28, 28, 96, 2, 1, A.RELU, {"pad_in": 1, "pad_out": 1, "residual": (A.RELU, True)}),
    (1, 16, 15, 18, 8, 2, 1, A.RELU, {"deep": False}),
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "k%d_%dx%dx%d_to%d_s%d_d%d" % (c[0], c[4], c[2], c[3], c[1], c[5], c[6]))
def test_conv_parity(case, storage):
    k, cout, h, w, cin, stride, dil, act, kw = case
    b = conv_builder(k, cout, h, w, cin, stride, dil, act, **kw)
    bn = kw.get("bn", False)
    wts = conv_block(100 + k, cout, k, cin, bn=bn)
    x = prng.uniform(7 * k + cin, (cin, h, w), -1, 1)
    inputs = [x]
    if "residual" in kw:
        inputs.append(prng.uniform(9, (cout, h // stride, w // stride), -1, 1))
    print("case", case, "storage", storage, flush=True)
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert got.shape == ref.shape
    assert err <= TOL[storage], info


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("k,cin,cout,size,ksplit,kcmax,kw", [
    (1, 512, 128, 14, 4, 128, {"bn": True}),                                   # 128-channel chunks, 4 slices
    (1, 192, 64, 9, 2, 128, {}),                                               # ragged last chunk (192 = 128 + 64)
    (3, 256, 256, 7, 8, 32, {"bn": True, "residual": (A.RELU, True)}),         # residual applied by the reduce pass
    (3, 96, 40, 13, 3, 32, {}),                                                # uneven slices (3 chunks over 3), cout not a tile multiple
    (1, 320, 100, 7, 1, 128, {}),                                              # wide chunks without split-K
])
def test_split_k_and_wide_chunks(k, cin, cout, size, ksplit, kcmax, kw, storage, monkeypatch):
    """The split-K path (partial sums + reduce pass) and the 64/128-channel chunk variants, forced through the
    engine's test switches instead of left to the tuner."""
    monkeypatch.setenv("FYNHIP_FORCE_KSPLIT", str(ksplit))
    monkeypatch.setenv("FYNHIP_CONV_KC_MAX", str(kcmax))
    b = conv_builder(k, cout, size, size, cin, 1, 1, A.RELU, **kw)
    wts = conv_block(300 + k + cin, cout, k, cin, bn=kw.get("bn", False))
    x = prng.uniform(11 * k + cin, (cin, size, size), -1, 1)
    inputs = [x]
    if "residual" in kw:
        inputs.append(prng.uniform(19, (cout, size, size), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    if ksplit > 1:
        assert "ksplit=%d" % ksplit in info
    assert err <= TOL[storage], info


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("tile", ["1,1,1,1", "1,1,2,1", "1,1,1,2"], ids=["32x32", "64x32", "32x64"])
@pytest.mark.parametrize("k,cin,cout,h,w,ksplit,kw", [
    (1, 512, 96, 7, 7, 0, {"bn": True}),                                        # 128-channel chunks, two steps per wave group
    (3, 64, 40, 14, 14, 0, {"bn": True, "residual": (A.RELU, True)}),           # 18 steps padded to a multiple of 8 (or 4)
    (1, 160, 33, 9, 5, 0, {}),                                                  # ragged last chunk, ragged channels and tile
    (3, 256, 64, 7, 7, 4, {"residual": (A.NONE, False)}),                       # together with split-K over workgroups
    (5, 32, 8, 20, 12, 0, {}),
])
def test_tiles_whose_waves_split_k(k, cin, cout, h, w, ksplit, kw, tile, storage, monkeypatch):
    """Small tiles (one or two 32x32 sub-tiles) whose remaining waves split the k16 steps of each chunk and add
    their partial sums in LDS; forced through the engine's tile switch."""
    monkeypatch.setenv("FYNHIP_CONV_TILE", tile)
    if ksplit:
        monkeypatch.setenv("FYNHIP_FORCE_KSPLIT", str(ksplit))
    b = conv_builder(k, cout, h, w, cin, 1, 1, A.RELU, **kw)
    wts = conv_block(500 + k + cin, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(13 * k + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(23, (cout, h, w), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    fm, fn, wm, wn = (int(v) for v in tile.split(","))
    assert "tile=%dx%d" % (32 * fm * wm, 32 * fn * wn) in info and "waves=%dx%d" % (wm, wn) in info
    if ksplit:
        assert "ksplit=%d" % ksplit in info
    assert err <= TOL[storage], info


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("tile", ["1,1,1,1", "1,1,2,1", "1,1,1,2"], ids=["32x32", "64x32", "32x64"])
@pytest.mark.parametrize("kc", [256, 512, 1024])
@pytest.mark.parametrize("cin,cout,h,w,stride,ksplit,kw", [
    (1024, 96, 7, 7, 1, 0, {"bn": True}),                                   # whole chunks
    (600, 33, 9, 5, 1, 0, {"residual": (A.RELU, True)}),                    # ragged last chunk, ragged channels and tile
    (1100, 40, 14, 14, 2, 0, {"bn": True}),                                 # stride 2, more than one chunk at every width
    (2048, 64, 7, 7, 1, 2, {"residual": (A.NONE, False)}),                  # together with split-K over workgroups
], ids=["1024ch", "600ch_ragged", "1100ch_s2", "2048ch_ksplit"])
def test_wide_chunks_on_pointwise_layers(cin, cout, h, w, stride, ksplit, kw, kc, tile, storage, monkeypatch):
    """1x1 convolutions over many input channels staged 256 to 1024 channels at a time (the tiles whose waves split
    K), forced through the engine's tile and chunk-width switches."""
    monkeypatch.setenv("FYNHIP_CONV_TILE", tile)
    monkeypatch.setenv("FYNHIP_CONV_KC", str(kc))
    if ksplit:
        monkeypatch.setenv("FYNHIP_FORCE_KSPLIT", str(ksplit))
    b = conv_builder(1, cout, h, w, cin, stride, 1, A.RELU, **kw)
    wts = conv_block(700 + cin, cout, 1, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(17 + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(29, (cout, (h + stride - 1) // stride, (w + stride - 1) // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    fm, fn, wm, wn = (int(v) for v in tile.split(","))
    planes, buffers = (2 if storage == fa.STORAGE_F32 else 1), (2 if cin > kc else 1)
    if stride == 1 and 1024 + buffers * planes * 32 * fn * wn * (2 * kc + 16) <= 150 * 1024:   # the chunk fits in LDS
        assert "kc=%d" % kc in info and "waves=%dx%d" % (wm, wn) in info
    assert err <= TOL[storage], info


WIDE_CASES = [
    # k, cout, h, w, cin, kwargs: few output channels under a wide kernel (the kx taps become output channels)
    (9, 3, 40, 56, 32, {}),
    (9, 3, 70, 200, 32, {"residual": (A.NONE, False), "pad_out": 1}),      # 64-column tiles, residual, padded output
    (7, 4, 33, 47, 24, {"bn": True, "residual": (A.RELU, True)}),
    (5, 2, 19, 90, 40, {"bn": True}),
    (3, 1, 25, 31, 64, {}),                                                 # two channel chunks
    (9, 3, 12, 3, 32, {}),                                                  # narrower than the kernel: no tile is wide enough
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("two_pass", [False, True], ids=["one_launch", "two_pass"])
@pytest.mark.parametrize("case", WIDE_CASES, ids=lambda c: "k%d_%dx%dx%d_to%d" % (c[0], c[4], c[2], c[3], c[1]))
def test_wide_kernel_few_output_channels(case, two_pass, storage, monkeypatch):
    """Both forms of the folded-kx convolution: partial sums summed inside the workgroup (one launch) and written out
    and summed by a second pass."""
    k, cout, h, w, cin, kw = case
    monkeypatch.setenv("FYNHIP_NO_FUSED_WIDE_CONV" if two_pass else "FYNHIP_FORCE_FUSED_WIDE_CONV", "1")   # (else: whichever is faster)
    monkeypatch.setenv("FYNHIP_NO_ROWS_WIDE_CONV", "1")   # (the third form has a test of its own)
    b = conv_builder(k, cout, h, w, cin, 1, 1, A.RELU, **kw)
    wts = conv_block(800 + k, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(31 * k + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(37, (cout, h, w), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert "wide-kernel" in info
    one_launch = "summed in the epilogue" in info
    assert one_launch == (not two_pass and w + k - 1 > 16)
    assert err <= TOL[storage], info


ROWS_CASES = WIDE_CASES[:3] + [
    (9, 3, 37, 113, 16, {"bn": True}),                                       # one k16 step per input row, ragged strips and rounds
    (9, 3, 5, 60, 32, {"residual": (A.RELU, False)}),                        # fewer rows than one round of a full block
    (9, 3, 300, 130, 32, {}),                                                # several row blocks per strip
    (3, 4, 21, 64, 8, {}),
    (5, 3, 44, 71, 24, {"pad_out": 2}),
]


@pytest.mark.parametrize(*combos(
    # (the shallow variant is run on the plain cases)
    lambda case, shallow, storage: not (shallow and ("residual" in case[5] or "pad_out" in case[5])),
    case=(ROWS_CASES, lambda c: "k%d_%dx%dx%d_to%d" % (c[0], c[4], c[2], c[3], c[1])), shallow=SHALLOW_AXIS, storage=STORAGE_AXIS))
def test_wide_kernel_row_rolling_form(case, shallow, storage, monkeypatch):
    """The folded-kx convolution with the input rows rolled through an LDS ring and the weights held in registers."""
    k, cout, h, w, cin, kw = case
    monkeypatch.setenv("FYNHIP_FORCE_ROWS_WIDE_CONV", "1")
    if shallow:   # unpadded shallow input: the sampler repeats the edge
        kw = dict(kw, deep=False, pad_in=0)
    b = conv_builder(k, cout, h, w, cin, 1, 1, A.RELU, **kw)
    wts = conv_block(900 + k, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(41 * k + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(43, (cout, h, w), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    # (fp32 tensors: the correction terms of the operand split run as fp8 MFMAs on 32-channel rows)
    fp8_form = storage == fa.STORAGE_F32 and cin > 16
    assert ("conv_rows f16+fp8-split" if fp8_form else ("conv_rows f16x2-split" if storage == fa.STORAGE_F32 else "conv_rows f16 ")) in info
    assert err <= TOL[storage], info
    if fp8_form and not shallow:
        monkeypatch.setenv("FYNHIP_EXACT_SPLIT", "1")   # three fp16 passes
        b2 = conv_builder(k, cout, h, w, cin, 1, 1, A.RELU, **kw)
        exact, info2 = run_single(b2, storage, inputs, wts)
        assert "conv_rows f16x2-split" in info2
        assert rel_l2(exact, ref) <= 2e-6, info2
        assert rel_l2(got, exact) <= 3e-5


P16_CASES = [
    # (cin, cout, h, w, stride, tile "h,w,channel groups", kw)  -- h, w: input size
    (128, 128, 16, 20, 1, "8,10,4", {}),                                           # whole tiles
    (128, 128, 19, 23, 1, "8,10,4", {"bn": True, "residual": (A.RELU, True)}),     # ragged in both directions
    (64, 128, 9, 7, 1, "8,8,4", {"residual": (A.NONE, False)}),                    # two chunks, one partial tile
    (192, 256, 13, 30, 1, "8,6,4", {"bn": True}),                                  # six chunks, two blocks of output channels
    (128, 128, 11, 17, 1, "4,8,4", {"pad_out": 2}),
    (64, 128, 6, 5, 1, "4,4,4", {"residual": (A.RELU, False)}),
    (128, 128, 30, 41, 1, None, {"residual": (A.NONE, False)}),                    # the engine's own choice of tile
    (96, 128, 21, 18, 1, "10,8,4", {"bn": True}),                                  # three chunks: a pair and an odd one
    (32, 128, 12, 9, 1, "8,8,4", {"residual": (A.RELU, True), "bn": True}),        # a single chunk (one staging buffer)
    (64, 128, 40, 34, 2, "10,8,4", {"bn": True}),                                  # stride 2: even/odd column halves
    (64, 128, 26, 44, 2, "8,10,4", {"pad_out": 1}),
    (96, 256, 18, 30, 2, "8,8,4", {}),
    (32, 64, 50, 46, 2, "8,6,2", {"bn": True}),                                    # two channel groups x two tiles side by side
    (32, 64, 22, 70, 2, "4,8,2", {"pad_out": 1}),
    (64, 192, 34, 20, 2, "8,4,2", {}),
    (64, 128, 70, 71, 1, "4,4,4", {"bn": True, "residual": (A.RELU, False)}),      # 324 tiles: workgroups walk two tiles, residual tile per tile
    (32, 128, 66, 68, 1, "4,4,4", {"residual": (A.NONE, True), "bn": True}),       # one chunk and a residual input: one workgroup per tile
    (32, 64, 150, 130, 2, "4,8,2", {"bn": True}),                                  # one chunk, 380 tiles: a stage per tile, weight ring wraps
    (96, 128, 82, 66, 2, "8,8,4", {"pad_out": 1}),                                 # three chunks per tile, odd stage count per tile
    (64, 64, 40, 37, 1, "8,8,2", {"bn": True, "residual": (A.RELU, True)}),        # stride 1, 64-channel blocks: two tiles side by side
    (32, 192, 21, 50, 1, "8,6,2", {}),
    (64, 64, 90, 100, 1, "4,8,2", {"residual": (A.NONE, False)}),                  # 161 tiles x 1 block
    (64, 64, 256, 256, 1, None, {}),                                               # BASELINE's single-layer case
    # channel counts that are not whole chunks / blocks: zeros behind the input's pitch, nothing stored behind the output's
    (40, 40, 21, 26, 1, "8,8,2", {"bn": True, "residual": (A.RELU, True)}),         # the residual layers of the reference's sample style nets, reduced
    (40, 40, 39, 32, 1, None, {"residual": (A.NONE, False)}),
    (24, 72, 30, 22, 2, "8,6,2", {"bn": True}),                                    # one ragged chunk; the second block of 64 output channels holds 8
    (72, 136, 17, 19, 1, "8,8,2", {"residual": (A.NONE, False)}),                  # three chunks, the last with 8 channels; three blocks of output channels
    (48, 200, 20, 20, 1, "4,8,2", {"pad_out": 1}),
    (20, 40, 38, 44, 2, "8,6,2", {"bn": True}),                                    # fewer channels than the tensors' pitch (conv3 and conv2 of those nets)
    (12, 20, 50, 36, 2, "4,8,2", {}),
    (44, 48, 23, 19, 1, "8,8,2", {"residual": (A.RELU, False)}),
]


def _p16_runs(case, act, shallow, storage):
    cin, cout, h, w, stride, tile, kw = case
    if shallow and ("residual" in kw or "pad_out" in kw):
        return False   # the shallow variant is run on the plain cases
    if act is not A.RELU and ("pad_out" in kw or tile in ("4,4,4", "8,6,4", "8,8,4", "8,4,2", "4,8,2") or h > 60):
        return False   # activations are varied on some of the cases
    return not (storage == fa.STORAGE_F16 and (act is A.NONE or (shallow and h > 30)))   # fp16 storage on some of the combinations


@pytest.mark.parametrize(*combos(_p16_runs, case=(P16_CASES, lambda c: "%dx%dx%d_to%d_s%d_%s" % (c[0], c[2], c[3], c[1], c[4], (c[5] or "auto").replace(",", "x"))),
                                 act=ACT3_AXIS, shallow=SHALLOW_AXIS, storage=STORAGE_AXIS))
def test_sixteen_position_fragment_form(case, act, shallow, storage, monkeypatch):
    """The 3x3 convolution on 16-position fragments: every compiled tile, ragged edges, the residual tile through LDS;
    fp32 storage (operand split, value ranges on both sides) and fp16 storage (one plane, one pass)."""
    cin, cout, h, w, stride, tile, kw = case
    if storage == fa.STORAGE_F16:
        monkeypatch.setenv("FYNHIP_NO_H16_CONV", "1")   # (the form with 64-channel wave tiles has its own test)
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    if tile:
        monkeypatch.setenv("FYNHIP_P16_TILE", tile)
    if shallow:
        kw = dict(kw, deep=False, pad_in=0)
    if act is A.LEAKY_RELU:
        kw = dict(kw, leak=0.1)
    b = conv_builder(3, cout, h, w, cin, stride, 1, act, **kw)
    wts = conv_block(1000 + cin, cout, 3, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(47 * cin + h, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(53, (cout, h // stride, w // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    # (fp32 tensors: the correction terms of the operand split run as fp8 MFMAs where the 32-channel chunks pair up)
    assert ("conv_p16 f16+fp8-split" if ((cin + 31) // 32) % 2 == 0 else "conv_p16 f16x2-split") in info if storage == fa.STORAGE_F32 else "conv_p16 f16 " in info
    if tile:
        th, tw, wm = tile.split(",")
        assert "waves=%sx" % wm in info and "th=%s tw=%s" % (th, tw) in info
    assert err <= TOL[storage], info
    if storage == fa.STORAGE_F32 and cin % 64 == 0 and act is A.RELU and not shallow:
        # the same layer with three fp16 passes (22-bit operands): fp32-class agreement with the oracle, and the two
        # forms agree to what four-bit correction terms leave (2^-11 * 2^-4 of the result, measured 1e-5)
        monkeypatch.setenv("FYNHIP_EXACT_SPLIT", "1")
        b2 = conv_builder(3, cout, h, w, cin, stride, 1, act, **kw)
        exact, info2 = run_single(b2, storage, inputs, wts)
        assert "conv_p16 f16x2-split" in info2
        assert rel_l2(exact, ref) <= 2e-6, info2
        assert rel_l2(got, exact) <= 3e-5


H16_CASES = [
    # (k, cin, cout, h, w, tile "h,w", kw)
    (9, 64, 128, 30, 40, "12,8", {}),                                              # two chunks, ragged in both directions
    (9, 128, 128, 25, 33, "8,8", {"bn": True, "residual": (A.RELU, True)}),
    (9, 64, 256, 14, 20, "4,8", {"residual": (A.NONE, False)}),                    # two blocks of output channels
    (9, 96, 128, 24, 32, "12,8", {"bn": True, "pad_out": 2}),                      # whole tiles, three chunks
    (9, 64, 128, 130, 150, "4,8", {"bn": True, "residual": (A.RELU, False)}),      # 330 tiles: workgroups walk two tiles
    (9, 128, 128, 60, 70, None, {"residual": (A.NONE, False)}),                    # the engine's own choice of tile
    (3, 128, 128, 40, 50, "12,8", {"bn": True, "residual": (A.NONE, True)}),
    (3, 64, 128, 150, 130, "4,8", {"pad_out": 1}),                                 # 342 tiles
    (3, 32, 128, 66, 68, "4,8", {"residual": (A.RELU, True), "bn": True}),         # one chunk and a residual input: one workgroup per tile
    (3, 32, 128, 150, 140, "4,8", {"bn": True}),                                   # one chunk, tiles walked: a stage per tile
    (3, 96, 384, 19, 23, "8,8", {}),                                               # three blocks of output channels
    # two bands of rows with different tile heights (two launches): "h,w;rows of the first band,h of the second"
    (9, 64, 128, 44, 30, "12,8;24,8", {"bn": True, "residual": (A.RELU, True)}),
    (3, 128, 128, 37, 50, "8,8;32,4", {"residual": (A.NONE, False), "pad_out": 1}),
    (9, 64, 128, 21, 18, "4,8;12,12", {}),
]


def _h16_runs(case, act, shallow):
    k, cin, cout, h, w, tile, kw = case
    if shallow and ("residual" in kw or "pad_out" in kw or h > 100):
        return False   # the shallow variant is run on the plain cases
    return not (act is not A.RELU and ("pad_out" in kw or h > 100 or cout > 128))   # activations are varied on some of the cases


@pytest.mark.parametrize(*combos(_h16_runs, case=(H16_CASES, lambda c: "k%d_%dx%dx%d_to%d_%s" % (c[0], c[1], c[3], c[4], c[2], (c[5] or "auto").replace(",", "x").replace(";", "_"))),
                                 act=ACT3_AXIS, shallow=SHALLOW_AXIS))
def test_fp16_sixteen_position_fragment_form(case, act, shallow, monkeypatch):
    """The 3x3 / 9x9 convolution between wide fp16 tensors on 16-position fragments: every compiled tile, ragged edges,
    tile walking, the residual tile through LDS."""
    k, cin, cout, h, w, tile, kw = case
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    split = None
    if tile and ";" in tile:
        tile, split = tile.split(";")
        monkeypatch.setenv("FYNHIP_H16_SPLIT", split)
    if tile:
        monkeypatch.setenv("FYNHIP_P16_TILE", tile)
    if shallow:
        kw = dict(kw, deep=False, pad_in=0)
    if act is A.LEAKY_RELU:
        kw = dict(kw, leak=0.1)
    b = conv_builder(k, cout, h, w, cin, 1, 1, act, **kw)
    wts = conv_block(2000 + cin + k, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(43 * cin + h, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(59, (cout, h, w), -1, 1))
    got, info = run_single(b, fa.STORAGE_F16, inputs, wts)
    ref = oracle_single(b, fa.STORAGE_F16, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert "conv_h16" in info
    if tile:
        th, tw = tile.split(",")
        assert "th=%s tw=%s" % (th, tw) in info
    if split:
        rows1, th2 = split.split(",")
        assert "second launch from row %s: th=%s" % (rows1, th2) in info
    assert err <= TOL[fa.STORAGE_F16], info


KR16_CASES = [
    # (k, cin, cout, h, w, fragments per block, kw)
    (1, 1024, 256, 14, 14, 1, {}),                                              # a ResNet stage-3 reduction layer
    (1, 1024, 64, 7, 9, 2, {"bn": True, "residual": (A.RELU, True)}),           # ragged tiles, residual read in the epilogue
    (1, 256, 48, 5, 6, 1, {"pad_out": 1}),                                      # two chunks per wave
    (1, 512, 32, 13, 3, 2, {"bn": True}),
    (3, 256, 256, 14, 14, 2, {"bn": True}),                                     # a ResNet stage-3 3x3 layer
    (3, 512, 32, 7, 7, 1, {"residual": (A.NONE, False)}),
    (3, 256, 48, 9, 6, 1, {"pad_out": 2, "bn": True}),
    (3, 512, 64, 18, 30, 2, {}),                                                # 40 tiles x 2 blocks
    (1, 128, 96, 11, 10, 2, {"bn": True, "residual": (A.NONE, False)}),         # one chunk per wave: a single step
    (3, 128, 128, 28, 28, 1, {"bn": True}),                                     # one chunk per wave, nine steps
    (1, 256, 64, 22, 30, 1, {"stride": 2, "bn": True}),                         # stride 2: positions read every other pixel
    (1, 512, 128, 13, 15, 2, {"stride": 2, "residual": (A.RELU, True)}),        # odd input size with stride 2
    # channel counts that are no multiple of 128: the chunk count is rounded up to four per wave, the rest reads as zero
    (1, 64, 256, 20, 20, 2, {"bn": True}),
    (1, 96, 48, 9, 9, 1, {}),
    (1, 160, 32, 7, 7, 2, {"residual": (A.NONE, False)}),
    (1, 320, 64, 7, 7, 1, {"bn": True}),                                        # 10 -> 12 chunks
    (1, 576, 96, 14, 14, 2, {}),                                                # 18 -> 20 chunks
    (1, 24, 144, 10, 12, 1, {"bn": True}),                                      # less than one chunk
    (3, 64, 64, 12, 12, 1, {"bn": True, "residual": (A.RELU, True)}),
    (1, 2048, 64, 7, 7, 1, {"bn": True}),                                       # 64 chunks: unpadded pixel pitch in LDS
    (1, 2048, 32, 5, 9, 2, {}),
    # output channel counts that are no multiple of the block: the last block is partly empty
    (1, 96, 24, 20, 20, 1, {"bn": True}),
    (1, 64, 20, 8, 8, 1, {"residual": (A.RELU, True)}),                         # 20 channels in a pitch of 24
    (1, 128, 56, 7, 7, 2, {"bn": True, "residual": (A.NONE, False)}),
    (3, 128, 40, 10, 9, 1, {}),
    # larger tiles (fragments per block, tile h, tile w)
    (1, 64, 256, 56, 56, "2,8,8", {"bn": True}),
    (1, 256, 64, 30, 44, "1,4,8", {"residual": (A.RELU, True)}),
    (3, 64, 64, 29, 35, "2,8,8", {"bn": True, "residual": (A.NONE, False)}),
    (3, 96, 48, 20, 12, "1,4,8", {"pad_out": 1}),
    (1, 24, 144, 56, 56, "1,8,8", {}),
    # 3x3 with stride 2: a window of 9x9 pixels per chunk under a tile of 4x4 positions
    (3, 128, 128, 56, 56, 1, {"stride": 2, "bn": True}),                        # the first 3x3 layer of ResNet's stage 2
    (3, 256, 64, 28, 28, 2, {"stride": 2}),
    (3, 256, 48, 13, 15, 1, {"stride": 2, "bn": True, "residual": (A.RELU, True)}),   # odd input size
    (3, 64, 32, 10, 22, 2, {"stride": 2, "pad_out": 1}),
    (3, 512, 32, 14, 14, 2, {"stride": 2}),                                     # 16 chunks: in fp32 in two rounds through the LDS
    (3, 512, 64, 15, 13, 1, {"stride": 2, "bn": True, "residual": (A.RELU, True)}),
    # reductions in two rounds through the LDS
    (3, 1024, 32, 7, 7, 1, {"bn": True}),
    (3, 1024, 64, 6, 9, 2, {"residual": (A.NONE, False)}),
    (1, 4096, 32, 5, 6, 2, {"bn": True}),
    (1, 4096, 48, 7, 7, 1, {"residual": (A.RELU, True)}),
]


def _kr16_runs(case, act, shallow, storage):
    k, cin, cout, h, w, fm, kw = case
    if shallow and (k == 1 or "residual" in kw or "pad_out" in kw):
        return False   # the shallow variant is run on the plain 3x3 cases
    return not (act is A.LEAKY_RELU and (cin > 512 or "pad_out" in kw))   # activations are varied on some of the cases


@pytest.mark.parametrize(*combos(_kr16_runs, case=(KR16_CASES, lambda c: "k%d_%dx%dx%d_to%d_fm%s%s" % (c[0], c[1], c[3], c[4], c[2], str(c[5]).replace(",", "x"), "_s2" if c[6].get("stride") == 2 else "")),
                                 act=([A.RELU, A.LEAKY_RELU], lambda a: "relu" if a is A.RELU else "leaky"), shallow=SHALLOW_AXIS, storage=STORAGE_AXIS))
def test_reduction_resident_form(case, act, shallow, storage, monkeypatch):
    """1x1 / 3x3 convolutions on few positions and many input channels with a tile's whole reduction resident in LDS and
    the four MFMA waves of a workgroup splitting the chunks."""
    k, cin, cout, h, w, fm, kw = case
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV", "1")
    monkeypatch.setenv("FYNHIP_KR16_FM", str(fm))
    if shallow:
        kw = dict(kw, deep=False, pad_in=0)
    if act is A.LEAKY_RELU:
        kw = dict(kw, leak=0.1)
    kw = dict(kw)
    stride = kw.pop("stride", 1)
    b = conv_builder(k, cout, h, w, cin, stride, 1, act, **kw)
    wts = conv_block(3000 + cin + k, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(41 * cin + h, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(67, (cout, h // stride, w // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    if isinstance(fm, str):
        f, th, tw = (int(v) for v in fm.split(","))
        assert "conv_kr16" in info and "tile=%dx%d" % (16 * f, th * tw) in info
    else:
        assert "conv_kr16" in info and "tile=%dx16" % (16 * fm) in info
    assert err <= TOL[storage], info


D16_CASES = [
    # (cin, cout, h, w, kw)
    (16, 96, 112, 112, {"bn": True}),                                            # an expand layer at the largest resolution
    (32, 16, 56, 60, {"residual": (A.NONE, False)}),
    (24, 144, 28, 31, {"bn": True, "pad_out": 1}),                               # 24 channels in a chunk of 32; positions no multiple of 16
    (96, 24, 37, 29, {"bn": True, "residual": (A.RELU, True)}),                  # three chunks, 24 output channels (second fragment half empty)
    (144, 40, 20, 20, {}),                                                       # five chunks
    (192, 64, 37, 45, {"stride": 2, "bn": True}),                                # six chunks, step 2 on an odd-sized input
    (64, 256, 56, 56, {"bn": True, "residual": (A.NONE, False)}),                # ResNet stage 1: 16 fragments, four per wave
    (256, 64, 40, 40, {"stride": 2}),                                            # eight chunks
    (8, 12, 40, 40, {}),                                                         # a quarter of a chunk, 12 output channels
    (32, 320, 24, 24, {"bn": True}),                                             # 20 fragments: five per wave, one ahead of their use
    # the fragments of output channels dealt to two or four workgroups per 16 positions
    (64, 256, 28, 28, {"bn": True, "residual": (A.RELU, True), "blocks": 2}),
    (32, 320, 24, 24, {"blocks": 4}),
    (96, 24, 30, 30, {"blocks": 2}),                                             # more waves than fragments
    # a wave per 16 positions and fragment (layers with up to four fragments of output channels)
    (32, 16, 56, 60, {"residual": (A.NONE, False), "blocks": -1}),
    (96, 24, 37, 29, {"bn": True, "blocks": -2}),
    (144, 40, 20, 20, {"blocks": -3}),
]


@pytest.mark.parametrize(*combos(
    # (activation and the shallow variant are varied on the plain cases)
    lambda case, variant, storage: variant == "relu" or not ("residual" in case[4] or "pad_out" in case[4] or "blocks" in case[4] or case[0] > 100),
    case=(D16_CASES, lambda c: "%dx%dx%d_to%d%s%s" % (c[0], c[2], c[3], c[1], "_s2" if c[4].get("stride") == 2 else "", ("_b%d" % c[4]["blocks"]).replace("-", "w") if "blocks" in c[4] else "")),
    variant=(["relu", "leaky", "shallow"], str), storage=STORAGE_AXIS))
def test_pointwise_without_lds(case, variant, storage, monkeypatch):
    """1x1 convolutions on many positions whose B fragments come straight from the tensor: a workgroup of four waves per
    16 positions, the waves sharing the fragments of output channels."""
    cin, cout, h, w, kw = case
    monkeypatch.setenv("FYNHIP_FORCE_D16_CONV", "1")
    kw = dict(kw)
    stride = kw.pop("stride", 1)
    blocks = kw.pop("blocks", None)
    if blocks:
        monkeypatch.setenv("FYNHIP_D16_BLOCKS", str(blocks))
    if variant == "shallow":
        kw.update(deep=False, pad_in=0)
    act = A.LEAKY_RELU if variant == "leaky" else A.RELU
    if variant == "leaky":
        kw["leak"] = 0.1
    b = conv_builder(1, cout, h, w, cin, stride, 1, act, **kw)
    wts = conv_block(5000 + cin + cout, cout, 1, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(43 * cin + h, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(71, (cout, h // stride, w // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert "conv_d16" in info and (not blocks or ("%d workgroup(s)" % blocks if blocks > 0 else "a wave per 16 positions") in info)
    assert err <= TOL[storage], info


SMALL_INPUT_CASES = [
    # (k, cin, cout, h, w, stride, kw)
    (3, 3, 32, 224, 224, 2, {"bn": True}),                      # the first layer of the MobileNetV2-style stack
    (7, 3, 64, 64, 72, 2, {"bn": True}),                        # a ResNet stem, reduced
    (5, 4, 24, 40, 36, 1, {"pad_out": 1}),                      # four channels, 24 output channels
    (3, 1, 16, 33, 47, 1, {"residual": (A.RELU, True)}),        # one channel, odd size, residual
    (7, 2, 40, 50, 50, 1, {"bn": True, "blocks": -3}),          # a wave per 16 positions and fragment
    (3, 3, 96, 40, 40, 2, {"blocks": 2}),                       # six fragments on two workgroups per tile
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("act", [A.NONE, A.LEAKY_RELU], ids=["linear", "leaky"])
@pytest.mark.parametrize("case", SMALL_INPUT_CASES, ids=lambda c: "k%d_%dx%dx%d_to%d_s%d" % (c[0], c[1], c[3], c[4], c[2], c[5]))
def test_small_input_convolution_without_lds(case, act, storage, monkeypatch):
    """K x K convolutions (3, 5, 7) on at most four input channels whose B fragments are gathered from the image, two
    taps of four channels per lane and step."""
    k, cin, cout, h, w, stride, kw = case
    monkeypatch.setenv("FYNHIP_FORCE_D16_CONV", "1")
    kw = dict(kw)
    blocks = kw.pop("blocks", None)
    if blocks:
        monkeypatch.setenv("FYNHIP_D16_BLOCKS", str(blocks))
    if act is A.LEAKY_RELU:
        kw["leak"] = 0.1
    b = conv_builder(k, cout, h, w, cin, stride, 1, act, **kw)
    wts = conv_block(6000 + k * cin + cout, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(47 * cin + h, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(73, (cout, h // stride, w // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert "conv_d16" in info and "KxK" in info
    assert err <= TOL[storage], info


ALL_TILES = ["2,2,2,2", "2,2,1,4", "2,1,2,2", "2,1,1,4", "1,2,1,4", "1,1,1,4", "1,1,4,1", "1,1,2,2", "1,2,4,1", "1,3,4,1", "1,4,4,1",
             "1,2,2,2", "1,4,2,2", "1,3,2,2", "1,4,1,4", "1,3,1,4", "1,1,1,1", "1,1,2,1", "1,1,1,2"]


# Combinations for which the engine has no such tile and says so: the halo tile of the widest shape (32 x 512 positions)
# in two fp32 operand planes is more than a CU's LDS (for the 5x5 kernel with step 2 also the next narrower), and the
# tiles whose waves split the reduction exist for chunks of 32 channels and more.
NO_SUCH_TILE = {(kk, "1,4,1,4", fa.STORAGE_F32) for kk in (3, 1, 5)} | {(5, "1,3,1,4", fa.STORAGE_F32)} | \
               {(5, t, st) for t in ("1,1,1,1", "1,1,2,1", "1,1,1,2") for st in (fa.STORAGE_F32, fa.STORAGE_F16)}


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("tile", ALL_TILES)
@pytest.mark.parametrize("k,cin,cout,h,w,stride,kw", [
    (3, 64, 40, 20, 24, 1, {"bn": True, "residual": (A.RELU, True)}),
    (1, 160, 24, 9, 13, 1, {}),
    (5, 16, 130, 12, 10, 2, {"bn": True}),
], ids=["k3_res", "k1_wide_chunks", "k5_s2_16ch"])
def test_every_tile_shape(k, cin, cout, h, w, stride, kw, tile, storage, monkeypatch):
    """Every workgroup shape of the convolution kernel (fragments per wave x wave arrangement), forced through the
    engine's tile switch: the tuner only ever picks a few of them for a given layer."""
    monkeypatch.setenv("FYNHIP_CONV_TILE", tile)
    b = conv_builder(k, cout, h, w, cin, stride, 1, A.RELU, **kw)
    wts = conv_block(600 + k + cin, cout, k, cin, bn=kw.get("bn", False))
    inputs = [prng.uniform(15 * k + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(27, (cout, h // stride, w // stride), -1, 1))
    if (k, tile, storage) in NO_SUCH_TILE:
        with pytest.raises(fa.FynException, match="no MFMA tile configuration fits"):
            run_single(b, storage, inputs, wts)
        return
    got, info = run_single(b, storage, inputs, wts)
    fm, fn, wm, wn = (int(v) for v in tile.split(","))
    assert "tile=%dx%d" % (32 * fm * wm, 32 * fn * wn) in info and "waves=%dx%d" % (wm, wn) in info
    err = rel_l2(got, oracle_single(b, storage, inputs, wts))
    assert err <= TOL[storage], info


def test_kernel_too_large_for_the_step_table_is_rejected():
    # 13x13 on 32 channels = 338 k16 steps per chunk, more than the 256-entry step table
    b = conv_builder(13, 8, 32, 32, 32)
    with pytest.raises(fa.FynException, match="too many kernel taps"):
        run_single(b, fa.STORAGE_F32, [np.zeros((32, 32, 32), np.float32)], conv_block(1, 8, 13, 32))
    with pytest.raises(fa.FynException):          # even kernel sizes do not exist in the reference either
        run_single(conv_builder(4, 8, 16, 16, 8), fa.STORAGE_F32, [np.zeros((8, 16, 16), np.float32)], conv_block(1, 8, 4, 8))


def test_reference_known_answer_patterns_on_gpu():
    # antisymmetric kernel on ones (convlayertests.cpp:242-261) and 1x1 ones (:165-182): exact
    for storage in (fa.STORAGE_F32, fa.STORAGE_F16):
        cin, cout, size = 8, 8, 32
        w = np.zeros((cout, 3, 3, cin), np.float32)
        w[:, 0], w[:, 2] = -1.0, 1.0
        block = np.concatenate([np.zeros(cout, np.float32), w.ravel()])
        got, _ = run_single(conv_builder(3, cout, size, size, cin), storage, [np.ones((cin, size, size), np.float32)], block)
        assert np.all(got[:, 1:size - 1] == 0)
        assert np.all(got[:, 0, 1:size - 1] == 3 * cin) and np.all(got[:, size - 1, 1:size - 1] == -3 * cin)
        block = np.concatenate([np.zeros(16, np.float32), np.ones(16 * 12, np.float32)])
        got, _ = run_single(conv_builder(1, 16, 20, 24, 12), storage, [np.ones((12, 20, 24), np.float32)], block)
        assert np.all(got == 12)


def test_shallow_unpadded_conv_edge_clamps():
    # networktests.cpp:85-97,173-186: shallow 3x3 4->8 @32x32 without padding, zero-sum kernel on ones => 0
    cin, cout = 4, 8
    w = np.zeros((cout, 3, 3, cin), np.float32)
    w[:, 0], w[:, 2] = -1.0, 1.0
    block = np.concatenate([np.zeros(cout, np.float32), w.ravel()])
    b = conv_builder(3, cout, 32, 32, cin, deep=False, pad_in=0)
    got, info = run_single(b, fa.STORAGE_F32, [np.ones((cin, 32, 32), np.float32)], block)
    assert "edge-clamp" in info
    assert np.all(got == 0.0)
    x = prng.uniform(3, (cin, 32, 32), -1, 1)
    wts = conv_block(5, cout, 3, cin)
    got, _ = run_single(b, fa.STORAGE_F32, [x], wts)
    assert rel_l2(got, oracle_single(b, fa.STORAGE_F32, [x], wts)) < 1e-5


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("k,crop,cin,cout,h,w", [(3, 0, 16, 8, 12, 10), (3, 1, 128, 64, 39, 32), (2, 0, 24, 16, 9, 17), (3, 1, 64, 32, 20, 26),
                                                 (3, 0, 1, 1, 1, 1), (2, 0, 3, 5, 1, 2), (3, 1, 7, 33, 2, 3), (3, 0, 40, 3, 5, 1)])
def test_transconv_parity(k, crop, cin, cout, h, w, storage):
    b = fa.ConvLayerBuilder(k, "tconv").type(fa.LayerType.TRANSCONVOLUTION2D).number(1).shape(cout, h, w, cin)
    b.upsample(2).inputPadding(1).outputPadding(1).prefixAct(A.RELU).deep().crop(crop)
    wts = conv_block(31, cout, k, cin)
    x = prng.uniform(32, (cin, h, w), -1, 1)
    print("transconv", k, crop, cin, cout, h, w, storage, flush=True)
    got, info = run_single(b, storage, [x], wts)
    ref = oracle_single(b, storage, [x], wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert got.shape == ref.shape == (cout, 2 * h + k - 2 - crop, 2 * w + k - 2 - crop)
    assert err <= TOL[storage]


C4_CASES = [
    # cin, cout, h, w, tile "h,w", kw
    (3, 32, 40, 56, "8,8", {"bn": True}),            # the style net's first layer, reduced
    (3, 32, 19, 37, "4,8", {}),                      # ragged
    (4, 64, 23, 30, "8,4", {"pad_out": 1}),          # four channels, two blocks of output channels
    (1, 32, 12, 70, "4,8", {"bn": True}),
    (3, 32, 90, 300, "8,8", {}),                     # 360 tiles: workgroups walk
    (3, 32, 33, 50, None, {"pad_out": 2}),
    (3, 12, 30, 70, "8,8", {"bn": True}),            # fewer output channels than a block of 32 (the first layer of the reference's sample style nets)
    (3, 40, 21, 33, "4,8", {}),                      # a second block that holds 8 channels
    (3, 12, 40, 64, "8,8", {"k": 3}),                # 3x3: a stage of three steps, two turns of it in the weight ring
    (4, 32, 19, 37, "4,8", {"k": 3, "bn": True}),
    (3, 24, 50, 41, None, {"k": 3}),
]


@pytest.mark.parametrize(*combos(
    # (the shallow variant is run on the plain cases)
    lambda case, shallow, storage: not (shallow and ("pad_out" in case[5] or case[2] > 60)),
    case=(C4_CASES, lambda c: "%dx%dx%d_to%d_%s" % (c[0], c[2], c[3], c[1], (c[4] or "auto").replace(",", "x"))), shallow=SHALLOW_AXIS, storage=STORAGE_AXIS))
def test_small_input_sixteen_position_fragment_form(case, shallow, storage, monkeypatch):
    """The 9x9 convolution on at most four input channels with two taps of a 4-channel pixel per lane and step."""
    cin, cout, h, w, tile, kw = case
    kw = dict(kw)
    k = kw.pop("k", 9)
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    monkeypatch.setenv("FYNHIP_NO_D16_CONV", "1")   # (the LDS-free form for first layers has its own test)
    if tile:
        monkeypatch.setenv("FYNHIP_P16_TILE", tile)
    if shallow:
        kw = dict(kw, deep=False, pad_in=0)
    b = conv_builder(k, cout, h, w, cin, 1, 1, A.NONE, **kw)
    wts = conv_block(1200 + cin, cout, k, cin, bn=kw.get("bn", False))
    x = prng.uniform(61 * cin + w, (cin, h, w), 0, 1)
    got, info = run_single(b, storage, [x], wts)
    ref = oracle_single(b, storage, [x], wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    # (fp32 tensors: the correction terms of the operand split run as fp8 MFMAs where a stage has an even number of steps)
    assert ("conv_p16c4 f16+fp8-split" if k == 9 else "conv_p16c4 f16x2-split") in info if storage == fa.STORAGE_F32 else "conv_p16c4 f16 " in info
    if tile:
        assert "th=%s tw=%s" % tuple(tile.split(",")) in info
    assert err <= TOL[storage], info
    if storage == fa.STORAGE_F32 and k == 9 and not shallow:
        # the same layer with three fp16 passes: fp32-class agreement with the oracle, and the two forms agree to what
        # four-bit correction terms leave
        monkeypatch.setenv("FYNHIP_EXACT_SPLIT", "1")
        b2 = conv_builder(k, cout, h, w, cin, 1, 1, A.NONE, **kw)
        exact, info2 = run_single(b2, storage, [x], wts)
        assert "conv_p16c4 f16x2-split" in info2
        assert rel_l2(exact, ref) <= 2e-6, info2
        assert rel_l2(got, exact) <= 3e-5


TP16_CASES = [
    # cin, cout, h, w, tile "h,w,channel groups", batch-norm
    (64, 32, 20, 26, "4,8,1", True),        # four tiles of positions side by side, ragged on both sides
    (128, 64, 39, 32, "4,8,2", False),      # the style net's first up-sampling layer, reduced
    (32, 32, 9, 70, "8,4,1", True),         # a single chunk
    (96, 64, 33, 17, "8,4,2", False),       # three chunks
    (64, 96, 7, 11, "2,8,1", True),         # three blocks of output channels
    (64, 128, 21, 40, "2,8,2", False),
    (128, 64, 29, 37, "6,8,2", True),       # three position fragments per wave: weight ring of three steps
    (64, 32, 15, 70, "6,8,1", False),
    (96, 64, 20, 26, "8,6,2", True),
    (64, 32, 80, 150, "4,8,1", True),       # 375 tiles: workgroups walk
    (64, 32, 31, 45, None, False),          # the engine's own choice
]


@pytest.mark.parametrize(*combos(
    # (the activation is varied on the small cases)
    lambda case, act, storage: not (act is A.NONE and (case[4] is None or case[2] > 60 or storage == fa.STORAGE_F16)),
    case=(TP16_CASES, lambda c: "%dx%dx%d_to%d_%s" % (c[0], c[2], c[3], c[1], (c[4] or "auto").replace(",", "x"))),
    act=([A.RELU, A.NONE], lambda a: "relu" if a is A.RELU else "none"), storage=STORAGE_AXIS))
def test_transconv_sixteen_position_fragment_form(case, act, storage, monkeypatch):
    """The doubling transposed 3x3 convolution on 16-position fragments: all four output parities from one staged input
    tile; fp32 and fp16 storage."""
    cin, cout, h, w, tile, bn = case
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    if tile:
        monkeypatch.setenv("FYNHIP_P16_TILE", tile)
    b = fa.ConvLayerBuilder(3, "tconv").type(fa.LayerType.TRANSCONVOLUTION2D).number(1).shape(cout, h, w, cin)
    b.upsample(2).inputPadding(1).outputPadding(2).prefixAct(act).deep().crop(1)
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    wts = conv_block(1100 + cin, cout, 3, cin, bn=bn)
    x = prng.uniform(57 * cin + w, (cin, h, w), -1, 1)
    got, info = run_single(b, storage, [x], wts)
    ref = oracle_single(b, storage, [x], wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    assert "tconv_p16 f16x2-split" in info if storage == fa.STORAGE_F32 else "tconv_p16 f16 " in info
    if tile:
        th, tw, wm = tile.split(",")
        assert "waves=%sx" % wm in info and "th=%s tw=%s" % (th, tw) in info
    assert got.shape == ref.shape == (cout, 2 * h, 2 * w)
    assert err <= TOL[storage], info


FRAC_CASES = [
    # k, cin, cout, h, w, step, stride, pad_in, act, kwargs
    (3, 40, 20, 12, 16, 0.5, 2, 0, A.NONE, {}),                   # deconv1 of the reference's style nets (stylenet3x3.cpp:163)
    (3, 20, 12, 12, 16, 0.25, 2, 0, A.RELU, {}),                  # deconv2 (:167): twice the size
    (3, 12, 3, 24, 32, 0.5, 1, 0, A.RELU, {}),                    # deconv3 (:171)
    (9, 12, 3, 10, 14, 0.5, 1, 0, A.RELU, {}),                    # deconv3 of stylenet9x9.cpp:201
    (5, 7, 9, 6, 5, 0.5, 1, 2, A.LEAKY_RELU, {"bn": True, "leak": 0.2}),
    (7, 4, 8, 5, 9, 0.25, 1, 1, A.CLIP, {"clip": (-0.5, 0.5)}),
    (5, 16, 33, 8, 8, 0.5, 2, 1, A.RELU, {"bn": True, "residual": (A.RELU, True), "pad_out": 2}),
    (3, 5, 4, 3, 2, 0.125, 2, 1, A.NONE, {"residual": (A.NONE, False)}),
    (9, 3, 2, 4, 4, 1.0, 1, 4, A.NONE, {}),                       # step 1: the ordinary convolution
    (3, 1, 1, 1, 1, 0.5, 1, 0, A.NONE, {}),
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", FRAC_CASES, ids=lambda c: "k%d_%dx%dx%d_to%d_step%g_s%d_p%d" % (c[0], c[1], c[3], c[4], c[2], c[5], c[6], c[7]))
def test_fractional_convolution_parity(case, storage, expect="conv_mfma"):
    k, cin, cout, h, w, step, stride, pad_in, act, kw = case
    b = fa.ConvLayerBuilder(k, "fracconv").type(fa.LayerType.FRACCONVOLUTION2D).number(1).shape(cout, h, w, cin)
    b.downsample(stride).sourceStep(step).prefixAct(act).inputPadding(pad_in).outputPadding(kw.get("pad_out", 0))
    bn = kw.get("bn", False)
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    if "residual" in kw:
        b.residual(*kw["residual"]).residualPadding(kw.get("pad_out", 0))
    if "leak" in kw:
        b.leakyReLU(kw["leak"])
    if "clip" in kw:
        b.clip(*kw["clip"])
    inv = int(round(1 / step))
    oh, ow = h * inv // stride, w * inv // stride
    wts = conv_block(700 + k, cout, k, cin, bn=bn)
    inputs = [prng.uniform(17 * k + cin, (cin, h, w), -1, 1)]
    if "residual" in kw:
        inputs.append(prng.uniform(29, (cout, oh, ow), -1, 1))
    print("case", case, "storage", storage, flush=True)
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    err = rel_l2(got, ref)
    print("  ", info, "rel_l2=%.3e" % err, flush=True)
    # (a layer with at most four output channels may also take the row-rolling form, a 3x3 layer the 16-position-fragment
    # form, whichever the engine times faster)
    assert "fractional step 1/%d" % inv in info and (expect in info or (expect == "conv_mfma" and (("conv_rows" in info and cout <= 4) or ("conv_p16" in info and k == 3))))
    assert got.shape == ref.shape == (cout, oh, ow)
    assert err <= TOL[storage], info


FRAC_ROWS_CASES = [
    FRAC_CASES[2], FRAC_CASES[3],                                 # the last layers of the reference's style nets, reduced
    (9, 12, 3, 70, 41, 0.5, 1, 0, A.RELU, {}),                    # three strips, several row blocks
    (5, 12, 4, 9, 40, 0.5, 1, 1, A.RELU, {"bn": True, "residual": (A.RELU, True)}),
    (7, 24, 2, 13, 11, 0.25, 1, 0, A.NONE, {}),                   # two k16 steps per row, pixels repeated four times
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", FRAC_ROWS_CASES, ids=lambda c: "k%d_%dx%dx%d_to%d_step%g" % (c[0], c[1], c[3], c[4], c[2], c[5]))
def test_fractional_convolution_row_rolling_form(case, storage, monkeypatch):
    """The fractional-step convolution onto at most four channels on the row-rolling kernel: the rows it stages are rows
    of the frame of repeated pixels."""
    monkeypatch.setenv("FYNHIP_FORCE_ROWS_WIDE_CONV", "1")
    test_fractional_convolution_parity(case, storage, expect="conv_rows")


FRAC_P16_CASES = [
    FRAC_CASES[0], FRAC_CASES[1],                                  # deconv1 and deconv2 of the reference's style nets, reduced
    (3, 40, 20, 37, 45, 0.5, 2, 0, A.RELU, {}),                    # several tiles, ragged on both sides
    (3, 24, 16, 19, 23, 0.5, 1, 1, A.RELU, {"bn": True, "residual": (A.NONE, False), "pad_out": 1}),   # no down-sampling, padded tensors
    (3, 64, 64, 9, 12, 0.25, 2, 0, A.NONE, {"bn": True}),          # whole chunks and blocks, pixels repeated four times
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", FRAC_P16_CASES, ids=lambda c: "k%d_%dx%dx%d_to%d_step%g_s%d" % (c[0], c[1], c[3], c[4], c[2], c[5], c[6]))
def test_fractional_convolution_sixteen_position_form(case, storage, monkeypatch):
    """The fractional-step 3x3 convolution on the 16-position-fragment kernel: its staging waves fetch the halo tile of
    the frame of repeated pixels."""
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    monkeypatch.setenv("FYNHIP_NO_H16_CONV", "1")
    test_fractional_convolution_parity(case, storage, expect="conv_p16")


@pytest.mark.parametrize("case", [FRAC_CASES[1], FRAC_CASES[3], FRAC_CASES[6]], ids=["deconv2", "deconv3_9x9", "k5_bn_residual"])
def test_fractional_convolution_on_the_plain_kernel(case, monkeypatch):
    """The fp32 FMA kernel (one thread per output pixel), kept as the engine's second implementation of the shallow
    sampling rules, selected by the engine's test switch."""
    monkeypatch.setenv("FYNHIP_FORCE_DIRECT_CONV", "1")
    test_fractional_convolution_parity(case, fa.STORAGE_F32, expect="conv_direct")


def test_fractional_convolution_rejections():
    """gpu/gpulayerfactory.cpp:447-456 and gpu/vanilla/fractionalconvlayerNxN_vanilla.cpp:44: deep tensors, 1x1
    kernels and dilation are refused; so are steps and sizes whose sample positions would not be dyadic."""
    def builder(k=3, step=0.5, h=8, w=8, stride=1):
        return fa.ConvLayerBuilder(k, "fracconv").type(fa.LayerType.FRACCONVOLUTION2D).number(1).shape(4, h, w, 4).sourceStep(step).downsample(stride)

    x = np.zeros((4, 8, 8), np.float32)
    with pytest.raises(fa.FynException, match="not supported for deep layers"):
        run_single(builder().deep(), fa.STORAGE_F32, [x], conv_block(1, 4, 3, 4))
    with pytest.raises(fa.FynException, match="Kernel size 1 not supported"):
        run_single(builder(k=1), fa.STORAGE_F32, [x], conv_block(1, 4, 1, 4))
    with pytest.raises(fa.FynException, match="Dilations not supported"):
        run_single(builder().dilation(2), fa.STORAGE_F32, [x], conv_block(1, 4, 3, 4))
    with pytest.raises(fa.FynException, match="sourceStep"):
        run_single(builder(step=0.3), fa.STORAGE_F32, [x], conv_block(1, 4, 3, 4))
    with pytest.raises(fa.FynException, match="not a multiple"):
        run_single(builder(step=1.0, h=7, w=7, stride=2), fa.STORAGE_F32, [np.zeros((4, 7, 7), np.float32)], conv_block(1, 4, 3, 4))


_CACHE_CHILD = r"""
import sys
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import fyusenet_amd as fa
from fyusenet_amd import prng
from util import conv_block, run_single
from test_gpu_conv import conv_builder
A = fa.ActType
for k, cout, h, w, cin, stride in ((9, 3, 70, 200, 32, 1), (1, 64, 14, 14, 512, 1), (3, 48, 30, 30, 48, 1), (1, 96, 28, 28, 64, 2)):
    b = conv_builder(k, cout, h, w, cin, stride, 1, A.RELU)
    out, info = run_single(b, fa.STORAGE_F16, [prng.uniform(5, (cin, h, w), -1, 1)], conv_block(900 + k, cout, k, cin))
    print(info, "%.6e" % float(abs(out).sum()))
"""


def test_tuning_choices_are_remembered_across_processes(tmp_path):
    """FYNHIP_TUNE_CACHE: a second process finds the first one's measured choices (tile, tile width, chunk width, split-K
    factor) in the file, sets up the same kernels without measuring and adds nothing to the file."""
    import os
    import subprocess
    import sys
    if os.environ.get("FYNHIP_AUTOTUNE", "").startswith("0"):
        pytest.skip("nothing is measured with FYNHIP_AUTOTUNE=0")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cache = tmp_path / "tune.txt"
    env = dict(os.environ, FYNHIP_TUNE_CACHE=str(cache))
    runs = []
    for _ in range(2):
        r = subprocess.run([sys.executable, "-c", _CACHE_CHILD, root], env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        runs.append((r.stdout, cache.read_text()))
    assert runs[0][0] == runs[1][0]                      # same kernels, same results
    assert runs[0][1] == runs[1][1]                      # nothing measured again
    lines = runs[0][1].splitlines()
    assert len(lines) >= 4 and all(len(ln.split()) == 8 for ln in lines)
