"""Parity of the function-type HIP layers (scale / padding / relu / clip / deep<->shallow, sigmoid, tanh, singleton
arithmetic, cast, transpose, image-patch extraction, RGB<->BGR, non-maximum suppression, blur) against the CPU oracle,
through the C ABI.  Layers that only move or select values must be bit-exact; those that compute stay within the storage
tolerance (rel-L2 1e-4 fp32 storage, 2e-3 fp16 storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import prng
from util import oracle_single, rel_l2, run_single

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}
A, T = fa.ActType, fa.LayerType
STORAGES = pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])


def _check(b, storage, x, exact, kind):
    got, info = run_single(b, storage, [x])
    ref = oracle_single(b, storage, [x])
    assert info == kind and got.shape == ref.shape
    if exact:
        assert np.array_equal(got, ref)
    else:
        assert rel_l2(got, ref) <= TOL[storage]
    return got


@STORAGES
@pytest.mark.parametrize("c,h,w,up,down,deep,pad,act", [
    (3, 40, 52, (2, 2), (1, 1), True, 0, A.NONE), (32, 39, 31, (2, 2), (1, 1), True, 1, A.RELU), (12, 20, 24, (3, 3), (1, 1), False, 0, A.NONE),
    (64, 56, 56, (1, 1), (2, 2), True, 0, A.RELU), (23, 30, 42, (1, 1), (3, 3), True, 1, A.NONE), (8, 32, 48, (1, 1), (2, 2), False, 0, A.NONE),
    (16, 18, 22, (4, 2), (1, 1), True, 0, A.CLIP), (5, 1, 9, (2, 2), (1, 1), True, 0, A.NONE)])
def test_scale_nearest_parity(c, h, w, up, down, deep, pad, act, storage):
    b = fa.ScaleLayerBuilder("scale").number(1).shape(c, h, w, c).upsample(*up).downsample(*down).inputPadding(pad).prefixAct(act).clip(-0.5, 0.5)
    if deep:
        b.deep()
    _check(b, storage, prng.normal(100, (c, h, w)), True, "scale-nearest")


@STORAGES
@pytest.mark.parametrize("c,h,w,up,down,deep,pad,act", [
    (3, 40, 52, (2, 2), (1, 1), True, 0, A.NONE), (32, 39, 31, (2, 2), (1, 1), True, 1, A.RELU), (12, 20, 24, (3, 3), (1, 1), False, 1, A.NONE),
    (8, 32, 48, (1, 1), (2, 2), False, 0, A.NONE), (16, 18, 22, (4, 2), (1, 1), True, 0, A.NONE)])
def test_scale_linear_parity(c, h, w, up, down, deep, pad, act, storage):
    b = fa.ScaleLayerBuilder("scale").number(1).shape(c, h, w, c).upsample(*up).downsample(*down).inputPadding(pad).prefixAct(act)
    b.scaleType(fa.ScalingType.LINEAR)
    if deep:
        b.deep()
    _check(b, storage, prng.normal(101, (c, h, w)), False, "scale-linear")


@STORAGES
def test_scale_builder_factor_interface(storage):
    # ScaleLayerBuilder::scale(float) (gpu/scalelayerbuilder.h:82-114)
    b = fa.ScaleLayerBuilder("s").number(1).shape(8, 12, 16, 8).scale(2.0).deep()
    assert b.upsample_ == [2, 2] and b.equal()
    got = _check(b, storage, prng.normal(102, (8, 12, 16)), True, "scale-nearest")
    assert got.shape == (8, 24, 32)
    b = fa.ScaleLayerBuilder("s").number(1).shape(8, 12, 16, 8).scale(0.5).deep()
    assert b.downsample_ == [2, 2]
    with pytest.raises(fa.FynException):
        fa.ScaleLayerBuilder("s").scale(1.5)


@STORAGES
@pytest.mark.parametrize("ltype,act,pad_in,pad_out,deep", [(T.RELU, A.RELU, 0, 1, True), (T.CLIP, A.CLIP, 1, 0, True), (T.PADDING2D, A.NONE, 0, 2, False),
                                                          (T.DEEP2SHALLOW, A.RELU, 1, 1, True), (T.SHALLOW2DEEP, A.NONE, 0, 1, False)])
def test_copy_type_layers(ltype, act, pad_in, pad_out, deep, storage):
    # RELU / CLIP / PADDING2D are scale layers of factor 1 in the reference (gpu/gpulayerfactory.cpp:125-140);
    # the activation is the builder's prefix activation
    c, h, w = 20, 14, 18
    b = fa.ScaleLayerBuilder("copy").type(ltype).number(1).shape(c, h, w, c).inputPadding(pad_in).outputPadding(pad_out).prefixAct(act).clip(-1.0, 0.25)
    if deep:
        b.deep()
    x = prng.normal(103, (c, h, w))
    got = _check(b, storage, x, True, "scale-nearest")
    if act == A.RELU:
        assert got.min() == 0.0
    if act == A.CLIP:
        assert got.max() == 0.25 and got.min() == -1.0


@STORAGES
@pytest.mark.parametrize("ltype,kind", [(T.SIGMOID, "sigmoid"), (T.TANH, "tanh")])
@pytest.mark.parametrize("c,h,w,deep,act", [(3, 64, 80, False, A.NONE), (40, 16, 16, True, A.RELU), (23, 9, 13, True, A.NONE)])
def test_sigmoid_tanh_parity(ltype, kind, c, h, w, deep, act, storage):
    b = fa.GPULayerBuilder(kind).type(ltype).number(1).shape(c, h, w, c).prefixAct(act)
    if deep:
        b.deep()
    got = _check(b, storage, prng.normal(104, (c, h, w), 0.0, 3.0), False, kind)
    assert np.all(np.abs(got) <= 1.0)


# unit_tests/arithtests.cpp:205-234: constant tensor (op) scalar
@STORAGES
@pytest.mark.parametrize("deep", [False, True])
@pytest.mark.parametrize("op", list(fa.ArithType))
@pytest.mark.parametrize("a,b_,w,h,c", [(3.0, 30.0, 400, 300, 4), (-2.0, 1.0, 200, 200, 5), (10.0, -10.0, 16, 16, 40), (-100.0, 23.0, 55, 57, 30),
                                        (15.0, -16.0, 99, 52, 47)])
def test_singleton_arith_reference_cases(op, a, b_, w, h, c, deep, storage):
    b = fa.SingletonArithLayerBuilder("single", op).number(1).shape(c, h, w, c).operand(b_)
    if deep:
        b.deep()
    x = np.full((c, h, w), a, np.float32)
    got, info = run_single(b, storage, [x])
    expect = {0: a + b_, 1: a - b_, 2: a * b_, 3: a / b_}[int(op)]
    assert info == "singleton-arith"
    assert np.all(np.abs(got - expect) < 0.5)                       # the reference's criterion (arithtests.cpp:131)
    ref = oracle_single(b, storage, [x])
    assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("op", list(fa.ArithType))
def test_singleton_arith_random(op, storage):
    b = fa.SingletonArithLayerBuilder("single", op).number(1).shape(19, 21, 17, 19).operand(-1.75).prefixAct(A.RELU).deep()
    _check(b, storage, prng.normal(105, (19, 21, 17)), False, "singleton-arith")


@STORAGES
@pytest.mark.parametrize("target", list(fa.CastTarget))
def test_cast_parity(target, storage):
    c, h, w = 7, 24, 30
    x = prng.uniform(106, (c, h, w), -400.0, 400.0)
    x[0, 0, :8] = [0.49, -0.49, 1.51, -1.51, 254.6, 255.4, 70000.0, -70000.0]
    frac = np.abs(x - np.floor(x) - 0.5)
    x = np.where(frac < 1e-2, x + 0.25, x).astype(np.float32)        # keep away from exact halves (also after fp16 rounding)
    if storage == fa.STORAGE_F16:
        x = np.clip(x, -60000.0, 60000.0)
        x = x.astype(np.float16).astype(np.float32)
        frac = np.abs(x - np.floor(x) - 0.5)
        x = np.where(frac < 1e-2, np.floor(x), x).astype(np.float32)
    b = fa.CastLayerBuilder("cast", target).number(1).shape(c, h, w, c).deep()
    got = _check(b, storage, x, True, "cast")
    if int(target) < 6:
        assert np.array_equal(got, np.rint(got))


@STORAGES
@pytest.mark.parametrize("c,h,w,act", [(4, 16, 24, A.NONE), (32, 56, 40, A.RELU), (23, 7, 31, A.NONE), (128, 1, 64, A.NONE)])
def test_transpose_parity(c, h, w, act, storage):
    b = fa.TransposeLayerBuilder("tr").number(1).shape(c, h, w, c).prefixAct(act).deep()
    got = _check(b, storage, prng.normal(107, (c, h, w)), True, "transpose")
    assert got.shape == (c, w, h)
    with pytest.raises(fa.FynException, match="shallow transpose"):
        run_single(fa.TransposeLayerBuilder("tr").number(1).shape(c, h, w, c), storage, [np.zeros((c, h, w), np.float32)])


@STORAGES
@pytest.mark.parametrize("cin,window,h,w,act", [(4, 2, 16, 24, A.NONE), (8, 2, 30, 18, A.RELU), (12, 3, 27, 33, A.NONE), (6, 2, 8, 12, A.NONE), (32, 4, 64, 64, A.NONE)])
def test_imgextract_parity(cin, window, h, w, act, storage):
    cout = ((cin + 3) // 4 * 4) * window * window
    b = fa.ImgExtractLayerBuilder(window, "patch").number(1).shape(cout, h, w, cin).prefixAct(act)
    got = _check(b, storage, prng.normal(108, (cin, h, w)), True, "imgextract")
    assert got.shape == (cout, h // window, w // window)


@STORAGES
def test_imgextract_rejections(storage):
    z = np.zeros((4, 8, 8), np.float32)
    with pytest.raises(fa.FynException):      # createImgExtractLayer rejects builders flagged deep
        run_single(fa.ImgExtractLayerBuilder(2, "p").number(1).shape(16, 8, 8, 4).deep(), storage, [z])
    with pytest.raises(fa.FynException):      # more output channels than the window yields
        run_single(fa.ImgExtractLayerBuilder(2, "p").number(1).shape(20, 8, 8, 4), storage, [z])
    with pytest.raises(fa.FynException):      # size not divisible by the window
        run_single(fa.ImgExtractLayerBuilder(3, "p").number(1).shape(36, 8, 8, 4), storage, [z])


@STORAGES
@pytest.mark.parametrize("c,h,w,pad", [(3, 20, 30, 0), (4, 33, 17, 1), (11, 16, 16, 0)])
def test_rgb2bgr_nonmax_blur_parity(c, h, w, pad, storage):
    x = prng.uniform(109, (c, h, w), 0.0, 1.0)
    b = fa.GPULayerBuilder("bgr").type(T.RGB2BGR).number(1).shape(c, h, w, c).inputPadding(pad)
    _check(b, storage, x, True, "rgb2bgr")
    b = fa.GPULayerBuilder("nms").type(T.NONMAX2D).number(1).shape(c, h, w, c).inputPadding(pad)
    got = _check(b, storage, x, True, "nonmax2d")
    assert 0 < np.count_nonzero(got) < got.size // 3
    for k in (3, 5, 7):
        for typ in fa.BlurKernelType:
            b = fa.BlurLayerBuilder("blur").number(1).shape(c, h, w, c).inputPadding(pad).kernel(k).blurType(typ)
            _check(b, storage, x, False, "blur2d")
    for ltype in (T.RGB2BGR, T.NONMAX2D, T.BLUR2D):      # shallow tensors only (gpu/gpulayerfactory.cpp)
        with pytest.raises(fa.FynException):
            bb = (fa.BlurLayerBuilder("x") if ltype == T.BLUR2D else fa.GPULayerBuilder("x").type(ltype)).number(1).shape(c, h, w, c).deep()
            run_single(bb, storage, [x])
    with pytest.raises(fa.FynException, match="odd kernel"):
        run_single(fa.BlurLayerBuilder("x").number(1).shape(c, h, w, c).kernel(4), storage, [x])


@STORAGES
def test_style_net_tail_with_sigmoid(storage):
    """Transposed convolution -> sigmoid -> download, the tail of the reference's style-transfer samples
    (samples/samplenetworks/stylenet3x3.cpp:171-176,209-211)."""
    from oracle import oracle as O
    from util import conv_block

    class Tail(fa.NeuralNetwork):
        def buildLayers(self, f):
            fa.ConvLayerBuilder(3, "deconv3").type(T.TRANSCONVOLUTION2D).number(1).shape(3, 24, 32, 12).upsample(2).crop(1).prefixAct(A.RELU).deep().push(f)
            fa.GPULayerBuilder("sigmoid").type(T.SIGMOID).number(2).shape(3, 48, 64, 3).deep().push(f)
            fa.UpDownLayerBuilder(fa.UpDownLayerBuilder.DOWNLOAD, "down").number(3).shape(3, 48, 64, 3).deep().push(f)

        def connectLayers(self, layers, bm):
            for i in (1, 2):
                bm.connectLayers(layers[i], layers[i + 1], 0)

        def initializeWeights(self, layers):
            layers[1].loadWeightsAndBiases(conv_block(110, 3, 3, 12), 0)

    net = Tail(storage)
    net.setup()
    x = prng.normal(111, (12, 24, 32))
    net.layers[1].setInput(x, 0)
    net.forward()
    net.finish()
    got = net.getOutput(3)
    ref = O.run_network(net.describe(), {(1, 0): x})[3]
    assert got.shape == (3, 48, 64) and rel_l2(got, ref) <= TOL[storage]
    assert got.min() > 0.0 and got.max() < 1.0
    net.cleanup()


def _hip():
    import ctypes
    lib = ctypes.CDLL("libamdhip64.so")
    lib.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    lib.hipMemcpyAsync.restype = ctypes.c_int
    return lib


class _CopyLayer:
    """A user layer: device-to-device copy of its input (same geometry on both sides), enqueued on the given stream."""
    calls = 0

    def __init__(self, fail_forward=False):
        self.hip = _hip()
        self.fail_forward = fail_forward
        self.was_set_up = self.cleaned = False

    def setup(self, inputs, output):
        i = inputs[0]
        assert (i.channels, i.height, i.width, i.padding, i.channel_pitch, i.storage) == \
               (output.channels, output.height, output.width, output.padding, output.channel_pitch, output.storage)
        self.nbytes = (i.height + 2 * i.padding) * (i.width + 2 * i.padding) * i.channel_pitch * (2 if i.storage else 4)
        self.was_set_up = True

    def forward(self, inputs, output, stream, sequence):
        if self.fail_forward:
            raise RuntimeError("told to fail")
        type(self).calls += 1
        assert self.hip.hipMemcpyAsync(output.data, inputs[0].data, self.nbytes, 3, stream) == 0   # hipMemcpyDeviceToDevice

    def cleanup(self):
        self.cleaned = True


@STORAGES
def test_custom_layer_hook(storage):
    """CustomLayerBuilder (gpu/customlayerbuilder.h:53-90): a layer supplied by the application sits between two engine
    layers, receives device views of its tensors and the stream, and its work is ordered with theirs."""
    from util import conv_block
    made = []

    def init(builder):
        made.append(_CopyLayer())
        return made[-1]

    class Net(fa.NeuralNetwork):
        def buildLayers(self, f):
            fa.ConvLayerBuilder(3, "conv").type(T.CONVOLUTION2D).number(1).shape(16, 20, 24, 8).inputPadding(1).outputPadding(1).deep().push(f)
            fa.CustomLayerBuilder("mine", init).number(2).shape(16, 20, 24, 16).inputPadding(1).outputPadding(1).deep().push(f)
            fa.GPULayerBuilder("sig").type(T.SIGMOID).number(3).shape(16, 20, 24, 16).inputPadding(1).prefixAct(A.RELU).deep().push(f)

        def connectLayers(self, layers, bm):
            bm.connectLayers(layers[1], layers[2], 0)
            bm.connectLayers(layers[2], layers[3], 0)

        def initializeWeights(self, layers):
            layers[1].loadWeightsAndBiases(conv_block(120, 16, 3, 8), 0)

    net = Net(storage)
    net.setup()
    assert made[0].was_set_up and net.layers[2].kernelInfo() == "custom"
    x = prng.normal(121, (8, 20, 24))
    net.layers[1].setInput(x, 0)
    for graph in (False, True):
        net.useGraph(graph)
        for _ in range(3):
            net.forward()
            net.finish()
            conv = net.layers[1].copyResult()
            assert np.array_equal(net.layers[2].copyResult(), conv)
            want = 1.0 / (1.0 + np.exp(-np.maximum(conv.astype(np.float64), 0)))
            assert rel_l2(net.getOutput(3), want) <= TOL[storage]
    assert _CopyLayer.calls >= 4          # every eager pass plus the captured one
    net.cleanup()
    assert made[0].cleaned

    class Failing(Net):
        def buildLayers(self, f):
            fa.ConvLayerBuilder(3, "conv").type(T.CONVOLUTION2D).number(1).shape(16, 20, 24, 8).inputPadding(1).outputPadding(1).deep().push(f)
            fa.CustomLayerBuilder("mine", lambda b: _CopyLayer(fail_forward=True)).number(2).shape(16, 20, 24, 16).inputPadding(1).outputPadding(1).deep().push(f)
            fa.GPULayerBuilder("sig").type(T.SIGMOID).number(3).shape(16, 20, 24, 16).inputPadding(1).deep().push(f)

    bad = Failing(storage)
    bad.setup()
    bad.layers[1].setInput(x, 0)
    with pytest.raises(fa.FynException, match="forward callback failed"):
        bad.forward()
    bad.cleanup()
    with pytest.raises(fa.FynException):     # a custom type without its implementation
        run_single(fa.GPULayerBuilder("x").type(T.CUSTOM).number(1).shape(4, 8, 8, 4), storage, [np.zeros((4, 8, 8), np.float32)])
