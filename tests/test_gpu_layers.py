"""Parity of the bandwidth-bound HIP layers (depthwise conv, pooling, batch-norm, add, concat,
arg-max, fully connected) and of the upload/download formats against the CPU oracle, through the
C ABI.  Max-pool, concat and arg-max indices must be bit-exact; the others stay within the storage
tolerance (rel-L2 1e-4 fp32 storage, 2e-3 fp16 storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import prng
from oracle import oracle as O
from util import conv_block, make_single_layer_net, oracle_single, rel_l2, run_single

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}
A = fa.ActType
STORAGES = pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])


@STORAGES
@pytest.mark.parametrize("c,h,w,stride,dil,res,bn", [(2, 1, 1, 1, 1, False, False), (5, 3, 2, 1, 1, True, True), (8, 2, 9, 2, 1, False, False),
                                                      (16, 5, 4, 1, 1, False, False), (24, 7, 6, 2, 1, False, True), (40, 4, 33, 1, 1, True, False),
                                                      (32, 112, 112, 1, 1, False, True), (96, 56, 56, 2, 1, False, False),
                                                      (144, 28, 28, 1, 1, True, True), (24, 17, 19, 1, 2, False, False),
                                                      (960, 7, 7, 1, 1, False, True), (12, 9, 9, 1, 1, True, False)])
def test_depthwise_parity(c, h, w, stride, dil, res, bn, storage):
    b = fa.ConvLayerBuilder(3, "dw").type(fa.LayerType.CONVOLUTION2D).number(1).shape(c, h, w, c).groupSize(c)
    b.downsample(stride).dilation(dil).inputPadding(dil).prefixAct(A.CLIP).clip(0.0, 6.0).deep()
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    if res:
        b.residual()
    wts = conv_block(40, c, 3, c, bn=bn, depthwise=True)
    inputs = [prng.uniform(41, (c, h, w), -2, 8)]
    if res:
        inputs.append(prng.uniform(42, (c, h // stride, w // stride), -1, 1))
    got, info = run_single(b, storage, inputs, wts)
    ref = oracle_single(b, storage, inputs, wts)
    assert info == "dwconv3x3" and got.shape == ref.shape
    assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("op,pool,stride,pad,c,h,w,act", [
    ("max", 2, 2, 0, 1, 2, 2, A.NONE), ("avg", 2, 2, 0, 3, 2, 6, A.RELU), ("max", 3, 2, 1, 9, 5, 3, A.RELU), ("avg", 3, 1, 1, 2, 1, 1, A.NONE),
    ("max", 4, 4, 0, 8, 8, 4, A.NONE), ("max", 2, 2, 0, 4, 8, 8, A.NONE), ("max", 2, 2, 0, 23, 200, 200, A.NONE), ("max", 3, 2, 1, 64, 112, 112, A.RELU),
    ("max", 2, 2, 0, 80, 40, 30, A.RELU), ("avg", 2, 2, 0, 12, 32, 32, A.NONE), ("avg", 3, 1, 1, 16, 20, 20, A.RELU),
    ("avg", 4, 4, 0, 80, 64, 48, A.NONE), ("avg", 2, 2, 0, 23, 200, 200, A.NONE)])  # shapes of pooltests.cpp:323-354
def test_pool_parity(op, pool, stride, pad, c, h, w, act, storage):
    kind = fa.PoolLayerBuilder.POOL_MAX if op == "max" else fa.PoolLayerBuilder.POOL_AVG
    b = fa.PoolLayerBuilder(kind, "pool").number(1).shape(c, h, w, c).poolSize(pool).downsample(stride)
    b.inputPadding(pad).prefixAct(act).deep()
    x = prng.uniform(50, (c, h, w), -100, 100)
    got, _ = run_single(b, storage, [x])
    ref = oracle_single(b, storage, [x])
    if op == "max":
        assert np.array_equal(got, ref)  # bit-exact
    else:
        assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("op,c,h,w", [("avg", 1, 1, 1), ("max", 3, 1, 5), ("avg", 9, 2, 2), ("avg", 2048, 7, 7), ("max", 4, 200, 200), ("avg", 4, 200, 200), ("avg", 23, 13, 9), ("max", 80, 16, 16),
                                        # images of 16384 pixels and more: the pixels are dealt to many workgroups, a second launch pools their results
                                        ("avg", 23, 160, 130), ("max", 12, 300, 200), ("avg", 128, 200, 200), ("max", 4, 128, 128)])
def test_global_pool_parity(op, c, h, w, storage):
    kind = fa.PoolLayerBuilder.POOL_MAX if op == "max" else fa.PoolLayerBuilder.POOL_AVG
    b = fa.PoolLayerBuilder(kind, "gpool").number(1).shape(c, h, w, c).prefixAct(A.RELU).deep().global_pool()
    x = prng.normal(51, (c, h, w))
    got, _ = run_single(b, storage, [x])
    ref = oracle_single(b, storage, [x])
    assert got.shape == (c, 1, 1)
    if op == "max":
        assert np.array_equal(got, ref)
    else:
        assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("c,h,w,res", [(64, 56, 56, None), (23, 17, 9, None), (32, 20, 20, (A.RELU, True)), (8, 12, 12, (A.NONE, False))])
def test_batchnorm_parity(c, h, w, res, storage):
    b = fa.GPULayerBuilder("bn").type(fa.LayerType.BATCHNORM).number(1).shape(c, h, w, c).prefixAct(A.RELU).deep()
    if res:
        b.residual(*res)
    sb = np.concatenate([prng.uniform(60, (c,), 0.5, 1.5), prng.normal(61, (c,), 0, 0.3)]).astype(np.float32)
    inputs = [prng.normal(62, (c, h, w))]
    if res:
        inputs.append(prng.normal(63, (c, h, w)))
    net = make_single_layer_net(b, storage, scale_bias=sb)
    lyr = net.layers[1]
    for p, x in enumerate(inputs):
        lyr.setInput(x, p)
    net.forward()
    got = lyr.copyResult()
    net.cleanup()
    desc = {"layers": [{"builder": b, "number": 1, "weights": sb}], "connections": [], "storage": storage}
    ref = O.run_network(desc, {(1, p): x for p, x in enumerate(inputs)})[1]
    assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("sub", [False, True])
@pytest.mark.parametrize("c,h,w", [(24, 30, 40), (20, 5, 333)], ids=["24x30x40", "wide-rows"])   # (rows of 256 items and more take their indices from a 2-D grid)
def test_addsub_parity(sub, c, h, w, storage):
    b = fa.GPULayerBuilder("add").type(fa.LayerType.SUB if sub else fa.LayerType.ADD).number(1).shape(c, h, w, c)
    xs = [prng.normal(70, (c, h, w)), prng.normal(71, (c, h, w))]
    got, _ = run_single(b, storage, xs)
    ref = oracle_single(b, storage, xs)
    assert rel_l2(got, ref) <= TOL[storage]


@STORAGES
@pytest.mark.parametrize("chans,relu", [([32, 32], False), ([23, 52], False), ([3, 5, 12], True), ([8, 4, 4, 16], False)])
@pytest.mark.parametrize("w,h", [(28, 20), (301, 6)], ids=["28x20", "wide-rows"])   # (rows of 256 items and more take their indices from a 2-D grid)
def test_concat_bit_exact(chans, relu, w, h, storage):
    b = fa.ConcatLayerBuilder("cat").number(1).deep()
    flags = fa.LayerFlags.PRE_RELU if relu else fa.LayerFlags.NO_LAYER_FLAGS
    for c in chans:
        b.input(c, 0, flags)
    b.size(w, h)
    b.outputChannels_ = sum(chans)
    xs = [prng.normal(80 + i, (c, h, w)) for i, c in enumerate(chans)]
    got, _ = run_single(b, storage, xs)
    ref = oracle_single(b, storage, xs)
    assert got.shape == (sum(chans), h, w)
    assert np.array_equal(got, ref)


@STORAGES
@pytest.mark.parametrize("c,h,w", [(1, 1, 1), (2, 3, 1), (5, 1, 7), (1000, 1, 1), (64, 128, 256), (128, 40, 40), (21, 33, 17), (2048, 3, 5),
                                   (128, 259, 257), (12, 725, 724)])  # misctests.cpp:269-275 shapes; the last two: four pixels per lane group, ragged end
def test_argmax_indices_exact(c, h, w, storage):
    b = fa.ArgMaxLayerBuilder("argmax").number(1).shape(2, h, w, c).deep()
    x = prng.normal(90, (c, h, w))
    if storage == fa.STORAGE_F16:
        x = O.round_fp16(x)
    x[:, 0, 0] = x[3 % c, 0, 0]  # full tie at one pixel: lowest index must win
    net = make_single_layer_net(b, storage)
    net.layers[1].setInput(x)
    net.forward()
    idx, val = net.getArgMax(1)
    chw = net.layers[1].copyResult()
    net.cleanup()
    ridx, rval = O.argmax(x)
    assert np.array_equal(idx, ridx) and idx[0, 0] == 0
    assert np.array_equal(val, rval)
    assert np.array_equal(chw[0].astype(np.int32), ridx) and np.array_equal(chw[1], rval)


@STORAGES
@pytest.mark.parametrize("cin,cout,bn", [(1, 1, False), (3, 7, True), (1025, 2, False), (2048, 1000, False), (512, 256, False), (100, 10, True)])
def test_gemm_parity(cin, cout, bn, storage):
    b = fa.GPULayerBuilder("fc").type(fa.LayerType.GEMM).number(1).shape(cout, 1, 1, cin).prefixAct(A.RELU).deep()
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    wts = conv_block(95, cout, 1, cin, bn=bn)
    x = prng.normal(96, (cin, 1, 1))
    got, info = run_single(b, storage, [x], wts)
    ref = oracle_single(b, storage, [x], wts)
    assert rel_l2(got, ref) <= TOL[storage]


_FC_CASES = [(32, 16, False, A.NONE, 1.0), (40, 7, True, A.RELU, 1.0), (1025, 2, False, A.RELU, 1.0), (2048, 1000, False, A.RELU, 1.0),
             (512, 256, True, A.LEAKY_RELU, 3.0e5), (100, 10, True, A.CLIP, 1.0), (4096, 24, False, A.NONE, 1.0e-7), (8192, 40, False, A.RELU, 1.0)]
# (fp16 tensors cannot hold the value ranges that the scaled cases are about)
_FC_PARAMS = [pytest.param(*c, st, id="%dx%d-%s-%g-%s" % (c[0], c[1], c[3].name, c[4], "f32" if st == fa.STORAGE_F32 else "f16"))
              for c in _FC_CASES for st in (fa.STORAGE_F32, fa.STORAGE_F16) if st == fa.STORAGE_F32 or c[4] == 1.0]


@pytest.mark.parametrize("form", ["mfma", "vector"])
@pytest.mark.parametrize("cin,cout,bn,act,xscale,storage", _FC_PARAMS)
def test_gemm_parity_of_both_forms(cin, cout, bn, act, xscale, form, storage, monkeypatch):
    """The fully connected layer on the matrix cores (fc_mfma_kernel) and on the vector units (gemv_kernel), each forced
    (gpu/deep/deepgemmlayer.cpp:66-236): reductions that are not whole steps of 32, fragments of 16 rows that reach
    behind the last output, inputs far above fp16's range and far below it (the vector is scaled by a power of two
    before it is split), all four activations on the fetch."""
    monkeypatch.setenv("FYNHIP_FORCE_MFMA_GEMM" if form == "mfma" else "FYNHIP_NO_MFMA_GEMM", "1")
    b = fa.GPULayerBuilder("fc").type(fa.LayerType.GEMM).number(1).shape(cout, 1, 1, cin).prefixAct(act).deep()
    if act == A.LEAKY_RELU:
        b.leakyReLU(0.1)
    if act == A.CLIP:
        b.clip(-0.5, 1.5)
    if bn:
        b.postfixNorm(fa.NormType.BATCHNORM)
    wts = conv_block(195, cout, 1, cin, bn=bn)
    x = (prng.normal(196, (cin, 1, 1)) * xscale).astype(np.float32)
    got, info = run_single(b, storage, [x], wts)
    ref = oracle_single(b, storage, [x], wts)
    wide = cin <= (8192 if storage == fa.STORAGE_F32 else 16384)
    assert info.startswith("fc_mfma" if form == "mfma" and wide else "gemv"), info
    assert rel_l2(got, ref) <= TOL[storage]


def test_gemm_reference_pattern():
    # misctests.cpp:238-265: 512 -> 256, alternating +-1 rows on ones => exactly 0
    cin, cout = 512, 256
    block = np.concatenate([np.zeros(cout, np.float32), np.tile(np.tile(np.array([1, -1], np.float32), cin // 2), cout)])
    b = fa.GPULayerBuilder("fc").type(fa.LayerType.GEMM).number(1).shape(cout, 1, 1, cin).deep()
    got, _ = run_single(b, fa.STORAGE_F32, [np.ones((cin, 1, 1), np.float32)], block)
    assert np.all(got == 0.0)


class _UpDownNet(fa.NeuralNetwork):
    """upload -> 3x3 conv -> download, the shape of unit_tests/networktests.cpp:85-140."""

    def __init__(self, storage, cin, cout, size, pad):
        super().__init__(storage)
        self.cin, self.cout, self.size, self.pad = cin, cout, size, pad
        self.w = conv_block(5, cout, 3, cin)

    def buildLayers(self, f):
        s = self.size
        fa.UpDownLayerBuilder(fa.UpDownLayerBuilder.UPLOAD, "up").number(0).shape(self.cin, s, s, self.cin).outputPadding(1).push(f)
        fa.ConvLayerBuilder(3, "conv").type(fa.LayerType.CONVOLUTION2D).number(1).shape(self.cout, s, s, self.cin).inputPadding(1).outputPadding(self.pad).deep().push(f)
        fa.UpDownLayerBuilder(fa.UpDownLayerBuilder.DOWNLOAD, "down").number(2).shape(self.cout, s, s, self.cout).inputPadding(self.pad).deep().push(f)

    def connectLayers(self, layers, bm):
        bm.connectLayers(layers[0], layers[1], 0)
        bm.connectLayers(layers[1], layers[2], 0)

    def initializeWeights(self, layers):
        layers["conv"].loadWeightsAndBiases(self.w, 0)


@pytest.mark.parametrize("pad", [0, 1])
def test_upload_download_formats(pad):
    cin, cout, size = 3, 12, 16
    net = _UpDownNet(fa.STORAGE_F32, cin, cout, size, pad)
    net.setup()
    x = prng.uniform(1, (cin, size, size), 0, 1)
    net.layers[0].setInput(O.chw_to_shallow(x, cin), 0, fa.ORDER_GPU_SHALLOW)  # RGB triplets in
    net.forward()
    net.finish()
    chw = net.getOutput(2, fa.ORDER_CHANNELWISE)
    ref = O.conv2d(O.pad_chw(x, 1), 1, net.w, cout, 3)
    assert rel_l2(chw, ref) < 1e-4
    deep = net.getOutput(2, fa.ORDER_GPU_DEEP)
    assert np.array_equal(deep, O.chw_to_deep(chw, pad))
    assert np.array_equal(O.deep_to_chw(deep, cout, size, size, pad), chw)
    net.cleanup()
    # RGBA out of a 3-channel layer
    b = fa.GPULayerBuilder("bn").type(fa.LayerType.BATCHNORM).number(1).shape(3, 8, 10, 3)
    n2 = make_single_layer_net(b, fa.STORAGE_F32, scale_bias=np.array([1, 1, 1, 0, 0, 0], np.float32))
    y = prng.uniform(2, (3, 8, 10), 0, 1)
    n2.layers[1].setInput(y)
    n2.forward()
    rgba = n2.getOutput(1, fa.ORDER_GPU_SHALLOW)
    assert rgba.shape == (8, 10, 4) and np.array_equal(rgba, O.chw_to_shallow(y, 4))
    n2.cleanup()


def test_error_paths_on_device():
    # forward on a layer without weights, reference: deepconvlayerNxN.cpp:130 ("uninitialised layer")
    b = fa.ConvLayerBuilder(3, "conv").type(fa.LayerType.CONVOLUTION2D).number(1).shape(8, 8, 8, 8).inputPadding(1).deep()
    net = make_single_layer_net(b, fa.STORAGE_F32)
    with pytest.raises(fa.FynException):
        net.forward()
    net.cleanup()
