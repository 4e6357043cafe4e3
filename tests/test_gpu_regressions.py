"""Regression tests of engine behaviour around buffer reuse, captured graphs and the Python wrappers' argument checks."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import capi, networks, prng
from util import conv_block, rel_l2

pytestmark = pytest.mark.gpu
A = fa.ActType
STORAGES = pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])


class _ConcatAfterWide(fa.NeuralNetwork):
    """wide (16 real channels) -> two 5-channel branches -> concat (10 channels, pitch 16) -> a consumer that names 12
    input channels.  With buffer reuse the concat result lands in the buffer the 16-channel tensor occupied; lanes
    10..15 of every pixel must read as zero there."""
    H, W = 20, 28

    def buildLayers(self, f):
        H, W = self.H, self.W
        fa.ConvLayerBuilder(1, "wide").type(fa.LayerType.CONVOLUTION2D).number(1).shape(16, H, W, 8).deep().push(f)
        fa.ConvLayerBuilder(1, "left").type(fa.LayerType.CONVOLUTION2D).number(2).shape(5, H, W, 16).deep().push(f)
        fa.ConvLayerBuilder(1, "right").type(fa.LayerType.CONVOLUTION2D).number(3).shape(5, H, W, 16).deep().push(f)
        b = fa.ConcatLayerBuilder("cat").number(4).deep().input(5, 0).input(5, 0)
        b.size(W, H)
        b.outputChannels_ = 10
        b.push(f)
        fa.ConvLayerBuilder(1, "reader").type(fa.LayerType.CONVOLUTION2D).number(5).shape(4, H, W, 12).deep().push(f)

    def connectLayers(self, layers, bm):
        bm.connectLayers(layers[1], layers[2], 0)
        bm.connectLayers(layers[1], layers[3], 0)
        bm.connectLayers(layers[2], layers[4], 0)
        bm.connectLayers(layers[3], layers[4], 1)
        bm.connectLayers(layers[4], layers[5], 0)

    def initializeWeights(self, layers):
        big = conv_block(300, 16, 1, 8)
        big[:16] = 1000.0   # every lane of the wide tensor holds something large
        layers[1].loadWeightsAndBiases(big, 0)
        layers[2].loadWeightsAndBiases(conv_block(304, 5, 1, 16), 0)
        layers[3].loadWeightsAndBiases(conv_block(308, 5, 1, 16), 0)
        w = conv_block(312, 4, 1, 12)
        w[4:] = 1.0         # the two channels beyond the ten real ones carry weight too
        layers[5].loadWeightsAndBiases(w, 0)


@STORAGES
def test_concat_pad_lanes_are_zero_after_buffer_reuse(storage):
    x = prng.uniform(320, (8, _ConcatAfterWide.H, _ConcatAfterWide.W), -1, 1)
    outs = []
    for reuse in (False, True):
        net = _ConcatAfterWide(storage)
        net.setup(reuseBuffers=reuse)
        net.layers[1].setInput(x, 0)
        net.forward()
        net.finish()
        outs.append(net.getOutput(5))
        if not reuse:
            cat = net.layers[4].copyResult()
            assert cat.shape[0] == 10
        net.cleanup()
    assert np.isfinite(outs[1]).all()
    assert np.array_equal(outs[0], outs[1])
    # (without reuse the concat result sits in a buffer of its own, zero-filled at setup: lanes 10..15 are zero there)


@STORAGES
def test_weights_loaded_after_a_graph_launch_take_effect(storage):
    """A captured forward pass holds kernel arguments by value, among them the power of two that undoes a layer's
    weight pre-scaling; loading weights of another magnitude must not leave the replay with stale arguments."""
    net = networks.StyleNet(storage, width=64, height=48)
    net.setup()
    x = net.makeInput()
    net.setInput(x)
    net.useGraph(True)
    net.forward()
    net.finish()
    first = net.getOutput(net.output_layer)
    # the same stream with every convolution's weights scaled by 1/64 (bias and batch-norm left alone would change the
    # function in a less controlled way: scale whole blocks, the comparison below is graph against eager anyway)
    net.weightStream = (net.weightStream * np.float32(1.0 / 64.0)).astype(np.float32)
    net.initializeWeights(net.layers)
    net.forward()
    net.finish()
    replayed = net.getOutput(net.output_layer)
    net.useGraph(False)
    net.forward()
    net.finish()
    eager = net.getOutput(net.output_layer)
    net.cleanup()
    assert np.array_equal(replayed, eager)
    assert not np.array_equal(replayed, first)


def test_python_wrappers_check_buffer_sizes():
    net = networks.StyleNet(fa.STORAGE_F32, width=64, height=48)
    net.setup()
    x = net.makeInput()
    with pytest.raises(capi.FynException, match="takes 9216 floats"):
        net.layers[0].setInput(x[:, :-1], 0)
    net.setInput(x)
    net.forward()
    net.finish()
    y = net.getOutput(net.output_layer)
    net.asyncBegin(0, net.output_layer, depth=2)
    with pytest.raises(capi.FynException, match="floats in and"):
        net.asyncSubmit(x, np.empty(y.size - 1, np.float32))
    with pytest.raises(capi.FynException, match="floats in and"):
        net.asyncSubmit(x[:2], np.empty_like(y))
    out = np.empty_like(y)
    t = net.asyncSubmit(x, out)
    assert t in net._async_outs   # kept alive until delivered
    net.asyncWait(t)
    assert t not in net._async_outs
    net.asyncEnd()
    assert np.array_equal(out, y)
    net.cleanup()


@pytest.mark.parametrize("magnitude", [1e5, 3e2, 1.0, 1e-5, 1e-9], ids=lambda m: "x%g" % m)
@pytest.mark.parametrize("k,cin,cout", [(3, 64, 64), (1, 256, 32), (9, 32, 3), (9, 3, 32)])
def test_fp32_storage_keeps_its_accuracy_over_the_value_range(magnitude, k, cin, cout):
    """With fp32 storage the matrix path splits operands into fp16 pairs; the engine moves a tensor's magnitudes into
    the window where the split is exact (a power of two taken from the largest magnitude written), so inputs far from
    1 -- beyond fp16's largest number or deep in its subnormal range -- keep the 1e-4 bound against the oracle."""
    from util import oracle_single, run_single
    h, w = 24, 40
    b = fa.ConvLayerBuilder(k, "conv").type(fa.LayerType.CONVOLUTION2D).number(1).shape(cout, h, w, cin).deep()
    b.inputPadding((k - 1) // 2).prefixAct(A.RELU)
    wts = conv_block(500 + k, cout, k, cin)
    x = (prng.uniform(501, (cin, h, w), -1, 1) * magnitude).astype(np.float32)
    got, info = run_single(b, fa.STORAGE_F32, [x], wts)
    ref = oracle_single(b, fa.STORAGE_F32, [x], wts)
    assert np.isfinite(got).all(), info
    # (the bias of about 0.01 dominates the tiny cases; compare what the convolution adds to it as well)
    bias = wts[:cout].astype(np.float64)[:, None, None]
    assert rel_l2(got, ref) <= 1e-4, info
    if magnitude >= 1e-5:
        assert rel_l2(got.astype(np.float64) - bias, ref.astype(np.float64) - bias) <= 1e-4, info


class _RangeChain(fa.NeuralNetwork):
    """Three convolutions whose weights make the intermediate tensors huge (first layer x 3e5) and small again."""
    H, W = 20, 24

    def buildLayers(self, f):
        H, W = self.H, self.W
        fa.UpDownLayerBuilder(fa.UpDownLayerBuilder.UPLOAD, "in").number(0).shape(8, H, W, 8).outputPadding(1).push(f)
        for no, (ci, co) in enumerate([(8, 32), (32, 32), (32, 16)], start=1):
            b = fa.ConvLayerBuilder(3, "c%d" % no).type(fa.LayerType.CONVOLUTION2D).number(no).shape(co, H, W, ci).deep()
            b.inputPadding(1).outputPadding(1 if no < 3 else 0).prefixAct(A.RELU if no > 1 else A.NONE)
            if no == 3:
                b.residual(A.RELU).residualPadding(0)
            b.push(f)

    def connectLayers(self, layers, bm):
        bm.connectLayers(layers[0], layers[1], 0)
        bm.connectLayers(layers[1], layers[2], 0)
        bm.connectLayers(layers[2], layers[3], 0)

    def initializeWeights(self, layers):
        self.blocks = []
        for no, (ci, co, gain) in enumerate([(8, 32, 3e5), (32, 32, 1.0), (32, 16, 1e-7)], start=1):
            blk = conv_block(520 + 4 * no, co, 3, ci)
            blk[co:] *= np.float32(gain)
            layers[no].loadWeightsAndBiases(blk, 0)


def test_value_range_words_start_over_every_frame():
    """A frame's result does not depend on the frames before it: the per-tensor magnitude words are cleared between
    passes (bit-identical outputs for a frame run after a frame of 1e6 times its magnitude and on a fresh network),
    and the chain stays within the fp32-storage bound although its middle tensors reach 1e6."""
    from oracle import oracle as O
    small = prng.uniform(540, (8, _RangeChain.H, _RangeChain.W), -1, 1)
    res = prng.uniform(541, (16, _RangeChain.H, _RangeChain.W), -1, 1)
    huge = (small * 1e6).astype(np.float32)

    def run(net, x, graph):
        net.useGraph(graph)
        net.layers[0].setInput(x, 0)
        net.layers[3].setInput(res, 1)
        net.forward()
        net.finish()
        return net.getOutput(3)

    fresh = _RangeChain(fa.STORAGE_F32)
    fresh.setup()
    want = run(fresh, small, False)
    ref = O.run_network(fresh.describe(), {(0, 0): small, (3, 1): res})[3]
    assert rel_l2(want, ref) <= 1e-4
    assert np.abs(fresh.layers[2].copyResult()).max() > 1e5     # the middle tensors are far beyond fp16's range
    fresh.cleanup()
    for graph in (False, True):
        net = _RangeChain(fa.STORAGE_F32)
        net.setup()
        first = run(net, huge, graph)
        assert np.isfinite(first).all()
        again = run(net, small, graph)
        net.cleanup()
        assert np.array_equal(again, want), "graph=%s" % graph
