"""Network descriptions of the benchmark configurations, written the way the reference's sample
networks are (samples/samplenetworks/resnet50.cpp:200-536, stylenet3x3.cpp:114-234): builders pushed
into a factory, explicit connectLayers calls, one headerless fp32 weight stream sliced by offsets.

Weights are synthetic (He-normal, bias ~ N(0, 0.01), folded batch-norm as scale ~ U(lo, hi) and
bias ~ N(0, 0.1)); the reference's pretrained .dat files are git-LFS stubs and unavailable.
"""
import numpy as np

from . import prng
from .builders import (ActType, ArgMaxLayerBuilder, ConvLayerBuilder, GPULayerBuilder, LayerType, NormType, PoolLayerBuilder,
                       UpDownLayerBuilder)
from .capi import STORAGE_F16, STORAGE_F32
from .network import NeuralNetwork

SEED_BASE = 0xF7A5E000


def conv_block(seed, cout, k, cin, bn=False, depthwise=False, bn_scale=(0.5, 1.5)):
    """One layer's block of a .dat stream: [bias][W [o][ky][kx][i]][bnScale][bnBias]
    (fyusenet/base/convlayerinterface.h:71-95; depthwise: [i][ky][kx], gpu/deep/deepdwconvlayerbase.cpp:242)."""
    if depthwise:
        w = prng.he_normal(seed, (cin * k * k,), k * k)
    else:
        w = prng.he_normal(seed, (cout * k * k * cin,), k * k * cin)
    parts = [prng.normal(seed + 1, (cout,), 0.0, 0.01), w]
    if bn:
        parts += [prng.uniform(seed + 2, (cout,), bn_scale[0], bn_scale[1]), prng.normal(seed + 3, (cout,), 0.0, 0.1)]
    return np.concatenate(parts).astype(np.float32)


class _StreamNet(NeuralNetwork):
    """Common plumbing: layers are declared with their weight-block generator; initializeWeights walks
    the stream by offsets like ResNet50::initializeWeights (samples/samplenetworks/resnet50.cpp:522-536)."""

    config_id = 0

    def __init__(self, storage, device=0):
        super().__init__(storage, device)
        self._builders = []
        self._edges = []
        self._blocks = []   # (layer number, generator)
        self._seed = SEED_BASE + self.config_id * 256
        self.weightStream = None
        self.offsets = {}

    def _add(self, b, block=None):
        self._builders.append(b)
        if block is not None:
            self._blocks.append((b.number_, block))
        return b

    def _next_seed(self):
        self._seed += 4
        return self._seed

    def buildLayers(self, factory):
        self.define()
        for b in self._builders:
            b.push(factory)

    def connectLayers(self, layers, bm):
        for (src, dst, port) in self._edges:
            bm.connectLayers(layers[src], layers[dst], port)

    def initializeWeights(self, layers):
        if self.weightStream is None:
            chunks, off = [], 0
            for no, gen in self._blocks:
                blk = gen()
                self.offsets[no] = off
                off += blk.size
                chunks.append(blk)
            self.weightStream = np.concatenate(chunks) if chunks else np.zeros(0, np.float32)
        for no, _ in self._blocks:
            lyr = layers[no]
            if int(lyr.builder.type_) == int(LayerType.BATCHNORM):
                lyr.loadScaleAndBias(self.weightStream, self.offsets[no])
            else:
                lyr.loadWeightsAndBiases(self.weightStream, self.offsets[no])

    # helpers -------------------------------------------------------------------------------
    def conv(self, no, name, k, cin, cout, h, w, src, stride=1, act=ActType.NONE, pad_out=0, bn=True, residual=None,
             res_act=ActType.NONE, clip=None, bn_scale=(0.5, 1.5), groups=1, res_pad=0):
        b = ConvLayerBuilder(k, name).type(LayerType.CONVOLUTION2D).number(no).shape(cout, h, w, cin).deep()
        b.downsample(stride).inputPadding((k - 1) // 2).outputPadding(pad_out).prefixAct(act)
        if clip:
            b.clip(*clip)
        if bn:
            b.postfixNorm(NormType.BATCHNORM)
        if groups != 1:
            b.groupSize(groups)
        if residual is not None:
            b.residual(res_act).residualPadding(res_pad)
            self._edges.append((residual, no, 1))
        seed = self._next_seed()
        dw = groups != 1
        self._add(b, lambda: conv_block(seed, cout, k, cin, bn=bn, depthwise=dw, bn_scale=bn_scale))
        if src is not None:
            self._edges.append((src, no, 0))
        return no


class SingleConvNet(_StreamNet):
    """Config 1: one 3x3 s1 p1 convolution 64->64 @256x256 with ReLU on input fetch
    (ConvLayerBuilder(3).shape(64,256,256,64).deep().inputPadding(1).prefixAct(RELU))."""
    config_id = 1

    def __init__(self, storage=STORAGE_F32, size=256, channels=64, device=0, width=None, height=None, residual=False):
        super().__init__(storage, device)
        self.width, self.height, self.ch, self.residual = width or size, height or size, channels, residual

    def define(self):
        self.conv(1, "conv3x3", 3, self.ch, self.ch, self.height, self.width, None, act=ActType.RELU, bn=False)
        if self.residual:   # residual tensor on port 1, fed from the host like the input (ReLU applied on its fetch)
            self._builders[-1].residual(ActType.RELU)

    def makeInput(self):
        return prng.uniform(SEED_BASE + 256 + 200, (self.ch, self.height, self.width), -1.0, 1.0)

    def setInput(self, x):
        self.layers[1].setInput(x, 0)
        if self.residual:
            self.layers[1].setInput(prng.uniform(SEED_BASE + 256 + 201, (self.ch, self.height, self.width), -1.0, 1.0), 1)

    output_layer = 1
    input_key = (1, 0)


class StyleNet(_StreamNet):
    """Configs 2 and 5: Johnson-style transfer net.  9x9 conv 3->32; 3x3 s2 convs 32->64->128; five residual
    blocks of two KxK 128->128 convs (K = 3 for config 2, 9 for config 5) with the residual add fused into the
    second conv; 3x3 s2 transposed convs 128->64->32 cropped to exactly 2x; 9x9 conv 32->3.  ReLU on every
    fetch but the first, batch-norm folded into scale/bias."""

    def __init__(self, storage=STORAGE_F32, width=512, height=624, res_kernel=3, device=0):
        self.config_id = 2 if res_kernel == 3 else 5
        super().__init__(storage, device)
        if width % 4 or height % 4:
            raise ValueError("style net needs sizes divisible by 4")
        self.W, self.H, self.rk = width, height, res_kernel

    def define(self):
        W, H, rk = self.W, self.H, self.rk
        rp = (rk - 1) // 2
        R = ActType.RELU
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(3, H, W, 3).outputPadding(4))
        self.conv(1, "conv1", 9, 3, 32, H, W, 0, pad_out=1)
        self.conv(2, "conv2", 3, 32, 64, H, W, 1, stride=2, act=R, pad_out=1)
        self.conv(3, "conv3", 3, 64, 128, H // 2, W // 2, 2, stride=2, act=R, pad_out=rp)
        h4, w4 = H // 4, W // 4
        prev, no = 3, 4
        for blk in range(5):
            self.conv(no, "res%d_1" % (blk + 1), rk, 128, 128, h4, w4, prev, act=R, pad_out=rp)
            last = blk == 4
            self.conv(no + 1, "res%d_2" % (blk + 1), rk, 128, 128, h4, w4, no, act=R, pad_out=1 if last else rp, residual=prev,
                      res_act=R, res_pad=rp, bn_scale=(0.25, 0.75))
            prev, no = no + 1, no + 2
        for i, (cin, cout, hh, ww, po) in enumerate([(128, 64, h4, w4, 1), (64, 32, H // 2, W // 2, 4)]):
            b = ConvLayerBuilder(3, "tconv%d" % (i + 1)).type(LayerType.TRANSCONVOLUTION2D).number(no).shape(cout, hh, ww, cin).deep()
            b.upsample(2).inputPadding(1).outputPadding(po).prefixAct(R).postfixNorm(NormType.BATCHNORM).crop(1)
            seed = self._next_seed()
            self._add(b, (lambda s=seed, ci=cin, co=cout: conv_block(s, co, 3, ci, bn=True)))
            self._edges.append((prev, no, 0))
            prev, no = no, no + 1
        self.conv(no, "conv_out", 9, 32, 3, H, W, prev, act=R, pad_out=0, bn=False)
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(no + 1).shape(3, H, W, 3).deep())
        self._edges.append((no, no + 1, 0))
        self.output_layer = no + 1
        self.last_conv = no

    def makeInput(self):
        return prng.uniform(SEED_BASE + self.config_id * 256 + 200, (3, self.H, self.W), 0.0, 1.0)

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


class ResNet50(_StreamNet):
    """Config 3: ResNet-50 v1 at batch 1.  7x7 s2 stem, 3x3 s2 max-pool, bottleneck stages [3,4,6,3] at widths
    256/512/1024/2048 (stride on the 3x3 and on the 1x1 projection shortcut, as samples/samplenetworks/
    resnet50.cpp:260-265 places it), global average pool, FC 2048->1000 (GEMM layer), arg-max.  Batch-norm is
    folded into every convolution (POST_BATCHNORM blocks); each ReLU is applied by the consumer on fetch, the
    residual add is fused into the last 1x1 convolution of a block (residual on port 1)."""
    config_id = 3

    def __init__(self, storage=STORAGE_F32, size=224, classes=1000, device=0):
        super().__init__(storage, device)
        self.size, self.classes = size, classes

    def define(self):
        S = self.size
        R = ActType.RELU
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(3, S, S, 3).outputPadding(3))
        self.conv(1, "stem", 7, 3, 64, S, S, 0, stride=2, pad_out=1)
        s = S // 2
        self._add(PoolLayerBuilder(PoolLayerBuilder.POOL_MAX, "maxpool").number(2).shape(64, s, s, 64).poolSize(3).downsample(2)
                  .inputPadding(1).prefixAct(R).deep())
        self._edges.append((1, 2, 0))
        s //= 2
        prev, no, cin = 2, 3, 64
        prev_act_res = R   # how a block input is read as residual (its ReLU is applied on fetch)
        for stage, (blocks, width) in enumerate(zip([3, 4, 6, 3], [256, 512, 1024, 2048])):
            mid = width // 4
            for blk in range(blocks):
                stride = 2 if (blk == 0 and stage > 0) else 1
                name = "s%db%d" % (stage + 1, blk + 1)
                if blk == 0:
                    sc = self.conv(no, name + "_proj", 1, cin, width, s, s, prev, stride=stride, act=R)
                    no += 1
                    res, res_act = sc, ActType.NONE
                else:
                    res, res_act = prev, prev_act_res
                self.conv(no, name + "_a", 1, cin, mid, s, s, prev, act=R, pad_out=1)
                self.conv(no + 1, name + "_b", 3, mid, mid, s, s, no, stride=stride, act=R)
                so = s // stride
                self.conv(no + 2, name + "_c", 1, mid, width, so, so, no + 1, act=R, residual=res, res_act=res_act,
                          bn_scale=(0.25, 0.75))
                prev, no, cin, s = no + 2, no + 3, width, so
        self._add(PoolLayerBuilder(PoolLayerBuilder.POOL_AVG, "avgpool").number(no).shape(cin, s, s, cin).prefixAct(R).deep().global_pool())
        self._edges.append((prev, no, 0))
        fc = GPULayerBuilder("fc").type(LayerType.GEMM).number(no + 1).shape(self.classes, 1, 1, cin).deep()
        seed = self._next_seed()
        self._add(fc, lambda: conv_block(seed, self.classes, 1, cin, bn=False))
        self._edges.append((no, no + 1, 0))
        self._add(ArgMaxLayerBuilder("argmax").number(no + 2).shape(2, 1, 1, self.classes).deep())
        self._edges.append((no + 1, no + 2, 0))
        self.logits_layer, self.argmax_layer = no + 1, no + 2
        self.output_layer = no + 1

    def makeInput(self):
        return prng.normal(SEED_BASE + 3 * 256 + 200, (3, self.size, self.size))

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


class MobileNetV2(_StreamNet):
    """Config 4: MobileNetV2-style stack: 3x3 s2 stem 3->32, then 17 inverted-residual blocks (expansion 6 except
    the first): 1x1 expand, 3x3 depthwise (groupSize == channels), 1x1 project with the residual add fused where
    stride is 1 and the channel count is kept.  ReLU6 is clip(0,6) applied on fetch by the depthwise and the
    project convolutions; the expand convolution of the next block reads the linear bottleneck without
    activation, and the residual tensor is read raw."""
    config_id = 4
    # (expansion, cout, stride)
    BLOCKS = [(1, 16, 1), (6, 24, 2), (6, 24, 1), (6, 32, 2), (6, 32, 1), (6, 32, 1), (6, 64, 2), (6, 64, 1), (6, 64, 1),
              (6, 64, 1), (6, 96, 1), (6, 96, 1), (6, 96, 1), (6, 160, 2), (6, 160, 1), (6, 160, 1), (6, 320, 1)]

    def __init__(self, storage=STORAGE_F16, size=224, device=0):
        super().__init__(storage, device)
        self.size = size

    def define(self):
        S = self.size
        C = ActType.CLIP
        c6 = (0.0, 6.0)
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(3, S, S, 3).outputPadding(1))
        self.conv(1, "stem", 3, 3, 32, S, S, 0, stride=2, pad_out=1)
        s, cin, prev, no = S // 2, 32, 1, 2
        for i, (t, cout, stride) in enumerate(self.BLOCKS):
            name = "b%d" % i
            exp = cin * t
            if t != 1:
                self.conv(no, name + "_expand", 1, cin, exp, s, s, prev, pad_out=1)
                dw_src, no = no, no + 1
            else:
                dw_src = prev
            self.conv(no, name + "_dw", 3, exp, exp, s, s, dw_src, stride=stride, act=C, clip=c6, groups=exp)
            so = s // stride
            use_res = stride == 1 and cin == cout
            last = i == len(self.BLOCKS) - 1
            # a block output feeds the next block's expand conv (no halo needed) -- or, for block 0's successor, too
            nxt_needs_halo = (not last) and False
            self.conv(no + 1, name + "_project", 1, exp, cout, so, so, no, act=C, clip=c6, residual=prev if use_res else None,
                      pad_out=1 if nxt_needs_halo else 0)
            prev, no, cin, s = no + 1, no + 2, cout, so
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(no).shape(cin, s, s, cin).deep())
        self._edges.append((prev, no, 0))
        self.output_layer = no

    def makeInput(self):
        return prng.normal(SEED_BASE + 4 * 256 + 200, (3, self.size, self.size))

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)
