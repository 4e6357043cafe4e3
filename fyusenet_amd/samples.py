"""The reference's own sample graphs (ResNet-50, style transfer) and their weight-file layouts.

`ResNet50Sample` builds the network of samples/samplenetworks/resnet50.cpp with the same layer numbers, names,
flags and connections (builders: resnet50.cpp:200-423, edges: :427-515), so that a weight file written for the
reference (`data/resnet_50.dat`, 102,304,184 bytes of headerless little-endian fp32) loads unchanged:
`weight_layout()` reproduces the byte offsets of ResNet50::initializeWeightOffsets (resnet50.cpp:539-677) from the
layer descriptions instead of a table.

Structure of that graph (it differs from the folded-BN benchmark graph in networks.py): an explicit batch-norm
layer on the RGB input and after the max-pool; bottleneck stages [3, 4, 6, 3]; in the first block of a stage the
block input feeds the 1x1 reduce convolution and the 1x1 projection shortcut directly; every later block starts
with an explicit batch-norm layer and takes the previous block's (un-normalised) output as residual; the last block
of a stage applies its batch-norm to the residual as well (BATCHNORM_ON_RESIDUAL); stride 2 sits on the 3x3
convolution and on the projection.  ReLU is always applied by the consumer on fetch.

`StyleNetSample` builds the reference's style-transfer samples (samples/samplenetworks/stylenet3x3.cpp:114-211,
stylenet9x9.cpp:118-251): all layers shallow and unpadded (every convolution repeats the edge of its input), 12 / 20 /
40 channels, two or five residual blocks at a quarter of the size, three fractional-step convolutions back up and a
sigmoid; `weight_layout()` reproduces the float offsets the reference hard-codes (stylenet3x3.cpp:41-50,
stylenet9x9.cpp:41-56) for its 77,235- and 169,059-float weight streams.  The OESCONV input variant (an Android
external-texture format) is not provided.
"""
import os

import numpy as np

from . import prng
from .builders import ActType, ConvLayerBuilder, GPULayerBuilder, LayerType, NormType, PoolLayerBuilder, UpDownLayerBuilder
from .capi import ERR_INVALID, STORAGE_F32, FynException
from .network import NeuralNetwork

RESNET50_TOTAL_WEIGHT_BYTES = 102304184   # samples/samplenetworks/resnet50.cpp:676


class _SampleNet(NeuralNetwork):
    """A graph described by (number, builder, weight floats) entries, edges and the order of the layers' blocks in
    the weight stream.  `weights`: None (synthetic weights from the in-repo PRNG), a float32 array, or the path of
    a headerless little-endian fp32 file."""

    def __init__(self, storage=STORAGE_F32, weights=None, device=0):
        super().__init__(storage, device)
        self._weights = weights
        self._specs = []     # (number, builder, weight floats or 0)
        self._edges = []
        self._file_order = []
        self._define()

    def weight_layout(self):
        """{layer number: (byte offset, byte size)} in the file order of the reference's `.dat`."""
        floats = {no: n for no, _, n in self._specs}
        layout, off = {}, 0
        for no in self._file_order:
            layout[no] = (off, 4 * floats[no])
            off += 4 * floats[no]
        return layout

    def total_weight_bytes(self):
        return sum(size for _, size in self.weight_layout().values())

    # ---- NeuralNetwork interface ----
    def buildLayers(self, factory):
        for _, b, _ in sorted(self._specs, key=lambda s: s[0]):
            b.push(factory)

    def connectLayers(self, layers, bm):
        for src, dst, port in self._edges:
            bm.connectLayers(layers[src], layers[dst], port)

    def _stream(self):
        w = self._weights
        if w is None:
            return self.synthetic_weights()
        if isinstance(w, (str, os.PathLike)):
            if os.path.getsize(w) != self.total_weight_bytes():
                raise FynException(ERR_INVALID, "%s: expected %d bytes of weights, file has %d" % (w, self.total_weight_bytes(), os.path.getsize(w)))
            return np.memmap(w, dtype="<f4", mode="r")
        w = np.ascontiguousarray(w, dtype=np.float32).ravel()
        if w.size * 4 != self.total_weight_bytes():
            raise FynException(ERR_INVALID, "expected %d floats of weights, got %d" % (self.total_weight_bytes() // 4, w.size))
        return w

    def initializeWeights(self, layers):
        # ResNet50::initializeWeights (resnet50.cpp:522-536): convolution-type layers take weights and biases,
        # batch-norm layers scale and bias, both addressed by float offset into the one stream
        stream = self._stream()
        for no, (off, size) in self.weight_layout().items():
            lyr = layers[no]
            block = np.asarray(stream[off // 4:(off + size) // 4], dtype=np.float32)
            if int(lyr.builder.type_) == int(LayerType.BATCHNORM):
                lyr.loadScaleAndBias(block, 0)
            else:
                lyr.loadWeightsAndBiases(block, 0)

    def synthetic_weights(self, seed=0xF7A5E300):
        """A weight stream of the file's exact size: He-normal weights, small biases, batch-norm scales in a range
        that keeps activations O(1) through all 16 blocks."""
        out = np.empty(self.total_weight_bytes() // 4, np.float32)
        spec = {no: b for no, b, _ in self._specs}
        for i, (no, (off, size)) in enumerate(sorted(self.weight_layout().items())):
            b, o, n = spec[no], off // 4, size // 4
            s = seed + 8 * i
            if int(b.type_) == int(LayerType.BATCHNORM):
                c = n // 2
                out[o:o + c] = prng.uniform(s, (c,), 0.5, 1.5)
                out[o + c:o + n] = prng.normal(s + 1, (c,), 0.0, 0.1)
                continue
            cout, cin = b.outputChannels_, b.inputChannels_
            k = getattr(b, "kernel_", 1)
            nw = cout * k * k * cin
            out[o:o + cout] = prng.normal(s, (cout,), 0.0, 0.01)
            out[o + cout:o + cout + nw] = prng.he_normal(s + 1, (nw,), k * k * cin)
            if n > cout + nw:
                lo, hi = (0.25, 0.75) if (int(b.getFlags()) & 1) else (0.5, 1.5)
                out[o + cout + nw:o + 2 * cout + nw] = prng.uniform(s + 2, (cout,), lo, hi)
                out[o + 2 * cout + nw:o + n] = prng.normal(s + 3, (cout,), 0.0, 0.1)
        return out


class ResNet50Sample(_SampleNet):
    IMAGE_SIZE = 224
    STAGES = ((3, 64), (4, 128), (6, 256), (3, 512))   # (blocks, bottleneck width); output width = 4x
    UPLOAD, INPUT_BN, STEM, MAXPOOL, POOL_BN, FIRST_BLOCK = 0, 2, 3, 4, 5, 6
    GLOBAL_POOL, GEMM, DOWNLOAD = 70, 72, 73

    # ---- graph description ----
    def _conv(self, no, k, cout, size, cin, stride=1, pad_in=0, pad_out=0, act=ActType.RELU, bn=False, residual=None):
        b = ConvLayerBuilder(k, "Conv%d" % no).type(LayerType.CONVOLUTION2D).number(no).shape(cout, size, size, cin).deep()
        b.downsample(stride).inputPadding(pad_in).outputPadding(pad_out).prefixAct(act)
        if bn:
            b.postfixNorm(NormType.BATCHNORM)
        if residual is not None:
            b.residual(ActType.NONE, residual == "bn")
        floats = cout + cout * k * k * cin + (2 * cout if bn else 0)
        self._specs.append((no, b, floats))
        return no

    def _bn(self, no, channels, size, deep=True, pad_out=0):
        b = GPULayerBuilder("BN%d" % no).type(LayerType.BATCHNORM).number(no).shape(channels, size, size, channels).outputPadding(pad_out)
        if deep:
            b.deep()
        self._specs.append((no, b, 2 * channels))
        return no

    def _define(self):
        S = self.IMAGE_SIZE
        up = UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(self.UPLOAD).shape(3, S, S, 3)
        self._specs.append((self.UPLOAD, up, 0))
        self._bn(self.INPUT_BN, 3, S, deep=False, pad_out=1)
        self._file_order.append(self.INPUT_BN)
        # 7x7 stride-2 stem reading a halo of 1 (resnet50.cpp:211-212): what lies beyond it reads as zero
        self._conv(self.STEM, 7, 64, S, 3, stride=2, pad_in=1, pad_out=1, act=ActType.NONE, bn=True)
        self._file_order.append(self.STEM)
        mp = PoolLayerBuilder(PoolLayerBuilder.POOL_MAX, "MaxPool4").type(LayerType.MAXPOOL2D).number(self.MAXPOOL)
        mp.shape(64, S // 2, S // 2, 64).poolSize(3, 3).downsample(2).deep().inputPadding(1).prefixAct(ActType.RELU)
        self._specs.append((self.MAXPOOL, mp, 0))
        size = S // 4
        self._bn(self.POOL_BN, 64, size)
        self._file_order.append(self.POOL_BN)
        self._edges += [(self.UPLOAD, self.INPUT_BN, 0), (self.INPUT_BN, self.STEM, 0), (self.STEM, self.MAXPOOL, 0),
                        (self.MAXPOOL, self.POOL_BN, 0)]
        no, prev, cin = self.FIRST_BLOCK, self.POOL_BN, 64
        for stage, (blocks, width) in enumerate(self.STAGES):
            out = 4 * width
            for blk in range(blocks):
                last = blk == blocks - 1
                if blk == 0:
                    stride = 2 if stage > 0 else 1
                    a = self._conv(no, 1, width, size, cin, pad_out=1, bn=True)
                    proj = self._conv(no + 1, 1, out, size, cin, stride=stride)
                    b3 = self._conv(no + 2, 3, width, size, width, stride=stride, pad_in=1, bn=True)
                    size //= stride
                    c = self._conv(no + 3, 1, out, size, width, residual="plain")
                    self._edges += [(prev, a, 0), (prev, proj, 0), (a, b3, 0), (proj, c, 1), (b3, c, 0)]
                    self._file_order += [a, b3, c, proj]          # the projection is stored behind its block
                else:
                    n = self._bn(no, out, size)
                    a = self._conv(no + 1, 1, width, size, out, pad_out=1, bn=True)
                    b3 = self._conv(no + 2, 3, width, size, width, pad_in=1, bn=True)
                    c = self._conv(no + 3, 1, out, size, width, bn=last, residual="bn" if last else "plain")
                    self._edges += [(prev, n, 0), (prev, c, 1), (n, a, 0), (a, b3, 0), (b3, c, 0)]
                    self._file_order += [n, a, b3, c]
                prev, no, cin = no + 3, no + 4, out
        assert no == self.GLOBAL_POOL
        gp = PoolLayerBuilder(PoolLayerBuilder.POOL_AVG, "GlobAvg70").type(LayerType.AVGPOOL2D).number(self.GLOBAL_POOL)
        gp.shape(cin, size, size, cin).global_pool().deep().prefixAct(ActType.RELU)
        self._specs.append((self.GLOBAL_POOL, gp, 0))
        fc = GPULayerBuilder("GEMM72").type(LayerType.GEMM).number(self.GEMM).shape(1000, 1, 1, cin).deep()
        self._specs.append((self.GEMM, fc, 1000 + cin * 1000))
        self._file_order.append(self.GEMM)
        down = UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(self.DOWNLOAD).shape(1000, 1, 1, 1000).deep()
        self._specs.append((self.DOWNLOAD, down, 0))
        self._edges += [(prev, self.GLOBAL_POOL, 0), (self.GLOBAL_POOL, self.GEMM, 0), (self.GEMM, self.DOWNLOAD, 0)]
        self.output_layer = self.GEMM
        self.input_key = (self.UPLOAD, 0)

    def makeInput(self):
        return prng.normal(0xF7A5E3F0, (3, self.IMAGE_SIZE, self.IMAGE_SIZE))

    def setInput(self, x):
        """x: CHW fp32 (3, 224, 224)."""
        self.layers[self.UPLOAD].setInput(x, 0)


STYLENET3X3_WEIGHT_FLOATS = 77235     # samples/samplenetworks/stylenet3x3.h:53
STYLENET9X9_WEIGHT_FLOATS = 169059    # samples/samplenetworks/stylenet9x9.h:59


class StyleNetSample(_SampleNet):
    """kernel 3: StyleNet3x3 (two residual blocks); kernel 9: StyleNet9x9 (9x9 first and last layer, five blocks).
    Width and height must be multiples of 4.  Input: CHW fp32 RGB in [0, 1]; output: layer SIGMOID, (3, H, W)."""

    UPLOAD, CONV1, CONV2, CONV3, FIRST_RES = 0, 1, 2, 3, 4

    def __init__(self, kernel=3, width=512, height=624, storage=STORAGE_F32, weights=None, device=0):
        if kernel not in (3, 9):
            raise FynException(ERR_INVALID, "the reference has style nets with 3x3 and 9x9 outer kernels, not %d" % kernel)
        if width % 4 or height % 4:
            raise FynException(ERR_INVALID, "style net: %dx%d is not a multiple of 4" % (width, height))
        self.kernel, self.width, self.height = kernel, width, height
        self.blocks = 2 if kernel == 3 else 5
        self.DECONV1 = self.FIRST_RES + 2 * self.blocks
        self.DECONV2, self.DECONV3, self.SIGMOID, self.DOWNLOAD = self.DECONV1 + 1, self.DECONV1 + 2, self.DECONV1 + 3, self.DECONV1 + 4
        super().__init__(storage, weights, device)

    def _conv(self, no, name, k, cout, h, w, cin, act=ActType.NONE, stride=1, residual=None, frac=None):
        b = ConvLayerBuilder(k, name).number(no).shape(cout, h, w, cin).prefixAct(act)
        b.type(LayerType.CONVOLUTION2D if frac is None else LayerType.FRACCONVOLUTION2D).downsample(stride)
        if frac is not None:
            b.sourceStep(frac)
        if residual is not None:
            b.residual(residual)
        self._specs.append((no, b, cout + cout * k * k * cin))
        return no

    def _define(self):
        W, H, K, R = self.width, self.height, self.kernel, ActType.RELU
        up = UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(self.UPLOAD).shape(3, H, W, 3)
        self._specs.append((self.UPLOAD, up, 0))
        self._conv(self.CONV1, "conv1", K, 12, H, W, 3, R)
        self._conv(self.CONV2, "conv2", 3, 20, H, W, 12, R, stride=2)
        self._conv(self.CONV3, "conv3", 3, 40, H // 2, W // 2, 20, R, stride=2)
        self._edges += [(self.UPLOAD, self.CONV1, 0), (self.CONV1, self.CONV2, 0), (self.CONV2, self.CONV3, 0)]
        prev, res = self.CONV3, []
        for i in range(self.blocks):
            a, c = self.FIRST_RES + 2 * i, self.FIRST_RES + 2 * i + 1
            # the first convolution of the second block reads its input without ReLU; the first block applies ReLU to its
            # shortcut, the others do not (stylenet3x3.cpp:147-159, stylenet9x9.cpp:153-189)
            self._conv(a, "res%d_1" % (i + 1), 3, 40, H // 4, W // 4, 40, ActType.NONE if i == 1 else R)
            self._conv(c, "res%d_2" % (i + 1), 3, 40, H // 4, W // 4, 40, R, residual=R if i == 0 else ActType.NONE)
            self._edges += [(prev, a, 0), (prev, c, 1), (a, c, 0)]
            res += [a, c]
            prev = c
        self._conv(self.DECONV1, "deconv1", 3, 20, H // 4, W // 4, 40, ActType.NONE, stride=2, frac=0.5)
        self._conv(self.DECONV2, "deconv2", 3, 12, H // 4, W // 4, 20, R, stride=2, frac=0.25)
        self._conv(self.DECONV3, "deconv3", K, 3, H // 2, W // 2, 12, R, frac=0.5)
        sg = GPULayerBuilder("sigmoid").type(LayerType.SIGMOID).number(self.SIGMOID).shape(3, H, W, 3)
        self._specs.append((self.SIGMOID, sg, 0))
        down = UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(self.DOWNLOAD).shape(4, H, W, 4)
        self._specs.append((self.DOWNLOAD, down, 0))
        self._edges += [(prev, self.DECONV1, 0), (self.DECONV1, self.DECONV2, 0), (self.DECONV2, self.DECONV3, 0),
                        (self.DECONV3, self.SIGMOID, 0), (self.SIGMOID, self.DOWNLOAD, 0)]
        # order of the blocks in the weight stream: the outer layers first, then the residual blocks
        self._file_order = [self.CONV1, self.CONV2, self.CONV3, self.DECONV1, self.DECONV2, self.DECONV3] + res
        self.output_layer = self.SIGMOID
        self.input_key = (self.UPLOAD, 0)

    def weight_offsets(self):
        """{layer number: float offset}, the reference's weightOffsets_ table."""
        return {no: off // 4 for no, (off, _) in self.weight_layout().items()}

    def makeInput(self):
        return prng.uniform(0x57A1E000 + self.kernel, (3, self.height, self.width), 0.0, 1.0)

    def setInput(self, x):
        """x: CHW fp32 (3, height, width)."""
        self.layers[self.UPLOAD].setInput(x, 0)
