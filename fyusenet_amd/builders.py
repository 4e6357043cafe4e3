"""Layer description surface, mirroring the reference's fluent builders method for method.

LayerBuilder        -> fyusenet/base/layerbuilder.h:53-558 (LayerBuilderTempl)
GPULayerBuilder     -> fyusenet/gpu/gpulayerbuilder.h
ConvLayerBuilder    -> fyusenet/gpu/convlayerbuilder.h
PoolLayerBuilder    -> fyusenet/gpu/poollayerbuilder.h
ConcatLayerBuilder  -> fyusenet/gpu/concatlayerbuilder.h
ArgMaxLayerBuilder  -> fyusenet/gpu/argmaxlayerbuilder.h
UpDownLayerBuilder  -> fyusenet/gpu/updownlayerbuilder.h
ScaleLayerBuilder   -> fyusenet/gpu/scalelayerbuilder.h
SingletonArithLayerBuilder -> fyusenet/gpu/singleton_arithlayerbuilder.h
CastLayerBuilder    -> fyusenet/gpu/castlayerbuilder.h
TransposeLayerBuilder -> fyusenet/gpu/transposelayerbuilder.h
ImgExtractLayerBuilder -> fyusenet/gpu/imgextractlayerbuilder.h
BlurLayerBuilder    -> fyusenet/gpu/blurlayerbuilder.h

Method names keep the reference's spelling (inputPadding, prefixAct, ...) so that a network
description reads like samples/samplenetworks/resnet50.cpp.  A builder only collects fields; the
engine is reached when LayerFactory.compileLayers() hands the descriptions to the C ABI.
"""
import enum

from . import capi


class LayerFlags(enum.IntFlag):
    """fyusenet/base/layerflags.h:33-50."""
    NO_LAYER_FLAGS = 0
    RESIDUAL_INPUT = 1
    RELU_ON_RESIDUAL = 2
    BATCHNORM_ON_RESIDUAL = 4
    POST_BATCHNORM = 8
    DEEP = 16
    POST_RELU = 32
    PRE_RELU = 64
    PRE_CLIP = 128


class ActType(enum.IntEnum):
    """fyusenet/base/layerflags.h:61-68."""
    NONE = 0
    RELU = 1
    LEAKY_RELU = 2
    CLIP = 3
    SIGMOID = 4
    TANH = 5


class ScalingType(enum.IntEnum):
    """fyusenet/base/layerflags.h:89-92."""
    NEAREST = 0
    LINEAR = 1


class BlurKernelType(enum.IntEnum):
    """fyusenet/base/layerflags.h:99-102."""
    AVERAGE = 0
    GAUSSIAN = 1


class ArithType(enum.IntEnum):
    """fyusenet/base/layerflags.h:109-114."""
    ADD = 0
    SUB = 1
    MUL = 2
    DIV = 3


class CastTarget(enum.IntEnum):
    """fyusenet/base/layerflags.h:121-130."""
    CT_INT32 = 0
    CT_INT16 = 1
    CT_INT8 = 2
    CT_UINT32 = 3
    CT_UINT16 = 4
    CT_UINT8 = 5
    CT_FLOAT16 = 6
    CT_FLOAT32 = 7


class NormType(enum.IntEnum):
    NONE = 0
    BATCHNORM = 1


class LayerType(enum.IntEnum):
    """fyusenet/base/layerflags.h:125-160 (same numeric values)."""
    ADD = 1
    SUB = 2
    ARGMAX = 3
    CAST = 4
    CONCAT = 5
    CONVOLUTION2D = 6
    FRACCONVOLUTION2D = 7
    TRANSCONVOLUTION2D = 8
    AVGPOOL2D = 9
    MAXPOOL2D = 10
    PADDING2D = 11
    SCALE2D = 12
    SINGLETON_ARITH = 13
    RELU = 14
    CLIP = 15
    TANH = 16
    SIGMOID = 17
    REDUCE = 18
    TRANSPOSE = 19
    IMGEXTRACT = 20
    BLUR2D = 21
    NONMAX2D = 22
    RGB2BGR = 23
    DEEP2SHALLOW = 24
    SHALLOW2DEEP = 25
    DOWNLOAD = 26
    UPLOAD = 27
    RESIDUAL = 28
    OESCONV = 29
    BATCHNORM = 30
    GEMM = 31
    CUSTOM = 32
    LAST_SUPPORTED = 33
    ILLEGAL = 1000


class LayerBuilder:
    def __init__(self, name):
        self.name_ = name
        self.inputPadding_ = 0
        self.outputPadding_ = 0
        self.residualPadding_ = 0
        self.downsample_ = [1, 1]
        self.upsample_ = [1, 1]
        self.preAct_ = ActType.NONE
        self.postAct_ = ActType.NONE
        self.resAct_ = ActType.NONE
        self.postNorm_ = NormType.NONE
        self.leakyReLU_ = 0.0
        self.clipLow_ = 0.0
        self.clipHigh_ = 0.0
        self.number_ = -1
        self.type_ = LayerType.ILLEGAL
        self.residualNorm_ = False
        self.width_ = 0
        self.height_ = 0
        self.inputChannels_ = 0
        self.outputChannels_ = 0
        self.flags_ = LayerFlags.NO_LAYER_FLAGS

    # -- fluent setters (base/layerbuilder.h:88-410) --
    def push(self, factory):
        factory.pushBuilder(self)
        return self

    def type(self, t):
        self.type_ = LayerType(t)
        return self

    def number(self, no):
        assert no >= 0
        self.number_ = no
        return self

    def size(self, width, height):
        self.width_, self.height_ = width, height
        return self

    def downsample(self, horizontal, vertical=None):
        self.downsample_ = [horizontal, horizontal if vertical is None else vertical]
        return self

    def upsample(self, horizontal, vertical=None):
        self.upsample_ = [horizontal, horizontal if vertical is None else vertical]
        return self

    def inputPadding(self, padding):
        self.inputPadding_ = padding
        return self

    def residualPadding(self, padding):
        self.residualPadding_ = padding
        return self

    def outputPadding(self, padding):
        self.outputPadding_ = padding
        return self

    def prefixAct(self, act):
        self.preAct_ = ActType(act)
        return self

    def postfixAct(self, act):
        self.postAct_ = ActType(act)
        return self

    def postfixNorm(self, nrm):
        self.postNorm_ = NormType(nrm)
        return self

    def deep(self):
        self.flags_ |= LayerFlags.DEEP
        return self

    def residual(self, act=ActType.NONE, postfixNorm=False):
        if act not in (ActType.RELU, ActType.NONE):
            raise capi.FynException(capi.ERR_INVALID, "Activation type %d not supported on residual" % int(act))
        self.flags_ |= LayerFlags.RESIDUAL_INPUT
        if act == ActType.RELU:
            self.flags_ |= LayerFlags.RELU_ON_RESIDUAL
        else:
            self.flags_ &= ~LayerFlags.RELU_ON_RESIDUAL
        self.residualNorm_ = postfixNorm
        return self

    def shape(self, *args):
        """shape(outChannels, height, width, inChannels) or shape(height, width, channels)."""
        if len(args) == 4:
            self.outputChannels_, self.height_, self.width_, self.inputChannels_ = args
        elif len(args) == 3:
            self.height_, self.width_, ch = args
            self.inputChannels_ = self.outputChannels_ = ch
        else:
            raise TypeError("shape() takes 3 or 4 arguments")
        return self

    def channels(self, channels):
        self.inputChannels_ = self.outputChannels_ = channels
        return self

    def inChannels(self, channels):
        self.inputChannels_ = channels
        return self

    def outChannels(self, channels):
        self.outputChannels_ = channels
        return self

    def leakyReLU(self, leak):
        self.leakyReLU_ = leak
        return self

    def clip(self, low, high):
        self.clipLow_, self.clipHigh_ = low, high
        return self

    def width(self):
        return self.width_

    def height(self):
        return self.height_

    def in_(self):
        return self.inputChannels_

    def out(self):
        return self.outputChannels_

    def isDeep(self):
        return bool(self.flags_ & LayerFlags.DEEP)

    def getFlags(self):
        """base/layerbuilder.h:445-493, including its quirk that residual(act, True) always sets
        BATCHNORM_ON_RESIDUAL (the test `residualNorm_ && POST_BATCHNORM` is constant-true)."""
        full = LayerFlags(self.flags_)
        if self.preAct_ in (ActType.RELU, ActType.LEAKY_RELU):
            full |= LayerFlags.PRE_RELU
        elif self.preAct_ == ActType.CLIP:
            full |= LayerFlags.PRE_CLIP
        elif self.preAct_ in (ActType.SIGMOID, ActType.TANH):
            raise capi.FynException(capi.ERR_UNSUPPORTED, "Activation type not supported yet")
        if self.postAct_ in (ActType.RELU, ActType.LEAKY_RELU):
            full |= LayerFlags.POST_RELU
        elif self.postAct_ != ActType.NONE:
            raise capi.FynException(capi.ERR_UNSUPPORTED, "Activation type not supported yet")
        if self.postNorm_ == NormType.BATCHNORM:
            full |= LayerFlags.POST_BATCHNORM
        if self.resAct_ == ActType.RELU:
            full |= LayerFlags.RELU_ON_RESIDUAL
        if self.residualNorm_:
            full |= LayerFlags.BATCHNORM_ON_RESIDUAL
        return full

    # -- conversion to the C ABI struct --
    def desc(self):
        d = capi.LayerDesc()
        d.struct_size = capi.ctypes.sizeof(capi.LayerDesc)
        d.type = int(self.type_)
        d.number = self.number_
        d.name = self.name_.encode()[: capi.FYN_NAME_LEN - 1]
        flags = self.getFlags()
        if flags & LayerFlags.POST_RELU:
            # base/layerflags.h:41: POST_RELU is "not supported by GPU layers"
            raise capi.FynException(capi.ERR_UNSUPPORTED, "postfix activation is not supported by GPU layers")
        d.flags = int(flags)
        d.width, d.height = self.width_, self.height_
        d.in_channels, d.out_channels = self.inputChannels_, self.outputChannels_
        d.input_padding, d.output_padding, d.residual_padding = self.inputPadding_, self.outputPadding_, self.residualPadding_
        d.downsample[0], d.downsample[1] = self.downsample_
        d.upsample[0], d.upsample[1] = self.upsample_
        d.leaky_relu = self.leakyReLU_ if self.preAct_ == ActType.LEAKY_RELU else 0.0
        d.clip_low, d.clip_high = self.clipLow_, self.clipHigh_
        d.kernel = 1
        d.dilation[0] = d.dilation[1] = 1
        d.group_size = 1
        d.pool_size[0] = d.pool_size[1] = 1
        self._fill(d)
        return d

    def _fill(self, d):
        pass


class GPULayerBuilder(LayerBuilder):
    def context(self, ctx):  # GL context link of the reference; no meaning here
        return self


class ConvLayerBuilder(GPULayerBuilder):
    def __init__(self, kernel, name):
        super().__init__(name)
        self.kernel_ = kernel
        self.dilation_ = [1, 1]
        self.groupSize_ = 1
        self.sourceStep_ = 1.0
        self.transconvCrop_ = 0
        self.type_ = LayerType.CONVOLUTION2D

    def dilation(self, horizontal, vertical=None):
        self.dilation_ = [horizontal, horizontal if vertical is None else vertical]
        return self

    def sourceStep(self, step):
        self.sourceStep_ = step
        return self

    def groupSize(self, gs):
        self.groupSize_ = gs
        return self

    def crop(self, n):
        """Extension (no reference counterpart): crop of a transposed convolution's full result."""
        self.transconvCrop_ = n
        return self

    def _fill(self, d):
        d.kernel = self.kernel_
        d.dilation[0], d.dilation[1] = self.dilation_
        d.group_size = self.groupSize_
        d.transconv_crop = self.transconvCrop_
        d.source_step = self.sourceStep_


class PoolLayerBuilder(GPULayerBuilder):
    POOL_AVG = 0
    POOL_MAX = 1

    def __init__(self, poolOp, name):
        super().__init__(name)
        self.operation_ = poolOp
        self.poolsize_ = [1, 1]
        self.global_ = False
        self.type_ = LayerType.AVGPOOL2D if poolOp == self.POOL_AVG else LayerType.MAXPOOL2D

    def poolSize(self, winx, winy=None):
        self.poolsize_ = [winx, winx if winy is None else winy]
        return self

    def global_pool(self):
        """PoolLayerBuilderTempl::global() (gpu/poollayerbuilder.h); `global` is a Python keyword."""
        if self.width_ == 0 or self.height_ == 0:
            raise capi.FynException(capi.ERR_INVALID, "Must set size before specifying global pooling")
        self.downsample_ = [self.width_, self.height_]
        self.global_ = True
        self.poolsize_ = [self.width_, self.height_]
        return self

    def _fill(self, d):
        d.pool_size[0], d.pool_size[1] = self.poolsize_
        d.global_pool = 1 if self.global_ else 0


class ConcatLayerBuilder(GPULayerBuilder):
    def __init__(self, name):
        super().__init__(name)
        self.type_ = LayerType.CONCAT
        self.inputs_ = []

    def input(self, channels, padding, flags=LayerFlags.NO_LAYER_FLAGS):
        self.inputs_.append((channels, padding, int(flags)))
        self.inputChannels_ += channels
        return self

    def _fill(self, d):
        if len(self.inputs_) > capi.FYN_MAX_CONCAT_INPUTS:
            raise capi.FynException(capi.ERR_UNSUPPORTED, "too many concat inputs")
        d.num_inputs = len(self.inputs_)
        for i, (c, p, f) in enumerate(self.inputs_):
            d.inputs[i].channels, d.inputs[i].padding, d.inputs[i].flags = c, p, f


class ArgMaxLayerBuilder(GPULayerBuilder):
    def __init__(self, name):
        super().__init__(name)
        self.type_ = LayerType.ARGMAX


class UpDownLayerBuilder(GPULayerBuilder):
    UPLOAD = 0
    DOWNLOAD = 1

    def __init__(self, direction, name):
        super().__init__(name)
        self.direction_ = direction
        self.type_ = LayerType.UPLOAD if direction == self.UPLOAD else LayerType.DOWNLOAD


class ScaleLayerBuilder(GPULayerBuilder):
    """gpu/scalelayerbuilder.h:38-135: integer up-/down-scaling, nearest or linear; also the builder of RELU,
    CLIP and PADDING2D layers, which the factory maps to a scale layer (gpu/gpulayerfactory.cpp:125-140)."""

    def __init__(self, name):
        super().__init__(name)
        self.type_ = LayerType.SCALE2D
        self.scaleType_ = ScalingType.NEAREST
        self.rotation_ = 0

    def scaleType(self, typ):
        self.scaleType_ = ScalingType(typ)
        return self

    def rotate(self, angle):
        self.rotation_ = angle
        return self

    def scale(self, scaleX, scaleY=None):
        scaleY = scaleX if scaleY is None else scaleY
        for axis, sc in ((0, scaleX), (1, scaleY)):
            if sc > 1.0:
                self.upsample_[axis] = int(sc)
                if abs(self.upsample_[axis] - sc) > 1e-4:
                    raise capi.FynException(capi.ERR_INVALID, "Only supporting integer upscales for now")
            elif sc < 1.0:
                dn = 1.0 / sc
                self.downsample_[axis] = int(dn + 1e-6)
                if abs(self.downsample_[axis] - dn) > 1e-4:
                    raise capi.FynException(capi.ERR_INVALID, "Only supporting integer downscales for now")
        return self

    def equal(self):
        return self.upsample_[0] == self.upsample_[1] and self.downsample_[0] == self.downsample_[1]

    def _fill(self, d):
        if self.rotation_ % 360 != 0:
            raise capi.FynException(capi.ERR_UNSUPPORTED, "rotation in scale layers is not supported")
        d.scale_type = int(self.scaleType_)


class SingletonArithLayerBuilder(GPULayerBuilder):
    def __init__(self, name, optype):
        super().__init__(name)
        self.type_ = LayerType.SINGLETON_ARITH
        self.opType_ = ArithType(optype)
        self.operand_ = 0.0

    def operand(self, opd):
        self.operand_ = float(opd)
        return self

    def _fill(self, d):
        d.arith_op = int(self.opType_)
        d.operand = self.operand_


class CastLayerBuilder(GPULayerBuilder):
    def __init__(self, name, target):
        super().__init__(name)
        self.type_ = LayerType.CAST
        self.target_ = CastTarget(target)

    def target(self, tgt):
        self.target_ = CastTarget(tgt)
        return self

    def _fill(self, d):
        d.cast_target = int(self.target_)


class TransposeLayerBuilder(GPULayerBuilder):
    def __init__(self, name):
        super().__init__(name)
        self.type_ = LayerType.TRANSPOSE

    def equal(self):
        return True


class ImgExtractLayerBuilder(GPULayerBuilder):
    def __init__(self, window, name):
        super().__init__(name)
        self.type_ = LayerType.IMGEXTRACT
        self.window_ = window
        self.downsample_ = [window, window]

    def _fill(self, d):
        d.window = self.window_


class BlurLayerBuilder(GPULayerBuilder):
    def __init__(self, name):
        super().__init__(name)
        self.type_ = LayerType.BLUR2D
        self.kernel_ = 3
        self.blurType_ = BlurKernelType.AVERAGE

    def kernel(self, sz):
        self.kernel_ = sz
        return self

    def blurType(self, typ):
        self.blurType_ = BlurKernelType(typ)
        return self

    def _fill(self, d):
        d.kernel = self.kernel_
        d.blur_type = int(self.blurType_)


class CustomLayerBuilder(GPULayerBuilder):
    """gpu/customlayerbuilder.h:53-90: `initCallback(builder)` returns the layer object.  Here that object provides
    forward(inputs, output, stream, sequence) and optionally setup(inputs, output) and cleanup(); inputs/output are
    capi.TensorView structures of device tensors, `stream` the hipStream_t (as an integer) to enqueue work on."""

    def __init__(self, name, initCallback):
        super().__init__(name)
        self.type_ = LayerType.CUSTOM
        self.initCallback_ = initCallback
        self.inputs_ = []

    def input(self, channels, padding):
        self.inputs_.append((channels, padding))
        return self

    def init(self):
        return self.initCallback_(self)

    def _fill(self, d):
        d.num_inputs = len(self.inputs_)
        for i, (c, p) in enumerate(self.inputs_):
            d.inputs[i].channels, d.inputs[i].padding, d.inputs[i].flags = c, p, 0
