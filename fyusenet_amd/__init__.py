"""fyusenet_amd: MI355X (gfx950) engine for FyuseNet's GPU layer stack.

The arithmetic lives in libfynhip.so (hand-written HIP kernels + C++ host engine, C ABI in
include/fynhip.h); this package is the ctypes binding plus a Python mirror of the reference's
LayerBuilder / LayerFactory / NeuralNetwork description surface.  There is no CPU fallback: using the
package without the built library raises ImportError at the first call.
"""
from . import capi  # noqa: F401
from .builders import (ActType, ArgMaxLayerBuilder, ArithType, BlurKernelType, BlurLayerBuilder, CastLayerBuilder,  # noqa: F401
                       CastTarget, ConcatLayerBuilder, ConvLayerBuilder, CustomLayerBuilder, GPULayerBuilder, ImgExtractLayerBuilder,
                       LayerBuilder, LayerFlags, LayerType, NormType, PoolLayerBuilder, ScaleLayerBuilder, ScalingType,
                       SingletonArithLayerBuilder, TransposeLayerBuilder, UpDownLayerBuilder)
from .capi import FynException, ORDER_CHANNELWISE, ORDER_GPU_DEEP, ORDER_GPU_SHALLOW, STORAGE_F16, STORAGE_F32  # noqa: F401
from .network import BufferManager, CompiledLayers, FramePool, Layer, LayerFactory, NeuralNetwork  # noqa: F401
