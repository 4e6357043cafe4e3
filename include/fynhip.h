/*
 * fynhip -- C ABI of the MI355X (gfx950) engine for FyuseNet's GPU layer stack.
 *
 * The reference exposes this path only as C++ classes; every entry point below names the reference
 * interface it stands in for (paths relative to the reference tree).  All functions return 0 on
 * success and a negative fyn_status on failure (exceptions never cross this boundary; the message the
 * reference would have put into a FynException is available from fyn_last_error()).
 *
 * Threading: like NeuralNetwork::forward (fyusenet/base/neuralnetwork.cpp:169) a network is not
 * re-entrant; one thread drives one network.  Different networks may be driven from different
 * threads.  Pointers passed in are borrowed for the duration of the call only (weights are copied
 * and repacked, as in fyusenet/gpu/deep/deepconvlayerbase.cpp:308-353).
 */
#ifndef FYNHIP_H
#define FYNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct fyn_net fyn_net; /* opaque: NeuralNetwork + Engine + BufferManager of one network */

enum fyn_status {
    FYN_OK = 0,
    FYN_ERR_INVALID = -1,     /* bad argument / inconsistent description (reference: FynException)   */
    FYN_ERR_UNSUPPORTED = -2, /* layer type / kernel size not supported (gpulayerfactory.cpp:182)    */
    FYN_ERR_STATE = -3,       /* call out of order (forward before setup, add after setup ...)       */
    FYN_ERR_DEVICE = -4,      /* HIP runtime error                                                  */
    FYN_ERR_NOTFOUND = -5,    /* unknown layer number                                               */
    FYN_ERR_DUPLICATE = -6    /* layer number already in use (base/layerfactory.cpp:73)              */
};

/* Storage type of activations and weights.  FYN_STORAGE_F32 is the reference's HIGH_PRECISION build,
 * FYN_STORAGE_F16 its default build (fyusenet/gpu/gpulayerbase.h:100-110). */
enum fyn_storage { FYN_STORAGE_F32 = 0, FYN_STORAGE_F16 = 1 };

/* Numeric values of LayerType (fyusenet/base/layerflags.h:125-160); only the types of the GPU layer
 * stack handled here are listed, any other value yields FYN_ERR_UNSUPPORTED. */
enum fyn_layer_type {
    FYN_LAYER_ADD = 1,
    FYN_LAYER_SUB = 2,
    FYN_LAYER_ARGMAX = 3,
    FYN_LAYER_CAST = 4,
    FYN_LAYER_CONCAT = 5,
    FYN_LAYER_CONVOLUTION2D = 6,
    FYN_LAYER_FRACCONVOLUTION2D = 7, /* shallow only, like the reference (gpu/gpulayerfactory.cpp:447-456) */
    FYN_LAYER_TRANSCONVOLUTION2D = 8,
    FYN_LAYER_AVGPOOL2D = 9,
    FYN_LAYER_MAXPOOL2D = 10,
    FYN_LAYER_PADDING2D = 11,
    FYN_LAYER_SCALE2D = 12,
    FYN_LAYER_SINGLETON_ARITH = 13,
    FYN_LAYER_RELU = 14,
    FYN_LAYER_CLIP = 15,
    FYN_LAYER_TANH = 16,
    FYN_LAYER_SIGMOID = 17,
    FYN_LAYER_TRANSPOSE = 19,
    FYN_LAYER_IMGEXTRACT = 20,
    FYN_LAYER_BLUR2D = 21,
    FYN_LAYER_NONMAX2D = 22,
    FYN_LAYER_RGB2BGR = 23,
    FYN_LAYER_DEEP2SHALLOW = 24,
    FYN_LAYER_SHALLOW2DEEP = 25,
    FYN_LAYER_DOWNLOAD = 26,
    FYN_LAYER_UPLOAD = 27,
    FYN_LAYER_BATCHNORM = 30,
    FYN_LAYER_GEMM = 31,
    FYN_LAYER_CUSTOM = 32 /* only through fyn_net_add_custom_layer */
};

/* LayerFlags bits (fyusenet/base/layerflags.h:33-50), as LayerBuilderTempl::getFlags() composes them
 * (fyusenet/base/layerbuilder.h:445-493). */
enum fyn_layer_flags {
    FYN_FLAG_RESIDUAL_INPUT = 1,
    FYN_FLAG_RELU_ON_RESIDUAL = 2,
    FYN_FLAG_BATCHNORM_ON_RESIDUAL = 4,
    FYN_FLAG_POST_BATCHNORM = 8,
    FYN_FLAG_DEEP = 16,
    FYN_FLAG_PRE_RELU = 64,
    FYN_FLAG_PRE_CLIP = 128
};

/* ActType (fyusenet/base/layerflags.h:61-68). */
enum fyn_act { FYN_ACT_NONE = 0, FYN_ACT_RELU = 1, FYN_ACT_LEAKY_RELU = 2, FYN_ACT_CLIP = 3 };

/* Host buffer orders (CPUBufferShape::order, fyusenet/cpu/cpubuffershape.h). */
enum fyn_order {
    FYN_ORDER_CHANNELWISE = 0, /* [C][H][W]                                                         */
    FYN_ORDER_GPU_SHALLOW = 1, /* [H][W][pc] interleaved, pc = channels (<= 4 channels per texel)    */
    FYN_ORDER_GPU_DEEP = 2     /* tiled RGBA, cpu/cpubuffer.cpp:413-442, cpubuffershape.cpp:430-448  */
};

#define FYN_MAX_CONCAT_INPUTS 8
#define FYN_NAME_LEN 64

/*
 * One layer description: the fields of LayerBuilderTempl (fyusenet/base/layerbuilder.h:497-521) plus
 * those of ConvLayerBuilder (gpu/convlayerbuilder.h), PoolLayerBuilder (gpu/poollayerbuilder.h),
 * ConcatLayerBuilder (gpu/concatlayerbuilder.h) and the builders of the function-type layers.  The struct is copied by fyn_net_add_layer; no
 * ownership is taken.  Zero-initialise it, set struct_size = sizeof(fyn_layer_desc), fill what the
 * builder would have filled.  width/height/in_channels describe the INPUT tensor, as shape() does.
 */
typedef struct fyn_layer_desc {
    uint32_t struct_size;
    int32_t type;   /* fyn_layer_type                                                   type()            */
    int32_t number; /* unique, layers execute in ascending number                       number()          */
    char name[FYN_NAME_LEN];
    uint32_t flags; /* fyn_layer_flags                                                  getFlags()        */
    int32_t width, height, in_channels, out_channels; /*                               shape()           */
    int32_t input_padding, output_padding, residual_padding; /*          inputPadding() ...               */
    int32_t downsample[2]; /* x, y                                                      downsample()      */
    int32_t upsample[2];   /* x, y                                                      upsample()        */
    float leaky_relu;      /* != 0 with PRE_RELU: leaky ReLU                            leakyReLU()       */
    float clip_low, clip_high; /* with PRE_CLIP                                         clip()            */
    /* convolution family */
    int32_t kernel;      /* isotropic kernel size                                       ConvLayerBuilder  */
    int32_t dilation[2]; /*                                                             dilation()        */
    int32_t group_size;  /* == in_channels and kernel 3: depthwise                      groupSize()       */
    /* pooling */
    int32_t pool_size[2]; /*                                                            poolSize()        */
    int32_t global_pool;  /*                                                            global()          */
    /* concatenation */
    int32_t num_inputs;
    struct {
        int32_t channels, padding;
        uint32_t flags;
    } inputs[FYN_MAX_CONCAT_INPUTS]; /*                                                  input()           */
    /* Extension without a reference counterpart: rows/columns cropped from the end of a transposed
     * convolution's full (2H+K-2) result; 0 reproduces the reference's deep layer size
     * (gpu/deep/deeptiler.cpp:71-74), 1 with K=3 yields the 2H size of the shallow layer
     * (gpu/vanilla/transconvlayerbase_vanilla.cpp:61-62). */
    int32_t transconv_crop;
    /* function-type layers */
    int32_t scale_type;  /* SCALE2D: ScalingType 0 nearest, 1 linear      ScaleLayerBuilder::scaleType() (gpu/scalelayerbuilder.h) */
    int32_t arith_op;    /* SINGLETON_ARITH: ArithType 0 add 1 sub 2 mul 3 div  (gpu/singleton_arithlayerbuilder.h)             */
    float operand;       /*                                                SingletonArithLayerBuilder::operand()                */
    int32_t cast_target; /* CAST: CastTarget 0..7 (base/layerflags.h:121-130)  CastLayerBuilder::target()                       */
    int32_t window;      /* IMGEXTRACT: window size                        ImgExtractLayerBuilder (gpu/imgextractlayerbuilder.h) */
    int32_t blur_type;   /* BLUR2D: BlurKernelType 0 average, 1 Gaussian; size in `kernel`  (gpu/blurlayerbuilder.h)            */
    float source_step;   /* FRACCONVOLUTION2D: step on the input per tap, 1/2, 1/4 ...; 0 reads as 1  ConvLayerBuilder::sourceStep() (gpu/convlayerbuilder.h:80) */
} fyn_layer_desc;

/* Thread-local text of the last failure (what the reference would have thrown). */
const char* fyn_last_error(void);

/* Library / device information: writes a short text (device name, CU count, arch) into buf. */
int fyn_device_info(int device, char* buf, size_t buflen);

/* NeuralNetwork construction (fyusenet/base/neuralnetwork.h:62-261); storage = fyn_storage. */
int fyn_net_create(int device, int storage, fyn_net** out);
/* NeuralNetwork::cleanup + destructor (base/neuralnetwork.cpp:57-79). */
int fyn_net_destroy(fyn_net* net);

/* LayerFactory::pushBuilder + LayerFactoryBackend::createLayer (base/layerfactory.cpp:67-101,
 * gpu/gpulayerfactory.cpp:112-184). */
int fyn_net_add_layer(fyn_net* net, const fyn_layer_desc* desc);

/* A device tensor as a custom layer sees it: channel-packed NHWC with a zero halo.  Element (y, x, c) of the net
 * area lives at data[((y + padding) * (width + 2*padding) + (x + padding)) * channel_pitch + c]; the element type is
 * float (storage FYN_STORAGE_F32) or IEEE half (FYN_STORAGE_F16).  Channels [channels, channel_pitch) and the halo
 * of an output must stay zero. */
typedef struct fyn_tensor_view {
    void* data;
    int32_t channels, height, width, padding, channel_pitch, storage;
} fyn_tensor_view;

/* User-supplied layer: the C form of CustomLayerBuilder's init callback returning a GPULayerBase subclass
 * (fyusenet/gpu/customlayerbuilder.h:53-90, gpu/gpulayerfactory.cpp:586-589).  `forward` must only ENQUEUE work on
 * the given hipStream_t (it is called once while a forward pass is being captured when fyn_net_use_graph is on, and
 * the enqueued work is what later passes replay); a non-zero return fails the pass.  `setup` (after the tensors
 * exist) and `cleanup` (when the network is destroyed) may be NULL.  The struct is copied. */
typedef struct fyn_custom_layer {
    void* user;
    int (*setup)(void* user, const fyn_tensor_view* inputs, int num_inputs, const fyn_tensor_view* output);
    int (*forward)(void* user, const fyn_tensor_view* inputs, int num_inputs, const fyn_tensor_view* output, void* hip_stream,
                   uint64_t sequence);
    void (*cleanup)(void* user);
} fyn_custom_layer;
/* desc->type must be FYN_LAYER_CUSTOM.  Input ports: desc->num_inputs ports of desc->inputs[i].channels/.padding (all
 * width x height), or, with num_inputs == 0, one port of in_channels/input_padding (plus a residual port with
 * FYN_FLAG_RESIDUAL_INPUT).  Output: out_channels x (height*upsample/downsample) x (width*...), output_padding. */
int fyn_net_add_custom_layer(fyn_net* net, const fyn_layer_desc* desc, const fyn_custom_layer* impl);

/* BufferManager::connectLayers(outputLayer, inputLayer, port) (base/buffermanager.cpp:160-184):
 * port 0 = data, port 1 = residual; concat ports 0..N-1. */
int fyn_net_connect(fyn_net* net, int out_layer, int in_layer, int port);

/* ConvLayerInterface::loadWeightsAndBiases(const float*, size_t offset) (base/convlayerinterface.h:95):
 * block at wb+offset = [bias][weights [o][ky][kx][i]][bnScale][bnBias].  May be called again after
 * setup to swap weights (samples/samplenetworks/stylenet3x3.cpp:81-89); a captured forward pass (fyn_net_use_graph) is
 * captured again on the next fyn_net_forward. */
int fyn_layer_load_weights(fyn_net* net, int layer, const float* wb, size_t offset_floats);
/* BatchNormInterface::loadScaleAndBias (base/batchnorminterface.h:146): [scale C][bias C]. */
int fyn_layer_load_scale_bias(fyn_net* net, int layer, const float* sb, size_t offset_floats);
/* Number of floats the layer's block occupies (to step through a .dat stream). */
int fyn_layer_weight_floats(fyn_net* net, int layer, size_t* count);

/* NeuralNetwork::setup -> glSetup (base/neuralnetwork.cpp:88-103,238-250): allocates device tensors,
 * packs weights, selects kernels. */
int fyn_net_setup(fyn_net* net);

/* UploadLayer::setInputBuffer + upload (gpu/uploadlayer.cpp:92-186): host fp32 buffer in `order`
 * for the UPLOAD layer `layer`; for any other layer: writes the tensor on input port `port`
 * directly (what LayerTestBase::generateTextures does, unit_tests/layertestbase.cpp:208-417). */
int fyn_net_set_input(fyn_net* net, int layer, int port, const float* data, int order);
/* Number of floats fyn_net_set_input reads from `data` for that layer and port (channels x height x width; the size
 * the CPUBuffer handed to UploadLayer::setInputBuffer must have). */
int fyn_net_input_floats(fyn_net* net, int layer, int port, size_t* count);

/* NeuralNetwork::forward (base/neuralnetwork.cpp:173-187): runs all layers in ascending number on
 * the network's stream; returns the sequence number used.  Asynchronous w.r.t. the host. */
int fyn_net_forward(fyn_net* net, uint64_t* seq_out);
/* NeuralNetwork::finish (base/neuralnetwork.cpp:196-206): waits for the stream. */
int fyn_net_finish(fyn_net* net);

/* GPULayerBase::copyResult(float*, bool) (gpu/gpulayerbase.cpp:525-564): output of `layer` as CHW
 * fp32; include_padding != 0 keeps the output halo.  Synchronises. */
int fyn_layer_copy_result(fyn_net* net, int layer, float* chw, int include_padding);
/* fyn_layer_copy_result for callers that cannot allocate (code under HIP graph capture on another stream, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The layout conversion goes through
 * a fixed device array of FYN_STATIC_SCRATCH_FLOATS floats that is part of the library's code object (one per GPU, held
 * until the process ends; its device address is looked up when the network is created) instead of the growable staging
 * area of fyn_layer_copy_result; no hipMalloc/hipFree is called.  A result with more floats is refused with
 * FYN_ERR_INVALID.  `chw` may be host memory (pinned memory keeps the HIP runtime from staging the copy itself) or
 * device memory.  All networks on one GPU share the array: calls that overlap on one GPU (from different threads) race;
 * every call overwrites all of the part it uses, so nothing of an earlier call is ever read.  Synchronises. */
#define FYN_STATIC_SCRATCH_FLOATS (8u << 20) /* 32 MiB */
int fyn_layer_copy_result_noalloc(fyn_net* net, int layer, float* chw, int include_padding);
/* Output geometry of a layer: channels, height, width (net size) and padding. */
int fyn_layer_output_shape(fyn_net* net, int layer, int* channels, int* height, int* width, int* padding);
/* DownloadLayer / CPUBuffer formats (gpu/deep/deepdownloadlayer.cpp:136-162, cpu/cpubuffer.cpp):
 * output of `layer` (padding stripped unless GPU_DEEP, which keeps the layer's output padding) as
 * fp32 in the requested fyn_order.  Synchronises. */
int fyn_net_get_output(fyn_net* net, int layer, float* data, int order);
/* ArgMax result as integers (index per pixel), the exact form of deepargmax2.frag's first channel. */
int fyn_layer_copy_argmax(fyn_net* net, int layer, int32_t* idx, float* val);

/* Engine::enableTimings / resetTimings (base/engine.cpp:208-233); here per-layer GPU time from
 * hipEvents.  fyn_net_get_timing returns the accumulated milliseconds and run count of one layer. */
int fyn_net_enable_timings(fyn_net* net, int enable);
int fyn_net_get_timing(fyn_net* net, int layer, float* ms_total, int* runs);
/* Engine::enableIntermediateOutput(dir) (base/engine.cpp:174-181): <name>_<seq>.bin CHW fp32 dumps. */
int fyn_net_enable_intermediate_output(fyn_net* net, const char* dir);

/* Output-buffer sharing between layers whose lifetimes do not overlap (the texture pool of
 * BufferManager::findTexture, base/buffermanager.cpp:512-525).  On by default; switch off before
 * fyn_net_setup to keep every intermediate tensor readable with fyn_layer_copy_result after forward.
 * With sharing on, an intermediate tensor may also never be written: a depthwise 3x3 layer and a 1x1
 * convolution next to it can run as one launch when nothing else reads the tensor between them, a
 * plain batch-norm layer is applied on fetch by the convolutions that read it, and a 1x1 shortcut
 * projection is computed by the 1x1 layer that adds it. */
int fyn_net_set_buffer_reuse(fyn_net* net, int enable);

/* Replays forward() from a captured hipGraph (launch-latency removal; no reference counterpart). */
int fyn_net_use_graph(fyn_net* net, int enable);

/* Measurement helpers (no reference counterpart): time `iters` forwards between two hipEvents on the
 * network's stream; per-layer variant times one layer's kernels alone.  Milliseconds total. */
int fyn_net_time_forward(fyn_net* net, int iters, float* ms_total);
int fyn_layer_time(fyn_net* net, int layer, int iters, float* ms_total);
/* `iters` forward passes queued back to back with an event after each; ms_each[i] receives the GPU time between the
 * events around pass i (for medians and percentiles). */
int fyn_net_time_steps(fyn_net* net, int iters, float* ms_each);
/* Frame pipeline for streams of frames handed over in host memory -- the reference engine's asynchronous mode
 * (fyusenet/base/engine.cpp:386-683, two upload/download buffer sets: gpu/uploadlayer.h:74).  The upload of frame
 * i+1 and the download of frame i-1 overlap the layers of frame i (pinned staging buffers, three streams).
 *   begin : input = an upload layer (or an unconnected input port), output = any layer; `depth` frames in flight.
 *   submit: copies `in` (borrowed for the call) and queues the frame; `out` must stay valid until the frame's
 *           ticket has been waited for (it is filled then, or when its slot is reused `depth` submits later).
 *   wait  : blocks until the frame (and all earlier ones) has been delivered.   end: drains and frees the pipeline.
 * Orders: input CHANNELWISE or GPU_SHALLOW, output CHANNELWISE or GPU_SHALLOW.
 * copy_streams != 0: uploads and downloads run on two streams of the pipeline's own (overlap inside this network).
 * copy_streams == 0: they are queued on the network's stream, between the frames' layers; for several networks that
 * run side by side, whose frames overlap each other, and whose streams would otherwise outnumber the hardware queues
 * of the process (streams that share a queue wait for each other's events). */
int fyn_net_async_begin(fyn_net* net, int in_layer, int in_port, int in_order, int out_layer, int out_order, int depth, int copy_streams);
int fyn_net_async_submit(fyn_net* net, const float* in, float* out, uint64_t* ticket);
int fyn_net_async_wait(fyn_net* net, uint64_t ticket);
/* Floats per frame that submit reads from `in` and writes to `out` (between begin and end). */
int fyn_net_async_sizes(fyn_net* net, size_t* in_floats, size_t* out_floats);
int fyn_net_async_end(fyn_net* net);
/* Device allocations this network has made since fyn_net_create: number of hipMalloc calls and the bytes asked for
 * (both only ever grow).  A diagnostic without a counterpart in the reference, whose textures belong to the GL driver;
 * it lets a caller check that a call sequence of its serving loop allocates nothing. */
int fyn_net_device_allocations(fyn_net* net, size_t* calls, size_t* bytes);
/* Text description of the kernel variant chosen for a layer (for profiles / reports). */
int fyn_layer_kernel_info(fyn_net* net, int layer, char* buf, size_t buflen);

#ifdef __cplusplus
}
#endif
#endif /* FYNHIP_H */
