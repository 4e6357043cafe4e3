/*
 * C++ description surface over the C ABI of fynhip.h: the builders, LayerFactory, CompiledLayers, BufferManager and
 * NeuralNetwork of the reference with their names, argument meaning and error behaviour, so that a network written
 * for the reference (samples/samplenetworks/resnet50.cpp, stylenet3x3.cpp) or one of its unit tests reads the same
 * here.  Header-only; link against libfynhip.so.  Nothing in here computes: every call ends in the C ABI.
 *
 *   LayerBuilderTempl        fyusenet/base/layerbuilder.h:53-558
 *   GPULayerBuilder          fyusenet/gpu/gpulayerbuilder.h
 *   ConvLayerBuilder         fyusenet/gpu/convlayerbuilder.h
 *   PoolLayerBuilder         fyusenet/gpu/poollayerbuilder.h
 *   ConcatLayerBuilder       fyusenet/gpu/concatlayerbuilder.h
 *   ArgMaxLayerBuilder       fyusenet/gpu/argmaxlayerbuilder.h
 *   UpDownLayerBuilder       fyusenet/gpu/updownlayerbuilder.h
 *   ScaleLayerBuilder        fyusenet/gpu/scalelayerbuilder.h
 *   SingletonArithLayerBuilder / CastLayerBuilder / TransposeLayerBuilder / ImgExtractLayerBuilder / BlurLayerBuilder /
 *   CustomLayerBuilder       fyusenet/gpu/ (one header per builder)
 *   LayerFactory             fyusenet/base/layerfactory.h:56-138, layerfactory.cpp:67-101
 *   CompiledLayers           fyusenet/base/compiledlayers.h:50-291
 *   BufferManager            fyusenet/base/buffermanager.cpp:160-184
 *   NeuralNetwork            fyusenet/base/neuralnetwork.h:62-261, neuralnetwork.cpp:88-250
 *   ConvLayerInterface       fyusenet/base/convlayerinterface.h:95
 *   BatchNormInterface       fyusenet/base/batchnorminterface.h:146
 *
 * The classes live in namespace fynhip (builders of GPU layers in fynhip::gpu).  Define FYNHIP_REFERENCE_NAMESPACE before
 * including this file to also reach them as fyusion::fyusenet / fyusion::fyusenet::gpu, the reference's namespaces.
 */
#ifndef FYNHIP_HPP
#define FYNHIP_HPP

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "fynhip.h"

namespace fynhip {

/* What the reference throws (fyusenet/common/fynexception.h); `status` is the C ABI's code. */
class FynException : public std::exception {
  public:
    FynException(int status, std::string msg) : status_(status), msg_(std::move(msg)) {}
    const char* what() const noexcept override { return msg_.c_str(); }
    int status() const { return status_; }

  private:
    int status_;
    std::string msg_;
};

namespace detail {
[[noreturn]] inline void raise(int status, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    throw FynException(status, buf);
}
inline void check(int status) {
    if (status != FYN_OK) {
        const char* m = fyn_last_error();
        throw FynException(status, m && *m ? m : "error " + std::to_string(status));
    }
}
}  // namespace detail

/* fyusenet/base/layerflags.h */
enum class LayerType : int {
    ADD = 1, SUB, ARGMAX, CAST, CONCAT, CONVOLUTION2D, FRACCONVOLUTION2D, TRANSCONVOLUTION2D, AVGPOOL2D, MAXPOOL2D,
    PADDING2D, SCALE2D, SINGLETON_ARITH, RELU, CLIP, TANH, SIGMOID, REDUCE, TRANSPOSE, IMGEXTRACT, BLUR2D, NONMAX2D,
    RGB2BGR, DEEP2SHALLOW, SHALLOW2DEEP, DOWNLOAD, UPLOAD, RESIDUAL, OESCONV, BATCHNORM, GEMM, CUSTOM, LAST_SUPPORTED,
    ILLEGAL = 1000
};
enum class ActType : int { NONE = 0, RELU, LEAKY_RELU, CLIP, SIGMOID, TANH };
enum class NormType : int { NONE = 0, BATCHNORM };
enum class ScalingType : int { NEAREST = 0, LINEAR };
enum class BlurKernelType : int { AVERAGE = 0, GAUSSIAN };
enum class ArithType : int { ADD = 0, SUB, MUL, DIV };
enum class CastTarget : int { CT_INT32 = 0, CT_INT16, CT_INT8, CT_UINT32, CT_UINT16, CT_UINT8, CT_FLOAT16, CT_FLOAT32 };
using layerflags = uint32_t;
namespace LayerFlags {
constexpr layerflags NO_LAYER_FLAGS = 0, RESIDUAL_INPUT = 1, RELU_ON_RESIDUAL = 2, BATCHNORM_ON_RESIDUAL = 4, POST_BATCHNORM = 8,
                     DEEP = 16, POST_RELU = 32, PRE_RELU = 64, PRE_CLIP = 128;
}

/* The GL context link that every reference builder carries; it has no meaning here and is accepted and ignored. */
struct GfxContextLink {};

class LayerFactory;

/* Fields of LayerBuilderTempl (base/layerbuilder.h:497-521) without the fluent interface. */
struct LayerBuilderData {
    explicit LayerBuilderData(std::string name) : name_(std::move(name)) {}
    virtual ~LayerBuilderData() = default;

    bool isDeep() const { return (flags_ & LayerFlags::DEEP) != 0; }
    int width() const { return width_; }
    int height() const { return height_; }
    int in() const { return inputChannels_; }
    int out() const { return outputChannels_; }

    /* base/layerbuilder.h:445-493, including its quirk that residual(act, true) always sets BATCHNORM_ON_RESIDUAL */
    layerflags getFlags() const {
        layerflags full = flags_;
        if (preAct_ == ActType::RELU || preAct_ == ActType::LEAKY_RELU) full |= LayerFlags::PRE_RELU;
        else if (preAct_ == ActType::CLIP) full |= LayerFlags::PRE_CLIP;
        else if (preAct_ != ActType::NONE) detail::raise(FYN_ERR_UNSUPPORTED, "Activation type not supported yet");
        if (postAct_ == ActType::RELU || postAct_ == ActType::LEAKY_RELU) full |= LayerFlags::POST_RELU;
        else if (postAct_ != ActType::NONE) detail::raise(FYN_ERR_UNSUPPORTED, "Activation type not supported yet");
        if (postNorm_ == NormType::BATCHNORM) full |= LayerFlags::POST_BATCHNORM;
        if (resAct_ == ActType::RELU) full |= LayerFlags::RELU_ON_RESIDUAL;
        if (residualNorm_) full |= LayerFlags::BATCHNORM_ON_RESIDUAL;
        return full;
    }

    /* The description handed to fyn_net_add_layer. */
    fyn_layer_desc desc() const {
        fyn_layer_desc d;
        std::memset(&d, 0, sizeof(d));
        d.struct_size = sizeof(d);
        d.type = static_cast<int32_t>(type_);
        d.number = number_;
        std::strncpy(d.name, name_.c_str(), FYN_NAME_LEN - 1);
        const layerflags f = getFlags();
        // base/layerflags.h:41: POST_RELU is "not supported by GPU layers"
        if (f & LayerFlags::POST_RELU) detail::raise(FYN_ERR_UNSUPPORTED, "postfix activation is not supported by GPU layers");
        d.flags = f;
        d.width = width_; d.height = height_;
        d.in_channels = inputChannels_; d.out_channels = outputChannels_;
        d.input_padding = inputPadding_; d.output_padding = outputPadding_; d.residual_padding = residualPadding_;
        d.downsample[0] = downsample_[0]; d.downsample[1] = downsample_[1];
        d.upsample[0] = upsample_[0]; d.upsample[1] = upsample_[1];
        d.leaky_relu = preAct_ == ActType::LEAKY_RELU ? leakyReLU_ : 0.f;
        d.clip_low = clipLow_; d.clip_high = clipHigh_;
        d.kernel = 1;
        d.dilation[0] = d.dilation[1] = 1;
        d.group_size = 1;
        d.pool_size[0] = d.pool_size[1] = 1;
        fill(d);
        return d;
    }

    std::string name_;
    short inputPadding_ = 0, outputPadding_ = 0, residualPadding_ = 0;
    short downsample_[2] = {1, 1}, upsample_[2] = {1, 1};
    ActType preAct_ = ActType::NONE, postAct_ = ActType::NONE, resAct_ = ActType::NONE;
    NormType postNorm_ = NormType::NONE;
    float leakyReLU_ = 0.f, clipLow_ = 0.f, clipHigh_ = 0.f;
    int number_ = -1;
    LayerType type_ = LayerType::ILLEGAL;
    bool residualNorm_ = false;
    int width_ = 0, height_ = 0, inputChannels_ = 0, outputChannels_ = 0;
    layerflags flags_ = LayerFlags::NO_LAYER_FLAGS;

  protected:
    virtual void fill(fyn_layer_desc&) const {}
};

/* The fluent setters (base/layerbuilder.h:88-410); every setter returns the most derived builder, as in the reference. */
template <typename D>
struct LayerBuilderTempl : LayerBuilderData {
    using LayerBuilderData::LayerBuilderData;
    D& self() { return *static_cast<D*>(this); }

    /* Hands the builder to the factory, which owns and deletes it from then on: create builders with `new`, as the
     * reference's networks do (samples/samplenetworks/resnet50.cpp:200-423). */
    D& push(const std::shared_ptr<LayerFactory>& factory);
    D& push(LayerFactory& factory);

    D& type(LayerType t) { type_ = t; return self(); }
    D& number(int no) {
        if (no < 0) detail::raise(FYN_ERR_INVALID, "Illegal layer number %d", no);
        number_ = no;
        return self();
    }
    D& size(int width, int height) { width_ = width; height_ = height; return self(); }
    D& downsample(short ds) { downsample_[0] = downsample_[1] = ds; return self(); }
    D& downsample(short horizontal, short vertical) { downsample_[0] = horizontal; downsample_[1] = vertical; return self(); }
    D& upsample(short us) { upsample_[0] = upsample_[1] = us; return self(); }
    D& upsample(short horizontal, short vertical) { upsample_[0] = horizontal; upsample_[1] = vertical; return self(); }
    D& inputPadding(short padding) { inputPadding_ = padding; return self(); }
    D& residualPadding(short padding) { residualPadding_ = padding; return self(); }
    D& outputPadding(short padding) { outputPadding_ = padding; return self(); }
    D& prefixAct(ActType act) { preAct_ = act; return self(); }
    D& postfixAct(ActType act) { postAct_ = act; return self(); }
    D& postfixNorm(NormType nrm) { postNorm_ = nrm; return self(); }
    D& deep() { flags_ |= LayerFlags::DEEP; return self(); }
    D& residual(ActType act = ActType::NONE, bool postfixNorm = false) {
        if (act != ActType::RELU && act != ActType::NONE) detail::raise(FYN_ERR_INVALID, "Activation type %d not supported on residual", (int)act);
        flags_ |= LayerFlags::RESIDUAL_INPUT;
        if (act == ActType::RELU) flags_ |= LayerFlags::RELU_ON_RESIDUAL;
        else flags_ &= ~LayerFlags::RELU_ON_RESIDUAL;
        residualNorm_ = postfixNorm;
        return self();
    }
    D& shape(int outChannels, int height, int width, int inChannels) {
        outputChannels_ = outChannels; height_ = height; width_ = width; inputChannels_ = inChannels;
        return self();
    }
    D& shape(int height, int width, int channels) {
        height_ = height; width_ = width; inputChannels_ = outputChannels_ = channels;
        return self();
    }
    D& channels(int ch) { inputChannels_ = outputChannels_ = ch; return self(); }
    D& inChannels(int ch) { inputChannels_ = ch; return self(); }
    D& outChannels(int ch) { outputChannels_ = ch; return self(); }
    D& leakyReLU(float leak) { leakyReLU_ = leak; return self(); }
    D& clip(float low, float high) { clipLow_ = low; clipHigh_ = high; return self(); }
};

struct LayerBuilder : LayerBuilderTempl<LayerBuilder> {
    using LayerBuilderTempl<LayerBuilder>::LayerBuilderTempl;
};

namespace gpu {

template <typename D>
struct GPULayerBuilderTempl : LayerBuilderTempl<D> {
    using LayerBuilderTempl<D>::LayerBuilderTempl;
    D& context(const GfxContextLink&) { return this->self(); }
};
struct GPULayerBuilder : GPULayerBuilderTempl<GPULayerBuilder> {
    using GPULayerBuilderTempl<GPULayerBuilder>::GPULayerBuilderTempl;
};

template <typename D>
struct ConvLayerBuilderTempl : GPULayerBuilderTempl<D> {
    ConvLayerBuilderTempl(short kernel, const std::string& name) : GPULayerBuilderTempl<D>(name), kernel_(kernel) {
        this->type_ = LayerType::CONVOLUTION2D;
    }
    D& dilation(short dilate) { dilation_[0] = dilation_[1] = dilate; return this->self(); }
    D& dilation(short horizontal, short vertical) { dilation_[0] = horizontal; dilation_[1] = vertical; return this->self(); }
    D& sourceStep(float step) { sourceStep_ = step; return this->self(); }
    D& groupSize(short gs) { groupSize_ = gs; return this->self(); }
    /* Extension without a reference counterpart: rows/columns cropped from the end of a transposed convolution's result. */
    D& crop(int n) { transconvCrop_ = n; return this->self(); }

    short kernel_ = 1;
    short dilation_[2] = {1, 1};
    short groupSize_ = 1;
    float sourceStep_ = 1.f;
    int transconvCrop_ = 0;

  protected:
    void fill(fyn_layer_desc& d) const override {
        d.kernel = kernel_;
        d.dilation[0] = dilation_[0]; d.dilation[1] = dilation_[1];
        d.group_size = groupSize_;
        d.transconv_crop = transconvCrop_;
        d.source_step = sourceStep_;
    }
};
struct ConvLayerBuilder : ConvLayerBuilderTempl<ConvLayerBuilder> {
    using ConvLayerBuilderTempl<ConvLayerBuilder>::ConvLayerBuilderTempl;
};

template <typename D>
struct PoolLayerBuilderTempl : GPULayerBuilderTempl<D> {
    enum op { POOL_AVG = 0, POOL_MAX };
    PoolLayerBuilderTempl(op poolOp, const std::string& name) : GPULayerBuilderTempl<D>(name), operation_(poolOp) {
        this->type_ = poolOp == POOL_AVG ? LayerType::AVGPOOL2D : LayerType::MAXPOOL2D;
    }
    D& poolSize(short win) { poolsize_[0] = poolsize_[1] = win; return this->self(); }
    D& poolSize(short winx, short winy) { poolsize_[0] = winx; poolsize_[1] = winy; return this->self(); }
    D& global() {
        if (this->width_ == 0 || this->height_ == 0) detail::raise(FYN_ERR_INVALID, "Must set size before specifying global pooling");
        this->downsample_[0] = (short)this->width_; this->downsample_[1] = (short)this->height_;
        poolsize_[0] = (short)this->width_; poolsize_[1] = (short)this->height_;
        global_ = true;
        return this->self();
    }
    op operation_;
    short poolsize_[2] = {1, 1};
    bool global_ = false;

  protected:
    void fill(fyn_layer_desc& d) const override {
        d.pool_size[0] = poolsize_[0]; d.pool_size[1] = poolsize_[1];
        d.global_pool = global_ ? 1 : 0;
    }
};
struct PoolLayerBuilder : PoolLayerBuilderTempl<PoolLayerBuilder> {
    using PoolLayerBuilderTempl<PoolLayerBuilder>::PoolLayerBuilderTempl;
};

template <typename D>
struct ConcatLayerBuilderTempl : GPULayerBuilderTempl<D> {
    struct InputSpec {
        int channels, padding;
        layerflags flags;
    };
    explicit ConcatLayerBuilderTempl(const std::string& name) : GPULayerBuilderTempl<D>(name) { this->type_ = LayerType::CONCAT; }
    D& input(int channels, int padding, layerflags flags = LayerFlags::NO_LAYER_FLAGS) {
        inputs_.push_back(InputSpec{channels, padding, flags});
        this->inputChannels_ += channels;
        return this->self();
    }
    std::vector<InputSpec> inputs_;

  protected:
    void fill(fyn_layer_desc& d) const override {
        if (inputs_.size() > FYN_MAX_CONCAT_INPUTS) detail::raise(FYN_ERR_UNSUPPORTED, "too many concat inputs");
        d.num_inputs = (int)inputs_.size();
        for (size_t i = 0; i < inputs_.size(); i++) {
            d.inputs[i].channels = inputs_[i].channels; d.inputs[i].padding = inputs_[i].padding; d.inputs[i].flags = inputs_[i].flags;
        }
    }
};
struct ConcatLayerBuilder : ConcatLayerBuilderTempl<ConcatLayerBuilder> {
    using ConcatLayerBuilderTempl<ConcatLayerBuilder>::ConcatLayerBuilderTempl;
};

struct ArgMaxLayerBuilder : GPULayerBuilderTempl<ArgMaxLayerBuilder> {
    explicit ArgMaxLayerBuilder(const std::string& name) : GPULayerBuilderTempl<ArgMaxLayerBuilder>(name) { type_ = LayerType::ARGMAX; }
};

struct UpDownLayerBuilder : GPULayerBuilderTempl<UpDownLayerBuilder> {
    enum direction { UPLOAD = 0, DOWNLOAD };
    UpDownLayerBuilder(direction dir, const std::string& name) : GPULayerBuilderTempl<UpDownLayerBuilder>(name), direction_(dir) {
        type_ = dir == UPLOAD ? LayerType::UPLOAD : LayerType::DOWNLOAD;
    }
    /* The reference's asynchronous transfers with per-layer callbacks; frames overlap through the frame pipeline of
     * NeuralNetwork::asyncBegin here, so these only record the request. */
    UpDownLayerBuilder& async() { async_ = true; return *this; }
    direction direction_;
    bool async_ = false;
};

struct ScaleLayerBuilder : GPULayerBuilderTempl<ScaleLayerBuilder> {
    explicit ScaleLayerBuilder(const std::string& name) : GPULayerBuilderTempl<ScaleLayerBuilder>(name) { type_ = LayerType::SCALE2D; }
    ScaleLayerBuilder& scaleType(ScalingType typ) { scaleType_ = typ; return *this; }
    ScaleLayerBuilder& rotate(int angle) { rotation_ = angle; return *this; }
    /* gpu/scalelayerbuilder.h: isotropic or anisotropic integer factors, > 1 up, < 1 down */
    ScaleLayerBuilder& scale(float scaleX, float scaleY) {
        const float sc[2] = {scaleX, scaleY};
        for (int axis = 0; axis < 2; axis++) {
            if (sc[axis] > 1.f) {
                upsample_[axis] = (short)sc[axis];
                if (std::fabs((float)upsample_[axis] - sc[axis]) > 1e-4f) detail::raise(FYN_ERR_INVALID, "Only supporting integer upscales for now");
            } else if (sc[axis] < 1.f) {
                const float dn = 1.f / sc[axis];
                downsample_[axis] = (short)(dn + 1e-6f);
                if (std::fabs((float)downsample_[axis] - dn) > 1e-4f) detail::raise(FYN_ERR_INVALID, "Only supporting integer downscales for now");
            }
        }
        return *this;
    }
    ScaleLayerBuilder& scale(float s) { return scale(s, s); }
    bool equal() const { return upsample_[0] == upsample_[1] && downsample_[0] == downsample_[1]; }
    ScalingType scaleType_ = ScalingType::NEAREST;
    int rotation_ = 0;

  protected:
    void fill(fyn_layer_desc& d) const override {
        if (rotation_ % 360 != 0) detail::raise(FYN_ERR_UNSUPPORTED, "rotation in scale layers is not supported");
        d.scale_type = (int)scaleType_;
    }
};

struct SingletonArithLayerBuilder : GPULayerBuilderTempl<SingletonArithLayerBuilder> {
    SingletonArithLayerBuilder(const std::string& name, ArithType op) : GPULayerBuilderTempl<SingletonArithLayerBuilder>(name), opType_(op) {
        type_ = LayerType::SINGLETON_ARITH;
    }
    SingletonArithLayerBuilder& operand(float opd) { operand_ = opd; return *this; }
    ArithType opType_;
    float operand_ = 0.f;

  protected:
    void fill(fyn_layer_desc& d) const override { d.arith_op = (int)opType_; d.operand = operand_; }
};

struct CastLayerBuilder : GPULayerBuilderTempl<CastLayerBuilder> {
    CastLayerBuilder(const std::string& name, CastTarget tgt) : GPULayerBuilderTempl<CastLayerBuilder>(name), target_(tgt) { type_ = LayerType::CAST; }
    CastLayerBuilder& target(CastTarget tgt) { target_ = tgt; return *this; }
    CastTarget target_;

  protected:
    void fill(fyn_layer_desc& d) const override { d.cast_target = (int)target_; }
};

struct TransposeLayerBuilder : GPULayerBuilderTempl<TransposeLayerBuilder> {
    explicit TransposeLayerBuilder(const std::string& name) : GPULayerBuilderTempl<TransposeLayerBuilder>(name) { type_ = LayerType::TRANSPOSE; }
};

struct ImgExtractLayerBuilder : GPULayerBuilderTempl<ImgExtractLayerBuilder> {
    ImgExtractLayerBuilder(short window, const std::string& name) : GPULayerBuilderTempl<ImgExtractLayerBuilder>(name), window_(window) {
        type_ = LayerType::IMGEXTRACT;
        downsample_[0] = downsample_[1] = window;
    }
    short window_;

  protected:
    void fill(fyn_layer_desc& d) const override { d.window = window_; }
};

struct BlurLayerBuilder : GPULayerBuilderTempl<BlurLayerBuilder> {
    explicit BlurLayerBuilder(const std::string& name) : GPULayerBuilderTempl<BlurLayerBuilder>(name) { type_ = LayerType::BLUR2D; }
    BlurLayerBuilder& kernel(short sz) { kernel_ = sz; return *this; }
    BlurLayerBuilder& blurType(BlurKernelType typ) { blurType_ = typ; return *this; }
    short kernel_ = 3;
    BlurKernelType blurType_ = BlurKernelType::AVERAGE;

  protected:
    void fill(fyn_layer_desc& d) const override { d.kernel = kernel_; d.blur_type = (int)blurType_; }
};

/* A user-supplied layer: what the init callback of the reference's CustomLayerBuilder returns (a GPULayerBase
 * subclass there, gpu/customlayerbuilder.h:53-90).  forward() must only enqueue work on the given hipStream_t. */
class CustomLayer {
  public:
    virtual ~CustomLayer() = default;
    virtual void setup(const fyn_tensor_view* /*inputs*/, int /*numInputs*/, const fyn_tensor_view& /*output*/) {}
    virtual void forward(const fyn_tensor_view* inputs, int numInputs, const fyn_tensor_view& output, void* hipStream, uint64_t sequence) = 0;
};

struct CustomLayerBuilder : GPULayerBuilderTempl<CustomLayerBuilder> {
    using initfunc = std::function<CustomLayer*(const CustomLayerBuilder&)>;
    CustomLayerBuilder(const std::string& name, initfunc init) : GPULayerBuilderTempl<CustomLayerBuilder>(name), initCallback_(std::move(init)) {
        type_ = LayerType::CUSTOM;
    }
    CustomLayerBuilder& input(int channels, int padding) { inputs_.emplace_back(channels, padding); return *this; }
    CustomLayer* init() const { return initCallback_(*this); }
    initfunc initCallback_;
    std::vector<std::pair<int, int>> inputs_;

  protected:
    void fill(fyn_layer_desc& d) const override {
        d.num_inputs = (int)inputs_.size();
        for (size_t i = 0; i < inputs_.size(); i++) {
            d.inputs[i].channels = inputs_[i].first; d.inputs[i].padding = inputs_[i].second; d.inputs[i].flags = 0;
        }
    }
};

}  // namespace gpu

/* base/convlayerinterface.h:95 and base/batchnorminterface.h:146: what initializeWeights() casts layers to. */
class ConvLayerInterface {
  public:
    virtual ~ConvLayerInterface() = default;
    virtual void loadWeightsAndBiases(const float* weightsAndBiases, size_t offset = 0) = 0;
};
class BatchNormInterface {
  public:
    virtual ~BatchNormInterface() = default;
    virtual void loadScaleAndBias(const float* scaleBias, size_t sbOffset = 0) = 0;
};

/* Handle of one compiled layer (LayerBase / GPULayerBase of the reference). */
class LayerBase {
  public:
    LayerBase(fyn_net* net, const LayerBuilderData& b) : net_(net), number_(b.number_), name_(b.name_), type_(b.type_) {}
    virtual ~LayerBase() = default;
    int getNumber() const { return number_; }
    const std::string& getName() const { return name_; }
    LayerType getType() const { return type_; }

    /* Output geometry: channels, height, width (net size), padding. */
    void outputShape(int& channels, int& height, int& width, int& padding) const {
        detail::check(fyn_layer_output_shape(net_, number_, &channels, &height, &width, &padding));
    }
    /* GPULayerBase::copyResult(float*, bool) (gpu/gpulayerbase.cpp:525-564): channel-wise fp32. */
    void copyResult(float* memory, bool includePadding = false) const {
        detail::check(fyn_layer_copy_result(net_, number_, memory, includePadding ? 1 : 0));
    }
    std::vector<float> copyResult(bool includePadding = false) const {
        int c, h, w, p;
        outputShape(c, h, w, p);
        if (includePadding) { h += 2 * p; w += 2 * p; }
        std::vector<float> out((size_t)c * h * w);
        copyResult(out.data(), includePadding);
        return out;
    }
    /* Writes the tensor on an input port (what the reference's layer tests do with textures, unit_tests/
     * layertestbase.cpp:208-417); for an upload layer: its input buffer (UploadLayer::setInputBuffer). */
    void setInput(const float* data, int port = 0, int order = FYN_ORDER_CHANNELWISE) {
        detail::check(fyn_net_set_input(net_, number_, port, data, order));
    }
    size_t weightFloats() const {
        size_t n = 0;
        detail::check(fyn_layer_weight_floats(net_, number_, &n));
        return n;
    }
    std::string kernelInfo() const {
        char buf[512];
        detail::check(fyn_layer_kernel_info(net_, number_, buf, sizeof(buf)));
        return buf;
    }

  protected:
    fyn_net* net_;
    int number_;
    std::string name_;
    LayerType type_;
};

namespace detail {
class WeightedLayer : public LayerBase, public ConvLayerInterface {
  public:
    using LayerBase::LayerBase;
    void loadWeightsAndBiases(const float* wb, size_t offset = 0) override { check(fyn_layer_load_weights(net_, number_, wb, offset)); }
};
class ScaleBiasLayer : public LayerBase, public BatchNormInterface {
  public:
    using LayerBase::LayerBase;
    void loadScaleAndBias(const float* sb, size_t offset = 0) override { check(fyn_layer_load_scale_bias(net_, number_, sb, offset)); }
};
}  // namespace detail

/* base/compiledlayers.h:50-291: layers by number and by name, iterated in ascending number; an iterator exposes
 * `first` (number) and `second` (layer), as the reference's does (`it.second`). */
class CompiledLayers {
  public:
    using store = std::map<int, std::shared_ptr<LayerBase>>;
    class iterator {
      public:
        iterator(store::const_iterator it, store::const_iterator end) : it_(it), end_(end) { load(); }
        iterator& operator++() { ++it_; load(); return *this; }
        bool operator!=(const iterator& o) const { return it_ != o.it_; }
        bool operator==(const iterator& o) const { return it_ == o.it_; }
        const iterator& operator*() const { return *this; }
        int first = -1;
        LayerBase* second = nullptr;

      private:
        void load() {
            first = it_ == end_ ? -1 : it_->first;
            second = it_ == end_ ? nullptr : it_->second.get();
        }
        store::const_iterator it_, end_;
    };
    LayerBase* operator[](int number) const {
        auto it = byNumber_.find(number);
        if (it == byNumber_.end()) detail::raise(FYN_ERR_NOTFOUND, "no layer %d", number);
        return it->second.get();
    }
    LayerBase* operator[](const std::string& name) const {
        auto it = byName_.find(name);
        if (it == byName_.end()) detail::raise(FYN_ERR_NOTFOUND, "no layer %s", name.c_str());
        return it->second;
    }
    LayerBase* operator[](const char* name) const { return (*this)[std::string(name)]; }
    size_t size() const { return byNumber_.size(); }
    iterator begin() const { return iterator(byNumber_.begin(), byNumber_.end()); }
    iterator end() const { return iterator(byNumber_.end(), byNumber_.end()); }
    void add(const std::shared_ptr<LayerBase>& l) {
        byNumber_[l->getNumber()] = l;
        byName_[l->getName()] = l.get();
    }

  private:
    store byNumber_;
    std::map<std::string, LayerBase*> byName_;
};

/* base/layerfactory.h:56-138.  The factory owns the builders pushed into it. */
class LayerFactory {
  public:
    explicit LayerFactory(fyn_net* net) : net_(net) {}

    void pushBuilder(LayerBuilderData* builder) {
        std::unique_ptr<LayerBuilderData> own(builder);
        // base/layerfactory.cpp:67-76
        if (builder->number_ < 0) detail::raise(FYN_ERR_INVALID, "Must identify each layer with a valid number (found %d in the builder)", builder->number_);
        if ((int)builder->type_ >= (int)LayerType::LAST_SUPPORTED) detail::raise(FYN_ERR_UNSUPPORTED, "Unsupported layer type %d", (int)builder->type_);
        if (builders_.count(builder->number_)) detail::raise(FYN_ERR_DUPLICATE, "Trying to insert a layer on a position that is already taken (%d)", builder->number_);
        builders_[builder->number_] = std::move(own);
    }

    /* LayerFactory::compileLayers (base/layerfactory.cpp:83-101): creates every layer in ascending number. */
    CompiledLayers compileLayers() {
        CompiledLayers layers;
        for (auto& kv : builders_) {
            const LayerBuilderData& b = *kv.second;
            const fyn_layer_desc d = b.desc();
            if (b.type_ == LayerType::CUSTOM) addCustom(b, d);
            else detail::check(fyn_net_add_layer(net_, &d));
            switch (b.type_) {
                case LayerType::CONVOLUTION2D: case LayerType::FRACCONVOLUTION2D: case LayerType::TRANSCONVOLUTION2D: case LayerType::GEMM:
                    layers.add(std::make_shared<detail::WeightedLayer>(net_, b));
                    break;
                case LayerType::BATCHNORM:
                    layers.add(std::make_shared<detail::ScaleBiasLayer>(net_, b));
                    break;
                default:
                    layers.add(std::make_shared<LayerBase>(net_, b));
            }
        }
        return layers;
    }

  private:
    void addCustom(const LayerBuilderData& b, const fyn_layer_desc& d) {
        // gpu/gpulayerfactory.cpp:586-589: the builder's callback creates the layer
        const auto* cb = dynamic_cast<const gpu::CustomLayerBuilder*>(&b);
        if (!cb || !cb->initCallback_) detail::raise(FYN_ERR_INVALID, "layer %s: a CUSTOM layer needs a CustomLayerBuilder with its init callback", b.name_.c_str());
        gpu::CustomLayer* impl = cb->init();
        if (!impl) detail::raise(FYN_ERR_INVALID, "layer %s: the init callback returned no layer", b.name_.c_str());
        fyn_custom_layer c;
        c.user = impl;   // owned by the engine from here: deleted by the cleanup callback
        c.setup = [](void* u, const fyn_tensor_view* in, int n, const fyn_tensor_view* out) -> int {
            try { static_cast<gpu::CustomLayer*>(u)->setup(in, n, *out); return 0; } catch (...) { return 1; }
        };
        c.forward = [](void* u, const fyn_tensor_view* in, int n, const fyn_tensor_view* out, void* stream, uint64_t seq) -> int {
            try { static_cast<gpu::CustomLayer*>(u)->forward(in, n, *out, stream, seq); return 0; } catch (...) { return 1; }
        };
        c.cleanup = [](void* u) { delete static_cast<gpu::CustomLayer*>(u); };
        const int rc = fyn_net_add_custom_layer(net_, &d, &c);
        if (rc != FYN_OK) {
            delete impl;
            detail::check(rc);
        }
    }

    fyn_net* net_;
    std::map<int, std::unique_ptr<LayerBuilderData>> builders_;
};

template <typename D>
D& LayerBuilderTempl<D>::push(const std::shared_ptr<LayerFactory>& factory) {
    factory->pushBuilder(this);
    return self();
}
template <typename D>
D& LayerBuilderTempl<D>::push(LayerFactory& factory) {
    factory.pushBuilder(this);
    return self();
}

/* base/buffermanager.cpp:160-184 (connectLayers); the tensors live in the engine. */
class BufferManager {
  public:
    explicit BufferManager(fyn_net* net) : net_(net) {}
    void connectLayers(LayerBase* outputLayer, LayerBase* inputLayer, int port = 0) {
        if (!outputLayer || !inputLayer) detail::raise(FYN_ERR_INVALID, "Illegal parameters out=%p in=%p", (void*)outputLayer, (void*)inputLayer);
        detail::check(fyn_net_connect(net_, outputLayer->getNumber(), inputLayer->getNumber(), port));
    }

  private:
    fyn_net* net_;
};

/*
 * base/neuralnetwork.h:62-261.  A network description derives from this class and provides buildLayers(),
 * connectLayers() and initializeWeights(); setup() runs them in the order of NeuralNetwork::glSetup
 * (base/neuralnetwork.cpp:238-250).  storage: FYN_STORAGE_F32 (the reference's HIGH_PRECISION build) or FYN_STORAGE_F16.
 */
class NeuralNetwork {
  public:
    enum state { EXEC_DONE = 0, EXEC_ERROR, EXEC_STOPPED };   // base/neuralnetwork.h:70-74 (the execution states in use here)
    struct execstate {
        state status;
        uint64_t sequenceNo;
    };

    explicit NeuralNetwork(const GfxContextLink& = GfxContextLink(), int storage = FYN_STORAGE_F32, int device = 0) {
        detail::check(fyn_net_create(device, storage, &net_));
    }
    NeuralNetwork(const NeuralNetwork&) = delete;
    NeuralNetwork& operator=(const NeuralNetwork&) = delete;
    virtual ~NeuralNetwork() { cleanup(); }

    /* NeuralNetwork::setup (base/neuralnetwork.cpp:88-103) */
    virtual void setup() {
        if (setup_) detail::raise(FYN_ERR_STATE, "network is already set up");
        layers_ = buildLayers();
        buffers_.reset(new BufferManager(net_));
        connectLayers(layers_, buffers_.get());
        initializeWeights(layers_);
        detail::check(fyn_net_setup(net_));
        setup_ = true;
    }
    /* NeuralNetwork::forward (base/neuralnetwork.cpp:173-187): all layers in ascending number; asynchronous to the host */
    virtual execstate forward() {
        uint64_t seq = 0;
        detail::check(fyn_net_forward(net_, &seq));
        return execstate{EXEC_DONE, seq};
    }
    /* NeuralNetwork::finish (base/neuralnetwork.cpp:196-206) */
    virtual void finish() { detail::check(fyn_net_finish(net_)); }
    /* NeuralNetwork::cleanup (base/neuralnetwork.cpp:57-79) */
    virtual void cleanup() {
        if (net_) (void)fyn_net_destroy(net_);
        net_ = nullptr;
        setup_ = false;
    }

    CompiledLayers& getLayers() { return layers_; }
    GfxContextLink context() const { return GfxContextLink(); }
    bool isSetup() const { return setup_; }

    /* Output of a layer in a CPUBuffer order (download layer formats, cpu/cpubuffer.cpp); synchronises. */
    void getOutput(int layer, float* data, int order = FYN_ORDER_CHANNELWISE) { detail::check(fyn_net_get_output(net_, layer, data, order)); }
    void useGraph(bool enable) { detail::check(fyn_net_use_graph(net_, enable ? 1 : 0)); }
    void setBufferReuse(bool enable) { detail::check(fyn_net_set_buffer_reuse(net_, enable ? 1 : 0)); }
    /* Engine::enableIntermediateOutput (base/engine.cpp:174-181) */
    void enableDebugOutput(const std::string& dir) { detail::check(fyn_net_enable_intermediate_output(net_, dir.c_str())); }

    /* Frame pipeline = the reference engine's asynchronous mode (base/engine.cpp:386-683). */
    void asyncBegin(int inLayer, int outLayer, int inOrder = FYN_ORDER_CHANNELWISE, int outOrder = FYN_ORDER_CHANNELWISE, int depth = 2,
                    int inPort = 0, bool copyStreams = true) {
        detail::check(fyn_net_async_begin(net_, inLayer, inPort, inOrder, outLayer, outOrder, depth, copyStreams ? 1 : 0));
    }
    uint64_t asyncSubmit(const float* frame, float* out) {
        uint64_t t = 0;
        detail::check(fyn_net_async_submit(net_, frame, out, &t));
        return t;
    }
    void asyncWait(uint64_t ticket) { detail::check(fyn_net_async_wait(net_, ticket)); }
    void asyncEnd() { detail::check(fyn_net_async_end(net_)); }

    fyn_net* handle() const { return net_; }

  protected:
    virtual CompiledLayers buildLayers() = 0;
    virtual void connectLayers(CompiledLayers& layers, BufferManager* buffers) = 0;
    virtual void initializeWeights(CompiledLayers& layers) = 0;

    /* NeuralNetwork::getLayerFactory (base/neuralnetwork.cpp:213-221) */
    std::shared_ptr<LayerFactory> getLayerFactory() { return std::make_shared<LayerFactory>(net_); }

    fyn_net* net_ = nullptr;
    bool setup_ = false;
    CompiledLayers layers_;
    std::unique_ptr<BufferManager> buffers_;
};

/*
 * Several instances of one network, each with its own stream, frame pipeline and captured graph; frames are dealt to the
 * instances in turn, so that the kernels of up to `instances` frames share the GPU (batch-1 networks of small layers are
 * bound by launch latency and leave most of the chip idle).  Results are delivered in submission order through
 * tickets.  The reference runs one frame pipeline per network (base/engine.cpp:386-683); several side by side are several
 * NeuralNetwork objects there as well.  More instances than hardware queues per process (4 by default) add nothing.
 *   Net: a NeuralNetwork subclass; make(): returns a new, not yet set up instance.
 */
template <typename Net>
class FramePool {
  public:
    FramePool(const std::function<std::unique_ptr<Net>()>& make, int inLayer, int outLayer, int instances = 4, int depth = 2,
              int inOrder = FYN_ORDER_CHANNELWISE, int outOrder = FYN_ORDER_CHANNELWISE, bool graph = true) {
        if (instances < 1) detail::raise(FYN_ERR_INVALID, "a frame pool needs at least one network instance");
        for (int i = 0; i < instances; i++) {
            nets_.push_back(make());
            Net& n = *nets_.back();
            n.setup();
            if (graph) n.useGraph(true);
            // one stream per instance: the instances overlap each other, and more streams than hardware queues would
            // wait for each other's events
            n.asyncBegin(inLayer, outLayer, inOrder, outOrder, depth, 0, instances == 1);
        }
    }
    ~FramePool() {
        for (auto& n : nets_) {
            try { n->asyncEnd(); } catch (...) {}
        }
    }
    /* Queues one frame on the next instance; `out` is filled once wait(ticket) has returned. */
    uint64_t submit(const float* frame, float* out) {
        Net& n = *nets_[submitted_ % nets_.size()];
        open_[++submitted_] = std::make_pair(&n, n.asyncSubmit(frame, out));
        return submitted_;
    }
    /* Returns when the frame of `ticket` and every frame submitted before it have been delivered. */
    void wait(uint64_t ticket) {
        if (ticket < 1 || ticket > submitted_) detail::raise(FYN_ERR_INVALID, "unknown frame ticket %llu", (unsigned long long)ticket);
        while (!open_.empty() && open_.begin()->first <= ticket) {
            open_.begin()->second.first->asyncWait(open_.begin()->second.second);
            open_.erase(open_.begin());
        }
    }
    size_t instances() const { return nets_.size(); }

  private:
    std::vector<std::unique_ptr<Net>> nets_;
    std::map<uint64_t, std::pair<Net*, uint64_t>> open_;
    uint64_t submitted_ = 0;
};

}  // namespace fynhip

#ifdef FYNHIP_REFERENCE_NAMESPACE
namespace fyusion {
namespace fyusenet = ::fynhip;
}
#endif

#endif /* FYNHIP_HPP */
