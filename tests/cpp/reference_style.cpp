// A program written against include/fynhip.hpp the way the reference's samples and unit tests are written against
// FyuseNet: the style-transfer network of samples/samplenetworks/stylenet3x3.cpp as a NeuralNetwork subclass, and the
// known-answer patterns of unit_tests/convlayertests.cpp:165-182,242-261 and networktests.cpp:85-97,173-186.
//
//   reference_style <weights.bin> <input.bin> <output.bin> <width> <height>
//
// weights.bin: 77235 floats (StyleNet3x3::STYLENET_SIZE); input.bin: width*height RGB triplets in [0,1] (GPU_SHALLOW
// order, what StyleNetBase::setInputBuffer takes); output.bin: width*height RGBA quadruples, written here.
// Exit status 0 when every check passed.
#define FYNHIP_REFERENCE_NAMESPACE
#include <cstdio>
#include <cstdlib>
#include <string>
#include <unordered_map>
#include <vector>

#include "fynhip.hpp"

using namespace fyusion::fyusenet;

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::fprintf(stderr, "%s:%d: EXPECT(%s) failed\n", __FILE__, __LINE__, #cond); \
            failures++;                                                     \
        }                                                                   \
    } while (0)

// ---- the sample network, as stylenet3x3.cpp:114-211 describes it ---------------------------------------------------
class StyleNet3x3 : public NeuralNetwork {
  public:
    enum { UPLOAD = 0, CONV1, CONV2, CONV3, RES1_1, RES1_2, RES2_1, RES2_2, DECONV1, DECONV2, DECONV3, SIGMOID, DOWNLOAD };
    constexpr static int STYLENET_SIZE = 77235;

    StyleNet3x3(int width, int height) : width_(width), height_(height) {
        weightOffsets_ = {{CONV1, 0},      {CONV2, 336},     {CONV3, 2516},    {RES1_1, 19475},  {RES1_2, 33915},
                          {RES2_1, 48355}, {RES2_2, 62795},  {DECONV1, 9756},  {DECONV2, 16976}, {DECONV3, 19148}};
        wbData_.assign(STYLENET_SIZE, 0.f);
    }
    void loadWeightsAndBiases(const float* weightsAndBiases, size_t size) {
        EXPECT(size == (size_t)STYLENET_SIZE);
        wbData_.assign(weightsAndBiases, weightsAndBiases + size);
        if (setup_) initializeWeights(getLayers());
    }
    void setInputBuffer(const float* rgb) { getLayers()["upload"]->setInput(rgb, 0, FYN_ORDER_GPU_SHALLOW); }

  protected:
    CompiledLayers buildLayers() override {
        std::shared_ptr<LayerFactory> factory = getLayerFactory();
        auto* up = new gpu::UpDownLayerBuilder(gpu::UpDownLayerBuilder::UPLOAD, "upload");
        up->shape(3, height_, width_, 3).context(context()).number(UPLOAD);
        up->push(factory);
        auto* conv1 = new gpu::ConvLayerBuilder(3, "conv1");
        conv1->shape(12, height_, width_, 3).type(LayerType::CONVOLUTION2D).prefixAct(ActType::RELU).context(context()).number(CONV1);
        conv1->push(factory);
        auto* conv2 = new gpu::ConvLayerBuilder(3, "conv2");
        conv2->shape(20, height_, width_, 12).type(LayerType::CONVOLUTION2D).downsample(2).prefixAct(ActType::RELU).context(context()).number(CONV2);
        conv2->push(factory);
        auto* conv3 = new gpu::ConvLayerBuilder(3, "conv3");
        conv3->shape(40, height_ / 2, width_ / 2, 20).type(LayerType::CONVOLUTION2D).downsample(2).prefixAct(ActType::RELU).context(context()).number(CONV3);
        conv3->push(factory);
        auto* res11 = new gpu::ConvLayerBuilder(3, "res1_1");
        res11->shape(40, height_ / 4, width_ / 4, 40).type(LayerType::CONVOLUTION2D).prefixAct(ActType::RELU).context(context()).number(RES1_1);
        res11->push(factory);
        auto* res12 = new gpu::ConvLayerBuilder(3, "res1_2");
        res12->shape(40, height_ / 4, width_ / 4, 40).type(LayerType::CONVOLUTION2D).prefixAct(ActType::RELU).residual(ActType::RELU).context(context()).number(RES1_2);
        res12->push(factory);
        auto* res21 = new gpu::ConvLayerBuilder(3, "res2_1");
        res21->shape(40, height_ / 4, width_ / 4, 40).type(LayerType::CONVOLUTION2D).context(context()).number(RES2_1);
        res21->push(factory);
        auto* res22 = new gpu::ConvLayerBuilder(3, "res2_2");
        res22->shape(40, height_ / 4, width_ / 4, 40).type(LayerType::CONVOLUTION2D).prefixAct(ActType::RELU).residual().context(context()).number(RES2_2);
        res22->push(factory);
        auto* deconv1 = new gpu::ConvLayerBuilder(3, "deconv1");
        deconv1->shape(20, height_ / 4, width_ / 4, 40).type(LayerType::FRACCONVOLUTION2D).downsample(2).sourceStep(0.5f).context(context()).number(DECONV1);
        deconv1->push(factory);
        auto* deconv2 = new gpu::ConvLayerBuilder(3, "deconv2");
        deconv2->shape(12, height_ / 4, width_ / 4, 20).type(LayerType::FRACCONVOLUTION2D).sourceStep(0.25f).downsample(2).prefixAct(ActType::RELU).context(context()).number(DECONV2);
        deconv2->push(factory);
        auto* deconv3 = new gpu::ConvLayerBuilder(3, "deconv3");
        deconv3->shape(3, height_ / 2, width_ / 2, 12).type(LayerType::FRACCONVOLUTION2D).sourceStep(0.5f).prefixAct(ActType::RELU).context(context()).number(DECONV3);
        deconv3->push(factory);
        auto* sigmoid = new gpu::GPULayerBuilder("sigmoid");
        sigmoid->shape(3, height_, width_, 3).type(LayerType::SIGMOID).context(context()).number(SIGMOID);
        sigmoid->push(factory);
        auto* down = new gpu::UpDownLayerBuilder(gpu::UpDownLayerBuilder::DOWNLOAD, "download");
        down->shape(4, height_, width_, 4).context(context()).number(DOWNLOAD);
        down->push(factory);
        return factory->compileLayers();
    }

    void connectLayers(CompiledLayers& layers, BufferManager* buffers) override {
        buffers->connectLayers(layers[UPLOAD], layers[CONV1], 0);
        buffers->connectLayers(layers[CONV1], layers[CONV2], 0);
        buffers->connectLayers(layers[CONV2], layers[CONV3], 0);
        buffers->connectLayers(layers[CONV3], layers[RES1_1], 0);
        buffers->connectLayers(layers[CONV3], layers[RES1_2], 1);
        buffers->connectLayers(layers[RES1_1], layers[RES1_2], 0);
        buffers->connectLayers(layers[RES1_2], layers[RES2_1], 0);
        buffers->connectLayers(layers[RES1_2], layers[RES2_2], 1);
        buffers->connectLayers(layers[RES2_1], layers[RES2_2], 0);
        buffers->connectLayers(layers[RES2_2], layers[DECONV1], 0);
        buffers->connectLayers(layers[DECONV1], layers[DECONV2], 0);
        buffers->connectLayers(layers[DECONV2], layers[DECONV3], 0);
        buffers->connectLayers(layers[DECONV3], layers[SIGMOID], 0);
        buffers->connectLayers(layers[SIGMOID], layers[DOWNLOAD], 0);
    }

    void initializeWeights(CompiledLayers& layers) override {
        for (auto it = layers.begin(); it != layers.end(); ++it) {
            ConvLayerInterface* conv = dynamic_cast<ConvLayerInterface*>(it.second);
            if (conv) conv->loadWeightsAndBiases(wbData_.data(), weightOffsets_.at(it.second->getNumber()));
        }
    }

    int width_, height_;
    std::unordered_map<int, size_t> weightOffsets_;
    std::vector<float> wbData_;
};

// ---- a one-layer network, as the reference's layer tests set one up ----------------------------------------------------
class SingleConv : public NeuralNetwork {
  public:
    SingleConv(int kernel, int cout, int size, int cin, bool deep, int padding, std::vector<float> block)
        : kernel_(kernel), cout_(cout), size_(size), cin_(cin), deep_(deep), padding_(padding), block_(std::move(block)) {}

  protected:
    CompiledLayers buildLayers() override {
        std::shared_ptr<LayerFactory> factory = getLayerFactory();
        auto* conv = new gpu::ConvLayerBuilder((short)kernel_, "conv");
        conv->shape(cout_, size_, size_, cin_).type(LayerType::CONVOLUTION2D).inputPadding((short)padding_).number(1);
        if (deep_) conv->deep();
        conv->push(factory);
        return factory->compileLayers();
    }
    void connectLayers(CompiledLayers&, BufferManager*) override {}
    void initializeWeights(CompiledLayers& layers) override {
        dynamic_cast<ConvLayerInterface*>(layers[1])->loadWeightsAndBiases(block_.data(), 0);
    }
    int kernel_, cout_, size_, cin_;
    bool deep_;
    int padding_;
    std::vector<float> block_;
};

static std::vector<float> antisymmetric_block(int cout, int cin) {   // rows -1, 0, +1 (convlayertests.cpp:242-261)
    std::vector<float> b((size_t)cout + (size_t)cout * 9 * cin, 0.f);
    for (int o = 0; o < cout; o++)
        for (int kx = 0; kx < 3; kx++)
            for (int i = 0; i < cin; i++) {
                b[cout + (((size_t)o * 3 + 0) * 3 + kx) * cin + i] = -1.f;
                b[cout + (((size_t)o * 3 + 2) * 3 + kx) * cin + i] = 1.f;
            }
    return b;
}

static void known_answers() {
    {   // deep 3x3, zero halo: zero inside, +-3*cin on the first and last row
        const int cin = 8, cout = 8, size = 32;
        SingleConv net(3, cout, size, cin, true, 1, antisymmetric_block(cout, cin));
        net.setup();
        std::vector<float> ones((size_t)cin * size * size, 1.f);
        net.getLayers()[1]->setInput(ones.data());
        net.forward();
        net.finish();
        const std::vector<float> out = net.getLayers()["conv"]->copyResult();
        EXPECT(out.size() == (size_t)cout * size * size);
        bool ok = true;
        for (int o = 0; o < cout; o++)
            for (int y = 0; y < size; y++)
                for (int x = 1; x < size - 1; x++) {
                    const float want = y == 0 ? 3.f * cin : (y == size - 1 ? -3.f * cin : 0.f);
                    ok = ok && out[((size_t)o * size + y) * size + x] == want;
                }
        EXPECT(ok);
    }
    {   // shallow 3x3 without padding: the edge repeats, a zero-sum kernel on ones gives 0 everywhere (networktests.cpp:85-97)
        const int cin = 4, cout = 8, size = 32;
        SingleConv net(3, cout, size, cin, false, 0, antisymmetric_block(cout, cin));
        net.setup();
        std::vector<float> ones((size_t)cin * size * size, 1.f);
        net.getLayers()[1]->setInput(ones.data());
        net.forward();
        net.finish();
        bool ok = true;
        for (float v : net.getLayers()[1]->copyResult()) ok = ok && v == 0.f;
        EXPECT(ok);
    }
    {   // 1x1 all-ones weights on ones: every output equals cin (convlayertests.cpp:165-182)
        const int cin = 12, cout = 16, size = 20;
        std::vector<float> block((size_t)cout + (size_t)cout * cin, 1.f);
        for (int o = 0; o < cout; o++) block[o] = 0.f;
        SingleConv net(1, cout, size, cin, true, 0, block);
        net.setup();
        std::vector<float> ones((size_t)cin * size * size, 1.f);
        net.getLayers()[1]->setInput(ones.data());
        net.forward();
        net.finish();
        bool ok = true;
        for (float v : net.getLayers()[1]->copyResult()) ok = ok && v == (float)cin;
        EXPECT(ok);
    }
}

static void error_behaviour() {
    NeuralNetwork* raw = nullptr;
    (void)raw;
    struct Bad : NeuralNetwork {
        int variant;
        explicit Bad(int v) : variant(v) {}
        CompiledLayers buildLayers() override {
            auto factory = getLayerFactory();
            if (variant == 0) {          // two layers on one number (base/layerfactory.cpp:73)
                (new gpu::GPULayerBuilder("a"))->shape(4, 8, 8, 4).type(LayerType::RELU).number(1).push(factory);
                (new gpu::GPULayerBuilder("b"))->shape(4, 8, 8, 4).type(LayerType::RELU).number(1).push(factory);
            } else if (variant == 1) {   // fractional convolution on deep tensors (gpu/gpulayerfactory.cpp:447-450)
                (new gpu::ConvLayerBuilder(3, "f"))->shape(4, 8, 8, 4).type(LayerType::FRACCONVOLUTION2D).sourceStep(0.5f).deep().number(1).push(factory);
            } else {                     // a builder without a number (base/layerfactory.cpp:68)
                (new gpu::GPULayerBuilder("c"))->shape(4, 8, 8, 4).type(LayerType::RELU).push(factory);
            }
            return factory->compileLayers();
        }
        void connectLayers(CompiledLayers&, BufferManager*) override {}
        void initializeWeights(CompiledLayers&) override {}
    };
    const char* expect[3] = {"already taken", "not supported for deep layers", "valid number"};
    for (int v = 0; v < 3; v++) {
        bool thrown = false;
        try {
            Bad net(v);
            net.setup();
        } catch (const FynException& ex) {
            thrown = std::string(ex.what()).find(expect[v]) != std::string::npos;
            if (!thrown) std::fprintf(stderr, "unexpected message: %s\n", ex.what());
        }
        EXPECT(thrown);
    }
}

static std::vector<float> read_floats(const char* path, size_t count) {
    std::vector<float> v(count);
    FILE* f = std::fopen(path, "rb");
    if (!f || std::fread(v.data(), sizeof(float), count, f) != count) {
        std::fprintf(stderr, "cannot read %zu floats from %s\n", count, path);
        std::exit(2);
    }
    std::fclose(f);
    return v;
}

int main(int argc, char** argv) {
    if (argc != 6) {
        std::fprintf(stderr, "usage: %s weights.bin input.bin output.bin width height\n", argv[0]);
        return 2;
    }
    const int width = std::atoi(argv[4]), height = std::atoi(argv[5]);
    try {
        known_answers();
        error_behaviour();
        const std::vector<float> weights = read_floats(argv[1], StyleNet3x3::STYLENET_SIZE);
        const std::vector<float> rgb = read_floats(argv[2], (size_t)width * height * 3);
        StyleNet3x3 net(width, height);
        net.loadWeightsAndBiases(weights.data(), weights.size());
        net.setup();
        net.setInputBuffer(rgb.data());
        net.forward();
        net.finish();
        std::vector<float> rgba((size_t)width * height * 4);
        net.getOutput(StyleNet3x3::DOWNLOAD, rgba.data(), FYN_ORDER_GPU_SHALLOW);
        // the frame pipeline must deliver the same frame
        std::vector<float> again(rgba.size(), -1.f);
        net.asyncBegin(StyleNet3x3::UPLOAD, StyleNet3x3::DOWNLOAD, FYN_ORDER_GPU_SHALLOW, FYN_ORDER_GPU_SHALLOW, 2);
        net.asyncWait(net.asyncSubmit(rgb.data(), again.data()));
        net.asyncEnd();
        EXPECT(again == rgba);
        // weights can be loaded again after setup (stylenet3x3.cpp:81-89)
        net.loadWeightsAndBiases(weights.data(), weights.size());
        net.forward();
        net.finish();
        net.getOutput(StyleNet3x3::DOWNLOAD, again.data(), FYN_ORDER_GPU_SHALLOW);
        EXPECT(again == rgba);
        {   // three instances side by side: every frame's result under its own ticket, equal to the single network's
            std::vector<float> w = weights;
            FramePool<StyleNet3x3> pool(
                [&]() {
                    std::unique_ptr<StyleNet3x3> n(new StyleNet3x3(width, height));
                    n->loadWeightsAndBiases(w.data(), w.size());
                    return n;
                },
                StyleNet3x3::UPLOAD, StyleNet3x3::DOWNLOAD, 3, 2, FYN_ORDER_GPU_SHALLOW, FYN_ORDER_GPU_SHALLOW);
            std::vector<std::vector<float>> outs(7, std::vector<float>(rgba.size(), -1.f));
            uint64_t last = 0;
            for (auto& o : outs) last = pool.submit(rgb.data(), o.data());
            pool.wait(last);
            bool same = true;
            for (auto& o : outs) same = same && o == rgba;
            EXPECT(same);
            EXPECT(pool.instances() == 3);
        }
        FILE* f = std::fopen(argv[3], "wb");
        if (!f || std::fwrite(rgba.data(), sizeof(float), rgba.size(), f) != rgba.size()) {
            std::fprintf(stderr, "cannot write %s\n", argv[3]);
            return 2;
        }
        std::fclose(f);
        std::printf("%s\n", net.getLayers()[StyleNet3x3::DECONV2]->kernelInfo().c_str());
    } catch (const FynException& ex) {
        std::fprintf(stderr, "FynException (%d): %s\n", ex.status(), ex.what());
        return 1;
    }
    std::printf("%d check(s) failed\n", failures);
    return failures == 0 ? 0 : 1;
}
