// A program written against include/fynhip.hpp (builders, LayerFactory, CompiledLayers, BufferManager and a
// NeuralNetwork subclass, reachable under the reference's namespace) with the host compiler only.
//
//   surface_example <weights.bin> <input.bin> <output.bin> <width> <height>
//
// The network is an hourglass of this file's own making, described by one table: a 5x5 convolution, a strided 3x3
// convolution, a residual pair, a stride-2 transposed convolution back to full size and a 1x1 convolution read
// through a leaky ReLU.  weights.bin is the headerless fp32 stream of the table's layers in table order, each block
// [bias][W o,ky,kx,i][bnScale][bnBias]; input.bin is 3 x height x width (channel-wise); output.bin receives the last
// layer's 8 x height x width result.  The GPU test runs the same table through the Python surface and requires equal
// bits.  Besides the network the program checks known answers (zero-sum kernels on constant images, a 1x1
// convolution of ones), the factory's error texts, the frame pipeline and a pool of instances.
// Exit status 0 when every check passed.
#define FYNHIP_REFERENCE_NAMESPACE
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "fynhip.hpp"

namespace fn = fyusion::fyusenet;

static int g_failed = 0;
static void expect(bool ok, const char* what, int line) {
    if (!ok) {
        std::fprintf(stderr, "surface_example.cpp:%d: %s\n", line, what);
        g_failed++;
    }
}
#define CHECK(c) expect((c), "check failed: " #c, __LINE__)

// ---- the table -----------------------------------------------------------------------------------------------------
enum Kind { UP, CONV, TCONV, DOWN };
struct Row {
    int no;
    const char* name;
    Kind kind;
    int kernel, cin, cout;
    int shrink;        // the layer's input is (height/shrink) x (width/shrink)
    int stride;        // down-sampling (CONV) or up-sampling (TCONV) step
    fn::ActType act;   // applied while reading the input
    bool bn;           // block carries bnScale/bnBias
    int padOut;        // zero border the layer writes around its output
    int from;          // producer of port 0, -1: none
    int residualFrom;  // producer of port 1, -1: none
};
static const Row kTable[] = {
    {0, "in", UP, 0, 3, 3, 1, 1, fn::ActType::NONE, false, 2, -1, -1},
    {1, "wide", CONV, 5, 3, 16, 1, 1, fn::ActType::NONE, true, 1, 0, -1},
    {2, "down", CONV, 3, 16, 32, 1, 2, fn::ActType::RELU, true, 1, 1, -1},
    {3, "pair_a", CONV, 3, 32, 32, 2, 1, fn::ActType::RELU, true, 1, 2, -1},
    {4, "pair_b", CONV, 3, 32, 32, 2, 1, fn::ActType::RELU, true, 1, 3, 2},
    {5, "up", TCONV, 3, 32, 16, 2, 2, fn::ActType::RELU, true, 0, 4, -1},
    {6, "mix", CONV, 1, 16, 8, 1, 1, fn::ActType::LEAKY_RELU, false, 0, 5, -1},
    {7, "out", DOWN, 0, 8, 8, 1, 1, fn::ActType::NONE, false, 0, 6, -1},
};
static const float kLeak = 0.125f;
static size_t blockFloats(const Row& r) {
    if (r.kind != CONV && r.kind != TCONV) return 0;
    return (size_t)r.cout + (size_t)r.cout * r.kernel * r.kernel * r.cin + (r.bn ? 2 * (size_t)r.cout : 0);
}
static size_t streamFloats() {
    size_t n = 0;
    for (const Row& r : kTable) n += blockFloats(r);
    return n;
}

class Hourglass : public fn::NeuralNetwork {
  public:
    Hourglass(int width, int height, std::vector<float> stream) : width_(width), height_(height), stream_(std::move(stream)) {}
    void reload(const std::vector<float>& stream) {
        stream_ = stream;
        if (isSetup()) initializeWeights(getLayers());
    }
    static int first() { return kTable[0].no; }
    static int last() { return kTable[sizeof(kTable) / sizeof(kTable[0]) - 1].no; }

  protected:
    fn::CompiledLayers buildLayers() override {
        auto factory = getLayerFactory();
        for (const Row& r : kTable) {
            const int h = height_ / r.shrink, w = width_ / r.shrink;
            if (r.kind == UP || r.kind == DOWN) {
                auto* b = new fn::gpu::UpDownLayerBuilder(r.kind == UP ? fn::gpu::UpDownLayerBuilder::UPLOAD : fn::gpu::UpDownLayerBuilder::DOWNLOAD, r.name);
                b->shape(r.cout, h, w, r.cin).outputPadding((short)r.padOut).context(context()).number(r.no);
                if (r.kind == DOWN) b->deep();   // uploads are shallow (three channels), the download reads a deep tensor
                b->push(factory);
                continue;
            }
            auto* b = new fn::gpu::ConvLayerBuilder((short)r.kernel, r.name);
            b->shape(r.cout, h, w, r.cin).deep().inputPadding((short)((r.kernel - 1) / 2)).outputPadding((short)r.padOut);
            b->prefixAct(r.act).context(context()).number(r.no);
            if (r.act == fn::ActType::LEAKY_RELU) b->leakyReLU(kLeak);
            if (r.bn) b->postfixNorm(fn::NormType::BATCHNORM);
            if (r.kind == TCONV) {
                b->type(fn::LayerType::TRANSCONVOLUTION2D).upsample((short)r.stride).crop(1);
            } else {
                b->type(fn::LayerType::CONVOLUTION2D).downsample((short)r.stride);
            }
            if (r.residualFrom >= 0) b->residual(fn::ActType::RELU).residualPadding((short)r.padOut);
            b->push(factory);
        }
        return factory->compileLayers();
    }
    void connectLayers(fn::CompiledLayers& layers, fn::BufferManager* buffers) override {
        for (const Row& r : kTable) {
            if (r.from >= 0) buffers->connectLayers(layers[r.from], layers[r.no], 0);
            if (r.residualFrom >= 0) buffers->connectLayers(layers[r.residualFrom], layers[r.no], 1);
        }
    }
    void initializeWeights(fn::CompiledLayers& layers) override {
        size_t at = 0;
        for (const Row& r : kTable) {
            const size_t n = blockFloats(r);
            if (!n) continue;
            auto* weighted = dynamic_cast<fn::ConvLayerInterface*>(layers[r.name]);
            CHECK(weighted != nullptr);
            CHECK(layers[r.no]->weightFloats() == n);
            if (weighted) weighted->loadWeightsAndBiases(stream_.data(), at);
            at += n;
        }
        CHECK(at == stream_.size());
    }

  private:
    int width_, height_;
    std::vector<float> stream_;
};

// ---- one convolution on a constant image -------------------------------------------------------------------------------
struct OneConv : fn::NeuralNetwork {
    int kernel, cout, size, cin, pad;
    bool deep;
    std::vector<float> block;
    OneConv(int k, int co, int sz, int ci, bool dp, int pd, std::vector<float> blk)
        : kernel(k), cout(co), size(sz), cin(ci), pad(pd), deep(dp), block(std::move(blk)) {}
    fn::CompiledLayers buildLayers() override {
        auto factory = getLayerFactory();
        auto* b = new fn::gpu::ConvLayerBuilder((short)kernel, "only");
        b->shape(cout, size, size, cin).type(fn::LayerType::CONVOLUTION2D).inputPadding((short)pad).number(1);
        if (deep) b->deep();
        b->push(factory);
        return factory->compileLayers();
    }
    void connectLayers(fn::CompiledLayers&, fn::BufferManager*) override {}
    void initializeWeights(fn::CompiledLayers& layers) override {
        dynamic_cast<fn::ConvLayerInterface*>(layers[1])->loadWeightsAndBiases(block.data(), 0);
    }
    std::vector<float> runOnOnes() {
        setup();
        std::vector<float> ones((size_t)cin * size * size, 1.f);
        getLayers()[1]->setInput(ones.data());
        forward();
        finish();
        return getLayers()["only"]->copyResult();
    }
};

// kernel rows weighted rowWeight[ky], the same for every column, input and output channel; zero bias
static std::vector<float> rowKernel(int cout, int cin, int k, const std::vector<float>& rowWeight) {
    std::vector<float> b((size_t)cout + (size_t)cout * k * k * cin, 0.f);
    size_t at = (size_t)cout;
    for (int o = 0; o < cout; o++)
        for (int ky = 0; ky < k; ky++)
            for (int kx = 0; kx < k; kx++)
                for (int i = 0; i < cin; i++) b[at++] = rowWeight[(size_t)ky];
    return b;
}

static void knownAnswers() {
    // zero halo (deep, padded): a (-1, 0, +1) row kernel on ones cancels inside; the first row only sees the +1 row
    // (and the middle row), the last row only the -1 row: +-3*cin
    {
        const int cin = 8, cout = 8, size = 32;
        OneConv net(3, cout, size, cin, true, 1, rowKernel(cout, cin, 3, {-1.f, 0.f, 1.f}));
        const std::vector<float> out = net.runOnOnes();
        CHECK(out.size() == (size_t)cout * size * size);
        int wrong = 0;
        for (int o = 0; o < cout; o++)
            for (int y = 0; y < size; y++)
                for (int x = 1; x + 1 < size; x++) {
                    const float want = y == 0 ? 3.f * cin : (y + 1 == size ? -3.f * cin : 0.f);
                    wrong += out[((size_t)o * size + y) * size + x] != want;
                }
        CHECK(wrong == 0);
    }
    // repeated edge (shallow, unpadded): the same kernel gives zero on the border rows as well
    {
        OneConv net(3, 8, 32, 4, false, 0, rowKernel(8, 4, 3, {-1.f, 0.f, 1.f}));
        int wrong = 0;
        for (float v : net.runOnOnes()) wrong += v != 0.f;
        CHECK(wrong == 0);
    }
    // one tap of ones: every output is the number of input channels
    {
        const int cin = 12, cout = 16;
        OneConv net(1, cout, 20, cin, true, 0, rowKernel(cout, cin, 1, {1.f}));
        int wrong = 0;
        for (float v : net.runOnOnes()) wrong += v != (float)cin;
        CHECK(wrong == 0);
    }
}

// ---- descriptions the factory refuses ------------------------------------------------------------------------------------
struct Refused : fn::NeuralNetwork {
    int variant;
    explicit Refused(int v) : variant(v) {}
    fn::CompiledLayers buildLayers() override {
        auto factory = getLayerFactory();
        switch (variant) {
            case 0:  // one number used twice
                (new fn::gpu::GPULayerBuilder("first"))->shape(4, 8, 8, 4).type(fn::LayerType::RELU).number(1).push(factory);
                (new fn::gpu::GPULayerBuilder("second"))->shape(4, 8, 8, 4).type(fn::LayerType::RELU).number(1).push(factory);
                break;
            case 1:  // fractional-step convolution on a deep tensor
                (new fn::gpu::ConvLayerBuilder(3, "frac"))->shape(4, 8, 8, 4).type(fn::LayerType::FRACCONVOLUTION2D).sourceStep(0.5f).deep().number(1).push(factory);
                break;
            default:  // no number at all
                (new fn::gpu::GPULayerBuilder("nameless"))->shape(4, 8, 8, 4).type(fn::LayerType::RELU).push(factory);
        }
        return factory->compileLayers();
    }
    void connectLayers(fn::CompiledLayers&, fn::BufferManager*) override {}
    void initializeWeights(fn::CompiledLayers&) override {}
};

static void refusals() {
    const char* text[3] = {"already taken", "not supported for deep layers", "valid number"};
    for (int v = 0; v < 3; v++) {
        std::string got;
        try {
            Refused net(v);
            net.setup();
        } catch (const fn::FynException& ex) {
            got = ex.what();
        }
        if (got.find(text[v]) == std::string::npos) std::fprintf(stderr, "variant %d: message was '%s'\n", v, got.c_str());
        CHECK(got.find(text[v]) != std::string::npos);
    }
}

static std::vector<float> readFloats(const char* path, size_t count) {
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
        knownAnswers();
        refusals();
        const std::vector<float> stream = readFloats(argv[1], streamFloats());
        const std::vector<float> frame = readFloats(argv[2], (size_t)3 * width * height);
        const size_t outFloats = (size_t)8 * width * height;
        Hourglass net(width, height, stream);
        net.setup();
        net.getLayers()["in"]->setInput(frame.data());
        const auto state = net.forward();
        CHECK(state.status == fn::NeuralNetwork::EXEC_DONE);
        net.finish();
        std::vector<float> result(outFloats);
        net.getOutput(Hourglass::last(), result.data());
        CHECK(net.getLayers()[6]->copyResult() == result);

        // layers come out of CompiledLayers in ascending number
        int previous = -1, count = 0;
        for (auto it = net.getLayers().begin(); it != net.getLayers().end(); ++it, ++count) {
            CHECK(it.second->getNumber() > previous);
            previous = it.second->getNumber();
        }
        CHECK(count == (int)(sizeof(kTable) / sizeof(kTable[0])));

        // the frame pipeline delivers the same frame
        std::vector<float> again(outFloats, -1.f);
        net.asyncBegin(Hourglass::first(), Hourglass::last(), FYN_ORDER_CHANNELWISE, FYN_ORDER_CHANNELWISE, 2);
        net.asyncWait(net.asyncSubmit(frame.data(), again.data()));
        net.asyncEnd();
        CHECK(again == result);

        // a second load of the same stream after setup changes nothing; a different stream does
        net.reload(stream);
        net.forward();
        net.finish();
        net.getOutput(Hourglass::last(), again.data());
        CHECK(again == result);
        std::vector<float> halved = stream;
        for (float& v : halved) v *= 0.5f;
        net.reload(halved);
        net.forward();
        net.finish();
        net.getOutput(Hourglass::last(), again.data());
        CHECK(again != result);

        // three instances side by side: each frame's result arrives under its own ticket
        {
            fn::FramePool<Hourglass> pool([&]() { return std::unique_ptr<Hourglass>(new Hourglass(width, height, stream)); },
                                          Hourglass::first(), Hourglass::last(), 3, 2);
            std::vector<std::vector<float>> outs(7, std::vector<float>(outFloats, -1.f));
            uint64_t ticket = 0;
            for (auto& o : outs) ticket = pool.submit(frame.data(), o.data());
            pool.wait(ticket);
            int differing = 0;
            for (auto& o : outs) differing += o != result;
            CHECK(differing == 0);
            CHECK(pool.instances() == 3);
        }
        FILE* f = std::fopen(argv[3], "wb");
        if (!f || std::fwrite(result.data(), sizeof(float), result.size(), f) != result.size()) {
            std::fprintf(stderr, "cannot write %s\n", argv[3]);
            return 2;
        }
        std::fclose(f);
        std::printf("%s\n", net.getLayers()["up"]->kernelInfo().c_str());
    } catch (const fn::FynException& ex) {
        std::fprintf(stderr, "FynException (%d): %s\n", ex.status(), ex.what());
        return 1;
    }
    std::printf("%d check(s) failed\n", g_failed);
    return g_failed == 0 ? 0 : 1;
}
