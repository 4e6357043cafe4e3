// Network graph, device tensor management and the forward loop.
#include "engine.h"
#include "range.h"

#include <algorithm>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <vector>

namespace fynhip {

void fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    throw Error(code, buf);
}

// ---------------------------------------------------------------------------------------------
// Layer base
// ---------------------------------------------------------------------------------------------
Layer::Layer(Net* n, const fyn_layer_desc& desc) : d(desc), net(n) {}

Act Layer::act() const {
    // LayerBuilderTempl::getFlags (base/layerbuilder.h:445-493): RELU and LEAKY_RELU both set PRE_RELU,
    // the leak value distinguishes them (gpu/gpulayerbase.cpp:775-802).
    // Kernels may evaluate the activation branch-free as min(hi, max(lo, x)) + leak * min(x, 0); the
    // fields are normalised for that here.
    const float inf = std::numeric_limits<float>::infinity();
    Act a{ACT_NONE, 0.f, -inf, inf};
    if (d.flags & FYN_FLAG_PRE_RELU) {
        a.lo = 0.f;
        if (d.leaky_relu != 0.f) {
            a.kind = ACT_LEAKY;
            a.leak = d.leaky_relu;
        } else {
            a.kind = ACT_RELU;
        }
    } else if (d.flags & FYN_FLAG_PRE_CLIP) {
        a.kind = ACT_CLIP;
        a.lo = d.clip_low;
        a.hi = d.clip_high;
    }
    return a;
}

void Layer::port_shape(int port, int& c, int& h, int& w, int& pad) const {
    if (port == 0) {
        c = d.in_channels;
        h = d.height;
        w = d.width;
        pad = d.input_padding;
    } else {  // residual: same net size as the output (base/layerbase.h:266-274)
        c = oc;
        h = oh;
        w = ow;
        pad = d.residual_padding;
    }
}

const Tensor& Layer::tin(int port) const { return net->tensors[in[port]]; }
const Tensor& Layer::tout() const { return net->tensors[out]; }

// ---------------------------------------------------------------------------------------------
// Streams.  All streams of a device are created together, when the library first needs one there, and are leased to
// networks afterwards.  Measured on this runtime: streams created after the process has launched its first hipGraph
// overlap each other badly (four ResNet-50 instances side by side: 3000 frames/s instead of 4700), whereas streams
// that exist by then are unaffected by later graph launches.  Leasing also keeps the stream count of a process that
// builds and destroys many networks constant.  Streams are never destroyed; a network that finds none free gets a
// new one.  The first kMainStreams entries serve networks' own streams (consecutive ones land on different hardware
// queues), the rest their copy streams.
// ---------------------------------------------------------------------------------------------
namespace {
struct DeviceStreams {
    std::vector<hipStream_t> streams;
    std::vector<char> leased;
};
constexpr size_t kMainStreams = 8, kCopyStreams = 8;
std::mutex g_streams_mu;
std::map<int, DeviceStreams> g_streams;

hipStream_t lease_stream(int device, bool copy) {
    std::lock_guard<std::mutex> lk(g_streams_mu);
    DeviceStreams& ds = g_streams[device];
    if (ds.streams.empty()) {
        for (size_t i = 0; i < kMainStreams + kCopyStreams; i++) {
            hipStream_t st = nullptr;
            if (i < kMainStreams) FYN_HIP(hipStreamCreate(&st));
            else FYN_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
            ds.streams.push_back(st);
            ds.leased.push_back(0);
        }
    }
    const size_t lo = copy ? kMainStreams : 0, hi = copy ? kMainStreams + kCopyStreams : kMainStreams;
    for (size_t i = lo; i < hi; i++)
        if (!ds.leased[i]) {
            ds.leased[i] = 1;
            return ds.streams[i];
        }
    hipStream_t st = nullptr;   // all taken: one more, destroyed again when it comes back
    if (copy) FYN_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    else FYN_HIP(hipStreamCreate(&st));
    return st;
}

void return_stream(int device, hipStream_t st) {
    if (!st) return;
    std::lock_guard<std::mutex> lk(g_streams_mu);
    DeviceStreams& ds = g_streams[device];
    for (size_t i = 0; i < ds.streams.size(); i++)
        if (ds.streams[i] == st) {
            ds.leased[i] = 0;
            return;
        }
    (void)hipStreamDestroy(st);   // an overflow stream
}
}  // namespace

// ---------------------------------------------------------------------------------------------
// Fixed staging area for read-backs that must not allocate (Net::copy_result_static).  One array per GPU, part of the
// loaded code object and held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the address it yields on each device is what kernels and copies receive.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) __attribute__((used)) float scratch[FYN_STATIC_SCRATCH_FLOATS];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};

// The calling thread's current device must be `device`.
float* static_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) fail(FYN_ERR_DEVICE, "device %d beyond the %d devices the fixed staging area covers", device, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        float* p = nullptr;
        FYN_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
        if (!p) fail(FYN_ERR_DEVICE, "no device address for the fixed staging area on device %d", device);
        g_scratch_ptr[device] = p;
    }
    return g_scratch_ptr[device];
}
}  // namespace

// ---------------------------------------------------------------------------------------------
// Net
// ---------------------------------------------------------------------------------------------
extern "C" char** environ;

void Switches::read() {
    v_.clear();
    for (char** e = environ; e && *e; e++) {
        if (strncmp(*e, "FYNHIP_", 7) != 0) continue;
        const char* eq = strchr(*e, '=');
        if (eq) v_[std::string(*e, eq - *e)] = std::string(eq + 1);
    }
}
const char* Switches::get(const char* name) const {
    auto it = v_.find(name);
    return it == v_.end() ? nullptr : it->second.c_str();
}

Net::Net(int dev, int stor) : device(dev), storage(stor) {
    sw.read();
    if (stor != FYN_STORAGE_F32 && stor != FYN_STORAGE_F16) fail(FYN_ERR_INVALID, "unknown storage type %d", stor);
    int count = 0;
    FYN_HIP(hipGetDeviceCount(&count));
    if (dev < 0 || dev >= count) fail(FYN_ERR_DEVICE, "device %d not present (%d devices)", dev, count);
    FYN_HIP(hipSetDevice(dev));
    stream = lease_stream(dev, false);
    // resolved here, where the caller may still allocate: looking the symbol up loads the code object on this device
    static_scratch_ = static_scratch(dev);
}

Net::~Net() {
    (void)hipSetDevice(device);
    try {
        async_end();
    } catch (...) {
    }
    if (stream) (void)hipStreamSynchronize(stream);
    if (graph_exec_) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_) (void)hipGraphDestroy(graph_);
    for (auto& kv : layers) {
        if (kv.second->ev0) (void)hipEventDestroy(kv.second->ev0);
        if (kv.second->ev1) (void)hipEventDestroy(kv.second->ev1);
    }
    layers.clear();
    for (void* p : allocs_) (void)hipFree(p);
    return_stream(device, stream);
}

void* Net::dev_alloc(size_t bytes, bool zero) {
    void* p = nullptr;
    if (bytes == 0) bytes = 16;
    FYN_HIP(hipMalloc(&p, bytes));
    allocs_.push_back(p);
    alloc_calls_++;
    alloc_bytes_ += bytes;
    if (zero) {
        launch_fill_zero(p, bytes, stream);
        FYN_HIP(hipGetLastError());
    }
    return p;
}

void Net::dev_free(void* p) {
    auto it = std::find(allocs_.begin(), allocs_.end(), p);
    if (it == allocs_.end()) return;
    FYN_HIP(hipStreamSynchronize(stream));
    allocs_.erase(it);
    (void)hipFree(p);
}

void Net::dev_free_many(const std::vector<void*>& ptrs) {
    bool synced = false;
    for (void* p : ptrs) {
        auto it = std::find(allocs_.begin(), allocs_.end(), p);
        if (it == allocs_.end()) continue;
        if (!synced) {
            FYN_HIP(hipStreamSynchronize(stream));
            synced = true;
        }
        allocs_.erase(it);
        (void)hipFree(p);
    }
}

float* Net::staging(size_t floats) {
    if (floats > staging_floats_) {
        FYN_HIP(hipStreamSynchronize(stream));
        // the old area stays owned by allocs_ and is released with the net
        staging_ = static_cast<float*>(dev_alloc(floats * sizeof(float), false));
        staging_floats_ = floats;
    }
    return staging_;
}

Layer* Net::layer(int number) {
    auto it = layers.find(number);
    if (it == layers.end()) fail(FYN_ERR_NOTFOUND, "no layer with number %d", number);
    return it->second.get();
}

void Net::add_layer(const fyn_layer_desc& d) {
    if (is_setup) fail(FYN_ERR_STATE, "cannot add layers after setup");
    // LayerFactory::pushBuilder (base/layerfactory.cpp:67-76)
    if (d.number < 0) fail(FYN_ERR_INVALID, "Must identify each layer with a valid number (found %d in the builder)", d.number);
    if (layers.count(d.number)) fail(FYN_ERR_DUPLICATE, "Trying to insert a layer on a position that is already taken (%d)", d.number);
    std::unique_ptr<Layer> l(create_layer(this, d));   // may throw: nothing is registered then
    layers[d.number] = std::move(l);
}

void Net::add_custom_layer(const fyn_layer_desc& d, const fyn_custom_layer& impl) {
    if (is_setup) fail(FYN_ERR_STATE, "cannot add layers after setup");
    if (d.number < 0) fail(FYN_ERR_INVALID, "Must identify each layer with a valid number (found %d in the builder)", d.number);
    if (layers.count(d.number)) fail(FYN_ERR_DUPLICATE, "Trying to insert a layer on a position that is already taken (%d)", d.number);
    std::unique_ptr<Layer> l(create_custom_layer(this, d, impl));
    layers[d.number] = std::move(l);
}

void Net::connect(int out_layer, int in_layer, int port) {
    if (is_setup) fail(FYN_ERR_STATE, "cannot connect layers after setup");
    Layer* src = layer(out_layer);
    Layer* dst = layer(in_layer);
    if (port < 0 || port >= dst->num_ports())
        fail(FYN_ERR_INVALID, "layer %s has no input port %d", dst->d.name, port);
    if (!(in_layer > out_layer))
        fail(FYN_ERR_INVALID, "layer %s (%d) cannot feed layer %s (%d): execution is in ascending number", src->d.name,
             out_layer, dst->d.name, in_layer);
    if (dst->in[port] != -1) return;  // already connected (BufferManager::checkIOMatch returns no match)
    // I/O match (base/buffermanager.cpp:462-492): same geometry on both sides of the edge.  The reference compares
    // textures, four channels each, not channel counts: a consumer may name up to three channels more or fewer
    // than were produced (the style-transfer samples download 4 channels of a 3-channel result,
    // samples/samplenetworks/stylenet3x3.cpp:175,180).  Channels beyond the produced ones read as zero.
    int c, h, w, pad;
    dst->port_shape(port, c, h, w, pad);
    if ((c + 3) / 4 != (src->oc + 3) / 4 || h != src->oh || w != src->ow || pad != src->d.output_padding)
        fail(FYN_ERR_INVALID,
             "Inputs/outputs do not match (I/O) for layers %s and %s: producer %dx%dx%d pad %d, consumer port %d wants "
             "%dx%dx%d pad %d",
             dst->d.name, src->d.name, src->oc, src->oh, src->ow, src->d.output_padding, port, c, h, w, pad);
    // tensors are created lazily: the producer's output tensor id
    if (src->out == -1) {
        if (!src->has_own_output()) {
            fail(FYN_ERR_INVALID, "layer %s has no output that can be connected", src->d.name);
        }
        Tensor t;
        t.producer = src->d.number;
        tensors.push_back(t);
        src->out = (int)tensors.size() - 1;
    }
    dst->in[port] = src->out;
    tensors[src->out].last_reader = std::max(tensors[src->out].last_reader, in_layer);
}

void Net::setup() {
    if (is_setup) fail(FYN_ERR_STATE, "network is already set up");
    FYN_HIP(hipSetDevice(device));
    // 1. tensors: external inputs for unconnected ports, outputs for every layer
    for (auto& kv : layers) {
        Layer* l = kv.second.get();
        for (int p = 0; p < l->num_ports(); p++) {
            if (l->in[p] != -1) continue;
            Tensor t;
            t.producer = -1;
            t.locked = true;
            t.last_reader = l->d.number;
            tensors.push_back(t);
            l->in[p] = (int)tensors.size() - 1;
            int c, h, w, pad;
            l->port_shape(p, c, h, w, pad);
            TView& v = tensors.back().v;
            v.c = c; v.h = h; v.w = w; v.pad = pad; v.cp = channel_pitch(c); v.f16 = f16();
        }
        if (l->has_own_output()) {
            if (l->out == -1) {
                Tensor t;
                t.producer = l->d.number;
                t.locked = true;  // nobody consumes it: it is a network output
                tensors.push_back(t);
                l->out = (int)tensors.size() - 1;
            }
            if (l->d.type == FYN_LAYER_UPLOAD) tensors[l->out].locked = true;  // filled from the host
            TView& v = tensors[l->out].v;
            v.c = l->oc; v.h = l->oh; v.w = l->ow; v.pad = l->d.output_padding; v.cp = channel_pitch(l->oc); v.f16 = f16();
        } else {
            // pass-through (download): output aliases the input, which must survive
            l->out = l->in[0];
            tensors[l->out].locked = true;
        }
    }
    keep_projection_inputs(this);
    // 2. device buffers.  Liveness rule of BufferManager::findTexture (base/buffermanager.cpp:512-525)
    //    restated for in-order stream execution: a buffer can take layer N's output when every reader of
    //    its current tenant has a number < N; only buffers of identical geometry are shared so that the
    //    zero halo written at allocation stays valid.
    for (auto& kv : layers) {
        Layer* l = kv.second.get();
        for (int p = 0; p < l->num_ports(); p++) {
            Tensor& t = tensors[l->in[p]];
            if (t.buffer == -1 && t.producer == -1) {
                DevBuffer b;
                b.bytes = t.v.bytes();
                b.ptr = dev_alloc(b.bytes);
                b.locked = true;
                buffers.push_back(b);
                t.buffer = (int)buffers.size() - 1;
                t.v.ptr = b.ptr;
            }
        }
        if (!l->has_own_output()) continue;
        Tensor& t = tensors[l->out];
        int found = -1;
        if (reuse_buffers && !t.locked) {
            for (size_t i = 0; i < buffers.size(); i++) {
                DevBuffer& b = buffers[i];
                if (!b.locked && b.free_after < l->d.number && b.h == t.v.h && b.w == t.v.w && b.pad == t.v.pad &&
                    b.cp == t.v.cp && b.f16 == t.v.f16) {
                    found = (int)i;
                    break;
                }
            }
        }
        if (found == -1) {
            DevBuffer b;
            b.bytes = t.v.bytes();
            b.ptr = dev_alloc(b.bytes);
            b.h = t.v.h; b.w = t.v.w; b.pad = t.v.pad; b.cp = t.v.cp; b.f16 = t.v.f16;
            buffers.push_back(b);
            found = (int)buffers.size() - 1;
        }
        DevBuffer& b = buffers[found];
        b.locked = t.locked;
        b.free_after = std::max(t.last_reader, l->d.number);
        t.buffer = found;
        t.v.ptr = b.ptr;
    }
    // pass-through layers were given the tensor id only; nothing else to do for them
    assign_range_words();
    // 3. per-layer setup (weight packing, kernel selection)
    for (auto& kv : layers) {
        kv.second->setup();
        kv.second->set_up = true;
    }
    fuse_depthwise_layers(this);
    fuse_projection_layers(this);
    fuse_batchnorm_layers(this);
    assign_range_resets();
    poison_lds_ = sw.get("FYNHIP_POISON_LDS") != nullptr;
    FYN_HIP(hipStreamSynchronize(stream));
    is_setup = true;
}

// Value ranges (range.h), fp32 storage only.  A tensor gets a word when whoever writes it keeps the word up to date:
// tensors fed from the host (set_input and the frame pipeline clear and raise the word themselves) and the outputs of
// layers whose kernels do (tracks_range()).
void Net::assign_range_words() {
    if (f16() || sw.get("FYNHIP_NO_RANGE_TRACKING") || sw.get("FYNHIP_FORCE_DIRECT_CONV") || tensors.empty()) return;
    amax_dev_ = static_cast<unsigned*>(dev_alloc(tensors.size() * RANGE_WORDS * sizeof(unsigned), true));
    for (size_t i = 0; i < tensors.size(); i++) {
        Tensor& t = tensors[i];
        bool tracked = t.producer == -1;
        if (t.producer >= 0) {
            Layer* pl = layer(t.producer);
            tracked = pl->d.type == FYN_LAYER_UPLOAD || pl->tracks_range();
        }
        if (tracked) t.amax = amax_dev_ + i * RANGE_WORDS;
    }
}

// A word raised during a forward pass must read 0 again before the tensor's producer runs in the next pass.  The
// clearing is given to a convolution kernel that runs after the tensor's last reader (kernels of one stream run one
// after the other, so nothing else touches the word at that time): the first such layer behind the last reader,
// wrapping around to the layers in front of the producer.  A tensor for which no layer is found loses its word.
void Net::assign_range_resets() {
    if (!amax_dev_) return;
    std::vector<int> order;
    for (auto& kv : layers) order.push_back(kv.first);
    bool lost = false;
    for (Tensor& t : tensors) {
        if (!t.amax || t.producer < 0) continue;
        Layer* pl = layer(t.producer);
        if (pl->d.type == FYN_LAYER_UPLOAD) continue;   // cleared where it is written from the host
        const int last = std::max(t.last_reader, t.producer);
        bool done = false;
        // layers behind the last reader, in execution order ...
        for (int no : order)
            if (no > last && layer(no)->add_range_reset(t.amax)) { done = true; break; }
        // ... then the layers in front of the producer (they run in the next pass, before it)
        if (!done)
            for (int no : order)
                if (no < t.producer && layer(no)->add_range_reset(t.amax)) { done = true; break; }
        if (!done) {
            t.amax = nullptr;
            lost = true;
        }
    }
    if (lost) {
        // layers copied the word addresses into their kernel arguments during setup: let them look again
        for (auto& kv : layers) kv.second->setup_ranges();
    }
}

void Net::dump_layer(Layer* l) {
    // Engine::enableIntermediateOutput (base/engine.cpp:174-181,602-604): <name>_<seq>.bin, CHW fp32
    if (!l->has_own_output()) return;
    const TView& v = l->tout().v;
    std::vector<float> host((size_t)v.c * v.h * v.w);
    copy_result(l->d.number, host.data(), 0);
    char path[1024];
    snprintf(path, sizeof(path), "%s/%s_%llu.bin", dump_dir.c_str(), l->d.name, (unsigned long long)seq);
    FILE* f = fopen(path, "wb");
    if (!f) fail(FYN_ERR_INVALID, "cannot write %s", path);
    fwrite(host.data(), sizeof(float), host.size(), f);
    fclose(f);
}

void Net::run_layers(bool with_events) {
    for (auto& kv : layers) {
        Layer* l = kv.second.get();
        if (with_events) {
            if (!l->ev0) {
                FYN_HIP(hipEventCreate(&l->ev0));
                FYN_HIP(hipEventCreate(&l->ev1));
            }
            FYN_HIP(hipEventRecord(l->ev0, stream));
        }
        if (poison_lds_ && launch_poison_lds(stream) != 0) fail(FYN_ERR_DEVICE, "LDS fill failed");
        l->forward(stream);
        FYN_HIP(hipGetLastError());
        if (with_events) FYN_HIP(hipEventRecord(l->ev1, stream));
        if (!dump_dir.empty()) dump_layer(l);
    }
}

void Net::collect_timings() {
    if (!events_pending_) return;
    for (auto& kv : layers) {
        Layer* l = kv.second.get();
        if (!l->ev0) continue;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, l->ev0, l->ev1) == hipSuccess) {
            l->ms_total += ms;
            l->runs++;
        }
    }
    events_pending_ = false;
}

void Net::forward(uint64_t* seq_out) {
    if (!is_setup) fail(FYN_ERR_STATE, "forward() called on a network that was not set up");
    FYN_HIP(hipSetDevice(device));
    seq++;
    if (seq_out) *seq_out = seq;
    const bool plain = timings || !dump_dir.empty();
    if (graph_enabled_ && !plain) {
        if (!graph_exec_) {
            FYN_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
            try {
                run_layers(false);
            } catch (...) {
                hipGraph_t g = nullptr;
                (void)hipStreamEndCapture(stream, &g);
                if (g) (void)hipGraphDestroy(g);
                throw;
            }
            FYN_HIP(hipStreamEndCapture(stream, &graph_));
            FYN_HIP(hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0));
        }
        FYN_HIP(hipGraphLaunch(graph_exec_, stream));
        return;
    }
    if (timings) {
        FYN_HIP(hipStreamSynchronize(stream));
        collect_timings();
    }
    run_layers(timings);
    events_pending_ = timings;
}

void Net::finish() {
    FYN_HIP(hipSetDevice(device));
    FYN_HIP(hipStreamSynchronize(stream));
    collect_timings();
}

void Net::use_graph(bool enable) {
    graph_enabled_ = enable;
    if (!enable && graph_exec_) {
        FYN_HIP(hipStreamSynchronize(stream));
        (void)hipGraphExecDestroy(graph_exec_);
        (void)hipGraphDestroy(graph_);
        graph_exec_ = nullptr;
        graph_ = nullptr;
    }
}

const Tensor& Net::input_tensor(int layer_no, int port) {
    if (!is_setup) fail(FYN_ERR_STATE, "set_input() before setup()");
    Layer* l = layer(layer_no);
    if (l->d.type == FYN_LAYER_UPLOAD) return l->tout();
    if (port < 0 || port >= l->num_ports()) fail(FYN_ERR_INVALID, "layer %s has no input port %d", l->d.name, port);
    const Tensor& t = l->tin(port);
    if (t.producer != -1) fail(FYN_ERR_INVALID, "input port %d of layer %s is fed by layer %d", port, l->d.name, t.producer);
    return t;
}

size_t Net::input_floats(int layer_no, int port) {
    const TView& v = input_tensor(layer_no, port).v;
    return (size_t)v.c * v.h * v.w;
}

void Net::async_sizes(size_t* in_floats, size_t* out_floats) const {
    if (slots_.empty()) fail(FYN_ERR_STATE, "no frame pipeline is active");
    *in_floats = async_in_floats_;
    *out_floats = async_out_floats_;
}

void Net::set_input(int layer_no, int port, const float* data, int order) {
    if (!is_setup) fail(FYN_ERR_STATE, "set_input() before setup()");
    if (!data) fail(FYN_ERR_INVALID, "null input buffer");
    FYN_HIP(hipSetDevice(device));
    const TView& v = input_tensor(layer_no, port).v;
    const size_t n = (size_t)v.c * v.h * v.w;
    float* st = staging(n);
    FYN_HIP(hipMemcpyAsync(st, data, n * sizeof(float), hipMemcpyHostToDevice, stream));
    unsigned* amax = input_tensor(layer_no, port).amax;
    if (amax) launch_fill_zero(amax, RANGE_WORDS * sizeof(unsigned), stream);   // the tensor's value-range record starts over
    if (order == FYN_ORDER_CHANNELWISE) launch_chw_to_tensor(st, v, stream, amax);
    else if (order == FYN_ORDER_GPU_SHALLOW) launch_hwc_to_tensor(st, v.c, v, stream, amax);
    else fail(FYN_ERR_UNSUPPORTED, "input order %d not supported for upload", order);
    FYN_HIP(hipGetLastError());
    // the host buffer is borrowed for this call only
    FYN_HIP(hipStreamSynchronize(stream));
}

// What a layer hands out: its output tensor; a layer that only passes its input on (download) may name up to three
// channels more or fewer than were produced, inside the same group of four (the extra ones are zero).
static TView result_view(Layer* l) {
    TView v = l->tout().v;
    if (!l->has_own_output()) v.c = std::min(l->oc, v.cp);
    return v;
}

void Net::copy_result(int layer_no, float* chw, int include_padding) {
    if (!is_setup) fail(FYN_ERR_STATE, "copy_result() before setup()");
    FYN_HIP(hipSetDevice(device));
    Layer* l = layer(layer_no);
    const TView v = result_view(l);
    const size_t n = include_padding ? (size_t)v.c * v.hp() * v.wp() : (size_t)v.c * v.h * v.w;
    float* st = staging(n);
    launch_tensor_to_chw(v, st, include_padding, stream);
    FYN_HIP(hipGetLastError());
    FYN_HIP(hipMemcpyAsync(chw, st, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    FYN_HIP(hipStreamSynchronize(stream));
}

void Net::copy_result_static(int layer_no, float* chw, int include_padding) {
    if (!is_setup) fail(FYN_ERR_STATE, "copy_result() before setup()");
    if (!chw) fail(FYN_ERR_INVALID, "null result buffer");
    FYN_HIP(hipSetDevice(device));
    Layer* l = layer(layer_no);
    const TView v = result_view(l);
    const size_t n = include_padding ? (size_t)v.c * v.hp() * v.wp() : (size_t)v.c * v.h * v.w;
    if (n > (size_t)FYN_STATIC_SCRATCH_FLOATS)
        fail(FYN_ERR_INVALID, "result of layer %s (%d) has %zu floats, the fixed staging area holds %zu: use fyn_layer_copy_result",
             l->d.name, l->d.number, n, (size_t)FYN_STATIC_SCRATCH_FLOATS);
    // every element of [0, n) is written by the conversion kernel: nothing of an earlier call is read
    launch_tensor_to_chw(v, static_scratch_, include_padding, stream);
    FYN_HIP(hipGetLastError());
    FYN_HIP(hipMemcpyAsync(chw, static_scratch_, n * sizeof(float), hipMemcpyDefault, stream));
    FYN_HIP(hipStreamSynchronize(stream));
}

static void deep_tiling(int channels, int& tx, int& ty) {
    // CPUBufferShape::computeDeepTiling (cpu/cpubuffershape.cpp:430-448)
    const int tiles = (channels + 3) / 4;
    int best = 1 << 30;
    tx = tiles;
    ty = 1;
    for (int y = 1; y <= tiles; y++)
        for (int x = y; x <= tiles; x++)
            if (x * y >= tiles) {
                const int cost = (x - y) + (x * y - tiles);
                if (cost < best) {
                    best = cost;
                    tx = x;
                    ty = y;
                }
            }
}

void Net::get_output(int layer_no, float* data, int order) {
    if (!is_setup) fail(FYN_ERR_STATE, "get_output() before setup()");
    FYN_HIP(hipSetDevice(device));
    Layer* l = layer(layer_no);
    const TView v = result_view(l);
    if (order == FYN_ORDER_CHANNELWISE) {
        copy_result(layer_no, data, 0);
    } else if (order == FYN_ORDER_GPU_SHALLOW) {
        if (v.c > 4) fail(FYN_ERR_UNSUPPORTED, "GPU_SHALLOW download holds at most 4 channels per texel (layer has %d)", v.c);
        const int pc = v.c == 3 ? 4 : v.c;  // rendered textures are RGBA (base/buffermanager.cpp:478-483)
        const size_t n = (size_t)v.h * v.w * pc;
        float* st = staging(n);
        launch_tensor_to_hwc(v, st, pc, stream);
        FYN_HIP(hipGetLastError());
        FYN_HIP(hipMemcpyAsync(data, st, n * sizeof(float), hipMemcpyDeviceToHost, stream));
        FYN_HIP(hipStreamSynchronize(stream));
    } else if (order == FYN_ORDER_GPU_DEEP) {
        // tiled RGBA buffer, tile t at grid (t % tx, t / tx), padding shared between tiles
        // (gpu/deep/deeptiler.cpp:63-110)
        std::vector<float> chw((size_t)v.c * v.h * v.w);
        copy_result(layer_no, chw.data(), 0);
        int tx, ty;
        deep_tiling(v.c, tx, ty);
        const int pad = v.pad;
        const int dw = tx * (v.w + pad) + pad, dh = ty * (v.h + pad) + pad;
        memset(data, 0, (size_t)dw * dh * 4 * sizeof(float));
        for (int ch = 0; ch < v.c; ch++) {
            const int t = ch / 4, comp = ch % 4, gx = t % tx, gy = t / tx;
            for (int y = 0; y < v.h; y++)
                for (int x = 0; x < v.w; x++)
                    data[(((size_t)(pad + gy * (v.h + pad) + y)) * dw + pad + gx * (v.w + pad) + x) * 4 + comp] =
                        chw[((size_t)ch * v.h + y) * v.w + x];
        }
    } else {
        fail(FYN_ERR_INVALID, "unknown buffer order %d", order);
    }
}

void Net::time_forward(int iters, float* ms) {
    if (!is_setup) fail(FYN_ERR_STATE, "time_forward() before setup()");
    FYN_HIP(hipSetDevice(device));
    hipEvent_t a, b;
    FYN_HIP(hipEventCreate(&a));
    FYN_HIP(hipEventCreate(&b));
    const bool t = timings;
    timings = false;
    FYN_HIP(hipEventRecord(a, stream));
    for (int i = 0; i < iters; i++) forward(nullptr);
    FYN_HIP(hipEventRecord(b, stream));
    FYN_HIP(hipEventSynchronize(b));
    timings = t;
    FYN_HIP(hipEventElapsedTime(ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
}

void Net::time_steps(int iters, float* ms_each) {
    if (!is_setup) fail(FYN_ERR_STATE, "time_steps() before setup()");
    if (iters > 65536) fail(FYN_ERR_INVALID, "at most 65536 steps per call");
    FYN_HIP(hipSetDevice(device));
    // one event after every forward pass, all queued without waiting; differences of consecutive events are the steps
    std::vector<hipEvent_t> ev((size_t)iters + 1, nullptr);
    const bool t = timings;
    timings = false;
    try {
        for (auto& e : ev) FYN_HIP(hipEventCreate(&e));
        FYN_HIP(hipEventRecord(ev[0], stream));
        for (int i = 0; i < iters; i++) {
            forward(nullptr);
            FYN_HIP(hipEventRecord(ev[(size_t)i + 1], stream));
        }
        FYN_HIP(hipEventSynchronize(ev[(size_t)iters]));
        for (int i = 0; i < iters; i++) FYN_HIP(hipEventElapsedTime(&ms_each[i], ev[(size_t)i], ev[(size_t)i + 1]));
    } catch (...) {
        timings = t;
        (void)hipStreamSynchronize(stream);
        for (auto e : ev) if (e) (void)hipEventDestroy(e);
        throw;
    }
    timings = t;
    for (auto e : ev) (void)hipEventDestroy(e);
}

void Net::weights_changed() {
    if (!graph_exec_) return;
    FYN_HIP(hipSetDevice(device));
    FYN_HIP(hipStreamSynchronize(stream));
    (void)hipGraphExecDestroy(graph_exec_);
    (void)hipGraphDestroy(graph_);
    graph_exec_ = nullptr;
    graph_ = nullptr;
}

void Net::time_layer(int layer_no, int iters, float* ms) {
    if (!is_setup) fail(FYN_ERR_STATE, "time_layer() before setup()");
    FYN_HIP(hipSetDevice(device));
    Layer* l = layer(layer_no);
    // The launches are captured into one hipGraph so that host-side dispatch gaps do not enter the
    // measurement; the events bracket the graph on the network's stream.
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    FYN_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    try {
        for (int i = 0; i < iters; i++) l->forward(stream);
    } catch (...) {
        (void)hipStreamEndCapture(stream, &g);
        if (g) (void)hipGraphDestroy(g);
        throw;
    }
    FYN_HIP(hipStreamEndCapture(stream, &g));
    FYN_HIP(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
    hipEvent_t a, b;
    FYN_HIP(hipEventCreate(&a));
    FYN_HIP(hipEventCreate(&b));
    FYN_HIP(hipGraphLaunch(ge, stream));  // warm-up
    FYN_HIP(hipEventRecord(a, stream));
    FYN_HIP(hipGraphLaunch(ge, stream));
    FYN_HIP(hipEventRecord(b, stream));
    FYN_HIP(hipEventSynchronize(b));
    FYN_HIP(hipGetLastError());
    FYN_HIP(hipEventElapsedTime(ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    (void)hipGraphExecDestroy(ge);
    (void)hipGraphDestroy(g);
}

// ---------------------------------------------------------------------------------------------
// Frame pipeline (the counterpart of the reference engine's asynchronous mode, base/engine.cpp:386-683, with
// its two upload/download buffer sets, gpu/uploadlayer.h:74): three streams of equal priority joined by events.
// Frame i:   up stream    pinned host slot -> device staging slot
//            main stream  staging -> input tensor, all layers, output tensor -> device staging slot
//            down stream  device staging slot -> pinned host slot
// A slot is reused only after its download has completed, which also orders the staging buffers.
// ---------------------------------------------------------------------------------------------
void Net::async_begin(int in_layer, int in_port, int in_order, int out_layer, int out_order, int depth, bool copy_streams) {
    if (!is_setup) fail(FYN_ERR_STATE, "async_begin() before setup()");
    if (!slots_.empty()) fail(FYN_ERR_STATE, "frame pipeline is already active");
    if (depth < 1 || depth > 8) fail(FYN_ERR_INVALID, "pipeline depth %d out of range (1..8)", depth);
    FYN_HIP(hipSetDevice(device));
    Layer* li = layer(in_layer);
    if (li->d.type == FYN_LAYER_UPLOAD) {
        async_in_ = &li->tout();
    } else {
        if (in_port < 0 || in_port >= li->num_ports()) fail(FYN_ERR_INVALID, "layer %s has no input port %d", li->d.name, in_port);
        async_in_ = &li->tin(in_port);
        if (async_in_->producer != -1) fail(FYN_ERR_INVALID, "input port %d of layer %s is fed by layer %d", in_port, li->d.name, async_in_->producer);
    }
    async_out_ = &layer(out_layer)->tout();
    async_out_view_ = result_view(layer(out_layer));
    const TView& vi = async_in_->v;
    const TView& vo = async_out_view_;
    if (in_order != FYN_ORDER_CHANNELWISE && in_order != FYN_ORDER_GPU_SHALLOW) fail(FYN_ERR_UNSUPPORTED, "input order %d not supported for upload", in_order);
    if (out_order == FYN_ORDER_GPU_SHALLOW) {
        if (vo.c > 4) fail(FYN_ERR_UNSUPPORTED, "GPU_SHALLOW download holds at most 4 channels per texel (layer has %d)", vo.c);
        async_out_floats_ = (size_t)vo.h * vo.w * (vo.c == 3 ? 4 : vo.c);
    } else if (out_order == FYN_ORDER_CHANNELWISE) {
        async_out_floats_ = (size_t)vo.c * vo.h * vo.w;
    } else {
        fail(FYN_ERR_UNSUPPORTED, "output order %d not supported by the frame pipeline", out_order);
    }
    async_in_floats_ = (size_t)vi.c * vi.h * vi.w;
    async_in_order_ = in_order;
    async_out_order_ = out_order;
    async_own_streams_ = copy_streams;
    if (async_own_streams_) {
        up_stream_ = lease_stream(device, true);
        down_stream_ = lease_stream(device, true);
    } else {
        up_stream_ = down_stream_ = stream;
    }
    slots_.resize(depth);
    for (AsyncSlot& s : slots_) {
        FYN_HIP(hipHostMalloc(reinterpret_cast<void**>(&s.pin_in), async_in_floats_ * sizeof(float), hipHostMallocDefault));
        FYN_HIP(hipHostMalloc(reinterpret_cast<void**>(&s.pin_out), async_out_floats_ * sizeof(float), hipHostMallocDefault));
        FYN_HIP(hipMalloc(reinterpret_cast<void**>(&s.dev_in), async_in_floats_ * sizeof(float)));
        FYN_HIP(hipMalloc(reinterpret_cast<void**>(&s.dev_out), async_out_floats_ * sizeof(float)));
        FYN_HIP(hipEventCreateWithFlags(&s.up, hipEventDisableTiming));
        FYN_HIP(hipEventCreateWithFlags(&s.comp, hipEventDisableTiming));
        FYN_HIP(hipEventCreateWithFlags(&s.down, hipEventDisableTiming));
    }
}

void Net::async_complete(AsyncSlot& s) {
    if (!s.busy) return;
    FYN_HIP(hipEventSynchronize(s.down));
    if (s.user_out) memcpy(s.user_out, s.pin_out, async_out_floats_ * sizeof(float));
    s.busy = false;
}

void Net::async_submit(const float* in, float* out, uint64_t* ticket) {
    if (slots_.empty()) fail(FYN_ERR_STATE, "async_submit() without async_begin()");
    if (!in || !out) fail(FYN_ERR_INVALID, "null frame buffer");
    FYN_HIP(hipSetDevice(device));
    AsyncSlot& s = slots_[async_seq_ % slots_.size()];
    async_complete(s);  // oldest frame: its output is delivered before the slot is reused
    memcpy(s.pin_in, in, async_in_floats_ * sizeof(float));
    FYN_HIP(hipMemcpyAsync(s.dev_in, s.pin_in, async_in_floats_ * sizeof(float), hipMemcpyHostToDevice, up_stream_));
    FYN_HIP(hipEventRecord(s.up, up_stream_));
    FYN_HIP(hipStreamWaitEvent(stream, s.up, 0));
    if (async_in_->amax) launch_fill_zero(async_in_->amax, RANGE_WORDS * sizeof(unsigned), stream);   // the tensor's value-range record starts over
    if (async_in_order_ == FYN_ORDER_CHANNELWISE) launch_chw_to_tensor(s.dev_in, async_in_->v, stream, async_in_->amax);
    else launch_hwc_to_tensor(s.dev_in, async_in_->v.c, async_in_->v, stream, async_in_->amax);
    forward(nullptr);
    const TView& vo = async_out_view_;
    if (async_out_order_ == FYN_ORDER_CHANNELWISE) launch_tensor_to_chw(vo, s.dev_out, 0, stream);
    else launch_tensor_to_hwc(vo, s.dev_out, vo.c == 3 ? 4 : vo.c, stream);
    FYN_HIP(hipGetLastError());
    FYN_HIP(hipEventRecord(s.comp, stream));
    FYN_HIP(hipStreamWaitEvent(down_stream_, s.comp, 0));
    FYN_HIP(hipMemcpyAsync(s.pin_out, s.dev_out, async_out_floats_ * sizeof(float), hipMemcpyDeviceToHost, down_stream_));
    FYN_HIP(hipEventRecord(s.down, down_stream_));
    s.user_out = out;
    s.busy = true;
    s.ticket = ++async_seq_;
    if (ticket) *ticket = s.ticket;
}

void Net::async_wait(uint64_t ticket) {
    if (slots_.empty()) fail(FYN_ERR_STATE, "async_wait() without async_begin()");
    FYN_HIP(hipSetDevice(device));
    if (ticket == 0 || ticket > async_seq_) fail(FYN_ERR_INVALID, "unknown frame ticket %llu", (unsigned long long)ticket);
    // frames complete in submission order: deliver everything up to the requested one
    for (uint64_t t = (async_seq_ > slots_.size() ? async_seq_ - slots_.size() + 1 : 1); t <= ticket; t++) {
        AsyncSlot& s = slots_[(t - 1) % slots_.size()];
        if (s.busy && s.ticket == t) async_complete(s);
    }
}

void Net::async_end() {
    if (slots_.empty()) return;
    (void)hipSetDevice(device);
    for (uint64_t t = (async_seq_ > slots_.size() ? async_seq_ - slots_.size() + 1 : 1); t <= async_seq_; t++) {
        AsyncSlot& s = slots_[(t - 1) % slots_.size()];
        if (s.busy && s.ticket == t) async_complete(s);
    }
    if (stream) (void)hipStreamSynchronize(stream);
    for (AsyncSlot& s : slots_) {
        if (s.pin_in) (void)hipHostFree(s.pin_in);
        if (s.pin_out) (void)hipHostFree(s.pin_out);
        if (s.dev_in) (void)hipFree(s.dev_in);
        if (s.dev_out) (void)hipFree(s.dev_out);
        if (s.up) (void)hipEventDestroy(s.up);
        if (s.comp) (void)hipEventDestroy(s.comp);
        if (s.down) (void)hipEventDestroy(s.down);
    }
    slots_.clear();
    if (async_own_streams_) {
        if (up_stream_) (void)hipStreamSynchronize(up_stream_);
        if (down_stream_) (void)hipStreamSynchronize(down_stream_);
        return_stream(device, up_stream_);
        return_stream(device, down_stream_);
    }
    up_stream_ = down_stream_ = nullptr;
    async_seq_ = 0;
}

}  // namespace fynhip
