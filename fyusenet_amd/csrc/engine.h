// Host-side engine: network graph, device tensors, layer objects.  This is the part of the
// reference's base/ + gpu/ host code that survives the move from OpenGL to HIP:
//   LayerFactory / GPULayerFactoryBackend   -> Net::add_layer          (base/layerfactory.cpp, gpu/gpulayerfactory.cpp)
//   BufferManager                           -> Net::connect / assign_buffers (base/buffermanager.cpp)
//   NeuralNetwork / Engine (sync branch)    -> Net::setup / forward / finish (base/neuralnetwork.cpp, base/engine.cpp)
//   GPULayerBase subclasses                 -> Layer subclasses in layer_classes.h and layers.cpp
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/fynhip.h"
#include "kernels.h"

namespace fynhip {

// Error carried up to the C ABI (the reference throws FynException, common/fynexception.h).
struct Error : public std::runtime_error {
    int code;
    Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};
[[noreturn]] void fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define FYN_HIP(call)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess) ::fynhip::fail(FYN_ERR_DEVICE, "%s failed: %s (%s:%d)", #call,       \
                                             hipGetErrorString(e_), __FILE__, __LINE__);           \
    } while (0)

struct Tensor {
    TView v{};
    int producer = -1;     // layer number writing it (-1: external input)
    int last_reader = -1;  // highest layer number reading it
    bool locked = false;   // never reused (network outputs, external inputs)
    int buffer = -1;       // index into Net::buffers_
    unsigned* amax = nullptr;   // value-range word (range.h) when a producer keeps it, else null
};

struct DevBuffer {
    void* ptr = nullptr;
    size_t bytes = 0;
    int h = 0, w = 0, pad = 0, cp = 0, f16 = 0;  // geometry key (reuse only between identical geometries)
    int free_after = -1;                          // highest reader of the current tenant
    bool locked = false;
};

class Net;

// The FYNHIP_* environment switches (tests, experiments, tuning cache), read once when a network is created: nothing on
// a launch path, and nothing during a later setup or weight load, looks at the environment again.
class Switches {
  public:
    void read();                               // every variable of the environment whose name begins with FYNHIP_
    const char* get(const char* name) const;   // the value, or nullptr when the variable was not set (like getenv)
    bool on(const char* name) const { return get(name) != nullptr; }
  private:
    std::map<std::string, std::string> v_;
};

class Layer {
  public:
    Layer(Net* net, const fyn_layer_desc& d);
    virtual ~Layer() {}
    fyn_layer_desc d;
    Net* net;
    std::vector<int> in;  // tensor id per input port, -1 = not connected
    int out = -1;         // tensor id
    int oc = 0, oh = 0, ow = 0;  // output net shape

    virtual int num_ports() const { return (d.flags & FYN_FLAG_RESIDUAL_INPUT) ? 2 : 1; }
    // shape of the tensor expected on an input port (channels, h, w, padding)
    virtual void port_shape(int port, int& c, int& h, int& w, int& pad) const;
    virtual bool has_own_output() const { return true; }
    virtual size_t weight_floats() const { return 0; }
    virtual void load_weights(const float*) { fail(FYN_ERR_INVALID, "layer %s (%d) takes no weights", d.name, d.number); }
    virtual void setup() {}
    virtual void forward(hipStream_t s) = 0;
    virtual std::string info() const { return "none"; }
    // value ranges (range.h): whether this layer's kernels raise the word of their output tensor, and whether they can
    // take on clearing another tensor's word (true: taken)
    virtual bool tracks_range() const { return false; }
    virtual bool add_range_reset(unsigned*) { return false; }
    virtual void setup_ranges() {}   // (re)reads the words of the layer's tensors into its kernel arguments
    Act act() const;
    const Tensor& tin(int port) const;
    const Tensor& tout() const;
    bool set_up = false;
    // timing
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    float ms_total = 0.f;
    int runs = 0;
};

class Net {
  public:
    Net(int device, int storage);
    Switches sw;
    ~Net();
    void add_layer(const fyn_layer_desc& d);
    void add_custom_layer(const fyn_layer_desc& d, const fyn_custom_layer& impl);
    void connect(int out_layer, int in_layer, int port);
    void setup();
    void forward(uint64_t* seq);
    void finish();
    Layer* layer(int number);
    void set_input(int layer, int port, const float* data, int order);
    const Tensor& input_tensor(int layer, int port);     // what set_input writes: an upload layer's output or an unconnected port
    size_t input_floats(int layer, int port);            // floats that set_input reads from the host buffer
    void async_sizes(size_t* in_floats, size_t* out_floats) const;   // per frame, of the active frame pipeline
    void copy_result(int layer, float* chw, int include_padding);
    void copy_result_static(int layer, float* chw, int include_padding);   // through the fixed staging area, no allocation
    void get_output(int layer, float* data, int order);
    void copy_argmax(int layer, int32_t* idx, float* val);
    void time_forward(int iters, float* ms);
    void time_steps(int iters, float* ms_each);
    // A captured forward pass holds kernel arguments by value (among them the power of two that undoes a layer's weight
    // pre-scaling): after a weight load on a set-up network the next forward() captures again.
    void weights_changed();
    void time_layer(int layer, int iters, float* ms);
    void use_graph(bool enable);
    // frame pipeline: upload of frame i+1 and download of frame i-1 overlap the layers of frame i
    void async_begin(int in_layer, int in_port, int in_order, int out_layer, int out_order, int depth, bool copy_streams);
    void async_submit(const float* in, float* out, uint64_t* ticket);
    void async_wait(uint64_t ticket);
    void async_end();

    int device;
    int storage;  // fyn_storage
    bool f16() const { return storage == FYN_STORAGE_F16; }
    bool is_setup = false;
    bool timings = false;
    bool reuse_buffers = true;
    // Layers fused into their neighbour's launch (fuse_depthwise_layers) run that way only in passes that neither time
    // nor dump single layers, and only in networks whose intermediate tensors may share buffers.
    bool fusion_on() const { return reuse_buffers && !timings && dump_dir.empty(); }
    std::string dump_dir;
    hipStream_t stream = nullptr;
    std::map<int, std::unique_ptr<Layer>> layers;  // ascending number = execution order
    std::vector<Tensor> tensors;
    std::vector<DevBuffer> buffers;
    uint64_t seq = 0;

    // device allocations owned by the net
    void* dev_alloc(size_t bytes, bool zero = true);
    void dev_free(void* p);   // setup-time only (waits for the stream)
    void dev_free_many(const std::vector<void*>& ptrs);   // the same for several areas, one wait
    float* staging(size_t floats);  // fp32 staging area for layout conversion

  private:
    struct AsyncSlot {
        float *pin_in = nullptr, *pin_out = nullptr, *dev_in = nullptr, *dev_out = nullptr;
        hipEvent_t up = nullptr, comp = nullptr, down = nullptr;
        float* user_out = nullptr;
        uint64_t ticket = 0;
        bool busy = false;
    };
    std::vector<AsyncSlot> slots_;
    hipStream_t up_stream_ = nullptr, down_stream_ = nullptr;
    const Tensor* async_in_ = nullptr;
    const Tensor* async_out_ = nullptr;
    bool async_own_streams_ = true;
    TView async_out_view_{};   // what the output layer hands out (a download layer may name other channel counts)
    int async_in_order_ = 0, async_out_order_ = 0;
    size_t async_in_floats_ = 0, async_out_floats_ = 0;
    uint64_t async_seq_ = 0;
    void async_complete(AsyncSlot& s);
    void run_layers(bool with_events);
    void collect_timings();
    void dump_layer(Layer* l);
    std::vector<void*> allocs_;
  public:
    // device allocations made for this network since it was created (calls of hipMalloc, bytes asked for)
    size_t alloc_calls_ = 0, alloc_bytes_ = 0;
  private:
    float* staging_ = nullptr;
    size_t staging_floats_ = 0;
    float* static_scratch_ = nullptr;   // this device's address of the fixed staging area
    unsigned* amax_dev_ = nullptr;      // one value-range word per tensor
    void assign_range_words();
    void assign_range_resets();
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t graph_exec_ = nullptr;
    bool graph_enabled_ = false;
    bool events_pending_ = false;
    bool poison_lds_ = false;           // FYNHIP_POISON_LDS: fill the LDS with NaN patterns in front of every layer
};

Layer* create_layer(Net* net, const fyn_layer_desc& d);
void fuse_batchnorm_layers(Net* net);   // after every layer's setup(): batch-norm layers that their readers (K-resident convolutions) can apply while staging
void keep_projection_inputs(Net* net);    // before buffers are assigned: inputs of such projections live until the layer that may compute them has run
void fuse_projection_layers(Net* net);   // after every layer's setup(): 1x1 shortcut projections that the 1x1 layer adding them can compute in its own launch
void fuse_depthwise_layers(Net* net);   // after every layer's setup(): depthwise 3x3 layers that their 1x1 reader can compute itself
Layer* create_custom_layer(Net* net, const fyn_layer_desc& d, const fyn_custom_layer& impl);

}  // namespace fynhip
