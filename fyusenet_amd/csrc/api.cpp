// extern "C" surface declared in include/fynhip.h: translates C++ errors into status codes and a
// thread-local message (the text a FynException would have carried, common/fynexception.h).
#include <cstring>
#include <string>

#include "engine.h"

struct fyn_net {
    fynhip::Net* impl;
};

static thread_local std::string g_last_error;

#define FYN_API_BEGIN try {
#define FYN_API_END                                     \
    }                                                   \
    catch (const fynhip::Error& e) {                    \
        g_last_error = e.what();                        \
        return e.code;                                  \
    }                                                   \
    catch (const std::bad_alloc&) {                     \
        g_last_error = "out of host memory";            \
        return FYN_ERR_DEVICE;                          \
    }                                                   \
    catch (const std::exception& e) {                   \
        g_last_error = e.what();                        \
        return FYN_ERR_INVALID;                         \
    }                                                   \
    return FYN_OK;

static fynhip::Net* N(fyn_net* n) {
    if (!n || !n->impl) fynhip::fail(FYN_ERR_INVALID, "null network handle");
    return n->impl;
}

extern "C" {

const char* fyn_last_error(void) { return g_last_error.c_str(); }

int fyn_device_info(int device, char* buf, size_t buflen) {
    FYN_API_BEGIN
    if (!buf || buflen == 0) fynhip::fail(FYN_ERR_INVALID, "null buffer");
    hipDeviceProp_t prop;
    FYN_HIP(hipGetDeviceProperties(&prop, device));
    snprintf(buf, buflen, "%s arch=%s CUs=%d clock=%dMHz mem=%.1fGiB lds/block=%zu", prop.name, prop.gcnArchName,
             prop.multiProcessorCount, prop.clockRate / 1000, (double)prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0),
             (size_t)prop.sharedMemPerBlock);
    FYN_API_END
}

int fyn_net_create(int device, int storage, fyn_net** out) {
    FYN_API_BEGIN
    if (!out) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    fynhip::Net* impl = new fynhip::Net(device, storage);
    *out = new fyn_net{impl};
    FYN_API_END
}

int fyn_net_destroy(fyn_net* net) {
    FYN_API_BEGIN
    if (net) {
        delete net->impl;
        delete net;
    }
    FYN_API_END
}

int fyn_net_add_layer(fyn_net* net, const fyn_layer_desc* desc) {
    FYN_API_BEGIN
    if (!desc) fynhip::fail(FYN_ERR_INVALID, "No builder supplied to layer factory line");
    if (desc->struct_size != sizeof(fyn_layer_desc))
        fynhip::fail(FYN_ERR_INVALID, "fyn_layer_desc size mismatch (%u, library expects %zu)", desc->struct_size, sizeof(fyn_layer_desc));
    fyn_layer_desc d = *desc;
    d.name[FYN_NAME_LEN - 1] = 0;
    N(net)->add_layer(d);
    FYN_API_END
}

int fyn_net_add_custom_layer(fyn_net* net, const fyn_layer_desc* desc, const fyn_custom_layer* impl) {
    FYN_API_BEGIN
    if (!desc || !impl) fynhip::fail(FYN_ERR_INVALID, "No builder supplied to layer factory line");
    if (desc->struct_size != sizeof(fyn_layer_desc))
        fynhip::fail(FYN_ERR_INVALID, "fyn_layer_desc size mismatch (%u, library expects %zu)", desc->struct_size, sizeof(fyn_layer_desc));
    fyn_layer_desc d = *desc;
    d.name[FYN_NAME_LEN - 1] = 0;
    N(net)->add_custom_layer(d, *impl);
    FYN_API_END
}

int fyn_net_connect(fyn_net* net, int out_layer, int in_layer, int port) {
    FYN_API_BEGIN
    N(net)->connect(out_layer, in_layer, port);
    FYN_API_END
}

int fyn_layer_load_weights(fyn_net* net, int layer, const float* wb, size_t offset_floats) {
    FYN_API_BEGIN
    if (!wb) fynhip::fail(FYN_ERR_INVALID, "null weight pointer");
    fynhip::Layer* l = N(net)->layer(layer);
    if (l->d.type == FYN_LAYER_BATCHNORM) fynhip::fail(FYN_ERR_INVALID, "layer %s takes scale/bias, not weights", l->d.name);
    l->load_weights(wb + offset_floats);
    N(net)->weights_changed();
    FYN_API_END
}

int fyn_layer_load_scale_bias(fyn_net* net, int layer, const float* sb, size_t offset_floats) {
    FYN_API_BEGIN
    if (!sb) fynhip::fail(FYN_ERR_INVALID, "null scale/bias pointer");
    fynhip::Layer* l = N(net)->layer(layer);
    if (l->d.type != FYN_LAYER_BATCHNORM) fynhip::fail(FYN_ERR_INVALID, "layer %s is not a batchnorm layer", l->d.name);
    l->load_weights(sb + offset_floats);
    N(net)->weights_changed();
    FYN_API_END
}

int fyn_layer_weight_floats(fyn_net* net, int layer, size_t* count) {
    FYN_API_BEGIN
    if (!count) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    *count = N(net)->layer(layer)->weight_floats();
    FYN_API_END
}

int fyn_net_setup(fyn_net* net) {
    FYN_API_BEGIN
    N(net)->setup();
    FYN_API_END
}

int fyn_net_set_input(fyn_net* net, int layer, int port, const float* data, int order) {
    FYN_API_BEGIN
    N(net)->set_input(layer, port, data, order);
    FYN_API_END
}

int fyn_net_input_floats(fyn_net* net, int layer, int port, size_t* count) {
    FYN_API_BEGIN
    if (!count) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    *count = N(net)->input_floats(layer, port);
    FYN_API_END
}

int fyn_net_forward(fyn_net* net, uint64_t* seq_out) {
    FYN_API_BEGIN
    N(net)->forward(seq_out);
    FYN_API_END
}

int fyn_net_finish(fyn_net* net) {
    FYN_API_BEGIN
    N(net)->finish();
    FYN_API_END
}

int fyn_layer_copy_result(fyn_net* net, int layer, float* chw, int include_padding) {
    FYN_API_BEGIN
    if (!chw) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    N(net)->copy_result(layer, chw, include_padding);
    FYN_API_END
}

int fyn_layer_copy_result_noalloc(fyn_net* net, int layer, float* chw, int include_padding) {
    FYN_API_BEGIN
    if (!chw) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    N(net)->copy_result_static(layer, chw, include_padding);
    FYN_API_END
}

int fyn_layer_output_shape(fyn_net* net, int layer, int* channels, int* height, int* width, int* padding) {
    FYN_API_BEGIN
    fynhip::Layer* l = N(net)->layer(layer);
    if (channels) *channels = l->oc;
    if (height) *height = l->oh;
    if (width) *width = l->ow;
    // a pass-through (download) layer hands on its input tensor, halo included
    if (padding) *padding = (N(net)->is_setup && l->out >= 0) ? l->tout().v.pad : l->d.output_padding;
    FYN_API_END
}

int fyn_net_get_output(fyn_net* net, int layer, float* data, int order) {
    FYN_API_BEGIN
    if (!data) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    N(net)->get_output(layer, data, order);
    FYN_API_END
}

int fyn_layer_copy_argmax(fyn_net* net, int layer, int32_t* idx, float* val) {
    FYN_API_BEGIN
    N(net)->copy_argmax(layer, idx, val);
    FYN_API_END
}

int fyn_net_enable_timings(fyn_net* net, int enable) {
    FYN_API_BEGIN
    fynhip::Net* n = N(net);
    n->finish();
    n->timings = enable != 0;
    if (!enable) return FYN_OK;
    for (auto& kv : n->layers) {
        kv.second->ms_total = 0.f;
        kv.second->runs = 0;
    }
    FYN_API_END
}

int fyn_net_get_timing(fyn_net* net, int layer, float* ms_total, int* runs) {
    FYN_API_BEGIN
    fynhip::Net* n = N(net);
    n->finish();
    fynhip::Layer* l = n->layer(layer);
    if (ms_total) *ms_total = l->ms_total;
    if (runs) *runs = l->runs;
    FYN_API_END
}

int fyn_net_enable_intermediate_output(fyn_net* net, const char* dir) {
    FYN_API_BEGIN
    N(net)->dump_dir = dir ? dir : "";
    FYN_API_END
}

int fyn_net_set_buffer_reuse(fyn_net* net, int enable) {
    FYN_API_BEGIN
    fynhip::Net* n = N(net);
    if (n->is_setup) fynhip::fail(FYN_ERR_STATE, "buffer reuse must be chosen before setup");
    n->reuse_buffers = enable != 0;
    FYN_API_END
}

int fyn_net_use_graph(fyn_net* net, int enable) {
    FYN_API_BEGIN
    N(net)->use_graph(enable != 0);
    FYN_API_END
}

int fyn_net_time_forward(fyn_net* net, int iters, float* ms_total) {
    FYN_API_BEGIN
    if (!ms_total || iters < 1) fynhip::fail(FYN_ERR_INVALID, "invalid arguments");
    N(net)->time_forward(iters, ms_total);
    FYN_API_END
}

int fyn_net_time_steps(fyn_net* net, int iters, float* ms_each) {
    FYN_API_BEGIN
    if (!ms_each || iters < 1) fynhip::fail(FYN_ERR_INVALID, "need an output array and at least one step");
    N(net)->time_steps(iters, ms_each);
    FYN_API_END
}

int fyn_layer_time(fyn_net* net, int layer, int iters, float* ms_total) {
    FYN_API_BEGIN
    if (!ms_total || iters < 1) fynhip::fail(FYN_ERR_INVALID, "invalid arguments");
    N(net)->time_layer(layer, iters, ms_total);
    FYN_API_END
}

int fyn_net_async_begin(fyn_net* net, int in_layer, int in_port, int in_order, int out_layer, int out_order, int depth, int copy_streams) {
    FYN_API_BEGIN
    N(net)->async_begin(in_layer, in_port, in_order, out_layer, out_order, depth, copy_streams != 0);
    FYN_API_END
}

int fyn_net_async_submit(fyn_net* net, const float* in, float* out, uint64_t* ticket) {
    FYN_API_BEGIN
    N(net)->async_submit(in, out, ticket);
    FYN_API_END
}

int fyn_net_async_sizes(fyn_net* net, size_t* in_floats, size_t* out_floats) {
    FYN_API_BEGIN
    if (!in_floats || !out_floats) fynhip::fail(FYN_ERR_INVALID, "null output pointer");
    N(net)->async_sizes(in_floats, out_floats);
    FYN_API_END
}

int fyn_net_async_wait(fyn_net* net, uint64_t ticket) {
    FYN_API_BEGIN
    N(net)->async_wait(ticket);
    FYN_API_END
}

int fyn_net_async_end(fyn_net* net) {
    FYN_API_BEGIN
    N(net)->async_end();
    FYN_API_END
}

int fyn_net_device_allocations(fyn_net* net, size_t* calls, size_t* bytes) {
    FYN_API_BEGIN
    if (calls) *calls = N(net)->alloc_calls_;
    if (bytes) *bytes = N(net)->alloc_bytes_;
    FYN_API_END
}

int fyn_layer_kernel_info(fyn_net* net, int layer, char* buf, size_t buflen) {
    FYN_API_BEGIN
    if (!buf || buflen == 0) fynhip::fail(FYN_ERR_INVALID, "null buffer");
    std::string s = N(net)->layer(layer)->info();
    snprintf(buf, buflen, "%s", s.c_str());
    FYN_API_END
}

}  // extern "C"
