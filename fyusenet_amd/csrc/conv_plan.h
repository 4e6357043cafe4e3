// Planning, tuning and weight packing of the matrix-core convolution kernels, shared by the convolution and the
// transposed-convolution layers (layer_classes.h, layers.cpp), and the small host helpers of the layer code.
#pragma once
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "engine.h"

namespace fynhip {

inline uint16_t f2h_bits(float f) {
    _Float16 h = (_Float16)f;  // round to nearest even
    uint16_t b;
    memcpy(&b, &h, 2);
    return b;
}

inline float h2f(uint16_t b) {
    _Float16 h;
    memcpy(&h, &b, 2);
    return (float)h;
}

inline int pow2ceil(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

inline int ilog2(int x) {
    int l = 0;
    while ((1 << l) < x) l++;
    return l;
}

template <typename T>
T* upload(Net* net, const std::vector<T>& host) {
    T* dev = static_cast<T*>(net->dev_alloc(host.size() * sizeof(T), false));
    FYN_HIP(hipMemcpyAsync(dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice, net->stream));
    FYN_HIP(hipStreamSynchronize(net->stream));
    return dev;
}

template <typename T>
void reupload(Net* net, T* dev, const std::vector<T>& host) {
    FYN_HIP(hipStreamSynchronize(net->stream));
    FYN_HIP(hipMemcpyAsync(dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice, net->stream));
    FYN_HIP(hipStreamSynchronize(net->stream));
}

// scale / bias' of the convolution family from a weight block:
//   bias' = bias*bnScale + bnBias, scale = bnScale (gpu/deep/deepconvlayerbase.cpp:360-382)
void fold_bn(const float* bias, const float* bn, int cout, bool post_bn, int padded, std::vector<float>& scale,
                    std::vector<float>& biasp);

// =============================================================================================
// MFMA convolution planning (shared by convolution and transposed convolution)
// =============================================================================================
struct Tap {
    int oy, ox;  // offset (input pixels) inside the staged tile of the sample used by position (0,0)
    int ky, kx;  // weight tap
};

struct SubConv {
    std::vector<Tap> taps;
    int span_y = 1, span_x = 1;  // staged tile = (tile-1)*in_stride + span
    int in_y0 = 0, in_x0 = 0, in_stride = 1;
    int npos_y = 0, npos_x = 0;
    int out_step = 1, out_off_y = 0, out_off_x = 0;
    int res_off_y = 0, res_off_x = 0;
    int clamp = 0;     // shallow sampling rule: repeat the frame's edge
    int in_shift = 0;  // fractional-step convolution: coordinates count in the frame repeated 2^in_shift times
    int fuse_k = 0, fuse_cout = 0;   // kx taps folded into the output channels and summed in the epilogue (ConvMfmaParams::fuse_k)
    int in_sub = 0;    // one-tap layer with stride in_sub > 1: the kernel works in the sub-sampled frame (in_stride is 1,
                       // in_y0/in_x0 are the stored coordinates of its pixel (0,0))
};

struct MfmaLaunch {
    ConvVariant var{};
    ConvMfmaParams p{};
    size_t lds = 0;
    // host-side description of the k16 steps of one chunk: 16 (ky,kx,ci_rel) triples, ci_rel < 0 = zero
    struct Step {
        int aoff;
        int off4[4] = {0, 0, 0, 0};   // chunks of 4 channels: one LDS offset per tap of the step
        int ky[16], kx[16], ci[16];
    };
    std::vector<Step> steps;
    void* wpack_dev = nullptr;
    int* aoff_dev = nullptr;
    size_t wpack_halves = 0;  // halves used by this launch's layout
    size_t wpack_alloc = 0;   // halves allocated
    SplitKReduceParams red{};  // second pass when p.ksplit > 1
    int cin = 0, cout = 0;
};

struct TileChoice {
    int fm, fn, wm, wn, twl, th;
    double score;
    int rowpad;  // bytes added to each staged pixel row in LDS
    int kc;      // input channels per staged chunk
};

// All tile configurations that fit (possibly none), best heuristic score first.
std::vector<TileChoice> enumerate_tiles(Net* net, int cout, const SubConv& sc, int pitch, int npl, int slack, int nbuf);

// kc_force > 0 selects the chunk width, 0 the default for the geometry.
void conv_geometry(Net* net, const TView& in, bool split, int ntaps, int kc_force, int& kc, int& pitch, int& slack, int& npl);

// Builds the launch description of one (sub-)convolution for one tile configuration.  The packed
// weight layout does not depend on the tile configuration (cout fragments are padded to a multiple
// of 4), so candidates can share one weight buffer (`share`); weights are packed separately.
MfmaLaunch plan_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
                            int cout, const Act& act, int res_relu, int res_scale, const TileChoice& tc,
                            const float* scale, const float* bias, const MfmaLaunch* share = nullptr, int force_pd = 0);

// Launches a planned (sub-)convolution: the MFMA kernel and, with split-K, the reduce pass.
int run_mfma(const MfmaLaunch& L, hipStream_t s);

// Turns a planned launch into its split-K form (ksplit slices over the input-channel chunks).
void set_ksplit(Net* net, MfmaLaunch& L, int ksplit);

template <typename F>
float time_calls(Net* net, F&& call, int iters) {
    hipEvent_t a, b;
    FYN_HIP(hipEventCreate(&a));
    FYN_HIP(hipEventCreate(&b));
    call();
    FYN_HIP(hipEventRecord(a, net->stream));
    for (int i = 0; i < iters; i++) call();
    FYN_HIP(hipEventRecord(b, net->stream));
    FYN_HIP(hipEventSynchronize(b));
    FYN_HIP(hipGetLastError());
    float ms = 0.f;
    FYN_HIP(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    return ms / iters;
}

float time_launch(Net* net, const MfmaLaunch& L, int iters);

// switches that pin part of the choice are for experiments: choices are neither remembered nor recalled then
bool tune_cache_bypassed(Net* net);

const TileChoice* tune_cache_lookup(Net* net, const char* key, const std::vector<TileChoice>& cands, int* ksplit);

void tune_cache_store(Net* net, const char* key, const ConvVariant& v, int ksplit, int twl);

// a measured yes/no choice under a key of its own (same file, the first number is the flag)
bool tune_cache_flag(Net* net, const char* key, bool* flag);

void tune_cache_store_flag(Net* net, const char* key, bool flag);

// three numbers under a key of their own (same file)
bool tune_cache_triple(Net* net, const char* key, int (&out)[3]);

void tune_cache_store_triple(Net* net, const char* key, int a, int b, int c);

// Picks the tile configuration of one (sub-)convolution: by measurement on the layer's own tensors (default), or by
// the heuristic score when FYNHIP_AUTOTUNE=0.  Candidates are timed before the weights are packed, i.e. on zero
// operands; the matrix pipes run about a tenth faster on those than on real data (the part holds a higher clock when
// fewer operand bits toggle), for all candidates alike, so the ranking carries over while the figures do not.
MfmaLaunch tune_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
                            int cout, const Act& act, int res_relu, int res_scale, const float* scale, const float* bias);

// Several sub-convolutions of one layer (the output parities of a transposed convolution) that run as one launch.
struct MfmaGroup {
    std::vector<MfmaLaunch> subs;
    ConvMfmaMulti multi{};
    size_t lds = 0;
    ConvVariant var{};
    void sync() {
        multi.nsub = (int)subs.size();
        lds = 0;
        for (size_t i = 0; i < subs.size(); i++) {
            multi.sub[i] = subs[i].p;
            lds = std::max(lds, subs[i].lds);
        }
        if (!subs.empty()) var = subs[0].var;
    }
};

int run_group(const MfmaGroup& g, hipStream_t s);

float time_group(Net* net, const MfmaGroup& g, int iters);

// Picks ONE tile configuration and chunk width for a group of sub-convolutions (same tensors, different taps
// and output offsets) by timing the merged launch; the step group size is fixed so that all members fit it.
MfmaGroup tune_mfma_group(Net* net, const std::vector<SubConv>& scs, const TView& in, const TView& out, int cin, int cout,
                                 const Act& act, const float* scale, const float* bias);

// Packs weights W[o][ky][kx][i] (block order, base/convlayerinterface.h:71-95) into the per-lane A
// fragment order of the kernel: [(chunk, step)][mfrag][plane][lane][8 halves]; for tiles whose waves split the
// steps of a chunk into WK groups, [group][chunk][step of the group]... (a wave walks its steps over all chunks
// with one stride).
void pack_mfma_weights(Net* net, MfmaLaunch& L, const float* w, int k, float wmul, int kw = -1);

// power of two that brings the largest weight magnitude to [2^11, 2^12): keeps hi and lo parts of the
// fp16 split in the normal range; undone exactly by acc_mul in the epilogue
float weight_prescale(const float* w, size_t n);

// The planes behind the first of a packed fragment of the 16-position forms on fp32 tensors (three planes of 64 lanes x 8
// halves): plane 1 takes the fp16 lo part of weight j of a lane; c8 takes the sources of plane 2, the fp8 operands of
// the correction terms: hi / 32 in its first eight places, lo * 64 in the other eight (the staged activations carry the
// inverse factors, conv_p16.hip).
void p16_lo_planes(uint16_t* frag_base, float* c8_lane, int lane, int j, float v, uint16_t hi);

void upload_p16_pack(Net* net, void* dev, const std::vector<uint16_t>& pack, const std::vector<float>& c8, size_t frags);

std::string mfma_info(const MfmaLaunch& L);

}  // namespace fynhip
