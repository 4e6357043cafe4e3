// Layer objects: validation of the builder description (the rules of
// GPULayerFactoryBackend::createLayer, fyusenet/gpu/gpulayerfactory.cpp:112-184,358-430,490-571),
// weight-block parsing / repacking (gpu/deep/deepconvlayerbase.cpp:293-395 and friends) and kernel
// selection + launch.
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "engine.h"

namespace fynhip {

static inline uint16_t f2h_bits(float f) {
    _Float16 h = (_Float16)f;  // round to nearest even
    uint16_t b;
    memcpy(&b, &h, 2);
    return b;
}
static inline float h2f(uint16_t b) {
    _Float16 h;
    memcpy(&h, &b, 2);
    return (float)h;
}

static int pow2ceil(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}
static int ilog2(int x) {
    int l = 0;
    while ((1 << l) < x) l++;
    return l;
}

template <typename T>
static T* upload(Net* net, const std::vector<T>& host) {
    T* dev = static_cast<T*>(net->dev_alloc(host.size() * sizeof(T), false));
    FYN_HIP(hipMemcpyAsync(dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice, net->stream));
    FYN_HIP(hipStreamSynchronize(net->stream));
    return dev;
}
template <typename T>
static void reupload(Net* net, T* dev, const std::vector<T>& host) {
    FYN_HIP(hipStreamSynchronize(net->stream));
    FYN_HIP(hipMemcpyAsync(dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice, net->stream));
    FYN_HIP(hipStreamSynchronize(net->stream));
}

// scale / bias' of the convolution family from a weight block:
//   bias' = bias*bnScale + bnBias, scale = bnScale (gpu/deep/deepconvlayerbase.cpp:360-382)
static void fold_bn(const float* bias, const float* bn, int cout, bool post_bn, int padded, std::vector<float>& scale,
                    std::vector<float>& biasp) {
    scale.assign(padded, 0.f);
    biasp.assign(padded, 0.f);
    for (int o = 0; o < cout; o++) {
        if (post_bn) {
            scale[o] = bn[o];
            biasp[o] = bias[o] * bn[o] + bn[cout + o];
        } else {
            scale[o] = 1.f;
            biasp[o] = bias[o];
        }
    }
}

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
static std::vector<TileChoice> enumerate_tiles(Net* net, int cout, const SubConv& sc, int pitch, int npl, int slack, int nbuf) {
    std::vector<TileChoice> all;
    const char* force = net->sw.get("FYNHIP_CONV_TILE");  // "fm,fn,wm,wn" for experiments
    int ff[4] = {0, 0, 0, 0};
    if (force) sscanf(force, "%d,%d,%d,%d", &ff[0], &ff[1], &ff[2], &ff[3]);
    for (int ti = 0; ti < conv_mfma_tile_count(); ti++) {
        int fm, fn, wm, wn;
        conv_mfma_tile(ti, &fm, &fn, &wm, &wn);
        if (force && (fm != ff[0] || fn != ff[1] || wm != ff[2] || wn != ff[3])) continue;
        const int bm = wn * fn * 32;
        if (sc.fuse_k) {
            // folded kx taps: one row of 32 virtual channels, four waves along the positions; tiles overlap by K-1
            // columns, so they are made wide (32 and 64 columns where the image has them)
            if (fm != 1 || wm != 1 || wn != 4 || cout > 32) continue;
            for (int tw = 16; tw <= 64; tw *= 2) {
                if (tw < 2 * sc.fuse_k || tw > bm || (tw > 16 && tw / 2 >= sc.npos_x)) continue;
                const int th = bm / tw, step = tw - sc.fuse_k + 1;
                const int tiles = ((sc.npos_x - (sc.fuse_k - 1) + step - 1) / step) * ((sc.npos_y + th - 1) / th);
                const int halo_w = (tw - 1) * sc.in_stride + sc.span_x, halo_h = (th - 1) * sc.in_stride + sc.span_y;
                const size_t lds = 1024 + (size_t)nbuf * npl * ((size_t)halo_h * (halo_w * pitch) + slack);
                if (lds > 150 * 1024) continue;
                const double util = ((double)sc.npos_x * sc.npos_y) / ((double)tiles * bm);
                all.push_back(TileChoice{fm, fn, wm, wn, ilog2(tw), th, util, 0, 0});
            }
            continue;
        }
        // (at least 8 columns: the epilogue writes 8 / FM consecutive positions of one tile row per instruction)
        int tw = std::max(8, std::min(bm >= 128 ? 16 : 8, pow2ceil(sc.npos_x)));
        while (bm / tw > pow2ceil(sc.npos_y) && tw < pow2ceil(sc.npos_x) && tw < bm) tw *= 2;
        const int th = bm / tw;
        const int tiles = ((sc.npos_x + tw - 1) / tw) * ((sc.npos_y + th - 1) / th);
        const int cpb = wm * fm * 32;
        const int cblocks = (cout + cpb - 1) / cpb;
        const int halo_w = (tw - 1) * sc.in_stride + sc.span_x, halo_h = (th - 1) * sc.in_stride + sc.span_y;
        const char* rp = net->sw.get("FYNHIP_ROWPAD");
        const int rowpad = rp ? atoi(rp) : 0;
        const size_t lds = 1024 + (size_t)nbuf * npl * ((size_t)halo_h * (halo_w * pitch + rowpad) + slack);
        if (lds > 150 * 1024) continue;
        const double util = ((double)cout * sc.npos_x * sc.npos_y) / ((double)cblocks * cpb * (double)tiles * bm);
        const double blocks = (double)tiles * cblocks;
        const double slots = 256.0 * (lds > 72 * 1024 ? 1 : 2);
        const double par = blocks >= slots ? blocks / (std::ceil(blocks / slots) * slots) : blocks / slots;
        const double bonus = (fm * fn == 4) ? 1.0 : (fm * fn == 2 ? 0.85 : 0.7);
        all.push_back(TileChoice{fm, fn, wm, wn, ilog2(tw), th, util * par * bonus, rowpad, 0});
    }
    std::sort(all.begin(), all.end(), [](const TileChoice& x, const TileChoice& y) { return x.score > y.score; });
    return all;
}

// kc_force > 0 selects the chunk width, 0 the default for the geometry.
static void conv_geometry(Net* net, const TView& in, bool split, int ntaps, int kc_force, int& kc, int& pitch, int& slack, int& npl) {
    // input channels staged per chunk: kernels with few taps take wide chunks (fewer barriers per output)
    const char* kmax = net->sw.get("FYNHIP_CONV_KC_MAX");
    const int cap = kmax ? atoi(kmax) : 128;
    if (in.cp == 4) kc = 4;
    else if (in.cp <= 16) kc = 16;
    else if (ntaps <= 2 && in.cp >= 128 && cap >= 128) kc = 128;
    else if (ntaps <= 4 && in.cp >= 64 && cap >= 64) kc = 64;
    else kc = 32;
    if (kc_force > 0) kc = kc_force;
    pitch = (kc == 4) ? 8 : kc * 2 + 16;
    slack = 0;
    npl = split ? 2 : 1;
}

// Builds the launch description of one (sub-)convolution for one tile configuration.  The packed
// weight layout does not depend on the tile configuration (cout fragments are padded to a multiple
// of 4), so candidates can share one weight buffer (`share`); weights are packed separately.
static MfmaLaunch plan_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
                            int cout, const Act& act, int res_relu, int res_scale, const TileChoice& tc,
                            const float* scale, const float* bias, const MfmaLaunch* share = nullptr, int force_pd = 0) {
    MfmaLaunch L;
    L.cin = cin;
    L.cout = cout;
    const bool split = !net->f16();
    int kc, pitch, slack, npl;
    conv_geometry(net, in, split, (int)sc.taps.size(), tc.kc, kc, pitch, slack, npl);
    const int tw = 1 << tc.twl;
    ConvMfmaParams& p = L.p;
    p.in = in.ptr;
    p.out = out.ptr;
    p.res = res ? res->ptr : nullptr;
    p.in_hp = in.hp(); p.in_wp = in.wp(); p.in_cp = in.cp;
    p.in_y0 = sc.in_y0; p.in_x0 = sc.in_x0; p.in_stride = sc.in_stride;
    if (sc.in_sub > 1) {
        p.in_sub = sc.in_sub; p.in_oy = sc.in_y0; p.in_ox = sc.in_x0;
        p.in_y0 = p.in_x0 = 0;
    }
    p.in_clamp = sc.clamp; p.in_shift = sc.in_shift;
    p.npos_y = sc.npos_y; p.npos_x = sc.npos_x;
    p.out_wp = out.wp(); p.out_cp = out.cp; p.out_step = sc.out_step;
    p.out_off_y = sc.out_off_y; p.out_off_x = sc.out_off_x;
    if (res) {
        p.res_wp = res->wp(); p.res_cp = res->cp;
        p.res_off_y = sc.res_off_y; p.res_off_x = sc.res_off_x;
    }
    p.res_relu = res_relu; p.res_scale = res_scale;
    p.tile_w_log2 = tc.twl; p.tile_h = tc.th;
    p.tiles_x = (sc.npos_x + tw - 1) / tw;
    if (sc.fuse_k) {
        p.fuse_k = sc.fuse_k; p.fuse_cout = sc.fuse_cout;
        const int step = tw - sc.fuse_k + 1;
        p.tiles_x = (sc.npos_x - (sc.fuse_k - 1) + step - 1) / step;
    }
    p.tiles_y = (sc.npos_y + tc.th - 1) / tc.th;
    p.halo_w = (tw - 1) * sc.in_stride + sc.span_x;
    p.halo_h = (tc.th - 1) * sc.in_stride + sc.span_y;
    p.pitch = pitch;
    p.row_pitch = p.halo_w * pitch + ((kc == 4) ? 0 : tc.rowpad);
    p.plane = p.halo_h * p.row_pitch + slack;
    p.cin_chunks = (kc == 4) ? 1 : (in.cp + kc - 1) / kc;
    const int cpb = tc.wm * tc.fm * 32;
    p.cout_blocks = (cout + cpb - 1) / cpb;
    p.mfrags = ((cout + 31) / 32 + 3) / 4 * 4;
    p.scale = scale;
    p.bias = bias;
    p.acc_mul = 1.f;
    p.act = act;
    p.ksplit = 1;
    p.partial = nullptr;
    p.cout_pad = out.cp;
    L.lds = 1024 + (size_t)npl * p.plane * (p.cin_chunks > 1 ? 2 : 1);  // step table + tiles (double-buffered across chunks)
    L.lds = std::max(L.lds, (size_t)4 * tc.fn * 32 * (tc.fm * 32 + 4) * 4);  // epilogue transposition area (all waves, all fragments)
    if (in.elems() >= (size_t)1 << 31) fail(FYN_ERR_UNSUPPORTED, "input tensor too large for 32-bit element offsets");
    L.var = ConvVariant{in.f16, out.f16, split ? 1 : 0, tc.fm, tc.fn, tc.wm, tc.wn, kc, 2, 2};

    // k16 steps
    if (kc == 4) {
        // small-Cin layout: a pixel is 4 channels (8 bytes); a k16 step holds four taps wherever they are, each
        // with its own LDS offset (table entry = 4 offsets per step), so K is padded only at the very end
        std::vector<Tap> taps = sc.taps;
        std::sort(taps.begin(), taps.end(), [](const Tap& a, const Tap& b) { return a.oy != b.oy ? a.oy < b.oy : a.ox < b.ox; });
        for (size_t i = 0; i < taps.size(); i += 4) {
            MfmaLaunch::Step st;
            st.aoff = 0;
            for (int q = 0; q < 4; q++) {
                const bool have = i + q < taps.size();
                const Tap& t = taps[have ? i + q : i];      // an absent tap reads the step's first tap with zero weights
                st.off4[q] = t.oy * p.row_pitch + t.ox * pitch;
                for (int e = 0; e < 4; e++) {
                    st.ky[4 * q + e] = t.ky; st.kx[4 * q + e] = t.kx; st.ci[4 * q + e] = have ? e : -1;
                }
            }
            L.steps.push_back(st);
        }
    } else {
        for (const Tap& t : sc.taps)
            for (int sub = 0; sub < kc / 16; sub++) {
                MfmaLaunch::Step st;
                st.aoff = t.oy * p.row_pitch + t.ox * pitch + sub * 32;
                for (int e = 0; e < 16; e++) {
                    st.ky[e] = t.ky; st.kx[e] = t.kx; st.ci[e] = sub * 16 + e;
                }
                L.steps.push_back(st);
            }
    }
    // step group size = depth of the kernel's weight prefetch ring: the largest compiled one that divides
    // the step count (32-channel chunks: 6, 4, 2; otherwise 2); an odd count is padded with a zero-weight step
    {
        const int raw = (int)L.steps.size();
        int pd = 2;
        if (kc == 32) pd = (raw % 6 == 0) ? 6 : ((raw % 4 == 0) ? 4 : 2);
        if (kc >= 64) pd = 4;
        if (const char* e = net->sw.get("FYNHIP_CONV_PD")) pd = atoi(e);
        if (force_pd > 0 && kc <= 32) pd = force_pd;
        const bool ksplit_tile = tc.wm * tc.wn < 4;      // waves split the steps of a chunk: smallest step group
        if (ksplit_tile) pd = kc > 128 ? 4 : 2;
        L.var.pd = pd;
        L.var.unr = (pd == 6 && raw % 18 == 0 && force_pd == 0 && !net->sw.get("FYNHIP_CONV_NO_FULL_UNROLL")) ? 18 : pd;
        if (kc == 128 && !ksplit_tile) L.var.unr = 8;
        if (!conv_mfma_variant_exists(L.var)) fail(FYN_ERR_UNSUPPORTED, "MFMA convolution variant not compiled");
    }
    while (L.steps.size() % conv_mfma_step_multiple(L.var) != 0) {
        MfmaLaunch::Step st;
        st.aoff = 0;
        for (int e = 0; e < 16; e++) { st.ky[e] = st.kx[e] = 0; st.ci[e] = -1; }
        L.steps.push_back(st);
    }
    if (kc == 4 && L.steps.size() > 64) fail(FYN_ERR_UNSUPPORTED, "too many kernel taps for the MFMA convolution (%zu steps)", L.steps.size());
    if (L.steps.size() > 256) fail(FYN_ERR_UNSUPPORTED, "too many kernel taps for the MFMA convolution (%zu steps per chunk)", L.steps.size());
    p.nsteps = (int)L.steps.size();
    std::vector<int> aoff;
    for (const MfmaLaunch::Step& st : L.steps) {
        if (kc == 4) aoff.insert(aoff.end(), st.off4, st.off4 + 4);
        else aoff.push_back(st.aoff);
    }
    L.aoff_dev = upload(net, aoff);
    p.aoff = L.aoff_dev;
    L.wpack_halves = (size_t)p.cin_chunks * p.nsteps * p.mfrags * npl * 64 * 8;
    // the buffer is sized generously (any step padding, any chunk width, the prefetch slack behind the last
    // step), so that tuning candidates can share it
    const size_t slack_halves = (size_t)16 * p.mfrags * npl * 64 * 8;
    if (share && share->wpack_alloc >= L.wpack_halves + slack_halves) {
        L.wpack_dev = share->wpack_dev;
        L.wpack_alloc = share->wpack_alloc;
    } else {
        L.wpack_alloc = 2 * L.wpack_halves + 4 * slack_halves;
        L.wpack_dev = net->dev_alloc(L.wpack_alloc * 2, true);
    }
    p.wpack = L.wpack_dev;
    p.chunks_per_split = p.cin_chunks;
    return L;
}

static std::string mfma_info(const MfmaLaunch& L);

// Launches a planned (sub-)convolution: the MFMA kernel and, with split-K, the reduce pass.
static int run_mfma(const MfmaLaunch& L, hipStream_t s) {
    const int rc = launch_conv_mfma(L.var, L.p, L.lds, s);
    if (rc != 0) return rc;
    if (L.p.ksplit > 1) launch_splitk_reduce(L.red, s);
    return 0;
}

// Turns a planned launch into its split-K form (ksplit slices over the input-channel chunks).
static void set_ksplit(Net* net, MfmaLaunch& L, int ksplit) {
    ConvMfmaParams& p = L.p;
    if (ksplit <= 1) {
        p.ksplit = 1;
        p.chunks_per_split = p.cin_chunks;
        p.partial = nullptr;
        return;
    }
    p.ksplit = ksplit;
    p.chunks_per_split = (p.cin_chunks + ksplit - 1) / ksplit;
    const size_t floats = (size_t)ksplit * p.npos_y * p.npos_x * p.cout_pad;
    p.partial = reinterpret_cast<float*>(net->dev_alloc(floats * sizeof(float), true));
    SplitKReduceParams& r = L.red;
    r.partial = p.partial; r.ksplit = ksplit; r.npos_y = p.npos_y; r.npos_x = p.npos_x; r.cout_pad = p.cout_pad;
    r.out = p.out; r.res = p.res; r.out_f16 = L.var.out_f16;
    r.out_wp = p.out_wp; r.out_cp = p.out_cp; r.out_step = p.out_step; r.out_off_y = p.out_off_y; r.out_off_x = p.out_off_x;
    r.res_wp = p.res_wp; r.res_cp = p.res_cp; r.res_off_y = p.res_off_y; r.res_off_x = p.res_off_x;
    r.res_relu = p.res_relu; r.res_scale = p.res_scale;
    r.acc_mul = p.acc_mul; r.scale = p.scale; r.bias = p.bias;
}

template <typename F>
static float time_calls(Net* net, F&& call, int iters) {
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
static float time_launch(Net* net, const MfmaLaunch& L, int iters) {
    return time_calls(net, [&]() {
        if (run_mfma(L, net->stream) != 0) fail(FYN_ERR_DEVICE, "convolution launch failed while tuning");
    }, iters);
}

// ---- optional on-disk memory of tuning results (text: "<key> fm fn wm wn kc ksplit tile_w_log2" per line) ----
static std::mutex g_tune_mu;   // guards the map and the file: networks may be set up from several threads
static std::map<std::string, std::array<int, 7>>& tune_cache(Net* net) {
    static std::map<std::string, std::array<int, 7>> cache;
    static bool loaded = false;
    if (!loaded) {
        loaded = true;
        const char* path = net->sw.get("FYNHIP_TUNE_CACHE");
        FILE* f = path ? fopen(path, "r") : nullptr;
        if (f) {
            char k[160];
            int a, b, c, d, e, g, h;
            while (fscanf(f, "%159s %d %d %d %d %d %d %d", k, &a, &b, &c, &d, &e, &g, &h) == 8) cache[k] = {a, b, c, d, e, g, h};
            fclose(f);
        }
    }
    return cache;
}

// switches that pin part of the choice are for experiments: choices are neither remembered nor recalled then
static bool tune_cache_bypassed(Net* net) {
    for (const char* e : {"FYNHIP_FORCE_KSPLIT", "FYNHIP_CONV_TILE", "FYNHIP_CONV_KC_MAX", "FYNHIP_CONV_KC", "FYNHIP_CONV_PD"})
        if (net->sw.get(e)) return true;
    return false;
}

static const TileChoice* tune_cache_lookup(Net* net, const char* key, const std::vector<TileChoice>& cands, int* ksplit) {
    if (tune_cache_bypassed(net)) return nullptr;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = tune_cache(net).find(key);
    if (it == tune_cache(net).end()) return nullptr;
    for (const TileChoice& c : cands)
        if (c.fm == it->second[0] && c.fn == it->second[1] && c.wm == it->second[2] && c.wn == it->second[3] && c.kc == it->second[4] &&
            c.twl == it->second[6]) {
            *ksplit = it->second[5];
            return &c;
        }
    return nullptr;
}

static void tune_cache_store(Net* net, const char* key, const ConvVariant& v, int ksplit, int twl) {
    if (tune_cache_bypassed(net)) return;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    tune_cache(net)[key] = {v.fm, v.fn, v.wm, v.wn, v.kc, ksplit, twl};   // same geometry later in this process: same choice
    const char* path = net->sw.get("FYNHIP_TUNE_CACHE");
    if (!path) return;
    FILE* f = fopen(path, "a");
    if (!f) return;
    fprintf(f, "%s %d %d %d %d %d %d %d\n", key, v.fm, v.fn, v.wm, v.wn, v.kc, ksplit, twl);
    fclose(f);
}

// a measured yes/no choice under a key of its own (same file, the first number is the flag)
static bool tune_cache_flag(Net* net, const char* key, bool* flag) {
    if (tune_cache_bypassed(net)) return false;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = tune_cache(net).find(key);
    if (it == tune_cache(net).end()) return false;
    *flag = it->second[0] != 0;
    return true;
}
static void tune_cache_store_flag(Net* net, const char* key, bool flag) {
    ConvVariant v{};
    v.fm = flag ? 1 : 0;
    tune_cache_store(net, key, v, 0, 0);
}
// three numbers under a key of their own (same file)
static bool tune_cache_triple(Net* net, const char* key, int (&out)[3]) {
    if (tune_cache_bypassed(net)) return false;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = tune_cache(net).find(key);
    if (it == tune_cache(net).end()) return false;
    out[0] = it->second[0]; out[1] = it->second[1]; out[2] = it->second[2];
    return true;
}
static void tune_cache_store_triple(Net* net, const char* key, int a, int b, int c) {
    ConvVariant v{};
    v.fm = a; v.fn = b; v.wm = c;
    tune_cache_store(net, key, v, 0, 0);
}

// Picks the tile configuration of one (sub-)convolution: by measurement on the layer's own tensors (default), or by
// the heuristic score when FYNHIP_AUTOTUNE=0.  Candidates are timed before the weights are packed, i.e. on zero
// operands; the matrix pipes run about a tenth faster on those than on real data (the part holds a higher clock when
// fewer operand bits toggle), for all candidates alike, so the ranking carries over while the figures do not.
static MfmaLaunch tune_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
                            int cout, const Act& act, int res_relu, int res_scale, const float* scale, const float* bias) {
    // candidates: every tile that fits, for the geometry's default chunk width, where that is wider than 32
    // channels for 32-channel chunks too, and for one-tap layers with 256 and more input channels chunks of
    // 256 to 1024 channels (a workgroup then fetches its whole reduction in one to three memory round trips)
    std::vector<TileChoice> cands;
    {
        int kc0, pitch, slack, npl;
        conv_geometry(net, in, !net->f16(), (int)sc.taps.size(), 0, kc0, pitch, slack, npl);
        std::vector<int> kcs{kc0};
        if (kc0 > 32) kcs.push_back(32);
        // one-tap layers with many input channels: also chunks of 256 to 1024 channels (K-split tiles only)
        if (sc.taps.size() == 1 && !net->sw.get("FYNHIP_CONV_KC_MAX"))
            for (int big : {256, 512, 1024})
                if (in.cp >= big) kcs.push_back(big);
        if (const char* fk = net->sw.get("FYNHIP_CONV_KC")) {   // testing: this chunk width first, the others only if it fits no tile
            const int f = atoi(fk);
            const bool known = f == 32 || f == 64 || f == 128 || ((f == 256 || f == 512 || f == 1024) && sc.taps.size() == 1);
            if (known && in.cp >= 32) kcs.insert(kcs.begin(), f);
        }
        for (int kco : kcs) {
            if (net->sw.get("FYNHIP_CONV_KC") && kco != kcs[0] && !cands.empty()) break;
            int kc;
            conv_geometry(net, in, !net->f16(), (int)sc.taps.size(), kco, kc, pitch, slack, npl);
            const int chunks = (kc == 4) ? 1 : (in.cp + kc - 1) / kc;
            std::vector<TileChoice> c = enumerate_tiles(net, cout, sc, pitch, npl, slack, chunks > 1 ? 2 : 1);
            for (TileChoice& tc : c) {
                tc.kc = kc;
                if (kco != kc0) tc.score *= 0.9;
                if (kc > 128 && tc.wm * tc.wn == 4) continue;
                if (tc.wm * tc.wn < 4) {   // tiles whose waves split K exist for chunks of 32 and more channels
                    const int wk = 4 / (tc.wm * tc.wn);
                    const int unr = kc > 128 ? 4 : 2;
                    const int raw = (int)sc.taps.size() * (kc / 16);
                    if (kc < 32 || (raw + unr * wk - 1) / (unr * wk) * (unr * wk) > 256) continue;
                }
                cands.push_back(tc);
            }
        }
        std::stable_sort(cands.begin(), cands.end(), [](const TileChoice& x, const TileChoice& y) { return x.score > y.score; });
    }
    if (cands.empty()) fail(FYN_ERR_UNSUPPORTED, "no MFMA tile configuration fits this convolution");
    const char* at = net->sw.get("FYNHIP_AUTOTUNE");
    const bool tune = !(at && at[0] == '0') && cands.size() > 1;
    // FYNHIP_TUNE_CACHE=<file>: measured choices are remembered per problem geometry, so that later
    // processes (e.g. under a profiler, where timing is distorted) pick the same kernels
    char key[160];
    snprintf(key, sizeof(key), "%d%d:%dx%d:%dx%d:s%d:t%zu:%dx%d:o%d:r%d:cp%d:e%d%d%d:f%d", in.f16, out.f16, cin, cout, sc.npos_y, sc.npos_x,
             sc.in_stride, sc.taps.size(), sc.span_y, sc.span_x, sc.out_step, res ? 1 : 0, in.cp, sc.clamp, sc.in_shift, sc.in_sub, sc.fuse_k);
    if (tune) {
        int ks = 1;
        const TileChoice* hit = tune_cache_lookup(net, key, cands, &ks);
        if (hit) {
            MfmaLaunch L = plan_mfma(net, sc, in, out, res, cin, cout, act, res_relu, res_scale, *hit, scale, bias);
            // a remembered split factor is held to what this layer allows, like a forced one
            if (sc.fuse_k || ks < 1) ks = 1;
            while (ks > 1 && ((ks - 1) * ((L.p.cin_chunks + ks - 1) / ks) >= L.p.cin_chunks || ks > 16)) ks--;
            set_ksplit(net, L, ks);
            return L;
        }
    }
    MfmaLaunch best = plan_mfma(net, sc, in, out, res, cin, cout, act, res_relu, res_scale, cands[0], scale, bias);
    if (const char* fk = net->sw.get("FYNHIP_FORCE_KSPLIT")) {   // testing: fixed split-K factor (clamped to what the layer allows)
        int ks = sc.fuse_k ? 1 : atoi(fk);   // (the fused shift-sum needs the whole reduction in one workgroup)
        while (ks > 1 && (ks - 1) * ((best.p.cin_chunks + ks - 1) / ks) >= best.p.cin_chunks) ks--;
        set_ksplit(net, best, ks);
        return best;
    }
    if (!tune) return best;
    const bool verbose = net->sw.get("FYNHIP_TUNE_VERBOSE") != nullptr;
    float best_ms = std::min(time_launch(net, best, 4), time_launch(net, best, 4));
    if (verbose) fprintf(stderr, "[tune] %s -> %.1f us\n", mfma_info(best).c_str(), best_ms * 1e3f);
    std::vector<std::pair<float, MfmaLaunch>> timed;
    timed.emplace_back(best_ms, best);
    for (size_t i = 1; i < cands.size(); i++) {
        MfmaLaunch L = plan_mfma(net, sc, in, out, res, cin, cout, act, res_relu, res_scale, cands[i], scale, bias, &best);
        const float ms = std::min(time_launch(net, L, 4), time_launch(net, L, 4));
        if (verbose) fprintf(stderr, "[tune] %s -> %.1f us\n", mfma_info(L).c_str(), ms * 1e3f);
        timed.emplace_back(ms, L);
        if (ms < best_ms) {
            best_ms = ms;
            best = L;
        }
    }
    // the winner and the candidates within a few percent of it are measured again over more launches
    {
        std::sort(timed.begin(), timed.end(), [](const std::pair<float, MfmaLaunch>& a, const std::pair<float, MfmaLaunch>& b) { return a.first < b.first; });
        size_t finalists = 1;
        while (finalists < timed.size() && finalists < 4 && timed[finalists].first <= 1.06f * timed[0].first) finalists++;
        {
            best_ms = 1e30f;
            for (size_t i = 0; i < finalists; i++) {
                float ms = 1e30f;
                for (int r = 0; r < 3; r++) ms = std::min(ms, time_launch(net, timed[i].second, 10));
                if (verbose) fprintf(stderr, "[tune] again %s -> %.1f us\n", mfma_info(timed[i].second).c_str(), ms * 1e3f);
                if (ms < best_ms) {
                    best_ms = ms;
                    best = timed[i].second;
                }
            }
        }
    }
    // few workgroups and several channel chunks: try splitting the reduction over more workgroups (for the
    // winner and, if its waves already split K inside the workgroup, also for the best tile that does not)
    std::vector<MfmaLaunch> trials;   // split-K variants that were timed
    std::vector<MfmaLaunch> bases{best};
    if (best.var.wm * best.var.wn < 4)
        for (const auto& t : timed)
            if (t.second.var.wm * t.second.var.wn == 4) {
                bases.push_back(t.second);
                break;
            }
    for (const MfmaLaunch& base : bases) {
        const int blocks = base.p.tiles_x * base.p.tiles_y * base.p.cout_blocks;
        for (int ks = 2; ks <= 16 && blocks < 192 && !sc.fuse_k; ks *= 2) {
            const int cps = (base.p.cin_chunks + ks - 1) / ks;
            if (base.p.cin_chunks < 2 || (ks - 1) * cps >= base.p.cin_chunks || blocks * ks > 1024) break;
            MfmaLaunch L = base;
            set_ksplit(net, L, ks);
            trials.push_back(L);
            // (timed like the finalists above: the event pair's share of a short measurement would count against it)
            float ms = 1e30f;
            for (int r = 0; r < 3; r++) ms = std::min(ms, time_launch(net, L, 10));
            if (verbose) fprintf(stderr, "[tune] %s -> %.1f us\n", mfma_info(L).c_str(), ms * 1e3f);
            if (ms < best_ms) {
                best_ms = ms;
                best = L;
            }
        }
    }
    tune_cache_store(net, key, best.var, best.p.ksplit, best.p.tile_w_log2);
    // the losing candidates' device buffers (step tables, weight buffers of their own, split-K partial sums) go back
    {
        std::vector<void*> drop;
        auto consider = [&](const MfmaLaunch& L) {
            for (void* q : {static_cast<void*>(L.aoff_dev), L.wpack_dev, static_cast<void*>(L.p.partial)})
                if (q && q != best.aoff_dev && q != best.wpack_dev && q != best.p.partial && std::find(drop.begin(), drop.end(), q) == drop.end())
                    drop.push_back(q);
        };
        for (const auto& t : timed) consider(t.second);
        for (const MfmaLaunch& L : trials) consider(L);
        net->dev_free_many(drop);
    }
    return best;
}

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

static int run_group(const MfmaGroup& g, hipStream_t s) {
    if (conv_mfma_multi_exists(g.var)) return launch_conv_mfma_multi(g.var, g.multi, g.lds, s);
    for (const MfmaLaunch& L : g.subs)   // no merged entry point for this variant (narrow channel chunks): one launch each
        if (int rc = launch_conv_mfma(L.var, L.p, L.lds, s)) return rc;
    return 0;
}

static float time_group(Net* net, const MfmaGroup& g, int iters) {
    hipEvent_t a, b;
    FYN_HIP(hipEventCreate(&a));
    FYN_HIP(hipEventCreate(&b));
    if (run_group(g, net->stream) != 0) fail(FYN_ERR_DEVICE, "convolution launch failed while tuning");
    FYN_HIP(hipEventRecord(a, net->stream));
    for (int i = 0; i < iters; i++) run_group(g, net->stream);
    FYN_HIP(hipEventRecord(b, net->stream));
    FYN_HIP(hipEventSynchronize(b));
    FYN_HIP(hipGetLastError());
    float ms = 0.f;
    FYN_HIP(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    return ms / iters;
}

// Picks ONE tile configuration and chunk width for a group of sub-convolutions (same tensors, different taps
// and output offsets) by timing the merged launch; the step group size is fixed so that all members fit it.
static MfmaGroup tune_mfma_group(Net* net, const std::vector<SubConv>& scs, const TView& in, const TView& out, int cin, int cout,
                                 const Act& act, const float* scale, const float* bias) {
    if (scs.empty() || scs.size() > FYN_CONV_MAX_SUB) fail(FYN_ERR_INVALID, "internal: bad sub-convolution group");
    // candidates from the member with the most taps (largest staged tile)
    size_t big = 0;
    for (size_t i = 1; i < scs.size(); i++)
        if (scs[i].taps.size() > scs[big].taps.size()) big = i;
    std::vector<TileChoice> cands;
    {
        int kc0, pitch, slack, npl;
        conv_geometry(net, in, !net->f16(), (int)scs[big].taps.size(), 0, kc0, pitch, slack, npl);
        std::vector<int> kcs{kc0};
        if (kc0 > 32) kcs.push_back(32);
        for (int kco : kcs) {
            int kc;
            conv_geometry(net, in, !net->f16(), (int)scs[big].taps.size(), kco, kc, pitch, slack, npl);
            const int chunks = (kc == 4) ? 1 : (in.cp + kc - 1) / kc;
            std::vector<TileChoice> c = enumerate_tiles(net, cout, scs[big], pitch, npl, slack, chunks > 1 ? 2 : 1);
            for (TileChoice& tc : c) {
                tc.kc = kc;
                if (tc.wm * tc.wn < 4) continue;   // no merged entry point for tiles whose waves split K
                cands.push_back(tc);
            }
        }
        std::stable_sort(cands.begin(), cands.end(), [](const TileChoice& x, const TileChoice& y) { return x.score > y.score; });
    }
    if (cands.empty()) fail(FYN_ERR_UNSUPPORTED, "no MFMA tile configuration fits this convolution");
    auto plan_all = [&](const TileChoice& tc, const MfmaGroup* share) {
        MfmaGroup g;
        for (size_t i = 0; i < scs.size(); i++)
            g.subs.push_back(plan_mfma(net, scs[i], in, out, nullptr, cin, cout, act, 0, 0, tc, scale, bias, share ? &share->subs[i] : nullptr, 2));
        g.sync();
        return g;
    };
    const char* at = net->sw.get("FYNHIP_AUTOTUNE");
    const bool tune = !(at && at[0] == '0') && cands.size() > 1;
    char key[160];
    snprintf(key, sizeof(key), "g%zu:%d%d:%dx%d:%dx%d:t%zu:o%d:cp%d", scs.size(), in.f16, out.f16, cin, cout, scs[big].npos_y, scs[big].npos_x,
             scs[big].taps.size(), scs[big].out_step, in.cp);
    if (tune) {
        int ks = 1;
        const TileChoice* hit = tune_cache_lookup(net, key, cands, &ks);
        if (hit) return plan_all(*hit, nullptr);
    }
    MfmaGroup best = plan_all(cands[0], nullptr);
    if (!tune) return best;
    const bool verbose = net->sw.get("FYNHIP_TUNE_VERBOSE") != nullptr;
    float best_ms = std::min(time_group(net, best, 4), time_group(net, best, 4));
    if (verbose) fprintf(stderr, "[tune] group of %zu: %s -> %.1f us\n", scs.size(), mfma_info(best.subs[0]).c_str(), best_ms * 1e3f);
    for (size_t i = 1; i < cands.size(); i++) {
        MfmaGroup g = plan_all(cands[i], &best);
        const float ms = std::min(time_group(net, g, 4), time_group(net, g, 4));
        if (verbose) fprintf(stderr, "[tune] group of %zu: %s -> %.1f us\n", scs.size(), mfma_info(g.subs[0]).c_str(), ms * 1e3f);
        if (ms < best_ms) {
            best_ms = ms;
            best = g;
        }
    }
    tune_cache_store(net, key, best.var, 1, best.subs[0].p.tile_w_log2);
    return best;
}

// Packs weights W[o][ky][kx][i] (block order, base/convlayerinterface.h:71-95) into the per-lane A
// fragment order of the kernel: [(chunk, step)][mfrag][plane][lane][8 halves]; for tiles whose waves split the
// steps of a chunk into WK groups, [group][chunk][step of the group]... (a wave walks its steps over all chunks
// with one stride).
static void pack_mfma_weights(Net* net, MfmaLaunch& L, const float* w, int k, float wmul, int kw = -1) {
    if (kw < 0) kw = k;
    const ConvMfmaParams& p = L.p;
    const int npl = L.var.split ? 2 : 1;
    const int kc = L.var.kc;
    std::vector<uint16_t> pack(L.wpack_halves, 0);
    const int nsub = p.nsteps / (4 / (L.var.wm * L.var.wn));   // steps per chunk and K group of waves
    for (int chunk = 0; chunk < p.cin_chunks; chunk++)
        for (int t = 0; t < p.nsteps; t++) {
            const MfmaLaunch::Step& st = L.steps[t];
            for (int mf = 0; mf < p.mfrags; mf++) {
                uint16_t* base = pack.data() + (((((size_t)(t / nsub) * p.cin_chunks + chunk) * nsub + t % nsub) * p.mfrags + mf) * npl) * 64 * 8;
                for (int lane = 0; lane < 64; lane++) {
                    const int o = mf * 32 + (lane & 31);
                    if (o >= L.cout) continue;
                    for (int j = 0; j < 8; j++) {
                        const int e = 8 * (lane >> 5) + j;
                        if (st.ci[e] < 0) continue;
                        const int ci = chunk * kc + st.ci[e];
                        if (ci >= L.cin) continue;
                        const float v = w[(((size_t)o * k + st.ky[e]) * kw + st.kx[e]) * L.cin + ci] * wmul;
                        const uint16_t hi = f2h_bits(v);
                        base[(size_t)lane * 8 + j] = hi;
                        if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                    }
                }
            }
        }
    FYN_HIP(hipStreamSynchronize(net->stream));
    FYN_HIP(hipMemcpyAsync(L.wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
    FYN_HIP(hipStreamSynchronize(net->stream));
}

// power of two that brings the largest weight magnitude to [2^11, 2^12): keeps hi and lo parts of the
// fp16 split in the normal range; undone exactly by acc_mul in the epilogue
static float weight_prescale(const float* w, size_t n) {
    float mx = 0.f;
    for (size_t i = 0; i < n; i++) mx = std::max(mx, std::fabs(w[i]));
    if (mx == 0.f || !std::isfinite(mx)) return 1.f;
    int e;
    std::frexp(mx, &e);  // mx = m * 2^e, m in [0.5,1)
    return std::ldexp(1.f, 12 - e);
}

// The planes behind the first of a packed fragment of the 16-position forms on fp32 tensors (three planes of 64 lanes x 8
// halves): plane 1 takes the fp16 lo part of weight j of a lane; c8 takes the sources of plane 2, the fp8 operands of
// the correction terms: hi / 32 in its first eight places, lo * 64 in the other eight (the staged activations carry the
// inverse factors, conv_p16.hip).
static void p16_lo_planes(uint16_t* frag_base, float* c8_lane, int lane, int j, float v, uint16_t hi) {
    const float lo = v - h2f(hi);
    frag_base[(size_t)(64 + lane) * 8 + j] = f2h_bits(lo);
    c8_lane[j] = h2f(hi) * (1.0f / 32.0f);
    c8_lane[8 + j] = lo * 64.0f;
}
static void upload_p16_pack(Net* net, void* dev, const std::vector<uint16_t>& pack, const std::vector<float>& c8, size_t frags) {
    FYN_HIP(hipStreamSynchronize(net->stream));
    FYN_HIP(hipMemcpyAsync(dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
    if (!c8.empty()) {
        float* src = upload(net, c8);
        if (launch_pack_fp8_plane(src, dev, frags, net->stream) != 0) fail(FYN_ERR_DEVICE, "packing the fp8 weight plane failed");
        net->dev_free(src);   // (waits for the stream)
    }
    FYN_HIP(hipStreamSynchronize(net->stream));
}

static std::string mfma_info(const MfmaLaunch& L) {
    char buf[256];
    snprintf(buf, sizeof(buf), "conv_mfma %s tile=%dx%d(cout x pos) waves=%dx%d kc=%d th=%d tw=%d blocks=%d lds=%zu steps=%d chunks=%d ksplit=%d",
             L.var.split ? "f16x2-split" : "f16", L.var.wm * L.var.fm * 32, L.var.wn * L.var.fn * 32, L.var.wm, L.var.wn, L.var.kc,
             L.p.tile_h, 1 << L.p.tile_w_log2, L.p.tiles_x * L.p.tiles_y * L.p.cout_blocks, L.lds, L.p.nsteps, L.p.cin_chunks, L.p.ksplit);
    return buf;
}

// =============================================================================================
// Convolution (CONVOLUTION2D, non-depthwise)
// =============================================================================================
class ConvLayer : public Layer {
  public:
    ConvLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        k = d.kernel;
        dil = d.dilation[0] > 0 ? d.dilation[0] : 1;
        stride = d.downsample[0] > 0 ? d.downsample[0] : 1;
        if ((k & 1) == 0 || k < 1) fail(FYN_ERR_UNSUPPORTED, "Unsupported convolution kernel size %d (%s)", k, d.name);
        if (d.dilation[0] != d.dilation[1] && d.dilation[1] > 0) fail(FYN_ERR_UNSUPPORTED, "anisotropic dilation not supported (%s)", d.name);
        if (d.downsample[0] != d.downsample[1] && d.downsample[1] > 0) fail(FYN_ERR_UNSUPPORTED, "anisotropic downsampling not supported (%s)", d.name);
        oc = d.out_channels;
        oh = d.height / stride;  // gpu/convlayerbase.cpp:47-48
        ow = d.width / stride;
        const int r = (k - 1) / 2;
        if (d.type == FYN_LAYER_FRACCONVOLUTION2D) {
            // gpu/gpulayerfactory.cpp:447-456, gpu/vanilla/fractionalconvlayerNxN_vanilla.cpp:43-50
            if (d.flags & FYN_FLAG_DEEP) fail(FYN_ERR_UNSUPPORTED, "Fractional convolution is not supported for deep layers");
            if (k == 1) fail(FYN_ERR_UNSUPPORTED, "Kernel size 1 not supported for fractional convolution (%s)", d.name);
            if (k > 9) fail(FYN_ERR_UNSUPPORTED, "Unsupported fractional convolution kernel size %d (%s)", k, d.name);   // shaders exist for 3, 5, 7, 9
            if (dil > 1 || d.dilation[1] > 1) fail(FYN_ERR_UNSUPPORTED, "Dilations not supported for fractional convolution");
            const float step = d.source_step > 0.f ? d.source_step : 1.f;
            int inv = 0;
            for (int s = 1; s <= 16; s *= 2)
                if (step * (float)s == 1.f) inv = s;
            // other steps put sample positions on texel boundaries, where the nearest filter's choice is the
            // GL implementation's; sizes must divide so that the positions stay dyadic
            if (!inv) fail(FYN_ERR_UNSUPPORTED, "fractional convolution (%s): sourceStep %g is not 1, 1/2, 1/4, 1/8 or 1/16", d.name, step);
            if ((d.width * inv) % stride || (d.height * inv) % stride)
                fail(FYN_ERR_UNSUPPORTED, "fractional convolution (%s): %dx%d is not a multiple of sourceStep*downsample", d.name, d.width, d.height);
            frac_shift = 1;
            while ((1 << (frac_shift - 1)) < inv) frac_shift++;
            oh = d.height * inv / stride;
            ow = d.width * inv / stride;
            clamp = true;
            direct = net->sw.get("FYNHIP_FORCE_DIRECT_CONV") != nullptr;
            wide = !direct && oc <= 4 && oc * k <= 32 && stride == 1 && d.in_channels > 4 && net->sw.get("FYNHIP_NO_WIDE_CONV") == nullptr;
            return;
        }
        // shallow, unpadded input: the sampler clamps to the edge (gpu/gpulayerbase.h:80-90)
        clamp = !(d.flags & FYN_FLAG_DEEP) && d.input_padding < r * dil && k > 1;
        direct = net->sw.get("FYNHIP_FORCE_DIRECT_CONV") != nullptr;   // (testing: the plain fp32 kernel instead of the MFMA path)
        // few output channels under a wide kernel: fold the kx taps into the GEMM's M dimension
        // (cout*K virtual channels, K taps) and reduce the K shifted partial sums in a second pass
        wide = !direct && oc <= 4 && oc * k <= 32 && k >= 3 && stride == 1 && dil == 1 && d.in_channels > 4 &&
               net->sw.get("FYNHIP_NO_WIDE_CONV") == nullptr;
    }
    // the sub-convolution of the folded form: K vertical taps over the columns of q
    SubConv wide_subconv() {
        const TView& in_v = tin(0).v;
        const int r = (k - 1) / 2;
        SubConv sc;
        for (int ky = 0; ky < k; ky++) sc.taps.push_back(Tap{ky, 0, ky, 0});
        sc.clamp = clamp ? 1 : 0;
        sc.span_y = k; sc.span_x = 1;
        sc.in_y0 = in_v.pad - r;
        sc.in_x0 = in_v.pad - r;
        if (frac_shift) {   // (the frame of repeated pixels, as in the one-stage form)
            sc.in_shift = frac_shift - 1;
            sc.in_y0 = (in_v.pad << sc.in_shift) - r;
            sc.in_x0 = (in_v.pad << sc.in_shift) + ((k == 3) ? -2 : -r);
        }
        sc.in_stride = 1;
        sc.npos_y = oh; sc.npos_x = ow + k - 1;
        sc.out_step = 1;
        sc.out_off_y = sc.out_off_x = 0;
        return sc;
    }
    // q through memory: stage 1 writes it, shift_reduce sums it
    void setup_two_pass_wide(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        qv = TView{};
        qv.h = oh; qv.w = ow + k - 1; qv.pad = 0; qv.c = oc * k; qv.cp = channel_pitch(oc * k); qv.f16 = out_v.f16;
        qv.ptr = net->dev_alloc(qv.bytes());
        SubConv sc = wide_subconv();
        if (!scale_dev) padded = std::max((oc * k + 127) / 128 * 128, out_v.cp);
        if (!scale_dev) {
            scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
            bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
        }
        q_scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
        q_bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
        launch = tune_mfma(net, sc, in_v, qv, nullptr, d.in_channels, oc * k, act(), 0, 0, q_scale_dev, q_bias_dev);
        sr.q = qv; sr.out = out_v; sr.res = res_v ? *res_v : TView{};
        sr.k = k; sr.cout = oc;
        sr.scale = scale_dev; sr.bias = bias_dev;
        sr.res_relu = res_relu; sr.res_scale = res_scale;
    }
    // value ranges (range.h)
    bool tracks_range() const override { return !direct; }
    void setup_ranges() override {
        const unsigned* in_w = tin(0).amax;
        unsigned* out_w = tout().amax;
        launch.p.in_amax = in_w;
        launch.p.out_amax = (launch.p.ksplit > 1 || (wide && !fused)) ? nullptr : out_w;   // the pass that writes the tensor raises its word
        launch.red.out_amax = out_w;
        sr.out_amax = out_w;
        rp.in_amax = in_w;
        rp.out_amax = out_w;
        pp.in_amax = in_w;
        pp.out_amax = out_w;
    }
    bool add_range_reset(unsigned* w) override {
        if (direct || !set_up || pj_into >= 0) return false;   // (a projection computed by its reader has no launch to clear words in)
        int& n = rows ? rp.nreset : (p16 ? pp.nreset : launch.p.nreset);
        if (n >= 4) return false;
        (rows ? rp.reset : (p16 ? pp.reset : launch.p.reset))[n++] = w;
        return true;
    }
    // 16-position-fragment form of a 3x3 convolution (conv_p16.hip): the compiled combinations that fit the layer are
    // timed (the three with the fewest fragment rounds on 256 CUs), and the best is kept if it beats the tuned launch of
    // the general kernel.
    void setup_p16(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = res_v ? res_v->ptr : nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = stride;
        q.in_y0 = q.in_x0 = in_v.pad - 1;
        q.in_clamp = clamp ? 1 : 0;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        q.cin_chunks = in_v.cp / 32;
        q.mfrags = oc / 16;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        q.in_amax = tin(0).amax;   // (the candidates are timed in the form the frame will run: fp8 correction terms where the input has a range word)
        q.exact_split = net->sw.get("FYNHIP_EXACT_SPLIT") ? 1 : 0;
        int want_h = 0, want_w = 0, want_wm = 0;   // FYNHIP_P16_TILE=h,w[,wm] (tests): that combination
        if (const char* e = net->sw.get("FYNHIP_P16_TILE")) sscanf(e, "%d,%d,%d", &want_h, &want_w, &want_wm);
        struct Cand { double cost; ConvP16Params q; };
        std::vector<Cand> cands;
        for (int i = 0; i < conv_p16_tile_count(); i++) {
            int th, tw, st, wm;
            conv_p16_tile(i, &th, &tw, &st, &wm);
            if (st != stride || oc % (32 * wm) != 0) continue;
            if (want_h && (th != want_h || tw != want_w || (want_wm && wm != want_wm))) continue;
            ConvP16Params c = q;
            c.tile_h = th; c.tile_w = tw; c.wm = wm;
            const int twg = (4 / wm) * tw;
            c.tiles_x = (ow + twg - 1) / twg; c.tiles_y = (oh + th - 1) / th;
            c.rcp_tiles_x = 1.0f / (float)c.tiles_x;
            c.cout_blocks = oc / (32 * wm);
            // one workgroup per CU: as many tile walkers per block of output channels as the chip has room for
            c.pos_groups = std::max(1, std::min(c.tiles_x * c.tiles_y, 256 / c.cout_blocks));
            if (res_v && c.cin_chunks < 2) c.pos_groups = c.tiles_x * c.tiles_y;   // (residual tile: one stage per tile is too few to walk)
            const size_t lds = conv_p16_lds_bytes(c);
            if (lds == 0 || lds > 160 * 1024) continue;
            // (a workgroup's eight waves take 140-240 registers each: one workgroup per CU whatever its LDS share)
            const int rounds = (c.tiles_x * c.tiles_y * c.cout_blocks + 255) / 256;
            cands.push_back(Cand{(double)rounds * (th * tw + 8) + 16, c});   // (+8: a tile's fixed part, +16: the launch's, in positions)
        }
        if (cands.empty()) return;
        std::sort(cands.begin(), cands.end(), [](const Cand& a, const Cand& b) { return a.cost < b.cost; });
        if (cands.size() > 3) cands.resize(3);
        const size_t halves = ((size_t)q.cin_chunks * 9 + 8) * q.mfrags * (q.f16 ? 1 : 3) * 64 * 8;
        p16_wpack_dev = net->dev_alloc(halves * 2, true);
        for (Cand& c : cands) c.q.wpack = p16_wpack_dev;
        const bool always = net->sw.get("FYNHIP_FORCE_P16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        const bool timing = !(at && at[0] == '0');
        int pick = 0;   // index into cands, -1: the general kernel
        char key[160];
        snprintf(key, sizeof(key), "p16:%dx%d:%dx%d:s%d:cp%d:r%d:e%d:h%d", d.in_channels, oc, oh, ow, stride, in_v.cp, res_v ? 1 : 0, clamp ? 1 : 0, q.f16);
        int cached[3] = {0, 0, 0};
        bool have_cached = false;
        if (!want_h) have_cached = tune_cache_triple(net, key, cached);   // (the cache keeps: chosen?, tile_h*1000 + tile_w, wm)
        if (have_cached) {
            pick = -1;
            if (cached[0] || always)
                for (size_t i = 0; i < cands.size(); i++)
                    if (cands[i].q.tile_h * 1000 + cands[i].q.tile_w == cached[1] && cands[i].q.wm == cached[2]) pick = (int)i;
            if (always && pick < 0) pick = 0;
        } else if (timing) {
            float best = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_p16(cands[i].q, net->stream) != 0) fail(FYN_ERR_DEVICE, "16-position convolution launch failed while tuning");
                    }, 10);
                    if (t < best) { best = t; pick = (int)i; }
                }
                t_other = std::min(t_other, time_launch(net, launch, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] 3x3: 16-position fragments (%dx%d tiles, %d channel groups) %.1f us, general kernel %.1f us\n",
                        cands[pick].q.tile_h, cands[pick].q.tile_w, cands[pick].q.wm, best * 1e3f, t_other * 1e3f);
            const bool win = best < t_other;
            if (!want_h) tune_cache_store_triple(net, key, win ? 1 : 0, cands[pick].q.tile_h * 1000 + cands[pick].q.tile_w, cands[pick].q.wm);
            if (!win && !always) pick = -1;
        }
        if (pick >= 0) {
            p16 = true;
            pp = cands[pick].q;
        } else {
            net->dev_free(p16_wpack_dev);
            p16_wpack_dev = nullptr;
        }
    }
    // the small-input form (conv_p16.hip, conv_p16c4_kernel): 9x9 on at most four input channels
    void setup_c4(const TView& in_v, const TView& out_v) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = 1; q.wm = 1;
        q.in_y0 = q.in_x0 = in_v.pad - (k - 1) / 2;
        q.in_clamp = clamp ? 1 : 0;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        q.cin_chunks = 1;
        q.mfrags = oc / 16;
        q.cout_blocks = oc / 32;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        int want_h = 0, want_w = 0;
        if (const char* e = net->sw.get("FYNHIP_P16_TILE")) sscanf(e, "%d,%d", &want_h, &want_w);
        std::vector<ConvP16Params> cands;
        int steps = 0;
        for (int i = 0; i < conv_p16c4_tile_count(); i++) {
            int kk, th, tw, ns;
            conv_p16c4_tile(i, &kk, &th, &tw, &ns);
            if (kk != k || (want_h && (th != want_h || tw != want_w))) continue;
            ConvP16Params c = q;
            c.tile_h = th; c.tile_w = tw;
            c.tiles_x = (ow + 4 * tw - 1) / (4 * tw); c.tiles_y = (oh + th - 1) / th;
            c.rcp_tiles_x = 1.0f / (float)c.tiles_x;
            c.pos_groups = std::max(1, std::min(c.tiles_x * c.tiles_y, 256 / c.cout_blocks));
            const size_t lds = conv_p16c4_lds_bytes(c, k);
            if (lds == 0 || lds > 160 * 1024) continue;
            steps = ns;
            cands.push_back(c);
        }
        if (cands.empty()) return;
        c4_steps = steps;
        const size_t halves = ((size_t)steps + 8) * q.mfrags * (q.f16 ? 1 : 2) * 64 * 8;
        p16_wpack_dev = net->dev_alloc(halves * 2, true);
        for (ConvP16Params& c : cands) c.wpack = p16_wpack_dev;
        const bool always = net->sw.get("FYNHIP_FORCE_P16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        int pick = 0;
        char key[160];
        snprintf(key, sizeof(key), "c4p16:k%d:%dx%d:%dx%d:e%d:h%d", k, d.in_channels, oc, oh, ow, clamp ? 1 : 0, q.f16);
        int cached[3] = {0, 0, 0};
        if (!want_h && tune_cache_triple(net, key, cached)) {
            pick = -1;
            if (cached[0] || always)
                for (size_t i = 0; i < cands.size(); i++)
                    if (cands[i].tile_h * 1000 + cands[i].tile_w == cached[1]) pick = (int)i;
            if (always && pick < 0) pick = 0;
        } else if (!(at && at[0] == '0')) {
            float best = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_p16c4(cands[i], k, net->stream) != 0) fail(FYN_ERR_DEVICE, "small-input 16-position convolution launch failed while tuning");
                    }, 10);
                    if (t < best) { best = t; pick = (int)i; }
                }
                t_other = std::min(t_other, time_launch(net, launch, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] %dx%d on %d channels: 16-position fragments (%dx%d tiles) %.1f us, general kernel %.1f us\n", k, k, d.in_channels,
                        cands[pick].tile_h, cands[pick].tile_w, best * 1e3f, t_other * 1e3f);
            const bool win = best < t_other;
            if (!want_h) tune_cache_store_triple(net, key, win ? 1 : 0, cands[pick].tile_h * 1000 + cands[pick].tile_w, 1);
            if (!win && !always) pick = -1;
        }
        if (pick >= 0) {
            p16 = true; c4 = true;
            pp = cands[pick];
        } else {
            net->dev_free(p16_wpack_dev);
            p16_wpack_dev = nullptr;
        }
    }
    // the fp16-storage form for wide layers (conv_h16.hip): K = 3 or 9, stride 1, blocks of 128 output channels.  A
    // launch takes a whole number of rounds of tiles over the chip's 256 CUs; when the last round of the best single
    // tile size would be far from full, the image is cut into two bands of rows with different tile heights (two
    // launches: e.g. 384 rows as three full rounds of 12-row tiles, the remaining 80 as one round of 8-row tiles).
    void setup_h16(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = res_v ? res_v->ptr : nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = 1; q.wm = 2;
        q.in_y0 = q.in_x0 = in_v.pad - (k - 1) / 2;
        q.in_clamp = clamp ? 1 : 0;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        q.cin_chunks = in_v.cp / 32;
        q.mfrags = oc / 16;
        q.cout_blocks = oc / 128;
        q.f16 = 1;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        int want_h = 0, want_w = 0, want_rows1 = 0, want_h2 = 0;   // FYNHIP_P16_TILE=h,w and FYNHIP_H16_SPLIT=rows of the first band,h of the second (tests)
        if (const char* e = net->sw.get("FYNHIP_P16_TILE")) sscanf(e, "%d,%d", &want_h, &want_w);
        if (const char* e = net->sw.get("FYNHIP_H16_SPLIT")) sscanf(e, "%d,%d", &want_rows1, &want_h2);
        // a band of `rows` output rows from row `row0` on, in tiles of th x tw; cost in MFMA cycles per wave (0: cannot be built)
        auto band = [&](int th, int tw, int row0, int rows, ConvP16Params* c, double* cost) {
            *c = q;
            c->tile_h = th; c->tile_w = tw;
            c->npos_y = rows;
            c->in_y0 = q.in_y0 + row0; c->out_off_y = q.out_off_y + row0; c->res_off_y = q.res_off_y + row0;
            c->tiles_x = (ow + 2 * tw - 1) / (2 * tw); c->tiles_y = (rows + th - 1) / th;
            c->rcp_tiles_x = 1.0f / (float)c->tiles_x;
            c->pos_groups = std::max(1, std::min(c->tiles_x * c->tiles_y, 256 / c->cout_blocks));
            if (res_v && c->cin_chunks < 2) c->pos_groups = c->tiles_x * c->tiles_y;   // (residual tile: one stage per tile is too few to walk)
            const size_t lds = conv_h16_lds_bytes(*c, k);
            if (lds == 0 || lds > 160 * 1024) return false;
            const int rounds = (c->tiles_x * c->tiles_y * c->cout_blocks + 255) / 256;
            *cost = (double)rounds * ((double)c->cin_chunks * k * k * (th * tw / 16) * 64 + 5000) + 10000;
            return true;
        };
        struct Cand { double cost; ConvP16Params a, b; bool two; };
        std::vector<Cand> cands;
        std::vector<std::pair<int, int>> tiles;
        for (int i = 0; i < conv_h16_tile_count(); i++) {
            int kk, th, tw;
            conv_h16_tile(i, &kk, &th, &tw);
            if (kk == k) tiles.push_back({th, tw});
        }
        for (auto& t : tiles) {
            if (want_h && (t.first != want_h || t.second != want_w)) continue;
            Cand c{};
            if (!want_rows1 && band(t.first, t.second, 0, oh, &c.a, &c.cost)) cands.push_back(c);
        }
        // the best cut into two bands (whole tiles of the first band's height above the cut)
        {
            Cand best{};
            best.cost = 1e300;
            for (auto& t1 : tiles)
                for (auto& t2 : tiles) {
                    if (want_h && (t1.first != want_h || t1.second != want_w)) continue;
                    if (want_h2 && t2.first != want_h2) continue;
                    for (int rows1 = t1.first; rows1 < oh; rows1 += t1.first) {
                        if (want_rows1 && rows1 != want_rows1) continue;
                        Cand c{};
                        double c1, c2;
                        if (!band(t1.first, t1.second, 0, rows1, &c.a, &c1) || !band(t2.first, t2.second, rows1, oh - rows1, &c.b, &c2)) continue;
                        c.cost = c1 + c2;
                        c.two = true;
                        if (c.cost < best.cost) best = c;
                    }
                }
            if (best.cost < 1e299) cands.push_back(best);
        }
        if (cands.empty()) return;
        std::sort(cands.begin(), cands.end(), [](const Cand& a, const Cand& b) { return a.cost < b.cost; });
        if (cands.size() > 3) cands.resize(3);
        const size_t halves = ((size_t)q.cin_chunks * k * k + 8) * q.mfrags * 64 * 8;
        p16_wpack_dev = net->dev_alloc(halves * 2, true);
        for (Cand& c : cands) c.a.wpack = c.b.wpack = p16_wpack_dev;
        auto run = [&](const Cand& c) {
            if (launch_conv_h16(c.a, k, net->stream) != 0 || (c.two && launch_conv_h16(c.b, k, net->stream) != 0))
                fail(FYN_ERR_DEVICE, "fp16 16-position convolution launch failed while tuning");
        };
        const bool forced = want_h || want_rows1;
        const bool always = net->sw.get("FYNHIP_FORCE_P16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        int pick = 0;
        char key[160];
        snprintf(key, sizeof(key), "h16:k%d:%dx%d:%dx%d:cp%d:r%d:e%d", k, d.in_channels, oc, oh, ow, in_v.cp, res_v ? 1 : 0, clamp ? 1 : 0);
        // (the cache keeps: chosen?, tile_h*1000 + tile_w of the first band, rows*1000 + tile_h of the second or 0)
        auto code1 = [](const Cand& c) { return c.a.tile_h * 1000 + c.a.tile_w; };
        auto code2 = [](const Cand& c) { return c.two ? c.a.npos_y * 1000 + c.b.tile_h : 0; };
        int cached[3] = {0, 0, 0};
        if (!forced && tune_cache_triple(net, key, cached)) {
            pick = -1;
            if (cached[0] || always)
                for (size_t i = 0; i < cands.size(); i++)
                    if (code1(cands[i]) == cached[1] && code2(cands[i]) == cached[2]) pick = (int)i;
            if (always && pick < 0) pick = 0;
        } else if (!(at && at[0] == '0')) {
            float best = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 2; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() { run(cands[i]); }, 5);
                    if (t < best) { best = t; pick = (int)i; }
                }
                t_other = std::min(t_other, time_launch(net, launch, 5));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] %dx%d fp16: 16-position fragments (%dx%d tiles%s) %.1f us, general kernel %.1f us\n", k, k,
                        cands[pick].a.tile_h, cands[pick].a.tile_w, cands[pick].two ? ", two bands" : "", best * 1e3f, t_other * 1e3f);
            const bool win = best < t_other;
            if (!forced) tune_cache_store_triple(net, key, win ? 1 : 0, code1(cands[pick]), code2(cands[pick]));
            if (!win && !always) pick = -1;
        }
        if (pick >= 0) {
            p16 = true; h16 = true;
            pp = cands[pick].a;
            h16_two = cands[pick].two;
            pp2 = cands[pick].b;
        } else {
            net->dev_free(p16_wpack_dev);
            p16_wpack_dev = nullptr;
        }
    }
    // weights of that form: [(chunk*K + ky)*K + kx][cout fragment of 16][lane][8 halves], zero steps behind the last
    void pack_h16(const float* w, float wmul) {
        const int cin = d.in_channels;
        std::vector<uint16_t> pack(((size_t)pp.cin_chunks * k * k + 8) * pp.mfrags * 64 * 8, 0);
        for (int chunk = 0; chunk < pp.cin_chunks; chunk++)
            for (int tap = 0; tap < k * k; tap++)
                for (int mf = 0; mf < pp.mfrags; mf++) {
                    uint16_t* base = pack.data() + ((size_t)(chunk * k * k + tap) * pp.mfrags + mf) * 64 * 8;
                    for (int lane = 0; lane < 64; lane++) {
                        const int o = mf * 16 + (lane & 15);
                        if (o >= oc) continue;
                        for (int j = 0; j < 8; j++) {
                            const int ci = chunk * 32 + 8 * (lane >> 4) + j;
                            if (ci >= cin) continue;
                            base[(size_t)lane * 8 + j] = f2h_bits(w[((size_t)o * k * k + tap) * cin + ci] * wmul);
                        }
                    }
                }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(p16_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    // the K-resident form for layers with few positions and many input channels (conv_p16.hip, conv_kr16_kernel)
    void setup_kr16(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = res_v ? res_v->ptr : nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = stride;   // (k = 1: position (y, x) reads pixel (y, x) * stride; k = 3: the kernel variant's stride)
        q.in_y0 = q.in_x0 = in_v.pad - (k - 1) / 2;
        q.in_clamp = clamp ? 1 : 0;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        q.cin_chunks = (in_v.cp + 127) / 128 * 4;   // (four waves share the chunks: rounded up, the channels behind the pitch read as zero)
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        int want_fm = 0, want_th = 0, want_tw = 0;   // FYNHIP_KR16_FM=fragments per block of output channels[,tile h,tile w] (tests)
        if (const char* e = net->sw.get("FYNHIP_KR16_FM")) sscanf(e, "%d,%d,%d", &want_fm, &want_th, &want_tw);
        std::vector<ConvP16Params> cands;
        for (int i = 0; i < conv_kr16_variant_count(); i++) {
            int taps, chunks, fm, th, tw, vstride;
            conv_kr16_variant(i, &taps, &chunks, &fm, &th, &tw, &vstride);
            if (taps != k * k || chunks != q.cin_chunks || (want_fm && fm != want_fm) || (k != 1 && vstride != stride)) continue;
            if (fm == 2 && oc % 32 != 0 && oc % 32 <= 16) continue;   // (the last block would be half empty: the 16-channel blocks do)
            if (want_th ? (th != want_th || tw != want_tw) : (want_fm && th * tw != 16)) continue;
            // (larger tiles are for layers that would need several rounds of 16-position workgroups)
            if (th * tw > 16 && !want_th && ((oh + 3) / 4) * ((ow + 3) / 4) * ((oc + 16 * fm - 1) / (16 * fm)) <= 512) continue;
            ConvP16Params c = q;
            c.tile_h = th; c.tile_w = tw;
            c.tiles_x = (ow + tw - 1) / tw; c.tiles_y = (oh + th - 1) / th;
            c.rcp_tiles_x = 1.0f / (float)c.tiles_x;
            c.pos_groups = c.tiles_x * c.tiles_y;
            c.wm = fm;
            c.cout_blocks = (oc + 16 * fm - 1) / (16 * fm);   // (the last block may be partly empty: zero weights, rows beyond the pitch not stored)
            c.mfrags = c.cout_blocks * fm;
            const size_t lds = conv_kr16_lds_bytes(c, k);
            if (lds == 0 || lds > 160 * 1024 || (long long)c.pos_groups * c.cout_blocks > 65535) continue;
            bool listed = false;   // (a one-round and a two-round variant of the same shape are one launch: the first that fits the LDS)
            for (const ConvP16Params& o : cands) listed = listed || (o.wm == c.wm && o.tile_h == c.tile_h && o.tile_w == c.tile_w);
            if (!listed) cands.push_back(c);
        }
        if (cands.empty()) return;
        // (large enough for every candidate: cout blocks x 4 waves x steps x fragments x planes)
        const size_t halves = (size_t)((oc + 31) / 32 * 2) * 4 * (q.cin_chunks / 4) * k * k * (q.f16 ? 1 : 2) * 64 * 8;
        void* const kr_wpack = net->dev_alloc(halves * 2, true);
        for (ConvP16Params& c : cands) c.wpack = kr_wpack;
        const bool had_p16 = p16;   // the 3x3 16-position form was chosen over the general kernel: this form has to beat it instead
        const bool always = net->sw.get("FYNHIP_FORCE_KR16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        int pick = 0;
        char key[160];
        snprintf(key, sizeof(key), "kr16:k%d:%dx%d:%dx%d:s%d:r%d:e%d:h%d:p%d", k, d.in_channels, oc, oh, ow, stride, res_v ? 1 : 0, clamp ? 1 : 0, q.f16, had_p16 ? 1 : 0);
        int cached[3] = {0, 0, 0};
        if (!want_fm && tune_cache_triple(net, key, cached)) {
            pick = -1;
            if (cached[0] || always)
                for (size_t i = 0; i < cands.size(); i++)
                    if (cands[i].wm == cached[1] && cands[i].tile_h * 100 + cands[i].tile_w == cached[2]) pick = (int)i;
            if (always && pick < 0) pick = 0;
        } else if (!(at && at[0] == '0')) {
            float best = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_kr16(cands[i], k, net->stream) != 0) fail(FYN_ERR_DEVICE, "K-resident convolution launch failed while tuning");
                    }, 10);
                    if (t < best) { best = t; pick = (int)i; }
                }
                if (had_p16)
                    t_other = std::min(t_other, time_calls(net, [&]() {
                        if (launch_conv_p16(pp, net->stream) != 0) fail(FYN_ERR_DEVICE, "16-position convolution launch failed while tuning");
                    }, 10));
                else
                    t_other = std::min(t_other, time_launch(net, launch, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] %dx%d on %d channels, %dx%d positions: K-resident form (%d-channel blocks, %dx%d tiles) %.1f us, %s %.1f us\n", k, k,
                        d.in_channels, oh, ow, 16 * cands[pick].wm, cands[pick].tile_h, cands[pick].tile_w, best * 1e3f,
                        had_p16 ? "16-position 3x3 form" : "general kernel", t_other * 1e3f);
            const bool win = best < t_other;
            if (!want_fm) tune_cache_store_triple(net, key, win ? 1 : 0, cands[pick].wm, cands[pick].tile_h * 100 + cands[pick].tile_w);
            if (!win && !always) pick = -1;
        }
        if (pick >= 0) {
            if (had_p16) net->dev_free(p16_wpack_dev);
            p16_wpack_dev = kr_wpack;
            p16 = true; kr16 = true;
            pp = cands[pick];
        } else {
            net->dev_free(kr_wpack);
        }
    }
    // The LDS-free 1x1 form (conv_d16.hip) against what has been chosen so far (the general kernel or the K-resident form).
    void setup_d16(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = res_v ? res_v->ptr : nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = stride;
        const int ks = k == 1 ? 0 : k;   // a K x K convolution on an input of at most four channels: steps of eight taps
        q.tile_h = ks;
        q.in_y0 = q.in_x0 = in_v.pad - (k - 1) / 2;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        q.cin_chunks = ks ? (ks * ks + 7) / 8 : (in_v.cp + 31) / 32;
        q.mfrags = (oc + 15) / 16;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        const size_t halves = (size_t)q.mfrags * q.cin_chunks * (q.f16 ? 1 : 2) * 64 * 8;
        void* const wp = net->dev_alloc(halves * 2, true);
        q.wpack = wp;
        q.wm = 1;
        q.cout_blocks = 1;   // workgroups per 16 positions (they share the fragments of output channels): 1, 2 or 4, timed
        const int min_blocks = ks ? (q.mfrags + 3) / 4 : 1;   // (the K x K form: one fragment per wave)
        if (ks && min_blocks > 4) { net->dev_free(wp); return; }
        q.cout_blocks = min_blocks;
        if (const char* e = net->sw.get("FYNHIP_D16_BLOCKS")) q.cout_blocks = std::max(-4, std::min(4, atoi(e))) ? std::max(-4, std::min(4, atoi(e))) : 1;   // (negative: a wave per 16 positions)
        const bool always = net->sw.get("FYNHIP_FORCE_D16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        bool pick = true;
        char key[160];
        snprintf(key, sizeof(key), "d16:k%d:%dx%d:%dx%d:s%d:r%d:h%d:kr%d", k, d.in_channels, oc, oh, ow, stride, res_v ? 1 : 0, q.f16, kr16 ? 1 : 0);
        int cached[3] = {0, 0, 0};
        if (net->sw.get("FYNHIP_D16_BLOCKS")) {
            pick = always;
        } else if (tune_cache_triple(net, key, cached)) {
            pick = cached[0] != 0 || always;
            q.cout_blocks = cached[1] ? cached[1] : 1;
        } else if (!(at && at[0] == '0')) {
            float t_new = 1e30f, t_other = 1e30f;
            int best_blocks = 1;
            for (int rep = 0; rep < 3; rep++) {
                for (int blocks = min_blocks; blocks <= 4 && 4 * blocks <= std::max(4 * min_blocks, q.mfrags); blocks *= 2) {
                    ConvP16Params c = q;
                    c.cout_blocks = blocks;
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_d16(c, net->stream) != 0) fail(FYN_ERR_DEVICE, "LDS-free 1x1 convolution launch failed while tuning");
                    }, 10);
                    if (t < t_new) { t_new = t; best_blocks = blocks; }
                }
                if (q.mfrags <= 4) {   // few fragments: a wave per 16 positions and fragment instead (noted as a negative count)
                    ConvP16Params c = q;
                    c.wm = 4; c.cout_blocks = q.mfrags;
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_d16(c, net->stream) != 0) fail(FYN_ERR_DEVICE, "LDS-free 1x1 convolution launch failed while tuning");
                    }, 10);
                    if (t < t_new) { t_new = t; best_blocks = -q.mfrags; }
                }
                if (kr16)
                    t_other = std::min(t_other, time_calls(net, [&]() {
                        if (launch_conv_kr16(pp, k, net->stream) != 0) fail(FYN_ERR_DEVICE, "K-resident convolution launch failed while tuning");
                    }, 10));
                else
                    t_other = std::min(t_other, time_launch(net, launch, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] %dx%d on %d channels, %dx%d positions, to %d: LDS-free form (%d %s per 16 positions) %.1f us, %s %.1f us\n", k, k, d.in_channels, oh, ow,
                        oc, best_blocks < 0 ? 1 : best_blocks, best_blocks < 0 ? "wave per fragment" : "workgroup(s)", t_new * 1e3f, kr16 ? "K-resident form" : "general kernel", t_other * 1e3f);
            pick = t_new < t_other || always;
            q.cout_blocks = best_blocks;
            tune_cache_store_triple(net, key, t_new < t_other ? 1 : 0, best_blocks, 0);
        }
        if (q.cout_blocks < 0) { q.wm = 4; q.cout_blocks = -q.cout_blocks; }
        if (pick) {
            if (p16) net->dev_free(p16_wpack_dev);
            p16_wpack_dev = wp;
            p16 = true; kr16 = false; d16 = true;
            pp = q;
        } else {
            net->dev_free(wp);
        }
    }
    // weights of that form: [cout fragment][chunk][plane][lane][8 halves]
    void pack_d16(const float* w, float wmul) {
        if (pp.tile_h) pack_taps16(w, wmul);
        else pack_frag16(pp, p16_wpack_dev, w, wmul);
    }
    // the K x K form on four-channel pixels: [cout fragment][step][plane][lane][8 halves], a lane's eight values being
    // the four channels of taps 8*step + 2*(lane/16) and the next one, in row-major order
    void pack_taps16(const float* w, float wmul) {
        const int cin = d.in_channels, npl = pp.f16 ? 1 : 2;
        std::vector<uint16_t> pack((size_t)pp.mfrags * pp.cin_chunks * npl * 64 * 8, 0);
        for (int mf = 0; mf < pp.mfrags; mf++)
            for (int c = 0; c < pp.cin_chunks; c++) {
                uint16_t* base = pack.data() + ((size_t)(mf * pp.cin_chunks + c) * npl) * 64 * 8;
                for (int lane = 0; lane < 64; lane++) {
                    const int o = mf * 16 + (lane & 15);
                    if (o >= oc) continue;
                    for (int j = 0; j < 8; j++) {
                        const int tap = c * 8 + 2 * (lane >> 4) + j / 4, ci = j % 4;
                        if (tap >= k * k || ci >= cin) continue;
                        const float v = w[((size_t)o * k * k + tap) * cin + ci] * wmul;
                        const uint16_t hi = f2h_bits(v);
                        base[(size_t)lane * 8 + j] = hi;
                        if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                    }
                }
            }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(p16_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    void pack_frag16(const ConvP16Params& q, void* dev, const float* w, float wmul) {
        const int cin = d.in_channels, npl = q.f16 ? 1 : 2;
        std::vector<uint16_t> pack((size_t)q.mfrags * q.cin_chunks * npl * 64 * 8, 0);
        for (int mf = 0; mf < q.mfrags; mf++)
            for (int c = 0; c < q.cin_chunks; c++) {
                uint16_t* base = pack.data() + ((size_t)(mf * q.cin_chunks + c) * npl) * 64 * 8;
                for (int lane = 0; lane < 64; lane++) {
                    const int o = mf * 16 + (lane & 15);
                    if (o >= oc) continue;
                    for (int j = 0; j < 8; j++) {
                        const int ci = c * 32 + 8 * (lane >> 4) + j;
                        if (ci >= cin) continue;
                        const float v = w[(size_t)o * cin + ci] * wmul;
                        const uint16_t hi = f2h_bits(v);
                        base[(size_t)lane * 8 + j] = hi;
                        if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                    }
                }
            }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    // weights of that form: [cout block][wave][step][fragment][plane][lane][8 halves]; step s of wave w = (chunk w + 4*(s / taps), tap s % taps)
    void pack_kr16(const float* w, float wmul) {
        const int cin = d.in_channels, taps = k * k, fm_n = pp.wm, npl = pp.f16 ? 1 : 2;
        const int steps = pp.cin_chunks / 4 * taps;
        std::vector<uint16_t> pack((size_t)pp.cout_blocks * 4 * steps * fm_n * npl * 64 * 8, 0);
        for (int cb = 0; cb < pp.cout_blocks; cb++)
            for (int wv = 0; wv < 4; wv++)
                for (int st = 0; st < steps; st++) {
                    const int chunk = wv + 4 * (st / taps), tap = st % taps;
                    for (int fm = 0; fm < fm_n; fm++) {
                        uint16_t* base = pack.data() + ((((size_t)(cb * 4 + wv) * steps + st) * fm_n + fm) * npl) * 64 * 8;
                        for (int lane = 0; lane < 64; lane++) {
                            const int o = (cb * fm_n + fm) * 16 + (lane & 15);
                            if (o >= oc) continue;
                            for (int j = 0; j < 8; j++) {
                                const int ci = chunk * 32 + 8 * (lane >> 4) + j;
                                if (ci >= cin) continue;
                                const float v = w[((size_t)o * taps + tap) * cin + ci] * wmul;
                                const uint16_t hi = f2h_bits(v);
                                base[(size_t)lane * 8 + j] = hi;
                                if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                            }
                        }
                    }
                }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(p16_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    // weights of that form: [step][cout fragment of 16][plane][lane][8 halves]; lane = (channel lane%16, tap pair 4*step + lane/16)
    void pack_c4(const float* w, float wmul) {
        const int cin = d.in_channels, ppr = (k + 1) / 2;
        const int npl = pp.f16 ? 1 : 2;   // (fp16 tensors: the hi plane only)
        std::vector<uint16_t> pack(((size_t)c4_steps + 8) * pp.mfrags * npl * 64 * 8, 0);
        for (int st = 0; st < c4_steps; st++)
            for (int mf = 0; mf < pp.mfrags; mf++) {
                uint16_t* base = pack.data() + (((size_t)st * pp.mfrags + mf) * npl) * 64 * 8;
                for (int lane = 0; lane < 64; lane++) {
                    const int o = p16_row_channel(mf, lane & 15, pp.f16 ? 2 : 1), pi = 4 * st + (lane >> 4);
                    const int ky = pi / ppr, kx0 = 2 * (pi % ppr);
                    if (o >= oc || ky >= k) continue;
                    for (int j = 0; j < 8; j++) {
                        const int kx = kx0 + j / 4, ci = j % 4;
                        if (kx >= k || ci >= cin) continue;
                        const float v = w[(((size_t)o * k + ky) * k + kx) * cin + ci] * wmul;
                        const uint16_t hi = f2h_bits(v);
                        base[(size_t)lane * 8 + j] = hi;
                        if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                    }
                }
            }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(p16_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    // weights of that form: [(chunk*9 + tap)][cout fragment of 16][plane][lane][8 halves], zero steps behind the last
    void pack_p16(const float* w, float wmul) {
        const int cin = d.in_channels;
        const int npl = pp.f16 ? 1 : 3;   // fp32 tensors: hi, lo, and the fp8 operands of the correction terms
        const size_t frags = ((size_t)pp.cin_chunks * 9 + 8) * pp.mfrags;
        std::vector<uint16_t> pack(frags * npl * 64 * 8, 0);
        std::vector<float> c8(npl == 3 ? frags * 64 * 16 : 0, 0.f);
        for (int chunk = 0; chunk < pp.cin_chunks; chunk++)
            for (int tap = 0; tap < 9; tap++)
                for (int mf = 0; mf < pp.mfrags; mf++) {
                    const size_t frag = (size_t)(chunk * 9 + tap) * pp.mfrags + mf;
                    uint16_t* base = pack.data() + frag * npl * 64 * 8;
                    for (int lane = 0; lane < 64; lane++) {
                        const int o = p16_row_channel(mf, lane & 15, pp.f16 ? 2 : 1);
                        if (o >= oc) continue;
                        for (int j = 0; j < 8; j++) {
                            const int ci = chunk * 32 + 8 * (lane >> 4) + j;
                            if (ci >= cin) continue;
                            const float v = w[(((size_t)o * 3 + tap / 3) * 3 + tap % 3) * cin + ci] * wmul;
                            const uint16_t hi = f2h_bits(v);
                            base[(size_t)lane * 8 + j] = hi;
                            if (npl == 3) p16_lo_planes(base, c8.data() + (frag * 64 + lane) * 16, lane, j, v, hi);
                        }
                    }
                }
        upload_p16_pack(net, p16_wpack_dev, pack, c8, frags);
    }
    void setup_rows_wide(const TView& in_v, const TView& out_v, const TView* res_v, int res_relu, int res_scale) {
        const int r = (k - 1) / 2;
        ConvRowsParams q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = res_v ? res_v->ptr : nullptr;
        q.k = k; q.cs = (in_v.cp + 15) / 16; q.fn = 2;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.in_y0 = in_v.pad - r; q.in_x0 = in_v.pad - r;
        q.in_clamp = clamp ? 1 : 0;
        q.out_h = oh; q.out_w = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        const int strip_w = 32 * q.fn - (k - 1);
        q.strips = (ow + strip_w - 1) / strip_w;
        // one workgroup per CU (the ring takes most of the LDS): as many row blocks as fill the chip in one round
        int blocks = std::max(1, 256 / q.strips);
        q.rows_per_block = ((oh + blocks - 1) / blocks + 3) / 4 * 4;
        q.row_blocks = (oh + q.rows_per_block - 1) / q.rows_per_block;
        q.cout = oc;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        if (conv_rows_lds_bytes(q, out_v.f16 != 0) > 160 * 1024) return;
        const size_t halves = (size_t)k * q.cs * (out_v.f16 ? 1 : 2) * 64 * 8;
        q.wpack = rows_wpack_dev = net->dev_alloc(halves * 2, true);
        const bool always = net->sw.get("FYNHIP_FORCE_ROWS_WIDE_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        bool pick = true;
        char key[160];
        snprintf(key, sizeof(key), "rows:%d:%dx%d:%dx%d:k%d:cp%d:r%d:e%d", out_v.f16, d.in_channels, oc, oh, ow, k, in_v.cp, res_v ? 1 : 0, clamp ? 1 : 0);
        if (always) {
        } else if (tune_cache_flag(net, key, &pick)) {
        } else if (!(at && at[0] == '0')) {
            float t_rows = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                t_rows = std::min(t_rows, time_calls(net, [&]() {
                    if (launch_conv_rows(q, out_v.f16 != 0, net->stream) != 0) fail(FYN_ERR_DEVICE, "row-rolling convolution launch failed while tuning");
                }, 10));
                t_other = std::min(t_other, time_calls(net, [&]() {
                    run_mfma(launch, net->stream);
                    if (!fused) launch_shift_reduce(sr, net->stream);
                }, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE")) fprintf(stderr, "[tune] folded kx taps: row-rolling %.1f us, %s %.1f us\n", t_rows * 1e3f, fused ? "one launch" : "two passes", t_other * 1e3f);
            pick = t_rows < t_other;
            tune_cache_store_flag(net, key, pick);
        }
        if (pick) {
            rows = true;
            rp = q;
            if (qv.ptr) { net->dev_free(qv.ptr); qv.ptr = nullptr; }
        } else {
            net->dev_free(rows_wpack_dev);
            rows_wpack_dev = nullptr;
        }
    }
    // weights of the row-rolling form: [step = ky*cs + sub][plane][lane][8 halves]
    void pack_rows(const float* w, float wmul) {
        const int cin = d.in_channels, npl = tout().v.f16 ? 1 : 2;
        std::vector<uint16_t> pack((size_t)k * rp.cs * npl * 64 * 8, 0);
        for (int ky = 0; ky < k; ky++)
            for (int sub = 0; sub < rp.cs; sub++)
                for (int lane = 0; lane < 64; lane++) {
                    const int vch = lane & 31, o = vch / k, kx = vch % k;
                    if (o >= oc) continue;
                    for (int j = 0; j < 8; j++) {
                        const int ci = sub * 16 + 8 * (lane >> 5) + j;
                        if (ci >= cin) continue;
                        const float v = w[(((size_t)o * k + ky) * k + kx) * cin + ci] * wmul;
                        const uint16_t hi = f2h_bits(v);
                        const size_t base = ((size_t)(ky * rp.cs + sub) * npl) * 64 * 8;
                        pack[base + (size_t)lane * 8 + j] = hi;
                        if (npl == 2) pack[base + (size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                    }
                }
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(rows_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    size_t weight_floats() const override {
        return (size_t)oc + (size_t)oc * k * k * d.in_channels + ((d.flags & FYN_FLAG_POST_BATCHNORM) ? 2 * (size_t)oc : 0);
    }
    void load_weights(const float* blk) override {
        block.assign(blk, blk + weight_floats());
        if (set_up) pack();
    }
    void setup() override {
        const TView& in_v = tin(0).v;
        const TView& out_v = tout().v;
        const TView* res_v = (d.flags & FYN_FLAG_RESIDUAL_INPUT) ? &tin(1).v : nullptr;
        const int r = (k - 1) / 2;
        const int res_relu = (d.flags & FYN_FLAG_RELU_ON_RESIDUAL) ? 1 : 0;
        const int res_scale = ((d.flags & FYN_FLAG_BATCHNORM_ON_RESIDUAL) && (d.flags & FYN_FLAG_POST_BATCHNORM)) ? 1 : 0;
        if (direct) {
            dp.in = in_v; dp.out = out_v;
            dp.in.c = std::min(d.in_channels, in_v.cp);   // the weights' channel count (the producer may name up to 3 more or fewer)
            dp.res = res_v ? *res_v : TView{};
            dp.k = k; dp.dil = dil; dp.stride = stride;
            dp.in_y0 = dp.in_x0 = in_v.pad - r * dil;
            dp.clamp = clamp ? 1 : 0;
            dp.frac_shift = frac_shift;
            // taps sit at kx - r steps, except under the 3x3 kernel, whose shader samples at -2, -1 and 0 steps
            // (shaders/vanilla/fraconv3x3.frag:14-19 against fraconv5x5.frag:14-22); rows are offset through the
            // proxy polygons, symmetrically for every size (gpu/vanilla/convlayerbase_vanilla.cpp:365)
            dp.tap_x0 = (k == 3) ? -2 : -r;
            dp.tap_y0 = -r;
            dp.res_relu = res_relu; dp.res_scale = res_scale;
            dp.act = act();
            padded = out_v.cp;
            wdirect_dev = static_cast<float*>(net->dev_alloc((size_t)k * k * d.in_channels * out_v.cp * sizeof(float)));
        } else if (wide) {
            // q[y][x'][o*K+kx], x' in [0, W+K-1) <-> input column x'-r; out[y][x][o] = sum_kx q[y][x+kx][o*K+kx].
            // One launch when a tile as wide as two kernels fits (q stays in the workgroup's LDS), else q goes through
            // memory and a second pass sums it.
            const bool never = net->sw.get("FYNHIP_NO_FUSED_WIDE_CONV") != nullptr, always = net->sw.get("FYNHIP_FORCE_FUSED_WIDE_CONV") != nullptr;
            MfmaLaunch one;
            bool have_one = false;
            if (!never) {
                SubConv sc = wide_subconv();
                sc.fuse_k = k; sc.fuse_cout = oc;
                sc.out_off_y = sc.out_off_x = out_v.pad;
                if (res_v) sc.res_off_y = sc.res_off_x = res_v->pad;
                padded = std::max((oc * k + 127) / 128 * 128, out_v.cp);
                scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
                bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
                try {
                    one = tune_mfma(net, sc, in_v, out_v, res_v, d.in_channels, oc * k, act(), res_relu, res_scale, scale_dev, bias_dev);
                    have_one = true;
                } catch (const Error& e) {
                    if (e.code != FYN_ERR_UNSUPPORTED) throw;   // (no tile fits)
                }
            }
            if (have_one && always) {
                fused = true;
                launch = one;
            } else {
                setup_two_pass_wide(in_v, out_v, res_v, res_relu, res_scale);
                if (have_one) {
                    // The one-launch form needs halo rows and columns, i.e. large tiles and few workgroups per CU; which
                    // form is faster depends on the image size and the storage type, so both are timed.
                    const char* at = net->sw.get("FYNHIP_AUTOTUNE");
                    bool pick = out_v.f16 != 0;
                    char key[160];
                    snprintf(key, sizeof(key), "folded:%d:%dx%d:%dx%d:k%d:cp%d:r%d:e%d%d", out_v.f16, d.in_channels, oc, oh, ow, k, in_v.cp,
                             res_v ? 1 : 0, clamp ? 1 : 0, frac_shift);
                    if (tune_cache_flag(net, key, &pick)) {
                    } else if (!(at && at[0] == '0')) {
                        float t1 = 1e30f, t2 = 1e30f;
                        for (int rep = 0; rep < 3; rep++) {
                            t1 = std::min(t1, time_launch(net, one, 10));
                            t2 = std::min(t2, time_calls(net, [&]() {
                                run_mfma(launch, net->stream);
                                launch_shift_reduce(sr, net->stream);
                            }, 10));
                        }
                        if (net->sw.get("FYNHIP_TUNE_VERBOSE")) fprintf(stderr, "[tune] folded kx taps: one launch %.1f us, two passes %.1f us\n", t1 * 1e3f, t2 * 1e3f);
                        pick = t1 < t2;
                        tune_cache_store_flag(net, key, pick);
                    }
                    if (pick) {
                        fused = true;
                        launch = one;
                        net->dev_free(qv.ptr);
                        qv.ptr = nullptr;
                    }
                }
            }
            // Third form: a workgroup walks down a strip of the image with the input rows in an LDS ring and the weights
            // in registers (conv_rows.hip); every input row is fetched once per strip and q never leaves the wave.
            if (!frac_shift && conv_rows_supported(k, in_v.cp, oc, out_v.f16 != 0) && out_v.cp == 4 && !net->sw.get("FYNHIP_NO_ROWS_WIDE_CONV"))
                setup_rows_wide(in_v, out_v, res_v, res_relu, res_scale);
        } else {
            SubConv sc;
            for (int ky = 0; ky < k; ky++)
                for (int kx = 0; kx < k; kx++) sc.taps.push_back(Tap{ky * dil, kx * dil, ky, kx});
            sc.span_y = sc.span_x = (k - 1) * dil + 1;
            sc.in_y0 = sc.in_x0 = in_v.pad - r * dil;
            sc.clamp = clamp ? 1 : 0;
            if (frac_shift) {
                // an ordinary strided convolution in the frame whose pixels are repeated 1/sourceStep times: taps one
                // virtual pixel apart, rows centred, columns centred except under the 3x3 kernel, whose shader samples
                // at -2, -1 and 0 steps (shaders/vanilla/fraconv3x3.frag:14-19 against fraconv5x5.frag:14-22)
                sc.in_shift = frac_shift - 1;
                sc.in_y0 = (in_v.pad << sc.in_shift) - r;
                sc.in_x0 = (in_v.pad << sc.in_shift) + ((k == 3) ? -2 : -r);
            }
            sc.in_stride = stride;
            if (k == 1 && stride > 1 && !frac_shift && !net->sw.get("FYNHIP_NO_SUBSAMPLED_STAGING")) {
                // strided pointwise layer: stage the pixels it reads and nothing between them
                sc.in_sub = stride;
                sc.in_stride = 1;
                sc.clamp = 0;   // (every position reads a pixel of the frame)
            }
            sc.npos_y = oh; sc.npos_x = ow;
            sc.out_step = 1;
            sc.out_off_y = sc.out_off_x = out_v.pad;
            if (res_v) sc.res_off_y = sc.res_off_x = res_v->pad;
            padded = std::max((oc + 127) / 128 * 128, out_v.cp);
            scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
            bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
            launch = tune_mfma(net, sc, in_v, out_v, res_v, d.in_channels, oc, act(), res_relu, res_scale, scale_dev, bias_dev);
            // the 16-position-fragment forms, each against the tuned launch of the general kernel: for wide fp16 layers the
            // one with 64-channel wave tiles first, then the 3x3 form, then the small-input form
            const bool same_storage = in_v.f16 == out_v.f16 && (!res_v || res_v->f16 == out_v.f16);
            // (tests: the K-resident form or nothing; a forced variant of the general kernel means the general kernel)
            const bool only_kr = net->sw.get("FYNHIP_FORCE_KR16_CONV") || net->sw.get("FYNHIP_FORCE_KSPLIT") || net->sw.get("FYNHIP_CONV_TILE") || net->sw.get("FYNHIP_CONV_KC") ||
                                 net->sw.get("FYNHIP_CONV_KC_MAX") || net->sw.get("FYNHIP_CONV_PD");
            if (!only_kr && !frac_shift && same_storage && conv_h16_supported(k, stride, dil, in_v.cp, oc, out_v.cp, out_v.f16 != 0) && d.in_channels == in_v.cp &&
                (!res_v || res_v->cp >= oc) && !net->sw.get("FYNHIP_NO_P16_CONV") && !net->sw.get("FYNHIP_NO_H16_CONV"))
                setup_h16(in_v, out_v, res_v, res_relu, res_scale);
            if (!only_kr && !p16 && !frac_shift && same_storage && !sc.in_sub && conv_p16_supported(k, stride, dil, in_v.cp, oc, out_v.cp, out_v.f16 != 0) &&
                d.in_channels == in_v.cp && (!res_v || (res_v->cp >= oc && res_v->cp % 8 == 0)) && !net->sw.get("FYNHIP_NO_P16_CONV"))
                setup_p16(in_v, out_v, res_v, res_relu, res_scale);
            if (!only_kr && !p16 && !frac_shift && same_storage && !res_v && conv_p16c4_supported(k, stride, dil, in_v.cp, oc, out_v.cp, out_v.f16 != 0) &&
                !net->sw.get("FYNHIP_NO_P16_CONV"))
                setup_c4(in_v, out_v);
            // few positions, many input channels: the whole reduction of a 4x4 tile resident in LDS instead of K-split launches
            if ((!p16 || (!h16 && !c4)) && !frac_shift && same_storage && (k == 1 || (k == 3 && (stride == 1 || stride == 2))) && dil == 1 && in_v.cp % 8 == 0 &&
                d.in_channels == in_v.cp && in_v.cp >= 16 && oc % 4 == 0 && oc >= 8 && out_v.cp >= oc && oh * ow <= 4096 && (!res_v || (res_v->cp >= out_v.cp && res_v->cp % 8 == 0)) &&
                !net->sw.get("FYNHIP_NO_P16_CONV") && !net->sw.get("FYNHIP_NO_KR16_CONV") && !net->sw.get("FYNHIP_FORCE_P16_CONV") &&
                // (a test that forces a variant of the general kernel wants the general kernel)
                !net->sw.get("FYNHIP_FORCE_KSPLIT") && !net->sw.get("FYNHIP_CONV_TILE") && !net->sw.get("FYNHIP_CONV_KC") && !net->sw.get("FYNHIP_CONV_KC_MAX") && !net->sw.get("FYNHIP_CONV_PD"))
                setup_kr16(in_v, out_v, res_v, res_relu, res_scale);
            // many positions, few input channels, 1x1: fragments straight from the tensor, no LDS
            if ((!p16 || kr16) && !frac_shift && same_storage && d.in_channels == in_v.cp && oc % 4 == 0 && oc >= 8 && oh * ow >= 256 &&
                conv_d16_supported(k, dil, in_v.cp, (in_v.cp + 31) / 32, oc, out_v.cp) && (!res_v || (res_v->cp >= out_v.cp && res_v->cp % 8 == 0)) &&
                !net->sw.get("FYNHIP_NO_P16_CONV") && !net->sw.get("FYNHIP_NO_D16_CONV") && !net->sw.get("FYNHIP_FORCE_P16_CONV") && !net->sw.get("FYNHIP_FORCE_KR16_CONV") &&
                !net->sw.get("FYNHIP_FORCE_KSPLIT") && !net->sw.get("FYNHIP_CONV_TILE") && !net->sw.get("FYNHIP_CONV_KC") && !net->sw.get("FYNHIP_CONV_KC_MAX") && !net->sw.get("FYNHIP_CONV_PD"))
                setup_d16(in_v, out_v, res_v, res_relu, res_scale);
            // the same kernel's K x K form for a first layer on at most four channels (3x3, 5x5, 7x7)
            if (!p16 && !frac_shift && !clamp && same_storage && oc % 4 == 0 && oc >= 8 && oh * ow >= 256 && conv_d16_small_supported(k, dil, in_v.cp, oc, out_v.cp) &&
                (!res_v || (res_v->cp >= out_v.cp && res_v->cp % 8 == 0)) && !net->sw.get("FYNHIP_NO_P16_CONV") && !net->sw.get("FYNHIP_NO_D16_CONV") && !net->sw.get("FYNHIP_FORCE_P16_CONV") &&
                !net->sw.get("FYNHIP_FORCE_KSPLIT") && !net->sw.get("FYNHIP_CONV_TILE") && !net->sw.get("FYNHIP_CONV_KC") && !net->sw.get("FYNHIP_CONV_KC_MAX") && !net->sw.get("FYNHIP_CONV_PD"))
                setup_d16(in_v, out_v, res_v, res_relu, res_scale);
        }
        if (direct) {
            scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
            bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
            dp.w = wdirect_dev; dp.scale = scale_dev; dp.bias = bias_dev;
        }
        set_up = true;
        setup_ranges();
        if (!block.empty()) pack();
    }
    void pack() {
        const float* bias = block.data();
        const float* w = bias + oc;
        const float* bn = w + (size_t)oc * k * k * d.in_channels;
        std::vector<float> sc, bi;
        fold_bn(bias, bn, oc, (d.flags & FYN_FLAG_POST_BATCHNORM) != 0, padded, sc, bi);
        reupload(net, scale_dev, sc);
        reupload(net, bias_dev, bi);
        if (direct) {
            const int cp = tout().v.cp, cin = d.in_channels;
            std::vector<float> wd((size_t)k * k * cin * cp, 0.f);
            for (int o = 0; o < oc; o++)
                for (int ky = 0; ky < k; ky++)
                    for (int kx = 0; kx < k; kx++)
                        for (int i = 0; i < cin; i++)
                            wd[(((size_t)ky * k + kx) * cin + i) * cp + o] = w[(((size_t)o * k + ky) * k + kx) * cin + i];
            reupload(net, wdirect_dev, wd);
        } else if (p16) {
            const float wmul = weight_prescale(w, (size_t)oc * k * k * d.in_channels);
            pp.acc_mul = pp2.acc_mul = 1.0f / wmul;
            if (c4) pack_c4(w, wmul);
            else if (d16) pack_d16(w, wmul);
            else if (kr16) pack_kr16(w, wmul);
            else if (h16) pack_h16(w, wmul);
            else pack_p16(w, wmul);
        } else if (wide && rows) {
            const float wmul = weight_prescale(w, (size_t)oc * k * k * d.in_channels);
            rp.acc_mul = 1.0f / wmul;
            pack_rows(w, wmul);
        } else if (wide) {
            const int cin = d.in_channels;
            const float wmul = weight_prescale(w, (size_t)oc * k * k * cin);
            // virtual weights Wv[o*K+kx][ky][0][ci] = W[o][ky][kx][ci]
            std::vector<float> wv((size_t)oc * k * k * cin);
            for (int o = 0; o < oc; o++)
                for (int ky = 0; ky < k; ky++)
                    for (int kx = 0; kx < k; kx++)
                        memcpy(&wv[(((size_t)(o * k + kx)) * k + ky) * cin], &w[(((size_t)o * k + ky) * k + kx) * cin], cin * sizeof(float));
            std::vector<float> ones(padded, 0.f), zeros(padded, 0.f);
            for (int i = 0; i < oc * k; i++) ones[i] = 1.f;
            if (!fused) {
                reupload(net, q_scale_dev, ones);
                reupload(net, q_bias_dev, zeros);
            }
            // the pre-scaling is undone on the way into the intermediate tensor (a power of two: no rounding), so that
            // fp16 storage holds the partial sums at their own magnitude
            launch.p.acc_mul = 1.0f / wmul;
            launch.red.acc_mul = 1.0f / wmul;
            sr.acc_mul = 1.0f;
            pack_mfma_weights(net, launch, wv.data(), k, wmul, 1);
        } else {
            const float wmul = weight_prescale(w, (size_t)oc * k * k * d.in_channels);
            launch.p.acc_mul = 1.0f / wmul;
            launch.red.acc_mul = 1.0f / wmul;
            pack_mfma_weights(net, launch, w, k, wmul);
        }
        if (edw_fused) pack_edw();
        have_weights = true;
        if (pj_fused) pack_two_sources();
        if (pj_into >= 0) static_cast<ConvLayer*>(net->layer(pj_into))->pack_two_sources();
    }
    // the weights once more, in the layout of the launch that also runs the depthwise layer behind this one
    void pack_edw() {
        if (block.empty()) return;
        const float* w = block.data() + oc;
        const float wmul = weight_prescale(w, (size_t)oc * k * k * d.in_channels);
        edw.acc_mul = 1.0f / wmul;
        pack_frag16(edw, edw_wpack_dev, w, wmul);
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without weights", d.name, d.number);
        if (pj_into >= 0 && net->fusion_on() && static_cast<ConvLayer*>(net->layer(pj_into))->pj_spread_ok) return;   // computed by the layer that adds it
        if (pj_fused && pj_spread_ok && net->fusion_on()) {
            ConvP16Params q = pj;   // (value-range words as the layer's own launch carries them)
            q.in_amax = tin(0).amax;
            q.in2_amax = net->layer(pj_layer_no)->tin(0).amax;
            q.out_amax = tout().amax;
            const int n = rows ? rp.nreset : (p16 ? pp.nreset : launch.p.nreset);
            unsigned* const* r = rows ? rp.reset : (p16 ? pp.reset : launch.p.reset);
            q.nreset = n;
            for (int i = 0; i < n; i++) q.reset[i] = r[i];
            if (launch_conv_kr16(q, 1, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        if (edw_fused && net->fusion_on()) {
            ConvP16Params q = edw;   // (value-range words as the layer's own launch carries them)
            q.in_amax = tin(0).amax;
            const int n = rows ? rp.nreset : (p16 ? pp.nreset : launch.p.nreset);
            unsigned* const* r = rows ? rp.reset : (p16 ? pp.reset : launch.p.reset);
            q.nreset = n;
            for (int i = 0; i < n; i++) q.reset[i] = r[i];
            if (launch_conv_e16dw(q, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        run(s);
    }
    void run(hipStream_t s) {
        if (rows) {
            if (launch_conv_rows(rp, tout().v.f16 != 0, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        if (p16 && (kr16 || d16) && dw_fused && net->fusion_on()) {
            if ((d16 ? launch_conv_d16(with_depthwise(), s) : launch_conv_kr16(with_depthwise(), k, s)) != 0) fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        if (p16 && (kr16 || d16) && bn_fused && net->fusion_on()) {
            if ((d16 ? launch_conv_d16(with_batchnorm(), s) : launch_conv_kr16(with_batchnorm(), k, s)) != 0) fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        if (p16) {
            if ((c4 ? launch_conv_p16c4(pp, k, s) : (d16 ? launch_conv_d16(pp, s) : (kr16 ? launch_conv_kr16(pp, k, s) : (h16 ? launch_conv_h16(pp, k, s) : launch_conv_p16(pp, s))))) != 0 ||
                (h16 && h16_two && launch_conv_h16(pp2, k, s) != 0))
                fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
            return;
        }
        if (direct) launch_conv_direct(dp, s);
        else if (run_mfma(launch, s) != 0)
            fail(FYN_ERR_DEVICE, "layer %s: convolution launch failed", d.name);
        if (wide && !fused) launch_shift_reduce(sr, s);
    }
    std::string info() const override {
        if (pj_into >= 0 && static_cast<ConvLayer*>(net->layer(pj_into))->pj_spread_ok)
            return "conv 1x1 projection (runs inside the launch of layer " + std::to_string(pj_into) + "; no launch of its own); apart: " + own_info();
        if (pj_fused && pj_spread_ok) {
            char buf[300];
            snprintf(buf, sizeof(buf), "conv_kr16 %s tile=%dx16(cout x pos) K-resident over two tensors, 4 waves split %d chunks (%d of them of the 1x1 projection %d, whose result the layer adds), blocks=%d lds=%zu; apart: ",
                     pj.f16 ? "f16" : "f16x2-split", 16 * pj.wm, pj.cin_chunks, pj.cin_chunks - pj.in2_chunk0, pj_layer_no, pj.pos_groups * pj.cout_blocks, conv_kr16_lds_bytes(pj, 1));
            return buf + own_info();
        }
        if (edw_fused)
            return "conv_e16dw " + std::string(edw.f16 ? "f16" : "f16x2-split") + " 1x1 and the depthwise 3x3 layer " + std::to_string(edw_dw_no) +
                   " behind it in one launch: a workgroup per 4x4 output positions and " + (edw.wm == 2 ? "16" : "64") + " expanded channels, blocks=" +
                   std::to_string(edw.tiles_x * edw.tiles_y * (edw.wm == 2 ? edw.mfrags : (edw.dw_cp + 63) / 64)) + "; apart: " + own_info();
        return own_info();
    }
    std::string own_info() const {
        const std::string mode = frac_shift ? "(fractional step 1/" + std::to_string(1 << (frac_shift - 1)) + ") " : (clamp ? "(edge-clamp) " : "");
        if (direct) return "conv_direct" + mode;
        if (rows) {
            char buf[200];
            snprintf(buf, sizeof(buf), "conv_rows %s(kx folded into cout, rows rolled through an LDS ring) strips=%d x %d row blocks of %d rows, lds=%zu",
                     tout().v.f16 ? "f16 " : "f16x2-split ", rp.strips, rp.row_blocks, rp.rows_per_block, conv_rows_lds_bytes(rp, tout().v.f16 != 0));
            return mode + buf;
        }
        if (p16 && c4) {
            char buf[220];
            snprintf(buf, sizeof(buf), "conv_p16c4 %s (tap pairs of a 4-channel pixel) tile=32x%d(cout x pos) th=%d tw=%d blocks=%d tiles=%d lds=%zu steps=%d",
                     pp.f16 ? "f16" : "f16x2-split", pp.tile_h * pp.tile_w * 4, pp.tile_h, pp.tile_w, pp.pos_groups * pp.cout_blocks, pp.tiles_x * pp.tiles_y * pp.cout_blocks,
                     conv_p16c4_lds_bytes(pp, k), c4_steps);
            return mode + buf;
        }
        if (p16 && d16) {
            char buf[360];
            snprintf(buf, sizeof(buf), "conv_d16 %s %s without LDS: %s, %d chunks in registers, %d fragments of 16 output channels, blocks=%d",
                     pp.f16 ? "f16" : "f16x2-split", (pp.tile_h ? "KxK on four-channel pixels (steps of eight taps)" : "1x1"), (pp.wm == 4 ? "a wave per 16 positions and fragment" : (std::to_string(pp.cout_blocks) + " workgroup(s) of 4 waves per 16 positions").c_str()),
                     pp.cin_chunks, pp.mfrags, (pp.npos_y * pp.npos_x + 16 * pp.wm - 1) / (16 * pp.wm) * pp.cout_blocks);
            if (dw_fused) return mode + buf + "; the depthwise 3x3 layer " + std::to_string(dw_layer_no) + " in front of it is computed by the waves themselves";
            if (bn_fused) return mode + buf + "; the batch-norm layer " + std::to_string(bn_layer_no) + " in front of it is applied on fetch";
            return mode + buf;
        }
        if (p16 && kr16) {
            char buf[220];
            snprintf(buf, sizeof(buf), "conv_kr16 %s tile=%dx%d(cout x pos) K-resident, 4 waves split %d chunks, blocks=%d lds=%zu steps=%d", pp.f16 ? "f16" : "f16x2-split",
                     16 * pp.wm, pp.tile_h * pp.tile_w, pp.cin_chunks, pp.pos_groups * pp.cout_blocks, conv_kr16_lds_bytes(pp, k), pp.cin_chunks / 4 * k * k);
            if (dw_fused) return mode + buf + "; the depthwise 3x3 layer " + std::to_string(dw_layer_no) + " in front of it is computed by the staging waves";
            if (bn_fused) return mode + buf + "; the batch-norm layer " + std::to_string(bn_layer_no) + " in front of it is applied while staging";
            return mode + buf;
        }
        if (p16 && h16) {
            char buf[220];
            snprintf(buf, sizeof(buf), "conv_h16 f16 tile=128x%d(cout x pos) waves=2x2 th=%d tw=%d blocks=%d tiles=%d lds=%zu steps=%d chunks=%d",
                     pp.tile_h * pp.tile_w * 2, pp.tile_h, pp.tile_w, pp.pos_groups * pp.cout_blocks, pp.tiles_x * pp.tiles_y * pp.cout_blocks,
                     conv_h16_lds_bytes(pp, k), k * k, pp.cin_chunks);
            std::string info = mode + buf;
            if (h16_two) {
                snprintf(buf, sizeof(buf), "; second launch from row %d: th=%d tw=%d blocks=%d tiles=%d lds=%zu", pp.npos_y, pp2.tile_h, pp2.tile_w,
                         pp2.pos_groups * pp2.cout_blocks, pp2.tiles_x * pp2.tiles_y * pp2.cout_blocks, conv_h16_lds_bytes(pp2, k));
                info += buf;
            }
            return info;
        }
        if (p16) {
            char buf[200];
            snprintf(buf, sizeof(buf), "conv_p16 %s tile=%dx%d(cout x pos) waves=%dx%d th=%d tw=%d blocks=%d tiles=%d lds=%zu steps=9 chunks=%d",
                     pp.f16 ? "f16" : (conv_p16_uses_fp8(pp) ? "f16+fp8-split" : "f16x2-split"), 32 * pp.wm, pp.tile_h * pp.tile_w * (4 / pp.wm), pp.wm, 4 / pp.wm, pp.tile_h, pp.tile_w, pp.pos_groups * pp.cout_blocks,
                     pp.tiles_x * pp.tiles_y * pp.cout_blocks, conv_p16_lds_bytes(pp), pp.cin_chunks);
            return mode + buf;
        }
        if (wide) return mode + (fused ? "wide-kernel(kx folded into cout, summed in the epilogue) " : "wide-kernel(kx folded into cout)+shift_reduce ") + mfma_info(launch);
        return mode + mfma_info(launch);
    }

    int k, dil, stride;
    int frac_shift = 0;   // fractional-step convolution: log2(1/sourceStep) + 1
    bool clamp = false, direct = false, wide = false, fused = false, rows = false, have_weights = false;
    int padded = 0;
    std::vector<float> block;
    MfmaLaunch launch;
    ConvRowsParams rp{};          // row-rolling form of the folded convolution (conv_rows.hip)
    void* rows_wpack_dev = nullptr;
    bool p16 = false;             // 16-position-fragment form of a 3x3 convolution (conv_p16.hip)
    bool c4 = false;              // ... its variant for inputs of at most four channels
    int c4_steps = 0;
    bool h16 = false;             // ... its fp16-storage form for wide layers (conv_h16.hip)
    bool kr16 = false;            // ... the K-resident form for layers with few positions (conv_p16.hip, conv_kr16_kernel)
    bool d16 = false;             // ... the LDS-free 1x1 form for many positions and few input channels (conv_d16.hip)
    // A depthwise 3x3 layer whose only reader is this 1x1 layer in the K-resident form can be computed inside this
    // layer's staging (fuse_depthwise_layers below): the fields of ConvP16Params that describe it
    // ... or, where this is a 1x1 layer and the depthwise layer its only reader, both run as one launch of
    // conv_e16dw_kernel (conv_d16.hip), with the weights packed once more in that kernel's layout
    bool edw_fused = false;
    int edw_dw_no = -1;
    ConvP16Params edw{};
    void* edw_wpack_dev = nullptr;
    bool dw_fused = false;
    int dw_layer_no = -1;
    ConvP16Params dw_fields{};
    ConvP16Params with_depthwise() const {
        ConvP16Params q = pp;
        q.dw_in = dw_fields.dw_in; q.dw_w = dw_fields.dw_w; q.dw_scale = dw_fields.dw_scale; q.dw_bias = dw_fields.dw_bias;
        q.dw_hp = dw_fields.dw_hp; q.dw_wp = dw_fields.dw_wp; q.dw_cp = dw_fields.dw_cp;
        q.dw_y0 = dw_fields.dw_y0; q.dw_x0 = dw_fields.dw_x0; q.dw_stride = dw_fields.dw_stride; q.dw_act = dw_fields.dw_act;
        return q;
    }
    // A batch-norm layer in front of this layer applied while the K-resident form stages its tile or the LDS-free 1x1
    // form fetches its fragments (fuse_batchnorm_layers below): the layer's input tensor -- same geometry as its output -- and its scale / bias arrays.
    bool bn_fused = false;
    int bn_layer_no = -1;
    const void* bn_in = nullptr;
    const float *bn_mul = nullptr, *bn_add = nullptr;
    ConvP16Params with_batchnorm() const {
        ConvP16Params q = pp;
        q.in = bn_in; q.in_mul = bn_mul; q.in_add = bn_add;
        q.in_amax = nullptr;   // (the batch-norm layer keeps no value-range word: its readers stage unscaled either way)
        return q;
    }
    bool takes_batchnorm() const {
        if (!p16 || dw_fused || edw_fused || pj_fused || pj_into >= 0 || pp.in_amax) return false;
        if (d16) return k == 1;
        if (!kr16) return false;
        ConvP16Params t = pp;   // (a variant of the K-resident form that applies the layer: 1x1 on 4x4 tiles)
        t.in_mul = t.in_add = scale_dev;
        return conv_kr16_lds_bytes(t, k) != 0;
    }
    // A 1x1 projection whose result this 1x1 layer adds (its residual input) computed in the layer's own launch, as one
    // reduction over two tensors (fuse_projection_layers below): the rows of both weight matrices carry their layers'
    // folded scales, the bias is the sum of both, and the projection's tensor is never written.
    bool pj_fused = false;
    bool pj_spread_ok = true;   // set with the weights (pack_two_sources): false keeps the two launches
    int pj_layer_no = -1;   // the projection this layer computes
    int pj_into = -1;       // on the projection: the layer that computes it
    ConvP16Params pj{};
    void* pj_wpack_dev = nullptr;
    float *pj_scale_dev = nullptr, *pj_bias_dev = nullptr;
    void pack_two_sources() {
        ConvLayer* P = static_cast<ConvLayer*>(net->layer(pj_layer_no));
        if (block.empty() || P->block.empty()) return;
        const int c1 = d.in_channels, c2 = P->d.in_channels, n1 = pj.in2_chunk0, fm_n = pj.wm, npl = pj.f16 ? 1 : 2, steps = pj.cin_chunks / 4;
        const float *b1 = block.data(), *w1 = b1 + oc, *bn1 = w1 + (size_t)oc * c1;
        const float *b2 = P->block.data(), *w2 = b2 + oc, *bn2 = w2 + (size_t)oc * c2;
        std::vector<float> s1, o1, s2, o2;
        fold_bn(b1, bn1, oc, (d.flags & FYN_FLAG_POST_BATCHNORM) != 0, oc, s1, o1);
        fold_bn(b2, bn2, oc, (P->d.flags & FYN_FLAG_POST_BATCHNORM) != 0, oc, s2, o2);
        // (batch-norm on the residual: the layer's scale multiplies what it adds, convlayerbase's residual variant)
        const bool rs = (d.flags & FYN_FLAG_BATCHNORM_ON_RESIDUAL) && (d.flags & FYN_FLAG_POST_BATCHNORM);
        std::vector<float> wa((size_t)oc * c1), wb((size_t)oc * c2), ones(padded, 0.f), bias(padded, 0.f);
        float mx = 0.f, row_lo = 0.f;
        for (int o = 0; o < oc; o++) {
            const float r2 = rs ? s1[o] * s2[o] : s2[o];
            float row = 0.f;
            for (int i = 0; i < c1; i++) row = std::max(row, std::fabs(wa[(size_t)o * c1 + i] = w1[(size_t)o * c1 + i] * s1[o]));
            for (int i = 0; i < c2; i++) row = std::max(row, std::fabs(wb[(size_t)o * c2 + i] = w2[(size_t)o * c2 + i] * r2));
            mx = std::max(mx, row);
            if (row > 0.f) row_lo = row_lo == 0.f ? row : std::min(row_lo, row);
            ones[o] = 1.f;
            bias[o] = o1[o] + (rs ? s1[o] * o2[o] : o2[o]);
        }
        // The folded scales ride on the weights and one power of two brings the largest of them to the top of fp16's
        // range: a row 2^16 times smaller than the largest still keeps 20 bits (11 in a single fp16 plane); beyond that
        // spread the pair runs as two launches, where each layer's scale multiplies its fp32 sum.
        pj_spread_ok = !(row_lo > 0.f) || mx <= row_lo * 65536.f;
        const float wmul = weight_prescale(&mx, 1);
        pj.acc_mul = 1.0f / wmul;
        std::vector<uint16_t> pack((size_t)pj.cout_blocks * 4 * steps * fm_n * npl * 64 * 8, 0);
        for (int cb = 0; cb < pj.cout_blocks; cb++)
            for (int wv = 0; wv < 4; wv++)
                for (int st = 0; st < steps; st++) {
                    const int chunk = wv + 4 * st;
                    const bool second = chunk >= n1;
                    const float* src = second ? wb.data() : wa.data();
                    const int cn = second ? c2 : c1, cbase = (second ? chunk - n1 : chunk) * 32;
                    for (int fm = 0; fm < fm_n; fm++) {
                        uint16_t* base = pack.data() + ((((size_t)(cb * 4 + wv) * steps + st) * fm_n + fm) * npl) * 64 * 8;
                        for (int lane = 0; lane < 64; lane++) {
                            const int o = (cb * fm_n + fm) * 16 + (lane & 15);
                            if (o >= oc) continue;
                            for (int j = 0; j < 8; j++) {
                                const int ci = cbase + 8 * (lane >> 4) + j;
                                if (ci >= cn) continue;
                                const float v = src[(size_t)o * cn + ci] * wmul;
                                const uint16_t hi = f2h_bits(v);
                                base[(size_t)lane * 8 + j] = hi;
                                if (npl == 2) base[(size_t)(64 + lane) * 8 + j] = f2h_bits(v - h2f(hi));
                            }
                        }
                    }
                }
        reupload(net, pj_scale_dev, ones);
        reupload(net, pj_bias_dev, bias);
        FYN_HIP(hipStreamSynchronize(net->stream));
        FYN_HIP(hipMemcpyAsync(pj_wpack_dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
        FYN_HIP(hipStreamSynchronize(net->stream));
    }
    bool takes_depthwise() const {
        // (not a layer that already runs the depthwise layer behind it: one launch cannot do both)
        return p16 && !edw_fused && ((kr16 && pp.tile_h == 4 && pp.tile_w == 4) || d16) && k == 1 && stride == 1 && !clamp && !pp.in_amax && !pp.in_clamp;
    }
    int launch_with_depthwise(const ConvP16Params& q, hipStream_t s) const { return d16 ? launch_conv_d16(q, s) : launch_conv_kr16(q, 1, s); }
    int launch_own(hipStream_t s) const { return d16 ? launch_conv_d16(pp, s) : launch_conv_kr16(pp, 1, s); }
    bool h16_two = false;         // ...... as two launches on two bands of rows (pp, pp2)
    ConvP16Params pp{}, pp2{};
    void* p16_wpack_dev = nullptr;
    ConvDirectParams dp{};
    ShiftReduceParams sr{};
    TView qv{};
    float *q_scale_dev = nullptr, *q_bias_dev = nullptr;
    float *scale_dev = nullptr, *bias_dev = nullptr, *wdirect_dev = nullptr;
};

// =============================================================================================
// Depthwise 3x3 convolution
// =============================================================================================
class DwConvLayer : public Layer {
  public:
    DwConvLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        dil = d.dilation[0] > 0 ? d.dilation[0] : 1;
        stride = d.downsample[0] > 0 ? d.downsample[0] : 1;
        if (d.out_channels != d.in_channels)
            fail(FYN_ERR_UNSUPPORTED, "depthwise channel multiplier %d/%d not supported (%s)", d.out_channels, d.in_channels, d.name);
        oc = d.out_channels;
        oh = d.height / stride;
        ow = d.width / stride;
    }
    size_t weight_floats() const override {
        return (size_t)oc + 9 * (size_t)d.in_channels + ((d.flags & FYN_FLAG_POST_BATCHNORM) ? 2 * (size_t)oc : 0);
    }
    void load_weights(const float* blk) override {
        block.assign(blk, blk + weight_floats());
        if (set_up) pack();
    }
    void setup() override {
        p.in = tin(0).v; p.out = tout().v;
        p.res = (d.flags & FYN_FLAG_RESIDUAL_INPUT) ? tin(1).v : TView{};
        p.dil = dil; p.stride = stride;
        p.res_relu = (d.flags & FYN_FLAG_RELU_ON_RESIDUAL) ? 1 : 0;
        p.res_scale = ((d.flags & FYN_FLAG_BATCHNORM_ON_RESIDUAL) && (d.flags & FYN_FLAG_POST_BATCHNORM)) ? 1 : 0;
        p.no_strips = net->sw.on("FYNHIP_NO_DW_STRIPS") ? 1 : 0;
        p.act = act();
        const int cp = p.out.cp;
        w_dev = static_cast<float*>(net->dev_alloc(9 * (size_t)cp * sizeof(float)));
        scale_dev = static_cast<float*>(net->dev_alloc(cp * sizeof(float)));
        bias_dev = static_cast<float*>(net->dev_alloc(cp * sizeof(float)));
        p.w = w_dev; p.scale = scale_dev; p.bias = bias_dev;
        set_up = true;
        if (!block.empty()) pack();
    }
    void pack() {
        const int cp = tout().v.cp;
        const float* bias = block.data();
        const float* w = bias + oc;  // [(i*9 + ky*3+kx)] (gpu/deep/deepdwconvlayerbase.cpp:242, multiplier 1)
        const float* bn = w + 9 * (size_t)d.in_channels;
        std::vector<float> sc, bi, wd(9 * (size_t)cp, 0.f);
        fold_bn(bias, bn, oc, (d.flags & FYN_FLAG_POST_BATCHNORM) != 0, cp, sc, bi);
        for (int i = 0; i < oc; i++)
            for (int t = 0; t < 9; t++) wd[(size_t)t * cp + i] = w[(size_t)i * 9 + t];
        reupload(net, w_dev, wd);
        reupload(net, scale_dev, sc);
        reupload(net, bias_dev, bi);
        have_weights = true;
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without weights", d.name, d.number);
        if (fused_into >= 0 && net->fusion_on()) return;   // computed inside the pointwise layer behind it
        launch_dwconv3x3(p, s);
    }
    std::string info() const override {
        return fused_into >= 0 ? "dwconv3x3 (runs inside the launch of layer " + std::to_string(fused_into) + "; no launch of its own)" : "dwconv3x3";
    }
    int fused_into = -1;
    int dil, stride;
    bool have_weights = false;
    std::vector<float> block;
    DwConvParams p{};
    float *w_dev = nullptr, *scale_dev = nullptr, *bias_dev = nullptr;
};

// Depthwise 3x3 -> pointwise 1x1 (the second half of an inverted-residual block) as one launch.  Where the pointwise
// layer runs the K-resident form on 4x4 tiles and is the depthwise layer's only reader, its staging waves can compute
// the depthwise layer for the tile instead of fetching that layer's output (conv_kr16_kernel, DWS): every workgroup of
// a tile -- one per block of 16 or 32 output channels -- repeats the depthwise arithmetic for its tile, which costs
// less than a launch as long as the blocks are few.  Both ways are timed; the depthwise layer's tensor is not written
// when the fused way is taken, so the fusion is tied to buffer reuse (a caller who switches reuse off wants every
// layer's tensor) and is left out of passes that time or dump single layers.
void fuse_depthwise_layers(Net* net) {
    if (net->sw.get("FYNHIP_NO_DW_FUSION") || !net->reuse_buffers) return;
    std::map<int, int> readers;
    for (auto& kv : net->layers)
        for (int t : kv.second->in)
            if (t >= 0) readers[t]++;
    const char* at = net->sw.get("FYNHIP_AUTOTUNE");
    // First the other half of the block: a 1x1 layer (expand) whose only reader is the depthwise layer.  Every expanded
    // channel depends on the 1x1 layer's input only, so a workgroup can compute the window of the expanded tensor that
    // its tile of the depthwise layer needs (conv_e16dw_kernel); the expanded tensor is then never written.
    for (auto& kv : net->layers) {
        if (net->sw.get("FYNHIP_NO_EDW_FUSION")) break;
        DwConvLayer* dw = dynamic_cast<DwConvLayer*>(kv.second.get());
        if (!dw || dw->dil != 1 || (dw->stride != 1 && dw->stride != 2) || dw->p.res.ptr || dw->p.in.cp % 8 != 0 || dw->p.in.cp != dw->p.out.cp || dw->p.in.f16 != dw->p.out.f16)
            continue;
        const Tensor& t = net->tensors[dw->in[0]];
        if (t.producer < 0 || t.locked || readers[dw->in[0]] != 1) continue;
        ConvLayer* ex = dynamic_cast<ConvLayer*>(net->layer(t.producer));
        if (!ex || ex->k != 1 || ex->stride != 1 || ex->dil != 1 || ex->clamp || ex->frac_shift || ex->direct || (ex->d.flags & FYN_FLAG_RESIDUAL_INPUT)) continue;
        const TView& in_v = ex->tin(0).v;
        // The launch writes the depthwise layer's output in the 1x1 layer's place in the order, i.e. earlier than the
        // buffer was handed over for: every other tenant of that buffer must be through by then -- neither read at or
        // behind the 1x1 layer (its own input included: the launch reads it while it writes) nor produced between the two.
        bool early_ok = true;
        for (const Tensor& o : net->tensors)
            if (&o != &net->tensors[dw->out] && o.buffer == net->tensors[dw->out].buffer && o.producer < dw->d.number &&
                std::max(o.last_reader, o.producer) >= ex->d.number)
                early_ok = false;
        if (!early_ok) continue;
        if (in_v.f16 != dw->p.out.f16 || ex->d.in_channels != in_v.cp || ex->tout().v.cp != dw->p.in.cp || ex->oc % 4 != 0 ||
            !conv_e16dw_supported(in_v.cp, (in_v.cp + 31) / 32, dw->stride))
            continue;
        ConvP16Params q{};
        q.in = in_v.ptr; q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = 1; q.in_y0 = q.in_x0 = in_v.pad;
        q.cin_chunks = (in_v.cp + 31) / 32;
        q.mfrags = (ex->oc + 15) / 16;
        q.f16 = in_v.f16 ? 1 : 0;
        q.scale = ex->scale_dev; q.bias = ex->bias_dev;
        q.acc_mul = 1.f;
        q.act = ex->act();
        q.dw_hp = ex->oh; q.dw_wp = ex->ow;
        q.out = dw->p.out.ptr; q.out_wp = dw->p.out.wp(); q.out_cp = dw->p.out.cp; q.out_off_y = q.out_off_x = dw->p.out.pad;
        q.npos_y = dw->p.out.h; q.npos_x = dw->p.out.w;
        q.tiles_x = (q.npos_x + 3) / 4; q.tiles_y = (q.npos_y + 3) / 4;
        q.dw_w = dw->w_dev; q.dw_scale = dw->scale_dev; q.dw_bias = dw->bias_dev;
        q.dw_cp = dw->p.in.cp; q.dw_stride = dw->stride; q.dw_act = dw->p.act;
        const size_t halves = (size_t)q.mfrags * q.cin_chunks * (q.f16 ? 1 : 2) * 64 * 8;
        void* const wp = net->dev_alloc(halves * 2, true);
        q.wpack = wp;
        bool pick = true;
        char key[200];
        snprintf(key, sizeof(key), "edw:%d:%dto%d:%dx%d:s%d", q.f16, in_v.cp, ex->oc, ex->oh, ex->ow, dw->stride);
        // (q.wm = 2: a workgroup per 16 expanded channels instead of 64, for layers with few tiles; by rule when nothing is timed)
        q.wm = (q.tiles_x * q.tiles_y * ((q.dw_cp + 63) / 64) < 128) ? 2 : 0;
        if (const char* e = net->sw.get("FYNHIP_EDW_NARROW")) q.wm = atoi(e) ? 2 : 0;
        int cached[3] = {0, 0, 0};
        if (net->sw.get("FYNHIP_FORCE_DW_FUSION") || net->sw.get("FYNHIP_EDW_NARROW")) {
        } else if (tune_cache_triple(net, key, cached)) {
            pick = cached[0] != 0;
            q.wm = cached[1];
        } else if (!(at && at[0] == '0')) {
            float t_fused = 1e30f, t_two = 1e30f;
            int best_wm = 0;
            for (int rep = 0; rep < 3; rep++) {
                for (int wm : {0, 2}) {
                    ConvP16Params c = q;
                    c.wm = wm;
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_e16dw(c, net->stream) != 0) fail(FYN_ERR_DEVICE, "1x1 + depthwise convolution launch failed while tuning");
                    }, 10);
                    if (t < t_fused) { t_fused = t; best_wm = wm; }
                }
                t_two = std::min(t_two, time_calls(net, [&]() {
                    ex->run(net->stream);
                    launch_dwconv3x3(dw->p, net->stream);
                }, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] 1x1 %d to %d at %dx%d + depthwise 3x3 (step %d): one launch (blocks of %d channels) %.1f us, two %.1f us\n", in_v.cp, ex->oc, ex->oh,
                        ex->ow, dw->stride, best_wm == 2 ? 16 : 64, t_fused * 1e3f, t_two * 1e3f);
            // (a near tie goes to the single launch: it leaves the expanded tensor unwritten, which a timing loop that
            // finds everything in the caches does not reward)
            pick = t_fused < t_two * 1.05f;
            q.wm = best_wm;
            tune_cache_store_triple(net, key, pick ? 1 : 0, best_wm, 0);
        }
        if (!pick) {
            net->dev_free(wp);
            continue;
        }
        ex->edw = q;
        ex->edw_wpack_dev = wp;
        ex->edw_fused = true;
        ex->edw_dw_no = dw->d.number;
        dw->fused_into = ex->d.number;
        ex->pack_edw();
    }
    for (auto& kv : net->layers) {
        ConvLayer* pw = dynamic_cast<ConvLayer*>(kv.second.get());
        if (!pw || !pw->takes_depthwise()) continue;
        const Tensor& t = net->tensors[pw->in[0]];
        if (t.producer < 0 || t.locked || readers[pw->in[0]] != 1) continue;
        DwConvLayer* dw = dynamic_cast<DwConvLayer*>(net->layer(t.producer));
        if (dw && dw->fused_into >= 0) continue;   // (already part of the 1x1 layer in front of it)
        if (!dw || dw->dil != 1 || (dw->stride != 1 && dw->stride != 2) || dw->p.res.ptr || dw->p.in.cp % 8 != 0 || dw->p.in.cp != dw->p.out.cp ||
            dw->p.in.f16 != dw->p.out.f16 || dw->p.out.f16 != pw->pp.f16 || dw->p.out.cp != pw->pp.in_cp)
            continue;
        // The launch reads the depthwise layer's input in the 1x1 layer's place in the order, i.e. later than the buffer
        // was kept for: no tensor produced behind the depthwise layer up to and including the 1x1 layer (whose output
        // the launch writes while it reads) may live in that buffer.
        bool late_ok = true;
        for (const Tensor& o : net->tensors)
            if (&o != &net->tensors[dw->in[0]] && o.buffer == net->tensors[dw->in[0]].buffer && o.producer > dw->d.number &&
                o.producer <= pw->d.number)
                late_ok = false;
        if (!late_ok) continue;
        ConvP16Params& f = pw->dw_fields;
        f.dw_in = dw->p.in.ptr; f.dw_w = dw->w_dev; f.dw_scale = dw->scale_dev; f.dw_bias = dw->bias_dev;
        f.dw_hp = dw->p.in.hp(); f.dw_wp = dw->p.in.wp(); f.dw_cp = dw->p.in.cp;
        f.dw_y0 = f.dw_x0 = dw->p.in.pad - 1;
        f.dw_stride = dw->stride; f.dw_act = dw->p.act;
        const ConvP16Params q = pw->with_depthwise();
        if (pw->d16 ? !conv_d16_dw_supported(q.cin_chunks, q.dw_stride) : (conv_kr16_lds_bytes(q, 1) == 0 || conv_kr16_lds_bytes(q, 1) > 160 * 1024)) continue;
        bool pick = true;
        char key[200];
        snprintf(key, sizeof(key), "dwpw:%d:%dx%dx%d:s%d:to%d:fm%d:d%d", q.f16, dw->p.in.cp, dw->p.in.h, dw->p.in.w, dw->stride, pw->oc, q.wm, pw->d16 ? 1 : 0);
        if (net->sw.get("FYNHIP_FORCE_DW_FUSION")) {
        } else if (tune_cache_flag(net, key, &pick)) {
        } else if (!(at && at[0] == '0')) {
            float t_fused = 1e30f, t_two = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                t_fused = std::min(t_fused, time_calls(net, [&]() {
                    if (pw->launch_with_depthwise(q, net->stream) != 0) fail(FYN_ERR_DEVICE, "1x1 convolution with a depthwise layer in front: launch failed while tuning");
                }, 10));
                t_two = std::min(t_two, time_calls(net, [&]() {
                    launch_dwconv3x3(dw->p, net->stream);
                    if (pw->launch_own(net->stream) != 0) fail(FYN_ERR_DEVICE, "1x1 convolution launch failed while tuning");
                }, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] depthwise 3x3 (step %d) on %d channels at %dx%d + 1x1 to %d: one launch %.1f us, two %.1f us\n", dw->stride, dw->p.in.cp,
                        dw->p.in.h, dw->p.in.w, pw->oc, t_fused * 1e3f, t_two * 1e3f);
            pick = t_fused < t_two;
            tune_cache_store_flag(net, key, pick);
        }
        if (!pick) continue;
        pw->dw_fused = true;
        pw->dw_layer_no = dw->d.number;
        dw->fused_into = pw->d.number;
    }
}

// The projection that layer `c` could compute itself (fuse_projection_layers below), by the graph alone: `c` a 1x1 layer
// without step that adds, unactivated, the result of a 1x1 layer nothing else reads.
static ConvLayer* projection_of(Net* net, ConvLayer* c) {
    if (!c || c->k != 1 || c->stride != 1 || c->dil != 1 || c->clamp || c->frac_shift || c->direct || !(c->d.flags & FYN_FLAG_RESIDUAL_INPUT) ||
        (c->d.flags & FYN_FLAG_RELU_ON_RESIDUAL) || c->in.size() < 2 || c->in[1] < 0 || c->in[0] == c->in[1])
        return nullptr;
    const Tensor& rt = net->tensors[c->in[1]];
    if (rt.producer < 0 || rt.locked) return nullptr;
    int readers = 0;
    for (auto& kv : net->layers)
        for (int t : kv.second->in) readers += t == c->in[1];
    if (readers != 1) return nullptr;
    ConvLayer* pr = dynamic_cast<ConvLayer*>(net->layer(rt.producer));
    if (!pr || pr->k != 1 || pr->dil != 1 || pr->clamp || pr->frac_shift || pr->direct || (pr->d.flags & FYN_FLAG_RESIDUAL_INPUT) || pr->oc != c->oc ||
        pr->d.number >= c->d.number || pr->in.empty() || pr->in[0] < 0)
        return nullptr;
    return pr;
}
// Before buffers are assigned: the input of such a projection stays whole until the layer that may compute it has run
// (a few more buffers in networks with such pairs, whether the pair is joined in the end or not).
void keep_projection_inputs(Net* net) {
    if (net->sw.get("FYNHIP_NO_PROJECTION_FUSION") || !net->reuse_buffers) return;
    for (auto& kv : net->layers) {
        ConvLayer* c = dynamic_cast<ConvLayer*>(kv.second.get());
        ConvLayer* pr = projection_of(net, c);
        if (!pr) continue;
        Tensor& x2 = net->tensors[pr->in[0]];
        x2.last_reader = std::max(x2.last_reader, c->d.number);
    }
}
// A 1x1 projection (a residual block's shortcut convolution) whose only reader adds it to its own 1x1 convolution: both
// are sums over channels at the same output position, so they run as ONE reduction over two tensors on the K-resident
// form -- the projection's chunks behind the layer's own, each weight row carrying its layer's folded scale -- and the
// projection's tensor is never written.  Conditions: both 1x1 without dilation on tensors of one storage type, the same
// activation on fetch, no activation on the residual, the projection's input still whole when the reader runs, and a
// compiled variant for the joint chunk count; timed against the two launches.
void fuse_projection_layers(Net* net) {
    if (net->sw.get("FYNHIP_NO_PROJECTION_FUSION") || net->sw.get("FYNHIP_NO_P16_CONV") || net->sw.get("FYNHIP_NO_KR16_CONV") || !net->reuse_buffers) return;
    const char* at = net->sw.get("FYNHIP_AUTOTUNE");
    for (auto& kv : net->layers) {
        ConvLayer* c = dynamic_cast<ConvLayer*>(kv.second.get());
        ConvLayer* pr = projection_of(net, c);
        if (!pr || c->dw_fused || c->edw_fused || c->bn_fused || pr->dw_fused || pr->edw_fused || pr->bn_fused || pr->pj_fused || pr->pj_into >= 0) continue;
        const Tensor& rt = net->tensors[c->in[1]];
        const Act a1 = c->act(), a2 = pr->act();
        if (a1.kind != a2.kind || a1.lo != a2.lo || a1.hi != a2.hi || a1.leak != a2.leak) continue;
        const TView& v1 = c->tin(0).v;
        const TView& v2 = pr->tin(0).v;
        const TView& ov = c->tout().v;
        Tensor& x2 = net->tensors[pr->in[0]];
        if (v1.f16 != ov.f16 || v2.f16 != ov.f16 || rt.v.f16 != ov.f16 || c->d.in_channels != v1.cp || pr->d.in_channels != v2.cp || v1.cp % 8 != 0 || v2.cp % 8 != 0 ||
            v1.cp < 8 || v2.cp < 8 || c->oc % 4 != 0 || c->oc < 8 || ov.cp < c->oc || c->oh * c->ow > 4096)
            continue;
        bool live = true;   // (the projection's input must still hold its values when the reader runs)
        for (const Tensor& o : net->tensors)
            if (&o != &x2 && o.buffer == x2.buffer && o.producer > pr->d.number && o.producer <= c->d.number) live = false;
        if (!live) continue;
        const int n1 = (v1.cp + 31) / 32, n2 = (v2.cp + 31) / 32;
        ConvP16Params q{};
        q.in = v1.ptr; q.out = ov.ptr;
        q.in_hp = v1.hp(); q.in_wp = v1.wp(); q.in_cp = v1.cp;
        q.stride = 1; q.in_y0 = q.in_x0 = v1.pad;
        q.in2 = v2.ptr; q.in2_hp = v2.hp(); q.in2_wp = v2.wp(); q.in2_cp = v2.cp;
        q.in2_stride = pr->stride; q.in2_y0 = q.in2_x0 = v2.pad; q.in2_chunk0 = n1;
        q.npos_y = c->oh; q.npos_x = c->ow;
        q.out_wp = ov.wp(); q.out_cp = ov.cp; q.out_off_y = q.out_off_x = ov.pad;
        q.f16 = ov.f16 ? 1 : 0;
        q.acc_mul = 1.f;
        q.act = a1;
        q.tile_h = q.tile_w = 4;
        q.tiles_x = (c->ow + 3) / 4; q.tiles_y = (c->oh + 3) / 4;
        q.rcp_tiles_x = 1.0f / (float)q.tiles_x;
        q.pos_groups = q.tiles_x * q.tiles_y;
        // (the last pixel either tensor is read at lies inside it)
        if ((c->oh - 1) * pr->stride + v2.pad >= v2.hp() || (c->ow - 1) * pr->stride + v2.pad >= v2.wp()) continue;
        // the joint chunk count, rounded up to the next one a variant is compiled for (the chunks behind both tensors read as zero)
        int chunks = 0;
        for (int n = (n1 + n2 + 3) / 4 * 4; n <= 64 && !chunks; n += 4) {
            ConvP16Params t = q;
            t.cin_chunks = n; t.wm = 1; t.cout_blocks = (c->oc + 15) / 16; t.mfrags = t.cout_blocks;
            if (conv_kr16_lds_bytes(t, 1) != 0) chunks = n;
        }
        if (!chunks) continue;
        q.cin_chunks = chunks;
        std::vector<ConvP16Params> cands;
        for (int fm : {1, 2}) {
            if (fm == 2 && c->oc % 32 != 0 && c->oc % 32 <= 16) continue;
            ConvP16Params t = q;
            t.wm = fm;
            t.cout_blocks = (c->oc + 16 * fm - 1) / (16 * fm);
            t.mfrags = t.cout_blocks * fm;
            const size_t lds = conv_kr16_lds_bytes(t, 1);
            if (lds == 0 || lds > 160 * 1024 || (long long)t.pos_groups * t.cout_blocks > 65535) continue;
            cands.push_back(t);
        }
        if (cands.empty()) continue;
        const size_t halves = (size_t)((c->oc + 31) / 32 * 2) * 4 * (chunks / 4) * (q.f16 ? 1 : 2) * 64 * 8;
        void* const wp = net->dev_alloc(halves * 2, true);
        float* const sc = static_cast<float*>(net->dev_alloc(c->padded * sizeof(float), true));
        float* const bi = static_cast<float*>(net->dev_alloc(c->padded * sizeof(float), true));
        for (ConvP16Params& t : cands) { t.wpack = wp; t.scale = sc; t.bias = bi; }
        int pick = 0;
        bool win = true;
        char key[200];
        snprintf(key, sizeof(key), "pj:%d:%dand%dto%d:%dx%d:s%d", q.f16, v1.cp, v2.cp, c->oc, c->oh, c->ow, pr->stride);
        int cached[3] = {0, 0, 0};
        if (net->sw.get("FYNHIP_FORCE_PROJECTION_FUSION")) {
        } else if (tune_cache_triple(net, key, cached)) {
            win = cached[0] != 0;
            for (size_t i = 0; i < cands.size(); i++)
                if (cands[i].wm == cached[1]) pick = (int)i;
        } else if (!(at && at[0] == '0')) {
            float t_fused = 1e30f, t_two = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() {
                        if (launch_conv_kr16(cands[i], 1, net->stream) != 0) fail(FYN_ERR_DEVICE, "1x1 convolution over two tensors: launch failed while tuning");
                    }, 10);
                    if (t < t_fused) { t_fused = t; pick = (int)i; }
                }
                t_two = std::min(t_two, time_calls(net, [&]() {
                    pr->run(net->stream);
                    c->run(net->stream);
                }, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] 1x1 on %d channels + 1x1 projection on %d (step %d) to %d at %dx%d: one launch %.1f us, two %.1f us\n", v1.cp, v2.cp, pr->stride, c->oc,
                        c->oh, c->ow, t_fused * 1e3f, t_two * 1e3f);
            win = t_fused < t_two;
            tune_cache_store_triple(net, key, win ? 1 : 0, cands[pick].wm, 0);
        }
        if (!win) {
            net->dev_free(wp); net->dev_free(sc); net->dev_free(bi);
            continue;
        }
        c->pj = cands[pick];
        c->pj_wpack_dev = wp; c->pj_scale_dev = sc; c->pj_bias_dev = bi;
        c->pj_fused = true;
        c->pj_layer_no = pr->d.number;
        pr->pj_into = c->d.number;
        x2.last_reader = std::max(x2.last_reader, c->d.number);   // (its value-range word is cleared behind its last reader)
        c->pack_two_sources();
    }
}

// =============================================================================================
// Transposed convolution, stride 2, K in {2,3}: one MFMA sub-convolution per output parity
// =============================================================================================
class TransConvLayer : public Layer {
  public:
    TransConvLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        k = d.kernel;
        // gpu/gpulayerfactory.cpp:410-411
        if (k != 2 && k != 3) fail(FYN_ERR_UNSUPPORTED, "Transpose convolution is currently only implemented for 2x2 and 3x3 kernels");
        if (d.upsample[0] != 2 || d.upsample[1] != 2) fail(FYN_ERR_UNSUPPORTED, "Transpose convolution requires upsample(2) (%s)", d.name);
        if (d.flags & FYN_FLAG_RESIDUAL_INPUT) fail(FYN_ERR_UNSUPPORTED, "Residual input is not supported on transpose convolution (%s)", d.name);
        crop = d.transconv_crop;
        if (crop < 0 || crop >= k) fail(FYN_ERR_INVALID, "invalid transconv_crop %d (%s)", crop, d.name);
        oc = d.out_channels;
        oh = 2 * d.height + k - 2 - crop;  // gpu/deep/deeptiler.cpp:71-74
        ow = 2 * d.width + k - 2 - crop;
    }
    size_t weight_floats() const override {
        return (size_t)oc + (size_t)oc * k * k * d.in_channels + ((d.flags & FYN_FLAG_POST_BATCHNORM) ? 2 * (size_t)oc : 0);
    }
    void load_weights(const float* blk) override {
        block.assign(blk, blk + weight_floats());
        if (set_up) pack();
    }
    void setup() override {
        const TView& in_v = tin(0).v;
        const TView& out_v = tout().v;
        padded = std::max((oc + 127) / 128 * 128, out_v.cp);
        scale_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
        bias_dev = static_cast<float*>(net->dev_alloc(padded * sizeof(float)));
        for (int py = 0; py < 2; py++)
            for (int px = 0; px < 2; px++) {
                SubConv sc;
                // out[2a+py, 2b+px] = sum over dy,dx of W[py+2dy, px+2dx] * in[a-dy, b-dx]
                const int ndy = (k - py + 1) / 2, ndx = (k - px + 1) / 2;
                for (int dy = 0; dy < ndy; dy++)
                    for (int dx = 0; dx < ndx; dx++) sc.taps.push_back(Tap{ndy - 1 - dy, ndx - 1 - dx, py + 2 * dy, px + 2 * dx});
                sc.span_y = ndy; sc.span_x = ndx;
                sc.in_y0 = in_v.pad - (ndy - 1);
                sc.in_x0 = in_v.pad - (ndx - 1);
                sc.in_stride = 1;
                sc.npos_y = (oh - py + 1) / 2;
                sc.npos_x = (ow - px + 1) / 2;
                if (sc.npos_y <= 0 || sc.npos_x <= 0) continue;
                sc.out_step = 2;
                sc.out_off_y = out_v.pad + py;
                sc.out_off_x = out_v.pad + px;
                subconvs.push_back(sc);
            }
        group = tune_mfma_group(net, subconvs, in_v, out_v, d.in_channels, oc, act(), scale_dev, bias_dev);
        if (tconv_p16_supported(k, crop, in_v.cp, in_v.pad, oc, out_v.cp, out_v.f16 != 0) && in_v.f16 == out_v.f16 && d.in_channels == in_v.cp &&
            !net->sw.get("FYNHIP_NO_P16_CONV"))
            setup_p16(in_v, out_v);
        set_up = true;
        setup_ranges();
        if (!block.empty()) pack();
    }
    // 16-position-fragment form (conv_p16.hip): all four output parities from one staged input tile; the compiled
    // combinations that fit are timed and the best is kept if it beats the grouped launch of the general kernel
    void setup_p16(const TView& in_v, const TView& out_v) {
        ConvP16Params q{};
        q.in = in_v.ptr; q.out = out_v.ptr; q.res = nullptr;
        q.in_hp = in_v.hp(); q.in_wp = in_v.wp(); q.in_cp = in_v.cp;
        q.stride = 1;
        q.in_y0 = q.in_x0 = in_v.pad - 1;
        q.npos_y = d.height; q.npos_x = d.width;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        q.cin_chunks = in_v.cp / 32;
        q.mfrags = oc / 16;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        q.in_amax = tin(0).amax;   // (timed in the form the frame will run)
        int want_h = 0, want_w = 0, want_wm = 0;   // FYNHIP_P16_TILE=h,w[,wm] (tests): that combination
        if (const char* e = net->sw.get("FYNHIP_P16_TILE")) sscanf(e, "%d,%d,%d", &want_h, &want_w, &want_wm);
        std::vector<ConvP16Params> cands;
        for (int i = 0; i < tconv_p16_tile_count(); i++) {
            int th, tw, wm;
            tconv_p16_tile(i, &th, &tw, &wm);
            if (oc % (32 * wm) != 0) continue;
            if (want_h && (th != want_h || tw != want_w || (want_wm && wm != want_wm))) continue;
            ConvP16Params c = q;
            c.tile_h = th; c.tile_w = tw; c.wm = wm;
            const int twg = (4 / wm) * tw;
            c.tiles_x = (d.width + twg - 1) / twg; c.tiles_y = (d.height + th - 1) / th;
            c.rcp_tiles_x = 1.0f / (float)c.tiles_x;
            c.cout_blocks = oc / (32 * wm);
            c.pos_groups = std::max(1, std::min(c.tiles_x * c.tiles_y, 256 / c.cout_blocks));
            const size_t lds = tconv_p16_lds_bytes(c);
            if (lds == 0 || lds > 160 * 1024) continue;
            cands.push_back(c);
        }
        if (cands.empty()) return;
        const size_t halves = ((size_t)q.cin_chunks * 9 + 8) * q.mfrags * (q.f16 ? 1 : 3) * 64 * 8;
        p16_wpack_dev = net->dev_alloc(halves * 2, true);
        for (ConvP16Params& c : cands) c.wpack = p16_wpack_dev;
        const bool always = net->sw.get("FYNHIP_FORCE_P16_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        int pick = 0;
        char key[160];
        snprintf(key, sizeof(key), "tp16:%dx%d:%dx%d:cp%d:h%d", d.in_channels, oc, d.height, d.width, in_v.cp, q.f16);
        int cached[3] = {0, 0, 0};
        if (!want_h && tune_cache_triple(net, key, cached)) {
            pick = -1;
            if (cached[0] || always)
                for (size_t i = 0; i < cands.size(); i++)
                    if (cands[i].tile_h * 1000 + cands[i].tile_w == cached[1] && cands[i].wm == cached[2]) pick = (int)i;
            if (always && pick < 0) pick = 0;
        } else if (!(at && at[0] == '0')) {
            float best = 1e30f, t_other = 1e30f;
            for (int rep = 0; rep < 3; rep++) {
                for (size_t i = 0; i < cands.size(); i++) {
                    const float t = time_calls(net, [&]() {
                        if (launch_tconv_p16(cands[i], net->stream) != 0) fail(FYN_ERR_DEVICE, "16-position transposed convolution launch failed while tuning");
                    }, 10);
                    if (t < best) { best = t; pick = (int)i; }
                }
                t_other = std::min(t_other, time_group(net, group, 10));
            }
            if (net->sw.get("FYNHIP_TUNE_VERBOSE"))
                fprintf(stderr, "[tune] transposed 3x3: 16-position fragments (%dx%d tiles, %d channel groups) %.1f us, general kernel %.1f us\n",
                        cands[pick].tile_h, cands[pick].tile_w, cands[pick].wm, best * 1e3f, t_other * 1e3f);
            const bool win = best < t_other;
            if (!want_h) tune_cache_store_triple(net, key, win ? 1 : 0, cands[pick].tile_h * 1000 + cands[pick].tile_w, cands[pick].wm);
            if (!win && !always) pick = -1;
        }
        if (pick >= 0) {
            p16 = true;
            pp = cands[pick];
        } else {
            net->dev_free(p16_wpack_dev);
            p16_wpack_dev = nullptr;
        }
    }
    // weights of that form: [(chunk*9 + step)][cout fragment of 16][plane][lane][8 halves], steps in the kernel's tap order
    void pack_p16(const float* w, float wmul) {
        const int cin = d.in_channels;
        const int npl = pp.f16 ? 1 : 3;   // fp32 tensors: hi, lo, and the fp8 operands of the correction terms
        const size_t frags = ((size_t)pp.cin_chunks * 9 + 8) * pp.mfrags;
        std::vector<uint16_t> pack(frags * npl * 64 * 8, 0);
        std::vector<float> c8(npl == 3 ? frags * 64 * 16 : 0, 0.f);
        for (int chunk = 0; chunk < pp.cin_chunks; chunk++)
            for (int t = 0; t < 9; t++) {
                int ky, kx;
                tconv_p16_tap(t, &ky, &kx);
                for (int mf = 0; mf < pp.mfrags; mf++) {
                    const size_t frag = (size_t)(chunk * 9 + t) * pp.mfrags + mf;
                    uint16_t* base = pack.data() + frag * npl * 64 * 8;
                    for (int lane = 0; lane < 64; lane++) {
                        const int o = p16_row_channel(mf, lane & 15, pp.f16 ? 2 : 1);
                        if (o >= oc) continue;
                        for (int j = 0; j < 8; j++) {
                            const int ci = chunk * 32 + 8 * (lane >> 4) + j;
                            if (ci >= cin) continue;
                            const float v = w[(((size_t)o * 3 + ky) * 3 + kx) * cin + ci] * wmul;
                            const uint16_t hi = f2h_bits(v);
                            base[(size_t)lane * 8 + j] = hi;
                            if (npl == 3) p16_lo_planes(base, c8.data() + (frag * 64 + lane) * 16, lane, j, v, hi);
                        }
                    }
                }
            }
        upload_p16_pack(net, p16_wpack_dev, pack, c8, frags);
    }
    // value ranges (range.h): every parity reads the input's word and raises the output's; the first one clears
    bool tracks_range() const override { return true; }
    void setup_ranges() override {
        for (auto& L : group.subs) {
            L.p.in_amax = tin(0).amax;
            L.p.out_amax = tout().amax;
        }
        group.sync();
        pp.in_amax = tin(0).amax;
        pp.out_amax = tout().amax;
    }
    bool add_range_reset(unsigned* w) override {
        if (p16) {
            if (!set_up || pp.nreset >= 4) return false;
            pp.reset[pp.nreset++] = w;
            return true;
        }
        if (!set_up || group.subs.empty() || group.subs[0].p.nreset >= 4) return false;
        group.subs[0].p.reset[group.subs[0].p.nreset++] = w;
        group.sync();
        return true;
    }
    void pack() {
        const float* bias = block.data();
        const float* w = bias + oc;
        const float* bn = w + (size_t)oc * k * k * d.in_channels;
        std::vector<float> sc, bi;
        fold_bn(bias, bn, oc, (d.flags & FYN_FLAG_POST_BATCHNORM) != 0, padded, sc, bi);
        reupload(net, scale_dev, sc);
        reupload(net, bias_dev, bi);
        const float wmul = weight_prescale(w, (size_t)oc * k * k * d.in_channels);
        if (p16) {
            pp.acc_mul = 1.0f / wmul;
            pack_p16(w, wmul);
            have_weights = true;
            return;
        }
        for (auto& L : group.subs) {
            L.p.acc_mul = 1.0f / wmul;
            pack_mfma_weights(net, L, w, k, wmul);
        }
        group.sync();
        have_weights = true;
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without weights", d.name, d.number);
        if (p16) {
            if (launch_tconv_p16(pp, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: transposed convolution launch failed", d.name);
            return;
        }
        if (run_group(group, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: transposed convolution launch failed", d.name);
    }
    std::string info() const override {
        if (p16) {
            char buf[220];
            snprintf(buf, sizeof(buf), "transconv, tconv_p16 %s 4 parities per tile, tile=%dx%d(cout x input pos) waves=%dx%d th=%d tw=%d blocks=%d tiles=%d lds=%zu steps=9 chunks=%d", pp.f16 ? "f16" : "f16x2-split",
                     32 * pp.wm, pp.tile_h * pp.tile_w * (4 / pp.wm), pp.wm, 4 / pp.wm, pp.tile_h, pp.tile_w, pp.pos_groups * pp.cout_blocks,
                     pp.tiles_x * pp.tiles_y * pp.cout_blocks, tconv_p16_lds_bytes(pp), pp.cin_chunks);
            return buf;
        }
        return group.subs.empty() ? "transconv" : "transconv, " + std::to_string(group.subs.size()) + " parities in one launch: " + mfma_info(group.subs[0]);
    }
    int k, crop;
    bool have_weights = false;
    int padded = 0;
    std::vector<float> block;
    std::vector<SubConv> subconvs;
    MfmaGroup group;
    bool p16 = false;             // 16-position-fragment form (conv_p16.hip)
    ConvP16Params pp{};
    void* p16_wpack_dev = nullptr;
    float *scale_dev = nullptr, *bias_dev = nullptr;
};

// =============================================================================================
// GEMM (fully connected; 1x1 spatial)
// =============================================================================================
class GemmLayer : public Layer {
  public:
    GemmLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        if (d.width != 1 || d.height != 1) fail(FYN_ERR_UNSUPPORTED, "GEMM layer expects a 1x1 spatial input (%s)", d.name);
        oc = d.out_channels;
        oh = ow = 1;
    }
    size_t weight_floats() const override {
        return (size_t)oc + (size_t)oc * d.in_channels + ((d.flags & FYN_FLAG_POST_BATCHNORM) ? 2 * (size_t)oc : 0);
    }
    void load_weights(const float* blk) override {
        block.assign(blk, blk + weight_floats());
        if (set_up) pack();
    }
    void setup() override {
        p.in = tin(0).v; p.out = tout().v;
        p.act = act();
        p.w_f16 = net->f16() ? 1 : 0;
        const size_t n = (size_t)p.out.cp * p.in.cp;
        w_dev = net->dev_alloc(n * (p.w_f16 ? 2 : 4));
        scale_dev = static_cast<float*>(net->dev_alloc(p.out.cp * sizeof(float)));
        bias_dev = static_cast<float*>(net->dev_alloc(p.out.cp * sizeof(float)));
        p.w = w_dev; p.scale = scale_dev; p.bias = bias_dev;
        set_up = true;
        if (!block.empty()) pack();
    }
    void pack() {
        const int cinp = p.in.cp, cin = d.in_channels;
        const float* bias = block.data();
        const float* w = bias + oc;
        const float* bn = w + (size_t)oc * cin;
        std::vector<float> sc, bi;
        fold_bn(bias, bn, oc, (d.flags & FYN_FLAG_POST_BATCHNORM) != 0, p.out.cp, sc, bi);
        reupload(net, scale_dev, sc);
        reupload(net, bias_dev, bi);
        if (p.w_f16) {
            std::vector<uint16_t> wd((size_t)p.out.cp * cinp, 0);
            for (int o = 0; o < oc; o++)
                for (int i = 0; i < cin; i++) wd[(size_t)o * cinp + i] = f2h_bits(w[(size_t)o * cin + i]);
            reupload(net, static_cast<uint16_t*>(w_dev), wd);
        } else {
            std::vector<float> wd((size_t)p.out.cp * cinp, 0.f);
            for (int o = 0; o < oc; o++)
                for (int i = 0; i < cin; i++) wd[(size_t)o * cinp + i] = w[(size_t)o * cin + i];
            reupload(net, static_cast<float*>(w_dev), wd);
        }
        have_weights = true;
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without weights", d.name, d.number);
        launch_gemv(p, s);
    }
    std::string info() const override { return "gemv"; }
    bool have_weights = false;
    std::vector<float> block;
    GemvParams p{};
    void* w_dev = nullptr;
    float *scale_dev = nullptr, *bias_dev = nullptr;
};

// =============================================================================================
// Pooling
// =============================================================================================
class PoolLayer : public Layer {
  public:
    PoolLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        is_max = d.type == FYN_LAYER_MAXPOOL2D;
        global = d.global_pool != 0;
        oc = d.in_channels;
        if (d.out_channels != 0 && d.out_channels != d.in_channels)
            fail(FYN_ERR_INVALID, "pooling layer %s must keep the channel count", d.name);
        if (global) {
            oh = ow = 1;
        } else {
            pool = d.pool_size[0];
            // gpu/gpulayerfactory.cpp:542-544
            if (d.pool_size[0] == 1 && d.pool_size[1] == 1)
                fail(FYN_ERR_INVALID, "Pooling layer with a pool size of 1 does not make sense, clean your net (%s)", d.name);
            if (d.pool_size[0] != d.pool_size[1] || pool < 1) fail(FYN_ERR_UNSUPPORTED, "anisotropic pooling not supported (%s)", d.name);
            stride = d.downsample[0] > 0 ? d.downsample[0] : 1;
            oh = d.height / stride;
            ow = d.width / stride;
        }
    }
    void setup() override {
        p.in = tin(0).v; p.out = tout().v;
        p.pool = pool; p.stride = stride; p.is_max = is_max; p.act = act();
        // stored-frame window start relative to (y*stride, x*stride):
        //   max: window begins input_padding before the stride origin (deepmaxpool.frag:15-45) -> 0
        //   avg: P=3 window [-1,1], otherwise [0,P) from the origin (deepavgpool.frag:17-44)
        p.off = is_max ? 0 : p.in.pad + (pool == 3 ? -1 : 0);
        // a large image is pooled by many workgroups per run of channel groups (about 2048 pixels each) and a second launch
        const long long npix = (long long)p.in.h * p.in.w;
        if (global && npix >= 16384) {
            splits = (int)std::min<long long>(1024, (npix + 2047) / 2048);
            partial_dev = static_cast<float*>(net->dev_alloc((size_t)splits * p.in.cp * sizeof(float)));
        }
    }
    void forward(hipStream_t s) override {
        if (global) launch_global_pool(tin(0).v, tout().v, is_max, act(), s, partial_dev, splits);
        else launch_pool(p, s);
    }
    std::string info() const override {
        if (!global) return "pool";
        return splits > 1 ? "global_pool (pixels dealt to " + std::to_string(splits) + " workgroups per run of channel groups, then a second launch)" : "global_pool";
    }
    int splits = 1;
    float* partial_dev = nullptr;
    bool is_max, global;
    int pool = 1, stride = 1;
    PoolParams p{};
};

// =============================================================================================
// Explicit batch-norm, add/sub, concat, arg-max, upload, download
// =============================================================================================
class BatchNormLayer : public Layer {
  public:
    BatchNormLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        oc = d.in_channels;
        oh = d.height;
        ow = d.width;
    }
    size_t weight_floats() const override { return 2 * (size_t)oc; }
    void load_weights(const float* blk) override {
        block.assign(blk, blk + weight_floats());
        if (set_up) pack();
    }
    void setup() override {
        p.in = tin(0).v; p.out = tout().v;
        p.res = (d.flags & FYN_FLAG_RESIDUAL_INPUT) ? tin(1).v : TView{};
        p.res_relu = (d.flags & FYN_FLAG_RELU_ON_RESIDUAL) ? 1 : 0;
        p.res_bn = (d.flags & FYN_FLAG_BATCHNORM_ON_RESIDUAL) ? 1 : 0;
        p.act = act();
        scale_dev = static_cast<float*>(net->dev_alloc(p.out.cp * sizeof(float)));
        bias_dev = static_cast<float*>(net->dev_alloc(p.out.cp * sizeof(float)));
        p.scale = scale_dev; p.bias = bias_dev;
        set_up = true;
        if (!block.empty()) pack();
    }
    void pack() {
        std::vector<float> sc(p.out.cp, 0.f), bi(p.out.cp, 0.f);
        for (int c = 0; c < oc; c++) {
            sc[c] = block[c];
            bi[c] = block[oc + c];
        }
        reupload(net, scale_dev, sc);
        reupload(net, bias_dev, bi);
        have_weights = true;
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without scale/bias", d.name, d.number);
        if (fused_into >= 0 && net->fusion_on()) return;   // applied by the convolution layers that read it
        launch_batchnorm(p, s);
    }
    std::string info() const override {
        return fused_into >= 0 ? "batchnorm (runs inside the launch of layer " + std::to_string(fused_into) + "; no launch of its own)" : "batchnorm";
    }
    int fused_into = -1;
    bool have_weights = false;
    std::vector<float> block;
    BnParams p{};
    float *scale_dev = nullptr, *bias_dev = nullptr;
};

// Batch-norm layers whose readers can apply them: a plain x * scale + bias (no activation, no residual input) between
// tensors of one geometry without a halo, read only by convolution layers on the K-resident or the LDS-free 1x1 form, as
// their data input.  Each reader then fetches from the batch-norm layer's input and applies scale and bias per channel
// before its own activation; the layer's output is never written and its launch is gone (the reference's ResNet-50 sample graph has one such layer in
// front of most blocks).  The input tensor must still hold its values when the last reader runs: no tensor produced
// between the batch-norm layer and that reader may live in the same buffer.
void fuse_batchnorm_layers(Net* net) {
    if (net->sw.get("FYNHIP_NO_BN_FUSION") || !net->reuse_buffers) return;
    for (auto& kv : net->layers) {
        BatchNormLayer* bn = dynamic_cast<BatchNormLayer*>(kv.second.get());
        if (!bn || bn->p.res.ptr || bn->p.act.kind != ACT_NONE) continue;
        Tensor& x = net->tensors[bn->in[0]];
        const Tensor& y = net->tensors[bn->out];
        // (no halo: around the layer's output it holds zeros, which scale and bias applied to the input's halo would not give)
        if (y.locked || x.v.pad != 0 || y.v.pad != 0 || x.v.h != y.v.h || x.v.w != y.v.w || x.v.cp != y.v.cp || x.v.f16 != y.v.f16 || x.v.c != y.v.c) continue;
        std::vector<ConvLayer*> readers;
        bool all = true;
        int last = -1;
        for (auto& kr : net->layers) {
            Layer* l = kr.second.get();
            for (size_t port = 0; port < l->in.size(); port++) {
                if (l->in[port] != bn->out) continue;
                ConvLayer* c = dynamic_cast<ConvLayer*>(l);
                if (!c || port != 0 || !c->takes_batchnorm() || c->d.number <= bn->d.number) { all = false; continue; }
                readers.push_back(c);
                last = std::max(last, c->d.number);
            }
        }
        if (!all || readers.empty()) continue;
        bool live = true;
        for (const Tensor& o : net->tensors)
            if (&o != &x && o.buffer == x.buffer && o.producer > bn->d.number && o.producer <= last) live = false;
        if (!live) continue;
        for (ConvLayer* c : readers) {
            c->bn_fused = true;
            c->bn_layer_no = bn->d.number;
            c->bn_in = x.v.ptr; c->bn_mul = bn->scale_dev; c->bn_add = bn->bias_dev;
        }
        bn->fused_into = readers.front()->d.number;
        x.last_reader = std::max(x.last_reader, last);   // (its value-range word is cleared behind its last reader)
    }
}

class AddSubLayer : public Layer {
  public:
    AddSubLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        oc = d.in_channels;
        oh = d.height;
        ow = d.width;
    }
    int num_ports() const override { return 2; }
    void port_shape(int, int& c, int& h, int& w, int& pad) const override {
        c = d.in_channels; h = d.height; w = d.width; pad = d.input_padding;
    }
    void forward(hipStream_t s) override { launch_addsub(tin(0).v, tin(1).v, tout().v, d.type == FYN_LAYER_SUB, act(), s); }
    std::string info() const override { return "addsub"; }
};

// Function-type layers with one input and no weights: scale / padding / relu / clip / deep<->shallow conversion
// (all a scale layer in the reference, gpu/gpulayerfactory.cpp:125-140,471-476), sigmoid, tanh, singleton
// arithmetic, cast, transpose, image-patch extraction, RGB<->BGR, non-maximum suppression and blur.
class FuncLayer : public Layer {
  public:
    FuncLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        const bool deep = (d.flags & FYN_FLAG_DEEP) != 0;
        if (d.flags & FYN_FLAG_RESIDUAL_INPUT) fail(FYN_ERR_UNSUPPORTED, "layer %s: this layer does not support residual input", d.name);
        oc = d.out_channels > 0 ? d.out_channels : d.in_channels;
        oh = d.height;
        ow = d.width;
        p.map = FMAP_SCALE;
        p.fn = FFN_COPY;
        p.ux = p.uy = p.dx = p.dy = 1;
        switch (d.type) {
            case FYN_LAYER_SCALE2D:
            case FYN_LAYER_PADDING2D:
            case FYN_LAYER_RELU:
            case FYN_LAYER_CLIP:
            case FYN_LAYER_DEEP2SHALLOW:
            case FYN_LAYER_SHALLOW2DEEP: {
                p.ux = std::max(1, d.upsample[0]); p.uy = std::max(1, d.upsample[1]);
                p.dx = std::max(1, d.downsample[0]); p.dy = std::max(1, d.downsample[1]);
                if (d.type != FYN_LAYER_SCALE2D && (p.ux != 1 || p.uy != 1 || p.dx != 1 || p.dy != 1))
                    fail(FYN_ERR_INVALID, "layer %s: only SCALE2D layers change the spatial size", d.name);
                if (oc != d.in_channels) fail(FYN_ERR_INVALID, "layer %s: input and output channels differ", d.name);
                // output size as the tiler / viewport computes it (gpu/deep/deeptiler.cpp:47-48, gpu/scalelayer.cpp:41-44)
                ow = (int)((float)d.width * ((float)p.ux / (float)p.dx));
                oh = (int)((float)d.height * ((float)p.uy / (float)p.dy));
                if (ow < 1 || oh < 1) fail(FYN_ERR_INVALID, "layer %s: scaled size is empty", d.name);
                // deep tensors: the input quad starts (d-1)/2 texels early (gpu/deep/deeptiler.cpp:97-110)
                p.ox = deep ? p.ux * (p.dx - 1) : 0;
                p.oy = deep ? p.uy * (p.dy - 1) : 0;
                linear = d.type == FYN_LAYER_SCALE2D && d.scale_type == 1;
                if (d.scale_type != 0 && d.scale_type != 1) fail(FYN_ERR_INVALID, "layer %s: unknown scaling type %d", d.name, d.scale_type);
                if (deep && (d.width == 1 || d.height == 1)) linear = false;   // gpu/deep/deepscalelayer.cpp:44
                kind = linear ? "scale-linear" : "scale-nearest";
                break;
            }
            case FYN_LAYER_SIGMOID: p.fn = FFN_SIGMOID; kind = "sigmoid"; break;
            case FYN_LAYER_TANH: p.fn = FFN_TANH; kind = "tanh"; break;
            case FYN_LAYER_SINGLETON_ARITH:
                if (d.arith_op < 0 || d.arith_op > 3) fail(FYN_ERR_INVALID, "layer %s: unknown arithmetic operation %d", d.name, d.arith_op);
                p.fn = FFN_ARITH; p.op = d.arith_op; p.operand = d.operand; kind = "singleton-arith";
                break;
            case FYN_LAYER_CAST:
                if (d.cast_target < 0 || d.cast_target > 7) fail(FYN_ERR_INVALID, "layer %s: unknown cast target %d", d.name, d.cast_target);
                p.fn = FFN_CAST; p.op = d.cast_target; kind = "cast";
                break;
            case FYN_LAYER_TRANSPOSE:
                // gpu/gpulayerfactory.cpp (createTransposeLayer): deep tensors only
                if (!deep) fail(FYN_ERR_UNSUPPORTED, "No shallow transpose layer support (yet)");
                p.map = FMAP_TRANSPOSE; oh = d.width; ow = d.height; kind = "transpose";
                break;
            case FYN_LAYER_IMGEXTRACT:
                // createImgExtractLayer rejects builders flagged deep (the layer itself works on deep-format tensors)
                if (deep) fail(FYN_ERR_UNSUPPORTED, "Shallow imgextract currently not supported");
                if (d.window < 1) fail(FYN_ERR_INVALID, "layer %s: invalid window %d", d.name, d.window);
                if (d.width % d.window || d.height % d.window)
                    fail(FYN_ERR_INVALID, "layer %s: size %dx%d is not divisible by window size %d", d.name, d.width, d.height, d.window);
                p.map = FMAP_IMGEXTRACT; p.window = d.window; p.in_groups = (d.in_channels + 3) / 4;
                if ((oc + 3) / 4 > p.in_groups * d.window * d.window)
                    fail(FYN_ERR_INVALID, "layer %s: %d output channels exceed what a %dx%d window of %d channels yields", d.name, oc, d.window, d.window, d.in_channels);
                oh = d.height / d.window; ow = d.width / d.window; kind = "imgextract";
                break;
            case FYN_LAYER_RGB2BGR:
                if (deep) fail(FYN_ERR_UNSUPPORTED, "Deep rgb->bgr currently not supported");
                p.fn = FFN_BGR; kind = "rgb2bgr";
                break;
            case FYN_LAYER_NONMAX2D:
                if (deep) fail(FYN_ERR_UNSUPPORTED, "Deep nonmax suppression currently not supported");
                kind = "nonmax2d";
                break;
            case FYN_LAYER_BLUR2D:
                if (deep) fail(FYN_ERR_UNSUPPORTED, "Deep blurring currently not supported");
                if ((d.kernel & 1) == 0) fail(FYN_ERR_INVALID, "This layer only supports odd kernel sizes");
                if (d.kernel < 3 || d.kernel > 15) fail(FYN_ERR_UNSUPPORTED, "layer %s: blur kernel size %d outside 3..15", d.name, d.kernel);
                if (d.blur_type != 0 && d.blur_type != 1) fail(FYN_ERR_INVALID, "layer %s: unknown blur kernel type %d", d.name, d.blur_type);
                kind = "blur2d";
                break;
            default: fail(FYN_ERR_UNSUPPORTED, "Unsupported layer type %d", d.type);
        }
        if (d.type != FYN_LAYER_IMGEXTRACT && oc != d.in_channels) fail(FYN_ERR_INVALID, "layer %s: input and output channels differ", d.name);
    }
    void setup() override {
        p.in = tin(0).v;
        p.out = tout().v;
        p.act = act();
        if (d.type == FYN_LAYER_BLUR2D) {
            // gpu/blurlayer.cpp:86-113 in its own float arithmetic
            const int k = d.kernel;
            std::vector<float> coef((size_t)k * k);
            if (d.blur_type == 0) {
                const float c = 1.0f / (float)(k * k);
                for (float& v : coef) v = c;
            } else {
                std::vector<float> g(k);
                const float fac = (float)(1.0 / std::sqrt(2.0 * 3.14159265358979323846));
                for (int i = 0; i < k; i++) {
                    const float x = (float)(i - (k - 1) / 2);
                    g[i] = fac * expf(-(x * x));
                }
                float denom = 0.f;
                for (int y = 0; y < k; y++)
                    for (int x = 0; x < k; x++) {
                        coef[(size_t)y * k + x] = g[y] * g[x];
                        denom += coef[(size_t)y * k + x];
                    }
                for (float& v : coef) v /= denom;
            }
            coef_dev = upload(net, coef);
        }
    }
    void forward(hipStream_t s) override {
        if (d.type == FYN_LAYER_NONMAX2D) launch_nonmax(p.in, p.out, s);
        else if (d.type == FYN_LAYER_BLUR2D) {
            // shaders/generickernel.frag:83-107: 3x3 visits (-1..1)^2; larger kernels stop one short of the last
            // row and column and take the coefficients in running order
            const int r = (d.kernel - 1) / 2;
            launch_blur(p.in, p.out, coef_dev, r, d.kernel == 3 ? r : r - 1, s);
        } else if (linear) launch_scale_linear(p, s);
        else launch_func(p, s);
    }
    std::string info() const override { return kind; }
    FuncParams p{};
    bool linear = false;
    const char* kind = "function";
    float* coef_dev = nullptr;
};

class ConcatLayer : public Layer {
  public:
    ConcatLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        if (d.num_inputs < 1 || d.num_inputs > FYN_MAX_CONCAT_INPUTS) fail(FYN_ERR_INVALID, "concat layer %s needs 1..%d inputs", d.name, FYN_MAX_CONCAT_INPUTS);
        int total = 0;
        bool all_relu = true;
        for (int i = 0; i < d.num_inputs; i++) {
            total += d.inputs[i].channels;
            if (!(d.inputs[i].flags & FYN_FLAG_PRE_RELU)) all_relu = false;
        }
        oc = total;
        oh = d.height;
        ow = d.width;
        // ReLU on fetch only if every input asks for it (gpu/deep/deepconcatlayer.cpp:40-49)
        relu = all_relu || (d.flags & FYN_FLAG_PRE_RELU);
    }
    int num_ports() const override { return d.num_inputs; }
    void port_shape(int port, int& c, int& h, int& w, int& pad) const override {
        c = d.inputs[port].channels; h = d.height; w = d.width; pad = d.inputs[port].padding;
    }
    void forward(hipStream_t s) override {
        Act a = act();
        if (relu && a.kind == ACT_NONE) {
            a.kind = ACT_RELU;
            a.lo = 0.f;
        }
        int off = 0;
        for (int i = 0; i < d.num_inputs; i++) {
            launch_concat_part(tin(i).v, tout().v, off, a, s, i == d.num_inputs - 1);
            off += d.inputs[i].channels;
        }
    }
    std::string info() const override { return "concat"; }
    bool relu;
};

class ArgMaxLayer : public Layer {
  public:
    ArgMaxLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        oc = 2;  // index, value (shaders/deep/deepargmax2.frag:15-20)
        oh = d.height;
        ow = d.width;
    }
    void setup() override { idx_dev = static_cast<int32_t*>(net->dev_alloc((size_t)oh * ow * sizeof(int32_t))); }
    void forward(hipStream_t s) override { launch_argmax(tin(0).v, tout().v, idx_dev, act(), s); }
    std::string info() const override { return "argmax"; }
    int32_t* idx_dev = nullptr;
};

class UploadLayer : public Layer {
  public:
    UploadLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        // gpu/gpulayerfactory.cpp:276-278: uploads carry at most one texel's worth of channels
        if (d.flags & FYN_FLAG_DEEP) fail(FYN_ERR_UNSUPPORTED, "Deep upload layers are not supported (%s)", d.name);
        oc = d.out_channels ? d.out_channels : d.in_channels;
        oh = d.height;
        ow = d.width;
    }
    int num_ports() const override { return 0; }
    void forward(hipStream_t) override {}
    std::string info() const override { return "upload"; }
};

class DownloadLayer : public Layer {
  public:
    DownloadLayer(Net* n, const fyn_layer_desc& d_) : Layer(n, d_) {
        oc = d.in_channels;
        oh = d.height;
        ow = d.width;
    }
    bool has_own_output() const override { return false; }
    void forward(hipStream_t) override {}
    std::string info() const override { return "download"; }
};

// User-supplied layer behind C callbacks (the reference's CustomLayerBuilder hook, gpu/customlayerbuilder.h:53-90).
class CustomLayer : public Layer {
  public:
    CustomLayer(Net* n, const fyn_layer_desc& d_, const fyn_custom_layer& impl) : Layer(n, d_), cb(impl) {
        if (!cb.forward) fail(FYN_ERR_INVALID, "custom layer %s has no forward function", d.name);
        if (d.num_inputs < 0 || d.num_inputs > FYN_MAX_CONCAT_INPUTS) fail(FYN_ERR_INVALID, "custom layer %s: bad number of inputs %d", d.name, d.num_inputs);
        const int ux = std::max(1, d.upsample[0]), uy = std::max(1, d.upsample[1]);
        const int dx = std::max(1, d.downsample[0]), dy = std::max(1, d.downsample[1]);
        oc = d.out_channels > 0 ? d.out_channels : d.in_channels;
        ow = d.width * ux / dx;
        oh = d.height * uy / dy;
        if (ow < 1 || oh < 1) fail(FYN_ERR_INVALID, "custom layer %s: empty output", d.name);
    }
    ~CustomLayer() override {
        if (cb.cleanup) cb.cleanup(cb.user);
    }
    int num_ports() const override { return d.num_inputs > 0 ? d.num_inputs : ((d.flags & FYN_FLAG_RESIDUAL_INPUT) ? 2 : 1); }
    void port_shape(int port, int& c, int& h, int& w, int& pad) const override {
        if (d.num_inputs > 0) {
            c = d.inputs[port].channels; h = d.height; w = d.width; pad = d.inputs[port].padding;
        } else {
            Layer::port_shape(port, c, h, w, pad);
        }
    }
    static fyn_tensor_view view_of(const TView& v) {
        return fyn_tensor_view{v.ptr, v.c, v.h, v.w, v.pad, v.cp, v.f16 ? FYN_STORAGE_F16 : FYN_STORAGE_F32};
    }
    void setup() override {
        ins.clear();
        for (int i = 0; i < num_ports(); i++) ins.push_back(view_of(tin(i).v));
        outv = view_of(tout().v);
        if (cb.setup) {
            const int rc = cb.setup(cb.user, ins.data(), (int)ins.size(), &outv);
            if (rc != 0) fail(FYN_ERR_INVALID, "custom layer %s: setup callback failed (%d)", d.name, rc);
        }
    }
    void forward(hipStream_t s) override {
        const int rc = cb.forward(cb.user, ins.data(), (int)ins.size(), &outv, s, net->seq);
        if (rc != 0) fail(FYN_ERR_DEVICE, "custom layer %s: forward callback failed (%d)", d.name, rc);
    }
    std::string info() const override { return "custom"; }
    fyn_custom_layer cb;
    std::vector<fyn_tensor_view> ins;
    fyn_tensor_view outv{};
};

Layer* create_custom_layer(Net* net, const fyn_layer_desc& d, const fyn_custom_layer& impl) {
    if (d.type != FYN_LAYER_CUSTOM) fail(FYN_ERR_INVALID, "layer %s: a custom layer needs type FYN_LAYER_CUSTOM", d.name);
    if (d.width <= 0 || d.height <= 0 || d.width > 65535 || d.height > 65535)
        fail(FYN_ERR_INVALID, "layer %s: invalid spatial size %dx%d", d.name, d.width, d.height);
    if (d.in_channels < 0 || d.in_channels > 32767 || d.out_channels < 0 || d.out_channels > 32767 || (d.in_channels == 0 && d.num_inputs == 0))
        fail(FYN_ERR_INVALID, "layer %s: invalid channel counts %d -> %d", d.name, d.in_channels, d.out_channels);
    Layer* l = new CustomLayer(net, d, impl);
    l->in.assign(l->num_ports(), -1);
    return l;
}

Layer* create_layer(Net* net, const fyn_layer_desc& d) {
    if (d.width <= 0 || d.height <= 0 || d.width > 65535 || d.height > 65535)
        fail(FYN_ERR_INVALID, "layer %s: invalid spatial size %dx%d", d.name, d.width, d.height);
    if (d.in_channels <= 0 || d.in_channels > 32767 || d.out_channels < 0 || d.out_channels > 32767)
        fail(FYN_ERR_INVALID, "layer %s: invalid channel counts %d -> %d", d.name, d.in_channels, d.out_channels);
    if (d.input_padding < 0 || d.output_padding < 0 || d.residual_padding < 0)
        fail(FYN_ERR_INVALID, "layer %s: negative padding", d.name);
    Layer* l = nullptr;
    switch (d.type) {
        case FYN_LAYER_CONVOLUTION2D: {
            // gpu/gpulayerfactory.cpp:358-396
            const bool dw = d.group_size != 1 && d.group_size != 0 && d.group_size == d.in_channels;
            if (dw) {
                if (d.kernel == 1) fail(FYN_ERR_UNSUPPORTED, "No 1x1 depthwise layer supported");
                if (d.kernel != 3) fail(FYN_ERR_UNSUPPORTED, "No %dx%d depthwise layer supported", d.kernel, d.kernel);
                l = new DwConvLayer(net, d);
            } else {
                if (d.group_size > 1) fail(FYN_ERR_UNSUPPORTED, "grouped convolution (group size %d) not supported (%s)", d.group_size, d.name);
                l = new ConvLayer(net, d);
            }
            break;
        }
        case FYN_LAYER_TRANSCONVOLUTION2D: l = new TransConvLayer(net, d); break;
        case FYN_LAYER_GEMM: l = new GemmLayer(net, d); break;
        case FYN_LAYER_MAXPOOL2D:
        case FYN_LAYER_AVGPOOL2D: l = new PoolLayer(net, d); break;
        case FYN_LAYER_BATCHNORM: l = new BatchNormLayer(net, d); break;
        case FYN_LAYER_ADD:
        case FYN_LAYER_SUB: l = new AddSubLayer(net, d); break;
        case FYN_LAYER_CONCAT: l = new ConcatLayer(net, d); break;
        case FYN_LAYER_ARGMAX:
            // gpu/gpulayerfactory.cpp:791-815: arg-max exists for deep tensors only
            if (!(d.flags & FYN_FLAG_DEEP)) fail(FYN_ERR_UNSUPPORTED, "ArgMax layer is only supported on deep tensors (%s)", d.name);
            l = new ArgMaxLayer(net, d);
            break;
        case FYN_LAYER_SCALE2D:
        case FYN_LAYER_PADDING2D:
        case FYN_LAYER_RELU:
        case FYN_LAYER_CLIP:
        case FYN_LAYER_DEEP2SHALLOW:
        case FYN_LAYER_SHALLOW2DEEP:
        case FYN_LAYER_SIGMOID:
        case FYN_LAYER_TANH:
        case FYN_LAYER_SINGLETON_ARITH:
        case FYN_LAYER_CAST:
        case FYN_LAYER_TRANSPOSE:
        case FYN_LAYER_IMGEXTRACT:
        case FYN_LAYER_RGB2BGR:
        case FYN_LAYER_NONMAX2D:
        case FYN_LAYER_BLUR2D: l = new FuncLayer(net, d); break;
        case FYN_LAYER_FRACCONVOLUTION2D:
            if (d.group_size > 1) fail(FYN_ERR_UNSUPPORTED, "grouped convolution (group size %d) not supported (%s)", d.group_size, d.name);
            l = new ConvLayer(net, d);
            break;
        case FYN_LAYER_CUSTOM: fail(FYN_ERR_INVALID, "layer %s: custom layers are added with fyn_net_add_custom_layer", d.name);
        case FYN_LAYER_UPLOAD: l = new UploadLayer(net, d); break;
        case FYN_LAYER_DOWNLOAD: l = new DownloadLayer(net, d); break;
        default: fail(FYN_ERR_UNSUPPORTED, "Unsupported layer type %d", d.type);
    }
    l->in.assign(l->num_ports(), -1);
    return l;
}

void Net::copy_argmax(int layer_no, int32_t* idx, float* val) {
    if (!is_setup) fail(FYN_ERR_STATE, "copy_argmax() before setup()");
    FYN_HIP(hipSetDevice(device));
    ArgMaxLayer* l = dynamic_cast<ArgMaxLayer*>(layer(layer_no));
    if (!l) fail(FYN_ERR_INVALID, "layer %d is not an arg-max layer", layer_no);
    const size_t n = (size_t)l->oh * l->ow;
    FYN_HIP(hipStreamSynchronize(stream));
    if (idx) FYN_HIP(hipMemcpy(idx, l->idx_dev, n * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (val) {
        std::vector<float> chw(2 * n);
        copy_result(layer_no, chw.data(), 0);
        memcpy(val, chw.data() + n, n * sizeof(float));
    }
}

}  // namespace fynhip
