// Planning, tuning (with its optional on-disk memory) and weight packing of the matrix-core convolution kernels:
// tile enumeration and launch descriptions for conv_mfma.hip, the timing of candidates on a layer's own tensors, the
// per-lane fragment order of the packed weights (gpu/deep/deepconvlayerbase.cpp:293-395 is the reference's packing).
#include "conv_plan.h"

#include <map>
#include <mutex>

namespace fynhip {

// scale / bias' of the convolution family from a weight block:
//   bias' = bias*bnScale + bnBias, scale = bnScale (gpu/deep/deepconvlayerbase.cpp:360-382)
void fold_bn(const float* bias, const float* bn, int cout, bool post_bn, int padded, std::vector<float>& scale,
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

// All tile configurations that fit (possibly none), best heuristic score first.
std::vector<TileChoice> enumerate_tiles(Net* net, int cout, const SubConv& sc, int pitch, int npl, int slack, int nbuf) {
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
void conv_geometry(Net* net, const TView& in, bool split, int ntaps, int kc_force, int& kc, int& pitch, int& slack, int& npl) {
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
MfmaLaunch plan_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
                            int cout, const Act& act, int res_relu, int res_scale, const TileChoice& tc,
                            const float* scale, const float* bias, const MfmaLaunch* share, int force_pd) {
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

// Launches a planned (sub-)convolution: the MFMA kernel and, with split-K, the reduce pass.
int run_mfma(const MfmaLaunch& L, hipStream_t s) {
    const int rc = launch_conv_mfma(L.var, L.p, L.lds, s);
    if (rc != 0) return rc;
    if (L.p.ksplit > 1) launch_splitk_reduce(L.red, s);
    return 0;
}

// Turns a planned launch into its split-K form (ksplit slices over the input-channel chunks).
void set_ksplit(Net* net, MfmaLaunch& L, int ksplit) {
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

float time_launch(Net* net, const MfmaLaunch& L, int iters) {
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
bool tune_cache_bypassed(Net* net) {
    for (const char* e : {"FYNHIP_FORCE_KSPLIT", "FYNHIP_CONV_TILE", "FYNHIP_CONV_KC_MAX", "FYNHIP_CONV_KC", "FYNHIP_CONV_PD"})
        if (net->sw.get(e)) return true;
    return false;
}

const TileChoice* tune_cache_lookup(Net* net, const char* key, const std::vector<TileChoice>& cands, int* ksplit) {
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

void tune_cache_store(Net* net, const char* key, const ConvVariant& v, int ksplit, int twl) {
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
bool tune_cache_flag(Net* net, const char* key, bool* flag) {
    if (tune_cache_bypassed(net)) return false;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = tune_cache(net).find(key);
    if (it == tune_cache(net).end()) return false;
    *flag = it->second[0] != 0;
    return true;
}

void tune_cache_store_flag(Net* net, const char* key, bool flag) {
    ConvVariant v{};
    v.fm = flag ? 1 : 0;
    tune_cache_store(net, key, v, 0, 0);
}

// three numbers under a key of their own (same file)
bool tune_cache_triple(Net* net, const char* key, int (&out)[3]) {
    if (tune_cache_bypassed(net)) return false;
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = tune_cache(net).find(key);
    if (it == tune_cache(net).end()) return false;
    out[0] = it->second[0]; out[1] = it->second[1]; out[2] = it->second[2];
    return true;
}

void tune_cache_store_triple(Net* net, const char* key, int a, int b, int c) {
    ConvVariant v{};
    v.fm = a; v.fn = b; v.wm = c;
    tune_cache_store(net, key, v, 0, 0);
}

// Picks the tile configuration of one (sub-)convolution: by measurement on the layer's own tensors (default), or by
// the heuristic score when FYNHIP_AUTOTUNE=0.  Candidates are timed before the weights are packed, i.e. on zero
// operands; the matrix pipes run about a tenth faster on those than on real data (the part holds a higher clock when
// fewer operand bits toggle), for all candidates alike, so the ranking carries over while the figures do not.
MfmaLaunch tune_mfma(Net* net, const SubConv& sc, const TView& in, const TView& out, const TView* res, int cin,
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

int run_group(const MfmaGroup& g, hipStream_t s) {
    if (conv_mfma_multi_exists(g.var)) return launch_conv_mfma_multi(g.var, g.multi, g.lds, s);
    for (const MfmaLaunch& L : g.subs)   // no merged entry point for this variant (narrow channel chunks): one launch each
        if (int rc = launch_conv_mfma(L.var, L.p, L.lds, s)) return rc;
    return 0;
}

float time_group(Net* net, const MfmaGroup& g, int iters) {
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
MfmaGroup tune_mfma_group(Net* net, const std::vector<SubConv>& scs, const TView& in, const TView& out, int cin, int cout,
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
void pack_mfma_weights(Net* net, MfmaLaunch& L, const float* w, int k, float wmul, int kw) {
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
float weight_prescale(const float* w, size_t n) {
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
void p16_lo_planes(uint16_t* frag_base, float* c8_lane, int lane, int j, float v, uint16_t hi) {
    const float lo = v - h2f(hi);
    frag_base[(size_t)(64 + lane) * 8 + j] = f2h_bits(lo);
    c8_lane[j] = h2f(hi) * (1.0f / 32.0f);
    c8_lane[8 + j] = lo * 64.0f;
}

void upload_p16_pack(Net* net, void* dev, const std::vector<uint16_t>& pack, const std::vector<float>& c8, size_t frags) {
    FYN_HIP(hipStreamSynchronize(net->stream));
    FYN_HIP(hipMemcpyAsync(dev, pack.data(), pack.size() * 2, hipMemcpyHostToDevice, net->stream));
    if (!c8.empty()) {
        float* src = upload(net, c8);
        if (launch_pack_fp8_plane(src, dev, frags, net->stream) != 0) fail(FYN_ERR_DEVICE, "packing the fp8 weight plane failed");
        net->dev_free(src);   // (waits for the stream)
    }
    FYN_HIP(hipStreamSynchronize(net->stream));
}

std::string mfma_info(const MfmaLaunch& L) {
    char buf[256];
    snprintf(buf, sizeof(buf), "conv_mfma %s tile=%dx%d(cout x pos) waves=%dx%d kc=%d th=%d tw=%d blocks=%d lds=%zu steps=%d chunks=%d ksplit=%d",
             L.var.split ? "f16x2-split" : "f16", L.var.wm * L.var.fm * 32, L.var.wn * L.var.fn * 32, L.var.wm, L.var.wn, L.var.kc,
             L.p.tile_h, 1 << L.p.tile_w_log2, L.p.tiles_x * L.p.tiles_y * L.p.cout_blocks, L.lds, L.p.nsteps, L.p.cin_chunks, L.p.ksplit);
    return buf;
}

}  // namespace fynhip
