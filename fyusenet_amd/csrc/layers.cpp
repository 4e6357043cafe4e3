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
#include "conv_plan.h"
#include "layer_classes.h"

namespace fynhip {

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
        q.plain_stores = net->sw.get("FYNHIP_PLAIN_STORES") ? 1 : 0;
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
            return std::string(buf) + (conv_p16_stores_through(pp, 2) ? " stores=through" : "");
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
        float wmax = 0.f;
        for (size_t i = 0; i < (size_t)oc * cin; i++) wmax = std::max(wmax, std::fabs(w[i]));
        // the matrix once more for the matrix-core form on fp32 tensors: fp16 hi and lo halves, eight weights at a time
        p.w_split = nullptr;
        if (!p.w_f16 && wmax < 3.0e4f && !net->sw.get("FYNHIP_NO_MFMA_GEMM")) {
            std::vector<uint16_t> ws((size_t)p.out.cp * cinp * 2, 0);
            for (int o = 0; o < oc; o++)
                for (int i = 0; i < cin; i++) {
                    const float v = w[(size_t)o * cin + i];
                    const uint16_t hb = f2h_bits(v);
                    const size_t at = ((size_t)o * cinp + (i & ~7)) * 2 + (i & 7);
                    ws[at] = hb;
                    ws[at + 8] = f2h_bits(v - h2f(hb));
                }
            if (!w_split_dev) w_split_dev = net->dev_alloc(ws.size() * 2);
            reupload(net, static_cast<uint16_t*>(w_split_dev), ws);
            p.w_split = w_split_dev;
        }
        have_weights = true;
        choose(wmax);
    }
    // The matrix-core form (fc_mfma_kernel) where it fits -- fp32 weights are split into fp16 halves in registers, so
    // they must lie inside fp16's range -- and is measured to be faster than the vector-unit form on this layer (both
    // stream the matrix once and are bound by that; with one right-hand side the matrix-core form pays for staging the
    // vector in every workgroup and for two barriers: 7.3 against 3.1 us on 2048 -> 1000 in fp32, 23.3 against 22.5 us
    // on 8192 -> 8192 in fp16; FYNHIP_NO_MFMA_GEMM / FYNHIP_FORCE_MFMA_GEMM pin the choice).
    void choose(float wmax) {
        use_mfma = false;
        if (net->sw.get("FYNHIP_NO_MFMA_GEMM") || !fc_mfma_supported(p) || !(wmax < 3.0e4f)) return;
        if (net->sw.get("FYNHIP_FORCE_MFMA_GEMM")) { use_mfma = true; return; }
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        if (at && at[0] == '0') return;   // (unmeasured: the vector-unit form, which wins on every layer measured so far)
        float t_m = 1e30f, t_v = 1e30f;
        for (int rep = 0; rep < 3; rep++) {
            t_m = std::min(t_m, time_calls(net, [&]() {
                if (launch_fc_mfma(p, net->stream) != 0) fail(FYN_ERR_DEVICE, "layer %s: matrix-core launch failed while tuning", d.name);
            }, 10));
            t_v = std::min(t_v, time_calls(net, [&]() { launch_gemv(p, net->stream); }, 10));
        }
        use_mfma = t_m < t_v;
        if (net->sw.get("FYNHIP_TUNE_VERBOSE")) fprintf(stderr, "[tune] fully connected %s: matrix cores %.2f us, vector units %.2f us\n", d.name, t_m * 1e3f, t_v * 1e3f);
    }
    void forward(hipStream_t s) override {
        if (!have_weights) fail(FYN_ERR_STATE, "layer %s (%d): forward() without weights", d.name, d.number);
        if (use_mfma) {
            if (launch_fc_mfma(p, s) != 0) fail(FYN_ERR_DEVICE, "layer %s: matrix-core launch failed", d.name);
        } else {
            launch_gemv(p, s);
        }
    }
    std::string info() const override {
        return use_mfma ? (p.out.f16 ? "fc_mfma f16, 16 or 4 rows per workgroup, 4 waves split the reduction" : "fc_mfma f16x2-split, 16 or 4 rows per workgroup, 4 waves split the reduction") : "gemv";
    }
    bool have_weights = false, use_mfma = false;
    std::vector<float> block;
    GemvParams p{};
    void *w_dev = nullptr, *w_split_dev = nullptr;
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
// Add/sub, element functions, concat, arg-max, upload, download, custom layers
// =============================================================================================
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
