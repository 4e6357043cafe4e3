// The layer classes that the graph-rewrite passes (fusion.cpp) look into: convolution, depthwise convolution and
// explicit batch-norm.  The other layer classes live in layers.cpp.
#pragma once
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "conv_plan.h"
#include "engine.h"

namespace fynhip {

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
        if (frac_shift) {   // (the frame of repeated pixels; the 3x3 shader's columns at -2, -1, 0: as in the general kernel's sub-convolution)
            q.in_shift = frac_shift - 1;
            q.in_y0 = (in_v.pad << q.in_shift) - 1;
            q.in_x0 = (in_v.pad << q.in_shift) - 2;
        }
        q.in_clamp = clamp ? 1 : 0;
        q.npos_y = oh; q.npos_x = ow;
        q.out_wp = out_v.wp(); q.out_cp = out_v.cp; q.out_off_y = q.out_off_x = out_v.pad;
        if (res_v) { q.res_wp = res_v->wp(); q.res_cp = res_v->cp; q.res_off_y = q.res_off_x = res_v->pad; }
        q.res_relu = res_relu; q.res_scale = res_scale;
        // (ragged channel counts: the last chunk reads zeros behind the input's pitch, the weights are packed for whole
        // blocks of 64 output channels, and a block's channels behind the output's pitch are not stored)
        q.cin_chunks = (in_v.cp + 31) / 32;
        q.mfrags = (oc + 63) / 64 * 4;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        q.in_amax = tin(0).amax;   // (the candidates are timed in the form the frame will run: fp8 correction terms where the input has a range word)
        q.exact_split = net->sw.get("FYNHIP_EXACT_SPLIT") ? 1 : 0;
        q.plain_stores = net->sw.get("FYNHIP_PLAIN_STORES") ? 1 : 0;
        int want_h = 0, want_w = 0, want_wm = 0;   // FYNHIP_P16_TILE=h,w[,wm] (tests): that combination
        if (const char* e = net->sw.get("FYNHIP_P16_TILE")) sscanf(e, "%d,%d,%d", &want_h, &want_w, &want_wm);
        struct Cand { double cost; ConvP16Params q; };
        std::vector<Cand> cands;
        for (int i = 0; i < conv_p16_tile_count(); i++) {
            int th, tw, st, wm;
            conv_p16_tile(i, &th, &tw, &st, &wm);
            if (st != stride || (wm == 4 && oc % 128 != 0)) continue;
            if (want_h && (th != want_h || tw != want_w || (want_wm && wm != want_wm))) continue;
            ConvP16Params c = q;
            c.tile_h = th; c.tile_w = tw; c.wm = wm;
            const int twg = (4 / wm) * tw;
            c.tiles_x = (ow + twg - 1) / twg; c.tiles_y = (oh + th - 1) / th;
            c.rcp_tiles_x = 1.0f / (float)c.tiles_x;
            c.cout_blocks = (oc + 32 * wm - 1) / (32 * wm);
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
        snprintf(key, sizeof(key), "p16:%dx%d:%dx%d:s%d:cp%d:r%d:e%d:h%d:f%d", d.in_channels, oc, oh, ow, stride, in_v.cp, res_v ? 1 : 0, clamp ? 1 : 0, q.f16, frac_shift);
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
        q.mfrags = (oc + 31) / 32 * 2;
        q.cout_blocks = (oc + 31) / 32;
        q.f16 = out_v.f16 ? 1 : 0;
        q.scale = scale_dev; q.bias = bias_dev;
        q.acc_mul = 1.f;
        q.act = act();
        q.in_amax = tin(0).amax;   // (timed in the form the frame will run)
        q.exact_split = net->sw.get("FYNHIP_EXACT_SPLIT") ? 1 : 0;
        q.plain_stores = net->sw.get("FYNHIP_PLAIN_STORES") ? 1 : 0;
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
        const size_t halves = ((size_t)steps + 8) * q.mfrags * (q.f16 ? 1 : 3) * 64 * 8;
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
        const int npl = pp.f16 ? 1 : 3;   // (fp16 tensors: the hi plane only; fp32: hi, lo, fp8 operands of the correction terms)
        const size_t frags = ((size_t)c4_steps + 8) * pp.mfrags;
        std::vector<uint16_t> pack(frags * npl * 64 * 8, 0);
        // (sources of the third plane, per tap of a lane's pair: four hi parts / 32, then four lo parts * 64)
        std::vector<float> c8(npl == 3 ? frags * 64 * 16 : 0, 0.f);
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
                        if (npl == 3) {
                            const float lo = v - h2f(hi);
                            base[(size_t)(64 + lane) * 8 + j] = f2h_bits(lo);
                            float* c8_lane = c8.data() + (((size_t)st * pp.mfrags + mf) * 64 + lane) * 16;
                            c8_lane[(j / 4) * 8 + j % 4] = h2f(hi) * (1.0f / 32.0f);
                            c8_lane[(j / 4) * 8 + 4 + j % 4] = lo * 64.0f;
                        }
                    }
                }
            }
        upload_p16_pack(net, p16_wpack_dev, pack, c8, frags);
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
        if (frac_shift) {   // (the frame of repeated pixels, and the 3x3 shader's taps at -2, -1, 0: as in wide_subconv)
            q.in_shift = frac_shift - 1;
            q.in_y0 = (in_v.pad << q.in_shift) - r;
            q.in_x0 = (in_v.pad << q.in_shift) + ((k == 3) ? -2 : -r);
        }
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
        q.in_amax = tin(0).amax;   // (timed in the form the frame will run: fp8 correction terms where the input has a range word)
        q.exact_split = net->sw.get("FYNHIP_EXACT_SPLIT") ? 1 : 0;
        const size_t halves = (size_t)k * q.cs * (out_v.f16 ? 1 : 3) * 64 * 8;
        q.wpack = rows_wpack_dev = net->dev_alloc(halves * 2, true);
        const bool always = net->sw.get("FYNHIP_FORCE_ROWS_WIDE_CONV") != nullptr;
        const char* at = net->sw.get("FYNHIP_AUTOTUNE");
        bool pick = true;
        char key[160];
        snprintf(key, sizeof(key), "rows:%d:%dx%d:%dx%d:k%d:cp%d:r%d:e%d:f%d", out_v.f16, d.in_channels, oc, oh, ow, k, in_v.cp, res_v ? 1 : 0, clamp ? 1 : 0, frac_shift);
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
    // weights of the row-rolling form: [step = ky*cs + sub][plane][lane][8 halves]; fp32 tensors: fp16 hi, fp16 lo and the
    // fp8 operands of the correction terms, as in the fragments of the 16-position forms
    void pack_rows(const float* w, float wmul) {
        const int cin = d.in_channels, npl = tout().v.f16 ? 1 : 3;
        const size_t frags = (size_t)k * rp.cs;
        std::vector<uint16_t> pack(frags * npl * 64 * 8, 0);
        std::vector<float> c8(npl == 3 ? frags * 64 * 16 : 0, 0.f);
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
                        const size_t frag = (size_t)(ky * rp.cs + sub), base = frag * npl * 64 * 8;
                        pack[base + (size_t)lane * 8 + j] = hi;
                        if (npl == 3) p16_lo_planes(pack.data() + base, c8.data() + (frag * 64 + lane) * 16, lane, j, v, hi);
                    }
                }
        upload_p16_pack(net, rows_wpack_dev, pack, c8, frags);
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
            if (conv_rows_supported(k, in_v.cp, oc, out_v.f16 != 0) && out_v.cp == 4 && !net->sw.get("FYNHIP_NO_ROWS_WIDE_CONV"))
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
            // (channels between a layer's count and the tensor's pitch hold zeros and meet zero weights)
            if (!only_kr && !p16 && same_storage && !sc.in_sub && conv_p16_supported(k, stride, dil, in_v.cp, oc, out_v.cp, out_v.f16 != 0) &&
                d.in_channels <= in_v.cp && (!res_v || (res_v->cp >= oc && res_v->cp % 8 == 0)) && !net->sw.get("FYNHIP_NO_P16_CONV"))
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
                     tout().v.f16 ? "f16 " : (conv_rows_uses_fp8(rp, false) ? "f16+fp8-split " : "f16x2-split "), rp.strips, rp.row_blocks, rp.rows_per_block, conv_rows_lds_bytes(rp, tout().v.f16 != 0));
            return mode + buf;
        }
        if (p16 && c4) {
            char buf[220];
            snprintf(buf, sizeof(buf), "conv_p16c4 %s (tap pairs of a 4-channel pixel) tile=32x%d(cout x pos) th=%d tw=%d blocks=%d tiles=%d lds=%zu steps=%d",
                     pp.f16 ? "f16" : (conv_p16c4_uses_fp8(pp, k) ? "f16+fp8-split" : "f16x2-split"), pp.tile_h * pp.tile_w * 4, pp.tile_h, pp.tile_w, pp.pos_groups * pp.cout_blocks, pp.tiles_x * pp.tiles_y * pp.cout_blocks,
                     conv_p16c4_lds_bytes(pp, k), c4_steps);
            return mode + buf + (conv_p16_stores_through(pp, 1) ? " stores=through" : "");
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
            return mode + buf + (conv_p16_stores_through(pp, 1) ? " stores=through" : "");
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

// =============================================================================================
// Explicit batch-norm
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

}  // namespace fynhip
