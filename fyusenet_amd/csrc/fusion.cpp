// Graph-rewrite passes run once when a network is set up: layers whose work a neighbouring convolution launch can
// take over (depthwise convolutions, 1x1 projections of a residual branch, plain batch-norm layers) are folded into
// that launch, subject to the liveness of the tensors whose reads or writes move to another layer's slot.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "layer_classes.h"

namespace fynhip {

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


}  // namespace fynhip
