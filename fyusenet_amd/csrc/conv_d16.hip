// 1x1 convolution on many positions and few input channels (the expand and project layers of an inverted-residual
// stack at its large resolutions, the pointwise layers of a classification net's first stage) with no LDS at all.
//
// Replaces, for such layers, the render passes of DeepConvLayer1x1::forward (fyusenet/gpu/deep/deepconvlayer1x1.cpp:
// 67-117).  A 1x1 layer has no halo, so the B fragment of v_mfma_f32_16x16x32_f16 -- 16 positions x 32 channels, a
// lane holding eight consecutive channels of one position -- is what a lane reads from the tensor with one 16-byte
// (fp16 tensors) or two 16-byte (fp32 tensors) loads.  A workgroup of four waves owns 16 consecutive positions (in
// row-major order over the output); every wave loads the positions' whole reduction (up to 8 chunks of 32 channels)
// into registers, converts it once (activation, fp16 or the hi/lo split of fp32 tensors) and then walks the fragments
// of 16 output channels w, w + 4, ... of its share: the chunk loop is NCHK x 1 or 3 MFMAs, and the fragment is scaled,
// added to its residual and stored straight from the accumulator layout (a lane holds four consecutive channels of its
// position).  Where a wave has at most four fragments and their weights fit 64 registers (FW > 0), weights, scale,
// bias and residual of all of them are requested together with the positions' channels: the kernel is one memory
// round trip, a few dozen MFMAs and the stores.  Otherwise (FW = 0) they come one fragment ahead of their use.  No
// staging waves, no barrier before the end, no transposition.  Weights: [cout fragment][chunk][plane][lane][8 halves], output channel 16*fragment + lane%16, input
// channel 32*chunk + 8*(lane/16) + j.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <type_traits>

#include "kernels.h"
#include "p16_common.h"
#include "range.h"

namespace fynhip {

namespace {
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

// DWS = 1 or 2: the layer's input is the output of a depthwise 3x3 layer with step DWS that is not read from memory but
// computed by every wave for its positions (nine texels of the depthwise layer's input per lane and chunk instead of
// one of its output; that layer's own arithmetic and rounding), as in conv_kr16_kernel's staging.
// KS = 3, 5 or 7: not a 1x1 layer but a KS x KS convolution on an input of at most four channels (a classification
// net's first layer; reference: gpu/deep/deepconvlayerNxN.cpp:129-211): a stored pixel is four channels, a lane's eight
// values of a k32 step are two taps in row-major order (tap 8*step + 2*(lane/16) + {0, 1}), gathered from the image
// with two loads; taps beyond the kernel and pixels outside the stored frame are zeros.  p.stride = step, in_y0 /
// in_x0 = stored coordinate of tap (0,0) of position (0,0) (may be negative), p.tile_h = KS.
template <bool HS, int NCHK, int FW, int DWS = 0, int KS = 0>
__global__ __launch_bounds__(256) void conv_d16_kernel(const ConvP16Params p) {
    static_assert(KS == 0 || (DWS == 0 && NCHK == (KS * KS + 7) / 8), "a small-input convolution: steps of eight taps");
    constexpr int NPL = HS ? 1 : 2, NPASS = HS ? 1 : 3;
    typedef typename std::conditional<HS, _Float16, float>::type store_t;
    if (blockIdx.x == 0 && blockIdx.y == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    // this lane's position (positions beyond the last one repeat it and are not stored)
    // p.wm = 4: the layer has no more fragments of output channels than grid rows, and the four waves of a workgroup take
    // four tiles of 16 positions instead of sharing the fragments of one (p.wm = 1)
    const int wfr = p.wm == 4 ? 0 : w, fpw = p.wm == 4 ? 1 : 4;   // this wave's first fragment inside the workgroup; fragments per workgroup and round
    const int npos = p.npos_y * p.npos_x;
    const int pos = (p.wm == 4 ? blockIdx.x * 4 + w : blockIdx.x) * 16 + mq;
    const bool okp = pos < npos;
    const int pc = okp ? pos : npos - 1;
    // (row and column without an integer division in front of the first request: the reciprocal of the row length comes
    // with the launch, one step of correction makes the quotient exact; beyond 2^22 positions the division is used)
    int py, px;
    if (npos <= (1 << 22)) {
        py = (int)(((float)pc + 0.5f) * p.rcp_tiles_x);
        px = pc - py * p.npos_x;
        if (px < 0) { py--; px += p.npos_x; }
        else if (px >= p.npos_x) { py++; px -= p.npos_x; }
    } else {
        py = pc / p.npos_x;
        px = pc - py * p.npos_x;
    }
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HS, half8_t, RawF>::type raw_t;
    constexpr int NT = DWS > 0 ? 9 : 1;   // texels per lane and chunk
    raw_t raw[NCHK][NT];
    unsigned okm = 0u;                    // (depthwise input) taps inside the stored frame
    if constexpr (DWS > 0) {
        const store_t* din = reinterpret_cast<const store_t*>(p.dw_in);
#pragma unroll
        for (int t = 0; t < 9; t++) {
            const int iy = py * DWS + t / 3 + p.dw_y0, ix = px * DWS + t % 3 + p.dw_x0;
            const bool ok = (unsigned)iy < (unsigned)p.dw_hp && (unsigned)ix < (unsigned)p.dw_wp;
            okm |= ok ? 1u << t : 0u;
            const store_t* tap = din + (ok ? ((size_t)iy * p.dw_wp + ix) * p.dw_cp : 0) + kq * 8;
#pragma unroll
            for (int c = 0; c < NCHK; c++) {
                const store_t* src = (c * KC + kq * 8 < p.in_cp) ? tap + c * KC : din;
                if constexpr (HS) {
                    raw[c][t] = *reinterpret_cast<const half8_t*>(src);
                } else {
                    raw[c][t].a = *reinterpret_cast<const float4*>(src);
                    raw[c][t].b = *reinterpret_cast<const float4*>(src + 4);
                }
            }
        }
    } else if constexpr (KS > 0) {
        const store_t* in = reinterpret_cast<const store_t*>(p.in);
        typedef typename std::conditional<HS, half4_t, float4>::type pix_t;
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            pix_t pix[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int t = c * 8 + 2 * kq + h;
                const int ty = t / KS, tx = t - ty * KS;
                const int iy = py * p.stride + ty + p.in_y0, ix = px * p.stride + tx + p.in_x0;
                const bool ok = t < KS * KS && (unsigned)iy < (unsigned)p.in_hp && (unsigned)ix < (unsigned)p.in_wp;
                pix[h] = *reinterpret_cast<const pix_t*>(in + (ok ? ((size_t)iy * p.in_wp + ix) * 4 : 0));
                if (!ok) {
                    if constexpr (HS) pix[h] = (half4_t)((_Float16)0.f);
                    else pix[h] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            if constexpr (HS) {
                raw[c][0] = half8_t{pix[0][0], pix[0][1], pix[0][2], pix[0][3], pix[1][0], pix[1][1], pix[1][2], pix[1][3]};
            } else {
                raw[c][0].a = pix[0];
                raw[c][0].b = pix[1];
            }
        }
    } else {
        const store_t* in = reinterpret_cast<const store_t*>(p.in) + ((size_t)(py * p.stride + p.in_y0) * p.in_wp + px * p.stride + p.in_x0) * p.in_cp + kq * 8;
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            // (channels behind the tensor's pitch -- the pitch is a multiple of 8, not of 32 -- read as zero)
            const bool okc = c * KC + kq * 8 < p.in_cp;
            const store_t* src = okc ? in + c * KC : reinterpret_cast<const store_t*>(p.in);
            if constexpr (HS) {
                raw[c][0] = *reinterpret_cast<const half8_t*>(src);
            } else {
                raw[c][0].a = *reinterpret_cast<const float4*>(src);
                raw[c][0].b = *reinterpret_cast<const float4*>(src + 4);
            }
        }
    }
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + lane * 16;
    constexpr unsigned wfrag = NCHK * NPL * 1024;
    typedef typename std::conditional<HS, half4_t, f32x4_t>::type res_t;
    const store_t* res = reinterpret_cast<const store_t*>(p.res);
    const size_t rpos = ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp + kq * 4;
    const size_t opos = ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp + kq * 4;
    auto w_load = [&](half8_t (&a)[NCHK][NPL], int frag) {
        if (frag < p.mfrags) {
#pragma unroll
            for (int c = 0; c < NCHK; c++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a[c][pl] = *reinterpret_cast<const half8_t*>(wbase + (size_t)frag * wfrag + (c * NPL + pl) * 1024);
        }
    };
    auto res_load = [&](int frag) {
        res_t r;
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = 0;
        // (the last fragment may reach beyond the tensor's channel pitch: those rows are neither read nor stored)
        if (res && frag < p.mfrags && frag * 16 + kq * 4 + 4 <= p.out_cp) r = *reinterpret_cast<const res_t*>(res + rpos + frag * 16);
        return r;
    };
    // (scale and bias hold 16*mfrags values or more)
    auto sb_load = [&](const float* base, int frag) { return frag < p.mfrags ? *reinterpret_cast<const f32x4_t*>(base + frag * 16 + kq * 4) : (f32x4_t)(0.f); };
    // (the fragments of output channels may be dealt to p.cout_blocks workgroups per tile: grid rows)
    const int f0 = blockIdx.y * fpw + wfr, fstep = fpw * p.cout_blocks;
    constexpr int NF = FW > 0 ? FW : 1;
    half8_t a_q[NF][NCHK][NPL];
    res_t r_q[NF];
    f32x4_t sc_q[NF], bi_q[NF];
#pragma unroll
    for (int j = 0; j < NF; j++) {
        w_load(a_q[j], f0 + fstep * j);
        r_q[j] = res_load(f0 + fstep * j);
        sc_q[j] = sb_load(p.scale, f0 + fstep * j);
        bi_q[j] = sb_load(p.bias, f0 + fstep * j);
    }
    // activation and conversion of the positions' channels
    float in_scale = 1.f, inv_in_scale = 1.f;
    if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    auto texel = [&](const raw_t& rw, float (&x)[8]) {
        if constexpr (HS) {
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = (float)rw[e];
        } else {
            x[0] = rw.a.x; x[1] = rw.a.y; x[2] = rw.a.z; x[3] = rw.a.w; x[4] = rw.b.x; x[5] = rw.b.y; x[6] = rw.b.z; x[7] = rw.b.w;
        }
    };
    _Float16 act_lo, act_hi;
    const bool half_act = HS && act_half_exact(p.act, act_lo, act_hi);
    half8_t b[NCHK][NPL];
#ifndef FYN_AFFINE_ON
#define FYN_AFFINE_ON 1
#endif
    const bool affine = FYN_AFFINE_ON && DWS == 0 && KS == 0 && p.in_mul != nullptr;
    auto convert = [&](auto kind_, auto aff_) {
    constexpr int KIND = decltype(kind_)::value;
    constexpr bool AFF = decltype(aff_)::value;   // (with the batch-norm layer in front: chosen once per wave, like the kind)   // (the activation's kind, chosen once per wave: act_kind)
#pragma unroll
    for (int c = 0; c < NCHK; c++) {
        const bool okc = KS > 0 || c * KC + kq * 8 < p.in_cp;
        float r[8];   // the layer's input values of this lane: from the tensor, or the depthwise layer's results
        if constexpr (DWS > 0) {
            const int ch = okc ? c * KC + kq * 8 : 0;
#pragma unroll
            for (int e = 0; e < 8; e++) r[e] = 0.f;
#pragma unroll
            for (int t = 0; t < 9; t++) {   // (ky outer, kx inner, fused multiply-add: the depthwise kernel's order)
                float x[8];
                texel(raw[c][t], x);
                const float4 w0 = *reinterpret_cast<const float4*>(p.dw_w + t * p.dw_cp + ch), w1 = *reinterpret_cast<const float4*>(p.dw_w + t * p.dw_cp + ch + 4);
                const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
                for (int e = 0; e < 8; e++) r[e] = fmaf(act_p16(((okm >> t) & 1u) ? x[e] : 0.f, p.dw_act), wv[e], r[e]);
            }
            const float4 s0 = *reinterpret_cast<const float4*>(p.dw_scale + ch), s1 = *reinterpret_cast<const float4*>(p.dw_scale + ch + 4);
            const float4 b0 = *reinterpret_cast<const float4*>(p.dw_bias + ch), b1 = *reinterpret_cast<const float4*>(p.dw_bias + ch + 4);
            const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w}, bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                r[e] = r[e] * sv[e] + bv[e];
                if constexpr (HS) r[e] = (float)(_Float16)r[e];   // (what the depthwise layer would have stored)
            }
        } else {
            texel(raw[c][0], r);
            if constexpr (KS == 0) {
                if constexpr (AFF) {   // a batch-norm layer in front, applied here: x * in_mul[channel] + in_add[channel]
                    const int ch = okc ? c * KC + kq * 8 : 0;
                    const float4 m0 = *reinterpret_cast<const float4*>(p.in_mul + ch), m1 = *reinterpret_cast<const float4*>(p.in_mul + ch + 4);
                    const float4 a0 = *reinterpret_cast<const float4*>(p.in_add + ch), a1 = *reinterpret_cast<const float4*>(p.in_add + ch + 4);
                    const float mv[8] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w}, av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        r[e] = r[e] * mv[e] + av[e];
                        if constexpr (HS) r[e] = (float)(_Float16)r[e];   // (what the batch-norm layer would have stored)
                    }
                }
            }
        }
        if constexpr (HS) {
            if (DWS == 0 && half_act && !AFF) {
                b[c][0] = okc ? act_half(raw[c][0], act_lo, act_hi) : (half8_t)((_Float16)0.f);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) b[c][0][e] = okc ? (_Float16)act_p16(r[e], p.act) : (_Float16)0.f;
            }
        } else {
            split8<KIND>(r, okc, p.act, in_scale, b[c][0], b[c][NPL - 1]);
        }
    }
    };
    if (affine) {
        if (HS || p.act.kind == ACT_LEAKY || p.act.kind == ACT_CLIP) convert(std::integral_constant<int, ACT_LEAKY>(), std::true_type());
        else if (p.act.kind == ACT_RELU) convert(std::integral_constant<int, ACT_RELU>(), std::true_type());
        else convert(std::integral_constant<int, ACT_NONE>(), std::true_type());
    } else if (HS || p.act.kind == ACT_LEAKY || p.act.kind == ACT_CLIP) convert(std::integral_constant<int, ACT_LEAKY>(), std::false_type());
    else if (p.act.kind == ACT_RELU) convert(std::integral_constant<int, ACT_RELU>(), std::false_type());
    else convert(std::integral_constant<int, ACT_NONE>(), std::false_type());
    store_t* out = reinterpret_cast<store_t*>(p.out);
    float vmax = 0.f;
    auto fragment = [&](int f, const half8_t (&a)[NCHK][NPL], const res_t& rcur, const f32x4_t& sc, const f32x4_t& bi) {
        f32x4_t acc = (f32x4_t)(0.f);
#pragma unroll
        for (int c = 0; c < NCHK; c++)
#pragma unroll
            for (int i = 0; i < NPASS; i++) {
                const int apl = (i == 1) ? 1 : 0, bpl = (i == 2) ? 1 : 0;
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[c][apl], b[c][bpl], acc, 0, 0, 0);
            }
        const int ch = f * 16 + kq * 4;
        const bool okc = okp && ch + 4 <= p.out_cp;
        f32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = acc[e] * (sc[e] * acc_mul) + bi[e];
        if (res) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float r = (float)rcur[e];
                if (p.res_relu) r = fmaxf(r, 0.f);
                if (p.res_scale) r *= sc[e];
                v[e] += r;
            }
        }
        if constexpr (HS) {
            half4_t hv;
#pragma unroll
            for (int e = 0; e < 4; e++) hv[e] = (_Float16)v[e];
            if (okc) *reinterpret_cast<half4_t*>(out + opos + f * 16) = hv;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) vmax = fmaxf(vmax, okc ? fabsf(v[e]) : 0.f);
            if (okc) *reinterpret_cast<f32x4_t*>(out + opos + f * 16) = v;
        }
    };
    if constexpr (FW > 0) {
#pragma unroll
        for (int j = 0; j < FW; j++)
            if (f0 + fstep * j < p.mfrags) fragment(f0 + fstep * j, a_q[j], r_q[j], sc_q[j], bi_q[j]);
    } else {
        for (int f = f0; f < p.mfrags; f += fstep) {
            half8_t a[NCHK][NPL];
#pragma unroll
            for (int c = 0; c < NCHK; c++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a[c][pl] = a_q[0][c][pl];
            const res_t rcur = r_q[0];
            const f32x4_t sc = sc_q[0], bi = bi_q[0];
            w_load(a_q[0], f + fstep);
            r_q[0] = res_load(f + fstep);
            sc_q[0] = sb_load(p.scale, f + fstep);
            bi_q[0] = sb_load(p.bias, f + fstep);
            fragment(f, a, rcur, sc, bi);
        }
    }
    if (!HS && p.out_amax) range_publish_block256(p.out_amax, vmax);
}

typedef void (*d16_fn)(const ConvP16Params);
// fragments of 16 output channels per wave whose weights are all requested up front: as many as the layer has when they
// fit 64 registers, else 0 (one fragment ahead)
template <bool HS>
int d16_fw(int chunks, int mfrags, int cout_blocks, int wm) {
    const int per_round = (wm == 4 ? 1 : 4) * cout_blocks;
    const int fw = (mfrags + per_round - 1) / per_round;
    return (fw <= 4 && chunks * (HS ? 1 : 2) * fw <= 16) ? fw : 0;
}
template <bool HS, int NCHK>
d16_fn pick_d16_fw(int fw) {
    switch (fw) {
        case 0: return conv_d16_kernel<HS, NCHK, 0>;
        case 1: return conv_d16_kernel<HS, NCHK, 1>;
        case 2: return conv_d16_kernel<HS, NCHK, 2>;
        case 3: return conv_d16_kernel<HS, NCHK, 3>;
        case 4: return conv_d16_kernel<HS, NCHK, 4>;
        default: return nullptr;
    }
}
template <bool HS>
d16_fn pick_d16(int chunks, int mfrags, int cout_blocks, int wm) {
    const int fw = d16_fw<HS>(chunks, mfrags, cout_blocks, wm);
    switch (chunks) {
        case 1: return pick_d16_fw<HS, 1>(fw);
        case 2: return pick_d16_fw<HS, 2>(fw);
        case 3: return pick_d16_fw<HS, 3>(fw);
        case 4: return pick_d16_fw<HS, 4>(fw);
        case 5: return pick_d16_fw<HS, 5>(fw);
        case 6: return pick_d16_fw<HS, 6>(fw);
        case 8: return pick_d16_fw<HS, 8>(fw);
        default: return nullptr;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// A 1x1 layer and the depthwise 3x3 layer behind it (the first half of an inverted-residual block: expand, then the
// depthwise convolution with step DWS; reference: gpu/deep/deepconvlayer1x1.cpp:67-117 followed by
// gpu/deep/deepdwconvlayer3x3.cpp:67-102) as one launch.  A workgroup owns a tile of 4x4 positions of the depthwise
// layer's output and a block of 64 expanded channels (grid rows): the depthwise layer needs the expanded tensor on a
// window of WIN x WIN positions, WIN = 3*DWS + 3, and every expanded channel depends on the 1x1 layer's input only, so
// the four waves (16 channels each) compute that window -- its positions are B fragments read straight from the 1x1
// layer's input, as above -- scale it, round it to the storage type, apply the depthwise layer's activation (window
// positions outside the expanded tensor are its zero padding) and leave it in LDS; behind one barrier every thread
// computes four channels of one output position with the depthwise kernel's arithmetic (layers_direct.hip).  The
// expanded tensor is never written.  Parameters: those of the 1x1 layer as for conv_d16_kernel, dw_hp x dw_wp = its
// output size (net, without padding), out* = the depthwise layer's tensor, npos_* its size, dw_w / dw_scale / dw_bias /
// dw_cp / dw_act the depthwise layer's.
template <bool HS, int NCHK, int DWS>
__global__ __launch_bounds__(256) void conv_e16dw_kernel(const ConvP16Params p) {
    constexpr int NPL = HS ? 1 : 2, NPASS = HS ? 1 : 3;
    constexpr int WIN = 3 * DWS + 3, NWIN = WIN * WIN, NPF = (NWIN + 15) / 16;
    typedef typename std::conditional<HS, _Float16, float>::type store_t;
    __shared__ __align__(16) float win[NWIN][68];   // (68: the sixteen positions of a fragment write distinct banks)
    if ((blockIdx.x | blockIdx.y | blockIdx.z) == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    const int txi = blockIdx.x, tyi = blockIdx.y;   // (a grid of tile columns x tile rows x channel blocks: no division in front of the first request)
    const int ey0 = tyi * 4 * DWS - 1, ex0 = txi * 4 * DWS - 1;   // the window's first position in the expanded tensor
    // ---- depthwise phase operands (requested first: they are used last) ----
    const int t = threadIdx.x;
    const int dpos = t >> 4, dc = (t & 15) * 4;                   // output position of the tile, first of four channels of the block
    const int dch = blockIdx.z * 64 + dc;
    const bool dch_ok = dch + 4 <= p.dw_cp;
    f32x4_t dww[9], dsc, dbi;
#pragma unroll
    for (int i = 0; i < 9; i++) dww[i] = *reinterpret_cast<const f32x4_t*>(p.dw_w + i * p.dw_cp + (dch_ok ? dch : 0));
    dsc = *reinterpret_cast<const f32x4_t*>(p.dw_scale + (dch_ok ? dch : 0));
    dbi = *reinterpret_cast<const f32x4_t*>(p.dw_bias + (dch_ok ? dch : 0));
    // ---- the window's positions: B fragments from the 1x1 layer's input ----
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HS, half8_t, RawF>::type raw_t;
    raw_t raw[NPF][NCHK];
    bool inside[NPF];
#pragma unroll
    for (int pf = 0; pf < NPF; pf++) {
        const int wp_ = min(pf * 16 + mq, NWIN - 1);
        const int ey = ey0 + wp_ / WIN, ex = ex0 + wp_ % WIN;
        inside[pf] = (unsigned)ey < (unsigned)p.dw_hp && (unsigned)ex < (unsigned)p.dw_wp;
        const int cy = min(max(ey, 0), p.dw_hp - 1), cx = min(max(ex, 0), p.dw_wp - 1);
        const store_t* in = reinterpret_cast<const store_t*>(p.in) + ((size_t)(cy + p.in_y0) * p.in_wp + cx + p.in_x0) * p.in_cp + kq * 8;
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            const bool okc = c * KC + kq * 8 < p.in_cp;
            const store_t* src = okc ? in + c * KC : reinterpret_cast<const store_t*>(p.in);
            if constexpr (HS) {
                raw[pf][c] = *reinterpret_cast<const half8_t*>(src);
            } else {
                raw[pf][c].a = *reinterpret_cast<const float4*>(src);
                raw[pf][c].b = *reinterpret_cast<const float4*>(src + 4);
            }
        }
    }
    // ---- this wave's fragment of expanded channels: weights, scale, bias ----
    const int mf = blockIdx.z * 4 + w;
    const bool mf_ok = mf < p.mfrags;
    half8_t a[NCHK][NPL];
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)(mf_ok ? mf : 0) * (NCHK * NPL * 1024) + lane * 16;
#pragma unroll
    for (int c = 0; c < NCHK; c++)
#pragma unroll
        for (int pl = 0; pl < NPL; pl++) a[c][pl] = *reinterpret_cast<const half8_t*>(wbase + (c * NPL + pl) * 1024);
    const f32x4_t sc = *reinterpret_cast<const f32x4_t*>(p.scale + (mf_ok ? mf : 0) * 16 + kq * 4);
    const f32x4_t bi = *reinterpret_cast<const f32x4_t*>(p.bias + (mf_ok ? mf : 0) * 16 + kq * 4);
    float in_scale = 1.f, inv_in_scale = 1.f;
    if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    _Float16 act_lo, act_hi;
    const bool half_act = HS && act_half_exact(p.act, act_lo, act_hi);
    auto window = [&](auto kind_) {
    constexpr int KIND = decltype(kind_)::value;   // (the 1x1 layer's activation kind, chosen once per wave: act_kind)
#pragma unroll
    for (int pf = 0; pf < NPF; pf++) {
        f32x4_t acc = (f32x4_t)(0.f);
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            const bool okc = c * KC + kq * 8 < p.in_cp;
            half8_t b[NPL];
            if constexpr (HS) {
                if (half_act) {
                    b[0] = okc ? act_half(raw[pf][c], act_lo, act_hi) : (half8_t)((_Float16)0.f);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) b[0][e] = okc ? (_Float16)act_p16((float)raw[pf][c][e], p.act) : (_Float16)0.f;
                }
            } else {
                const float r[8] = {raw[pf][c].a.x, raw[pf][c].a.y, raw[pf][c].a.z, raw[pf][c].a.w, raw[pf][c].b.x, raw[pf][c].b.y, raw[pf][c].b.z, raw[pf][c].b.w};
                split8<KIND>(r, okc, p.act, in_scale, b[0], b[NPL - 1]);
            }
#pragma unroll
            for (int i = 0; i < NPASS; i++) {
                const int apl = (i == 1) ? 1 : 0, bpl = (i == 2) ? 1 : 0;
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[c][apl], b[bpl], acc, 0, 0, 0);
            }
        }
        // the expanded value as the 1x1 layer would have stored it, then the depthwise layer's activation on its fetch
        const int wp_ = pf * 16 + mq;
        f32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float x = acc[e] * (sc[e] * acc_mul) + bi[e];
            if constexpr (HS) x = (float)(_Float16)x;
            v[e] = act_p16((inside[pf] && mf_ok) ? x : 0.f, p.dw_act);
        }
        if (wp_ < NWIN) *reinterpret_cast<f32x4_t*>(&win[wp_][w * 16 + kq * 4]) = v;
    }
    };
    if (HS || p.act.kind == ACT_LEAKY || p.act.kind == ACT_CLIP) window(std::integral_constant<int, ACT_LEAKY>());
    else if (p.act.kind == ACT_RELU) window(std::integral_constant<int, ACT_RELU>());
    else window(std::integral_constant<int, ACT_NONE>());
    __syncthreads();
    // ---- depthwise 3x3 on the window: one position, four channels per thread (ky outer, kx inner, fused multiply-add) ----
    const int py = dpos >> 2, px = dpos & 3;
    f32x4_t dacc = (f32x4_t)(0.f);
#pragma unroll
    for (int ky = 0; ky < 3; ky++)
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const f32x4_t x = *reinterpret_cast<const f32x4_t*>(&win[(py * DWS + ky) * WIN + px * DWS + kx][dc]);
#pragma unroll
            for (int e = 0; e < 4; e++) dacc[e] = fmaf(x[e], dww[ky * 3 + kx][e], dacc[e]);
        }
    const int oy = tyi * 4 + py, ox = txi * 4 + px;
    if (oy < p.npos_y && ox < p.npos_x && dch_ok) {
        store_t* out = reinterpret_cast<store_t*>(p.out) + ((size_t)(p.out_off_y + oy) * p.out_wp + p.out_off_x + ox) * p.out_cp + dch;
        f32x4_t o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = dacc[e] * dsc[e] + dbi[e];
        if constexpr (HS) {
            half4_t hv;
#pragma unroll
            for (int e = 0; e < 4; e++) hv[e] = (_Float16)o[e];
            *reinterpret_cast<half4_t*>(out) = hv;
        } else {
            *reinterpret_cast<f32x4_t*>(out) = o;
        }
    }
}


// The same with a workgroup per 16 expanded channels (p.wm = 2; grid rows = fragments): for layers with few tiles, where
// blocks of 64 channels leave most of the chip idle and every wave with a long chain of fragments.  All four waves work
// on the one fragment of channels and deal the window's position fragments among themselves (wave w takes w, w + 4);
// behind the barrier a thread computes one channel of one output position.
template <bool HS, int NCHK, int DWS>
__global__ __launch_bounds__(256) void conv_e16dw_narrow_kernel(const ConvP16Params p) {
    constexpr int NPL = HS ? 1 : 2, NPASS = HS ? 1 : 3;
    constexpr int WIN = 3 * DWS + 3, NWIN = WIN * WIN, NPF = (NWIN + 15) / 16, PFW = (NPF + 3) / 4;
    typedef typename std::conditional<HS, _Float16, float>::type store_t;
    __shared__ __align__(16) float win[NWIN][20];   // (20: the sixteen positions of a fragment write distinct banks)
    if ((blockIdx.x | blockIdx.y | blockIdx.z) == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    const int txi = blockIdx.x, tyi = blockIdx.y;   // (a grid of tile columns x tile rows x channel blocks: no division in front of the first request)
    const int ey0 = tyi * 4 * DWS - 1, ex0 = txi * 4 * DWS - 1;
    const int mf = blockIdx.z;
    // depthwise phase operands (requested first: they are used last)
    const int t = threadIdx.x;
    const int dpos = t >> 4, dch = mf * 16 + (t & 15);
    const bool dch_ok = dch < p.dw_cp;
    float dww[9];
#pragma unroll
    for (int i = 0; i < 9; i++) dww[i] = p.dw_w[i * p.dw_cp + (dch_ok ? dch : 0)];
    const float dsc = p.dw_scale[dch_ok ? dch : 0], dbi = p.dw_bias[dch_ok ? dch : 0];
    // this wave's position fragments of the window
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HS, half8_t, RawF>::type raw_t;
    raw_t raw[PFW][NCHK];
    bool inside[PFW];
#pragma unroll
    for (int j = 0; j < PFW; j++) {
        const int pf = w + 4 * j;
        const int wp_ = min(pf * 16 + mq, NWIN - 1);
        const int ey = ey0 + wp_ / WIN, ex = ex0 + wp_ % WIN;
        inside[j] = (unsigned)ey < (unsigned)p.dw_hp && (unsigned)ex < (unsigned)p.dw_wp;
        const int cy = min(max(ey, 0), p.dw_hp - 1), cx = min(max(ex, 0), p.dw_wp - 1);
        const store_t* in = reinterpret_cast<const store_t*>(p.in) + ((size_t)(cy + p.in_y0) * p.in_wp + cx + p.in_x0) * p.in_cp + kq * 8;
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            const bool okc = c * KC + kq * 8 < p.in_cp;
            const store_t* src = okc ? in + c * KC : reinterpret_cast<const store_t*>(p.in);
            if constexpr (HS) {
                raw[j][c] = *reinterpret_cast<const half8_t*>(src);
            } else {
                raw[j][c].a = *reinterpret_cast<const float4*>(src);
                raw[j][c].b = *reinterpret_cast<const float4*>(src + 4);
            }
        }
    }
    half8_t a[NCHK][NPL];
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)mf * (NCHK * NPL * 1024) + lane * 16;
#pragma unroll
    for (int c = 0; c < NCHK; c++)
#pragma unroll
        for (int pl = 0; pl < NPL; pl++) a[c][pl] = *reinterpret_cast<const half8_t*>(wbase + (c * NPL + pl) * 1024);
    const f32x4_t sc = *reinterpret_cast<const f32x4_t*>(p.scale + mf * 16 + kq * 4);
    const f32x4_t bi = *reinterpret_cast<const f32x4_t*>(p.bias + mf * 16 + kq * 4);
    float in_scale = 1.f, inv_in_scale = 1.f;
    if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    _Float16 act_lo, act_hi;
    const bool half_act = HS && act_half_exact(p.act, act_lo, act_hi);
    auto window = [&](auto kind_) {
    constexpr int KIND = decltype(kind_)::value;
#pragma unroll
    for (int j = 0; j < PFW; j++) {
        const int pf = w + 4 * j;
        if (pf >= NPF) continue;
        f32x4_t acc = (f32x4_t)(0.f);
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            const bool okc = c * KC + kq * 8 < p.in_cp;
            half8_t b[NPL];
            if constexpr (HS) {
                if (half_act) {
                    b[0] = okc ? act_half(raw[j][c], act_lo, act_hi) : (half8_t)((_Float16)0.f);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) b[0][e] = okc ? (_Float16)act_p16((float)raw[j][c][e], p.act) : (_Float16)0.f;
                }
            } else {
                const float r[8] = {raw[j][c].a.x, raw[j][c].a.y, raw[j][c].a.z, raw[j][c].a.w, raw[j][c].b.x, raw[j][c].b.y, raw[j][c].b.z, raw[j][c].b.w};
                split8<KIND>(r, okc, p.act, in_scale, b[0], b[NPL - 1]);
            }
#pragma unroll
            for (int i = 0; i < NPASS; i++) {
                const int apl = (i == 1) ? 1 : 0, bpl = (i == 2) ? 1 : 0;
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[c][apl], b[bpl], acc, 0, 0, 0);
            }
        }
        const int wp_ = pf * 16 + mq;
        f32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float x = acc[e] * (sc[e] * acc_mul) + bi[e];
            if constexpr (HS) x = (float)(_Float16)x;
            v[e] = act_p16(inside[j] ? x : 0.f, p.dw_act);
        }
        if (wp_ < NWIN) *reinterpret_cast<f32x4_t*>(&win[wp_][kq * 4]) = v;
    }
    };
    if (HS || p.act.kind == ACT_LEAKY || p.act.kind == ACT_CLIP) window(std::integral_constant<int, ACT_LEAKY>());
    else if (p.act.kind == ACT_RELU) window(std::integral_constant<int, ACT_RELU>());
    else window(std::integral_constant<int, ACT_NONE>());
    __syncthreads();
    const int py = dpos >> 2, px = dpos & 3;
    float dacc = 0.f;
#pragma unroll
    for (int ky = 0; ky < 3; ky++)
#pragma unroll
        for (int kx = 0; kx < 3; kx++) dacc = fmaf(win[(py * DWS + ky) * WIN + px * DWS + kx][t & 15], dww[ky * 3 + kx], dacc);
    const int oy = tyi * 4 + py, ox = txi * 4 + px;
    if (oy < p.npos_y && ox < p.npos_x && dch_ok) {
        store_t* out = reinterpret_cast<store_t*>(p.out) + ((size_t)(p.out_off_y + oy) * p.out_wp + p.out_off_x + ox) * p.out_cp + dch;
        *out = (store_t)(dacc * dsc + dbi);
    }
}

template <bool HS, int DWS>
d16_fn pick_e16dw(int chunks, bool narrow) {
    switch (chunks) {
        case 1: return narrow ? conv_e16dw_narrow_kernel<HS, 1, DWS> : conv_e16dw_kernel<HS, 1, DWS>;
        case 2: return narrow ? conv_e16dw_narrow_kernel<HS, 2, DWS> : conv_e16dw_kernel<HS, 2, DWS>;
        case 3: return narrow ? conv_e16dw_narrow_kernel<HS, 3, DWS> : conv_e16dw_kernel<HS, 3, DWS>;
        case 4: return narrow ? conv_e16dw_narrow_kernel<HS, 4, DWS> : conv_e16dw_kernel<HS, 4, DWS>;
        case 5: return narrow ? conv_e16dw_narrow_kernel<HS, 5, DWS> : conv_e16dw_kernel<HS, 5, DWS>;
        default: return nullptr;
    }
}
// with a depthwise layer in front: up to 96 channels, one fragment per wave up front or one ahead
template <bool HS, int DWS>
d16_fn pick_d16_dw(int chunks, bool one) {
    switch (chunks) {
        case 1: return one ? conv_d16_kernel<HS, 1, 1, DWS> : conv_d16_kernel<HS, 1, 0, DWS>;
        case 2: return one ? conv_d16_kernel<HS, 2, 1, DWS> : conv_d16_kernel<HS, 2, 0, DWS>;
        case 3: return one ? conv_d16_kernel<HS, 3, 1, DWS> : conv_d16_kernel<HS, 3, 0, DWS>;
        default: return nullptr;
    }
}
// a K x K convolution on at most four input channels: one fragment per wave and round
template <bool HS>
d16_fn pick_d16_ks(int ks) {
    switch (ks) {
        case 3: return conv_d16_kernel<HS, 2, 1, 0, 3>;
        case 5: return conv_d16_kernel<HS, 4, 1, 0, 5>;
        case 7: return conv_d16_kernel<HS, 7, 1, 0, 7>;
        default: return nullptr;
    }
}
}  // namespace

bool conv_d16_small_supported(int k, int dil, int in_cp, int cout, int out_cp) {
    return (k == 3 || k == 5 || k == 7) && dil == 1 && in_cp == 4 && cout >= 4 && out_cp % 4 == 0 && out_cp >= cout;
}

bool conv_d16_dw_supported(int chunks, int dw_stride) { return chunks >= 1 && chunks <= 3 && (dw_stride == 1 || dw_stride == 2); }

bool conv_d16_supported(int k, int dil, int in_cp, int chunks, int cout, int out_cp) {
    return k == 1 && dil == 1 && in_cp % 8 == 0 && in_cp >= 8 && pick_d16<true>(chunks, 1, 1, 1) != nullptr && in_cp <= chunks * KC && cout >= 4 && out_cp % 4 == 0 && out_cp >= cout;
}

// p.cin_chunks = 32-channel chunks (1..6, 8; channels behind in_cp read as zero), p.mfrags = fragments of 16 output
// channels (scale and bias hold 16*mfrags values; rows beyond out_cp are not stored), in_y0/in_x0 = input padding,
// p.stride = pixel step per position; p.cout_blocks (1 or more) workgroups of 256 threads per 16 positions, which
// share the fragments of output channels, or (p.wm = 4 instead of 1) one wave per 16 positions and grid row
int launch_conv_d16(const ConvP16Params& p, hipStream_t s) {
    if (p.cout_blocks < 1 || p.cout_blocks > 64 || (p.wm != 1 && p.wm != 4)) return -5;
    d16_fn fn = p.f16 ? pick_d16<true>(p.cin_chunks, p.mfrags, p.cout_blocks, p.wm) : pick_d16<false>(p.cin_chunks, p.mfrags, p.cout_blocks, p.wm);
    const int ks = p.tile_h;   // 0: a 1x1 layer
    if (ks) {
        // (p.cin_chunks = steps of eight taps; every wave has at most one fragment per round)
        if (p.dw_in || p.in_cp != 4 || p.cin_chunks != (ks * ks + 7) / 8 || p.mfrags > (p.wm == 4 ? 1 : 4) * p.cout_blocks) return -5;
        fn = p.f16 ? pick_d16_ks<true>(ks) : pick_d16_ks<false>(ks);
    }
    if (p.dw_in) {
        // (the depthwise layer's tensor has the 1x1 layer's channels; the 1x1 layer does not step)
        if (!conv_d16_dw_supported(p.cin_chunks, p.dw_stride) || !p.dw_w || !p.dw_scale || !p.dw_bias || p.dw_cp != p.in_cp || p.stride != 1 || p.dw_hp < 1 || p.dw_wp < 1) return -5;
        const bool one = p.mfrags <= (p.wm == 4 ? 1 : 4) * p.cout_blocks;
        fn = p.f16 ? (p.dw_stride == 1 ? pick_d16_dw<true, 1>(p.cin_chunks, one) : pick_d16_dw<true, 2>(p.cin_chunks, one))
                   : (p.dw_stride == 1 ? pick_d16_dw<false, 1>(p.cin_chunks, one) : pick_d16_dw<false, 2>(p.cin_chunks, one));
    }
    // (a batch-norm layer applied on fetch: plain 1x1 launches only, both arrays or none)
    if ((p.in_mul != nullptr) != (p.in_add != nullptr) || (p.in_mul && (ks || p.dw_in))) return -5;
    const long long npos = (long long)p.npos_y * p.npos_x;
    if (!fn) return -1;
    if ((!ks && (p.in_cp > p.cin_chunks * KC || p.in_cp % 8 != 0 || p.in_cp < 8)) || p.mfrags < 1 || p.stride < 1 || npos < 1 || npos > (1ll << 30) || p.out_cp % 4 != 0 || p.out_cp < 4 ||
        (p.res && (p.res_cp < p.out_cp || p.res_cp % 4 != 0)) || p.nreset < 0 || p.nreset > 4 || p.in_clamp ||
        (!ks && ((long long)((p.npos_y - 1) * p.stride + p.in_y0) >= p.in_hp || (long long)((p.npos_x - 1) * p.stride + p.in_x0) >= p.in_wp || p.in_y0 < 0 || p.in_x0 < 0)))
        return -5;
    const long long per_wg = 16 * p.wm;
    ConvP16Params q = p;
    q.rcp_tiles_x = 1.0f / (float)p.npos_x;   // (this kernel's use of the field: the reciprocal of a row of positions)
    hipLaunchKernelGGL(fn, dim3((unsigned)((npos + per_wg - 1) / per_wg), (unsigned)p.cout_blocks), dim3(256), 0, s, q);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

bool conv_e16dw_supported(int in_cp, int chunks, int dw_stride) {
    return in_cp % 8 == 0 && in_cp >= 8 && chunks >= 1 && chunks <= 5 && in_cp <= chunks * KC && (dw_stride == 1 || dw_stride == 2);
}

// The 1x1 layer's parameters as for launch_conv_d16 (stride 1, no residual; wpack in that layout), dw_hp x dw_wp its
// output size, out* / npos_* the depthwise layer's tensor, tiles_x x tiles_y tiles of 4x4 of its positions, dw_*
// its weights [9][dw_cp], scale, bias, step and activation; dw_cp = out_cp = channels of both layers (multiple of 8);
// p.wm = 2: a workgroup per 16 expanded channels instead of 64
int launch_conv_e16dw(const ConvP16Params& p, hipStream_t s) {
    if (!conv_e16dw_supported(p.in_cp, p.cin_chunks, p.dw_stride)) return -1;
    const bool narrow = p.wm == 2;   // a workgroup per 16 expanded channels instead of 64
    const d16_fn fn = p.f16 ? (p.dw_stride == 1 ? pick_e16dw<true, 1>(p.cin_chunks, narrow) : pick_e16dw<true, 2>(p.cin_chunks, narrow))
                            : (p.dw_stride == 1 ? pick_e16dw<false, 1>(p.cin_chunks, narrow) : pick_e16dw<false, 2>(p.cin_chunks, narrow));
    if (!fn) return -1;
    if (p.mfrags < 1 || p.stride != 1 || p.res || p.in_clamp || !p.dw_w || !p.dw_scale || !p.dw_bias || p.dw_cp % 8 != 0 || p.dw_cp != p.out_cp || p.dw_cp > 16 * p.mfrags + 15 ||
        p.dw_hp < 1 || p.dw_wp < 1 || p.dw_hp - 1 + p.in_y0 >= p.in_hp || p.dw_wp - 1 + p.in_x0 >= p.in_wp || p.in_y0 < 0 || p.in_x0 < 0 || p.npos_y < 1 || p.npos_x < 1 ||
        p.tiles_x * 4 < p.npos_x || p.tiles_y * 4 < p.npos_y || (p.npos_y - 1) * p.dw_stride >= p.dw_hp + 1 || (p.npos_x - 1) * p.dw_stride >= p.dw_wp + 1 ||
        (long long)p.tiles_x * p.tiles_y > (1ll << 30) || p.tiles_y > 65535 || p.mfrags > 65535 || p.nreset < 0 || p.nreset > 4)
        return -5;
    hipLaunchKernelGGL(fn, dim3((unsigned)p.tiles_x, (unsigned)p.tiles_y, (unsigned)(narrow ? p.mfrags : (p.dw_cp + 63) / 64)), dim3(256), 0, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace fynhip
