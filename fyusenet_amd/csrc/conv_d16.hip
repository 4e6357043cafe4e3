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

template <bool HS, int NCHK, int FW>
__global__ __launch_bounds__(256) void conv_d16_kernel(const ConvP16Params p) {
    constexpr int NPL = HS ? 1 : 2, NPASS = HS ? 1 : 3;
    typedef typename std::conditional<HS, _Float16, float>::type store_t;
    if (blockIdx.x == 0 && blockIdx.y == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    // this lane's position (positions beyond the last one repeat it and are not stored)
    const int npos = p.npos_y * p.npos_x;
    const int pos = blockIdx.x * 16 + mq;
    const bool okp = pos < npos;
    const int pc = okp ? pos : npos - 1;
    const int py = pc / p.npos_x, px = pc - py * p.npos_x;
    const store_t* in = reinterpret_cast<const store_t*>(p.in) + ((size_t)(py * p.stride + p.in_y0) * p.in_wp + px * p.stride + p.in_x0) * p.in_cp + kq * 8;
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HS, half8_t, RawF>::type raw_t;
    raw_t raw[NCHK];
#pragma unroll
    for (int c = 0; c < NCHK; c++) {
        // (channels behind the tensor's pitch -- the pitch is a multiple of 8, not of 32 -- read as zero)
        const bool okc = c * KC + kq * 8 < p.in_cp;
        const store_t* src = okc ? in + c * KC : reinterpret_cast<const store_t*>(p.in);
        if constexpr (HS) {
            raw[c] = *reinterpret_cast<const half8_t*>(src);
        } else {
            raw[c].a = *reinterpret_cast<const float4*>(src);
            raw[c].b = *reinterpret_cast<const float4*>(src + 4);
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
    const int f0 = blockIdx.y * 4 + w, fstep = 4 * p.cout_blocks;
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
    half8_t b[NCHK][NPL];
#pragma unroll
    for (int c = 0; c < NCHK; c++) {
        const bool okc = c * KC + kq * 8 < p.in_cp;
        if constexpr (HS) {
#pragma unroll
            for (int e = 0; e < 8; e++) b[c][0][e] = okc ? (_Float16)act_p16((float)raw[c][e], p.act) : (_Float16)0.f;
        } else {
            const float r[8] = {raw[c].a.x, raw[c].a.y, raw[c].a.z, raw[c].a.w, raw[c].b.x, raw[c].b.y, raw[c].b.z, raw[c].b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = okc ? act_p16(r[e], p.act) * in_scale : 0.f;
                b[c][0][e] = (_Float16)v;
                b[c][NPL - 1][e] = (_Float16)(v - (float)b[c][0][e]);
            }
        }
    }
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
int d16_fw(int chunks, int mfrags, int cout_blocks) {
    const int fw = (mfrags + 4 * cout_blocks - 1) / (4 * cout_blocks);
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
d16_fn pick_d16(int chunks, int mfrags, int cout_blocks) {
    const int fw = d16_fw<HS>(chunks, mfrags, cout_blocks);
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
    if (blockIdx.x == 0 && blockIdx.y == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    const int tyi = blockIdx.x / p.tiles_x, txi = blockIdx.x - tyi * p.tiles_x;
    const int ey0 = tyi * 4 * DWS - 1, ex0 = txi * 4 * DWS - 1;   // the window's first position in the expanded tensor
    // ---- depthwise phase operands (requested first: they are used last) ----
    const int t = threadIdx.x;
    const int dpos = t >> 4, dc = (t & 15) * 4;                   // output position of the tile, first of four channels of the block
    const int dch = blockIdx.y * 64 + dc;
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
    const int mf = blockIdx.y * 4 + w;
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
#pragma unroll
    for (int pf = 0; pf < NPF; pf++) {
        f32x4_t acc = (f32x4_t)(0.f);
#pragma unroll
        for (int c = 0; c < NCHK; c++) {
            const bool okc = c * KC + kq * 8 < p.in_cp;
            half8_t b[NPL];
            if constexpr (HS) {
#pragma unroll
                for (int e = 0; e < 8; e++) b[0][e] = okc ? (_Float16)act_p16((float)raw[pf][c][e], p.act) : (_Float16)0.f;
            } else {
                const float r[8] = {raw[pf][c].a.x, raw[pf][c].a.y, raw[pf][c].a.z, raw[pf][c].a.w, raw[pf][c].b.x, raw[pf][c].b.y, raw[pf][c].b.z, raw[pf][c].b.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float v = okc ? act_p16(r[e], p.act) * in_scale : 0.f;
                    b[0][e] = (_Float16)v;
                    b[NPL - 1][e] = (_Float16)(v - (float)b[0][e]);
                }
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

template <bool HS, int DWS>
d16_fn pick_e16dw(int chunks) {
    switch (chunks) {
        case 1: return conv_e16dw_kernel<HS, 1, DWS>;
        case 2: return conv_e16dw_kernel<HS, 2, DWS>;
        case 3: return conv_e16dw_kernel<HS, 3, DWS>;
        case 4: return conv_e16dw_kernel<HS, 4, DWS>;
        case 5: return conv_e16dw_kernel<HS, 5, DWS>;
        default: return nullptr;
    }
}
}  // namespace

bool conv_d16_supported(int k, int dil, int in_cp, int chunks, int cout, int out_cp) {
    return k == 1 && dil == 1 && in_cp % 8 == 0 && in_cp >= 8 && pick_d16<true>(chunks, 1, 1) != nullptr && in_cp <= chunks * KC && cout >= 4 && out_cp % 4 == 0 && out_cp >= cout;
}

// p.cin_chunks = 32-channel chunks (1..6, 8; channels behind in_cp read as zero), p.mfrags = fragments of 16 output
// channels (scale and bias hold 16*mfrags values; rows beyond out_cp are not stored), in_y0/in_x0 = input padding,
// p.stride = pixel step per position; p.cout_blocks (1 or more) workgroups of 256 threads per 16 positions, which
// share the fragments of output channels
int launch_conv_d16(const ConvP16Params& p, hipStream_t s) {
    if (p.cout_blocks < 1 || p.cout_blocks > 64) return -5;
    const d16_fn fn = p.f16 ? pick_d16<true>(p.cin_chunks, p.mfrags, p.cout_blocks) : pick_d16<false>(p.cin_chunks, p.mfrags, p.cout_blocks);
    const long long npos = (long long)p.npos_y * p.npos_x;
    if (!fn) return -1;
    if (p.in_cp > p.cin_chunks * KC || p.in_cp % 8 != 0 || p.in_cp < 8 || p.mfrags < 1 || p.stride < 1 || npos < 1 || npos > (1ll << 30) || p.out_cp % 4 != 0 || p.out_cp < 4 ||
        (p.res && (p.res_cp < p.out_cp || p.res_cp % 4 != 0)) || p.nreset < 0 || p.nreset > 4 || p.in_clamp || p.dw_in ||
        (long long)((p.npos_y - 1) * p.stride + p.in_y0) >= p.in_hp || (long long)((p.npos_x - 1) * p.stride + p.in_x0) >= p.in_wp || p.in_y0 < 0 || p.in_x0 < 0)
        return -5;
    hipLaunchKernelGGL(fn, dim3((unsigned)((npos + 15) / 16), (unsigned)p.cout_blocks), dim3(256), 0, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

bool conv_e16dw_supported(int in_cp, int chunks, int dw_stride) {
    return in_cp % 8 == 0 && in_cp >= 8 && chunks >= 1 && chunks <= 5 && in_cp <= chunks * KC && (dw_stride == 1 || dw_stride == 2);
}

// The 1x1 layer's parameters as for launch_conv_d16 (stride 1, no residual; wpack in that layout), dw_hp x dw_wp its
// output size, out* / npos_* the depthwise layer's tensor, tiles_x x tiles_y tiles of 4x4 of its positions, dw_*
// its weights [9][dw_cp], scale, bias, step and activation; dw_cp = out_cp = channels of both layers (multiple of 8)
int launch_conv_e16dw(const ConvP16Params& p, hipStream_t s) {
    if (!conv_e16dw_supported(p.in_cp, p.cin_chunks, p.dw_stride)) return -1;
    const d16_fn fn = p.f16 ? (p.dw_stride == 1 ? pick_e16dw<true, 1>(p.cin_chunks) : pick_e16dw<true, 2>(p.cin_chunks))
                            : (p.dw_stride == 1 ? pick_e16dw<false, 1>(p.cin_chunks) : pick_e16dw<false, 2>(p.cin_chunks));
    if (!fn) return -1;
    if (p.mfrags < 1 || p.stride != 1 || p.res || p.in_clamp || !p.dw_w || !p.dw_scale || !p.dw_bias || p.dw_cp % 8 != 0 || p.dw_cp != p.out_cp || p.dw_cp > 16 * p.mfrags + 15 ||
        p.dw_hp < 1 || p.dw_wp < 1 || p.dw_hp - 1 + p.in_y0 >= p.in_hp || p.dw_wp - 1 + p.in_x0 >= p.in_wp || p.in_y0 < 0 || p.in_x0 < 0 || p.npos_y < 1 || p.npos_x < 1 ||
        p.tiles_x * 4 < p.npos_x || p.tiles_y * 4 < p.npos_y || (p.npos_y - 1) * p.dw_stride >= p.dw_hp + 1 || (p.npos_x - 1) * p.dw_stride >= p.dw_wp + 1 ||
        (long long)p.tiles_x * p.tiles_y > (1ll << 30) || p.nreset < 0 || p.nreset > 4)
        return -5;
    hipLaunchKernelGGL(fn, dim3((unsigned)(p.tiles_x * p.tiles_y), (unsigned)((p.dw_cp + 63) / 64)), dim3(256), 0, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace fynhip
