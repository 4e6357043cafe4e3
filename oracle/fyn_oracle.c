/*
 * CPU oracle for the FyuseNet GPU layer stack.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file;
 * it is used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py as
 * the checker / reported CPU baseline.
 *
 * Every function restates, in plain C on channel-wise (CHW) fp32 arrays -- the format
 * GPULayerBase::copyResult hands to the reference's unit tests
 * (fyusenet/gpu/gpulayerbase.cpp:525-564) -- the arithmetic that the reference's layers define.
 * The reference file:line each function follows is cited at the function.  Accumulation is done in
 * double so that the oracle is "truth" for the fp32 tolerance checks; this changes no definition.
 *
 * Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):
 *   fyo_conv2d        reference known-answer patterns (convlayertests.cpp:165-182,242-261,
 *                     networktests.cpp:85-97) + torch.nn.functional.conv2d in fp64
 *   fyo_fracconv      fyo_conv2d (pinned above) on a numpy.repeat up-sampled input, the exact identity of its
 *                     sampling rule, + a float restatement of the proxy polygon's texture coordinates on
 *                     tiny inputs (no reference test exists)
 *   fyo_dwconv        conv2d(groups=C) fp64 + brute force          (no reference test exists)
 *   fyo_transconv     conv_transpose2d(stride=2) fp64 + brute force (no reference test exists)
 *   fyo_gemm          reference pattern misctests.cpp:238-265 + torch linear fp64
 *   fyo_maxpool/avg   max_pool2d/avg_pool2d fp64 for pool==stride (pooltests.cpp:66-116 case)
 *                     + brute force for the padded 3x3 window rule
 *   fyo_global_pool   closed form (mean/max)
 *   fyo_batchnorm     closed form x*s+b (misctests.cpp:118-126)
 *   fyo_argmax        numpy argmax (first maximum) (misctests.cpp:84-102)
 *   fyo_concat        memcpy identity
 *   fyo_deep_*        round trip + hand-computed tilings + DeepTiler's arithmetic (gpu/deep/deeptiler.cpp:73-76,
 *                     97-110: tile origin and channel order) + the copy loop of cpu/cpubuffer.cpp:424-437 at padding 0
 *                     with its row stride corrected (the reference multiplies the row index by the pixel packing twice)
 *   activations       leaky ReLU on fetch: shaders/activation.inc's form against the library's leaky_relu in fp64,
 *                     through unary copy, batch-norm and convolution; clip: numpy clip
 *   fyo_batchnorm     residual variants (residual / ReLU on it / batch-norm on it / both): closed form of
 *                     shaders/deep/deepbatchnorm.frag:26-35 per flag
 *   fyo_unary         arithmetic: reference patterns arithtests.cpp:205-234; sigmoid/tanh: scipy expit /
 *                     numpy tanh fp64; cast: numpy rint + clip (exact halves: parity unpinned, GLSL
 *                     leaves the tie direction open)
 *   fyo_scale         nearest: numpy repeat / strided slices; linear: torch interpolate(bilinear,
 *                     align_corners=False) fp64 on the stored array, avg_pool2d for the shallow halving
 *                     (no reference test exists; GL's fixed-point filter weights: parity unpinned)
 *   fyo_transpose     numpy transpose, involution
 *   fyo_imgextract    numpy reshape/transpose space-to-depth + brute force for partial groups
 *   fyo_nonmax        scipy maximum_filter with the cross footprint
 *   fyo_blur          scipy correlate for 3x3; literal loop restatement for larger kernels
 *   fyo_rgb2bgr       index permutation
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FYO_RESIDUAL_INPUT 1u
#define FYO_RELU_ON_RESIDUAL 2u
#define FYO_BATCHNORM_ON_RESIDUAL 4u
#define FYO_POST_BATCHNORM 8u

enum { FYO_ACT_NONE = 0, FYO_ACT_RELU = 1, FYO_ACT_LEAKY = 2, FYO_ACT_CLIP = 3 };

/* activate() of fyusenet/gpu/shaders/activation.inc:3-18 (applied when a layer READS its input). */
static inline float fyo_activate(float x, int act, float leak, float lo, float hi) {
    switch (act) {
        case FYO_ACT_RELU: return x > 0.f ? x : 0.f;
        case FYO_ACT_LEAKY: return x >= 0.f ? x : leak * x;
        case FYO_ACT_CLIP: return x < lo ? lo : (x > hi ? hi : x);
        default: return x;
    }
}

/* Fetch from a stored tensor [c][hs][ws] (hs, ws include the zero halo of width pad).
 * (y, x) are coordinates in the stored frame.  border: 0 = outside reads 0 (the deep path's zero
 * halo, fyusenet/base/layerbase.h:66-73), 1 = clamp to the edge (shallow unpadded textures,
 * fyusenet/gpu/gpulayerbase.h:80-90). */
static inline float fyo_fetch(const float* plane, int hs, int ws, int y, int x, int border) {
    if (border) {
        if (y < 0) y = 0;
        if (y >= hs) y = hs - 1;
        if (x < 0) x = 0;
        if (x >= ws) x = ws - 1;
    } else if (y < 0 || y >= hs || x < 0 || x >= ws) {
        return 0.f;
    }
    return plane[(size_t)y * ws + x];
}

/* Epilogue shared by the convolution family, in the shader's order
 * (shaders/deep/deepconv3x3_tiled.frag:36-45, batchnorm.inc:2-12, residual.inc:2-13 and the bias
 * fold of gpu/deep/deepconvlayerbase.cpp:377-382):
 *   acc*scale + (bias*scale + bnBias)  [+ residual, optionally ReLU'd, optionally * scale]. */
static inline float fyo_epilogue(double acc, float bias, unsigned flags, const float* bn, int cout, int o,
                                 const float* residual, size_t ridx) {
    double v;
    float scale = 1.f;
    if (flags & FYO_POST_BATCHNORM) {
        scale = bn[o];
        float b = bias * scale + bn[cout + o];
        v = acc * (double)scale + (double)b;
    } else {
        v = acc + (double)bias;
    }
    if ((flags & FYO_RESIDUAL_INPUT) && residual) {
        float r = residual[ridx];
        if (flags & FYO_RELU_ON_RESIDUAL) r = r > 0.f ? r : 0.f;
        if (flags & FYO_BATCHNORM_ON_RESIDUAL) r = r * scale;
        v += (double)r;
    }
    return (float)v;
}

/*
 * 2D convolution.  Follows ConvLayerTest::paddedConvolution (unit_tests/convlayertests.cpp:83-118):
 * weights [o][ky][kx][i] after cout biases, accumulator starts from the bias, optional activation on
 * fetch, output position (yo,xo) centred on stored input (pad + yo*stride, pad + xo*stride);
 * generalised by dilation (taps at (k-r)*dil, shaders/deep/deepconv3x3_tiled.frag:26-35), the BN /
 * residual epilogue and the border rule.  Output size H/stride (gpu/convlayerbase.cpp:47-48).
 *   in        [cin][hs][ws], hs = H + 2*pad_in
 *   block     [bias cout][W cout*k*k*cin][bnScale cout][bnBias cout]  (base/convlayerinterface.h:71-95)
 *   residual  [cout][H/stride][W/stride] or NULL
 *   out       [cout][H/stride][W/stride]
 */
int fyo_conv2d(const float* in, int cin, int hs, int ws, int pad_in, const float* block, int cout, int k, int dil,
               int stride, int act, float leak, float lo, float hi, unsigned flags, const float* residual,
               int border, float* out) {
    if ((k & 1) == 0 || stride < 1 || dil < 1) return -1;
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    const int ho = H / stride, wo = W / stride, r = (k - 1) / 2;
    const float* wts = block + cout;
    const float* bn = wts + (size_t)cout * k * k * cin;
#pragma omp parallel for schedule(static)
    for (int o = 0; o < cout; o++) {
        for (int yo = 0; yo < ho; yo++) {
            for (int xo = 0; xo < wo; xo++) {
                double acc = 0.0;
                const int yc = pad_in + yo * stride, xc = pad_in + xo * stride;
                for (int i = 0; i < cin; i++) {
                    const float* plane = in + (size_t)i * hs * ws;
                    for (int ky = 0; ky < k; ky++) {
                        for (int kx = 0; kx < k; kx++) {
                            float v = fyo_fetch(plane, hs, ws, yc + (ky - r) * dil, xc + (kx - r) * dil, border);
                            v = fyo_activate(v, act, leak, lo, hi);
                            acc += (double)v * (double)wts[(((size_t)o * k + ky) * k + kx) * cin + i];
                        }
                    }
                }
                size_t oidx = ((size_t)o * ho + yo) * wo + xo;
                out[oidx] = fyo_epilogue(acc, block[o], flags, bn, cout, o, residual, oidx);
            }
        }
    }
    return 0;
}

/*
 * Fractional-step ("up-sampling") convolution of the shallow path, FRACCONVOLUTION2D.
 * gpu/vanilla/fractionalconvlayerNxN_vanilla.cpp:43-50: output size = int(size / (sourceStep * downsample));
 * :91: the shader's horizontal tap distance is sourceStep texels.  The proxy polygons
 * (gpu/vanilla/convlayerbase_vanilla.cpp:361-371) map the output's net area onto the input's, shift row
 * pass `ky` by sourceStep*(ky - r) texels and both axes by -sourceStep*(downsample-1)/2; the texture is read
 * with nearest filtering, so with sourceStep = 1/inv_step the stored texel of tap t at output x is
 *      pad + floor((downsample*x + t + 1/2) / inv_step)
 * (never on a texel boundary for an integer inv_step).  Vertical taps are t = ky - r.  Horizontal taps are
 * t = kx - r for 5x5, 7x7 and 9x9 (shaders/vanilla/fraconv5x5.frag:14-22, fraconv9x9.frag:14-30) but
 * t = kx - 2 for 3x3 (shaders/vanilla/fraconv3x3.frag:14-19 samples at -2, -1 and 0 steps): reproduced as is.
 * Activation on fetch, bias / BN / residual epilogue and the weight block are those of fyo_conv2d.
 * Sizes that sourceStep*downsample does not divide are refused (their sample positions are not dyadic).
 *   in        [cin][hs][ws], hs = H + 2*pad_in;  out / residual [cout][H*inv_step/stride][W*inv_step/stride]
 */
int fyo_fracconv(const float* in, int cin, int hs, int ws, int pad_in, const float* block, int cout, int k,
                 int stride, int inv_step, int act, float leak, float lo, float hi, unsigned flags,
                 const float* residual, int border, float* out) {
    if ((k & 1) == 0 || k < 3 || k > 9 || stride < 1 || inv_step < 1) return -1;
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    if ((H * inv_step) % stride || (W * inv_step) % stride) return -2;
    const int ho = H * inv_step / stride, wo = W * inv_step / stride, r = (k - 1) / 2;
    const int tx0 = (k == 3) ? -2 : -r;
    const float* wts = block + cout;
    const float* bn = wts + (size_t)cout * k * k * cin;
#pragma omp parallel for schedule(static)
    for (int o = 0; o < cout; o++) {
        for (int yo = 0; yo < ho; yo++) {
            for (int xo = 0; xo < wo; xo++) {
                double acc = 0.0;
                for (int i = 0; i < cin; i++) {
                    const float* plane = in + (size_t)i * hs * ws;
                    for (int ky = 0; ky < k; ky++) {
                        /* floor((2n + 1) / (2*inv_step)) for any sign of n */
                        const int ny = 2 * (stride * yo + ky - r) + 1;
                        const int sy = pad_in + (ny >= 0 ? ny / (2 * inv_step) : -((-ny + 2 * inv_step - 1) / (2 * inv_step)));
                        for (int kx = 0; kx < k; kx++) {
                            const int nx = 2 * (stride * xo + kx + tx0) + 1;
                            const int sx = pad_in + (nx >= 0 ? nx / (2 * inv_step) : -((-nx + 2 * inv_step - 1) / (2 * inv_step)));
                            float v = fyo_fetch(plane, hs, ws, sy, sx, border);
                            v = fyo_activate(v, act, leak, lo, hi);
                            acc += (double)v * (double)wts[(((size_t)o * k + ky) * k + kx) * cin + i];
                        }
                    }
                }
                size_t oidx = ((size_t)o * ho + yo) * wo + xo;
                out[oidx] = fyo_epilogue(acc, block[o], flags, bn, cout, o, residual, oidx);
            }
        }
    }
    return 0;
}

/*
 * Depthwise 3x3 (any odd k accepted) convolution.  Follows
 * shaders/deep/deepconv_dw3x3_tiled.frag:36-59 (9 activated taps at +-DILATION, then BN/bias,
 * then residual) and the source-weight indexing of
 * gpu/deep/deepdwconvlayerbase.cpp:242: w[(i*k*k + ky*k+kx)*mult + m]; output channel i*mult+m;
 * block = [bias cout][W cin*k*k*mult][bnScale cout][bnBias cout] (deepdwconvlayerbase.cpp:99-108).
 */
int fyo_dwconv(const float* in, int cin, int hs, int ws, int pad_in, const float* block, int mult, int k, int dil,
               int stride, int act, float leak, float lo, float hi, unsigned flags, const float* residual,
               float* out) {
    if ((k & 1) == 0) return -1;
    const int cout = cin * mult;
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    const int ho = H / stride, wo = W / stride, r = (k - 1) / 2;
    const float* wts = block + cout;
    const float* bn = wts + (size_t)cin * k * k * mult;
#pragma omp parallel for schedule(static)
    for (int o = 0; o < cout; o++) {
        const int i = o / mult, m = o % mult;
        const float* plane = in + (size_t)i * hs * ws;
        for (int yo = 0; yo < ho; yo++) {
            for (int xo = 0; xo < wo; xo++) {
                double acc = 0.0;
                const int yc = pad_in + yo * stride, xc = pad_in + xo * stride;
                for (int ky = 0; ky < k; ky++) {
                    for (int kx = 0; kx < k; kx++) {
                        float v = fyo_fetch(plane, hs, ws, yc + (ky - r) * dil, xc + (kx - r) * dil, 0);
                        v = fyo_activate(v, act, leak, lo, hi);
                        acc += (double)v * (double)wts[((size_t)i * k * k + ky * k + kx) * mult + m];
                    }
                }
                size_t oidx = ((size_t)o * ho + yo) * wo + xo;
                out[oidx] = fyo_epilogue(acc, block[o], flags, bn, cout, o, residual, oidx);
            }
        }
    }
    return 0;
}

/*
 * Stride-2 transposed convolution, scatter form
 *   out[o, 2y+ky, 2x+kx] += W[o,ky,kx,i] * act(in[i,y,x]),   full size 2H+k-2 (gpu/deep/deeptiler.cpp:71-74)
 * which is what the four stencil-selected parity passes of
 * shaders/deep/deeptransconv3x3_stride2.frag:27-51 / .vert:50-72 (k=3) and
 * deeptransconv2x2_stride2.frag:25-36 (k=2) compute; weights use the convolution block layout
 * (gpu/deep/deeptransconvlayerbase.cpp:148-160).  The epilogue (BN/bias on every output element)
 * follows deeptransconv3x3_stride2.frag:43-50.  `crop` drops the last `crop` rows/columns of the full
 * result (the 2H "doubling decoder" size).
 *   in [cin][hs][ws]; out [cout][2H+k-2-crop][2W+k-2-crop]; residual of the output size or NULL.
 */
int fyo_transconv(const float* in, int cin, int hs, int ws, int pad_in, const float* block, int cout, int k, int crop,
                  int act, float leak, float lo, float hi, unsigned flags, const float* residual, float* out) {
    if (k != 2 && k != 3) return -1;
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    const int hf = 2 * H + k - 2, wf = 2 * W + k - 2;
    const int ho = hf - crop, wo = wf - crop;
    const float* wts = block + cout;
    const float* bn = wts + (size_t)cout * k * k * cin;
#pragma omp parallel for schedule(static)
    for (int o = 0; o < cout; o++) {
        double* acc = (double*)calloc((size_t)hf * wf, sizeof(double));
        for (int i = 0; i < cin; i++) {
            const float* plane = in + (size_t)i * hs * ws;
            for (int y = 0; y < H; y++) {
                for (int x = 0; x < W; x++) {
                    float v = fyo_activate(plane[(size_t)(y + pad_in) * ws + x + pad_in], act, leak, lo, hi);
                    for (int ky = 0; ky < k; ky++)
                        for (int kx = 0; kx < k; kx++)
                            acc[(size_t)(2 * y + ky) * wf + 2 * x + kx] +=
                                (double)v * (double)wts[(((size_t)o * k + ky) * k + kx) * cin + i];
                }
            }
        }
        for (int y = 0; y < ho; y++)
            for (int x = 0; x < wo; x++) {
                size_t oidx = ((size_t)o * ho + y) * wo + x;
                out[oidx] = fyo_epilogue(acc[(size_t)y * wf + x], block[o], flags, bn, cout, o, residual, oidx);
            }
        free(acc);
    }
    return 0;
}

/*
 * Fully connected layer y[o] = sum_i W[o,i]*act(x[i]) + b[o]  (a 1x1 convolution on 1x1 spatial,
 * gpu/deep/deepgemmlayer.cpp:66-236); block = [bias cout][W cout*cin] (+ BN block).
 */
int fyo_gemm(const float* x, int cin, const float* block, int cout, int act, float leak, float lo, float hi,
             unsigned flags, float* y) {
    return fyo_conv2d(x, cin, 1, 1, 0, block, cout, 1, 1, 1, act, leak, lo, hi, flags & FYO_POST_BATCHNORM, NULL,
                      0, y);
}

/*
 * Max pooling, deep rule (shaders/deep/deepmaxpool.frag:12-59): window rows/cols
 * (yo*stride - pad_in + [0,P)) in net input coordinates, i.e. the window starts pad_in before the
 * stride origin; halo texels are 0 (not -inf) and are activated like any other texel.  For
 * pool == stride and pad_in == 0 this is PoolLayerTest::computeMaxPool (unit_tests/pooltests.cpp:66-90).
 */
int fyo_maxpool(const float* in, int c, int hs, int ws, int pad_in, int pool, int stride, int act, float leak,
                float lo, float hi, float* out) {
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in, ho = H / stride, wo = W / stride;
#pragma omp parallel for schedule(static)
    for (int ch = 0; ch < c; ch++) {
        const float* plane = in + (size_t)ch * hs * ws;
        for (int yo = 0; yo < ho; yo++)
            for (int xo = 0; xo < wo; xo++) {
                float m = 0.f;
                for (int py = 0; py < pool; py++)
                    for (int px = 0; px < pool; px++) {
                        /* stored coordinate = pad_in + (yo*stride - pad_in + py) */
                        float v = fyo_fetch(plane, hs, ws, yo * stride + py, xo * stride + px, 0);
                        v = fyo_activate(v, act, leak, lo, hi);
                        if ((py == 0 && px == 0) || v > m) m = v;
                    }
                out[((size_t)ch * ho + yo) * wo + xo] = m;
            }
    }
    return 0;
}

/*
 * Average pooling, deep rule (shaders/deep/deepavgpool.frag:15-58): P=3 uses the window [-1,1]
 * around the stride origin, every other size [0,P) from it; divisor always P*P.  For pool == stride,
 * P != 3 this is PoolLayerTest::computeAvgPool (unit_tests/pooltests.cpp:92-116).
 */
int fyo_avgpool(const float* in, int c, int hs, int ws, int pad_in, int pool, int stride, int act, float leak,
                float lo, float hi, float* out) {
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in, ho = H / stride, wo = W / stride;
    const int off = (pool == 3) ? -1 : 0;
#pragma omp parallel for schedule(static)
    for (int ch = 0; ch < c; ch++) {
        const float* plane = in + (size_t)ch * hs * ws;
        for (int yo = 0; yo < ho; yo++)
            for (int xo = 0; xo < wo; xo++) {
                double acc = 0.0;
                for (int py = 0; py < pool; py++)
                    for (int px = 0; px < pool; px++) {
                        float v = fyo_fetch(plane, hs, ws, pad_in + yo * stride + off + py,
                                            pad_in + xo * stride + off + px, 0);
                        acc += (double)fyo_activate(v, act, leak, lo, hi);
                    }
                out[((size_t)ch * ho + yo) * wo + xo] = (float)(acc / (double)(pool * pool));
            }
    }
    return 0;
}

/* Global pooling: mean (op 0) or max (op 1) over all H*W activated values per channel
 * (shaders/deep/deepglobavgpool.frag:15-24, deepglobmaxpool.frag). out [c]. */
int fyo_global_pool(const float* in, int c, int hs, int ws, int pad_in, int op, int act, float leak, float lo,
                    float hi, float* out) {
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    for (int ch = 0; ch < c; ch++) {
        const float* plane = in + (size_t)ch * hs * ws;
        double acc = 0.0;
        float m = 0.f;
        for (int y = 0; y < H; y++)
            for (int x = 0; x < W; x++) {
                float v = fyo_activate(plane[(size_t)(y + pad_in) * ws + x + pad_in], act, leak, lo, hi);
                acc += v;
                if ((y == 0 && x == 0) || v > m) m = v;
            }
        out[ch] = op ? m : (float)(acc / ((double)H * W));
    }
    return 0;
}

/*
 * Explicit batch-norm layer: out = act(in)*scale_c + bias_c, residual variants as in
 * shaders/deep/deepbatchnorm.frag:24-36 (here BATCHNORM_ON_RESIDUAL applies scale AND bias to the
 * residual).  sb = [scale c][bias c] (base/batchnorminterface.h:137-146).  Without activation and
 * residual this is BatchNormTest::referenceNorm (unit_tests/misctests.cpp:118-126).
 */
int fyo_batchnorm(const float* in, int c, int hs, int ws, int pad_in, const float* sb, int act, float leak, float lo,
                  float hi, unsigned flags, const float* residual, float* out) {
    const int H = hs - 2 * pad_in, W = ws - 2 * pad_in;
    for (int ch = 0; ch < c; ch++) {
        const float* plane = in + (size_t)ch * hs * ws;
        for (int y = 0; y < H; y++)
            for (int x = 0; x < W; x++) {
                size_t oidx = ((size_t)ch * H + y) * W + x;
                float v = fyo_activate(plane[(size_t)(y + pad_in) * ws + x + pad_in], act, leak, lo, hi);
                float r = v * sb[ch] + sb[c + ch];
                if ((flags & FYO_RESIDUAL_INPUT) && residual) {
                    float q = residual[oidx];
                    if (flags & FYO_RELU_ON_RESIDUAL) q = q > 0.f ? q : 0.f;
                    if (flags & FYO_BATCHNORM_ON_RESIDUAL) q = q * sb[ch] + sb[c + ch];
                    r += q;
                }
                out[oidx] = r;
            }
    }
    return 0;
}

/* Element-wise add (sub != 0: subtract) of two activated tensors (shaders/add.frag, gpu/addsublayer.cpp). */
int fyo_addsub(const float* a, const float* b, size_t n, int sub, int act, float leak, float lo, float hi,
               float* out) {
    for (size_t i = 0; i < n; i++) {
        float x = fyo_activate(a[i], act, leak, lo, hi), y = fyo_activate(b[i], act, leak, lo, hi);
        out[i] = sub ? x - y : x + y;
    }
    return 0;
}

/* Channel concatenation: port p's channels follow those of ports < p; one common activation
 * (shaders/deep/deepconcat.frag:45-76, gpu/concatlayerbuilder.h:40-84).  Unpadded [c][h][w] inputs. */
int fyo_concat(const float* const* ins, const int* chans, int n, int h, int w, int act, float leak, float lo,
               float hi, float* out) {
    size_t pos = 0;
    for (int p = 0; p < n; p++) {
        size_t cnt = (size_t)chans[p] * h * w;
        for (size_t i = 0; i < cnt; i++) out[pos + i] = fyo_activate(ins[p][i], act, leak, lo, hi);
        pos += cnt;
    }
    return 0;
}

/* Exact arg-max over channels, lowest index among maxima (strict '>' scan,
 * ArgMaxTest::referenceArgMax, unit_tests/misctests.cpp:84-102); also returns the maximum value, the
 * second output channel of shaders/deep/deepargmax2.frag:15-20.  in [c][h][w] unpadded. */
int fyo_argmax(const float* in, int c, int h, int w, int act, float leak, float lo, float hi, int* idx, float* val) {
    const size_t cs = (size_t)h * w;
    for (size_t p = 0; p < cs; p++) {
        float mx = fyo_activate(in[p], act, leak, lo, hi);
        int mi = 0;
        for (int ch = 1; ch < c; ch++) {
            float v = fyo_activate(in[ch * cs + p], act, leak, lo, hi);
            if (v > mx) {
                mx = v;
                mi = ch;
            }
        }
        idx[p] = mi;
        if (val) val[p] = mx;
    }
    return 0;
}

/* ---- fp16 storage emulation: round-to-nearest-even through IEEE binary16 ------------------- */
static inline uint16_t fyo_f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mant = x & 0x7fffffu;
    int32_t exp = (int32_t)((x >> 23) & 0xff);
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0));
    int32_t e = exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        mant |= 0x800000u;
        int shift = 14 - e;
        uint32_t h = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}
static inline float fyo_h2f(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, x;
    if (exp == 0) {
        if (!mant) x = sign;
        else {
            int e = -1;
            do { mant <<= 1; e++; } while (!(mant & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7f800000u | (mant << 13);
    else x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}
/* Round every element to the nearest binary16 value (what an fp16-stored tensor holds). */
void fyo_round_fp16(const float* in, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = fyo_h2f(fyo_f2h(in[i]));
}

/* ---- buffer formats at the upload / download boundary ------------------------------------- */

/* Deep tile grid: minimise |tx-ty| + unused tiles, first minimum in y-outer / x-inner ascending
 * order with x >= y (fyusenet/cpu/cpubuffershape.cpp:430-448, gpu/deep/deeptiler.cpp:63-110). */
void fyo_deep_tiling(int channels, int* tx, int* ty) {
    int tiles = (channels + 3) / 4;
    int best = 1 << 30, bx = tiles, by = 1;
    for (int y = 1; y <= tiles; y++)
        for (int x = y; x <= tiles; x++)
            if (x * y >= tiles) {
                int cost = (x - y) + (x * y - tiles);
                if (cost < best) {
                    best = cost;
                    bx = x;
                    by = y;
                }
            }
    *tx = bx;
    *ty = by;
}

/* CHW -> GPU_DEEP tiled RGBA buffer of size (tx*(W+p)+p) x (ty*(H+p)+p) x 4, tile t at grid
 * (t % tx, t / tx), shared padding between tiles (cpu/cpubuffer.cpp:413-442 inverse,
 * gpu/deep/deeptiler.cpp:63-110). */
int fyo_chw_to_deep(const float* chw, int c, int h, int w, int pad, float* deep) {
    int tx, ty;
    fyo_deep_tiling(c, &tx, &ty);
    const int dw = tx * (w + pad) + pad, dh = ty * (h + pad) + pad;
    memset(deep, 0, (size_t)dw * dh * 4 * sizeof(float));
    for (int ch = 0; ch < c; ch++) {
        int t = ch / 4, comp = ch % 4, gx = t % tx, gy = t / tx;
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                deep[(((size_t)(pad + gy * (h + pad) + y)) * dw + pad + gx * (w + pad) + x) * 4 + comp] =
                    chw[((size_t)ch * h + y) * w + x];
    }
    return 0;
}

/* GPU_DEEP -> CHW (CPUBuffer::deepToChannelWise, cpu/cpubuffer.cpp:413-442). */
int fyo_deep_to_chw(const float* deep, int c, int h, int w, int pad, float* chw) {
    int tx, ty;
    fyo_deep_tiling(c, &tx, &ty);
    const int dw = tx * (w + pad) + pad;
    for (int ch = 0; ch < c; ch++) {
        int t = ch / 4, comp = ch % 4, gx = t % tx, gy = t / tx;
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                chw[((size_t)ch * h + y) * w + x] =
                    deep[(((size_t)(pad + gy * (h + pad) + y)) * dw + pad + gx * (w + pad) + x) * 4 + comp];
    }
    return 0;
}

/* GPU_SHALLOW (HWC with `pc` interleaved components per pixel, pc = channels for <=4 channels)
 * <-> CHW (cpu/cpubuffer.cpp:121-158 toChannelWise for a single-texture tensor). */
int fyo_shallow_to_chw(const float* hwc, int c, int h, int w, int pc, float* chw) {
    for (int ch = 0; ch < c; ch++)
        for (size_t p = 0; p < (size_t)h * w; p++) chw[(size_t)ch * h * w + p] = hwc[p * pc + ch];
    return 0;
}
int fyo_chw_to_shallow(const float* chw, int c, int h, int w, int pc, float* hwc) {
    memset(hwc, 0, (size_t)h * w * pc * sizeof(float));
    for (int ch = 0; ch < c; ch++)
        for (size_t p = 0; p < (size_t)h * w; p++) hwc[p * pc + ch] = chw[(size_t)ch * h * w + p];
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Function-type layers (one input, no weights).
 * ------------------------------------------------------------------------------------------- */

/* Floor division for a positive divisor. */
static inline long fyo_floordiv(long a, long b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

/* Element-wise functions of the activated input; n elements.
 *   fn 0  copy                    shaders/deep/deepdefault.frag:20-22 (also RELU/CLIP/PADDING2D layers, which the
 *                                 factory maps to a scale layer of factor 1, gpu/gpulayerfactory.cpp:125-140)
 *   fn 1  sigmoid 1/(1+exp(-x))   shaders/deep/deepsigmoid.frag:19-22
 *   fn 2  tanh, written there as 2*(e^{2x}/(1+e^{2x}))-1   shaders/deep/deeptanh.frag:19-22
 *   fn 3  x (op) operand, op = ArithType 0 add, 1 sub, 2 mul, 3 div   shaders/deep/deep_singleton_arith.frag:21-39
 *   fn 4  cast: op = CastTarget 0..5 (int32, int16, int8, uint32, uint16, uint8): round, then clamp to the
 *         type's range, result kept as float; 6 (float16): value rounded to fp16; 7 (float32): unchanged
 *         (shaders/typecast.inc:10-35, shaders/deep/deepcast.frag:20-27).  GLSL leaves the direction of
 *         round() at exact halves to the implementation; ties go to even here. */
int fyo_unary(const float* in, size_t n, int fn, int op, float operand, int act, float leak, float lo, float hi,
              float* out) {
    static const double cast_lo[6] = {-2147483648.0, -32768.0, -128.0, 0.0, 0.0, 0.0};
    static const double cast_hi[6] = {2147483647.0, 32767.0, 127.0, 4294967295.0, 65535.0, 255.0};
    for (size_t i = 0; i < n; i++) {
        const double x = (double)fyo_activate(in[i], act, leak, lo, hi);
        double r = x;
        switch (fn) {
            case 0: break;
            case 1: r = 1.0 / (1.0 + exp(-x)); break;
            case 2: r = tanh(x); break;
            case 3:
                if (op == 0) r = x + (double)operand;
                else if (op == 1) r = x - (double)operand;
                else if (op == 2) r = x * (double)operand;
                else if (op == 3) r = x / (double)operand;
                else return -1;
                break;
            case 4:
                if (op >= 0 && op < 6) {
                    r = nearbyint(x);
                    if (r < cast_lo[op]) r = cast_lo[op];
                    if (r > cast_hi[op]) r = cast_hi[op];
                } else if (op == 6) {
                    float xf = (float)x, hf;
                    fyo_round_fp16(&xf, 1, &hf);
                    r = (double)hf;
                } else if (op != 7) {
                    return -1;
                }
                break;
            default: return -1;
        }
        out[i] = (float)r;
    }
    return 0;
}

/* Scale layer: integer up- or down-scaling with nearest or bilinear sampling
 * (gpu/deep/deepscalelayer.cpp:41-96, gpu/scalelayer.cpp:38-108, shaders/deep/deepdefault.frag, shaders/scaling.frag).
 * The sampling position of output column x in input texel units, relative to the first net texel, is what the
 * proxy polygon's texture coordinates interpolate to:
 *   deep    (x + 1/2) * d/u - (d - 1)/2     (gpu/deep/deeptiler.cpp:97-110: the quad starts (d-1)/2 texels early)
 *   shallow (x + 1/2) * d/u                 (gpu/functionlayer.cpp:194-219)
 * Nearest takes the texel containing that position, linear blends the two texels around it (per axis) with
 * GL_LINEAR weights; the RAW texels are blended and the activation is applied to the result.  Texels outside the
 * net area are the stored halo (zero) where the input has padding, beyond the stored texture the edge is repeated
 * (GL_CLAMP_TO_EDGE).  in_stored [c][hs][ws] with halo pad; out [c][H*uy/dy][W*ux/dx]. */
int fyo_scale(const float* in_stored, int c, int hs, int ws, int pad, int ux, int uy, int dx, int dy, int linear,
              int deep, int act, float leak, float lo, float hi, float* out) {
    if (ux < 1 || uy < 1 || dx < 1 || dy < 1) return -1;
    const int h = hs - 2 * pad, w = ws - 2 * pad;
    const int ho = h * uy / dy, wo = w * ux / dx;
    for (int ch = 0; ch < c; ch++) {
        const float* plane = in_stored + (size_t)ch * hs * ws;
        for (int y = 0; y < ho; y++) {
            const long ny = (long)(2 * y + 1) * dy - (deep ? (long)uy * (dy - 1) : 0);   /* position = ny / (2 uy) */
            for (int x = 0; x < wo; x++) {
                const long nx = (long)(2 * x + 1) * dx - (deep ? (long)ux * (dx - 1) : 0);
                double v;
                if (!linear) {
                    const int sy = (int)fyo_floordiv(ny, 2L * uy), sx = (int)fyo_floordiv(nx, 2L * ux);
                    v = fyo_fetch(plane, hs, ws, sy + pad, sx + pad, 1);
                } else {
                    const long y0 = fyo_floordiv(ny - uy, 2L * uy), x0 = fyo_floordiv(nx - ux, 2L * ux);
                    const double fy = (double)((ny - uy) - y0 * 2L * uy) / (double)(2L * uy);
                    const double fx = (double)((nx - ux) - x0 * 2L * ux) / (double)(2L * ux);
                    const double a = fyo_fetch(plane, hs, ws, (int)y0 + pad, (int)x0 + pad, 1);
                    const double b = fyo_fetch(plane, hs, ws, (int)y0 + pad, (int)x0 + 1 + pad, 1);
                    const double cc = fyo_fetch(plane, hs, ws, (int)y0 + 1 + pad, (int)x0 + pad, 1);
                    const double d = fyo_fetch(plane, hs, ws, (int)y0 + 1 + pad, (int)x0 + 1 + pad, 1);
                    v = (1.0 - fy) * ((1.0 - fx) * a + fx * b) + fy * ((1.0 - fx) * cc + fx * d);
                }
                out[((size_t)ch * ho + y) * wo + x] = fyo_activate((float)v, act, leak, lo, hi);
            }
        }
    }
    return 0;
}

/* Spatial transposition out[c][x][y] = act(in[c][y][x]) (gpu/deep/deeptransposelayer.cpp:141-156: the input quad's
 * texture coordinates are attached to the output quad in transposed vertex order). */
int fyo_transpose(const float* in, int c, int h, int w, int act, float leak, float lo, float hi, float* out) {
    for (int ch = 0; ch < c; ch++)
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                out[((size_t)ch * w + x) * h + y] = fyo_activate(in[((size_t)ch * h + y) * w + x], act, leak, lo, hi);
    return 0;
}

/* Image-patch extraction (space to depth) with window n (gpu/deep/deepextractimgpatches.cpp:150-186,
 * shaders/deep/deepimgpatch.frag:28-33): output 4-channel group g takes input group g mod G (G = groups of the
 * input) at in-window offset (xpix, ypix) = (b mod n, b / n), b = g / G; out(y, x) = act(in(y*n + ypix, x*n + xpix)).
 * Channels of an input group beyond cin read as zero.  in [cin][h][w], out [cout][h/n][w/n]. */
int fyo_imgextract(const float* in, int cin, int h, int w, int window, int cout, int act, float leak, float lo,
                   float hi, float* out) {
    const int groups = (cin + 3) / 4, ho = h / window, wo = w / window;
    if (window < 1 || (cout + 3) / 4 > groups * window * window) return -1;
    for (int o = 0; o < cout; o++) {
        const int g = o / 4, j = o % 4, b = g / groups, src = (g % groups) * 4 + j;
        const int xpix = b % window, ypix = b / window;
        for (int y = 0; y < ho; y++)
            for (int x = 0; x < wo; x++) {
                const float v = src < cin ? in[((size_t)src * h + y * window + ypix) * w + x * window + xpix] : 0.f;
                out[((size_t)o * ho + y) * wo + x] = fyo_activate(v, act, leak, lo, hi);
            }
    }
    return 0;
}

/* 2D non-maximum suppression over the 4-neighbourhood (shaders/nonmax2d.frag:88-101): a value survives if it is
 * >= its left, right, upper and lower neighbour and > 0.1, everything else becomes 0.  No activation.  Neighbours
 * outside the net area are the stored halo, beyond the stored texture the edge is repeated. */
int fyo_nonmax(const float* in_stored, int c, int hs, int ws, int pad, float* out) {
    const int h = hs - 2 * pad, w = ws - 2 * pad;
    for (int ch = 0; ch < c; ch++) {
        const float* p = in_stored + (size_t)ch * hs * ws;
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const int sy = y + pad, sx = x + pad;
                const float m = p[(size_t)sy * ws + sx];
                const int keep = m >= fyo_fetch(p, hs, ws, sy, sx + 1, 1) && m >= fyo_fetch(p, hs, ws, sy, sx - 1, 1) &&
                                 m >= fyo_fetch(p, hs, ws, sy - 1, sx, 1) && m >= fyo_fetch(p, hs, ws, sy + 1, sx, 1) &&
                                 m > 0.1f;
                out[((size_t)ch * h + y) * w + x] = keep ? m : 0.f;
            }
    }
    return 0;
}

/* Blur layer coefficients (gpu/blurlayer.cpp:86-113): box = 1/k^2; Gaussian = outer product of
 * exp(-x^2)/sqrt(2 pi), x = i - (k-1)/2, normalised to sum 1.  coef [k*k] row-major. */
int fyo_blur_coeffs(int k, int gaussian, float* coef) {
    if (k < 1 || !(k & 1)) return -1;
    if (!gaussian) {
        for (int i = 0; i < k * k; i++) coef[i] = 1.0f / (float)(k * k);
        return 0;
    }
    float g[64];
    if (k > 63) return -1;
    const float fac = (float)(1.0 / sqrt(2.0 * 3.14159265358979323846));
    for (int i = 0; i < k; i++) {
        const float x = (float)(i - (k - 1) / 2);
        g[i] = fac * expf(-(x * x));
    }
    float denom = 0.f;
    for (int y = 0; y < k; y++)
        for (int x = 0; x < k; x++) {
            coef[y * k + x] = g[y] * g[x];
            denom += coef[y * k + x];
        }
    for (int i = 0; i < k * k; i++) coef[i] /= denom;
    return 0;
}

/* Blur layer (shaders/generickernel.frag:83-107), no activation.  k == 3: the nine taps (-1..1)^2 with
 * coefficients in row-major order.  k > 3: the shader's loops run over offsets -(k-1)/2 .. (k-1)/2 - 1 in both
 * directions (the last row and column of the window are never visited) and take the coefficients in running
 * order from the start of the k*k array; that is restated literally.  Borders as in fyo_nonmax. */
int fyo_blur(const float* in_stored, int c, int hs, int ws, int pad, int k, int gaussian, float* out) {
    float coef[64 * 64];
    if (k > 15 || fyo_blur_coeffs(k, gaussian, coef) != 0) return -1;   /* MAX_KERNEL_SIZE 15, generickernel.frag:18 */
    const int h = hs - 2 * pad, w = ws - 2 * pad, r = (k - 1) / 2;
    const int last = (k == 3) ? r : r - 1;
    for (int ch = 0; ch < c; ch++) {
        const float* p = in_stored + (size_t)ch * hs * ws;
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                double acc = 0.0;
                int kidx = 0;
                for (int oy = -r; oy <= last; oy++)
                    for (int ox = -r; ox <= last; ox++)
                        acc += (double)coef[kidx++] * (double)fyo_fetch(p, hs, ws, y + pad + oy, x + pad + ox, 1);
                out[((size_t)ch * h + y) * w + x] = (float)acc;
            }
    }
    return 0;
}

/* RGB <-> BGR: within every group of four channels the first and third swap (val.bgra, shaders/rgb2bgr.frag:88-92).
 * No activation.  in/out [c][h][w]; a partner channel beyond c reads as zero. */
int fyo_rgb2bgr(const float* in, int c, int h, int w, float* out) {
    const size_t plane = (size_t)h * w;
    for (int ch = 0; ch < c; ch++) {
        const int j = ch % 4, src = (j == 0) ? ch + 2 : (j == 2) ? ch - 2 : ch;
        if (src < c) memcpy(out + ch * plane, in + src * plane, plane * sizeof(float));
        else memset(out + ch * plane, 0, plane * sizeof(float));
    }
    return 0;
}
