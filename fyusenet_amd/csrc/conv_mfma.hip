// Implicit-GEMM convolution on gfx950 matrix cores (v_mfma_f32_32x32x16_f16, fp32 accumulate).
//
// Replaces the additive-blend render passes of DeepConvLayerNxN::forward
// (fyusenet/gpu/deep/deepconvlayerNxN.cpp:129-211), DeepConvLayer1x1::forward
// (deepconvlayer1x1.cpp:67-117), the shallow ConvLayerNxN::forward
// (gpu/vanilla/convlayerNxN_vanilla.cpp:72-141) and, launched once per output parity, the stencil
// passes of DeepTransConvLayerBase::forward (gpu/deep/deeptransconvlayerbase.cpp:83-130).
//
// GEMM view: M = output channels (A operand = weights, pre-packed per lane in HBM, streamed
// through L2 straight into VGPRs), N = output positions (B operand = activations, staged once per
// input-channel chunk as a halo tile in LDS and re-read for every kernel tap at a shifted address),
// K = taps x input channels.  The activation of the producing layer is applied while staging
// (shaders/activation.inc:3-18 semantics: activation on input fetch).  Epilogue: acc*scale + bias
// (+ residual), the order of shaders/deep/deepconv3x3_tiled.frag:36-45.
//
// fp32 storage: both operands are split into fp16 hi + lo parts (x = hi + lo, 22 significant
// bits) and three MFMAs (hi*hi, lo*hi, hi*lo) are issued per fragment pair; fp16 storage: one.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace fynhip {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float act_apply(float x, const Act& a) {
    switch (a.kind) {
        case ACT_RELU: return fmaxf(x, 0.f);
        case ACT_LEAKY: return x >= 0.f ? x : a.leak * x;
        case ACT_CLIP: return fminf(a.hi, fmaxf(a.lo, x));
        default: return x;
    }
}

template <typename T>
__device__ __forceinline__ void load_vals(const T* src, float* v, int n);
template <>
__device__ __forceinline__ void load_vals<float>(const float* src, float* v, int n) {
    if (n == 8) {
        float4 a = *reinterpret_cast<const float4*>(src);
        float4 b = *reinterpret_cast<const float4*>(src + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        float4 a = *reinterpret_cast<const float4*>(src);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    }
}
template <>
__device__ __forceinline__ void load_vals<_Float16>(const _Float16* src, float* v, int n) {
    if (n == 8) {
        half8_t a = *reinterpret_cast<const half8_t*>(src);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)a[i];
    } else {
        half4_t a = *reinterpret_cast<const half4_t*>(src);
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = (float)a[i];
    }
}

template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN, int KC>
__global__ __launch_bounds__(256) void conv_mfma_kernel(const ConvMfmaParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int NPL = SPLIT ? 2 : 1;         // operand planes (hi, lo)
    constexpr int CPI = (KC == 4) ? 4 : 8;     // channels per staging item
    constexpr int G = (KC == 4) ? 1 : KC / 8;  // staging items per pixel
    static_assert(WM * WN == 4, "4 waves per block");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM;
    const int wn = wave / WM;

    // Workgroups are dealt round-robin to the 8 XCDs; remap so that neighbouring tiles (shared
    // halos, same input tile for all cout blocks) meet in one XCD's L2.
    int bid = blockIdx.x;
    {
        const int per = gridDim.x >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    const int cb = bid % p.cout_blocks;
    const int tile = bid / p.cout_blocks;
    const int tyi = tile / p.tiles_x;
    const int txi = tile - tyi * p.tiles_x;
    const int twl = p.tile_w_log2;
    const int TW = 1 << twl;
    const int pos_y0 = tyi * p.tile_h;
    const int pos_x0 = txi * TW;

    const int npix = p.halo_h * p.halo_w;
    const int nitems = npix * G;
    const int gy0 = pos_y0 * p.in_stride + p.in_y0;
    const int gx0 = pos_x0 * p.in_stride + p.in_x0;
    const float inv_hw = 1.0f / (float)p.halo_w;
    const TIn* in = reinterpret_cast<const TIn*>(p.in);

    if (KC == 4) {
        // slack behind each plane is read by the last (zero-weight) k elements of a row run
        if (tid < 16 * NPL) {
            int pl = tid >> 4;
            reinterpret_cast<uint32_t*>(lds + pl * p.plane + npix * p.pitch)[tid & 15] = 0u;
        }
    }

    // per-lane LDS byte offsets of the B (activation) fragments
    int boff[FN];
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = (wn * FN + fn) * 32 + (lane & 31);
        const int ty = m >> twl, tx = m & (TW - 1);
        boff[fn] = ((ty * p.in_stride) * p.halo_w + tx * p.in_stride) * p.pitch + (lane >> 5) * 16;
    }

    // A (weight) fragments: [(chunk*nsteps + step)][mfrag][plane][lane] x 8 halves
    const half8_t* wfrag = reinterpret_cast<const half8_t*>(p.wpack) +
                           (size_t)((cb * WM + wm) * FM) * NPL * 64 + lane;
    const size_t wstep = (size_t)p.mfrags * NPL * 64;
    const int total_steps = p.cin_chunks * p.nsteps;

    float16_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    half8_t a_cur[FM][NPL];
#pragma unroll
    for (int fm = 0; fm < FM; fm++)
#pragma unroll
        for (int pl = 0; pl < NPL; pl++) a_cur[fm][pl] = wfrag[(fm * NPL + pl) * 64];

    int gs = 0;
    for (int chunk = 0; chunk < p.cin_chunks; chunk++) {
        __syncthreads();
        // ---- stage the activated input halo tile of this channel chunk into LDS ----
        for (int idx = tid; idx < nitems; idx += 256) {
            const int pix = (G == 1) ? idx : idx / G;
            const int g = (G == 1) ? 0 : idx - pix * G;
            const int py = (int)(((float)pix + 0.5f) * inv_hw);
            const int px = pix - py * p.halo_w;
            const int gy = gy0 + py, gx = gx0 + px;
            const int c0 = chunk * KC + g * CPI;
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = 0.f;
            if ((unsigned)gy < (unsigned)p.in_hp && (unsigned)gx < (unsigned)p.in_wp && c0 < p.in_cp)
                load_vals<TIn>(in + ((size_t)gy * p.in_wp + gx) * p.in_cp + c0, v, CPI);
#pragma unroll
            for (int i = 0; i < CPI; i++) v[i] = act_apply(v[i], p.act);
            unsigned char* dst = lds + pix * p.pitch + g * 16;
            if (CPI == 8) {
                half8_t hi;
#pragma unroll
                for (int i = 0; i < 8; i++) hi[i] = (_Float16)v[i];
                *reinterpret_cast<half8_t*>(dst) = hi;
                if (SPLIT) {
                    half8_t lo;
#pragma unroll
                    for (int i = 0; i < 8; i++) lo[i] = (_Float16)(v[i] - (float)hi[i]);
                    *reinterpret_cast<half8_t*>(dst + p.plane) = lo;
                }
            } else {
                half4_t hi;
#pragma unroll
                for (int i = 0; i < 4; i++) hi[i] = (_Float16)v[i];
                *reinterpret_cast<half4_t*>(dst) = hi;
                if (SPLIT) {
                    half4_t lo;
#pragma unroll
                    for (int i = 0; i < 4; i++) lo[i] = (_Float16)(v[i] - (float)hi[i]);
                    *reinterpret_cast<half4_t*>(dst + p.plane) = lo;
                }
            }
        }
        __syncthreads();
        // ---- all k16 steps (taps x channel sub-blocks) of this chunk ----
        for (int t = 0; t < p.nsteps; t++, gs++) {
            const int ao = p.aoff[t];
            half8_t a_nxt[FM][NPL];
            if (gs + 1 < total_steps) {
                const half8_t* wn_ = wfrag + (size_t)(gs + 1) * wstep;
#pragma unroll
                for (int fm = 0; fm < FM; fm++)
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++) a_nxt[fm][pl] = wn_[(fm * NPL + pl) * 64];
            } else {
#pragma unroll
                for (int fm = 0; fm < FM; fm++)
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++) a_nxt[fm][pl] = a_cur[fm][pl];
            }
            half8_t b[FN][NPL];
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) {
                    const unsigned char* src = lds + pl * p.plane + boff[fn] + ao;
                    if (KC == 4) {
                        half4_t lo4 = *reinterpret_cast<const half4_t*>(src);
                        half4_t hi4 = *reinterpret_cast<const half4_t*>(src + 8);
                        half8_t r;
                        r[0] = lo4[0]; r[1] = lo4[1]; r[2] = lo4[2]; r[3] = lo4[3];
                        r[4] = hi4[0]; r[5] = hi4[1]; r[6] = hi4[2]; r[7] = hi4[3];
                        b[fn][pl] = r;
                    } else {
                        b[fn][pl] = *reinterpret_cast<const half8_t*>(src);
                    }
                }
#pragma unroll
            for (int fm = 0; fm < FM; fm++)
#pragma unroll
                for (int fn = 0; fn < FN; fn++) {
                    acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_cur[fm][0], b[fn][0], acc[fm][fn], 0, 0, 0);
                    if (SPLIT) {
                        acc[fm][fn] =
                            __builtin_amdgcn_mfma_f32_32x32x16_f16(a_cur[fm][1], b[fn][0], acc[fm][fn], 0, 0, 0);
                        acc[fm][fn] =
                            __builtin_amdgcn_mfma_f32_32x32x16_f16(a_cur[fm][0], b[fn][1], acc[fm][fn], 0, 0, 0);
                    }
                }
#pragma unroll
            for (int fm = 0; fm < FM; fm++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a_cur[fm][pl] = a_nxt[fm][pl];
        }
    }

    // ---- epilogue: lane holds, per fragment, column (position) lane%32 and rows (channels)
    //      8*(r/4) + 4*(lane/32) + r%4 ----
    TOut* out = reinterpret_cast<TOut*>(p.out);
    const TOut* res = reinterpret_cast<const TOut*>(p.res);
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = (wn * FN + fn) * 32 + (lane & 31);
        const int py = pos_y0 + (m >> twl), px = pos_x0 + (m & (TW - 1));
        if (py >= p.npos_y || px >= p.npos_x) continue;
        const size_t obase = ((size_t)(p.out_off_y + py * p.out_step) * p.out_wp + p.out_off_x + px * p.out_step) * p.out_cp;
        const size_t rbase = res ? ((size_t)(p.res_off_y + py * p.out_step) * p.res_wp + p.res_off_x + px * p.out_step) * p.res_cp : 0;
#pragma unroll
        for (int fm = 0; fm < FM; fm++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int c = ((cb * WM + wm) * FM + fm) * 32 + q * 8 + (lane >> 5) * 4;
                if (c >= p.out_cp) continue;
                const float4 sc = *reinterpret_cast<const float4*>(p.scale + c);
                const float4 bi = *reinterpret_cast<const float4*>(p.bias + c);
                float o[4];
                o[0] = (acc[fm][fn][q * 4 + 0] * p.acc_mul) * sc.x + bi.x;
                o[1] = (acc[fm][fn][q * 4 + 1] * p.acc_mul) * sc.y + bi.y;
                o[2] = (acc[fm][fn][q * 4 + 2] * p.acc_mul) * sc.z + bi.z;
                o[3] = (acc[fm][fn][q * 4 + 3] * p.acc_mul) * sc.w + bi.w;
                if (res) {
                    float r[8];
                    load_vals<TOut>(res + rbase + c, r, 4);
                    const float rs[4] = {sc.x, sc.y, sc.z, sc.w};
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        float rv = r[i];
                        if (p.res_relu) rv = fmaxf(rv, 0.f);
                        if (p.res_scale) rv *= rs[i];
                        o[i] += rv;
                    }
                }
                if (sizeof(TOut) == 4) {
                    *reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + obase + c) = make_float4(o[0], o[1], o[2], o[3]);
                } else {
                    half4_t hv;
#pragma unroll
                    for (int i = 0; i < 4; i++) hv[i] = (_Float16)o[i];
                    *reinterpret_cast<half4_t*>(reinterpret_cast<_Float16*>(out) + obase + c) = hv;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// variant table
// ---------------------------------------------------------------------------------------------
typedef void (*conv_kernel_fn)(const ConvMfmaParams);

template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN>
static conv_kernel_fn pick_kc(int kc) {
    switch (kc) {
        case 4: return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 4>;
        case 16: return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 16>;
        case 32: return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32>;
        default: return nullptr;
    }
}

template <typename TIn, typename TOut, bool SPLIT>
static conv_kernel_fn pick_tile(const ConvVariant& v) {
#define FYN_TILE(fm_, fn_, wm_, wn_) \
    if (v.fm == fm_ && v.fn == fn_ && v.wm == wm_ && v.wn == wn_) return pick_kc<TIn, TOut, SPLIT, fm_, fn_, wm_, wn_>(v.kc);
    FYN_TILE(2, 2, 2, 2)  // 128 cout x 128 positions
    FYN_TILE(2, 2, 1, 4)  //  64 cout x 256 positions
    FYN_TILE(2, 1, 2, 2)  // 128 cout x  64 positions
    FYN_TILE(2, 1, 1, 4)  //  64 cout x 128 positions
    FYN_TILE(1, 2, 1, 4)  //  32 cout x 256 positions
    FYN_TILE(1, 1, 1, 4)  //  32 cout x 128 positions
    FYN_TILE(1, 1, 4, 1)  // 128 cout x  32 positions
    FYN_TILE(1, 1, 2, 2)  //  64 cout x  64 positions
#undef FYN_TILE
    return nullptr;
}

static conv_kernel_fn pick_kernel(const ConvVariant& v) {
    if (v.split) {
        if (v.in_f16 || v.out_f16) return nullptr;  // split arithmetic is the fp32-storage path
        return pick_tile<float, float, true>(v);
    }
    if (v.in_f16 && v.out_f16) return pick_tile<_Float16, _Float16, false>(v);
    if (!v.in_f16 && v.out_f16) return pick_tile<float, _Float16, false>(v);
    if (!v.in_f16 && !v.out_f16) return pick_tile<float, float, false>(v);
    return nullptr;
}

bool conv_mfma_variant_exists(const ConvVariant& v) { return pick_kernel(v) != nullptr; }

int launch_conv_mfma(const ConvVariant& v, const ConvMfmaParams& p, size_t lds_bytes, hipStream_t s) {
    conv_kernel_fn fn = pick_kernel(v);
    if (!fn) return -1;
    if (lds_bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) != hipSuccess)
            return -2;
    }
    const int blocks = p.tiles_x * p.tiles_y * p.cout_blocks;
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(256), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace fynhip
