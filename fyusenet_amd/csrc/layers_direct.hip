// Bandwidth-bound layer kernels for gfx950 (no matrix cores): depthwise 3x3 convolution, pooling,
// global pooling, explicit batch-norm, add/sub, concat, exact arg-max, the fully connected
// matrix-vector product, a direct (fallback) convolution and the layout converters at the
// upload/download boundary.  All operate on the channel-packed NHWC layout described in kernels.h;
// one thread moves 4 consecutive channels of one pixel (16 B in fp32 storage, 8 B in fp16 storage),
// consecutive threads touch consecutive channels, so every wavefront access is one contiguous run.
// The activation of the producing layer is applied on input fetch (shaders/activation.inc:3-18).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "kernels.h"
#include "range.h"

namespace fynhip {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// Activation on fetch.  The host normalises every kind to act(x) = min(hi, max(lo, x)) + leak * min(x, 0)
// (none: lo = -inf, hi = +inf, leak = 0; ReLU: lo = 0; leaky: lo = 0, leak; clip: lo, hi), which is evaluated without
// branches; "none" skips the arithmetic altogether (one uniform branch per vector).
__device__ __forceinline__ float act1(float x, const Act& a) {
    return (a.kind == ACT_NONE) ? x : fminf(a.hi, fmaxf(a.lo, x)) + a.leak * fminf(x, 0.f);
}
__device__ __forceinline__ float4 act4(float4 v, const Act& a) {
    if (a.kind == ACT_NONE) return v;
    return make_float4(fminf(a.hi, fmaxf(a.lo, v.x)) + a.leak * fminf(v.x, 0.f), fminf(a.hi, fmaxf(a.lo, v.y)) + a.leak * fminf(v.y, 0.f),
                       fminf(a.hi, fmaxf(a.lo, v.z)) + a.leak * fminf(v.z, 0.f), fminf(a.hi, fmaxf(a.lo, v.w)) + a.leak * fminf(v.w, 0.f));
}

template <typename T>
__device__ __forceinline__ float4 ld4(const T* p);
template <>
__device__ __forceinline__ float4 ld4<float>(const float* p) {
    return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 ld4<_Float16>(const _Float16* p) {
    half4_t h = *reinterpret_cast<const half4_t*>(p);
    return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}
template <typename T>
__device__ __forceinline__ void st4(T* p, float4 v);
template <>
__device__ __forceinline__ void st4<float>(float* p, float4 v) {
    *reinterpret_cast<float4*>(p) = v;
}
template <>
__device__ __forceinline__ void st4<_Float16>(_Float16* p, float4 v) {
    half4_t h;
    h[0] = (_Float16)v.x; h[1] = (_Float16)v.y; h[2] = (_Float16)v.z; h[3] = (_Float16)v.w;
    *reinterpret_cast<half4_t*>(p) = h;
}

__device__ __forceinline__ size_t tv_off(const TView& t, int y, int x) {  // net coords -> element offset
    return ((size_t)(y + t.pad) * t.wp() + (x + t.pad)) * t.cp;
}

// V consecutive channels of one pixel as floats.  fp16 tensors whose channel pitch allows it are moved 8 channels
// (16 bytes) per thread, everything else 4 channels per thread.
template <int V>
struct FV {
    float v[V];
};
template <typename T, int V>
__device__ __forceinline__ FV<V> ldv(const T* p) {
    FV<V> r;
    if constexpr (V == 8 && sizeof(T) == 2) {
        const half8_t h = *reinterpret_cast<const half8_t*>(p);
#pragma unroll
        for (int i = 0; i < 8; i++) r.v[i] = (float)h[i];
    } else {
#pragma unroll
        for (int q = 0; q < V / 4; q++) {
            const float4 a = ld4<T>(p + 4 * q);
            r.v[4 * q + 0] = a.x; r.v[4 * q + 1] = a.y; r.v[4 * q + 2] = a.z; r.v[4 * q + 3] = a.w;
        }
    }
    return r;
}
template <typename T, int V>
__device__ __forceinline__ void stv(T* p, const FV<V>& r) {
    if constexpr (V == 8 && sizeof(T) == 2) {
        half8_t h;
#pragma unroll
        for (int i = 0; i < 8; i++) h[i] = (_Float16)r.v[i];
        *reinterpret_cast<half8_t*>(p) = h;
    } else {
#pragma unroll
        for (int q = 0; q < V / 4; q++) st4<T>(p + 4 * q, make_float4(r.v[4 * q + 0], r.v[4 * q + 1], r.v[4 * q + 2], r.v[4 * q + 3]));
    }
}
template <int V>
__device__ __forceinline__ FV<V> zerov() {
    FV<V> r;
#pragma unroll
    for (int i = 0; i < V; i++) r.v[i] = 0.f;
    return r;
}
template <int V>
__device__ __forceinline__ FV<V> actv(FV<V> r, const Act& a) {
    if (a.kind == ACT_NONE) return r;
#pragma unroll
    for (int i = 0; i < V; i++) r.v[i] = fminf(a.hi, fmaxf(a.lo, r.v[i])) + a.leak * fminf(r.v[i], 0.f);
    return r;
}

// wide: every tensor of the launch has a channel pitch that is a multiple of 8
#define FYN_DISPATCH_TV(f16, wide, KERNEL, grid, block, stream, ...)                                       \
    do {                                                                                                   \
        if ((f16) && (wide)) hipLaunchKernelGGL((KERNEL<_Float16, 8>), grid, block, 0, stream, __VA_ARGS__); \
        else if (f16) hipLaunchKernelGGL((KERNEL<_Float16, 4>), grid, block, 0, stream, __VA_ARGS__);       \
        else hipLaunchKernelGGL((KERNEL<float, 4>), grid, block, 0, stream, __VA_ARGS__);                  \
    } while (0)

#define FYN_DISPATCH_T(f16, KERNEL, grid, block, stream, ...)                                   \
    do {                                                                                        \
        if (f16) hipLaunchKernelGGL((KERNEL<_Float16>), grid, block, 0, stream, __VA_ARGS__);   \
        else hipLaunchKernelGGL((KERNEL<float>), grid, block, 0, stream, __VA_ARGS__);          \
    } while (0)

static inline dim3 grid1d(size_t n, int block) { return dim3((unsigned)((n + block - 1) / block)); }
// A thread's pixel and channel group in the element-wise kernels.  grid_rows() gives one grid row per tensor row where a
// row fills at least a workgroup and the height fits the grid's second dimension: the index arithmetic is then one
// 32-bit division instead of three 64-bit ones, which were most of the instructions of a thread that moves 16 bytes.
struct PixelIndex {
    int y, x, g;
    bool inside;
};
__device__ __forceinline__ PixelIndex pixel_index(int h, int w, int cg) {
    PixelIndex r;
    if (gridDim.y > 1) {
        const unsigned i = blockIdx.x * 256u + threadIdx.x;
        r.inside = i < (unsigned)w * (unsigned)cg;
        r.y = (int)blockIdx.y;
        r.x = (int)(i / (unsigned)cg);
        r.g = (int)(i - (unsigned)r.x * (unsigned)cg);
    } else {
        const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
        r.inside = idx < (size_t)h * w * cg;
        r.g = (int)(idx % cg);
        const size_t pix = idx / cg;
        r.x = (int)(pix % w);
        r.y = (int)(pix / w);
    }
    return r;
}
static inline dim3 grid_rows(int h, int w, int cg) {
    const long long row = (long long)w * cg;
    if (h > 1 && h <= 65535 && row >= 256 && row < (1ll << 31)) return dim3((unsigned)((row + 255) / 256), (unsigned)h);
    return grid1d((size_t)h * w * cg, 256);
}

// ---------------------------------------------------------------------------------------------
// depthwise 3x3  (DeepDepthwiseConvLayer3x3::forward, gpu/deep/deepdwconvlayer3x3.cpp:67-102;
//                 shaders/deep/deepconv_dw3x3_tiled.frag:36-59)
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dwconv3x3_kernel(const DwConvParams p) {
    const int cg = p.out.cp >> 2;
    const size_t n = (size_t)p.out.h * p.out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % p.out.w), y = (int)(pix / p.out.w);
    const int c = g * 4;
    const T* in = reinterpret_cast<const T*>(p.in.ptr);
    const int iwp = p.in.wp(), ihp = p.in.hp();
    const int yc = y * p.stride + p.in.pad, xc = x * p.stride + p.in.pad;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int ky = 0; ky < 3; ky++) {
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const int sy = yc + (ky - 1) * p.dil, sx = xc + (kx - 1) * p.dil;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if ((unsigned)sy < (unsigned)ihp && (unsigned)sx < (unsigned)iwp)
                v = ld4<T>(in + ((size_t)sy * iwp + sx) * p.in.cp + c);
            v = act4(v, p.act);
            const float4 w = *reinterpret_cast<const float4*>(p.w + (ky * 3 + kx) * p.out.cp + c);
            acc.x = fmaf(v.x, w.x, acc.x); acc.y = fmaf(v.y, w.y, acc.y);
            acc.z = fmaf(v.z, w.z, acc.z); acc.w = fmaf(v.w, w.w, acc.w);
        }
    }
    const float4 sc = *reinterpret_cast<const float4*>(p.scale + c);
    const float4 bi = *reinterpret_cast<const float4*>(p.bias + c);
    float4 o = make_float4(acc.x * sc.x + bi.x, acc.y * sc.y + bi.y, acc.z * sc.z + bi.z, acc.w * sc.w + bi.w);
    if (p.res.ptr) {
        float4 r = ld4<T>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x) + c);
        if (p.res_relu) r = make_float4(fmaxf(r.x, 0.f), fmaxf(r.y, 0.f), fmaxf(r.z, 0.f), fmaxf(r.w, 0.f));
        if (p.res_scale) r = make_float4(r.x * sc.x, r.y * sc.y, r.z * sc.z, r.w * sc.w);
        o = make_float4(o.x + r.x, o.y + r.y, o.z + r.z, o.w + r.w);
    }
    st4<T>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, o);
}
// V stored elements as they come from memory (one 8- or 16-byte load).
template <typename T, int V>
struct alignas(sizeof(T) * V) RawV {
    T v[V];
};

// Undilated depthwise 3x3, stride S: one thread produces PX (four, on small layers two or one: more threads, each
// done sooner) neighbouring output pixels of V channels from a 3 x ((PX-1)*S+3) input window, so that an input texel is
// fetched once per thread instead of up to three times and the nine weight vectors are loaded once per PX outputs.  All loads of the window are issued before the first
// use (one memory round trip per thread); the texels stay in their stored type until they are consumed.  Same
// accumulation order per output (ky outer, kx inner, fused multiply-add) as dwconv3x3_kernel.
template <typename T, int V, int S, int PX>
__global__ __launch_bounds__(256) void dwconv3x3_row_kernel(const DwConvParams p) {
    constexpr int WIN = (PX - 1) * S + 3;
    const int cg = p.out.cp / V;
    const int xb = (p.out.w + PX - 1) / PX;
    const size_t n = (size_t)p.out.h * xb * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t t = idx / cg;
    const int bx = (int)(t % xb), y = (int)(t / xb);
    const int c = g * V, x0 = bx * PX;
    const T* in = reinterpret_cast<const T*>(p.in.ptr);
    const int iwp = p.in.wp(), ihp = p.in.hp();
    const int sx0 = x0 * S + p.in.pad - 1;
    RawV<T, V> raw[3][WIN];
#pragma unroll
    for (int ky = 0; ky < 3; ky++) {
        const int sy = y * S + p.in.pad + (ky - 1);
        const bool row_ok = (unsigned)sy < (unsigned)ihp;
#pragma unroll
        for (int j = 0; j < WIN; j++) {
            const int sx = sx0 + j;
#pragma unroll
            for (int i = 0; i < V; i++) raw[ky][j].v[i] = (T)0.f;
            if (row_ok && (unsigned)sx < (unsigned)iwp) raw[ky][j] = *reinterpret_cast<const RawV<T, V>*>(in + ((size_t)sy * iwp + sx) * p.in.cp + c);
        }
    }
    // min(hi, max(lo, x)) in fp16 equals the fp32 evaluation when there is no leak and both bounds are fp16 values:
    // then it is applied to the packed halves, two elements per instruction, before the conversion
    const _Float16 hlo = (_Float16)p.act.lo, hhi = (_Float16)p.act.hi;
    const bool packed_act = sizeof(T) == 2 && V == 8 && p.act.leak == 0.f && (float)hlo == p.act.lo && (float)hhi == p.act.hi;
    FV<V> acc[PX];
#pragma unroll
    for (int px = 0; px < PX; px++) acc[px] = zerov<V>();
#pragma unroll
    for (int ky = 0; ky < 3; ky++) {
        FV<V> row[WIN];
#pragma unroll
        for (int j = 0; j < WIN; j++) {
            if constexpr (V == 8 && sizeof(T) == 2) {
                if (packed_act) {
                    half8_t h = __builtin_bit_cast(half8_t, raw[ky][j]);
                    h = __builtin_elementwise_min(__builtin_elementwise_max(h, (half8_t)hlo), (half8_t)hhi);
#pragma unroll
                    for (int i = 0; i < 8; i++) row[j].v[i] = (float)h[i];
                    continue;
                }
            }
            FV<V> v;
#pragma unroll
            for (int i = 0; i < V; i++) v.v[i] = (float)raw[ky][j].v[i];
            row[j] = actv<V>(v, p.act);
        }
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const FV<V> w = ldv<float, V>(p.w + (ky * 3 + kx) * p.out.cp + c);
#pragma unroll
            for (int px = 0; px < PX; px++)
#pragma unroll
                for (int i = 0; i < V; i++) acc[px].v[i] = fmaf(row[px * S + kx].v[i], w.v[i], acc[px].v[i]);
        }
    }
    const FV<V> sc = ldv<float, V>(p.scale + c), bi = ldv<float, V>(p.bias + c);
#pragma unroll
    for (int px = 0; px < PX; px++) {
        const int x = x0 + px;
        if (x >= p.out.w) break;
        FV<V> o;
#pragma unroll
        for (int i = 0; i < V; i++) o.v[i] = acc[px].v[i] * sc.v[i] + bi.v[i];
        if (p.res.ptr) {
            const FV<V> r = ldv<T, V>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x) + c);
#pragma unroll
            for (int i = 0; i < V; i++) {
                float rv = r.v[i];
                if (p.res_relu) rv = fmaxf(rv, 0.f);
                if (p.res_scale) rv *= sc.v[i];
                o.v[i] += rv;
            }
        }
        stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, o);
    }
}

// The same convolution with a thread walking DOWN a strip of four output columns: the three input rows of a window
// stay in registers (in their stored type, already activated) and every step fetches only the row(s) that enter the
// window, one step ahead of their use, so an input texel is fetched 1.5 times (the strips' horizontal overlap) instead
// of 4.5 times, and the nine weight vectors are loaded once per strip.  Same accumulation order per output as the
// kernels above.  fp16 tensors: the activation must be a clamp that is exact on halves (no leak, bounds representable;
// the caller checks), it is applied to the packed halves; products are formed from the halves with fp32 accumulation.
template <typename T, int V, int S>
__global__ __launch_bounds__(256) void dwconv3x3_col_kernel(const DwConvParams p, int rows_per_thread) {
    constexpr int PX = 4, WIN = (PX - 1) * S + 3;
    typedef RawV<T, V> Raw;
    const int cg = p.out.cp / V;
    const int xb = (p.out.w + PX - 1) / PX;
    const int yb = (p.out.h + rows_per_thread - 1) / rows_per_thread;
    const size_t n = (size_t)yb * xb * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t t = idx / cg;
    const int bx = (int)(t % xb), by = (int)(t / xb);
    const int c = g * V, x0 = bx * PX;
    const int y_begin = by * rows_per_thread, y_end = min(y_begin + rows_per_thread, p.out.h);
    const T* in = reinterpret_cast<const T*>(p.in.ptr);
    const int iwp = p.in.wp(), ihp = p.in.hp();
    const int sx0 = x0 * S + p.in.pad - 1;
    const _Float16 hlo = (_Float16)p.act.lo, hhi = (_Float16)p.act.hi;
    auto load_row = [&](Raw (&dst)[WIN], int sy) {
        const bool row_ok = (unsigned)sy < (unsigned)ihp;
#pragma unroll
        for (int j = 0; j < WIN; j++) {
            const int sx = sx0 + j;
#pragma unroll
            for (int i = 0; i < V; i++) dst[j].v[i] = (T)0.f;
            if (row_ok && (unsigned)sx < (unsigned)iwp) dst[j] = *reinterpret_cast<const Raw*>(in + ((size_t)sy * iwp + sx) * p.in.cp + c);
        }
    };
    auto activate = [&](Raw (&r)[WIN]) {
#pragma unroll
        for (int j = 0; j < WIN; j++) {
            if constexpr (sizeof(T) == 2) {
                typedef _Float16 halfv_t __attribute__((ext_vector_type(V)));
                halfv_t h = __builtin_bit_cast(halfv_t, r[j]);
                h = __builtin_elementwise_min(__builtin_elementwise_max(h, (halfv_t)hlo), (halfv_t)hhi);
                r[j] = __builtin_bit_cast(Raw, h);
            } else {
#pragma unroll
                for (int i = 0; i < V; i++) r[j].v[i] = (T)act1((float)r[j].v[i], p.act);
            }
        }
    };
    FV<V> w[9];
#pragma unroll
    for (int k = 0; k < 9; k++) w[k] = ldv<float, V>(p.w + k * p.out.cp + c);
    const FV<V> sc = ldv<float, V>(p.scale + c), bi = ldv<float, V>(p.bias + c);
    // window rows of output row y: stored rows y*S + pad - 1 + {0, 1, 2}
    Raw win[3][WIN], nxt[S][WIN];
    const int sy0 = y_begin * S + p.in.pad - 1;
#pragma unroll
    for (int ky = 0; ky < 3; ky++) load_row(win[ky], sy0 + ky);
#pragma unroll
    for (int ky = 0; ky < 3; ky++) activate(win[ky]);
    for (int y = y_begin; y < y_end; y++) {
        // the S rows that enter the window of the next output row are requested before this row is computed
        if (y + 1 < y_end) {
#pragma unroll
            for (int q = 0; q < S; q++) load_row(nxt[q], (y + 1) * S + p.in.pad - 1 + (3 - S) + q);
        }
        FV<V> acc[PX];
#pragma unroll
        for (int px = 0; px < PX; px++) acc[px] = zerov<V>();
#pragma unroll
        for (int ky = 0; ky < 3; ky++)
#pragma unroll
            for (int kx = 0; kx < 3; kx++)
#pragma unroll
                for (int px = 0; px < PX; px++)
#pragma unroll
                    for (int i = 0; i < V; i++) acc[px].v[i] = fmaf((float)win[ky][px * S + kx].v[i], w[ky * 3 + kx].v[i], acc[px].v[i]);
#pragma unroll
        for (int px = 0; px < PX; px++) {
            const int x = x0 + px;
            if (x >= p.out.w) break;
            FV<V> o;
#pragma unroll
            for (int i = 0; i < V; i++) o.v[i] = acc[px].v[i] * sc.v[i] + bi.v[i];
            if (p.res.ptr) {
                const FV<V> r = ldv<T, V>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x) + c);
#pragma unroll
                for (int i = 0; i < V; i++) {
                    float rv = r.v[i];
                    if (p.res_relu) rv = fmaxf(rv, 0.f);
                    if (p.res_scale) rv *= sc.v[i];
                    o.v[i] += rv;
                }
            }
            stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, o);
        }
        if (y + 1 < y_end) {
            // slide the window down by S rows
#pragma unroll
            for (int q = 0; q < S; q++) activate(nxt[q]);
#pragma unroll
            for (int ky = 0; ky + S < 3; ky++)
#pragma unroll
                for (int j = 0; j < WIN; j++) win[ky][j] = win[ky + S][j];
#pragma unroll
            for (int q = 0; q < S; q++)
#pragma unroll
                for (int j = 0; j < WIN; j++) win[3 - S + q][j] = nxt[q][j];
        }
    }
}

template <typename T, int V, int PX>
static void launch_dw_row_px(const DwConvParams& p, hipStream_t s) {
    const size_t n = (size_t)p.out.h * ((p.out.w + PX - 1) / PX) * (p.out.cp / V);
    if (p.stride == 1) hipLaunchKernelGGL((dwconv3x3_row_kernel<T, V, 1, PX>), grid1d(n, 256), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((dwconv3x3_row_kernel<T, V, 2, PX>), grid1d(n, 256), dim3(256), 0, s, p);
}
// (pixels per thread: four when that still gives every SIMD of the chip a wave, else two, else one)
template <typename T, int V>
static void launch_dw_row(const DwConvParams& p, hipStream_t s) {
    const size_t per_px = (size_t)p.out.h * (p.out.cp / V);
    const size_t want = 256 * 4 * 64;
    if (per_px * ((p.out.w + 3) / 4) >= want) launch_dw_row_px<T, V, 4>(p, s);
    else if (per_px * ((p.out.w + 1) / 2) >= want) launch_dw_row_px<T, V, 2>(p, s);
    else launch_dw_row_px<T, V, 1>(p, s);
}

// strips of `rows` output rows per thread, when the image is tall enough to leave the chip enough threads
template <typename T, int V>
static bool launch_dw_col(const DwConvParams& p, hipStream_t s) {
    if (p.no_strips) return false;
    const size_t per_row = (size_t)((p.out.w + 3) / 4) * (p.out.cp / V);
    int rows = 16;
    while (rows > 2 && per_row * ((p.out.h + rows - 1) / rows) < 256 * 256 * 2) rows /= 2;   // at least two waves per SIMD of work
    if (rows < 4 || p.out.h < rows) return false;
    const size_t n = per_row * ((p.out.h + rows - 1) / rows);
    if (p.stride == 1) hipLaunchKernelGGL((dwconv3x3_col_kernel<T, V, 1>), grid1d(n, 256), dim3(256), 0, s, p, rows);
    else hipLaunchKernelGGL((dwconv3x3_col_kernel<T, V, 2>), grid1d(n, 256), dim3(256), 0, s, p, rows);
    return true;
}

void launch_dwconv3x3(const DwConvParams& p, hipStream_t s) {
    if (p.dil == 1 && (p.stride == 1 || p.stride == 2) && p.out.w >= 4) {
        const bool wide = (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0) && (!p.res.ptr || p.res.cp % 8 == 0);
        // a clamp that is exact on halves (the strip kernel applies it to the packed halves)
        const _Float16 hlo = (_Float16)p.act.lo, hhi = (_Float16)p.act.hi;
        const bool half_act = p.act.leak == 0.f && (float)hlo == p.act.lo && (float)hhi == p.act.hi;
        if (p.out.f16 && half_act && launch_dw_col<_Float16, 4>(p, s)) return;
        if (!p.out.f16 && launch_dw_col<float, 4>(p, s)) return;
        if (p.out.f16 && wide) launch_dw_row<_Float16, 8>(p, s);
        else if (p.out.f16) launch_dw_row<_Float16, 4>(p, s);
        else launch_dw_row<float, 4>(p, s);
        return;
    }
    const size_t n = (size_t)p.out.h * p.out.w * (p.out.cp >> 2);
    FYN_DISPATCH_T(p.out.f16, dwconv3x3_kernel, grid1d(n, 256), dim3(256), s, p);
}

// ---------------------------------------------------------------------------------------------
// max / average pooling  (DeepPoolingLayer::forward, gpu/deep/deeppoolinglayer.cpp:109-131;
//                         shaders/deep/deepmaxpool.frag:12-59, deepavgpool.frag:15-58)
// ---------------------------------------------------------------------------------------------
// P: window size known at compile time (2, 3: all loads of a window are issued before the first use), 0: any size
template <typename T, int V, int P>
__global__ __launch_bounds__(256) void pool_kernel(const PoolParams p) {
    const int cg = p.out.cp / V;
    const PixelIndex pi = pixel_index(p.out.h, p.out.w, cg);
    if (!pi.inside) return;
    const int g = pi.g, x = pi.x, y = pi.y;
    const int c = g * V;
    const T* in = reinterpret_cast<const T*>(p.in.ptr);
    const int iwp = p.in.wp(), ihp = p.in.hp();
    const int y0 = y * p.stride + p.off, x0 = x * p.stride + p.off;  // stored coordinates
    FV<V> acc = zerov<V>();
    auto fold = [&](const FV<V>& v, bool first_tap) {
#pragma unroll
        for (int i = 0; i < V; i++) {
            if (p.is_max) acc.v[i] = first_tap ? v.v[i] : fmaxf(acc.v[i], v.v[i]);
            else acc.v[i] += v.v[i];
        }
    };
    auto fetch = [&](int sy, int sx) {
        FV<V> v = zerov<V>();
        if ((unsigned)sy < (unsigned)ihp && (unsigned)sx < (unsigned)iwp) v = ldv<T, V>(in + ((size_t)sy * iwp + sx) * p.in.cp + c);
        return v;
    };
    if constexpr (P > 0) {
        FV<V> win[P][P];
#pragma unroll
        for (int py = 0; py < P; py++)
#pragma unroll
            for (int px = 0; px < P; px++) win[py][px] = fetch(y0 + py, x0 + px);
#pragma unroll
        for (int py = 0; py < P; py++)
#pragma unroll
            for (int px = 0; px < P; px++) fold(actv<V>(win[py][px], p.act), py == 0 && px == 0);
    } else {
        for (int py = 0; py < p.pool; py++)
            for (int px = 0; px < p.pool; px++) fold(actv<V>(fetch(y0 + py, x0 + px), p.act), py == 0 && px == 0);
    }
    if (!p.is_max) {
        const float inv = 1.0f / (float)(p.pool * p.pool);
#pragma unroll
        for (int i = 0; i < V; i++) acc.v[i] *= inv;
    }
    stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, acc);
}
template <int P>
static void launch_pool_p(const PoolParams& p, hipStream_t s) {
    const bool wide = (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0);
    const dim3 grid = grid_rows(p.out.h, p.out.w, p.out.cp / ((p.out.f16 && wide) ? 8 : 4));
    if (p.out.f16 && wide) hipLaunchKernelGGL((pool_kernel<_Float16, 8, P>), grid, dim3(256), 0, s, p);
    else if (p.out.f16) hipLaunchKernelGGL((pool_kernel<_Float16, 4, P>), grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL((pool_kernel<float, 4, P>), grid, dim3(256), 0, s, p);
}
void launch_pool(const PoolParams& p, hipStream_t s) {
    if (p.pool == 2) launch_pool_p<2>(p, s);
    else if (p.pool == 3) launch_pool_p<3>(p, s);
    else launch_pool_p<0>(p, s);
}

// ---------------------------------------------------------------------------------------------
// global pooling  (DeepGlobalPoolLayer, gpu/deep/deepglobalpoollayer.cpp:55-135;
//                  shaders/deep/deepglobavgpool.frag:15-24).  One block per run of up to 64
// channel groups; the block's threads split the pixels, partial results meet in LDS.
// ---------------------------------------------------------------------------------------------
// Large images: the pixels are dealt to gridDim.y workgroups per run of channel groups, each of which leaves its
// sum (maximum) in row blockIdx.y of a small fp32 tensor (`out`, `mul` = 1), and a second launch of the same kernel
// pools that tensor (`mul` = 1 / pixels of the image).  TOut: the element type of `out`.
template <typename T, typename TOut>
__global__ __launch_bounds__(256) void global_pool_kernel(const TView in, const TView out, int is_max, const Act act,
                                                          int cgb_log2, float mul) {
    __shared__ float4 red[256];
    const int cgs = in.cp >> 2;
    const int cgb = 1 << cgb_log2;             // channel groups handled by this block
    const int parts = 256 >> cgb_log2;         // pixel partitions
    const int lg = threadIdx.x & (cgb - 1);
    const int part = threadIdx.x >> cgb_log2;
    const int g = blockIdx.x * cgb + lg;
    const int total = in.h * in.w;
    const int share = (total + gridDim.y - 1) / gridDim.y;
    const int pbeg = blockIdx.y * share;
    const int npix = min(total, pbeg + share);   // (end of this workgroup's pixels)
    const T* src = reinterpret_cast<const T*>(in.ptr);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    bool first = true;
    if (g < cgs) {
        // eight pixels per trip: their loads are issued together, then folded in pixel order (a tensor without a halo
        // is one run of pixels: no row arithmetic)
        constexpr int NJ = 8;
        const bool flat = in.pad == 0;
        for (int pix0 = pbeg + part; pix0 < npix; pix0 += NJ * parts) {
            float4 v4[NJ];
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int pix = pix0 + j * parts;
                const int pc = pix < npix ? pix : pix0;
                size_t off;
                if (flat) {
                    off = (size_t)pc * in.cp;
                } else {
                    const int y = pc / in.w, x = pc - y * in.w;
                    off = tv_off(in, y, x);
                }
                v4[j] = ld4<T>(src + off + g * 4);
            }
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                if (pix0 + j * parts >= npix) break;
                const float4 v = act4(v4[j], act);
                if (is_max) {
                    acc = first ? v : make_float4(fmaxf(acc.x, v.x), fmaxf(acc.y, v.y), fmaxf(acc.z, v.z), fmaxf(acc.w, v.w));
                    first = false;
                } else {
                    acc = make_float4(acc.x + v.x, acc.y + v.y, acc.z + v.z, acc.w + v.w);
                }
            }
        }
    }
    if (is_max && first) acc = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int st = parts >> 1; st > 0; st >>= 1) {
        if (part < st) {
            float4 a = red[threadIdx.x], b = red[threadIdx.x + st * cgb];
            red[threadIdx.x] = is_max ? make_float4(fmaxf(a.x, b.x), fmaxf(a.y, b.y), fmaxf(a.z, b.z), fmaxf(a.w, b.w))
                                      : make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
        }
        __syncthreads();
    }
    if (part == 0 && g < cgs) {
        float4 r = red[threadIdx.x];
        if (!is_max) r = make_float4(r.x * mul, r.y * mul, r.z * mul, r.w * mul);
        st4<TOut>(reinterpret_cast<TOut*>(out.ptr) + tv_off(out, 0, blockIdx.y) + g * 4, r);
    }
}
// splits > 1: `partial` holds splits x in.cp floats (the pixels are dealt to that many workgroups per run of channel groups)
void launch_global_pool(const TView& in, const TView& out, int is_max, const Act& act, hipStream_t s, float* partial, int splits) {
    const int cgs = in.cp >> 2;
    // few channel groups per workgroup: more workgroups, and more threads sharing the pixels of a group
    int l2 = 0;
    while ((1 << l2) < cgs && l2 < 4) l2++;
    const int cgb = 1 << l2;
    const dim3 grid((cgs + cgb - 1) / cgb);
    const float inv = 1.0f / (float)(in.h * in.w);
    if (partial && splits > 1) {
        TView pv{};
        pv.ptr = partial; pv.h = 1; pv.w = splits; pv.pad = 0; pv.c = in.c; pv.cp = in.cp; pv.f16 = 0;
        Act none{};
        none.kind = ACT_NONE;
        if (in.f16) hipLaunchKernelGGL((global_pool_kernel<_Float16, float>), dim3(grid.x, splits), dim3(256), 0, s, in, pv, is_max, act, l2, 1.0f);
        else hipLaunchKernelGGL((global_pool_kernel<float, float>), dim3(grid.x, splits), dim3(256), 0, s, in, pv, is_max, act, l2, 1.0f);
        if (out.f16) hipLaunchKernelGGL((global_pool_kernel<float, _Float16>), grid, dim3(256), 0, s, pv, out, is_max, none, l2, inv);
        else hipLaunchKernelGGL((global_pool_kernel<float, float>), grid, dim3(256), 0, s, pv, out, is_max, none, l2, inv);
        return;
    }
    if (in.f16) hipLaunchKernelGGL((global_pool_kernel<_Float16, _Float16>), grid, dim3(256), 0, s, in, out, is_max, act, l2, inv);
    else hipLaunchKernelGGL((global_pool_kernel<float, float>), grid, dim3(256), 0, s, in, out, is_max, act, l2, inv);
}

// ---------------------------------------------------------------------------------------------
// explicit batch-norm (DeepBatchNormLayer, shaders/deep/deepbatchnorm.frag:24-36), add/sub
// (shaders/add.frag) and one input of a concatenation (shaders/deep/deepconcat.frag:45-76)
// ---------------------------------------------------------------------------------------------
template <typename T, int V>
__global__ __launch_bounds__(256) void batchnorm_kernel(const BnParams p) {
    const int cg = p.out.cp / V;
    const PixelIndex pi = pixel_index(p.out.h, p.out.w, cg);
    if (!pi.inside) return;
    const int g = pi.g, x = pi.x, y = pi.y;
    const int c = g * V;
    FV<V> v = actv<V>(ldv<T, V>(reinterpret_cast<const T*>(p.in.ptr) + tv_off(p.in, y, x) + c), p.act);
    const FV<V> sc = ldv<float, V>(p.scale + c), bi = ldv<float, V>(p.bias + c);
    FV<V> o;
#pragma unroll
    for (int i = 0; i < V; i++) o.v[i] = v.v[i] * sc.v[i] + bi.v[i];
    if (p.res.ptr) {
        FV<V> r = ldv<T, V>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x) + c);
#pragma unroll
        for (int i = 0; i < V; i++) {
            float rv = r.v[i];
            if (p.res_relu) rv = fmaxf(rv, 0.f);
            if (p.res_bn) rv = rv * sc.v[i] + bi.v[i];
            o.v[i] += rv;
        }
    }
    stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, o);
}
void launch_batchnorm(const BnParams& p, hipStream_t s) {
    const bool wide = (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0) && (!p.res.ptr || p.res.cp % 8 == 0);
    FYN_DISPATCH_TV(p.out.f16, wide, batchnorm_kernel, grid_rows(p.out.h, p.out.w, p.out.cp / ((p.out.f16 && wide) ? 8 : 4)), dim3(256), s, p);
}

// ---------------------------------------------------------------------------------------------
// function-type layers: scale / padding / relu / clip / deep<->shallow (shaders/deep/deepdefault.frag, scaling.frag),
// sigmoid (deepsigmoid.frag), tanh (deeptanh.frag), singleton arithmetic (deep_singleton_arith.frag), cast
// (typecast.inc), transpose (deeptransposelayer.cpp:141-156), image-patch extraction (deepimgpatch.frag),
// RGB<->BGR (rgb2bgr.frag), non-maximum suppression (nonmax2d.frag), blur (generickernel.frag)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int floordiv_pos(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

// Texel at stored coordinates, edge repeated beyond the stored tensor; channels >= in.c read as zero.
template <typename T>
__device__ __forceinline__ float4 fetch_clamped(const TView& t, int sy, int sx, int c) {
    sy = min(max(sy, 0), t.hp() - 1);
    sx = min(max(sx, 0), t.wp() - 1);
    float4 v = ld4<T>(reinterpret_cast<const T*>(t.ptr) + ((size_t)sy * t.wp() + sx) * t.cp + c);
    if (c + 3 >= t.c) {
        if (c + 0 >= t.c) v.x = 0.f;
        if (c + 1 >= t.c) v.y = 0.f;
        if (c + 2 >= t.c) v.z = 0.f;
        if (c + 3 >= t.c) v.w = 0.f;
    }
    return v;
}

__device__ __forceinline__ float4 mask_channels(float4 v, int c, int nc) {
    if (c + 3 >= nc) {
        if (c + 0 >= nc) v.x = 0.f;
        if (c + 1 >= nc) v.y = 0.f;
        if (c + 2 >= nc) v.z = 0.f;
        if (c + 3 >= nc) v.w = 0.f;
    }
    return v;
}

__device__ __forceinline__ float func1(float x, int fn, int op, float operand) {
    switch (fn) {
        case FFN_SIGMOID: return __frcp_rn(1.0f + __expf(-x));
        case FFN_TANH: return 1.0f - 2.0f * __frcp_rn(1.0f + __expf(2.0f * x));   // = 2 e^{2x}/(1+e^{2x}) - 1 without the inf/inf of large x
        case FFN_ARITH: return op == 0 ? x + operand : op == 1 ? x - operand : op == 2 ? x * operand : x / operand;
        case FFN_CAST: {
            if (op == 7) return x;
            if (op == 6) return (float)(_Float16)x;
            const float r = rintf(x);   // ties to even
            switch (op) {
                case 0: return fminf(fmaxf(r, -2147483648.0f), 2147483647.0f);
                case 1: return fminf(fmaxf(r, -32768.0f), 32767.0f);
                case 2: return fminf(fmaxf(r, -128.0f), 127.0f);
                case 3: return fminf(fmaxf(r, 0.0f), 4294967295.0f);
                case 4: return fminf(fmaxf(r, 0.0f), 65535.0f);
                default: return fminf(fmaxf(r, 0.0f), 255.0f);
            }
        }
        default: return x;
    }
}

// Texel of V channels at stored coordinates, edge repeated beyond the stored tensor; channels >= in.c read as zero.
template <typename T, int V>
__device__ __forceinline__ FV<V> fetch_clamped_v(const TView& t, int sy, int sx, int c) {
    sy = min(max(sy, 0), t.hp() - 1);
    sx = min(max(sx, 0), t.wp() - 1);
    FV<V> v = ldv<T, V>(reinterpret_cast<const T*>(t.ptr) + ((size_t)sy * t.wp() + sx) * t.cp + c);
    if (c + V > t.c) {
#pragma unroll
        for (int i = 0; i < V; i++)
            if (c + i >= t.c) v.v[i] = 0.f;
    }
    return v;
}

template <typename T, int V>
__global__ __launch_bounds__(256) void func_kernel(const FuncParams p) {
    const int cg = p.out.cp / V;
    const size_t n = (size_t)p.out.h * p.out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % p.out.w), y = (int)(pix / p.out.w);
    int sy, sx, sc = g * V;   // source texel and first source channel
    if (p.map == FMAP_TRANSPOSE) {
        sy = x;
        sx = y;
    } else if (p.map == FMAP_IMGEXTRACT) {   // (always launched 4 channels wide: the groups of the reference are texels)
        const int b = g / p.in_groups;
        sc = (g - b * p.in_groups) * 4;
        sy = y * p.window + b / p.window;
        sx = x * p.window + b % p.window;
    } else {
        sy = floordiv_pos((2 * y + 1) * p.dy - p.oy, 2 * p.uy);
        sx = floordiv_pos((2 * x + 1) * p.dx - p.ox, 2 * p.ux);
    }
    FV<V> v = zerov<V>();
    if (sc < p.in.cp) v = fetch_clamped_v<T, V>(p.in, sy + p.in.pad, sx + p.in.pad, sc);
    if (p.fn == FFN_BGR) {
#pragma unroll
        for (int q = 0; q < V / 4; q++) {
            const float t = v.v[4 * q];
            v.v[4 * q] = v.v[4 * q + 2];
            v.v[4 * q + 2] = t;
        }
    } else {
        v = actv<V>(v, p.act);
        if (p.fn != FFN_COPY) {
#pragma unroll
            for (int i = 0; i < V; i++) v.v[i] = func1(v.v[i], p.fn, p.op, p.operand);
        }
    }
    const int c = g * V;
    if (c + V > p.out.c) {
#pragma unroll
        for (int i = 0; i < V; i++)
            if (c + i >= p.out.c) v.v[i] = 0.f;
    }
    stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, v);
}
// Scaling up by two (nearest): a thread owns a block of 2 x 2 output pixels and V channels.  The four source texels
// come from the same rule as above; where they coincide -- everywhere but at most at the frame's edges, by the
// offsets -- the texel is fetched and converted once and stored four times, instead of four threads fetching it.
template <typename T, int V>
__global__ __launch_bounds__(256) void func_up2_kernel(const FuncParams p) {
    const int cg = p.out.cp / V;
    const int bw = (p.out.w + 1) >> 1, bh = (p.out.h + 1) >> 1;
    const size_t n = (size_t)bh * bw * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t blk = idx / cg;
    const int x0 = 2 * (int)(blk % bw), y0 = 2 * (int)(blk / bw);
    const int c = g * V;
    int sy[2], sx[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        sy[i] = floordiv_pos((2 * (y0 + i) + 1) * p.dy - p.oy, 2 * p.uy);
        sx[i] = floordiv_pos((2 * (x0 + i) + 1) * p.dx - p.ox, 2 * p.ux);
    }
    FV<V> v[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (i == 1 && sy[1] == sy[0]) { v[1][j] = v[0][j]; continue; }
            if (j == 1 && sx[1] == sx[0]) { v[i][1] = v[i][0]; continue; }
            FV<V> t = zerov<V>();
            if (c < p.in.cp) t = fetch_clamped_v<T, V>(p.in, sy[i] + p.in.pad, sx[j] + p.in.pad, c);
            t = actv<V>(t, p.act);
            if (p.fn != FFN_COPY) {
#pragma unroll
                for (int e = 0; e < V; e++) t.v[e] = func1(t.v[e], p.fn, p.op, p.operand);
            }
            if (c + V > p.out.c) {
#pragma unroll
                for (int e = 0; e < V; e++)
                    if (c + e >= p.out.c) t.v[e] = 0.f;
            }
            v[i][j] = t;
        }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
            if (y0 + i < p.out.h && x0 + j < p.out.w) stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y0 + i, x0 + j) + c, v[i][j]);
}
// The same size in and out (the scaling map's steps equal and its offsets inside a texel): output texel (y, x) reads
// source texel (y, x).  One grid row per image row and 32-bit indices inside it, so that a thread's index arithmetic is
// a shift or one short division -- in func_kernel it is most of the instructions of a thread that moves 16 bytes in
// and 16 out, and holds a transcendental function like the sigmoid under the memory's speed.
template <typename T, int V>
__global__ __launch_bounds__(256) void func_same_kernel(const FuncParams p, int cg_shift) {
    const int cg = p.out.cp / V;
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= (unsigned)(p.out.w * cg)) return;
    const int y = blockIdx.y;
    const int x = cg_shift >= 0 ? (int)(i >> cg_shift) : (int)(i / (unsigned)cg);
    const int c = ((int)i - x * cg) * V;
    FV<V> v = zerov<V>();
    if (c < p.in.cp) v = fetch_clamped_v<T, V>(p.in, y + p.in.pad, x + p.in.pad, c);
    v = actv<V>(v, p.act);
    if (p.fn != FFN_COPY) {
#pragma unroll
        for (int e = 0; e < V; e++) v.v[e] = func1(v.v[e], p.fn, p.op, p.operand);
    }
    if (c + V > p.out.c) {
#pragma unroll
        for (int e = 0; e < V; e++)
            if (c + e >= p.out.c) v.v[e] = 0.f;
    }
    stv<T, V>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, v);
}
void launch_func(const FuncParams& p, hipStream_t s) {
    if (p.map == FMAP_SCALE && p.fn != FFN_BGR && p.dx == p.ux && p.dy == p.uy && p.ox > -p.ux && p.ox <= p.ux && p.oy > -p.uy && p.oy <= p.uy &&
        p.out.h <= 65535 && (long long)p.out.w * p.out.cp < (1ll << 30)) {
        const bool wide = (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0);
        const int cg = p.out.cp / ((p.out.f16 && wide) ? 8 : 4);
        int shift = -1;
        for (int b = 0; b < 16; b++)
            if ((1 << b) == cg) shift = b;
        const dim3 grid((unsigned)(((size_t)p.out.w * cg + 255) / 256), (unsigned)p.out.h);
        FYN_DISPATCH_TV(p.out.f16, wide, func_same_kernel, grid, dim3(256), s, p, shift);
        return;
    }
    if (p.map == FMAP_SCALE && p.ux == 2 && p.uy == 2 && p.dx == 1 && p.dy == 1 && p.fn != FFN_BGR) {
        const bool wide2 = (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0);
        const size_t n2 = (size_t)((p.out.h + 1) / 2) * ((p.out.w + 1) / 2) * (p.out.cp / ((p.out.f16 && wide2) ? 8 : 4));
        FYN_DISPATCH_TV(p.out.f16, wide2, func_up2_kernel, grid1d(n2, 256), dim3(256), s, p);
        return;
    }
    const bool wide = p.map != FMAP_IMGEXTRACT && (p.in.cp % 8 == 0) && (p.out.cp % 8 == 0);
    const size_t n = (size_t)p.out.h * p.out.w * (p.out.cp / ((p.out.f16 && wide) ? 8 : 4));
    FYN_DISPATCH_TV(p.out.f16, wide, func_kernel, grid1d(n, 256), dim3(256), s, p);
}

// Bilinear scaling: the raw texels around position ((2x+1)*dx - ox)/(2*ux) - 1/2 are blended, then activated.
template <typename T>
__global__ __launch_bounds__(256) void scale_linear_kernel(const FuncParams p) {
    const int cg = p.out.cp >> 2;
    const size_t n = (size_t)p.out.h * p.out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % p.out.w), y = (int)(pix / p.out.w);
    const int ny = (2 * y + 1) * p.dy - p.oy - p.uy, nx = (2 * x + 1) * p.dx - p.ox - p.ux;
    const int y0 = floordiv_pos(ny, 2 * p.uy), x0 = floordiv_pos(nx, 2 * p.ux);
    const float fy = (float)(ny - y0 * 2 * p.uy) / (float)(2 * p.uy), fx = (float)(nx - x0 * 2 * p.ux) / (float)(2 * p.ux);
    const int c = g * 4, sy = y0 + p.in.pad, sx = x0 + p.in.pad;
    const float4 a = fetch_clamped<T>(p.in, sy, sx, c), b = fetch_clamped<T>(p.in, sy, sx + 1, c);
    const float4 cc = fetch_clamped<T>(p.in, sy + 1, sx, c), d = fetch_clamped<T>(p.in, sy + 1, sx + 1, c);
    const float w00 = (1.f - fy) * (1.f - fx), w01 = (1.f - fy) * fx, w10 = fy * (1.f - fx), w11 = fy * fx;
    float4 v = make_float4(w00 * a.x + w01 * b.x + w10 * cc.x + w11 * d.x, w00 * a.y + w01 * b.y + w10 * cc.y + w11 * d.y,
                           w00 * a.z + w01 * b.z + w10 * cc.z + w11 * d.z, w00 * a.w + w01 * b.w + w10 * cc.w + w11 * d.w);
    v = act4(v, p.act);
    st4<T>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, mask_channels(v, c, p.out.c));
}
void launch_scale_linear(const FuncParams& p, hipStream_t s) {
    const size_t n = (size_t)p.out.h * p.out.w * (p.out.cp >> 2);
    FYN_DISPATCH_T(p.out.f16, scale_linear_kernel, grid1d(n, 256), dim3(256), s, p);
}

template <typename T>
__global__ __launch_bounds__(256) void nonmax_kernel(const TView in, const TView out) {
    const int cg = out.cp >> 2;
    const size_t n = (size_t)out.h * out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % out.w), y = (int)(pix / out.w);
    const int c = g * 4, sy = y + in.pad, sx = x + in.pad;
    const float4 m = fetch_clamped<T>(in, sy, sx, c);
    const float4 r = fetch_clamped<T>(in, sy, sx + 1, c), l = fetch_clamped<T>(in, sy, sx - 1, c);
    const float4 t = fetch_clamped<T>(in, sy - 1, sx, c), b = fetch_clamped<T>(in, sy + 1, sx, c);
    float4 v;
    v.x = (m.x >= r.x && m.x >= l.x && m.x >= t.x && m.x >= b.x && m.x > 0.1f) ? m.x : 0.f;
    v.y = (m.y >= r.y && m.y >= l.y && m.y >= t.y && m.y >= b.y && m.y > 0.1f) ? m.y : 0.f;
    v.z = (m.z >= r.z && m.z >= l.z && m.z >= t.z && m.z >= b.z && m.z > 0.1f) ? m.z : 0.f;
    v.w = (m.w >= r.w && m.w >= l.w && m.w >= t.w && m.w >= b.w && m.w > 0.1f) ? m.w : 0.f;
    st4<T>(reinterpret_cast<T*>(out.ptr) + tv_off(out, y, x) + c, v);
}
void launch_nonmax(const TView& in, const TView& out, hipStream_t s) {
    const size_t n = (size_t)out.h * out.w * (out.cp >> 2);
    FYN_DISPATCH_T(out.f16, nonmax_kernel, grid1d(n, 256), dim3(256), s, in, out);
}

template <typename T>
__global__ __launch_bounds__(256) void blur_kernel(const TView in, const TView out, const float* __restrict__ coef, int r, int last) {
    const int cg = out.cp >> 2;
    const size_t n = (size_t)out.h * out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % out.w), y = (int)(pix / out.w);
    const int c = g * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    int kidx = 0;
    for (int oy = -r; oy <= last; oy++)
        for (int ox = -r; ox <= last; ox++) {
            const float w = coef[kidx++];
            const float4 v = fetch_clamped<T>(in, y + in.pad + oy, x + in.pad + ox, c);
            acc.x = fmaf(w, v.x, acc.x); acc.y = fmaf(w, v.y, acc.y);
            acc.z = fmaf(w, v.z, acc.z); acc.w = fmaf(w, v.w, acc.w);
        }
    st4<T>(reinterpret_cast<T*>(out.ptr) + tv_off(out, y, x) + c, acc);
}
void launch_blur(const TView& in, const TView& out, const float* coef, int r, int last, hipStream_t s) {
    const size_t n = (size_t)out.h * out.w * (out.cp >> 2);
    FYN_DISPATCH_T(out.f16, blur_kernel, grid1d(n, 256), dim3(256), s, in, out, coef, r, last);
}

template <typename T, int V>
__global__ __launch_bounds__(256) void addsub_kernel(const TView a, const TView b, const TView out, int sub, const Act act) {
    const int cg = out.cp / V;
    const PixelIndex pi = pixel_index(out.h, out.w, cg);
    if (!pi.inside) return;
    const int g = pi.g, x = pi.x, y = pi.y;
    const int c = g * V;
    const FV<V> u = actv<V>(ldv<T, V>(reinterpret_cast<const T*>(a.ptr) + tv_off(a, y, x) + c), act);
    const FV<V> v = actv<V>(ldv<T, V>(reinterpret_cast<const T*>(b.ptr) + tv_off(b, y, x) + c), act);
    FV<V> o;
#pragma unroll
    for (int i = 0; i < V; i++) o.v[i] = sub ? u.v[i] - v.v[i] : u.v[i] + v.v[i];
    stv<T, V>(reinterpret_cast<T*>(out.ptr) + tv_off(out, y, x) + c, o);
}
void launch_addsub(const TView& a, const TView& b, const TView& out, int sub, const Act& act, hipStream_t s) {
    const bool wide = (a.cp % 8 == 0) && (b.cp % 8 == 0) && (out.cp % 8 == 0);
    FYN_DISPATCH_TV(out.f16, wide, addsub_kernel, grid_rows(out.h, out.w, out.cp / ((out.f16 && wide) ? 8 : 4)), dim3(256), s, a, b, out, sub, act);
}

// Channel offsets that are not multiples of the vector width (the "component shift" case of deepconcat.frag) are
// handled per element; aligned offsets move whole vectors.
template <typename T, int V>
__global__ __launch_bounds__(256) void concat_kernel(const TView in, const TView out, int c_off, const Act act, int zero_to) {
    const int cg = (in.c + V - 1) / V;
    const PixelIndex pi = pixel_index(out.h, out.w, cg);
    if (!pi.inside) return;
    const int g = pi.g, x = pi.x, y = pi.y;
    const int c = g * V;
    const T* src = reinterpret_cast<const T*>(in.ptr) + tv_off(in, y, x) + c;
    T* dst = reinterpret_cast<T*>(out.ptr) + tv_off(out, y, x) + c_off + c;
    if ((c_off % V) == 0 && c + V <= in.c) {
        stv<T, V>(dst, actv<V>(ldv<T, V>(src), act));
    } else {
        for (int i = 0; i < V && c + i < in.c; i++) dst[i] = (T)act1((float)src[i], act);
    }
    // last part: the pad lanes behind the last real channel are written as zero (the buffer may have held another tensor)
    if (g == cg - 1) {
        T* px = reinterpret_cast<T*>(out.ptr) + tv_off(out, y, x);
        for (int i = c_off + in.c; i < zero_to; i++) px[i] = (T)0.f;
    }
}
void launch_concat_part(const TView& in, const TView& out, int c_off, const Act& act, hipStream_t s, bool last) {
    const bool wide = (in.cp % 8 == 0) && (out.cp % 8 == 0);
    const int v = (out.f16 && wide) ? 8 : 4;
    FYN_DISPATCH_TV(out.f16, wide, concat_kernel, grid_rows(out.h, out.w, (in.c + v - 1) / v), dim3(256), s, in, out, c_off, act, last ? out.cp : 0);
}

// ---------------------------------------------------------------------------------------------
// exact arg-max over channels, lowest index among maxima (replaces the mantissa-bit approximation of
// DeepArgMaxLayer::forward, gpu/deep/deepargmaxlayer.cpp:113-152).  L lanes cooperate on one pixel and
// merge with cross-lane shuffles (DPP / ds_swizzle on gfx950).
// ---------------------------------------------------------------------------------------------
// One (value, index) pair per lane; the better of two: larger value, lower index among equals.
__device__ __forceinline__ void argmax_merge(float& best, int& bidx, float ob, int oi) {
    if (ob > best || (ob == best && oi < bidx)) {
        best = ob;
        bidx = oi;
    }
}
// The pair of the lane that the data-parallel path CTRL pairs this lane with (quad permutations and the mirrors of a row
// of 16 lanes: after xor 1, xor 2, half-row mirror and row mirror every lane of a row holds the row's result).
template <int CTRL>
__device__ __forceinline__ void argmax_dpp_step(float& best, int& bidx) {
    const float ob = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(best), CTRL, 0xf, 0xf, false));
    const int oi = __builtin_amdgcn_update_dpp(0, bidx, CTRL, 0xf, 0xf, false);
    argmax_merge(best, bidx, ob, oi);
}
// V channels per load (16 bytes of an fp16 tensor, 4 channels otherwise), L = 2^l_log2 lanes per pixel, R pixels per
// lane group with all their loads in flight before the first comparison.
template <typename T, int V, int R>
__global__ __launch_bounds__(256) void argmax_kernel(const TView in, const TView out, int32_t* idx_out, const Act act,
                                                     int l_log2) {
    const int L = 1 << l_log2;
    const int lane = threadIdx.x & 63;
    const int sub = lane & (L - 1);
    const int ppw = 64 >> l_log2;  // lane groups per wave
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const size_t pix0 = (wave * ppw + (lane >> l_log2)) * R;
    const size_t npix = (size_t)in.h * in.w;
    const int cgs = (in.c + V - 1) / V;   // (channels beyond in.c inside the last group are masked below; the pitch covers them)
    const T* src[R];
    bool valid[R];
    float best[R];
    int bidx[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        valid[r] = pix0 + r < npix;
        const size_t pix = valid[r] ? pix0 + r : 0;
        // (a tensor without a halo is one run of pixels: no row arithmetic)
        src[r] = reinterpret_cast<const T*>(in.ptr) + (in.pad == 0 ? pix * in.cp : tv_off(in, (int)(pix / in.w), (int)(pix % in.w)));
        best[r] = -INFINITY;
        bidx[r] = 0x7fffffff;
    }
    for (int g0 = sub; g0 < cgs; g0 += 2 * L) {   // two groups of every pixel per trip: loads first, then the scan in channel order
        FV<V> v[R][2];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < 2; j++) v[r][j] = ldv<T, V>(src[r] + (g0 + j * L < cgs ? g0 + j * L : g0) * V);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int g = g0 + j * L;
                if (g >= cgs) break;
                const FV<V> a = actv<V>(v[r][j], act);
                // (a lane meets its channels in rising order: a later equal value never replaces the first)
                if (g * V + V <= in.c) {
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        const bool up = a.v[i] > best[r];
                        best[r] = up ? a.v[i] : best[r];
                        bidx[r] = up ? g * V + i : bidx[r];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        const int c = g * V + i;
                        if (c < in.c && a.v[i] > best[r]) {
                            best[r] = a.v[i];
                            bidx[r] = c;
                        }
                    }
                }
            }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (L >= 2) argmax_dpp_step<0xB1>(best[r], bidx[r]);    // quad_perm [1,0,3,2]
        if (L >= 4) argmax_dpp_step<0x4E>(best[r], bidx[r]);    // quad_perm [2,3,0,1]
        if (L >= 8) argmax_dpp_step<0x141>(best[r], bidx[r]);   // row_half_mirror
        if (L >= 16) argmax_dpp_step<0x140>(best[r], bidx[r]);  // row_mirror
        if (L >= 32) {   // across rows of 16: swizzle inside a half wave (xor 16), then across the halves
            const float ob = __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(best[r]), 0x401f));
            const int oi = __builtin_amdgcn_ds_swizzle(bidx[r], 0x401f);
            argmax_merge(best[r], bidx[r], ob, oi);
        }
        if (L >= 64) argmax_merge(best[r], bidx[r], __shfl_xor(best[r], 32, 64), __shfl_xor(bidx[r], 32, 64));
        if (valid[r] && sub == 0) {
            const size_t pix = pix0 + r;
            T* dst = reinterpret_cast<T*>(out.ptr) + (out.pad == 0 ? pix * out.cp : tv_off(out, (int)(pix / in.w), (int)(pix % in.w)));
            st4<T>(dst, make_float4((float)bidx[r], best[r], 0.f, 0.f));
            if (idx_out) idx_out[pix] = bidx[r];
        }
    }
}
void launch_argmax(const TView& in, const TView& out, int32_t* idx_out, const Act& act, hipStream_t s) {
    const bool wide = in.f16 && in.cp % 8 == 0;
    const int v = wide ? 8 : 4;
    const int cgs = (in.c + v - 1) / v;
    int l2 = 0;
    while ((1 << l2) < cgs && l2 < 6) l2++;
    const size_t npix = (size_t)in.h * in.w;
    const size_t ppw = 64 >> l2;
    // four pixels per lane group where that still leaves every SIMD of the chip a few waves
    const bool many = npix / (ppw * 4) >= 4096;
    const size_t waves = (npix + ppw * (many ? 4 : 1) - 1) / (ppw * (many ? 4 : 1));
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (wide) {
        if (many) hipLaunchKernelGGL((argmax_kernel<_Float16, 8, 4>), grid, block, 0, s, in, out, idx_out, act, l2);
        else hipLaunchKernelGGL((argmax_kernel<_Float16, 8, 1>), grid, block, 0, s, in, out, idx_out, act, l2);
    } else if (in.f16) {
        if (many) hipLaunchKernelGGL((argmax_kernel<_Float16, 4, 4>), grid, block, 0, s, in, out, idx_out, act, l2);
        else hipLaunchKernelGGL((argmax_kernel<_Float16, 4, 1>), grid, block, 0, s, in, out, idx_out, act, l2);
    } else {
        if (many) hipLaunchKernelGGL((argmax_kernel<float, 4, 4>), grid, block, 0, s, in, out, idx_out, act, l2);
        else hipLaunchKernelGGL((argmax_kernel<float, 4, 1>), grid, block, 0, s, in, out, idx_out, act, l2);
    }
}

// ---------------------------------------------------------------------------------------------
// fully connected layer as a matrix-vector product (DeepGEMMLayer::forward,
// gpu/deep/deepgemmlayer.cpp:66-236): one wavefront per output row, the row of weights is streamed
// once from HBM in 16-byte pieces, partial sums meet on the DPP paths.
// ---------------------------------------------------------------------------------------------
// Sum of a wave's 64 values on the vector ALUs' data-parallel paths (prefix sums inside rows of 16 lanes, then the row
// sums carried into the following rows); every lane gets the total.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x111, 0xf, 0xf, false));   // row_shr:1
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x112, 0xf, 0xf, false));   // row_shr:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x114, 0xf, 0xf, false));   // row_shr:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x118, 0xf, 0xf, false));   // row_shr:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));   // row_bcast:15 into rows 1, 3
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xc, 0xf, false));   // row_bcast:31 into rows 2, 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

template <typename T, typename TW>
__global__ __launch_bounds__(256) void gemv_kernel(const GemvParams p) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.out.cp) return;
    const int cinp = p.in.cp;
    const T* x = reinterpret_cast<const T*>(p.in.ptr) + tv_off(p.in, 0, 0);
    const TW* w = reinterpret_cast<const TW*>(p.w) + (size_t)row * cinp;
    float acc = 0.f;
    if (row < p.out.c) {
        // eight 16-byte pieces of the row per trip (a row of 2048 fp32 weights in one): every load of a trip is on its
        // way before the first multiply-add, so the wave pays the memory latency once per trip
        constexpr int NP = 8;
        for (int c0 = lane * 4; c0 < cinp; c0 += NP * 256) {
            float4 xv[NP], wv[NP];
#pragma unroll
            for (int j = 0; j < NP; j++) {
                const int c = c0 + j * 256 < cinp ? c0 + j * 256 : c0;
                wv[j] = ld4<TW>(w + c);
            }
#pragma unroll
            for (int j = 0; j < NP; j++) {
                const int c = c0 + j * 256 < cinp ? c0 + j * 256 : c0;
                xv[j] = ld4<T>(x + c);
            }
#pragma unroll
            for (int j = 0; j < NP; j++) {
                if (c0 + j * 256 >= cinp) break;
                const float4 a = act4(xv[j], p.act);
                acc = fmaf(a.x, wv[j].x, acc); acc = fmaf(a.y, wv[j].y, acc);
                acc = fmaf(a.z, wv[j].z, acc); acc = fmaf(a.w, wv[j].w, acc);
            }
        }
    }
    acc = wave_sum_dpp(acc);
    if (lane == 0) {
        float r = (row < p.out.c) ? acc * p.scale[row] + p.bias[row] : 0.f;
        reinterpret_cast<T*>(p.out.ptr)[tv_off(p.out, 0, 0) + row] = (T)r;
    }
}
void launch_gemv(const GemvParams& p, hipStream_t s) {
    dim3 grid((p.out.cp + 3) / 4), block(256);
    if (p.out.f16) {
        if (p.w_f16) hipLaunchKernelGGL((gemv_kernel<_Float16, _Float16>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((gemv_kernel<_Float16, float>), grid, block, 0, s, p);
    } else {
        if (p.w_f16) hipLaunchKernelGGL((gemv_kernel<float, _Float16>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((gemv_kernel<float, float>), grid, block, 0, s, p);
    }
}

// ---------------------------------------------------------------------------------------------
// The same product on the matrix cores (v_mfma_f32_16x16x32_f16, fp32 accumulate).  A workgroup owns 16 output rows;
// its four waves take a quarter of the reduction each, in steps of 32 input channels: the A operand is the 16 x 32
// block of weights (lane = row, eight consecutive channels; fp16 weights as they lie in memory, fp32 weights from a
// copy packed at weight load as [row][group of 8 channels][8 x fp16 hi | 8 x fp16 lo], the same four bytes per weight,
// so that the matrix is streamed once as in gemv_kernel and nothing is converted on the way), the B
// operand the input vector's 32 values in every one of the 16 columns (staged once per workgroup in LDS as fp16, with
// fp32 tensors as hi and lo planes scaled by a power of two that puts the largest value at 2^14), so all columns of
// the result are equal and column 0 is taken.  fp32 tensors: hi*hi + lo*hi + hi*lo, 22 significant bits per operand.
// The four partial sums meet in LDS in a fixed order.  With one right-hand side 15 of the 16 columns are idle; what
// the kernel is bound by is the weight stream, like gemv_kernel.
// ---------------------------------------------------------------------------------------------
typedef float fc_f32x4 __attribute__((ext_vector_type(4)));
constexpr int FC_TRIP = 8;   // steps whose weight loads are in flight together (two such sets: one is converted while the next arrives)

template <typename T>
struct FcRaw;
template <>
struct FcRaw<float> { half8_t a, b; };   // hi and lo halves of eight weights
template <>
struct FcRaw<_Float16> { half8_t a; };

// R: output rows per workgroup, 16 or -- for matrices of few rows, so that every CU of the chip pulls a share of the
// stream -- 4 (the fragment's rows then repeat those four; lanes that ask for the same bytes cost no traffic).
template <typename T, int R>
__global__ __launch_bounds__(256) void fc_mfma_kernel(const GemvParams p) {
    constexpr bool F32 = sizeof(T) == 4;
    extern __shared__ __align__(16) unsigned char fc_lds[];   // x hi [kpad] halves, then (fp32 tensors) x lo [kpad] halves
    __shared__ float part[4][16];
    __shared__ float wmax[4];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mq = lane & 15, kq = lane >> 4;
    const int cinp = p.in.cp;
    const int nsteps = (cinp + 31) >> 5, kpad = nsteps * 32;
    const int per = (nsteps + 3) >> 2;
    const int s0 = wave * per, s1 = min(nsteps, s0 + per);
    const int row0 = blockIdx.x * R;
    const int wrow = min(row0 + (mq & (R - 1)), p.out.cp - 1);   // (the matrix has out.cp rows; fragment rows behind them repeat the last and are not stored)
    // (fp32 tensors: p.w_split, 16 halves per group of 8 weights)
    const _Float16* w = F32 ? reinterpret_cast<const _Float16*>(p.w_split) + ((size_t)wrow * cinp + kq * 8) * 2
                            : reinterpret_cast<const _Float16*>(p.w) + (size_t)wrow * cinp + kq * 8;
    auto load_trip = [&](FcRaw<T> (&raw)[FC_TRIP], int first) {
#pragma unroll
        for (int j = 0; j < FC_TRIP; j++) {
            const int s = first + j;
            const bool ok = s < s1 && s * 32 + kq * 8 < cinp;
            const _Float16* src = w + (ok ? s * 32 * (F32 ? 2 : 1) : 0);
            raw[j].a = *reinterpret_cast<const half8_t*>(src);
            if (!ok) raw[j].a = (half8_t)((_Float16)0.f);
            if constexpr (F32) {
                raw[j].b = *reinterpret_cast<const half8_t*>(src + 8);
                if (!ok) raw[j].b = (half8_t)((_Float16)0.f);
            }
        }
    };
    // the input vector's loads first (the counters retire loads in order: waiting for these must not wait for the weights),
    // unconditional, from a clamped address
    const T* x = reinterpret_cast<const T*>(p.in.ptr) + tv_off(p.in, 0, 0);
    constexpr int XG = 8;   // groups of 8 values per thread: up to 16384 inputs
    float4 x0[XG], x1[XG];
#pragma unroll
    for (int g = 0; g < XG; g++) {
        const int c = (tid + g * 256) * 8;
        if (g * 2048 < cinp) {   // (uniform)
            const int cc = min(c, cinp - 8);
            x0[g] = ld4<T>(x + cc);
            x1[g] = ld4<T>(x + cc + 4);
        } else {
            x0[g] = x1[g] = float4{0.f, 0.f, 0.f, 0.f};
        }
    }
    FcRaw<T> ra[FC_TRIP], rb[FC_TRIP];
    // (the weights do not depend on the vector: both sets of loads go out ahead of its staging, so that a reduction of up
    // to 2048 channels pays the memory's latency once)
    load_trip(ra, s0);
    load_trip(rb, s0 + FC_TRIP);

    // the input vector: activation, scale, fp16 planes
    float xv[XG][8];
    float amax = 0.f;
#pragma unroll
    for (int g = 0; g < XG; g++) {
        const int c = (tid + g * 256) * 8;
        const bool in = c < cinp;
        const float4 v0 = act4(x0[g], p.act), v1 = act4(x1[g], p.act);
        xv[g][0] = in ? v0.x : 0.f; xv[g][1] = in ? v0.y : 0.f; xv[g][2] = in ? v0.z : 0.f; xv[g][3] = in ? v0.w : 0.f;
        xv[g][4] = in ? v1.x : 0.f; xv[g][5] = in ? v1.y : 0.f; xv[g][6] = in ? v1.z : 0.f; xv[g][7] = in ? v1.w : 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(xv[g][e]));
    }
    float mul = 1.f, inv = 1.f;
    if constexpr (F32) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
        if (lane == 0) wmax[wave] = amax;
        __syncthreads();
        amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
        // a power of two that takes the largest value to [2^14, 2^15): no overflow in fp16, and the lo halves stay normal
        int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127;
        if (amax > 0.f && e > -100 && e < 128) {
            mul = __uint_as_float((unsigned)(127 + 14 - e) << 23);
            inv = __uint_as_float((unsigned)(127 - 14 + e) << 23);
        }
    }
#pragma unroll
    for (int g = 0; g < XG; g++) {
        const int c = (tid + g * 256) * 8;
        if (c < kpad) {
            half8_t hi, lo;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = xv[g][e] * mul;
                hi[e] = (_Float16)v;
                lo[e] = (_Float16)(v - (float)hi[e]);
            }
            *reinterpret_cast<half8_t*>(fc_lds + (size_t)c * 2) = hi;
            if constexpr (F32) *reinterpret_cast<half8_t*>(fc_lds + (size_t)(kpad + c) * 2) = lo;
        }
    }
    __syncthreads();

    fc_f32x4 acc = (fc_f32x4)(0.f), acc1 = (fc_f32x4)(0.f), acc2 = (fc_f32x4)(0.f);   // (one chain per pass: no MFMA waits for the one before it)
    auto run_trip = [&](const FcRaw<T> (&raw)[FC_TRIP], int first) {
#pragma unroll
        for (int j = 0; j < FC_TRIP; j++) {
            const int s = first + j;
            if (s >= s1) break;
            const half8_t bh = *reinterpret_cast<const half8_t*>(fc_lds + (size_t)(s * 32 + kq * 8) * 2);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(raw[j].a, bh, acc, 0, 0, 0);
            if constexpr (F32) {
                const half8_t bl = *reinterpret_cast<const half8_t*>(fc_lds + (size_t)(kpad + s * 32 + kq * 8) * 2);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(raw[j].b, bh, acc1, 0, 0, 0);
                acc2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(raw[j].a, bl, acc2, 0, 0, 0);
            }
        }
    };
    for (int t = s0; t < s1; t += 2 * FC_TRIP) {
        run_trip(ra, t);
        if (t + 2 * FC_TRIP < s1) load_trip(ra, t + 2 * FC_TRIP);
        if (t + FC_TRIP >= s1) break;
        run_trip(rb, t + FC_TRIP);
        if (t + 3 * FC_TRIP < s1) load_trip(rb, t + 3 * FC_TRIP);
    }
    // a lane of column 0 holds rows 4 * kq .. 4 * kq + 3
    if (mq == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) part[wave][kq * 4 + i] = acc[i] + (acc1[i] + acc2[i]);
    }
    __syncthreads();
    if (tid < R) {
        const int row = row0 + tid;
        if (row < p.out.cp) {
            const float sum = ((part[0][tid] + part[1][tid]) + part[2][tid]) + part[3][tid];
            const float r = (row < p.out.c) ? (sum * inv) * p.scale[row] + p.bias[row] : 0.f;
            reinterpret_cast<T*>(p.out.ptr)[tv_off(p.out, 0, 0) + row] = (T)r;
        }
    }
}
// fp16 tensors hold the vector and the matrix in fp16 already; fp32 weights must stay below fp16's range (the caller
// knows the matrix and checks: fc_mfma_supported says nothing about its values)
bool fc_mfma_supported(const GemvParams& p) {
    const int kpad = (p.in.cp + 31) / 32 * 32;
    return (p.out.f16 || p.w_split) && p.in.cp >= 32 && p.in.cp % 8 == 0 && (size_t)kpad * (p.out.f16 ? 2 : 4) <= 32768 && (p.w_f16 != 0) == (p.out.f16 != 0) && p.in.f16 == p.out.f16 && p.out.cp >= 1;
}
int launch_fc_mfma(const GemvParams& p, hipStream_t s) {
    if (!fc_mfma_supported(p)) return -1;
    const int kpad = (p.in.cp + 31) / 32 * 32;
    const bool few = (p.out.cp + 15) / 16 < 256;
    dim3 grid(few ? (p.out.cp + 3) / 4 : (p.out.cp + 15) / 16), block(256);
    const size_t lds = (size_t)kpad * (p.out.f16 ? 2 : 4);
    if (p.out.f16) {
        if (few) hipLaunchKernelGGL((fc_mfma_kernel<_Float16, 4>), grid, block, lds, s, p);
        else hipLaunchKernelGGL((fc_mfma_kernel<_Float16, 16>), grid, block, lds, s, p);
    } else {
        if (few) hipLaunchKernelGGL((fc_mfma_kernel<float, 4>), grid, block, lds, s, p);
        else hipLaunchKernelGGL((fc_mfma_kernel<float, 16>), grid, block, lds, s, p);
    }
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

// ---------------------------------------------------------------------------------------------
// direct convolution: the engine's second, plain implementation of the convolution family's sampling rules (zero halo,
// edge clamp of shallow layers, fractional steps), selected by FYNHIP_FORCE_DIRECT_CONV for cross-checks.
// fp32 FMA, one thread = one output pixel x 4 output channels.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void conv_direct_kernel(const ConvDirectParams p) {
    const int cg = p.out.cp >> 2;
    const size_t n = (size_t)p.out.h * p.out.w * cg;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int g = (int)(idx % cg);
    const size_t pix = idx / cg;
    const int x = (int)(pix % p.out.w), y = (int)(pix / p.out.w);
    const int c = g * 4;
    const T* in = reinterpret_cast<const T*>(p.in.ptr);
    const int iwp = p.in.wp(), ihp = p.in.hp();
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int ky = 0; ky < p.k; ky++) {
        for (int kx = 0; kx < p.k; kx++) {
            int sy = y * p.stride + p.in_y0 + ky * p.dil, sx = x * p.stride + p.in_x0 + kx * p.dil;
            if (p.frac_shift) {   // (an arithmetic shift: floor for negative numerators too)
                sy = p.in.pad + ((2 * (y * p.stride + ky + p.tap_y0) + 1) >> p.frac_shift);
                sx = p.in.pad + ((2 * (x * p.stride + kx + p.tap_x0) + 1) >> p.frac_shift);
            }
            bool ok = true;
            if (p.clamp) {
                sy = min(max(sy, 0), ihp - 1);
                sx = min(max(sx, 0), iwp - 1);
            } else {
                ok = (unsigned)sy < (unsigned)ihp && (unsigned)sx < (unsigned)iwp;
            }
            const T* src = in + ((size_t)sy * iwp + sx) * p.in.cp;
            const float* w = p.w + ((size_t)(ky * p.k + kx) * p.in.c) * p.out.cp + c;
            for (int ci = 0; ci < p.in.c; ci++) {
                const float v = act1(ok ? (float)src[ci] : 0.f, p.act);
                const float4 wv = *reinterpret_cast<const float4*>(w + (size_t)ci * p.out.cp);
                acc.x = fmaf(v, wv.x, acc.x); acc.y = fmaf(v, wv.y, acc.y);
                acc.z = fmaf(v, wv.z, acc.z); acc.w = fmaf(v, wv.w, acc.w);
            }
        }
    }
    const float4 sc = *reinterpret_cast<const float4*>(p.scale + c);
    const float4 bi = *reinterpret_cast<const float4*>(p.bias + c);
    float4 o = make_float4(acc.x * sc.x + bi.x, acc.y * sc.y + bi.y, acc.z * sc.z + bi.z, acc.w * sc.w + bi.w);
    if (p.res.ptr) {
        float4 r = ld4<T>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x) + c);
        if (p.res_relu) r = make_float4(fmaxf(r.x, 0.f), fmaxf(r.y, 0.f), fmaxf(r.z, 0.f), fmaxf(r.w, 0.f));
        if (p.res_scale) r = make_float4(r.x * sc.x, r.y * sc.y, r.z * sc.z, r.w * sc.w);
        o = make_float4(o.x + r.x, o.y + r.y, o.z + r.z, o.w + r.w);
    }
    st4<T>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x) + c, o);
}
void launch_conv_direct(const ConvDirectParams& p, hipStream_t s) {
    const size_t n = (size_t)p.out.h * p.out.w * (p.out.cp >> 2);
    FYN_DISPATCH_T(p.out.f16, conv_direct_kernel, grid1d(n, 256), dim3(256), s, p);
}

// ---------------------------------------------------------------------------------------------
// shift-reduce stage of the wide-kernel / few-output-channel convolution (see ShiftReduceParams):
// one thread per output pixel, the K neighbouring q pixels it reads are shared with its neighbours
// through L1/L2, so HBM sees q once.
// ---------------------------------------------------------------------------------------------
// A block takes 256 consecutive output pixels of one row: the 256+K-1 q pixels they need are one
// contiguous run in HBM, fetched once with 16-byte loads into LDS (row pitch cp+1 floats, so that the
// per-thread strided reads below fall into distinct banks), then every thread sums its K*cout values.
template <typename T>
__global__ __launch_bounds__(256) void shift_reduce_kernel(const ShiftReduceParams p) {
    extern __shared__ float sq[];
    const int tiles_x = (p.out.w + 255) / 256;
    const int y = blockIdx.x / tiles_x;
    const int x0 = (blockIdx.x - y * tiles_x) * 256;
    const int npx = min(256, p.out.w - x0) + p.k - 1;   // q pixels needed
    const int cp = p.q.cp, pitch = cp + 1;
    const T* q = reinterpret_cast<const T*>(p.q.ptr) + tv_off(p.q, y, x0);
    const int nvec = npx * (cp >> 2);
    for (int i = threadIdx.x; i < nvec; i += 256) {
        const float4 v = ld4<T>(q + (size_t)i * 4);
        const int px = i / (cp >> 2), c = (i - px * (cp >> 2)) * 4;
        float* d = sq + px * pitch + c;
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
    __syncthreads();
    const int x = x0 + threadIdx.x;
    float vmax = 0.f;
    if (x < p.out.w) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int kx = 0; kx < p.k; kx++) {
            const float* qp = sq + (threadIdx.x + kx) * pitch + kx;
#pragma unroll
            for (int o = 0; o < 4; o++)
                if (o < p.cout) acc[o] += qp[o * p.k];
        }
        float o4[4];
#pragma unroll
        for (int o = 0; o < 4; o++) o4[o] = (o < p.cout) ? (acc[o] * p.acc_mul) * p.scale[o] + p.bias[o] : 0.f;
        if (p.res.ptr) {
            float4 r = ld4<T>(reinterpret_cast<const T*>(p.res.ptr) + tv_off(p.res, y, x));
            float rv[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int o = 0; o < 4; o++) {
                if (o >= p.cout) continue;
                float v = rv[o];
                if (p.res_relu) v = fmaxf(v, 0.f);
                if (p.res_scale) v *= p.scale[o];
                o4[o] += v;
            }
        }
        st4<T>(reinterpret_cast<T*>(p.out.ptr) + tv_off(p.out, y, x), make_float4(o4[0], o4[1], o4[2], o4[3]));
        vmax = fmaxf(fmaxf(fabsf(o4[0]), fabsf(o4[1])), fmaxf(fabsf(o4[2]), fabsf(o4[3])));
    }
    if (p.out_amax) range_publish_block256(p.out_amax, vmax);   // (every thread takes part)
}
void launch_shift_reduce(const ShiftReduceParams& p, hipStream_t s) {
    const int tiles_x = (p.out.w + 255) / 256;
    const size_t lds = (size_t)(256 + p.k - 1) * (p.q.cp + 1) * sizeof(float);
    if (p.out.f16) hipLaunchKernelGGL((shift_reduce_kernel<_Float16>), dim3(tiles_x * p.out.h), dim3(256), lds, s, p);
    else hipLaunchKernelGGL((shift_reduce_kernel<float>), dim3(tiles_x * p.out.h), dim3(256), lds, s, p);
}

// ---------------------------------------------------------------------------------------------
// layout converters (UploadLayer / DownloadLayer / GPULayerBase::copyResult formats)
// ---------------------------------------------------------------------------------------------
// One thread converts four channels of one pixel; pixels are the fastest index, so that plane accesses are
// contiguous across a wavefront (image-like tensors of up to 4 channels are contiguous on the packed side too).
template <typename T>
__global__ __launch_bounds__(256) void chw_to_tensor_kernel(const float* chw, const TView t, unsigned* amax) {
    const size_t npix = (size_t)t.h * t.w;
    const size_t n = npix * (t.cp >> 2);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    float vmax = 0.f;
    if (idx < n) {
        const size_t pix = idx % npix;
        const int c = (int)(idx / npix) * 4;
        const int x = (int)(pix % t.w), y = (int)(pix / t.w);
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = c + i < t.c ? chw[(size_t)(c + i) * npix + pix] : 0.f;
            vmax = fmaxf(vmax, fabsf(v[i]));
        }
        st4<T>(reinterpret_cast<T*>(t.ptr) + tv_off(t, y, x) + c, make_float4(v[0], v[1], v[2], v[3]));
    }
    if (amax) range_publish_block256(amax, vmax);   // (every thread takes part)
}
void launch_chw_to_tensor(const float* chw, const TView& t, hipStream_t s, unsigned* amax) {
    FYN_DISPATCH_T(t.f16, chw_to_tensor_kernel, grid1d((size_t)t.h * t.w * (t.cp >> 2), 256), dim3(256), s, chw, t, amax);
}

template <typename T>
__global__ __launch_bounds__(256) void tensor_to_chw_kernel(const TView t, float* chw, int keep_pad) {
    const int oh = keep_pad ? t.hp() : t.h, ow = keep_pad ? t.wp() : t.w;
    const size_t npix = (size_t)oh * ow;
    const size_t n = npix * ((t.c + 3) >> 2);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const size_t pix = idx % npix;
    const int c = (int)(idx / npix) * 4;
    const int x = (int)(pix % ow), y = (int)(pix / ow);
    const int sy = keep_pad ? y : y + t.pad, sx = keep_pad ? x : x + t.pad;
    const float4 v = ld4<T>(reinterpret_cast<const T*>(t.ptr) + ((size_t)sy * t.wp() + sx) * t.cp + c);
    const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (c + i < t.c) chw[(size_t)(c + i) * npix + pix] = vv[i];
}
void launch_tensor_to_chw(const TView& t, float* chw, int include_padding, hipStream_t s) {
    const int oh = include_padding ? t.hp() : t.h, ow = include_padding ? t.wp() : t.w;
    FYN_DISPATCH_T(t.f16, tensor_to_chw_kernel, grid1d((size_t)oh * ow * ((t.c + 3) >> 2), 256), dim3(256), s, t, chw, include_padding);
}

template <typename T>
__global__ __launch_bounds__(256) void hwc_to_tensor_kernel(const float* hwc, int pc, const TView t, unsigned* amax) {
    const size_t n = (size_t)t.h * t.w * t.cp;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    float vmax = 0.f;
    if (idx < n) {
        const int c = (int)(idx % t.cp);
        const size_t pix = idx / t.cp;
        const int x = (int)(pix % t.w), y = (int)(pix / t.w);
        const float v = (c < t.c && c < pc) ? hwc[pix * pc + c] : 0.f;
        reinterpret_cast<T*>(t.ptr)[tv_off(t, y, x) + c] = (T)v;
        vmax = fabsf(v);
    }
    if (amax) range_publish_block256(amax, vmax);   // (every thread takes part)
}
void launch_hwc_to_tensor(const float* hwc, int pc, const TView& t, hipStream_t s, unsigned* amax) {
    FYN_DISPATCH_T(t.f16, hwc_to_tensor_kernel, grid1d((size_t)t.h * t.w * t.cp, 256), dim3(256), s, hwc, pc, t, amax);
}

template <typename T>
__global__ __launch_bounds__(256) void tensor_to_hwc_kernel(const TView t, float* hwc, int pc) {
    const size_t n = (size_t)t.h * t.w * pc;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int c = (int)(idx % pc);
    const size_t pix = idx / pc;
    const int x = (int)(pix % t.w), y = (int)(pix / t.w);
    hwc[idx] = c < t.c ? (float)reinterpret_cast<const T*>(t.ptr)[tv_off(t, y, x) + c] : 0.f;
}
void launch_tensor_to_hwc(const TView& t, float* hwc, int pc, hipStream_t s) {
    FYN_DISPATCH_T(t.f16, tensor_to_hwc_kernel, grid1d((size_t)t.h * t.w * pc, 256), dim3(256), s, t, hwc, pc);
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint4* p, size_t n16, unsigned char* tail, size_t ntail) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = idx; i < n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
    if (idx < ntail) tail[idx] = 0;
}
void launch_fill_zero(void* ptr, size_t bytes, hipStream_t s) {
    const size_t n16 = bytes / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, s, reinterpret_cast<uint4*>(ptr), n16,
                       reinterpret_cast<unsigned char*>(ptr) + n16 * 16, bytes - n16 * 16);
}

// Debugging aid: fills the LDS of every CU with all-ones words (a NaN as fp16 and as fp32, -1 as an integer).  The LDS
// keeps its contents from one kernel to the next, so a kernel that reads a location it never wrote shows it in its
// results when this ran just before it.  One workgroup takes a CU's whole LDS; there are several per CU, each busy long
// enough for the others to land elsewhere.
__global__ __launch_bounds__(256) void poison_lds_kernel(unsigned words) {
    extern __shared__ unsigned poison_words[];
    volatile unsigned* w = poison_words;
    for (unsigned i = threadIdx.x; i < words; i += 256) w[i] = 0xffffffffu;
}
int launch_poison_lds(hipStream_t s) {
    constexpr size_t bytes = 160 * 1024;
    if (ensure_lds(reinterpret_cast<const void*>(poison_lds_kernel), bytes) != 0) return -1;
    hipLaunchKernelGGL(poison_lds_kernel, dim3(1024), dim3(256), bytes, s, (unsigned)(bytes / 4));
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Second pass of a split-K convolution (see ConvMfmaParams::ksplit): one thread per (position, 4 channels).
template <typename TOut>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const SplitKReduceParams p) {
    const int cq = p.cout_pad >> 2;
    const size_t n = (size_t)p.npos_y * p.npos_x * cq;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int c = (int)(idx % cq) * 4;
    float vmax = 0.f;
    if (idx < n && c < p.out_cp) {
        const size_t pos = idx / cq;
        const int py = (int)(pos / p.npos_x), px = (int)(pos - (size_t)py * p.npos_x);
        const size_t slice = (size_t)p.npos_y * p.npos_x * p.cout_pad;
        // everything this thread reads is requested up front: residual, scale, bias and the first eight slices share
        // one memory round trip
        float rv[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.res) {
            const TOut* res = reinterpret_cast<const TOut*>(p.res);
            const size_t rbase = ((size_t)(p.res_off_y + py * p.out_step) * p.res_wp + p.res_off_x + px * p.out_step) * p.res_cp + c;
            const float4 r = ld4<TOut>(res + rbase);
            rv[0] = r.x; rv[1] = r.y; rv[2] = r.z; rv[3] = r.w;
        }
        const f32x4 sc = *reinterpret_cast<const f32x4*>(p.scale + c), bi = *reinterpret_cast<const f32x4*>(p.bias + c);
        // slices are summed in slice order; their loads are issued eight at a time (one round trip per eight slices)
        f32x4 a = (f32x4)(0.f);
        const float* src = p.partial + pos * p.cout_pad + c;
        for (int k0 = 0; k0 < p.ksplit; k0 += 8) {
            f32x4 v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = *reinterpret_cast<const f32x4*>(src + (size_t)(k0 + j < p.ksplit ? k0 + j : k0) * slice);
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (k0 + j < p.ksplit) a += v[j];
        }
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o[i] = (a[i] * p.acc_mul) * sc[i] + bi[i];
            if (p.res) {
                float r = rv[i];
                if (p.res_relu) r = fmaxf(r, 0.f);
                if (p.res_scale) r *= sc[i];
                o[i] += r;
            }
        }
        TOut* out = reinterpret_cast<TOut*>(p.out);
        const size_t obase = ((size_t)(p.out_off_y + py * p.out_step) * p.out_wp + p.out_off_x + px * p.out_step) * p.out_cp + c;
        st4<TOut>(out + obase, make_float4(o[0], o[1], o[2], o[3]));
        vmax = fmaxf(fmaxf(fabsf(o[0]), fabsf(o[1])), fmaxf(fabsf(o[2]), fabsf(o[3])));
    }
    if (p.out_amax) range_publish_block256(p.out_amax, vmax);   // (every thread takes part)
}

void launch_splitk_reduce(const SplitKReduceParams& p, hipStream_t s) {
    const size_t n = (size_t)p.npos_y * p.npos_x * (p.cout_pad >> 2);
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (p.out_f16) hipLaunchKernelGGL(splitk_reduce_kernel<_Float16>, dim3(blocks), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(splitk_reduce_kernel<float>, dim3(blocks), dim3(256), 0, s, p);
}

}  // namespace fynhip
