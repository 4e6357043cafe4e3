// What the 16-position-fragment convolution kernels (conv_p16.hip, conv_h16.hip) share: vector types, the LDS-only
// barrier, the activation, the staged pixel's pitch and the search for a bank-conflict-free row padding.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace fynhip {
namespace {
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Workgroup barrier that orders LDS traffic only (global loads and stores stay in flight across it).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ float act_p16(float x, const Act& a) { return __builtin_amdgcn_fmed3f(x, a.lo, a.hi) + a.leak * fminf(x, 0.f); }
// An activation that is exact on halves -- none, or a clamp without leak whose bounds are fp16 values -- is applied to
// the packed halves (two values per instruction, no conversions): act_half_exact says whether, act_half applies it.
__device__ __forceinline__ bool act_half_exact(const Act& a, _Float16& lo, _Float16& hi) {
    lo = (_Float16)fmaxf(a.lo, -65504.f);
    hi = (_Float16)fminf(a.hi, 65504.f);
    return a.leak == 0.f && (a.lo < -65504.f || (float)lo == a.lo) && (a.hi > 65504.f || (float)hi == a.hi);
}
__device__ __forceinline__ half8_t act_half(half8_t v, _Float16 lo, _Float16 hi) {
    return __builtin_elementwise_min(__builtin_elementwise_max(v, (half8_t)lo), (half8_t)hi);
}
// The same on four halves, and with an item outside the tensor (ok false) reading as zeros.
typedef _Float16 half4c_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4c_t act_half4(half4c_t v, _Float16 lo, _Float16 hi) {
    return __builtin_elementwise_min(__builtin_elementwise_max(v, (half4c_t)lo), (half4c_t)hi);
}
// The same with the kind known (a wave-uniform choice made outside the loop over a lane's values): nothing for ACT_NONE,
// one instruction for ACT_RELU, the general three otherwise.  Where a wave runs alone on its SIMD every vector
// instruction costs four cycles, and a staging thread converts dozens of values.
template <int KIND>
__device__ __forceinline__ float act_kind(float x, const Act& a) {
    if constexpr (KIND == ACT_NONE) return x;
    else if constexpr (KIND == ACT_RELU) return fmaxf(x, 0.f);
    else return act_p16(x, a);
}

// The fp16 hi/lo split of eight fp32 values of a staging item, scaled by the power of two s: hi = f16(s*x),
// lo = f16(s*x - hi), as packed halves.  Four instructions per pair of values: the mixed-precision multiply-adds take
// the fp32 value, the scale and (for lo) the half just written as their operands and round once, which is what the
// plain expression gives as well (s*x is exact); the compiler's own selection for that expression computes hi twice
// and needs eleven instructions per pair.  `ok` false: zeros.  KIND as for act_kind; ACT_NONE and ACT_RELU are clamps
// to +-3e38 and [0, 3e38] (one instruction, and the bounds collapse to 0 for an item outside the tensor).
__device__ __forceinline__ void split_pair(float x0, float x1, float s, unsigned& H, unsigned& L) {
    asm volatile(
        "v_fma_mixlo_f16 %0, %2, %3, 0\n\t"
        "v_fma_mixhi_f16 %0, %2, %4, 0\n\t"
        "v_fma_mixlo_f16 %1, %2, %3, -%0 op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %1, %2, %4, -%0 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
        : "=&v"(H), "=&v"(L)
        : "v"(s), "v"(x0), "v"(x1));
}
template <int KIND>
__device__ __forceinline__ void split8(const float (&r)[8], bool ok, const Act& a, float s, half8_t& hi, half8_t& lo) {
    typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
    float x[8];
    if constexpr (KIND == ACT_NONE || KIND == ACT_RELU) {
        const float top = ok ? 3.0e38f : 0.f, bottom = (KIND == ACT_RELU || !ok) ? 0.f : -3.0e38f;
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = __builtin_amdgcn_fmed3f(r[e], bottom, top);
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = ok ? act_p16(r[e], a) : 0.f;
    }
    u32x4_t H, L;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        unsigned h, l;
        split_pair(x[2 * e], x[2 * e + 1], s, h, l);
        H[e] = h;
        L[e] = l;
    }
    hi = __builtin_bit_cast(half8_t, H);
    lo = __builtin_bit_cast(half8_t, L);
}

// The second staged plane of the fp8 form of the correction terms, from the split halves of eight values:
// [8 x fp8(32 lo) | 8 x fp8(hi / 64)] (e4m3, round to nearest even).  With hi below 2^14 and lo below 2^3 (the value
// range's scale) both stay inside fp8's range, and values down to 2^-14 of the largest keep their four bits.
// (v_cvt_scalef32_pk_fp8_f16 converts two halves divided by a power of two: one instruction per pair)
typedef short c8_short2_t __attribute__((ext_vector_type(2)));
typedef _Float16 c8_half2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned c8_quad(_Float16 v0, _Float16 v1, _Float16 v2, _Float16 v3, float divisor) {
    c8_short2_t w = {0, 0};
    w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(w, c8_half2_t{v0, v1}, divisor, false);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(w, c8_half2_t{v2, v3}, divisor, true);
    return __builtin_bit_cast(unsigned, w);
}
__device__ __forceinline__ half8_t c8_plane(const half8_t& hi, const half8_t& lo) {
    typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
    u32x4_t w;
#pragma unroll
    for (int q = 0; q < 2; q++) {
        w[q] = c8_quad(lo[4 * q], lo[4 * q + 1], lo[4 * q + 2], lo[4 * q + 3], 0.03125f);
        w[2 + q] = c8_quad(hi[4 * q], hi[4 * q + 1], hi[4 * q + 2], hi[4 * q + 3], 64.f);
    }
    return __builtin_bit_cast(half8_t, w);
}

constexpr int KC = 32;        // input channels per chunk
constexpr int PITCH = KC * 2 + 16;   // bytes per staged pixel and plane: 8 neighbouring lanes' 16-byte reads cover all banks

// Row padding (bytes, a multiple of 16) with which the sixteen positions of every fragment of every wave read distinct
// LDS banks, for both ways the hardware may group the lanes of a 16-byte read (8 lanes over 32 banks, 16 over 64).
constexpr bool p16_pad_ok(int TH, int TW, int S, int WN, int row_pitch) {
    for (int model = 0; model < 2; model++) {
        const int banks = model ? 64 : 32, group = model ? 16 : 8;
        for (int wn = 0; wn < WN; wn++)
            for (int fn = 0; fn < TH * TW / 16; fn++)
                for (int g0 = 0; g0 < 64; g0 += group)
                    for (int i = g0; i < g0 + group; i++)
                        for (int j = i + 1; j < g0 + group; j++) {
                            const int mi = fn * 16 + (i & 15), mj = fn * 16 + (j & 15);
                            const int ai = (S * (mi / TW) * row_pitch + (wn * TW + mi % TW) * PITCH + (i >> 4) * 16) / 4;
                            const int aj = (S * (mj / TW) * row_pitch + (wn * TW + mj % TW) * PITCH + (j >> 4) * 16) / 4;
                            // (16-byte reads at 16-byte alignment: two of them meet in a bank exactly when they start in the same one)
                            if (ai % banks == aj % banks && ai != aj) return false;
                        }
    }
    return true;
}
constexpr int p16_row_pad(int TH, int TW, int S, int WN, int slots) {
    for (int pad = 0; pad < 256; pad += 16)
        if (p16_pad_ok(TH, TW, S, WN, slots * PITCH + pad)) return pad;
    return 96;
}
}  // namespace
}  // namespace fynhip
