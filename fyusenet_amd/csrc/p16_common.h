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
