// 3x3 convolution between wide layers with fp32 storage (the residual blocks of a style-transfer net) as an
// implicit GEMM on gfx950 matrix cores with 16-position fragments (v_mfma_f32_16x16x32_f16, fp32 accumulate).
//
// Replaces, for such layers, the render passes of DeepConvLayerNxN::forward (fyusenet/gpu/deep/deepconvlayerNxN.cpp:
// 129-211); epilogue order of shaders/deep/deepconv3x3_tiled.frag:36-45 (acc*scale + bias, then the residual).
//
// Why a second MFMA kernel: with 32x32 fragments a workgroup's tile is a multiple of 32 positions, and a layer of
// 128x156 positions then fills 208 of the 256 CUs for three fragment rounds.  16-position fragments allow tiles of
// 8x10 positions: 16x16 = 256 workgroups, one per CU, five fragments each (the work of 2.5 of the larger ones).
//
// GEMM view as in conv_mfma.hip: M = output channels (A = weights, packed per lane, streamed through L2 into a register
// ring), N = positions (B = activations, staged per 32-channel chunk as a halo tile in LDS, fp16 hi and lo planes),
// K = taps x input channels, one tap of one chunk (32 channels) per step.  Three MFMAs per fragment pair (hi*hi,
// lo*hi, hi*lo).  Tile size, halo pitch and the tap offsets are compile-time constants, so a B fragment read is one
// LDS instruction with an immediate offset and the step loop has no address arithmetic.
//
// Workgroup = 4 staging waves (next chunk: global loads, activation, hi/lo conversion, LDS writes; scale and bias at
// the start and, during the last chunk, the residual tile into LDS) + 4 MFMA waves (32 output channels each: 2 channel
// fragments x FN position fragments).  A lane's accumulators of one fragment are 4 consecutive fragment rows of one
// position, so the epilogue needs no transposition: residual and scale/bias from LDS, one 16-byte store per fragment
// (fp16 tensors: the weights are packed so that row r of fragment fm of a wave's pair is output channel
// 8*(r/4) + 4*fm + r%4 of the wave's 32, a lane's eight values are eight consecutive channels and go out in one store).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "kernels.h"
#include "p16_common.h"
#include "range.h"


namespace fynhip {

// The file is compiled twice: for fp32 tensors (operands split into fp16 hi and lo planes, three MFMA passes; this
// translation unit also holds the host entry points) and, with -DFYN_P16_HALF=1, for fp16 tensors (one plane, one pass).
#ifndef FYN_P16_HALF
#define FYN_P16_HALF 0
#endif

namespace {
constexpr int NT = 9;         // taps
constexpr int PD = 6;         // depth of the weight-fragment ring (steps)
constexpr bool HSTORE = FYN_P16_HALF != 0;   // fp16 tensors
constexpr int NPL = HSTORE ? 1 : 2;          // staged planes (hi, lo)
constexpr int NPASS = HSTORE ? 1 : 3;        // MFMAs per fragment pair (hi*hi, lo*hi, hi*lo)
// fp32 tensors, weight planes per fragment (launch_conv_p16, launch_tconv_p16): fp16 hi, fp16 lo, and the fp8 operands of
// the correction terms, [8 x fp8(hi / 32) | 8 x fp8(lo * 64)] per lane; a kernel reads plane 0 and one of the other two
constexpr int NPLW = HSTORE ? 1 : 3;
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
constexpr int ESZ = HSTORE ? 2 : 4;          // bytes per stored element
typedef std::conditional<HSTORE, _Float16, float>::type store_t;
// Output channel, inside a wave's 32, of accumulator element e of channel fragment fm in the lanes kq = lane / 16:
// kq * CHK + fm * CHF + e.  fp32 tensors: fragment rows are channels in order (a fragment's store is 64 contiguous bytes
// from the four lanes of a position).  fp16 tensors: the weights are packed so that a lane's eight values are eight
// consecutive channels (one 16-byte store per lane and position instead of two of 8 bytes; with fp32 tensors the same
// layout -- two 16-byte stores per lane, interleaved between lanes -- measured slower).
constexpr int CHK = HSTORE ? 8 : 4, CHF = HSTORE ? 4 : 16;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

// Geometry of one instantiation.  A workgroup's four MFMA waves are WM groups of 32 output channels x WN = 4 / WM tiles
// of TH x TW positions side by side; S is the input step per position (1 or 2).  With S = 2 the staged tile keeps even
// and odd columns in separate halves of a row, so that the positions of a fragment are neighbours in LDS whatever the
// tap: column c lives in slot (c & 1) * HWH + (c >> 1).
template <int TH_, int TW, int S, int WM, int KH = 2>
struct Geo {
    static constexpr int TH = TH_, STEP = S;
    static constexpr int WN = 4 / WM;
    static constexpr int TWG = WN * TW;                  // positions per row of the workgroup's tile
    static constexpr int HW = S * (TWG - 1) + 1 + KH, HH = S * (TH - 1) + 1 + KH;   // (KH: 2 for 3x3 taps, 1 for the transposed layer's)
    static constexpr int HWH = (HW + 1) / 2;
    static constexpr int SLOTS = (S == 1) ? HW : 2 * HWH;
    static constexpr int ROW_PITCH = SLOTS * PITCH + p16_row_pad(TH, TW, S, WN, SLOTS);
    static constexpr int PLANE = HH * ROW_PITCH;
    static constexpr int BUF = NPL * PLANE;              // hi, lo
    static constexpr int NPOS = TH * TW, FN = NPOS / 16;  // per wave
    static constexpr int NITEMS = HH * HW * (KC / 8);    // staging items: (pixel, 8 channels)
    static constexpr int NB = (NITEMS + 255) / 256;      // ... per staging thread
    static constexpr int CPB = 32 * WM;                  // output channels per workgroup
    static constexpr int RES_PITCH = CPB * ESZ + 16;     // bytes per position of the residual tile
    static constexpr int RPP = CPB * ESZ / 16;           // 16-byte pieces per position
    static constexpr int RPIECES = TH * TWG * RPP;       // residual 16-byte pieces
    static constexpr int RNB = (RPIECES + 255) / 256;    // ... per staging thread
    static constexpr int slot_off(int c) { return (S == 1) ? c * PITCH : ((c & 1) * HWH + (c >> 1)) * PITCH; }
    static constexpr int tap_off(int t) { return (t / 3) * ROW_PITCH + slot_off(t % 3); }
    static_assert(S == 1 || S == 2, "input step 1 or 2");
    static_assert(NPOS % 16 == 0, "whole position fragments");
    static_assert(PLANE + 2 * ROW_PITCH + 2 * PITCH + HWH * PITCH + 64 < 65536, "B fragment offsets inside a staging buffer fit the LDS instructions' immediate field");
};
// One stage = the nine steps of one 32-channel chunk of one tile, read from staging buffer BUFI (stages alternate between
// the two buffers; the B fragments of the stage's first step are in `b`, and the stage ends with those of the first step
// of the other buffer, i.e. of the stage that follows).  One slot per MFMA: the MFMA, then a share of the step's memory
// instructions, fenced so that the compiler keeps the order (a memory instruction issued right after an MFMA runs in
// its shadow).  Position fragment fn is used by six consecutive MFMAs; its registers are then refilled with the
// fragment of the next step, so one register set per fragment is enough.  The ring slot of the previous step is
// refilled with the weights of step t+PD-1 (the weight stream wraps from the last step of a tile to the first of the
// next).  The barrier of a stage sits in its last step, before the first read of the other buffer: the staging waves
// have filled that buffer by then, and all reads of this stage's buffer were issued a step earlier.
template <class G, int BUFI>
__device__ __forceinline__ void p16_stage(f32x4_t (&acc)[2][G::FN], half8_t (&a_q)[PD][2][NPL], half8_t (&b)[G::FN][NPL],
                                          const int (&bbase)[2][G::FN], const unsigned char* lds, const unsigned char*& wnext,
                                          const unsigned char* wbase, const unsigned char* wend, unsigned wstep, unsigned wlane) {
    constexpr int FN = G::FN;
#pragma unroll
    for (int dd = 0; dd < NT; dd++) {
        const int d = (BUFI * NT + dd) % PD, dprev = (d + PD - 1) % PD;   // (two stages = 18 steps = three turns of the ring)
        const int nbuf = (dd + 1 == NT) ? 1 - BUFI : BUFI, noff = G::tap_off((dd + 1) % NT);
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
        constexpr int SL = 2 * NPASS, NS = SL * FN, NW = 2 * NPL;   // slots per position fragment and per step; weight fragments per step
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const int fn = i / SL, r = i % SL, kind = r / 2, fm = r % 2;
            const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_q[d][fm][apl], b[fn][bpl], acc[fm][fn], 0, 0, 0);
            if (dd == NT - 1 && i == (SL - 1 < 3 ? SL - 1 : 3)) lds_barrier();   // (ahead of the slot's own fragment read)
            if (r == SL - 1) {
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) b[fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[nbuf][fn] + noff + pl * G::PLANE);
            }
#pragma unroll
            for (int j = 0; j < NW; j++)   // the weight fragments of a step, spread over its slots
                if (i == ((j * NS) / NW + 1 < NS ? (j * NS) / NW + 1 : NS - 1))
                    a_q[dprev][j % 2][j / 2] = *reinterpret_cast<const half8_t*>(w_ + ((j % 2) * NPLW + j / 2) * 1024 + wlane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The same stage with the two correction terms of the operand split (lo*hi and hi*lo, 2^-11 of the result) as fp8
// matrix instructions, v_mfma_f32_16x16x128_f8f6f4: 128 products per lane row and instruction at twice the fp16 rate.
// The second staged plane then holds, per pixel and eight channels, [8 x fp8(32 lo) | 8 x fp8(hi / 64)], the third
// weight plane [8 x fp8(hi / 32) | 8 x fp8(64 lo)]: element by element the products are lo*hi and hi*lo with the scales
// cancelling, so all passes add into one accumulator.  One instruction takes the sixteen bytes of two consecutive steps
// (two taps) on either side; steps are paired along the whole tile (s = 9 * chunk + tap even with s + 1), which needs an
// even number of chunks.  Per step: ten fp16 MFMAs (hi*hi), and in every second step ten fp8 ones in front of them --
// 304 matrix-pipe cycles per fragment pair and chunk instead of 432.  The correction terms keep four significant bits
// for operands down to 2^-14 of the largest a tensor holds, which needs the tensor's value range (range.h): the kernel
// runs on inputs that carry a range word; measured against the fp64 oracle: rel-L2 1e-5 (three fp16 passes: 3e-7).
// Registers: a0 = ring of the fp16 hi weights, a2 = ring of the fp8 weights in pairs of steps, b0 = fp16 hi fragments,
// b1 = the fp8 fragments of a pair of steps.  The refills follow the uses in program order: a fragment's registers for
// the next step after its own MFMAs, the ring slot of step s-1 (whose fp8 half this step's fp8 block may still read)
// behind that block.
template <class G, int PH>
__device__ __forceinline__ void p16_stage_c8(f32x4_t (&acc)[2][G::FN], half8_t (&a0)[PD][2], i32x8_t (&a2)[PD / 2][2], half8_t (&b0)[G::FN],
                                             i32x8_t (&b1)[G::FN], const int (&bbase)[2][G::FN], const unsigned char* lds,
                                             const unsigned char*& wnext, const unsigned char* wbase, const unsigned char* wend, unsigned wstep,
                                             unsigned wlane) {
    constexpr int FN = G::FN;
    static_assert(PD % 2 == 0 && (2 * NT) % PD == 0, "pairs of steps keep their ring slots over two stages");
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int s = PH * NT + t, d = s % PD, dprev = (d + PD - 1) % PD;
        const bool pair = (s & 1) != 0;                    // the second step of a pair: the fp8 block runs
        const int nbuf = (t + 1 == NT) ? 1 - PH : PH, noff = G::tap_off((t + 1) % NT);
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
        // the loads of the step: weights of step s + PD - 1 into the ring slot of step s - 1 (a0: two fragments, a2: two
        // halves of fragments), and every position fragment's operands of step s + 1
        auto load_a0 = [&](int wfm) { a0[dprev][wfm] = *reinterpret_cast<const half8_t*>(w_ + (wfm * NPLW) * 1024 + wlane); };
        auto load_a2 = [&](int wfm) {
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(w_ + (wfm * NPLW + 2) * 1024 + wlane);
            if ((dprev & 1) == 0) { a2[dprev / 2][wfm][0] = v[0]; a2[dprev / 2][wfm][1] = v[1]; a2[dprev / 2][wfm][2] = v[2]; a2[dprev / 2][wfm][3] = v[3]; }
            else { a2[dprev / 2][wfm][4] = v[0]; a2[dprev / 2][wfm][5] = v[1]; a2[dprev / 2][wfm][6] = v[2]; a2[dprev / 2][wfm][7] = v[3]; }
        };
        auto load_b0 = [&](int fn) { b0[fn] = *reinterpret_cast<const half8_t*>(lds + bbase[nbuf][fn] + noff); };
        auto load_b1 = [&](int fn) {
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(lds + bbase[nbuf][fn] + noff + G::PLANE);
            if (((s + 1) & 1) == 0) { b1[fn][0] = v[0]; b1[fn][1] = v[1]; b1[fn][2] = v[2]; b1[fn][3] = v[3]; }
            else { b1[fn][4] = v[0]; b1[fn][5] = v[1]; b1[fn][6] = v[2]; b1[fn][7] = v[3]; }
        };
        // (a pair step also fetches the second half of the NEXT pair, two steps ahead -- that half is free once the
        // step's fp8 block has run --, which leaves the short step between two pair steps with five LDS reads instead
        // of ten; not across the end of a stage, where the other buffer is handed over in the last step only)
        const bool ahead2 = pair && t + 2 < NT;
        const bool have_b1 = !pair && t > 0 && (((s - 1) & 1) != 0) && (t - 1) + 2 < NT;   // step s - 1 fetched this step's share
        auto load_b1_ahead = [&](int fn) {
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(lds + bbase[PH][fn] + G::tap_off(t + 2) + G::PLANE);
            b1[fn][4] = v[0]; b1[fn][5] = v[1]; b1[fn][6] = v[2]; b1[fn][7] = v[3];
        };
        if (pair) {
            // fp8 block: a fragment's fp8 operands of the next step (the half that this block has just read) behind its
            // two MFMAs, the fp16 weights in the first slots; the barrier of a stage's last step ahead of every read
            // of the other buffer
#pragma unroll
            for (int i = 0; i < 2 * FN; i++) {
                const int fn = i / 2, fm = i % 2;
                acc[fm][fn] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a2[d / 2][fm], b1[fn], acc[fm][fn], 0, 0, 0, 0, 0, 0);
                if (t == NT - 1 && i == 0) lds_barrier();
                if (fm == 1) load_b1(fn);
#pragma unroll
                for (int j = 0; j < 2; j++)
                    if ((j * 2 * FN) / 2 == i) load_a0(j);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int i = 0; i < 2 * FN; i++) {
            const int fn = i / 2, fm = i % 2;
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0[d][fm], b0[fn], acc[fm][fn], 0, 0, 0);
            if (!pair && t == NT - 1 && i == 0) lds_barrier();
            if (fm == 1) {   // the fragment's MFMAs of this step are issued: its operands of the next step
                load_b0(fn);
                if (!pair && !have_b1) load_b1(fn);
                if (ahead2) load_b1_ahead(fn);
            }
            if (pair) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    if ((j * 2 * FN) / 2 == i) load_a2(j);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if ((j * 2 * FN) / 4 == i) { if (j < 2) load_a0(j); else load_a2(j - 2); }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The staging waves of a workgroup (threads 0..255): stage after stage -- a 32-channel chunk of a tile's halo: global
// loads, activation, hi/lo conversion, LDS writes -- one stage ahead of the MFMA waves, across tile boundaries; scale and
// bias at the start and, during a tile's last chunk, its residual tile.  One barrier per stage, after the one that hands
// over the first.
// (C8: the second plane in the fp8 form, see p16_stage_c8)
template <class G, bool C8 = false>
__device__ __forceinline__ void p16_stager(const ConvP16Params& p, unsigned char* lds, int stid, int cb, int group, int ntiles,
                                           int nchunks, unsigned range_bits) {
    constexpr int CPB = G::CPB;
    constexpr int sb_off = 2 * G::BUF;
    constexpr int res_off = sb_off + 2 * CPB * 4;
    const store_t* in = reinterpret_cast<const store_t*>(p.in);
    int i_y[G::NB], i_x[G::NB];   // an item's pixel inside the halo tile (rows above 2^15: no such item)
    int l_off[G::NB];
#pragma unroll
    for (int i = 0; i < G::NB; i++) {
        const int idx = stid + i * 256;
        l_off[i] = -1; i_y[i] = 1 << 20; i_x[i] = 0;
        if (idx < G::NITEMS) {
            const int pix = idx >> 2, g = idx & 3;
            const int py = pix / G::HW, px = pix - py * G::HW;
            i_y[i] = py; i_x[i] = px;
            l_off[i] = py * G::ROW_PITCH + ((G::STEP == 1) ? px * PITCH : ((px & 1) * G::HWH + (px >> 1)) * PITCH) + g * 16;
        }
    }
    const int g8 = (stid & 3) * 8;
    // Two sets of staging registers: the loads of stage n+2 are issued before stage n+1 is converted, so a stage's
    // memory latency passes while the stage before it is written to LDS.
    int g_off[2][G::NB];       // element offsets of a set's items, -1: outside the frame (reads as 0)
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HSTORE, half8_t, RawF>::type raw_t;   // an item as it comes from memory: 8 channels
    raw_t raw[2][G::NB];
    float in_scale = 1.f, inv_unused;
    // (unconditional loads: items outside the tensor read its first element and are zeroed when stored)
    auto fetch = [&](auto set_, int tile, int chunk) {
        constexpr int SET = decltype(set_)::value;
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const int y0 = tyi * G::TH * G::STEP + p.in_y0, x0 = txi * G::TWG * G::STEP + p.in_x0;
#pragma unroll
        for (int i = 0; i < G::NB; i++) {
            // (coordinates in the frame of repeated pixels, which is the stored frame unless the step is fractional)
            int gy = y0 + i_y[i], gx = x0 + i_x[i];
            const int vhp = p.in_hp << p.in_shift, vwp = p.in_wp << p.in_shift;
            if (p.in_clamp && l_off[i] >= 0) {
                gy = min(max(gy, 0), vhp - 1);
                gx = min(max(gx, 0), vwp - 1);
            }
            // (the last chunk of a tensor whose channel pitch is not a multiple of 32: the groups of 8 behind the pitch are zeros)
            g_off[SET][i] = ((unsigned)gy < (unsigned)vhp && (unsigned)gx < (unsigned)vwp && g8 + chunk * KC < p.in_cp) ? ((gy >> p.in_shift) * p.in_wp + (gx >> p.in_shift)) * p.in_cp + g8 + chunk * KC : -1;
            const store_t* src = in + (g_off[SET][i] >= 0 ? g_off[SET][i] : 0);
            if constexpr (HSTORE) {
                raw[SET][i] = *reinterpret_cast<const half8_t*>(src);
            } else {
                raw[SET][i].a = *reinterpret_cast<const float4*>(src);
                raw[SET][i].b = *reinterpret_cast<const float4*>(src + 4);
            }
        }
    };
    const int act_kind_ = p.act.kind;
    auto store = [&](auto set_, unsigned char* buf) {
        constexpr int SET = decltype(set_)::value;
        if constexpr (HSTORE) {
            // (an activation that is exact on halves acts on the packed halves: two instructions per item instead of seven per value)
            _Float16 hlo, hhi;
            const bool half_act = act_half_exact(p.act, hlo, hhi);
#pragma unroll
            for (int i = 0; i < G::NB; i++) {
                if (l_off[i] < 0) continue;
                const bool ok = g_off[SET][i] >= 0;
                half8_t v;
                if (half_act) {
                    v = ok ? act_half(raw[SET][i], hlo, hhi) : (half8_t)((_Float16)0.f);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] = ok ? (_Float16)act_p16((float)raw[SET][i][e], p.act) : (_Float16)0.f;
                }
                *reinterpret_cast<half8_t*>(buf + l_off[i]) = v;
            }
        } else {
            // (the activation's kind chosen once per call, the hi/lo split in four instructions per pair: split8)
            auto split_all = [&](auto kind_) {
                constexpr int KIND = decltype(kind_)::value;
#pragma unroll
                for (int i = 0; i < G::NB; i++) {
                    if (l_off[i] < 0) continue;
                    const float4 r0 = raw[SET][i].a, r1 = raw[SET][i].b;
                    const float r[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
                    half8_t hi, lo;
                    split8<KIND>(r, g_off[SET][i] >= 0, p.act, in_scale, hi, lo);
                    *reinterpret_cast<half8_t*>(buf + l_off[i]) = hi;
                    *reinterpret_cast<half8_t*>(buf + G::PLANE + l_off[i]) = C8 ? c8_plane(hi, lo) : lo;
                }
            };
            if (act_kind_ == ACT_RELU) split_all(std::integral_constant<int, ACT_RELU>());
            else if (act_kind_ == ACT_NONE) split_all(std::integral_constant<int, ACT_NONE>());
            else split_all(std::integral_constant<int, ACT_LEAKY>());
        }
    };
    auto residual_in = [&](int tile) {   // the residual tile of a tile: [position][CPB channels] as stored, in 16-byte pieces
        const store_t* res = reinterpret_cast<const store_t*>(p.res);
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        f32x4_t rv[G::RNB];
#pragma unroll
        for (int i = 0; i < G::RNB; i++) {
            const int idx = stid + i * 256;
            const int m = idx / G::RPP, piece = idx % G::RPP;
            const int ty = m / G::TWG, tx = m - ty * G::TWG;
            const int py = tyi * G::TH + ty, px = txi * G::TWG + tx;
            const bool ok = idx < G::RPIECES && py < p.npos_y && px < p.npos_x && cb * CPB + piece * (16 / ESZ) < p.res_cp;
            rv[i] = *reinterpret_cast<const f32x4_t*>(res + (ok ? ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp + cb * CPB + piece * (16 / ESZ) : 0));
        }
#pragma unroll
        for (int i = 0; i < G::RNB; i++) {
            const int idx = stid + i * 256;
            if (idx < G::RPIECES) *reinterpret_cast<f32x4_t*>(lds + res_off + (idx / G::RPP) * G::RES_PITCH + (idx % G::RPP) * 16) = rv[i];
        }
    };
    // the stage after (tile, c); false: there is none
    auto advance = [&](int& tile, int& c) {
        if (++c == nchunks) { c = 0; tile += p.pos_groups; }
        return tile < ntiles;
    };
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;
    
    int tile = group, c = 0;          // the stage the MFMA waves are on (stage n)
    int t1 = group, c1 = 0;           // stage n+1
    fetch(Set0(), tile, 0);
    bool have1 = advance(t1, c1);
    int t2 = t1, c2 = c1;             // stage n+2
    bool have2 = have1 && advance(t2, c2);
    if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_unused);
    if (stid < CPB) {   // (scale and bias have one entry per channel of the output tensor's pitch)
        const bool have = cb * CPB + stid < p.out_cp;
        reinterpret_cast<float*>(lds + sb_off)[stid] = have ? p.scale[cb * CPB + stid] : 0.f;
        reinterpret_cast<float*>(lds + sb_off)[CPB + stid] = have ? p.bias[cb * CPB + stid] : 0.f;
    }
    store(Set0(), lds);
    
    lds_barrier();
    if (have1) fetch(Set1(), t1, c1);   // (not before the first stage is handed over: every workgroup of the launch is fetching at that moment; measured again with the fp8 form: 15.3 against 15.6 us)
    // One iteration per stage n of the MFMA waves: stage n+1 (fetched an iteration ago) is written to the other
    // buffer, then stage n+2 is fetched into the registers that stage n left.  Unrolled by two: set = parity of the stage.
    auto iteration = [&](auto next_set, auto free_set, unsigned char* next_buf) {
        if (c + 1 == nchunks && p.res) residual_in(tile);
        if (have1) store(next_set, next_buf);
        if (have2) fetch(free_set, t2, c2);
        lds_barrier();
        const bool go_on = have1;
        tile = t1; c = c1; t1 = t2; c1 = c2; have1 = have2;
        if (have2) have2 = advance(t2, c2);
        return go_on;
    };
    for (;;) {
        if (!iteration(Set1(), Set0(), lds + G::BUF)) break;   // stage n even: n+1 is in set 1, goes into buffer 1
        if (!iteration(Set0(), Set1(), lds)) break;
    }
}

// Grid: cout_blocks x pos_groups workgroups; a workgroup keeps its block of output channels and walks the tiles
// group, group + pos_groups, ... (one tile each when the layer has no more tiles than the chip has CUs).  The staging
// waves run one stage ahead of the MFMA waves, across tile boundaries, so that from the second tile on a tile's fetch
// and the previous tile's stores overlap with MFMA work.
// C8 (fp32 tensors, an even number of chunks, an input with a range word): the correction terms as fp8 MFMAs (p16_stage_c8)
template <int TH, int TW, int S, int WM, bool C8 = false>
__global__ __launch_bounds__(512) void conv_p16_kernel(const ConvP16Params p) {
    using G = Geo<TH, TW, S, WM>;
    constexpr int FN = G::FN, CPB = G::CPB;
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ unsigned range_box[2];   // meeting point of the MFMA waves' output maxima (range.h)
    if (blockIdx.x == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups are dealt round-robin to the 8 XCDs; remap so that neighbouring tiles (shared halos) meet in one L2.
    int bid = blockIdx.x;
    {
        const int nblk = p.pos_groups * p.cout_blocks;
        const int per = nblk >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    const int cb = bid % p.cout_blocks;
    const int group = bid / p.cout_blocks;
    const int ntiles = p.tiles_x * p.tiles_y;
    if (tid < 2) range_box[tid] = 0u;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    const int nchunks = p.cin_chunks;
    // LDS: two staging buffers, scale and bias, the residual tile
    constexpr int sb_off = 2 * G::BUF;
    constexpr int res_off = sb_off + 2 * CPB * 4;

    if (wave < 4) {   // the first four waves stage: they start first
        p16_stager<G, C8>(p, lds, tid & 255, cb, group, ntiles, nchunks, range_bits);
        return;
    }

    // ---------------------------------------------------------------------- MFMA waves
    const int mq = lane & 15, kq = lane >> 4;
    const int mw = (wave - 4) % WM;   // this wave's 32 output channels of the workgroup's CPB
    const int wn = (wave - 4) / WM;   // ... and its tile of positions
    int bbase[2][FN];   // per-lane LDS offset of the B fragments in either staging buffer: position, then the lane's 8 channels of the chunk
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = fn * 16 + mq;
        const int ty = m / TW, tx = m - ty * TW;
        bbase[0][fn] = S * ty * G::ROW_PITCH + (wn * TW + tx) * PITCH + kq * 16;
        bbase[1][fn] = bbase[0][fn] + G::BUF;
    }
    // A fragments: [(chunk*9 + tap)][cout fragment of 16][plane][lane] x 8 halves
    const unsigned wstep = (unsigned)p.mfrags * NPLW * 1024;
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)((cb * 2 * WM + mw * 2) * NPLW) * 1024;   // (uniform: the loads take it as their scalar base)
    const unsigned wlane = lane * 16;
    const unsigned char* wend = wbase + (size_t)nchunks * NT * wstep;
    half8_t a_q[C8 ? 1 : PD][2][NPL];   // exact form: hi and lo weights of a step
    half8_t a0[C8 ? PD : 1][2];         // fp8 form: hi weights of a step ...
    i32x8_t a2[C8 ? PD / 2 : 1][2];     // ... and the fp8 weights of a pair of steps
    if constexpr (C8) {
#pragma unroll
        for (int d = 0; d < PD; d++)
#pragma unroll
            for (int fm = 0; fm < 2; fm++) {
                a0[d][fm] = *reinterpret_cast<const half8_t*>(wbase + (size_t)d * wstep + (fm * NPLW) * 1024 + wlane);
                const i32x4_t v = *reinterpret_cast<const i32x4_t*>(wbase + (size_t)d * wstep + (fm * NPLW + 2) * 1024 + wlane);
#pragma unroll
                for (int e = 0; e < 4; e++) a2[d / 2][fm][(d & 1) * 4 + e] = v[e];
            }
    } else {
#pragma unroll
        for (int d = 0; d < PD; d++)
#pragma unroll
            for (int fm = 0; fm < 2; fm++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a_q[d][fm][pl] = *reinterpret_cast<const half8_t*>(wbase + (size_t)d * wstep + (fm * NPLW + pl) * 1024 + wlane);
    }
    f32x4_t acc[2][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int fm = 0; fm < 2; fm++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++) acc[fm][fn] = (f32x4_t)(0.f);
    };
    zero_acc();
    float inv_in_scale = 1.f;
    if (p.in_amax) (void)range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    store_t* out = reinterpret_cast<store_t*>(p.out);
    const bool have_res = p.res != nullptr;
    const bool through = store_through_pays(p.out, p.npos_y, p.npos_x, p.out_cp * ESZ, (p.cout_blocks == 1 || (CPB * ESZ) % 128 == 0) && !p.plain_stores, hw_block_count());
    bool drop = through && wave == 4 && hw_block_id() < 8;
    const bool res_scale = p.res_scale != 0;
    const float res_floor = p.res_relu ? 0.f : -__builtin_inff();
    float vmax = 0.f;

    // Epilogue of a tile.  A lane holds, per fragment, output channels 4*kq .. 4*kq+3 of position fn*16 + mq.  One
    // wave per SIMD pays four cycles per vector instruction, so the arithmetic is kept short (acc_mul is a power of two:
    // folding it into the scale changes no bit) and every fragment is stored as soon as it is finished.
    auto finish_tile = [&](int tile) {
        if (drop) {   // (ahead of this workgroup's first store: what it has read so far may go as well)
            drop_clean_l2_lines();
            drop = false;
        }
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const float* sb = reinterpret_cast<const float*>(lds + sb_off);
        f32x4_t rs[2], bi[2], scm[2];
#pragma unroll
        for (int fm = 0; fm < 2; fm++) {
            const f32x4_t sc = *reinterpret_cast<const f32x4_t*>(sb + mw * 32 + kq * CHK + fm * CHF);
            bi[fm] = *reinterpret_cast<const f32x4_t*>(sb + CPB + mw * 32 + kq * CHK + fm * CHF);
            scm[fm] = sc * acc_mul;
            rs[fm] = res_scale ? sc : (f32x4_t)(1.f);
        }
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            const int m = fn * 16 + mq;
            const int ty = m / TW, tx = wn * TW + (m - ty * TW);
            const int py = tyi * TH + ty, px = txi * G::TWG + tx;
            const bool inside = py < p.npos_y && px < p.npos_x;
            const size_t obase = ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp + cb * CPB + mw * 32 + kq * CHK;
            float fmax_ = 0.f;
            half8_t hv;
#pragma unroll
            for (int fm = 0; fm < 2; fm++) {
                // (a block of output channels may reach behind the tensor's channel pitch: those groups are not stored)
                const bool ok = inside && cb * CPB + mw * 32 + kq * CHK + (HSTORE ? 0 : fm * CHF) < p.out_cp;
                f32x4_t v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[fm][fn][e] * scm[fm][e] + bi[fm][e];
                if (have_res) {
                    // (the two options as operands instead of selects: max(r, 0 or -inf), times scale or 1)
                    const unsigned char* rsrc = lds + res_off + (ty * G::TWG + tx) * G::RES_PITCH + (mw * 32 + kq * CHK + fm * CHF) * ESZ;
                    f32x4_t rv;
                    if constexpr (HSTORE) {
                        const half4_t rh = *reinterpret_cast<const half4_t*>(rsrc);
#pragma unroll
                        for (int e = 0; e < 4; e++) rv[e] = (float)rh[e];
                    } else {
                        rv = *reinterpret_cast<const f32x4_t*>(rsrc);
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = fmaf(fmaxf(rv[e], res_floor), rs[fm][e], v[e]);
                }
                if constexpr (HSTORE) {
#pragma unroll
                    for (int e = 0; e < 4; e++) hv[fm * 4 + e] = (_Float16)v[e];
                    if (fm == 1 && ok) store_out(through, reinterpret_cast<half8_t*>(out + obase), hv);   // the lane's eight channels in one store
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) fmax_ = fmaxf(fmax_, ok ? fabsf(v[e]) : 0.f);
                    if (ok) store_out(through, reinterpret_cast<f32x4_t*>(out + obase + fm * CHF), v);
                }
            }
            vmax = fmaxf(vmax, fmax_);
        }
    };

    lds_barrier();   // the first stage is staged
    half8_t b[C8 ? 1 : FN][NPL];
    half8_t b0[C8 ? FN : 1];
    i32x8_t b1[C8 ? FN : 1];
    if constexpr (C8) {
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            b0[fn] = *reinterpret_cast<const half8_t*>(lds + bbase[0][fn]);
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(lds + bbase[0][fn] + G::PLANE);
#pragma unroll
            for (int e = 0; e < 4; e++) { b1[fn][e] = v[e]; b1[fn][4 + e] = 0; }
        }
    } else {
#pragma unroll
        for (int fn = 0; fn < FN; fn++)
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) b[fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[0][fn] + pl * G::PLANE);
    }

    const unsigned char* wnext = wbase + (size_t)((PD - 1) % (nchunks * NT)) * wstep;
    int tile = group, c = 0;
    if constexpr (C8) {
        // (an even number of chunks: a tile is whole pairs of stages)
        for (;;) {
            p16_stage_c8<G, 0>(acc, a0, a2, b0, b1, bbase, lds, wnext, wbase, wend, wstep, wlane);
            p16_stage_c8<G, 1>(acc, a0, a2, b0, b1, bbase, lds, wnext, wbase, wend, wstep, wlane);
            c += 2;
            if (c == nchunks) {
                finish_tile(tile);
                c = 0; tile += p.pos_groups;
                if (tile >= ntiles) break;
                zero_acc();
            }
        }
    } else {
    for (;;) {
        p16_stage<G, 0>(acc, a_q, b, bbase, lds, wnext, wbase, wend, wstep, wlane);
        if (++c == nchunks) {
            finish_tile(tile);
            c = 0; tile += p.pos_groups;
            if (tile >= ntiles) break;
            zero_acc();
        }
        p16_stage<G, 1>(acc, a_q, b, bbase, lds, wnext, wbase, wend, wstep, wlane);
        if (++c == nchunks) {
            finish_tile(tile);
            c = 0; tile += p.pos_groups;
            if (tile >= ntiles) break;
            zero_acc();
        }
    }
    }
    if (p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 4);
}

// ---------------------------------------------------------------------------------------------------------------
// Transposed 3x3 convolution that up-samples by two, cropped to exactly twice the input size (replaces the stencil
// passes of DeepTransConvLayerBase::forward, gpu/deep/deeptransconvlayerbase.cpp:83-130, for such layers):
//     out[2a+py, 2b+px] = sum over dy, dx of W[py+2dy, px+2dx] * in[a-dy, b-dx],   py+2dy <= 2, px+2dx <= 2.
// Positions are input pixels; every tap (ky, kx) feeds the accumulators of exactly one output parity (ky&1, kx&1) and
// reads the input shifted by (ky>>1, kx>>1), so a chunk is nine steps as in a 3x3 convolution, with four accumulator
// sets and four distinct B fragments per position fragment (two register sets: the next shift's fragments are read
// while the current shift's taps run).  Taps in the order of their shift:
constexpr int TT_KY[NT] = {0, 0, 1, 1, 0, 1, 2, 2, 2};
constexpr int TT_KX[NT] = {0, 1, 0, 1, 2, 2, 0, 1, 2};
constexpr int tt_shift(int t) { return (TT_KY[t] >> 1) * 2 + (TT_KX[t] >> 1); }
constexpr int tt_parity(int t) { return (TT_KY[t] & 1) * 2 + (TT_KX[t] & 1); }
constexpr bool tt_last_of_shift(int t) { return t == NT - 1 || tt_shift(t + 1) != tt_shift(t); }

// (PDT: depth of the weight ring; three position fragments per wave leave room for three steps only, which at 288 cycles
// per step still covers an L2 round trip)
template <class G, int BUFI, int PDT>
__device__ __forceinline__ void tp16_stage(f32x4_t (&acc)[4][2][G::FN], half8_t (&a_q)[PDT][2][NPL], half8_t (&b)[2][G::FN][NPL],
                                           const int (&bbase)[2][G::FN], const unsigned char* lds, const unsigned char*& wnext,
                                           const unsigned char* wbase, const unsigned char* wend, unsigned wstep, unsigned wlane) {
    constexpr int FN = G::FN;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int d = (BUFI * NT + t) % PDT, dprev = (d + PDT - 1) % PDT;
        const int sh = tt_shift(t), set = sh & 1, par = tt_parity(t);
        const int nsh = (sh + 1) & 3, nbuf = (t == NT - 1) ? 1 - BUFI : BUFI;
        // the tile is staged with one pixel of halo above and to the left: shift (dy, dx) reads pixel (1-dy, 1-dx) + position
        const int noff = (1 - (nsh >> 1)) * G::ROW_PITCH + (1 - (nsh & 1)) * PITCH;
        constexpr int SL = 2 * NPASS, NS = SL * FN, NW = 2 * NPL;
        constexpr int BAR = HSTORE ? 0 : 3;             // the slot of the stage's barrier in its last step
        const int first_read = (t == NT - 1) ? BAR + 1 : 0;
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const int fn = i / SL, r = i % SL, kind = r / 2, fm = r % 2;
            const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
            acc[par][fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_q[d][fm][apl], b[set][fn][bpl], acc[par][fm][fn], 0, 0, 0);
            if (t == NT - 1 && i == BAR) lds_barrier();
            if (tt_last_of_shift(t) && i >= first_read && i < first_read + NPL * FN) {
                const int j = i - first_read;
                b[1 - set][j / NPL][j % NPL] = *reinterpret_cast<const half8_t*>(lds + bbase[nbuf][j / NPL] + noff + (j % NPL) * G::PLANE);
            }
#pragma unroll
            for (int j = 0; j < NW; j++)   // the weight fragments of a step, spread over its slots
                if (i == ((j * NS) / NW + 1 < NS ? (j * NS) / NW + 1 : NS - 1))
                    a_q[dprev][j % 2][j / 2] = *reinterpret_cast<const half8_t*>(w_ + ((j % 2) * NPLW + j / 2) * 1024 + wlane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int TH, int TW, int WM>
__global__ __launch_bounds__(512) void tconv_p16_kernel(const ConvP16Params p) {
    using G = Geo<TH, TW, 1, WM, 1>;
    constexpr int FN = G::FN, CPB = G::CPB;
    constexpr int PDT = (FN >= 3) ? 3 : 6;
    static_assert((2 * NT) % PDT == 0, "two stages are whole turns of the weight ring");
    static_assert(2 * NPASS * FN >= (HSTORE ? 1 : 4) + NPL * FN, "the last step of a stage has room for the next stage's first fragments");
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ unsigned range_box[2];
    if (blockIdx.x == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bid = blockIdx.x;
    {
        const int nblk = p.pos_groups * p.cout_blocks;
        const int per = nblk >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    const int cb = bid % p.cout_blocks;
    const int group = bid / p.cout_blocks;
    const int ntiles = p.tiles_x * p.tiles_y;
    if (tid < 2) range_box[tid] = 0u;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    const int nchunks = p.cin_chunks;
    constexpr int sb_off = 2 * G::BUF;
    if (wave < 4) {
        p16_stager<G>(p, lds, tid & 255, cb, group, ntiles, nchunks, range_bits);
        return;
    }
    const int mq = lane & 15, kq = lane >> 4;
    const int mw = (wave - 4) % WM, wn = (wave - 4) / WM;
    int bbase[2][FN];
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = fn * 16 + mq;
        const int ty = m / TW, tx = m - ty * TW;
        bbase[0][fn] = ty * G::ROW_PITCH + (wn * TW + tx) * PITCH + kq * 16;
        bbase[1][fn] = bbase[0][fn] + G::BUF;
    }
    const unsigned wstep = (unsigned)p.mfrags * NPLW * 1024;
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)((cb * 2 * WM + mw * 2) * NPLW) * 1024;   // (uniform: the loads take it as their scalar base)
    const unsigned wlane = lane * 16;
    const unsigned char* wend = wbase + (size_t)nchunks * NT * wstep;
    half8_t a_q[PDT][2][NPL];
#pragma unroll
    for (int d = 0; d < PDT; d++)
#pragma unroll
        for (int fm = 0; fm < 2; fm++)
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) a_q[d][fm][pl] = *reinterpret_cast<const half8_t*>(wbase + (size_t)d * wstep + (fm * NPLW + pl) * 1024 + wlane);
    f32x4_t acc[4][2][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int par = 0; par < 4; par++)
#pragma unroll
            for (int fm = 0; fm < 2; fm++)
#pragma unroll
                for (int fn = 0; fn < FN; fn++) acc[par][fm][fn] = (f32x4_t)(0.f);
    };
    zero_acc();
    float inv_in_scale = 1.f;
    if (p.in_amax) (void)range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    store_t* out = reinterpret_cast<store_t*>(p.out);
    const bool through = store_through_pays(p.out, 2 * p.npos_y, 2 * p.npos_x, p.out_cp * ESZ, (p.cout_blocks == 1 || (CPB * ESZ) % 128 == 0) && !p.plain_stores, hw_block_count());
    bool drop = through && wave == 4 && hw_block_id() < 8;
    float vmax = 0.f;
    auto finish_tile = [&](int tile) {
        if (drop) {   // (ahead of this workgroup's first store: what it has read so far may go as well)
            drop_clean_l2_lines();
            drop = false;
        }
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const float* sb = reinterpret_cast<const float*>(lds + sb_off);
        f32x4_t bi[2], scm[2];
#pragma unroll
        for (int fm = 0; fm < 2; fm++) {
            scm[fm] = *reinterpret_cast<const f32x4_t*>(sb + mw * 32 + kq * CHK + fm * CHF) * acc_mul;
            bi[fm] = *reinterpret_cast<const f32x4_t*>(sb + CPB + mw * 32 + kq * CHK + fm * CHF);
        }
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            const int m = fn * 16 + mq;
            const int ty = m / TW, tx = wn * TW + (m - ty * TW);
            const int a = tyi * TH + ty, bx = txi * G::TWG + tx;
            const bool ok = a < p.npos_y && bx < p.npos_x;
            const size_t obase = ((size_t)(p.out_off_y + 2 * a) * p.out_wp + p.out_off_x + 2 * bx) * p.out_cp + cb * CPB + mw * 32 + kq * CHK;
            float fmax_ = 0.f;
#pragma unroll
            for (int par = 0; par < 4; par++) {
                const size_t o = obase + ((size_t)(par >> 1) * p.out_wp + (par & 1)) * p.out_cp;
                half8_t hv;
#pragma unroll
                for (int fm = 0; fm < 2; fm++) {
                    f32x4_t v;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        v[e] = acc[par][fm][fn][e] * scm[fm][e] + bi[fm][e];
                        if constexpr (!HSTORE) fmax_ = fmaxf(fmax_, fabsf(v[e]));
                    }
                    if constexpr (HSTORE) {
#pragma unroll
                        for (int e = 0; e < 4; e++) hv[fm * 4 + e] = (_Float16)v[e];
                        if (fm == 1 && ok) store_out(through, reinterpret_cast<half8_t*>(out + o), hv);
                    } else {
                        if (ok) store_out(through, reinterpret_cast<f32x4_t*>(out + o + fm * CHF), v);
                    }
                }
            }
            vmax = fmaxf(vmax, ok ? fmax_ : 0.f);
        }
    };
    lds_barrier();   // the first stage is staged
    half8_t b[2][FN][NPL];
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int pl = 0; pl < NPL; pl++) b[0][fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[0][fn] + G::ROW_PITCH + PITCH + pl * G::PLANE);
    const unsigned char* wnext = wbase + (size_t)((PDT - 1) % (nchunks * NT)) * wstep;
    int tile = group, c = 0;
    for (;;) {
        tp16_stage<G, 0, PDT>(acc, a_q, b, bbase, lds, wnext, wbase, wend, wstep, wlane);
        if (++c == nchunks) {
            finish_tile(tile);
            c = 0; tile += p.pos_groups;
            if (tile >= ntiles) break;
            zero_acc();
        }
        tp16_stage<G, 1, PDT>(acc, a_q, b, bbase, lds, wnext, wbase, wend, wstep, wlane);
        if (++c == nchunks) {
            finish_tile(tile);
            c = 0; tile += p.pos_groups;
            if (tile >= ntiles) break;
            zero_acc();
        }
    }
    if (p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 4);
}

// ---------------------------------------------------------------------------------------------------------------
// K x K convolution (K = 9) on an input of at most four channels (the first layer of a style-transfer net; replaces the
// render passes of DeepConvLayerNxN::forward, gpu/deep/deepconvlayerNxN.cpp:129-211, for such layers).  A staged pixel
// is four fp16 channels = 8 bytes per plane, so a lane's eight halves of a k32 step are two horizontally neighbouring
// taps: a kernel row is padded to (K+1)/2 tap pairs, a step takes four pairs in row-major order (45 pairs = 12 steps for
// 9x9, the last three pairs empty), and every lane keeps the LDS offset of its pair for each step in a register.  One
// group of 32 output channels, four tiles of positions side by side; a tile is one stage, walked as above.
template <int K, int TH_, int TW>
struct GeoC4 {
    static constexpr int TH = TH_, STEP = 1, WN = 4, TWG = 4 * TW;
    static constexpr int PPR = (K + 1) / 2, NPAIR = K * PPR;          // tap pairs per kernel row, in all
    // (the staged width covers the empty tap that pads an odd kernel row to whole pairs: its weight is zero, but the
    // pixel it is multiplied with must be a number)
    static constexpr int HW = TWG + 2 * PPR - 1, HH = TH + K - 1;
    static constexpr int NS = ((NPAIR + 3) / 4 + 2) / 3 * 3;          // steps per stage (two stages are whole turns of the weight ring)
    static constexpr int PIX = 8;                                     // bytes per staged pixel and plane
    static constexpr int ROW_PITCH = (HW * PIX + 15) / 16 * 16 + 16;
    // A plane is staged twice, the second copy eight bytes further on: the two pixels of a tap pair are then 16 aligned
    // bytes in one of the copies whatever the parity of the pair's first pixel, and a B fragment is one 16-byte LDS read
    // (with 8-byte reads the four tap pairs of a step meet in the same banks and the reads, not the MFMAs, set the pace:
    // 59 % MFMA issue inside the step loop).  The copies lie 64 bytes apart modulo the 128 of the banks: of eight
    // neighbouring positions the even ones read the first copy and the odd ones the second, all banks once.
    static constexpr int COPY = HH * ROW_PITCH;
    static constexpr int COPY2 = (COPY + 127) / 128 * 128 + 48;        // offset of the second copy (its pixel x at COPY2 + 8 + 8 x)
    static constexpr int PLANE = COPY2 + COPY + 16;
    static constexpr int BUF = NPL * PLANE;
    static constexpr int NPOS = TH * TW, FN = NPOS / 16;
    static constexpr int NITEMS = HH * HW;                            // staging items: pixels
    static constexpr int NB = (NITEMS + 255) / 256;
    static constexpr int CPB = 32;
    static_assert(NPOS % 16 == 0 && (2 * NS) % PD == 0, "whole position fragments; whole ring turns");
    static_assert(2 * BUF + PLANE < 65536, "offsets fit the LDS instructions' immediate field");
};

template <class G, bool C8>
__device__ __forceinline__ void c4_stager(const ConvP16Params& p, unsigned char* lds, int stid, int cb, int group, int ntiles, unsigned range_bits) {
    constexpr int sb_off = 2 * G::BUF;
    const store_t* in = reinterpret_cast<const store_t*>(p.in);
    int i_y[G::NB], i_x[G::NB], l_off[G::NB];
#pragma unroll
    for (int i = 0; i < G::NB; i++) {
        const int idx = stid + i * 256;
        l_off[i] = -1; i_y[i] = 1 << 20; i_x[i] = 0;
        if (idx < G::NITEMS) {
            const int py = idx / G::HW, px = idx - py * G::HW;
            i_y[i] = py; i_x[i] = px;
            l_off[i] = py * G::ROW_PITCH + px * G::PIX;
        }
    }
    int g_off[2][G::NB];
    typedef typename std::conditional<HSTORE, half4_t, float4>::type raw_t;   // a pixel as it comes from memory
    raw_t raw[2][G::NB];
    float in_scale = 1.f, inv_unused;
    auto fetch = [&](auto set_, int tile) {
        constexpr int SET = decltype(set_)::value;
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const int y0 = tyi * G::TH + p.in_y0, x0 = txi * G::TWG + p.in_x0;
#pragma unroll
        for (int i = 0; i < G::NB; i++) {
            int gy = y0 + i_y[i], gx = x0 + i_x[i];
            if (p.in_clamp && l_off[i] >= 0) {
                gy = min(max(gy, 0), p.in_hp - 1);
                gx = min(max(gx, 0), p.in_wp - 1);
            }
            g_off[SET][i] = ((unsigned)gy < (unsigned)p.in_hp && (unsigned)gx < (unsigned)p.in_wp) ? (gy * p.in_wp + gx) * 4 : -1;
            raw[SET][i] = *reinterpret_cast<const raw_t*>(in + (g_off[SET][i] >= 0 ? g_off[SET][i] : 0));
        }
    };
    const bool plain_act = p.act.kind == ACT_NONE;   // (a first layer reads its input as it is)
    auto store = [&](auto set_, unsigned char* buf) {
        constexpr int SET = decltype(set_)::value;
#pragma unroll
        for (int i = 0; i < G::NB; i++) {
            if (l_off[i] < 0) continue;
            const bool ok = g_off[SET][i] >= 0;
            if constexpr (HSTORE) {
                half4_t v;
                _Float16 hlo, hhi;
                if (act_half_exact(p.act, hlo, hhi)) {   // (on the packed halves, as in p16_stager)
                    v = ok ? act_half4(raw[SET][i], hlo, hhi) : (half4_t)((_Float16)0.f);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = ok ? (_Float16)act_p16((float)raw[SET][i][e], p.act) : (_Float16)0.f;
                }
                *reinterpret_cast<half4_t*>(buf + l_off[i]) = v;
                *reinterpret_cast<half4_t*>(buf + G::COPY2 + 8 + l_off[i]) = v;
            } else {
                // (the hi/lo split of a pair of values in four instructions, as in split8)
                const float r[4] = {raw[SET][i].x, raw[SET][i].y, raw[SET][i].z, raw[SET][i].w};
                float x[4];
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] = ok ? (plain_act ? r[e] : act_p16(r[e], p.act)) : 0.f;
                unsigned h0, l0, h1, l1;
                split_pair(x[0], x[1], in_scale, h0, l0);
                split_pair(x[2], x[3], in_scale, h1, l1);
                const half4_t hi = __builtin_bit_cast(half4_t, uint2{h0, h1}), lo = __builtin_bit_cast(half4_t, uint2{l0, l1});
                *reinterpret_cast<half4_t*>(buf + l_off[i]) = hi;
                *reinterpret_cast<half4_t*>(buf + G::COPY2 + 8 + l_off[i]) = hi;
                if constexpr (C8) {
                    // the pixel's fp8 operands of the correction terms: [4 x fp8(32 lo) | 4 x fp8(hi / 64)]
                    const int2 c8 = int2{(int)c8_quad(lo[0], lo[1], lo[2], lo[3], 0.03125f), (int)c8_quad(hi[0], hi[1], hi[2], hi[3], 64.f)};
                    *reinterpret_cast<int2*>(buf + G::PLANE + l_off[i]) = c8;
                    *reinterpret_cast<int2*>(buf + G::PLANE + G::COPY2 + 8 + l_off[i]) = c8;
                } else {
                    *reinterpret_cast<half4_t*>(buf + G::PLANE + l_off[i]) = lo;
                    *reinterpret_cast<half4_t*>(buf + G::PLANE + G::COPY2 + 8 + l_off[i]) = lo;
                }
            }
        }
    };
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;
    int tile = group;                       // the stage the MFMA waves are on
    int t1 = tile + p.pos_groups, t2 = t1 + p.pos_groups;
    fetch(Set0(), tile);
    if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_unused);
    if (stid < 32) {   // (scale and bias have one entry per channel of the output tensor's pitch)
        const bool have = cb * 32 + stid < p.out_cp;
        reinterpret_cast<float*>(lds + sb_off)[stid] = have ? p.scale[cb * 32 + stid] : 0.f;
        reinterpret_cast<float*>(lds + sb_off)[32 + stid] = have ? p.bias[cb * 32 + stid] : 0.f;
    }
    store(Set0(), lds);
    lds_barrier();
    if (t1 < ntiles) fetch(Set1(), t1);
    auto iteration = [&](auto next_set, auto free_set, unsigned char* next_buf) {
        if (t1 < ntiles) store(next_set, next_buf);
        if (t2 < ntiles) fetch(free_set, t2);
        lds_barrier();
        const bool go_on = t1 < ntiles;
        tile = t1; t1 = t2; t2 += p.pos_groups;
        return go_on;
    };
    for (;;) {
        if (!iteration(Set1(), Set0(), lds + G::BUF)) break;
        if (!iteration(Set0(), Set1(), lds)) break;
    }
}

template <class G, int BUFI>
__device__ __forceinline__ void c4_stage(f32x4_t (&acc)[2][G::FN], half8_t (&a_q)[PD][2][NPL], half8_t (&b)[G::FN][NPL], const int (&bbase)[G::FN],
                                         const int (&off)[G::NS], const unsigned char* lds, const unsigned char*& wnext,
                                         const unsigned char* wbase, const unsigned char* wend, unsigned wstep, unsigned wlane) {
    constexpr int FN = G::FN, NS = G::NS;
#pragma unroll
    for (int dd = 0; dd < NS; dd++) {
        const int d = (BUFI * NS + dd) % PD, dprev = (d + PD - 1) % PD;
        const int nbuf = (dd + 1 == NS) ? 1 - BUFI : BUFI, ns = (dd + 1) % NS;
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
        constexpr int SL = 2 * NPASS, NSL = SL * FN, NW = 2 * NPL;
#pragma unroll
        for (int i = 0; i < NSL; i++) {
            const int fn = i / SL, r = i % SL, kind = r / 2, fm = r % 2;
            const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_q[d][fm][apl], b[fn][bpl], acc[fm][fn], 0, 0, 0);
            if (dd == NS - 1 && i == (SL - 1 < 3 ? SL - 1 : 3)) lds_barrier();
            if (r == SL - 1) {
                const unsigned char* src = lds + nbuf * G::BUF + bbase[fn] + off[ns];
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) b[fn][pl] = *reinterpret_cast<const half8_t*>(src + pl * G::PLANE);
            }
#pragma unroll
            for (int j = 0; j < NW; j++)
                if (i == ((j * NSL) / NW + 1 < NSL ? (j * NSL) / NW + 1 : NSL - 1))
                    a_q[dprev][j % 2][j / 2] = *reinterpret_cast<const half8_t*>(w_ + ((j % 2) * NPLW + j / 2) * 1024 + wlane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The same stage with the correction terms as fp8 matrix instructions (see p16_stage_c8).  The second staged plane holds
// per pixel [4 x fp8(32 lo) | 4 x fp8(hi / 64)], the third weight plane per tap [4 x fp8(hi / 32) | 4 x fp8(64 lo)]; one
// v_mfma_f32_16x16x128_f8f6f4 takes the tap pairs of two consecutive steps.  Per pair of steps and fragment pair:
// four fp16 MFMAs and two fp8 ones, 128 matrix-pipe cycles instead of 192.  The stage has an even number of steps, so
// its last step is a pair step and the stage's barrier sits behind that step's first fp8 MFMA.
template <class G, int BUFI>
__device__ __forceinline__ void c4_stage_c8(f32x4_t (&acc)[2][G::FN], half8_t (&a0)[PD][2], i32x8_t (&a2)[PD / 2][2], half8_t (&b0)[G::FN], i32x8_t (&b1)[G::FN],
                                            const int (&bbase)[G::FN], const int (&off)[G::NS], const unsigned char* lds, const unsigned char*& wnext,
                                            const unsigned char* wbase, const unsigned char* wend, unsigned wstep, unsigned wlane) {
    constexpr int FN = G::FN, NS = G::NS;
    static_assert(NS % 2 == 0 && PD % 2 == 0, "pairs of steps");
#pragma unroll
    for (int dd = 0; dd < NS; dd++) {
        const int d = (BUFI * NS + dd) % PD, dprev = (d + PD - 1) % PD;
        const bool pair = (dd & 1) != 0;
        const int nbuf = (dd + 1 == NS) ? 1 - BUFI : BUFI, ns = (dd + 1) % NS;
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
        // weights of step s + PD - 1 into the ring slot of step s - 1; every position fragment's operands of step s + 1
        auto load_a0 = [&](int fm) { a0[dprev][fm] = *reinterpret_cast<const half8_t*>(w_ + (fm * NPLW) * 1024 + wlane); };
        auto load_a2 = [&](int fm) {
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(w_ + (fm * NPLW + 2) * 1024 + wlane);
            if ((dprev & 1) == 0) { a2[dprev / 2][fm][0] = v[0]; a2[dprev / 2][fm][1] = v[1]; a2[dprev / 2][fm][2] = v[2]; a2[dprev / 2][fm][3] = v[3]; }
            else { a2[dprev / 2][fm][4] = v[0]; a2[dprev / 2][fm][5] = v[1]; a2[dprev / 2][fm][6] = v[2]; a2[dprev / 2][fm][7] = v[3]; }
        };
        auto load_b0 = [&](int fn) { b0[fn] = *reinterpret_cast<const half8_t*>(lds + nbuf * G::BUF + bbase[fn] + off[ns]); };
        auto load_b1 = [&](int fn) {
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(lds + nbuf * G::BUF + bbase[fn] + off[ns] + G::PLANE);
            if (pair) { b1[fn][0] = v[0]; b1[fn][1] = v[1]; b1[fn][2] = v[2]; b1[fn][3] = v[3]; }   // (the next step opens a pair)
            else { b1[fn][4] = v[0]; b1[fn][5] = v[1]; b1[fn][6] = v[2]; b1[fn][7] = v[3]; }
        };
        if (pair) {
#pragma unroll
            for (int i = 0; i < 2 * FN; i++) {
                const int fn = i / 2, fm = i % 2;
                acc[fm][fn] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a2[d / 2][fm], b1[fn], acc[fm][fn], 0, 0, 0, 0, 0, 0);
                if (dd == NS - 1 && i == 0) lds_barrier();
                if (fm == 1) load_b1(fn);
                if (i == 0) load_a0(0);
                if (i == FN) load_a0(1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int i = 0; i < 2 * FN; i++) {
            const int fn = i / 2, fm = i % 2;
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0[d][fm], b0[fn], acc[fm][fn], 0, 0, 0);
            if (fm == 1) {
                load_b0(fn);
                if (!pair) load_b1(fn);
            }
            if (pair) {
                if (i == 0) load_a2(0);
                if (i == FN) load_a2(1);
            } else {
                if (i == 0) load_a0(0);
                if (i == FN / 2) load_a0(1);
                if (i == FN) load_a2(0);
                if (i == FN + FN / 2) load_a2(1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int K, int TH, int TW, bool C8>
__global__ __launch_bounds__(512) void conv_p16c4_kernel(const ConvP16Params p) {
    using G = GeoC4<K, TH, TW>;
    constexpr int FN = G::FN, NS = G::NS;
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ unsigned range_box[2];
    if (blockIdx.x == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bid = blockIdx.x;
    {
        const int nblk = p.pos_groups * p.cout_blocks;
        const int per = nblk >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    const int cb = bid % p.cout_blocks;
    const int group = bid / p.cout_blocks;
    const int ntiles = p.tiles_x * p.tiles_y;
    if (tid < 2) range_box[tid] = 0u;
    const unsigned range_bits = p.in_amax ? range_load(p.in_amax) : 0u;
    constexpr int sb_off = 2 * G::BUF;
    if (wave < 4) {
        c4_stager<G, C8>(p, lds, tid & 255, cb, group, ntiles, range_bits);
        return;
    }
    const int mq = lane & 15, kq = lane >> 4;
    const int wn = wave - 4;
    int bbase[FN];
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = fn * 16 + mq;
        const int ty = m / TW, tx = m - ty * TW;
        const int x = wn * TW + tx;   // (a tap pair starts an even number of pixels from its position: the position's parity picks the copy)
        bbase[fn] = ty * G::ROW_PITCH + x * G::PIX + ((x & 1) ? G::COPY2 + 8 : 0);
    }
    int off[NS];   // LDS offset of this lane's tap pair in each step (pairs beyond the kernel: pair 0, their weights are zero)
#pragma unroll
    for (int st = 0; st < NS; st++) {
        const int pi = 4 * st + kq;
        const int row = pi / G::PPR, col = 2 * (pi - row * G::PPR);
        off[st] = pi < G::NPAIR ? row * G::ROW_PITCH + col * G::PIX : 0;
    }
    const unsigned wstep = (unsigned)p.mfrags * NPLW * 1024;
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)(cb * 2 * NPLW) * 1024;   // (uniform: the loads take it as their scalar base)
    const unsigned wlane = lane * 16;
    const unsigned char* wend = wbase + (size_t)NS * wstep;
    // weight ring: fp16 planes (hi, lo), or with the fp8 form the hi plane and the fp8 plane in pairs of steps
    half8_t a_q[PD][2][C8 ? 1 : NPL];
    half8_t a0[C8 ? PD : 1][2];
    i32x8_t a2[C8 ? PD / 2 : 1][2];
#pragma unroll
    for (int d = 0; d < PD; d++)
#pragma unroll
        for (int fm = 0; fm < 2; fm++) {
            const unsigned char* wf = wbase + (size_t)(d % NS) * wstep + (fm * NPLW) * 1024 + wlane;   // (a stage of fewer steps than the ring holds: the next tile's)
            if constexpr (C8) {
                a0[d][fm] = *reinterpret_cast<const half8_t*>(wf);
                const i32x4_t v = *reinterpret_cast<const i32x4_t*>(wf + 2 * 1024);
#pragma unroll
                for (int e = 0; e < 4; e++) a2[d / 2][fm][(d & 1) * 4 + e] = v[e];
            } else {
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a_q[d][fm][pl] = *reinterpret_cast<const half8_t*>(wf + pl * 1024);
            }
        }
    f32x4_t acc[2][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int fm = 0; fm < 2; fm++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++) acc[fm][fn] = (f32x4_t)(0.f);
    };
    zero_acc();
    float inv_in_scale = 1.f;
    if (p.in_amax) (void)range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    store_t* out = reinterpret_cast<store_t*>(p.out);
    const bool through = store_through_pays(p.out, p.npos_y, p.npos_x, p.out_cp * ESZ, (p.cout_blocks == 1 || (32 * ESZ) % 128 == 0) && !p.plain_stores, hw_block_count());
    bool drop = through && wave == 4 && hw_block_id() < 8;
    float vmax = 0.f;
    auto finish_tile = [&](int tile) {
        if (drop) {   // (ahead of this workgroup's first store: what it has read so far may go as well)
            drop_clean_l2_lines();
            drop = false;
        }
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const float* sb = reinterpret_cast<const float*>(lds + sb_off);
        f32x4_t bi[2], scm[2];
#pragma unroll
        for (int fm = 0; fm < 2; fm++) {
            scm[fm] = *reinterpret_cast<const f32x4_t*>(sb + kq * CHK + fm * CHF) * acc_mul;
            bi[fm] = *reinterpret_cast<const f32x4_t*>(sb + 32 + kq * CHK + fm * CHF);
        }
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            const int m = fn * 16 + mq;
            const int ty = m / TW, tx = wn * TW + (m - ty * TW);
            const int py = tyi * TH + ty, px = txi * G::TWG + tx;
            const bool inside = py < p.npos_y && px < p.npos_x;
            const size_t obase = ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp + cb * 32 + kq * CHK;
            float fmax_ = 0.f;
            half8_t hv;
#pragma unroll
            for (int fm = 0; fm < 2; fm++) {
                // (the block of 32 output channels may reach behind the tensor's channel pitch: those groups are not stored)
                const bool ok = inside && cb * 32 + kq * CHK + (HSTORE ? 0 : fm * CHF) < p.out_cp;
                f32x4_t v;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[e] = acc[fm][fn][e] * scm[fm][e] + bi[fm][e];
                    if constexpr (!HSTORE) fmax_ = fmaxf(fmax_, ok ? fabsf(v[e]) : 0.f);
                }
                if constexpr (HSTORE) {
#pragma unroll
                    for (int e = 0; e < 4; e++) hv[fm * 4 + e] = (_Float16)v[e];
                    if (fm == 1 && ok) store_out(through, reinterpret_cast<half8_t*>(out + obase), hv);
                } else {
                    if (ok) store_out(through, reinterpret_cast<f32x4_t*>(out + obase + fm * CHF), v);
                }
            }
            vmax = fmaxf(vmax, fmax_);
        }
    };
    lds_barrier();   // the first stage is staged
    half8_t b[C8 ? 1 : FN][NPL];   // exact form: hi and lo fragments of a step
    half8_t b0[C8 ? FN : 1];       // fp8 form: hi fragments ...
    i32x8_t b1[C8 ? FN : 1];       // ... and the fp8 fragments of a pair of steps
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        if constexpr (C8) {
            b0[fn] = *reinterpret_cast<const half8_t*>(lds + bbase[fn] + off[0]);
            const i32x4_t v = *reinterpret_cast<const i32x4_t*>(lds + bbase[fn] + off[0] + G::PLANE);
#pragma unroll
            for (int e = 0; e < 4; e++) b1[fn][e] = v[e];
        } else {
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) b[fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[fn] + off[0] + pl * G::PLANE);
        }
    }
    const unsigned char* wnext = wbase + (size_t)((PD - 1) % NS) * wstep;
    int tile = group;
    auto stage = [&](auto bufi) {
        constexpr int BUFI = decltype(bufi)::value;
        if constexpr (C8) {
            c4_stage_c8<G, BUFI>(acc, a0, a2, b0, b1, bbase, off, lds, wnext, wbase, wend, wstep, wlane);
        } else {
            c4_stage<G, BUFI>(acc, a_q, b, bbase, off, lds, wnext, wbase, wend, wstep, wlane);
        }
    };
    for (;;) {
        stage(std::integral_constant<int, 0>());
        finish_tile(tile);
        tile += p.pos_groups;
        if (tile >= ntiles) break;
        zero_acc();
        stage(std::integral_constant<int, 1>());
        finish_tile(tile);
        tile += p.pos_groups;
        if (tile >= ntiles) break;
        zero_acc();
    }
    if (p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 4);
}

// ---------------------------------------------------------------------------------------------------------------
// 1x1 and 3x3 convolutions (stride 1) on layers with few positions and many input channels (the last stages of a
// classification net at batch 1: 14x14 or 7x7 positions, 256 to 1024 input channels).  There the general kernel cuts
// the reduction into slices for separate workgroups and sums them in a second launch.  Here a workgroup owns a tile of
// 4x4 positions and 16*FM output channels and keeps the tile's whole reduction resident in LDS: the staging waves fetch
// all 4*CPW chunks of 32 channels at once (one memory round trip), the four MFMA waves take every fourth chunk each --
// a stream of CPW*NTAPS steps, fully unrolled, weights through a register ring, B fragments read three steps ahead --
// and add their accumulators through LDS; wave 0 runs the epilogue.  Small tiles make many workgroups (13 tiles x 16
// blocks of 16 channels for 1024 -> 256 at 14x14), so the layer's activations and weights are pulled through many CUs.
// Weights: [cout block][wave][step][fragment][plane][lane][8 halves], the wave's steps being (chunk wave + 4*i, tap).
template <int NTAPS, int CPW, int FN_ = 1, int S_ = 1>
struct GeoR {
    static constexpr int FN = FN_;                      // position fragments per tile: 4x4, 4x8 or 8x8 positions
    static constexpr int S = S_;                        // stride of a 3x3 layer (a 1x1 layer's stride is a launch parameter: it only thins the pixels fetched)
    static constexpr int TH = (FN == 4) ? 8 : 4, TW = (FN == 1) ? 4 : 8, KH = (NTAPS == 9) ? 2 : 0;
    static_assert(FN == 1 || FN == 2 || FN == 4, "tiles of 16, 32 or 64 positions");
    static_assert(S == 1 || (S == 2 && NTAPS == 9), "stride 2 for 3x3");
    static constexpr int HW = S * (TW - 1) + 1 + KH, HH = S * (TH - 1) + 1 + KH;
    static constexpr int NCH = 4 * CPW;                 // chunks of the layer
    // (64 chunks -- 2048 input channels -- fit the LDS only without the padding that keeps the fragment reads free of
    // bank conflicts; the reads are a small part of this kernel)
    static constexpr int PIT = (NCH > 32) ? KC * 2 : PITCH;
    static constexpr int ROW_PITCH = HW * PIT + ((NCH > 32) ? 0 : p16_row_pad(TH, TW, 1, 1, HW));
    static constexpr int PLANE = HH * ROW_PITCH;
    static constexpr int BUFC = NPL * PLANE;            // one chunk of the tile
    static constexpr int NITEMS = HH * HW * (KC / 8);   // staging items per chunk
    static constexpr int TOTAL = NITEMS * NCH, NB = (TOTAL + 255) / 256;
    static constexpr int STEPS = CPW * NTAPS;           // per MFMA wave
    static constexpr int RPD = STEPS < 8 ? STEPS : 8;   // weight ring depth (steps; the step loop is unrolled, so any depth fits)
    static constexpr int BD = FN > 1 ? (STEPS < 2 ? STEPS : 2) : (STEPS < 4 ? STEPS : 4);    // B fragment ring depth (steps)
    static constexpr int RED_OFF = NCH * BUFC;          // [wave 1..3][fragment][lane] x 16 bytes, then scale and bias
    static constexpr int tap_off(int t) { return NTAPS == 9 ? (t / 3) * ROW_PITCH + (t % 3) * PIT : 0; }
    static_assert(NTAPS == 1 || NTAPS == 9, "1x1 or 3x3");
};

// DWS = 1 or 2: the input of a 1x1 layer is not read from memory but computed by the staging waves: it is the output of
// a depthwise 3x3 layer with step DWS (weights fp32, folded scale and bias, the arithmetic and the rounding to the
// storage type of the depthwise kernel in layers_direct.hip), whose tensor then never exists.  A staging item is a pair
// of horizontally neighbouring positions and 8 channels: 3 x (DWS + 3) texels of the depthwise layer's input.
#ifndef FYN_KR_STAGE_WAVES
#define FYN_KR_STAGE_WAVES 8
#endif
template <int NTAPS, int CPW, int FM, int FN, int S, int DWS = 0, int R = 1, int SRC = 0>
__global__ __launch_bounds__(512) void conv_kr16_kernel(const ConvP16Params p) {
    // SRC: 0 = the plain layer; 1 = a batch-norm layer in front applied while staging (p.in_mul, p.in_add); 2 = a reduction
    // over two tensors (p.in2...).  Kernels of their own, so that the plain one carries none of their instructions.
    static_assert(SRC == 0 || (NTAPS == 1 && FN == 1 && S == 1 && DWS == 0 && R == 1), "batch-norm in front / two tensors: 1x1, tiles of 4x4 positions, one round");
    // R > 1: the reduction passes through the LDS in R rounds of 4 * CPW chunks each (layers whose whole reduction does
    // not fit: 3x3 with stride 2 on 512 channels needs 166 KB).  The staging waves request round r + 1 while the MFMA
    // waves work on round r and write it once those are through.
    using G = GeoR<NTAPS, CPW, FN, S>;
    static_assert(DWS == 0 || (NTAPS == 1 && FN == 1 && S == 1 && DWS <= 2), "a fused depthwise layer: 1x1, tiles of 4x4 positions");
    static_assert(R >= 1 && (R == 1 || DWS == 0), "rounds: without a depthwise layer in the staging");
    constexpr int RPD = G::RPD, BD = G::BD, STEPS = G::STEPS;
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ unsigned range_box[2];
    if ((blockIdx.x | blockIdx.y | blockIdx.z) == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (a grid of output-channel blocks x tile columns x tile rows: no division stands between the kernel's start and its
    // first request; consecutive workgroups are the channel blocks of one tile)
    const int cb = blockIdx.x, txi = blockIdx.y, tyi = blockIdx.z;
    if (tid < 2) range_box[tid] = 0u;
    // (two source tensors: the larger of their value ranges scales both, or nothing is scaled when one keeps no word)
    const bool ranged = p.in_amax && (SRC != 2 || p.in2_amax);
    // (both loads are issued here and met where the scale is computed: nothing waits for them in between)
    const unsigned range_bits1 = ranged ? range_load(p.in_amax) : 0u;
    const unsigned range_bits2 = (SRC == 2 && ranged) ? range_load(p.in2_amax) : 0u;
    auto range_word = [&]() { return max(range_bits1, range_bits2); };
    constexpr int red_off = G::RED_OFF;
    constexpr int sb_off = red_off + 3 * FM * FN * 1024;
    // Staging waves: the four that only stage, and -- without a depthwise layer in front -- the four MFMA waves too,
    // after they have requested their weights: conversion and address arithmetic of the tile split eight ways.
    constexpr int SW = (DWS > 0 || R > 1) ? 4 : FYN_KR_STAGE_WAVES, NTH = SW * 64;

    // The tile's staging: every thread of the SW staging waves takes the items stid, stid + NTH, ...
    struct RawF { float4 a, b; };
    typedef typename std::conditional<HSTORE, half8_t, RawF>::type raw_t;
    auto stage_tile = [&](const int stid, const int round, const bool wait) {
        const int ch_r = round * G::NCH * KC;   // the round's first channel
        constexpr int NB = (G::TOTAL + NTH - 1) / NTH;
        const store_t* in = reinterpret_cast<const store_t*>(p.in);
        raw_t raw[NB];
        int l_off[NB];
        int ch_of[NB];   // the item's first channel
        bool ok[NB];
        // (a 1x1 layer may step over the input: position (y, x) reads pixel (y, x) * stride)
        // (a 3x3 layer with stride 2 stages every pixel under its tile: position (y, x) reads the window at (2y, 2x))
        const int st = NTAPS == 1 ? p.stride : 1, org = NTAPS == 1 ? p.stride : S;
        const int y0 = tyi * G::TH * org + p.in_y0, x0 = txi * G::TW * org + p.in_x0;
        if constexpr (NTH % G::NITEMS == 0) {
            // A chunk's items divide the staging threads (1x1 layers): a thread keeps its pixel and its 8 channels
            // of the chunk for all its items and only the chunk advances, by CPI per item -- the pixel's arithmetic is
            // done once, not once per item (a thread has up to 16 items, and nothing is requested before it is through).
            constexpr int CPI = NTH / G::NITEMS;
            const int chunk0 = stid / G::NITEMS, rem = stid - chunk0 * G::NITEMS;
            const int pix = rem >> 2, g = rem & 3;
            const int py = pix / G::HW, px = pix - py * G::HW;
            int gy = y0 + py * st, gx = x0 + px * st;
            if (p.in_clamp) {
                gy = min(max(gy, 0), p.in_hp - 1);
                gx = min(max(gx, 0), p.in_wp - 1);
            }
            const bool inb = (unsigned)gy < (unsigned)p.in_hp && (unsigned)gx < (unsigned)p.in_wp;
            const int l0 = chunk0 * G::BUFC + py * G::ROW_PITCH + px * G::PIT + g * 16;
            const int c0 = ch_r + chunk0 * KC + g * 8;
            const store_t* src0 = in + (inb ? (gy * p.in_wp + gx) * p.in_cp : 0) + c0;
            // the second source tensor (1x1 layers): the same pixel of the tile at that tensor's own step, origin and pitch
            [[maybe_unused]] bool inb2 = false;
            [[maybe_unused]] const store_t* src2 = in;
            [[maybe_unused]] int c2 = 0;
            if constexpr (SRC == 2) {
                {
                    const int gy2 = (tyi * G::TH + py) * p.in2_stride + p.in2_y0, gx2 = (txi * G::TW + px) * p.in2_stride + p.in2_x0;
                    inb2 = (unsigned)gy2 < (unsigned)p.in2_hp && (unsigned)gx2 < (unsigned)p.in2_wp;
                    c2 = (chunk0 - p.in2_chunk0) * KC + g * 8;   // (negative for the chunks of the first tensor)
                    src2 = reinterpret_cast<const store_t*>(p.in2) + (inb2 ? (gy2 * p.in2_wp + gx2) * p.in2_cp : 0) + c2;
                }
            }
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const bool in_tile = chunk0 + i * CPI < G::NCH;
                l_off[i] = in_tile ? l0 + i * CPI * G::BUFC : -1;
                // (channels behind the tensor's pitch -- the chunk count is rounded up to four per wave -- read as zero)
                ok[i] = in_tile && inb && c0 + i * CPI * KC < p.in_cp;
                ch_of[i] = c0 + i * CPI * KC;
                const store_t* src = ok[i] ? src0 + i * CPI * KC : in;
                if constexpr (SRC == 2) {
                    if (chunk0 + i * CPI >= p.in2_chunk0) {
                        ok[i] = in_tile && inb2 && c2 + i * CPI * KC < p.in2_cp;
                        src = ok[i] ? src2 + i * CPI * KC : in;
                    }
                }
                if constexpr (HSTORE) {
                    raw[i] = *reinterpret_cast<const half8_t*>(src);
                } else {
                    raw[i].a = *reinterpret_cast<const float4*>(src);
                    raw[i].b = *reinterpret_cast<const float4*>(src + 4);
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int idx = stid + i * NTH;
            const int chunk = idx / G::NITEMS, rem = idx - chunk * G::NITEMS;
            const int pix = rem >> 2, g = rem & 3;
            const int py = pix / G::HW, px = pix - py * G::HW;
            l_off[i] = idx < G::TOTAL ? chunk * G::BUFC + py * G::ROW_PITCH + px * G::PIT + g * 16 : -1;
            int gy = y0 + py * st, gx = x0 + px * st;
            if (p.in_clamp) {
                gy = min(max(gy, 0), p.in_hp - 1);
                gx = min(max(gx, 0), p.in_wp - 1);
            }
            // (channels behind the tensor's pitch -- the chunk count is rounded up to four per wave -- read as zero)
            ok[i] = idx < G::TOTAL && (unsigned)gy < (unsigned)p.in_hp && (unsigned)gx < (unsigned)p.in_wp && ch_r + chunk * KC + g * 8 < p.in_cp;
            ch_of[i] = ch_r + chunk * KC + g * 8;
            const store_t* src = in + (ok[i] ? (gy * p.in_wp + gx) * p.in_cp + ch_r + chunk * KC + g * 8 : 0);
            if constexpr (HSTORE) {
                raw[i] = *reinterpret_cast<const half8_t*>(src);
            } else {
                raw[i].a = *reinterpret_cast<const float4*>(src);
                raw[i].b = *reinterpret_cast<const float4*>(src + 4);
            }
        }
        }
        float in_scale = 1.f, inv_unused;
        if (ranged) in_scale = range_scale(range_after_act(range_reduce(range_word()), p.act), &inv_unused);
        // (fp16 tensors: no activation, or a clamp without leak whose bounds are fp16 values, is applied to the packed
        // halves -- two values per instruction, no conversions)
        _Float16 hlo, hhi;
        const bool half_act = act_half_exact(p.act, hlo, hhi) && HSTORE;
        // a batch-norm layer in front: x * in_mul[c] + in_add[c] on the item's eight channels (the arrays come through the L1)
        auto affine8 = [&](float (&x)[8], const int i) {
            const int c = ok[i] ? ch_of[i] : 0;
            const float4 m0 = *reinterpret_cast<const float4*>(p.in_mul + c), m1 = *reinterpret_cast<const float4*>(p.in_mul + c + 4);
            const float4 a0 = *reinterpret_cast<const float4*>(p.in_add + c), a1 = *reinterpret_cast<const float4*>(p.in_add + c + 4);
            const float m[8] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w}, a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = x[e] * m[e] + a[e];
        };
        if (wait) lds_barrier();   // the MFMA waves are through with the round before: its place in the LDS is free
        // (with or without the batch-norm layer: chosen once, outside the loops over the items)
        [[maybe_unused]] auto store_halves = [&](auto aff_) {
        constexpr bool AFF = decltype(aff_)::value;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            if (l_off[i] < 0) continue;
            if constexpr (HSTORE) {
                half8_t rv = raw[i];
                if constexpr (AFF) {
                    float x[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) x[e] = (float)rv[e];
                    affine8(x, i);
#pragma unroll
                    for (int e = 0; e < 8; e++) rv[e] = (_Float16)x[e];   // (what the batch-norm layer would have stored)
                }
                half8_t v;
                if (half_act) {
                    v = ok[i] ? act_half(rv, hlo, hhi) : (half8_t)((_Float16)0.f);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] = ok[i] ? (_Float16)act_p16((float)rv[e], p.act) : (_Float16)0.f;
                }
                *reinterpret_cast<half8_t*>(lds + l_off[i]) = v;
            }
        }
        };
        if constexpr (HSTORE) store_halves(std::integral_constant<bool, SRC == 1>());
        if constexpr (!HSTORE) {
            auto split_all = [&](auto kind_, auto aff_) {
                constexpr int KIND = decltype(kind_)::value;
                constexpr bool AFF = decltype(aff_)::value;
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    if (l_off[i] < 0) continue;
                    float r[8] = {raw[i].a.x, raw[i].a.y, raw[i].a.z, raw[i].a.w, raw[i].b.x, raw[i].b.y, raw[i].b.z, raw[i].b.w};
                    if constexpr (AFF) affine8(r, i);
                    half8_t hi, lo;
                    split8<KIND>(r, ok[i], p.act, in_scale, hi, lo);
                    *reinterpret_cast<half8_t*>(lds + l_off[i]) = hi;
                    *reinterpret_cast<half8_t*>(lds + G::PLANE + l_off[i]) = lo;
                }
            };
            constexpr std::integral_constant<bool, SRC == 1> aff;
            if (p.act.kind == ACT_NONE) split_all(std::integral_constant<int, ACT_NONE>(), aff);
            else if (p.act.kind == ACT_RELU) split_all(std::integral_constant<int, ACT_RELU>(), aff);
            else split_all(std::integral_constant<int, ACT_LEAKY>(), aff);
        }
    };

    if (wave < 4) {   // ------------------------------------------------------------ staging waves
        const int stid = tid & 255;
        if constexpr (DWS > 0) {
            constexpr int WINW = DWS + 3;
            constexpr int TOTAL = G::NCH * 32, NB = (TOTAL + 255) / 256;
            constexpr int IPP_MAX = (HSTORE && !(DWS == 2 && NB > 1)) ? 2 : 1;   // items whose texels are in flight together (registers)
            constexpr int IPP = NB < IPP_MAX ? NB : IPP_MAX;
            const store_t* din = reinterpret_cast<const store_t*>(p.dw_in);
            float in_scale = 1.f, inv_unused;
            if (p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_word()), p.act), &inv_unused);
            if (stid < 16 * FM) {
                reinterpret_cast<float*>(lds + sb_off)[stid] = p.scale[cb * 16 * FM + stid];
                reinterpret_cast<float*>(lds + sb_off)[16 * FM + stid] = p.bias[cb * 16 * FM + stid];
            }
            // (a clamp that is exact on halves is applied to the packed halves, as in the depthwise kernel)
            const _Float16 hlo = (_Float16)p.dw_act.lo, hhi = (_Float16)p.dw_act.hi;
            const bool packed_act = HSTORE && p.dw_act.leak == 0.f && (float)hlo == p.dw_act.lo && (float)hhi == p.dw_act.hi;
#pragma unroll
            for (int i0 = 0; i0 < NB; i0 += IPP) {
                raw_t raw[IPP][3][WINW];
                unsigned okm[IPP];
#pragma unroll
                for (int ii = 0; ii < IPP; ii++) {
                    if (i0 + ii >= NB) continue;
                    const int idx = stid + (i0 + ii) * 256;
                    const int chunk = idx >> 5, pair = (idx >> 2) & 7, g = idx & 3;
                    const int oy = tyi * 4 + (pair >> 1), ox = txi * 4 + (pair & 1) * 2;
                    const int ch = chunk * KC + g * 8;
                    const bool chan_ok = idx < TOTAL && ch < p.dw_cp;
                    okm[ii] = 0u;
#pragma unroll
                    for (int r = 0; r < 3; r++)
#pragma unroll
                        for (int c = 0; c < WINW; c++) {
                            const int iy = oy * DWS + r + p.dw_y0, ix = ox * DWS + c + p.dw_x0;
                            const bool ok = chan_ok && (unsigned)iy < (unsigned)p.dw_hp && (unsigned)ix < (unsigned)p.dw_wp;
                            okm[ii] |= ok ? 1u << (r * WINW + c) : 0u;
                            const store_t* src = din + (ok ? (iy * p.dw_wp + ix) * p.dw_cp + ch : 0);
                            if constexpr (HSTORE) {
                                raw[ii][r][c] = *reinterpret_cast<const half8_t*>(src);
                            } else {
                                raw[ii][r][c].a = *reinterpret_cast<const float4*>(src);
                                raw[ii][r][c].b = *reinterpret_cast<const float4*>(src + 4);
                            }
                        }
                }
#pragma unroll
                for (int ii = 0; ii < IPP; ii++) {
                    if (i0 + ii >= NB) continue;
                    const int idx = stid + (i0 + ii) * 256;
                    if (idx >= TOTAL) continue;
                    const int chunk = idx >> 5, pair = (idx >> 2) & 7, g = idx & 3;
                    const int ch = chunk * KC + g * 8;
                    const bool chan_ok = ch < p.dw_cp;
                    const int wch = chan_ok ? ch : 0;
                    float acc[2][8];
#pragma unroll
                    for (int j = 0; j < 2; j++)
#pragma unroll
                        for (int e = 0; e < 8; e++) acc[j][e] = 0.f;
#pragma unroll
                    for (int r = 0; r < 3; r++) {
                        // (a texel outside the stored frame is a zero that the activation is applied to, as in the depthwise kernel)
                        float row[WINW][8];
#pragma unroll
                        for (int c = 0; c < WINW; c++) {
                            const bool ok = (okm[ii] >> (r * WINW + c)) & 1u;
                            float x[8];
                            if constexpr (HSTORE) {
                                if (packed_act) {
                                    half8_t h = ok ? raw[ii][r][c] : (half8_t)((_Float16)0.f);
                                    h = __builtin_elementwise_min(__builtin_elementwise_max(h, (half8_t)hlo), (half8_t)hhi);
#pragma unroll
                                    for (int e = 0; e < 8; e++) row[c][e] = (float)h[e];
                                    continue;
                                }
#pragma unroll
                                for (int e = 0; e < 8; e++) x[e] = (float)raw[ii][r][c][e];
                            } else {
                                const float4 a = raw[ii][r][c].a, b = raw[ii][r][c].b;
                                x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
                            }
#pragma unroll
                            for (int e = 0; e < 8; e++) row[c][e] = act_p16(ok ? x[e] : 0.f, p.dw_act);
                        }
#pragma unroll
                        for (int kx = 0; kx < 3; kx++) {
                            // (the weights come through the L1: staging them in LDS first cost a barrier and measured slower)
                            const float* wp = p.dw_w + (r * 3 + kx) * p.dw_cp + wch;
                            const float4 w0 = *reinterpret_cast<const float4*>(wp), w1 = *reinterpret_cast<const float4*>(wp + 4);
                            const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
                            for (int j = 0; j < 2; j++)
#pragma unroll
                                for (int e = 0; e < 8; e++) acc[j][e] = fmaf(row[j * DWS + kx][e], w[e], acc[j][e]);
                        }
                    }
                    const float4 s0 = *reinterpret_cast<const float4*>(p.dw_scale + wch), s1 = *reinterpret_cast<const float4*>(p.dw_scale + wch + 4);
                    const float4 b0 = *reinterpret_cast<const float4*>(p.dw_bias + wch), b1 = *reinterpret_cast<const float4*>(p.dw_bias + wch + 4);
                    const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
                    const float bi[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                    const int lo0 = chunk * G::BUFC + (pair >> 1) * G::ROW_PITCH + (pair & 1) * 2 * G::PIT + g * 16;
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        half8_t hi, lo;
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            float o = acc[j][e] * sc[e] + bi[e];
                            if constexpr (HSTORE) o = (float)(_Float16)o;   // (what the depthwise layer would have stored)
                            const float v = chan_ok ? act_p16(o, p.act) * in_scale : 0.f;
                            hi[e] = (_Float16)v;
                            lo[e] = (_Float16)(v - (float)hi[e]);
                        }
                        *reinterpret_cast<half8_t*>(lds + lo0 + j * G::PIT) = hi;
                        if constexpr (!HSTORE) *reinterpret_cast<half8_t*>(lds + G::PLANE + lo0 + j * G::PIT) = lo;
                    }
                }
            }
            lds_barrier();   // the tile is staged
            lds_barrier();   // the MFMA waves have left their accumulators for wave 0
            return;
        }
        if (stid < 16 * FM) {
            reinterpret_cast<float*>(lds + sb_off)[stid] = p.scale[cb * 16 * FM + stid];
            reinterpret_cast<float*>(lds + sb_off)[16 * FM + stid] = p.bias[cb * 16 * FM + stid];
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            stage_tile(SW == 8 ? tid : stid, r, r > 0);
            lds_barrier();   // the round is staged
        }
        lds_barrier();   // the MFMA waves have left their accumulators for wave 0
        return;
    }

    // ---------------------------------------------------------------------- MFMA waves
    const int w = wave - 4;
    const int mq = lane & 15, kq = lane >> 4;
    int bbase[FN];   // chunk `w` of the tile, the lane's position of each fragment
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = fn * 16 + mq;
        bbase[fn] = (m / G::TW) * S * G::ROW_PITCH + (m % G::TW) * S * G::PIT + kq * 16 + w * G::BUFC;
    }
    constexpr unsigned wstep = FM * NPL * 1024;
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)((cb * 4 + w) * R * STEPS) * wstep + lane * 16;
    half8_t a_q[RPD][FM][NPL];
    auto ring_fill = [&](const unsigned char* wb) {   // the weights of a round's first RPD - 1 steps
#pragma unroll
        for (int d = 0; d < RPD - 1; d++)
#pragma unroll
            for (int fm = 0; fm < FM; fm++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) a_q[d][fm][pl] = *reinterpret_cast<const half8_t*>(wb + (size_t)d * wstep + (fm * NPL + pl) * 1024);
#pragma unroll
        for (int fm = 0; fm < FM; fm++)
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) a_q[RPD - 1][fm][pl] = a_q[0][fm][pl];   // (defined; replaced during the first step)
    };
    ring_fill(wbase);
    f32x4_t acc[FM][FN];
#pragma unroll
    for (int fm = 0; fm < FM; fm++)
#pragma unroll
        for (int fn = 0; fn < FN; fn++) acc[fm][fn] = (f32x4_t)(0.f);
    float inv_in_scale = 1.f;
    if (ranged) (void)range_scale(range_after_act(range_reduce(range_word()), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    // The residual values of the epilogue (wave 0) are requested here, so that their memory round trip passes under the
    // staging and the step stream instead of behind them (small tiles: the registers are there).
    constexpr bool RES_EARLY = FM * FN <= 4;
    typedef typename std::conditional<HSTORE, half4_t, f32x4_t>::type res_t;
    res_t res_early[RES_EARLY ? FM : 1][RES_EARLY ? FN : 1];
    if constexpr (RES_EARLY) {
        if (w == 0 && p.res) {
            const store_t* res = reinterpret_cast<const store_t*>(p.res);
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
#pragma unroll
                for (int fm = 0; fm < FM; fm++) {
                    const int m = fn * 16 + mq;
                    const int py = tyi * G::TH + m / G::TW, px = txi * G::TW + m % G::TW;
                    const int ch = cb * 16 * FM + fm * 16 + kq * 4;
                    const bool okc = py < p.npos_y && px < p.npos_x && ch + 4 <= p.out_cp;
                    res_early[fm][fn] = *reinterpret_cast<const res_t*>(res + (okc ? ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp + ch : 0));
                }
        }
    }

    if constexpr (SW == 8) stage_tile(tid, 0, false);
#pragma unroll
    for (int r = 0; r < R; r++) {
        const unsigned char* wb = wbase + (size_t)r * STEPS * wstep;
        lds_barrier();   // the round is staged
        // B fragment of step s: chunk w + 4*(s / NTAPS), tap s % NTAPS
        auto b_off = [&](int s) { return (s / NTAPS) * 4 * G::BUFC + G::tap_off(s % NTAPS); };
        half8_t b[BD][FN][NPL];
#pragma unroll
        for (int s = 0; s < BD - 1; s++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
#pragma unroll
                for (int pl = 0; pl < NPL; pl++) b[s][fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[fn] + b_off(s) + pl * G::PLANE);
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int d = s % RPD, dload = (s + RPD - 1) % RPD, bs = s % BD, bload = (s + BD - 1) % BD;
            // the weights of step s + RPD - 1 and the fragment of step s + BD - 1 go into the slots the previous step left
            if (s + RPD - 1 < STEPS) {
#pragma unroll
                for (int fm = 0; fm < FM; fm++)
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++)
                        a_q[dload][fm][pl] = *reinterpret_cast<const half8_t*>(wb + (size_t)(s + RPD - 1) * wstep + (fm * NPL + pl) * 1024);
            }
            if (s + BD - 1 < STEPS) {
#pragma unroll
                for (int fn = 0; fn < FN; fn++)
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++)
                        b[bload][fn][pl] = *reinterpret_cast<const half8_t*>(lds + bbase[fn] + b_off(s + BD - 1) + pl * G::PLANE);
            }
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
#pragma unroll
                for (int i = 0; i < NPASS * FM; i++) {
                    const int kind = i / FM, fm = i % FM;
                    const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
                    acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_q[d][fm][apl], b[bs][fn][bpl], acc[fm][fn], 0, 0, 0);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (r + 1 < R) {
            ring_fill(wb + (size_t)STEPS * wstep);
            lds_barrier();   // every MFMA wave is through with the round: the staging waves may write the next
        }
    }
    // the four partial sums meet in wave 0
    if (w > 0) {
#pragma unroll
        for (int fm = 0; fm < FM; fm++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
                *reinterpret_cast<f32x4_t*>(lds + red_off + (((w - 1) * FM + fm) * FN + fn) * 1024 + lane * 16) = acc[fm][fn];
    }
    lds_barrier();
    if (w > 0) return;
    float vmax = 0.f;
    {
        const float* sb = reinterpret_cast<const float*>(lds + sb_off);
        store_t* out = reinterpret_cast<store_t*>(p.out);
        const store_t* res = reinterpret_cast<const store_t*>(p.res);
#pragma unroll
        for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int fm = 0; fm < FM; fm++) {
            const int m = fn * 16 + mq;
            const int py = tyi * G::TH + m / G::TW, px = txi * G::TW + m % G::TW;
            const bool okp = py < p.npos_y && px < p.npos_x;
            f32x4_t v = acc[fm][fn];
#pragma unroll
            for (int o = 0; o < 3; o++) v += *reinterpret_cast<const f32x4_t*>(lds + red_off + ((o * FM + fm) * FN + fn) * 1024 + lane * 16);
            const f32x4_t sc = *reinterpret_cast<const f32x4_t*>(sb + fm * 16 + kq * 4);
            const f32x4_t bi = *reinterpret_cast<const f32x4_t*>(sb + 16 * FM + fm * 16 + kq * 4);
            const int ch = cb * 16 * FM + fm * 16 + kq * 4;
            // (the last block of output channels may reach beyond the tensor's channel pitch: those rows are not stored)
            const bool okc = okp && ch + 4 <= p.out_cp;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = v[e] * (sc[e] * acc_mul) + bi[e];
            if (res && okc) {
                [[maybe_unused]] const store_t* rp = res + ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp + ch;
                f32x4_t rv;
                if constexpr (RES_EARLY) {
#pragma unroll
                    for (int e = 0; e < 4; e++) rv[e] = (float)res_early[fm][fn][e];
                } else if constexpr (HSTORE) {
                    const half4_t rh = *reinterpret_cast<const half4_t*>(rp);
#pragma unroll
                    for (int e = 0; e < 4; e++) rv[e] = (float)rh[e];
                } else {
                    rv = *reinterpret_cast<const f32x4_t*>(rp);
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float r = p.res_relu ? fmaxf(rv[e], 0.f) : rv[e];
                    if (p.res_scale) r *= sc[e];
                    v[e] += r;
                }
            }
            store_t* op = out + ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp + ch;
            if constexpr (HSTORE) {
                half4_t hv;
#pragma unroll
                for (int e = 0; e < 4; e++) hv[e] = (_Float16)v[e];
                if (okc) *reinterpret_cast<half4_t*>(op) = hv;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) vmax = fmaxf(vmax, okc ? fabsf(v[e]) : 0.f);
                if (okc) *reinterpret_cast<f32x4_t*>(op) = v;
            }
        }
    }
    if (p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 1);
}

typedef void (*p16_fn)(const ConvP16Params);
struct P16Entry {
    int th, tw, stride, wm;
    p16_fn fn;
    size_t buf, res_bytes;   // one staging buffer; the residual tile
    p16_fn fn_c8;            // fp32 tensors: the form with the correction terms as fp8 MFMAs
};
template <int TH, int TW, int S, int WM>
constexpr P16Entry entry() {
    using G = Geo<TH, TW, S, WM>;
    P16Entry e{TH, TW, S, WM, conv_p16_kernel<TH, TW, S, WM>, (size_t)G::BUF, (size_t)TH * G::TWG * G::RES_PITCH, nullptr};
    if constexpr (!HSTORE) e.fn_c8 = conv_p16_kernel<TH, TW, S, WM, true>;
    return e;
}
const P16Entry kEntries[] = {
    entry<8, 10, 1, 4>(), entry<10, 8, 1, 4>(), entry<8, 8, 1, 4>(), entry<8, 6, 1, 4>(), entry<4, 8, 1, 4>(), entry<4, 4, 1, 4>(),
    entry<8, 8, 1, 2>(), entry<8, 6, 1, 2>(), entry<4, 8, 1, 2>(),
    entry<10, 8, 2, 4>(), entry<8, 10, 2, 4>(), entry<8, 8, 2, 4>(),
    entry<8, 6, 2, 2>(), entry<4, 8, 2, 2>(), entry<8, 4, 2, 2>(),
};
size_t entry_lds(const P16Entry& e, bool residual) {   // (e.buf and e.res_bytes are this translation unit's: they depend on the storage type)
    return 2 * e.buf + 2 * (size_t)(32 * e.wm) * 4 + (residual ? e.res_bytes : 0);
}
struct TP16Entry {
    int th, tw, wm;
    p16_fn fn;
    size_t buf;
};
template <int TH, int TW, int WM>
constexpr TP16Entry tentry() {
    return TP16Entry{TH, TW, WM, tconv_p16_kernel<TH, TW, WM>, (size_t)Geo<TH, TW, 1, WM, 1>::BUF};
}
const TP16Entry kTEntries[] = {
    tentry<4, 8, 1>(), tentry<8, 4, 1>(), tentry<2, 8, 1>(), tentry<6, 8, 1>(),
    tentry<4, 8, 2>(), tentry<8, 4, 2>(), tentry<2, 8, 2>(), tentry<6, 8, 2>(), tentry<8, 6, 2>(),
};
struct C4Entry {
    int k, th, tw;
    p16_fn fn, fn8;   // three fp16 passes; fp8 correction terms (fp32 tensors, an even number of steps) or null
    size_t buf;
    int steps;
};
template <int K, int TH, int TW>
constexpr C4Entry c4entry() {
    using G = GeoC4<K, TH, TW>;
    if constexpr (!HSTORE && G::NS % 2 == 0) return C4Entry{K, TH, TW, conv_p16c4_kernel<K, TH, TW, false>, conv_p16c4_kernel<K, TH, TW, true>, (size_t)G::BUF, G::NS};
    else return C4Entry{K, TH, TW, conv_p16c4_kernel<K, TH, TW, false>, nullptr, (size_t)G::BUF, G::NS};
}
const C4Entry kC4Entries[] = {c4entry<9, 8, 8>(), c4entry<9, 4, 8>(), c4entry<9, 8, 4>(), c4entry<3, 8, 8>(), c4entry<3, 4, 8>()};
struct KREntry {
    int taps, cpw, fm, nfrag, th, tw, stride, dws, rounds, src;   // (cpw: chunks per wave and round)
    p16_fn fn;
    size_t lds;
};
template <int NTAPS, int CPW, int FM, int FN = 1, int S = 1, int DWS = 0, int R = 1, int SRC = 0>
constexpr KREntry krentry() {
    using G = GeoR<NTAPS, CPW, FN, S>;
    return KREntry{NTAPS, CPW, FM, FN, G::TH, G::TW, S, DWS, R, SRC, conv_kr16_kernel<NTAPS, CPW, FM, FN, S, DWS, R, SRC>, (size_t)(G::RED_OFF + 3 * FM * FN * 1024 + 2 * 16 * FM * 4)};
}
const KREntry kKREntries[] = {
    krentry<1, 1, 1>(), krentry<1, 2, 1>(), krentry<1, 3, 1>(), krentry<1, 4, 1>(), krentry<1, 5, 1>(), krentry<1, 6, 1>(), krentry<1, 8, 1>(), krentry<1, 12, 1>(), krentry<1, 16, 1>(),
    krentry<1, 1, 2>(), krentry<1, 2, 2>(), krentry<1, 3, 2>(), krentry<1, 4, 2>(), krentry<1, 5, 2>(), krentry<1, 6, 2>(), krentry<1, 8, 2>(), krentry<1, 12, 2>(), krentry<1, 16, 2>(),
    krentry<9, 1, 1>(), krentry<9, 2, 1>(), krentry<9, 4, 1>(), krentry<9, 1, 2>(), krentry<9, 2, 2>(), krentry<9, 4, 2>(),
    // larger tiles for layers with more positions and a short reduction
    krentry<1, 1, 1, 2>(), krentry<1, 1, 2, 2>(), krentry<1, 2, 1, 2>(), krentry<1, 2, 2, 2>(), krentry<9, 1, 1, 2>(), krentry<9, 1, 2, 2>(),
    krentry<1, 1, 1, 4>(), krentry<1, 1, 2, 4>(), krentry<1, 2, 1, 4>(), krentry<1, 2, 2, 4>(), krentry<9, 1, 1, 4>(), krentry<9, 1, 2, 4>(),
    // 3x3 with stride 2 (a 9x9-pixel window per chunk under a tile of 4x4 positions)
    krentry<9, 1, 1, 1, 2>(), krentry<9, 1, 2, 1, 2>(), krentry<9, 2, 1, 1, 2>(), krentry<9, 2, 2, 1, 2>(),
#if FYN_P16_HALF   // (16 chunks in one round: 83 KB of fp16, 166 KB in two fp32 planes -- that unit takes the two-round variant below)
    krentry<9, 4, 1, 1, 2>(), krentry<9, 4, 2, 1, 2>(),
#endif
    // reductions that pass through the LDS in two rounds (taken where the one-round entry above is more than a CU's LDS):
    // 3x3 with stride 2 on 512 channels in fp32, 3x3 on 1024 channels, 1x1 on 4096
    krentry<9, 2, 1, 1, 2, 0, 2>(), krentry<9, 2, 2, 1, 2, 0, 2>(), krentry<9, 4, 1, 1, 1, 0, 2>(), krentry<9, 4, 2, 1, 1, 0, 2>(),
    krentry<1, 16, 1, 1, 1, 0, 2>(), krentry<1, 16, 2, 1, 1, 0, 2>(),
};
// 1x1 with a depthwise 3x3 layer (step 1 or 2) computed in the staging
#define FYN_KR_DW(CPW) krentry<1, CPW, 1, 1, 1, 1>(), krentry<1, CPW, 2, 1, 1, 1>(), krentry<1, CPW, 1, 1, 1, 2>(), krentry<1, CPW, 2, 1, 1, 2>()
const KREntry kKRDwEntries[] = {FYN_KR_DW(1), FYN_KR_DW(2), FYN_KR_DW(3), FYN_KR_DW(4)};   // (up to 512 channels: beyond, two launches are faster)
#undef FYN_KR_DW
// 1x1 on 4x4 tiles with a batch-norm layer applied while staging (1) or over two tensors (2)
#define FYN_KR_SRC(CPW) krentry<1, CPW, 1, 1, 1, 0, 1, 1>(), krentry<1, CPW, 2, 1, 1, 0, 1, 1>(), krentry<1, CPW, 1, 1, 1, 0, 1, 2>(), krentry<1, CPW, 2, 1, 1, 0, 1, 2>()
const KREntry kKRSrcEntries[] = {FYN_KR_SRC(1), FYN_KR_SRC(2), FYN_KR_SRC(3), FYN_KR_SRC(4), FYN_KR_SRC(5), FYN_KR_SRC(6), FYN_KR_SRC(8), FYN_KR_SRC(12), FYN_KR_SRC(16)};
#undef FYN_KR_SRC
}  // namespace

// Host entry points.  The fp32 unit holds the public ones and hands launches on fp16 tensors (p.f16) to the other
// unit's, which carry the suffix _half; tile tables are the same in both.
#if FYN_P16_HALF
#define P16_NAME(n) n##_half
#else
#define P16_NAME(n) n
size_t conv_p16_lds_bytes_half(const ConvP16Params& p);
int launch_conv_p16_half(const ConvP16Params& p, hipStream_t s);
size_t tconv_p16_lds_bytes_half(const ConvP16Params& p);
int launch_tconv_p16_half(const ConvP16Params& p, hipStream_t s);
size_t conv_p16c4_lds_bytes_half(const ConvP16Params& p, int k);
int launch_conv_p16c4_half(const ConvP16Params& p, int k, hipStream_t s);
size_t conv_kr16_lds_bytes_half(const ConvP16Params& p, int k);
int launch_conv_kr16_half(const ConvP16Params& p, int k, hipStream_t s);

int conv_p16_tile_count() { return (int)(sizeof(kEntries) / sizeof(kEntries[0])); }
void conv_p16_tile(int index, int* th, int* tw, int* stride, int* wm) {
    *th = kEntries[index].th; *tw = kEntries[index].tw; *stride = kEntries[index].stride; *wm = kEntries[index].wm;
}
bool conv_p16_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16) {
    // (16-byte loads of 8 channels, 16-byte stores of 4 fp32 or 8 fp16 channels; the last chunk and the last block of
    // output channels may be ragged: what lies behind a pitch is read as zero and not stored)
    const int og = f16 ? 8 : 4;
    return k == 3 && (stride == 1 || stride == 2) && dil == 1 && in_cp % 8 == 0 && in_cp >= 16 && cout >= 8 && out_cp % og == 0 && out_cp >= cout;
}
int tconv_p16_tile_count() { return (int)(sizeof(kTEntries) / sizeof(kTEntries[0])); }
void tconv_p16_tile(int index, int* th, int* tw, int* wm) {
    *th = kTEntries[index].th; *tw = kTEntries[index].tw; *wm = kTEntries[index].wm;
}
void tconv_p16_tap(int t, int* ky, int* kx) { *ky = TT_KY[t]; *kx = TT_KX[t]; }
bool tconv_p16_supported(int k, int crop, int in_cp, int in_pad, int cout, int out_cp, bool f16) {
    (void)f16;
    return k == 3 && crop == 1 && in_cp % KC == 0 && in_pad >= 1 && cout % 32 == 0 && out_cp % 4 == 0 && out_cp >= cout;
}
int conv_p16c4_tile_count() { return (int)(sizeof(kC4Entries) / sizeof(kC4Entries[0])); }
void conv_p16c4_tile(int index, int* k, int* th, int* tw, int* steps) {
    *k = kC4Entries[index].k; *th = kC4Entries[index].th; *tw = kC4Entries[index].tw; *steps = kC4Entries[index].steps;
}
int conv_kr16_variant_count() { return (int)(sizeof(kKREntries) / sizeof(kKREntries[0])); }
void conv_kr16_variant(int index, int* taps, int* chunks, int* fm, int* th, int* tw, int* stride) {
    *taps = kKREntries[index].taps; *chunks = 4 * kKREntries[index].cpw * kKREntries[index].rounds; *fm = kKREntries[index].fm;
    *th = kKREntries[index].th; *tw = kKREntries[index].tw; *stride = kKREntries[index].stride;
}
bool conv_p16c4_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16) {
    // (any number of output channels: the weights are packed for whole blocks of 32, what lies behind the pitch is not stored)
    return (k == 9 || k == 3) && stride == 1 && dil == 1 && in_cp == 4 && cout >= 8 && out_cp % (f16 ? 8 : 4) == 0 && out_cp >= cout;
}
#endif

#if !FYN_P16_HALF
// Third weight plane of the 16-position forms on fp32 tensors: src holds, per fragment and lane, sixteen floats -- the
// eight hi parts divided by 32, then the eight lo parts times 64 -- which become the sixteen fp8 values of the lane in
// plane 2 of the fragment (three planes of 1 KB each).  Converted on the device, so that the format is the one the
// matrix instruction reads.
__global__ __launch_bounds__(256) void pack_fp8_plane_kernel(const float* __restrict__ src, unsigned char* __restrict__ wpack, size_t n4) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;   // four values each
    if (i >= n4) return;
    const float4 v = reinterpret_cast<const float4*>(src)[i];
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(v.x, v.y, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(v.z, v.w, w, true);
    const size_t lane16 = i >> 2, frag = lane16 >> 6;   // sixteen values per lane, 64 lanes per fragment
    *reinterpret_cast<int*>(wpack + frag * 3072 + 2048 + (lane16 & 63) * 16 + (i & 3) * 4) = w;
}
int launch_pack_fp8_plane(const float* src, void* wpack, size_t frags, hipStream_t s) {
    const size_t n4 = frags * 64 * 4;
    if (n4 == 0) return 0;
    hipLaunchKernelGGL(pack_fp8_plane_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, src, static_cast<unsigned char*>(wpack), n4);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
#endif

static const KREntry* find_krentry(const ConvP16Params& p, int k) {
    if (p.dw_in) {
        for (const KREntry& c : kKRDwEntries)
            if (k == 1 && c.cpw * 4 == p.cin_chunks && c.fm == p.wm && c.th == p.tile_h && c.tw == p.tile_w && c.dws == p.dw_stride) return &c;
        return nullptr;
    }
    if (p.in_mul || p.in2) {
        const int src = p.in_mul ? 1 : 2;
        for (const KREntry& c : kKRSrcEntries)
            if (k == 1 && c.cpw * 4 == p.cin_chunks && c.fm == p.wm && c.th == p.tile_h && c.tw == p.tile_w && c.src == src && c.lds <= 160 * 1024) return &c;
        return nullptr;
    }
    for (const KREntry& c : kKREntries)
        if (c.taps == k * k && c.cpw * 4 * c.rounds == p.cin_chunks && c.fm == p.wm && c.th == p.tile_h && c.tw == p.tile_w && c.stride == (k == 1 ? 1 : p.stride) &&
            c.lds <= 160 * 1024)
            return &c;
    return nullptr;
}
size_t P16_NAME(conv_kr16_lds_bytes)(const ConvP16Params& p, int k) {
#if !FYN_P16_HALF
    if (p.f16) return conv_kr16_lds_bytes_half(p, k);
#endif
    const KREntry* e = find_krentry(p, k);
    return e ? e->lds : 0;
}
// The K-resident form: k = 1 (any stride) or 3 (stride 1, or 2 with 4x4 tiles); tiles of tile_h x tile_w = 4x4 (4x8, 8x8 for short reductions) positions, blocks of 16*p.wm output channels (p.wm = 1 or 2),
// p.cin_chunks = 4, 8, 12, 16, 20, 24, 32, 48, 64 or 128 (3x3: 4, 8, 16 or 32; with stride 2: 4, 8 or 16), channels behind in_cp reading as zero; in_y0/in_x0 = input padding - (k-1)/2; one workgroup per tile and block
int P16_NAME(launch_conv_kr16)(const ConvP16Params& p, int k, hipStream_t s) {
#if !FYN_P16_HALF
    if (p.f16) return launch_conv_kr16_half(p, k, s);
#endif
    const KREntry* e = find_krentry(p, k);
    if (!e) return -1;
    if (p.in_cp > p.cin_chunks * KC || p.in_cp % 8 != 0 || p.in_cp < 8 || p.cout_blocks < 1 || p.mfrags != p.cout_blocks * e->fm || p.stride < 1 ||
        p.tiles_x * e->tw < p.npos_x || p.tiles_y * e->th < p.npos_y || p.out_cp % 4 != 0 || p.out_cp < 4 || (p.res && p.res_cp < p.out_cp) || p.nreset < 0 || p.nreset > 4 || (p.f16 != 0) != HSTORE ||
        p.tiles_x < 1 || p.tiles_y < 1 || p.tiles_x > 65535 || p.tiles_y > 65535 || (long long)p.tiles_x * p.tiles_y * p.cout_blocks > 65535)
        return -5;
    // (a fused depthwise layer: its tensor has the pointwise layer's channels, in whole groups of 8, and the 1x1 layer does not step)
    if (p.dw_in && (!p.dw_w || !p.dw_scale || !p.dw_bias || p.dw_cp != p.in_cp || p.stride != 1 || p.in_clamp || p.dw_hp < 1 || p.dw_wp < 1)) return -5;
    // (a batch-norm layer applied while staging: not beside a depthwise layer, and both arrays or none)
    if ((p.in_mul != nullptr) != (p.in_add != nullptr) || (p.in_mul && (p.dw_in || p.in2))) return -5;
    // (a second source tensor: 1x1 in one round, the first tensor's channels end where the second's chunks begin)
    if (p.in2 && (k != 1 || e->rounds != 1 || p.dw_in || p.in_mul || p.in_clamp || p.in2_chunk0 < 1 || p.in2_chunk0 >= p.cin_chunks || p.in_cp > p.in2_chunk0 * KC ||
                  p.in2_cp % 8 != 0 || p.in2_cp < 8 || p.in2_cp > (p.cin_chunks - p.in2_chunk0) * KC || p.in2_stride < 1 || p.in2_hp < 1 || p.in2_wp < 1 || p.in2_y0 < 0 || p.in2_x0 < 0))
        return -5;
    if (e->lds > 160 * 1024) return -2;
    if (ensure_lds(reinterpret_cast<const void*>(e->fn), e->lds) != 0) return -2;
    hipLaunchKernelGGL(e->fn, dim3(p.cout_blocks, p.tiles_x, p.tiles_y), dim3(512), e->lds, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

// The correction terms run as fp8 MFMAs where the input carries a value-range word (fp32 tensors) and the chunks pair up,
// unless the layer asks for the three fp16 passes (p.exact_split).
static bool p16_uses_fp8(const ConvP16Params& p) {
    return !HSTORE && !p.f16 && !p.exact_split && p.in_amax != nullptr && p.cin_chunks % 2 == 0;
}
#if !FYN_P16_HALF
bool conv_p16_uses_fp8(const ConvP16Params& p) { return p16_uses_fp8(p); }
#endif

static const P16Entry* find_entry(const ConvP16Params& p) {
    for (const P16Entry& c : kEntries)
        if (c.th == p.tile_h && c.tw == p.tile_w && c.stride == p.stride && c.wm == p.wm) return &c;
    return nullptr;
}
size_t P16_NAME(conv_p16_lds_bytes)(const ConvP16Params& p) {
#if !FYN_P16_HALF
    if (p.f16) return conv_p16_lds_bytes_half(p);
#endif
    const P16Entry* e = find_entry(p);
    return e ? entry_lds(*e, p.res != nullptr) : 0;
}

int P16_NAME(launch_conv_p16)(const ConvP16Params& p, hipStream_t s) {
#if !FYN_P16_HALF
    if (p.f16) return launch_conv_p16_half(p, s);
#endif
    const P16Entry* e = find_entry(p);
    if (!e) return -1;
    const int cpb = 32 * e->wm, twg = (4 / e->wm) * e->tw;
    // what the kernel's indexing assumes
    if (p.cin_chunks < 1 || p.in_cp > p.cin_chunks * KC || p.in_cp <= (p.cin_chunks - 1) * KC || p.in_cp % 8 != 0 || p.in_shift < 0 || p.in_shift > 8 || p.cout_blocks < 1 || p.mfrags < p.cout_blocks * 2 * e->wm ||
        p.tiles_x * twg < p.npos_x || p.tiles_y * p.tile_h < p.npos_y || p.out_cp <= (p.cout_blocks - 1) * cpb || (p.out_cp * ESZ) % 16 != 0 ||
        (p.res && (p.res_cp <= (p.cout_blocks - 1) * cpb || (p.res_cp * ESZ) % 16 != 0)) || p.nreset < 0 || p.nreset > 4 || p.pos_groups < 1 ||
        p.pos_groups > p.tiles_x * p.tiles_y || (p.f16 != 0) != HSTORE ||
        // (a tile's residual tile may not be overwritten while its epilogue reads it: the next one comes a stage later)
        (p.res && p.cin_chunks < 2 && p.pos_groups < p.tiles_x * p.tiles_y) || p.rcp_tiles_x != 1.0f / (float)p.tiles_x ||
        p.tiles_x * p.tiles_y > 4000000)   // (tile index -> row and column through the reciprocal: exact below four million tiles)
        return -5;
    const size_t lds_bytes = entry_lds(*e, p.res != nullptr);
    if (lds_bytes > 160 * 1024) return -2;
    const p16_fn fn = p16_uses_fp8(p) ? e->fn_c8 : e->fn;
    if (ensure_lds(reinterpret_cast<const void*>(fn), lds_bytes) != 0) return -2;
    hipLaunchKernelGGL(fn, dim3(p.pos_groups * p.cout_blocks), dim3(512), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

static const TP16Entry* find_tentry(const ConvP16Params& p) {
    for (const TP16Entry& c : kTEntries)
        if (c.th == p.tile_h && c.tw == p.tile_w && c.wm == p.wm) return &c;
    return nullptr;
}
size_t P16_NAME(tconv_p16_lds_bytes)(const ConvP16Params& p) {
#if !FYN_P16_HALF
    if (p.f16) return tconv_p16_lds_bytes_half(p);
#endif
    const TP16Entry* e = find_tentry(p);
    return e ? 2 * e->buf + 2 * (size_t)(32 * e->wm) * 4 : 0;
}

// npos_y x npos_x: the input size (positions are input pixels); out_off_*: stored coordinate of output pixel (0, 0)
int P16_NAME(launch_tconv_p16)(const ConvP16Params& p, hipStream_t s) {
#if !FYN_P16_HALF
    if (p.f16) return launch_tconv_p16_half(p, s);
#endif
    const TP16Entry* e = find_tentry(p);
    if (!e) return -1;
    const int cpb = 32 * e->wm, twg = (4 / e->wm) * e->tw;
    if (p.cin_chunks < 1 || p.in_cp != p.cin_chunks * KC || p.cout_blocks < 1 || p.mfrags < p.cout_blocks * 2 * e->wm ||
        p.tiles_x * twg < p.npos_x || p.tiles_y * p.tile_h < p.npos_y || p.out_cp < p.cout_blocks * cpb || (p.out_cp * ESZ) % 16 != 0 || p.res || p.stride != 1 || p.in_shift != 0 ||
        p.nreset < 0 || p.nreset > 4 || p.pos_groups < 1 || p.pos_groups > p.tiles_x * p.tiles_y || (p.f16 != 0) != HSTORE ||
        p.rcp_tiles_x != 1.0f / (float)p.tiles_x || p.tiles_x * p.tiles_y > 4000000)
        return -5;
    const size_t lds_bytes = P16_NAME(tconv_p16_lds_bytes)(p);
    if (lds_bytes > 160 * 1024) return -2;
    if (ensure_lds(reinterpret_cast<const void*>(e->fn), lds_bytes) != 0) return -2;
    hipLaunchKernelGGL(e->fn, dim3(p.pos_groups * p.cout_blocks), dim3(512), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

// (the fp8 form of the correction terms: as p16_uses_fp8, for the kernels whose stage has an even number of steps)
static bool c4_uses_fp8(const ConvP16Params& p, const C4Entry* e) {
    return !HSTORE && !p.f16 && !p.exact_split && p.in_amax != nullptr && e->fn8 != nullptr;
}
static const C4Entry* find_c4entry(const ConvP16Params& p, int k) {
    for (const C4Entry& c : kC4Entries)
        if (c.k == k && c.th == p.tile_h && c.tw == p.tile_w) return &c;
    return nullptr;
}
size_t P16_NAME(conv_p16c4_lds_bytes)(const ConvP16Params& p, int k) {
#if !FYN_P16_HALF
    if (p.f16) return conv_p16c4_lds_bytes_half(p, k);
#endif
    const C4Entry* e = find_c4entry(p, k);
    return e ? 2 * e->buf + 2 * 32 * 4 : 0;
}

// k x k convolution on a four-channel input: wpack = [step][cout fragment of 16][plane][lane][8 halves], lane = (output
// channel lane%16, tap pair 4*step + lane/16 = kernel row pair/((k+1)/2), columns 2*(pair%((k+1)/2)) and +1), four input
// channels per tap; in_y0/in_x0 = input padding - (k-1)/2
int P16_NAME(launch_conv_p16c4)(const ConvP16Params& p, int k, hipStream_t s) {
#if !FYN_P16_HALF
    if (p.f16) return launch_conv_p16c4_half(p, k, s);
#endif
    const C4Entry* e = find_c4entry(p, k);
    if (!e) return -1;
    if (p.in_cp != 4 || p.cin_chunks != 1 || p.cout_blocks < 1 || p.mfrags < p.cout_blocks * 2 || p.wm != 1 || p.stride != 1 || p.res || p.in_shift != 0 ||
        p.tiles_x * 4 * e->tw < p.npos_x || p.tiles_y * e->th < p.npos_y || p.out_cp <= (p.cout_blocks - 1) * 32 || (p.out_cp * ESZ) % 16 != 0 ||
        p.nreset < 0 || p.nreset > 4 || p.pos_groups < 1 || p.pos_groups > p.tiles_x * p.tiles_y || (p.f16 != 0) != HSTORE ||
        p.rcp_tiles_x != 1.0f / (float)p.tiles_x || p.tiles_x * p.tiles_y > 4000000)
        return -5;
    const size_t lds_bytes = P16_NAME(conv_p16c4_lds_bytes)(p, k);
    if (lds_bytes > 160 * 1024) return -2;
    if (ensure_lds(reinterpret_cast<const void*>(e->fn), lds_bytes) != 0) return -2;
    const p16_fn fn = c4_uses_fp8(p, e) ? e->fn8 : e->fn;
    if (fn != e->fn && ensure_lds(reinterpret_cast<const void*>(fn), lds_bytes) != 0) return -2;
    hipLaunchKernelGGL(fn, dim3(p.pos_groups * p.cout_blocks), dim3(512), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
#if !FYN_P16_HALF
bool conv_p16c4_uses_fp8(const ConvP16Params& p, int k) {
    const C4Entry* e = find_c4entry(p, k);
    return e && c4_uses_fp8(p, e);
}
#endif

}  // namespace fynhip
