// K x K convolution (K = 3 or 9, stride 1) between wide layers with fp16 storage -- the residual blocks of a
// style-transfer net at full resolution -- as an implicit GEMM on gfx950 matrix cores with 16-position fragments
// (v_mfma_f32_16x16x32_f16, fp32 accumulate), one MFMA per fragment pair.
//
// Replaces, for such layers, the render passes of DeepConvLayerNxN::forward (fyusenet/gpu/deep/deepconvlayerNxN.cpp:
// 129-211); epilogue order of shaders/deep/deepconv3x3_tiled.frag:36-45 (acc*scale + bias, then the residual).
//
// Why another MFMA kernel: these layers run for hundreds of microseconds, and what bounds the general kernel on them is
// operand traffic and the rounds of a launch.  Its waves hold 32 output channels x 96 positions, so every wave reads the
// whole position tile from LDS for each k16 step (128 bytes per CU and MFMA cycle, about what the LDS delivers), and
// its 1872 workgroups, two per CU, make 3.7 rounds with a prologue and an epilogue per tile in the open.  Here a wave
// holds 64 channels x 96 positions (4 x 6 fragments, 96 accumulator registers): 64 bytes per cycle from LDS and 43 from
// the L1 (weights), and a workgroup walks its tiles with four staging waves running a stage ahead, as in conv_p16.hip.
//
// GEMM view: M = output channels (A = weights, packed per lane, streamed through L2/L1 into a register ring of three
// steps), N = positions (B = activations, a halo tile of one 32-channel chunk in LDS), K = taps x channels, one tap of one
// chunk per step.  A stage is one chunk of one tile: K kernel rows of K steps; the code of one kernel row is unrolled
// (the tap's column is an immediate offset of the LDS reads), the rows are a loop that moves the fragments' base
// registers by a row pitch.
//
// Workgroup = 4 staging waves + 4 MFMA waves (2 groups of 64 output channels x 2 tiles of TH x 8 positions side by
// side).  A lane's accumulators of one fragment are 4 consecutive output channels of one position: no transposition in
// the epilogue; residual (staged to LDS by the staging waves during a tile's last chunk) and scale/bias from LDS.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "kernels.h"
#include "p16_common.h"

namespace fynhip {

namespace {
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
constexpr int HPD = 3;    // depth of the weight-fragment ring (steps); a kernel row is a whole number of turns
constexpr int HFM = 4;    // fragments of 16 output channels per wave

template <int K_, int TH_, int TW_>
struct GeoH {
    static constexpr int K = K_, TH = TH_, TW = TW_;
    static constexpr int WM = 2, WN = 2, TWG = WN * TW;
    static constexpr int HW = TWG + K - 1, HH = TH + K - 1;
    static constexpr int ROW_PITCH = HW * PITCH + p16_row_pad(TH, TW, 1, WN, HW);
    static constexpr int BUF = HH * ROW_PITCH;            // one staging buffer (fp16 storage: one plane)
    static constexpr int NPOS = TH * TW, FN = NPOS / 16;  // per wave
    static constexpr int NITEMS = HH * HW * (KC / 8);     // staging items: (pixel, 8 channels)
    static constexpr int NB = (NITEMS + 255) / 256;
    static constexpr int CPB = 16 * HFM * WM;             // output channels per workgroup
    static constexpr int RES_PITCH = CPB * 2 + 16;        // bytes per position of the residual tile
    static constexpr int RPIECES = TH * TWG * (CPB / 8);  // residual 16-byte pieces
    static constexpr int RNB = (RPIECES + 255) / 256;
    static_assert(NPOS % 16 == 0, "whole position fragments");
    static_assert(K % HPD == 0, "a kernel row is whole turns of the weight ring");
    static_assert(K * PITCH < 65536, "the tap column fits the LDS instructions' immediate field");
};

// The K steps of one kernel row of a stage.  `brow`: per-lane LDS offsets of the row's fragments at tap column 0;
// `nxt`: offsets of the fragments of the step that follows the row (the next kernel row, or the first step of the next
// stage in the other staging buffer -- LAST: the stage's barrier sits in front of the first such read; the staging waves
// have filled that buffer by then, and all reads of this stage's buffer were issued a step earlier).  One slot per
// MFMA: the MFMA, then a share of the step's memory instructions, fenced so that the compiler keeps the order.
// Position fragment fn is used by four consecutive MFMAs, after which its registers take the fragment of the next
// step; the ring slot of the previous step takes the weights of the step after the next.
template <class G, bool LAST>
__device__ __forceinline__ void h16_row(f32x4_t (&acc)[HFM][G::FN], half8_t (&a_q)[HPD][HFM], half8_t (&b)[G::FN], const int (&brow)[G::FN],
                                        const int (&nxt)[G::FN], const unsigned char* lds, const unsigned char*& wnext,
                                        const unsigned char* wbase, const unsigned char* wend, unsigned wstep, unsigned wlane) {
    constexpr int FN = G::FN, K = G::K;
#pragma unroll
    for (int dd = 0; dd < K; dd++) {
        const int d = dd % HPD, dprev = (d + HPD - 1) % HPD;
        const unsigned char* w_ = wnext;
        wnext += wstep;
        if (wnext == wend) wnext = wbase;
#pragma unroll
        for (int i = 0; i < HFM * FN; i++) {
            const int fn = i / HFM, fm = i % HFM;
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_q[d][fm], b[fn], acc[fm][fn], 0, 0, 0);
            if (LAST && dd == K - 1 && i == 1) lds_barrier();
            if (fm == HFM - 1) {
                if (dd + 1 < K) b[fn] = *reinterpret_cast<const half8_t*>(lds + brow[fn] + (dd + 1) * PITCH);
                else b[fn] = *reinterpret_cast<const half8_t*>(lds + nxt[fn]);
            }
#pragma unroll
            for (int j = 0; j < HFM; j++)   // the weight fragments of the step after the next, spread over this step's slots
                if (i == j * FN + 1) a_q[dprev][j] = *reinterpret_cast<const half8_t*>(w_ + j * 1024 + wlane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The staging waves (threads 0..255): stage after stage -- a 32-channel chunk of a tile's halo: global loads, activation,
// LDS writes -- one stage ahead of the MFMA waves, across tile boundaries; scale and bias at the start and, during a
// tile's last chunk, its residual tile.  One barrier per stage, after the one that hands over the first.  (A stage of
// the MFMA waves lasts thousands of cycles; the staging waves spend most of it waiting at the barrier.)
template <class G>
__device__ __forceinline__ void h16_stager(const ConvP16Params& p, unsigned char* lds, int stid, int cb, int group, int ntiles, int nchunks) {
    constexpr int CPB = G::CPB;
    constexpr int sb_off = 2 * G::BUF;
    constexpr int res_off = sb_off + 2 * CPB * 4;
    const _Float16* in = reinterpret_cast<const _Float16*>(p.in);
    int i_y[G::NB], i_x[G::NB], l_off[G::NB];
#pragma unroll
    for (int i = 0; i < G::NB; i++) {
        const int idx = stid + i * 256;
        l_off[i] = -1; i_y[i] = 1 << 20; i_x[i] = 0;
        if (idx < G::NITEMS) {
            const int pix = idx >> 2, g = idx & 3;
            const int py = pix / G::HW, px = pix - py * G::HW;
            i_y[i] = py; i_x[i] = px;
            l_off[i] = py * G::ROW_PITCH + px * PITCH + g * 16;
        }
    }
    const int g8 = (stid & 3) * 8;
    int g_off[G::NB];          // element offsets of the items, -1: outside the frame (reads as 0)
    half8_t raw[G::NB];
    // (unconditional loads: items outside the tensor read its first element and are zeroed when stored)
    auto fetch = [&](int tile, int chunk) {
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const int y0 = tyi * G::TH + p.in_y0, x0 = txi * G::TWG + p.in_x0;
#pragma unroll
        for (int i = 0; i < G::NB; i++) {
            int gy = y0 + i_y[i], gx = x0 + i_x[i];
            if (p.in_clamp && l_off[i] >= 0) {
                gy = min(max(gy, 0), p.in_hp - 1);
                gx = min(max(gx, 0), p.in_wp - 1);
            }
            g_off[i] = ((unsigned)gy < (unsigned)p.in_hp && (unsigned)gx < (unsigned)p.in_wp) ? (gy * p.in_wp + gx) * p.in_cp + g8 + chunk * KC : -1;
            raw[i] = *reinterpret_cast<const half8_t*>(in + (g_off[i] >= 0 ? g_off[i] : 0));
        }
    };
    auto store = [&](unsigned char* buf) {
#pragma unroll
        for (int i = 0; i < G::NB; i++) {
            if (l_off[i] < 0) continue;
            const bool ok = g_off[i] >= 0;
            half8_t v;
            _Float16 hlo, hhi;
            if (act_half_exact(p.act, hlo, hhi)) {
                // (on the packed halves: two instructions per item instead of seven per value; the staging waves share their
                // SIMDs' issue slots with the MFMA waves)
                v = ok ? act_half(raw[i], hlo, hhi) : (half8_t)((_Float16)0.f);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = ok ? (_Float16)act_p16((float)raw[i][e], p.act) : (_Float16)0.f;
            }
            *reinterpret_cast<half8_t*>(buf + l_off[i]) = v;
        }
    };
    auto residual_in = [&](int tile) {   // the residual tile of a tile: [position][CPB channels] fp16
        const _Float16* res = reinterpret_cast<const _Float16*>(p.res);
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        half8_t rv[G::RNB];
#pragma unroll
        for (int i = 0; i < G::RNB; i++) {
            const int idx = stid + i * 256;
            const int m = idx / (CPB / 8), c8 = idx % (CPB / 8);
            const int ty = m / G::TWG, tx = m - ty * G::TWG;
            const int py = tyi * G::TH + ty, px = txi * G::TWG + tx;
            const bool ok = idx < G::RPIECES && py < p.npos_y && px < p.npos_x;
            rv[i] = *reinterpret_cast<const half8_t*>(res + (ok ? ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp + cb * CPB + c8 * 8 : 0));
        }
#pragma unroll
        for (int i = 0; i < G::RNB; i++) {
            const int idx = stid + i * 256;
            if (idx < G::RPIECES) *reinterpret_cast<half8_t*>(lds + res_off + (idx / (CPB / 8)) * G::RES_PITCH + (idx % (CPB / 8)) * 16) = rv[i];
        }
    };
    auto advance = [&](int& tile, int& c) {
        if (++c == nchunks) { c = 0; tile += p.pos_groups; }
        return tile < ntiles;
    };
    int tile = group, c = 0;          // the stage the MFMA waves are on (stage n)
    int t1 = group, c1 = 0;           // stage n+1
    fetch(tile, 0);
    bool have1 = advance(t1, c1);
    if (stid < CPB) {
        reinterpret_cast<float*>(lds + sb_off)[stid] = p.scale[cb * CPB + stid];
        reinterpret_cast<float*>(lds + sb_off)[CPB + stid] = p.bias[cb * CPB + stid];
    }
    store(lds);
    lds_barrier();
    int buf = 0;                      // the buffer of stage n
    for (;;) {
        if (have1) fetch(t1, c1);
        if (c + 1 == nchunks && p.res) residual_in(tile);
        if (have1) store(lds + (1 - buf) * G::BUF);
        lds_barrier();
        if (!have1) break;
        tile = t1; c = c1; buf = 1 - buf;
        have1 = advance(t1, c1);
    }
}

// Grid: cout_blocks x pos_groups workgroups; a workgroup keeps its block of 128 output channels and walks the tiles
// group, group + pos_groups, ...
template <int K, int TH, int TW>
__global__ __launch_bounds__(512) void conv_h16_kernel(const ConvP16Params p) {
    using G = GeoH<K, TH, TW>;
    constexpr int FN = G::FN, CPB = G::CPB;
    extern __shared__ __align__(16) unsigned char lds[];
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
    const int nchunks = p.cin_chunks;
    constexpr int sb_off = 2 * G::BUF;
    constexpr int res_off = sb_off + 2 * CPB * 4;

    if (wave < 4) {   // the first four waves stage: they start first
        h16_stager<G>(p, lds, tid & 255, cb, group, ntiles, nchunks);
        return;
    }

    // ---------------------------------------------------------------------- MFMA waves
    const int mq = lane & 15, kq = lane >> 4;
    const int mw = (wave - 4) % G::WM;   // this wave's 64 output channels of the workgroup's 128
    const int wn = (wave - 4) / G::WM;   // ... and its tile of positions
    int base[FN];    // per-lane LDS offset of the B fragments at tap (0, 0) in staging buffer 0
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = fn * 16 + mq;
        const int ty = m / TW, tx = m - ty * TW;
        base[fn] = ty * G::ROW_PITCH + (wn * TW + tx) * PITCH + kq * 16;
    }
    // A fragments: [(chunk*K + ky)*K + kx][cout fragment of 16][lane] x 8 halves
    const unsigned wstep = (unsigned)p.mfrags * 1024;
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)(cb * (CPB / 16) + mw * HFM) * 1024;   // (uniform)
    const unsigned wlane = lane * 16;
    const unsigned char* wend = wbase + (size_t)nchunks * K * K * wstep;
    half8_t a_q[HPD][HFM];
#pragma unroll
    for (int d = 0; d < HPD - 1; d++)
#pragma unroll
        for (int fm = 0; fm < HFM; fm++) a_q[d][fm] = *reinterpret_cast<const half8_t*>(wbase + (size_t)d * wstep + fm * 1024 + wlane);
#pragma unroll
    for (int fm = 0; fm < HFM; fm++) a_q[HPD - 1][fm] = a_q[0][fm];   // (defined; overwritten by the first step's loads)
    f32x4_t acc[HFM][FN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int fm = 0; fm < HFM; fm++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++) acc[fm][fn] = (f32x4_t)(0.f);
    };
    zero_acc();
    _Float16* out = reinterpret_cast<_Float16*>(p.out);
    const bool have_res = p.res != nullptr;
    const bool res_scale = p.res_scale != 0;
    const float res_floor = p.res_relu ? 0.f : -__builtin_inff();

    auto finish_tile = [&](int tile) {
        const int tyi = (int)(((float)tile + 0.5f) * p.rcp_tiles_x), txi = tile - tyi * p.tiles_x;
        const float* sb = reinterpret_cast<const float*>(lds + sb_off);
        f32x4_t rs[HFM], bi[HFM], scm[HFM];
#pragma unroll
        for (int fm = 0; fm < HFM; fm++) {
            const f32x4_t sc = *reinterpret_cast<const f32x4_t*>(sb + mw * 64 + fm * 16 + kq * 4);
            bi[fm] = *reinterpret_cast<const f32x4_t*>(sb + CPB + mw * 64 + fm * 16 + kq * 4);
            scm[fm] = sc * p.acc_mul;
            rs[fm] = res_scale ? sc : (f32x4_t)(1.f);
        }
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            const int m = fn * 16 + mq;
            const int ty = m / TW, tx = wn * TW + (m - ty * TW);
            const int py = tyi * TH + ty, px = txi * G::TWG + tx;
            const bool ok = py < p.npos_y && px < p.npos_x;
            const size_t obase = ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp + cb * CPB + mw * 64 + kq * 4;
#pragma unroll
            for (int fm = 0; fm < HFM; fm++) {
                f32x4_t v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[fm][fn][e] * scm[fm][e] + bi[fm][e];
                if (have_res) {
                    const half4_t rv = *reinterpret_cast<const half4_t*>(lds + res_off + (ty * G::TWG + tx) * G::RES_PITCH + (mw * 64 + fm * 16 + kq * 4) * 2);
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = fmaf(fmaxf((float)rv[e], res_floor), rs[fm][e], v[e]);
                }
                half4_t hv;
#pragma unroll
                for (int e = 0; e < 4; e++) hv[e] = (_Float16)v[e];
                if (ok) *reinterpret_cast<half4_t*>(out + obase + fm * 16) = hv;
            }
        }
    };

    lds_barrier();   // the first stage is staged
    half8_t b[FN];
    int brow[FN], nxt[FN];
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        brow[fn] = base[fn];
        b[fn] = *reinterpret_cast<const half8_t*>(lds + brow[fn]);
    }
    const unsigned char* wnext = wbase + (size_t)((HPD - 1) % (nchunks * K * K)) * wstep;
    int tile = group, c = 0, buf = 0;
    for (;;) {
        for (int ky = 0; ky < K - 1; ky++) {
#pragma unroll
            for (int fn = 0; fn < FN; fn++) nxt[fn] = brow[fn] + G::ROW_PITCH;
            h16_row<G, false>(acc, a_q, b, brow, nxt, lds, wnext, wbase, wend, wstep, wlane);
#pragma unroll
            for (int fn = 0; fn < FN; fn++) brow[fn] = nxt[fn];
        }
        buf = 1 - buf;
#pragma unroll
        for (int fn = 0; fn < FN; fn++) nxt[fn] = base[fn] + buf * G::BUF;
        h16_row<G, true>(acc, a_q, b, brow, nxt, lds, wnext, wbase, wend, wstep, wlane);
#pragma unroll
        for (int fn = 0; fn < FN; fn++) brow[fn] = nxt[fn];
        if (++c == nchunks) {
            finish_tile(tile);
            c = 0; tile += p.pos_groups;
            if (tile >= ntiles) break;
            zero_acc();
        }
    }
}

struct H16Entry {
    int k, th, tw;
    void (*fn)(const ConvP16Params);
    size_t buf_bytes, res_bytes;
};
template <int K, int TH, int TW>
constexpr H16Entry h16_entry() {
    using G = GeoH<K, TH, TW>;
    return H16Entry{K, TH, TW, conv_h16_kernel<K, TH, TW>, (size_t)(2 * G::BUF + 2 * G::CPB * 4), (size_t)(TH * G::TWG * G::RES_PITCH)};
}
const H16Entry H16_TABLE[] = {
    h16_entry<9, 12, 8>(), h16_entry<9, 8, 8>(), h16_entry<9, 4, 8>(),
    h16_entry<3, 12, 8>(), h16_entry<3, 8, 8>(), h16_entry<3, 4, 8>(),
};
constexpr int H16_COUNT = sizeof(H16_TABLE) / sizeof(H16_TABLE[0]);
const H16Entry* h16_find(const ConvP16Params& p, int k) {
    for (int i = 0; i < H16_COUNT; i++)
        if (H16_TABLE[i].k == k && H16_TABLE[i].th == p.tile_h && H16_TABLE[i].tw == p.tile_w) return &H16_TABLE[i];
    return nullptr;
}
}  // namespace

bool conv_h16_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16_storage) {
    bool have_k = false;
    for (int i = 0; i < H16_COUNT; i++) have_k = have_k || H16_TABLE[i].k == k;
    return f16_storage && have_k && stride == 1 && dil == 1 && in_cp % KC == 0 && cout % 128 == 0 && out_cp >= cout;
}
int conv_h16_tile_count() { return H16_COUNT; }
void conv_h16_tile(int i, int* k, int* th, int* tw) {
    *k = H16_TABLE[i].k; *th = H16_TABLE[i].th; *tw = H16_TABLE[i].tw;
}
size_t conv_h16_lds_bytes(const ConvP16Params& p, int k) {
    const H16Entry* e = h16_find(p, k);
    if (!e) return 0;
    return e->buf_bytes + (p.res ? e->res_bytes : 0);
}
int launch_conv_h16(const ConvP16Params& p, int k, hipStream_t s) {
    const H16Entry* e = h16_find(p, k);
    if (!e) return -1;
    // what the kernel and its grid assume
    if (p.cin_chunks < 1 || p.in_cp < p.cin_chunks * KC || p.mfrags % 8 != 0 || p.cout_blocks * 8 != p.mfrags || p.out_cp < p.cout_blocks * 128 ||
        (p.res && p.res_cp < p.cout_blocks * 128) || (p.res && p.cin_chunks < 2 && p.pos_groups != p.tiles_x * p.tiles_y) ||
        p.pos_groups < 1 || p.pos_groups > p.tiles_x * p.tiles_y || p.tiles_x < 1 || p.tiles_y < 1 || !p.f16 ||
        p.rcp_tiles_x != 1.0f / (float)p.tiles_x || p.tiles_x * p.tiles_y > 4000000 || p.in_cp % 8 != 0 || p.out_cp % 4 != 0 || (p.res && p.res_cp % 8 != 0) ||
        p.tiles_x * 2 * e->tw < p.npos_x || p.tiles_y * e->th < p.npos_y || !p.in || !p.out || !p.wpack || !p.scale || !p.bias)
        return -1;
    const size_t lds = conv_h16_lds_bytes(p, k);
    if (ensure_lds(reinterpret_cast<const void*>(e->fn), lds) != 0) return -2;
    hipLaunchKernelGGL(e->fn, dim3((unsigned)(p.pos_groups * p.cout_blocks)), dim3(512), lds, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace fynhip
