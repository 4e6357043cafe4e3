// Implicit-GEMM convolution on gfx950 matrix cores (v_mfma_f32_32x32x16_f16, fp32 accumulate).
//
// Replaces the additive-blend render passes of DeepConvLayerNxN::forward
// (fyusenet/gpu/deep/deepconvlayerNxN.cpp:129-211), DeepConvLayer1x1::forward
// (deepconvlayer1x1.cpp:67-117), the shallow ConvLayerNxN::forward
// (gpu/vanilla/convlayerNxN_vanilla.cpp:72-141) with its sampler's edge clamp, the fractional-step
// FractionalConvLayerNxN (gpu/vanilla/fractionalconvlayerNxN_vanilla.cpp:43-91; both applied while a
// halo tile is staged: in_clamp, in_shift) and, launched once per output parity, the stencil
// passes of DeepTransConvLayerBase::forward (gpu/deep/deeptransconvlayerbase.cpp:83-130).
//
// GEMM view: M = output channels (A operand = weights, pre-packed per lane in HBM, streamed
// through L2 straight into VGPRs), N = output positions (B operand = activations, staged once per
// input-channel chunk as a halo tile in LDS and re-read for every kernel tap at a shifted address),
// K = taps x input channels.  The activation of the producing layer is applied while staging
// (shaders/activation.inc:3-18 semantics: activation on input fetch).  Epilogue: acc*scale + bias
// (+ residual), the order of shaders/deep/deepconv3x3_tiled.frag:36-45.
//
// Two more sampling and output rules, described at their fields in ConvMfmaParams: strided one-tap layers work in the
// sub-sampled frame (in_sub), and a K x K convolution with at most four output channels can run with its kx taps
// folded into the output channels, the epilogue summing them inside the workgroup (fuse_k).
//
// fp32 storage: both operands are split into fp16 hi + lo parts (x = hi + lo, 22 significant
// bits) and three MFMAs (hi*hi, lo*hi, hi*lo) are issued per fragment pair; fp16 storage: one.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <vector>

#include "kernels.h"
#include "range.h"


namespace fynhip {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Branch-free activation: the host normalises every activation kind to
//   act(x) = min(hi, max(lo, x)) + leak * min(x, 0)
// (none: lo=-inf, hi=+inf, leak=0; ReLU: lo=0; leaky: lo=0, leak; clip: lo, hi).
// (the clamp is one median-of-three instruction: lo <= hi always)
__device__ __forceinline__ float act_apply(float x, const Act& a) {
    return __builtin_amdgcn_fmed3f(x, a.lo, a.hi) + a.leak * fminf(x, 0.f);
}

template <typename T>
__device__ __forceinline__ void load_vals(const T* src, float* v, int n);
template <>
__device__ __forceinline__ void load_vals<float>(const float* src, float* v, int n) {
    float4 a = *reinterpret_cast<const float4*>(src);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    if (n == 8) {
        float4 b = *reinterpret_cast<const float4*>(src + 4);
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
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

// Raw (unconverted) staging item as it comes from HBM/L2: CPI channels of one pixel.
template <typename T, int CPI>
struct RawItem;
template <>
struct RawItem<float, 8> {
    float4 a, b;
    __device__ __forceinline__ void zero() { a = b = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ void load(const float* p) {
        a = *reinterpret_cast<const float4*>(p);
        b = *reinterpret_cast<const float4*>(p + 4);
    }
    __device__ __forceinline__ void get(float* v) const {
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
};
template <>
struct RawItem<float, 4> {
    float4 a;
    __device__ __forceinline__ void zero() { a = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ void load(const float* p) { a = *reinterpret_cast<const float4*>(p); }
    __device__ __forceinline__ void get(float* v) const { v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; }
};
template <>
struct RawItem<_Float16, 8> {
    half8_t a;
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 8; i++) a[i] = (_Float16)0.f;
    }
    __device__ __forceinline__ void load(const _Float16* p) { a = *reinterpret_cast<const half8_t*>(p); }
    __device__ __forceinline__ void get(float* v) const {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)a[i];
    }
};
template <>
struct RawItem<_Float16, 4> {
    half4_t a;
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 4; i++) a[i] = (_Float16)0.f;
    }
    __device__ __forceinline__ void load(const _Float16* p) { a = *reinterpret_cast<const half4_t*>(p); }
    __device__ __forceinline__ void get(float* v) const {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = (float)a[i];
    }
};

// Activates, converts (hi / lo fp16 planes when SPLIT) and writes one staging item to LDS.
// (SPLIT: `scale` is the power of two that moves the tensor's magnitudes into the window where hi + lo is exact)
template <bool SPLIT, int CPI>
__device__ __forceinline__ void stage_store(unsigned char* dst, int plane, const float* raw, const Act& act, float scale) {
    float v[8];
#pragma unroll
    for (int i = 0; i < CPI; i++) v[i] = SPLIT ? act_apply(raw[i], act) * scale : act_apply(raw[i], act);
    if (CPI == 8) {
        half8_t hi;
#pragma unroll
        for (int i = 0; i < 8; i++) hi[i] = (_Float16)v[i];
        *reinterpret_cast<half8_t*>(dst) = hi;
        if (SPLIT) {
            half8_t lo;
#pragma unroll
            for (int i = 0; i < 8; i++) lo[i] = (_Float16)(v[i] - (float)hi[i]);
            *reinterpret_cast<half8_t*>(dst + plane) = lo;
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
            *reinterpret_cast<half4_t*>(dst + plane) = lo;
        }
    }
}

// Per-step LDS offset(s) of the B fragments.  Chunks of 8 or more channels: one offset per step, a lane's 8 halves
// are consecutive channels of one tap.  Small-Cin layout (KC == 4, pixels of 4 channels = 8 bytes): a lane's 8 halves
// are two taps, each with an offset of its own (taps are packed densely, four per k16 step, whatever their
// positions), selected by the lane's half of the wavefront.
template <int KC>
struct StepOff {
    int v;
};
template <>
struct StepOff<4> {
    int2 v;
};
template <int KC>
__device__ __forceinline__ StepOff<KC> load_step_off(const int* steptab, int step, int lane) {
    StepOff<KC> r;
    if constexpr (KC == 4) r.v = reinterpret_cast<const int2*>(steptab)[2 * step + (lane >> 5)];
    else r.v = steptab[step];
    return r;
}

// One B (activation) fragment of a lane: 8 halves.
template <int KC>
__device__ __forceinline__ half8_t load_b_frag(const unsigned char* base, const StepOff<KC>& ao) {
    if constexpr (KC == 4) {
        const half4_t lo4 = *reinterpret_cast<const half4_t*>(base + ao.v.x);
        const half4_t hi4 = *reinterpret_cast<const half4_t*>(base + ao.v.y);
        half8_t r;
        r[0] = lo4[0]; r[1] = lo4[1]; r[2] = lo4[2]; r[3] = lo4[3];
        r[4] = hi4[0]; r[5] = hi4[1]; r[6] = hi4[2]; r[7] = hi4[3];
        return r;
    } else {
        return *reinterpret_cast<const half8_t*>(base + ao.v);
    }
}

template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN, int KC, int PD, int UNR>
__device__ __forceinline__ void conv_mfma_body(const ConvMfmaParams& p, unsigned char* lds) {
    // Tiles with two or more fragments per wave run one MFMA wave per SIMD; such workgroups get four more
    // waves (threads 256..511) that do nothing but stage the next input chunk (global loads, activation,
    // fp32 -> fp16 hi/lo conversion, LDS writes), so that this work shares the SIMDs with the MFMA waves
    // instead of interrupting them.  Single-fragment tiles (two to three workgroups per CU) stage with the
    // MFMA waves themselves.
    constexpr bool SPEC = FM * FN >= 2;
    constexpr int NPL = SPLIT ? 2 : 1;         // operand planes (hi, lo)
    constexpr int CPI = (KC == 4) ? 4 : 8;     // channels per staging item
    constexpr int G = (KC == 4) ? 1 : KC / 8;  // staging items per pixel
    // The four MFMA waves are arranged WM x WN over the tile; when WM*WN < 4 the remaining factor WK splits the
    // k16 steps of every chunk among waves that share an output sub-tile (their accumulators meet in LDS in the
    // epilogue): small tiles keep four waves busy and the reduction of a layer with few positions is spread
    // over more workgroups without a second pass.
    static_assert(WM * WN == 1 || WM * WN == 2 || WM * WN == 4, "1, 2 or 4 sub-tiles per block");
    constexpr int WK = 4 / (WM * WN);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps tile/fragment index math scalar
    const bool consumer = !SPEC || wave < 4;   // issues MFMAs, owns accumulators, writes the output
    const bool stager = !SPEC || wave >= 4;    // stages input tiles
    const int stid = SPEC ? (tid & 255) : tid; // thread index among the staging threads
    const int wm = (wave & 3) % WM;
    const int wn = ((wave & 3) / WM) % WN;
    const int wk = (wave & 3) / (WM * WN);      // 0 when WK == 1

    // Workgroups are dealt round-robin to the 8 XCDs; remap so that neighbouring tiles (shared
    // halos, same input tile for all cout blocks) meet in one XCD's L2.
    int bid = blockIdx.x;
    {
        const int nblk = p.tiles_x * p.tiles_y * p.cout_blocks * (p.ksplit > 1 ? p.ksplit : 1);
        if (bid >= nblk) return;   // rows are as long as the largest member
        const int per = nblk >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    // value ranges (range.h): read the input tensor's record (the records in this launch's care are cleared by the
    // kernel entry points)
    float in_scale = 1.f, inv_in_scale = 1.f;   // (set once the first tile's loads are on their way)
    const unsigned range_bits = (SPLIT && p.in_amax) ? range_load(p.in_amax) : 0u;
    const int ntile_blocks = p.tiles_x * p.tiles_y * p.cout_blocks;
    const int ks = bid / ntile_blocks;           // split-K slice (0 without split-K)
    bid -= ks * ntile_blocks;
    const int cb = bid % p.cout_blocks;
    const int tile = bid / p.cout_blocks;
    const int tyi = tile / p.tiles_x;
    const int txi = tile - tyi * p.tiles_x;
    const int twl = p.tile_w_log2;
    const int TW = 1 << twl;
    const int pos_y0 = tyi * p.tile_h;
    const int pos_x0 = txi * (TW - (p.fuse_k ? p.fuse_k - 1 : 0));

    const int npix = p.halo_h * p.halo_w;
    const int nitems = npix * G;
    const int gy0 = pos_y0 * p.in_stride + p.in_y0;
    const int gx0 = pos_x0 * p.in_stride + p.in_x0;
    const float inv_hw = 1.0f / (float)p.halo_w;
    // frame that gy0/gx0 and the taps count in, and its step and origin in the stored frame
    const int vhp = p.in_sub ? p.npos_y : p.in_hp << p.in_shift, vwp = p.in_sub ? p.npos_x : p.in_wp << p.in_shift;
    const int gstep = p.in_sub ? p.in_sub : 1;
    const TIn* in = reinterpret_cast<const TIn*>(p.in);

    // LDS holds two staging buffers (double buffering across channel chunks) when there is more
    // than one chunk; each buffer = NPL planes.
    const int bufsz = NPL * p.plane;

    // per-lane LDS byte offsets of the B (activation) fragments
    int boff[FN];
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        const int m = (wn * FN + fn) * 32 + (lane & 31);
        const int ty = m >> twl, tx = m & (TW - 1);
        boff[fn] = (ty * p.in_stride) * p.row_pitch + (tx * p.in_stride) * p.pitch + ((KC == 4) ? 0 : (lane >> 5) * 16);
    }

    // A (weight) fragments: [(chunk*nsteps + step)][mfrag][plane][lane] x 8 halves
    // (uniform base + per-lane 32-bit offset: the loads use the scalar-base addressing form and stepping
    // through K costs two scalar adds; the buffer has PD steps of zero slack behind the last step, so the
    // prefetch needs no clamp)
    const unsigned wstep = (unsigned)p.mfrags * NPL * 1024;   // bytes per k16 step
    const int chunk0 = ks * p.chunks_per_split;                // this workgroup's channel chunks: [chunk0, chunk1)
    const int chunk1 = (chunk0 + p.chunks_per_split < p.cin_chunks) ? chunk0 + p.chunks_per_split : p.cin_chunks;
    // (WK > 1: the steps of wave group wk are stored as a contiguous run over all chunks, [wk][chunk][step of the group])
    const int nsub = p.nsteps / WK;                            // steps per chunk of this wave
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(p.wpack) + (size_t)((cb * WM + wm) * FM) * NPL * 1024 +
                                 ((size_t)wk * p.cin_chunks + chunk0) * nsub * wstep;
    const unsigned wlane = lane * 16;

    float16_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // A fragments are prefetched PD-1 steps ahead into a register ring that is indexed statically (the
    // step loop is unrolled PD-fold; nsteps is a multiple of PD): with one to three waves per SIMD the L2
    // round trip of a weight fragment is several times longer than one step's MFMAs.
    half8_t a_q[PD][FM][NPL];
    if (consumer)
#pragma unroll
    for (int d = 0; d < PD; d++) {
        const unsigned char* w_ = wbase + (size_t)d * wstep;
#pragma unroll
        for (int fm = 0; fm < FM; fm++)
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) a_q[d][fm][pl] = *reinterpret_cast<const half8_t*>(w_ + (fm * NPL + pl) * 1024 + wlane);
    }
    // LDS byte offsets of the (up to 256) k16 steps of a chunk: a 1 KB table at the start of LDS.  A step
    // reads the entry of step t+2 with an ordinary (asynchronous) LDS load into a VGPR; the value is only
    // consumed one step later, so the lookup never stalls the instruction stream.
    int* steptab = reinterpret_cast<int*>(lds);
    if (tid < p.nsteps * ((KC == 4) ? 4 : 1)) steptab[tid] = p.aoff[tid];   // (KC == 4: four tap offsets per step)
    __shared__ unsigned range_box[2];   // meeting point of the waves' output maxima (range.h); zero before the first barrier
    if (tid < 2) range_box[tid] = 0u;
    unsigned char* const sbase = lds + 1024;   // staging buffers follow the table

    // ---- staging machinery: items (pixel, 8-channel group) of the halo tile; the first NB items of a
    //      thread are described once (their addresses only shift by the chunk's channel offset) and
    //      are fetched for chunk c+1 while the MFMAs of chunk c run ----
    constexpr int NB = (KC >= 64) ? 8 : 4;
    int g_off[NB];   // element offset of the pixel in the input tensor, -1: outside (reads as 0)
    int l_off[NB];   // LDS byte offset inside a plane, -1: no such item
    int c_off[NB];   // channel offset of the group inside a chunk
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int idx = stid + i * 256;
        g_off[i] = -1; l_off[i] = -1; c_off[i] = 0;
        if (idx < nitems) {
            const int pix = (G == 1) ? idx : idx / G;
            const int g = (G == 1) ? 0 : idx - pix * G;
            const int py = (int)(((float)pix + 0.5f) * inv_hw);
            const int px = pix - py * p.halo_w;
            int gy = gy0 + py, gx = gx0 + px;
            l_off[i] = py * p.row_pitch + px * p.pitch + g * 16;
            c_off[i] = g * CPI;
            if (p.in_clamp) {
                gy = min(max(gy, 0), vhp - 1);
                gx = min(max(gx, 0), vwp - 1);
            }
            if ((unsigned)gy < (unsigned)vhp && (unsigned)gx < (unsigned)vwp) g_off[i] = (((gy >> p.in_shift) * gstep + p.in_oy) * p.in_wp + (gx >> p.in_shift) * gstep + p.in_ox) * p.in_cp;
        }
    }
    RawItem<TIn, CPI> raw[NB];
    // The loads are unconditional (items outside the tensor read its first element and are zeroed when
    // stored), so that the number of loads in flight is known at compile time.
    auto fetch_first = [&](int chunk_) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int c0 = chunk_ * KC + c_off[i];
            const bool ok = g_off[i] >= 0 && c0 < p.in_cp;
            raw[i].load(in + (ok ? g_off[i] + c0 : 0));
        }
    };
    auto store_first = [&](int chunk_, unsigned char* buf) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            if (l_off[i] >= 0) {
                const int c0 = chunk_ * KC + c_off[i];
                const bool ok = g_off[i] >= 0 && c0 < p.in_cp;
                float v[8];
                raw[i].get(v);
#pragma unroll
                for (int e = 0; e < CPI; e++) v[e] = ok ? v[e] : 0.f;
                stage_store<SPLIT, CPI>(buf + l_off[i], p.plane, v, p.act, in_scale);
            }
        }
    };
    // items beyond the first NB*256 (large halo tiles) are staged without prefetch, NB at a time
    auto stage_rest = [&](int chunk, unsigned char* buf) {
        for (int base = NB * 256; base < nitems; base += NB * 256) {
            RawItem<TIn, CPI> r2[NB];
            int lo2[NB];
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int idx = base + stid + i * 256;
                lo2[i] = -1;
                r2[i].zero();
                if (idx < nitems) {
                    const int pix = (G == 1) ? idx : idx / G;
                    const int g = (G == 1) ? 0 : idx - pix * G;
                    const int py = (int)(((float)pix + 0.5f) * inv_hw);
                    const int px = pix - py * p.halo_w;
                    int gy = gy0 + py, gx = gx0 + px;
                    const int c0 = chunk * KC + g * CPI;
                    lo2[i] = py * p.row_pitch + px * p.pitch + g * 16;
                    if (p.in_clamp) {
                        gy = min(max(gy, 0), vhp - 1);
                        gx = min(max(gx, 0), vwp - 1);
                    }
                    if ((unsigned)gy < (unsigned)vhp && (unsigned)gx < (unsigned)vwp && c0 < p.in_cp)
                        r2[i].load(in + (((gy >> p.in_shift) * gstep + p.in_oy) * p.in_wp + (gx >> p.in_shift) * gstep + p.in_ox) * p.in_cp + c0);
                }
            }
#pragma unroll
            for (int i = 0; i < NB; i++) {
                if (lo2[i] >= 0) {
                    float v[8];
                    r2[i].get(v);
                    stage_store<SPLIT, CPI>(buf + lo2[i], p.plane, v, p.act, in_scale);
                }
            }
        }
    };

    // prologue: chunk 0 into buffer 0
    if (stager) fetch_first(chunk0);
    if (SPLIT && p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_bits), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;
    if (stager) {
        store_first(chunk0, sbase);
        stage_rest(chunk0, sbase);
    }
    __syncthreads();

    // ---- main loop: channel chunks, each nsteps k16 steps in groups of PD.  B fragments of step t+1 are
    //      read from LDS while the MFMAs of step t run; the next chunk's tile is fetched from HBM/L2 at the
    //      start of a chunk and converted into the other LDS buffer at its end, one barrier per chunk. ----
    const unsigned char* wnext = wbase + (size_t)(PD - 1) * wstep;   // next ring refill: step PD-1 (again), PD, ...
    // B fragments ping-pong between two statically indexed register sets (PD is even, so the set of a
    // step is the parity of its position in the group): the LDS reads of step t+1 are issued before the
    // MFMAs of step t and nothing is copied.
    static_assert(PD % 2 == 0 && UNR % PD == 0, "the B fragment ping-pong needs an even step group; the unrolled group covers whole ring turns");
    half8_t b_buf[2][FN][NPL];
    unsigned char* cur = sbase;
    // step offsets of the next two steps (ping-pong like the B fragments)
    StepOff<KC> ao_reg[2];
    const int tab0 = wk * nsub;                                // this wave's first step in the table
    ao_reg[0] = load_step_off<KC>(steptab, tab0, lane);
    ao_reg[1] = load_step_off<KC>(steptab, tab0 + (nsub > 1 ? 1 : 0), lane);
    // PD steps starting at step t0 of the current chunk.  The body is branch-free (after the chunk's last
    // step the B prefetch re-reads step 0, unused) and written as one slot per MFMA: the MFMA, then a share
    // of the step's memory instructions -- LDS reads of the B fragments of step t+1, and the refill of the
    // ring slot used by step t-1 with the A fragments of step t+PD-1 -- fenced so that the compiler keeps
    // this order.  A memory instruction issued right after an MFMA runs in that MFMA's shadow; a block of
    // memory instructions between two MFMAs leaves the matrix pipe idle (one wave cannot queue MFMAs).
    constexpr int NMF = FM * FN * (SPLIT ? 3 : 1);     // MFMAs per step
    constexpr int NDS = FN * NPL;                      // B fragment reads per step
    constexpr int NVM = FM * NPL;                      // A fragment loads per step
    auto run_group = [&](int t0) {
#pragma unroll
        for (int dd = 0; dd < UNR; dd++) {
            const int d = dd % PD;                            // ring slot of this step
            const StepOff<KC> ao = ao_reg[(dd + 1) & 1];      // offset of step t+1 (loaded one step ago)
            const int t2 = t0 + dd + 2;                       // the table wraps: the next chunk starts at step 0 again
            const int step2 = tab0 + (t2 < nsub ? t2 : t2 - nsub);
            const int dprev = (d + PD - 1) % PD;       // ring slot of the previous step: free for refill
            const unsigned char* w_ = wnext;                  // fragments of step gs+PD-1
            wnext += wstep;
#pragma unroll
            for (int i = 0; i < NMF; i++) {
                const int kind = i / (FM * FN), rem = i % (FM * FN);
                const int fm = rem / FN, fn = rem % FN;
                const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
                acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_q[d][fm][apl], b_buf[dd & 1][fn][bpl], acc[fm][fn], 0, 0, 0);
                if (i == 0) ao_reg[dd & 1] = load_step_off<KC>(steptab, step2, lane);   // this parity's old value (step t) was consumed during step t-1
#pragma unroll
                for (int j = i * NDS / NMF; j < (i + 1) * NDS / NMF; j++)   // plane 0 of all fragments first
                    b_buf[(dd + 1) & 1][j % FN][j / FN] = load_b_frag<KC>(cur + (j / FN) * p.plane + boff[j % FN], ao);
#pragma unroll
                for (int j = i * NVM / NMF; j < (i + 1) * NVM / NMF; j++)
                    a_q[dprev][j % FM][j / FM] = *reinterpret_cast<const half8_t*>(w_ + ((j % FM) * NPL + j / FM) * 1024 + wlane);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // One loop per role where the roles are separate waves: a wave's registers then hold either the staging items or
    // the fragments and accumulators, not both (the two kinds of waves execute the same barriers, one per chunk).
    if (SPEC && !consumer) {
        for (int chunk = chunk0; chunk < chunk1; chunk++) {
            const bool more_chunks = chunk + 1 < chunk1;
            if (more_chunks) {
                fetch_first(chunk + 1);
                unsigned char* nxt = sbase + ((chunk - chunk0 + 1) & 1) * bufsz;
                store_first(chunk + 1, nxt);
                stage_rest(chunk + 1, nxt);
                __syncthreads();  // everyone is done reading the current buffer and writing `nxt`
            }
        }
    } else {
        for (int chunk = chunk0; chunk < chunk1; chunk++) {
            const bool more_chunks = chunk + 1 < chunk1;
            // (after the last chunk the fetch is unused; it keeps the number of loads in flight static)
            if (!SPEC) fetch_first(more_chunks ? chunk + 1 : chunk);
            {
                const StepOff<KC> ao = ao_reg[0];
#pragma unroll
                for (int fn = 0; fn < FN; fn++)
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++) b_buf[0][fn][pl] = load_b_frag<KC>(cur + pl * p.plane + boff[fn], ao);
                for (int t0 = 0; t0 < nsub; t0 += UNR) run_group(t0);
            }
            if (more_chunks) {
                unsigned char* nxt = sbase + ((chunk - chunk0 + 1) & 1) * bufsz;
                if (!SPEC) {
                    store_first(chunk + 1, nxt);
                    stage_rest(chunk + 1, nxt);
                }
                __syncthreads();  // everyone is done reading `cur` and writing `nxt`
                cur = nxt;
            }
        }
    }

    // ---- epilogue.  A lane holds, per fragment, column (position) lane%32 and rows (channels)
    //      8*(r/4) + 4*(lane/32) + r%4.  The wave transposes its accumulators through a private LDS area
    //      so that it writes, per position, one contiguous run of FM*32 channels (128-256 B) instead of
    //      16-byte pieces; scale, bias' and the residual are applied on the way out
    //      (shaders/deep/deepconv3x3_tiled.frag:36-45 order). ----
    __syncthreads();  // all waves are done with the staged tiles; LDS is reused below
    constexpr int ROWF = FM * 32 + 4;                 // floats per position row (+4: bank spread)
    constexpr int LPP = FM * 8;                       // lanes per position on the way out
    constexpr int PPI = 64 / LPP;                     // positions per store instruction
    constexpr int ITS = 32 / PPI;                     // store instructions per fragment ...
    constexpr int ITW = ITS / WK;                     // ... of which a wave issues this many (K groups share the rows out)
    static_assert(ITS % WK == 0, "rows of a fragment divide among the K groups");
    float* tr = reinterpret_cast<float*>(lds) + (wave & 3) * (FN * 32 * ROWF);   // FN fragments of 32 rows per wave
    auto acc_to_lds = [&]() {
#pragma unroll
        for (int fn = 0; fn < FN; fn++)
#pragma unroll
            for (int fm = 0; fm < FM; fm++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    f32x4_t v;
                    v[0] = acc[fm][fn][q * 4 + 0]; v[1] = acc[fm][fn][q * 4 + 1];
                    v[2] = acc[fm][fn][q * 4 + 2]; v[3] = acc[fm][fn][q * 4 + 3];
                    *reinterpret_cast<f32x4_t*>(tr + (fn * 32 + (lane & 31)) * ROWF + fm * 32 + q * 8 + (lane >> 5) * 4) = v;
                }
    };
    // With K groups, every wave first publishes its partial accumulators; a wave then finishes the rows
    // it = i*WK + wk of its sub-tile, adding the groups' partial sums in group order.
    if constexpr (WK > 1) {
        if (consumer) acc_to_lds();
        __syncthreads();
    }
    if constexpr (FM == 1 && WM == 1 && WN == 4) {
        if (p.fuse_k) {
            // Folded kx taps: position m of the tile is row m of the transposed accumulators (the four waves' areas
            // are consecutive), its virtual channels are consecutive floats.  Every thread sums whole outputs.
            if (consumer) acc_to_lds();
            __syncthreads();
            if (!consumer) return;
            const int K = p.fuse_k, nox = TW - K + 1, ow = p.npos_x - (K - 1);
            const float* q = reinterpret_cast<const float*>(lds);
            TOut* outp = reinterpret_cast<TOut*>(p.out);
            const TOut* resp = reinterpret_cast<const TOut*>(p.res);
            float sc4[4], bi4[4];
#pragma unroll
            for (int o = 0; o < 4; o++) {
                sc4[o] = o < p.fuse_cout ? p.scale[o] : 0.f;
                bi4[o] = o < p.fuse_cout ? p.bias[o] : 0.f;
            }
            const float inv_nox = 1.0f / (float)nox;
            float vmax = 0.f;
            for (int idx = tid & 255; idx < p.tile_h * nox; idx += 256) {
                const int ty = (int)(((float)idx + 0.5f) * inv_nox);
                const int tx = idx - ty * nox;
                const int py = pos_y0 + ty, px = pos_x0 + tx;
                if (py >= p.npos_y || px >= ow) continue;
                float a[4] = {0.f, 0.f, 0.f, 0.f};
                const float* row = q + ((ty << twl) + tx) * ROWF;
                for (int kx = 0; kx < K; kx++) {
#pragma unroll
                    for (int o = 0; o < 4; o++)
                        if (o < p.fuse_cout) a[o] += row[kx * ROWF + o * K + kx];
                }
                float rv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (resp) load_vals<TOut>(resp + ((size_t)(p.res_off_y + py) * p.res_wp + p.res_off_x + px) * p.res_cp, rv, 4);
                f32x4_t v;
#pragma unroll
                for (int o = 0; o < 4; o++) {
                    float r = rv[o];
                    if (p.res_relu) r = fmaxf(r, 0.f);
                    if (p.res_scale) r *= sc4[o];
                    v[o] = o < p.fuse_cout ? ((a[o] * acc_mul) * sc4[o] + bi4[o]) + r : 0.f;
                    vmax = fmaxf(vmax, fabsf(v[o]));
                }
                const size_t oidx = ((size_t)(p.out_off_y + py) * p.out_wp + p.out_off_x + px) * p.out_cp;
                if (sizeof(TOut) == 4) {
                    *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(outp) + oidx) = v;
                } else {
                    half4_t hv;
#pragma unroll
                    for (int o = 0; o < 4; o++) hv[o] = (_Float16)v[o];
                    *reinterpret_cast<half4_t*>(reinterpret_cast<_Float16*>(outp) + oidx) = hv;
                }
            }
            if (SPLIT && p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 4);
            return;
        }
    }
    if (!consumer) return;
    const float* tr0 = reinterpret_cast<const float*>(lds) + ((wave & 3) % (WM * WN)) * (FN * 32 * ROWF);   // K group 0's area of this sub-tile
    constexpr int TRK = WM * WN * FN * 32 * ROWF;     // floats between the areas of consecutive K groups
    auto row_from_lds = [&](int fn, int it) {
        f32x4_t v = *reinterpret_cast<const f32x4_t*>(tr0 + (fn * 32 + it * PPI + lane / LPP) * ROWF + (lane % LPP) * 4);
#pragma unroll
        for (int k = 1; k < WK; k++) v += *reinterpret_cast<const f32x4_t*>(tr0 + k * TRK + (fn * 32 + it * PPI + lane / LPP) * ROWF + (lane % LPP) * 4);
        return v;
    };
    TOut* out = reinterpret_cast<TOut*>(p.out);
    const TOut* res = reinterpret_cast<const TOut*>(p.res);
    const int c4 = (lane % LPP) * 4;                                   // channel offset inside the wave's range
    const int c = ((cb * WM + wm) * FM) * 32 + c4;                     // absolute output channel
    const bool c_ok = c < p.out_cp;
    f32x4_t sc = (f32x4_t)(0.f), bi = (f32x4_t)(0.f);
    if (c_ok) {
        sc = *reinterpret_cast<const f32x4_t*>(p.scale + c);
        bi = *reinterpret_cast<const f32x4_t*>(p.bias + c);
    }
    // Phases instead of a per-fragment round trip (one wave per SIMD cannot hide latencies behind other
    // waves): (1) all residual loads, (2) all accumulators into LDS, (3) all rows back, (4) arithmetic and
    // stores.
    if (p.ksplit > 1) {
        // split-K: raw partial sums, [ks][position][cout_pad] fp32; the reduce pass finishes the layer
        float* part = p.partial + (size_t)ks * p.npos_y * p.npos_x * p.cout_pad;
        const bool cp_ok = c < p.cout_pad;
        if constexpr (WK == 1) acc_to_lds();
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
#pragma unroll
            for (int i = 0; i < ITW; i++) {
                const int it = (WK == 1) ? i : i * WK + wk;
                const int row = it * PPI + lane / LPP;
                f32x4_t v = row_from_lds(fn, it);
                if (SPLIT) v *= inv_in_scale;   // partial sums in the units the reduce pass expects (a power of two)
                const int m = (wn * FN + fn) * 32 + row;
                const int py = pos_y0 + (m >> twl), px = pos_x0 + (m & (TW - 1));
                if (cp_ok && py < p.npos_y && px < p.npos_x)
                    *reinterpret_cast<f32x4_t*>(part + ((size_t)py * p.npos_x + px) * p.cout_pad + c) = v;
            }
        }
        return;
    }
    // Row r of a fragment is position m = frag*32 + it*PPI + lane/LPP; PPI divides the tile width, so the
    // tile row (and with it the image row) of an (fn, it) pair is wave-uniform and only the column carries a
    // per-lane part: base addresses are scalar, the per-lane offset is computed once.
    const int lrow = lane / LPP;
    const int out_lane = lrow * p.out_step * p.out_cp + c;
    const int res_lane = lrow * p.out_step * p.res_cp + c;
    bool ok[FN][ITW];
    size_t obase[FN][ITW];
    float rres[FN][ITW][4];
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int it = 0; it < ITW; it++) {
            const int m0 = (wn * FN + fn) * 32 + ((WK == 1) ? it : it * WK + wk) * PPI;
            const int py = pos_y0 + (m0 >> twl), px0 = pos_x0 + (m0 & (TW - 1));
            ok[fn][it] = c_ok && py < p.npos_y && px0 + lrow < p.npos_x;
            obase[fn][it] = ((size_t)(p.out_off_y + py * p.out_step) * p.out_wp + p.out_off_x + px0 * p.out_step) * p.out_cp + out_lane;
#pragma unroll
            for (int i = 0; i < 4; i++) rres[fn][it][i] = 0.f;
            if (res && ok[fn][it]) {
                const size_t rbase = ((size_t)(p.res_off_y + py * p.out_step) * p.res_wp + p.res_off_x + px0 * p.out_step) * p.res_cp + res_lane;
                float r[8];
                load_vals<TOut>(res + rbase, r, 4);
#pragma unroll
                for (int i = 0; i < 4; i++) rres[fn][it][i] = r[i];
            }
        }
    if constexpr (WK == 1) acc_to_lds();
    f32x4_t a4[FN][ITW];
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int it = 0; it < ITW; it++) a4[fn][it] = row_from_lds(fn, (WK == 1) ? it : it * WK + wk);
    // arithmetic for every row unconditionally (one wait for the loads above), then predicated stores only:
    // a wait inside a predicated region would also wait for the stores issued before it
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int it = 0; it < ITW; it++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float rv = rres[fn][it][i];   // zero without a residual input
                if (p.res_relu) rv = fmaxf(rv, 0.f);
                if (p.res_scale) rv *= sc[i];
                a4[fn][it][i] = ((a4[fn][it][i] * acc_mul) * sc[i] + bi[i]) + rv;
            }
    // pin the results in registers here: the compiler would otherwise sink the arithmetic (and the waits for
    // its inputs) into the predicated store regions below
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int it = 0; it < ITW; it++) asm volatile("" : "+v"(a4[fn][it]));
    if (SPLIT && p.out_amax) {
        float vmax = 0.f;
#pragma unroll
        for (int fn = 0; fn < FN; fn++)
#pragma unroll
            for (int it = 0; it < ITW; it++)
#pragma unroll
                for (int i = 0; i < 4; i++) vmax = fmaxf(vmax, ok[fn][it] ? fabsf(a4[fn][it][i]) : 0.f);
        range_publish_waves(p.out_amax, vmax, range_box, 4);
    }
#pragma unroll
    for (int fn = 0; fn < FN; fn++)
#pragma unroll
        for (int it = 0; it < ITW; it++) {
            if (!ok[fn][it]) continue;
            if (sizeof(TOut) == 4) {
                *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + obase[fn][it]) = a4[fn][it];
            } else {
                half4_t hv;
#pragma unroll
                for (int i = 0; i < 4; i++) hv[i] = (_Float16)a4[fn][it][i];
                *reinterpret_cast<half4_t*>(reinterpret_cast<_Float16*>(out) + obase[fn][it]) = hv;
            }
        }
}

// Entry points: one convolution per launch (parameters by value), or up to four sub-convolutions of one layer
// per launch (grid row blockIdx.y works on sub[blockIdx.y]; rows are as long as the largest member).
template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN, int KC, int PD, int UNR>
__global__ __launch_bounds__((FM * FN >= 2) ? 512 : 256) void conv_mfma_kernel(const ConvMfmaParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    if (blockIdx.x == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    conv_mfma_body<TIn, TOut, SPLIT, FM, FN, WM, WN, KC, PD, UNR>(p, lds);
}

template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN, int KC, int PD, int UNR>
__global__ __launch_bounds__((FM * FN >= 2) ? 512 : 256) void conv_mfma_multi_kernel(const ConvMfmaMulti P) {
    extern __shared__ __align__(16) unsigned char lds[];
    if (blockIdx.x == 0 && blockIdx.y == 0) range_clear(P.sub[0].reset[0], P.sub[0].reset[1], P.sub[0].reset[2], P.sub[0].reset[3], P.sub[0].nreset);
    conv_mfma_body<TIn, TOut, SPLIT, FM, FN, WM, WN, KC, PD, UNR>(P.sub[blockIdx.y], lds);
}

// ---------------------------------------------------------------------------------------------
// variant table.  This file is compiled FYN_CONV_PARTS times with -DFYN_CONV_PART=0..N-1 (in parallel);
// every part instantiates the kernels of the tiles whose table index is congruent to it, and part 0
// also holds the dispatcher.
// ---------------------------------------------------------------------------------------------
typedef void (*conv_kernel_fn)(const ConvMfmaParams);
typedef void (*conv_multi_fn)(const ConvMfmaMulti);
struct ConvEntry {
    conv_kernel_fn single = nullptr;
    conv_multi_fn multi = nullptr;   // may be absent for a variant
};

#ifndef FYN_CONV_PARTS
#define FYN_CONV_PARTS 1
#endif
#ifndef FYN_CONV_PART
#define FYN_CONV_PART 0
#endif

// (index, fm, fn, wm, wn): cout tile = wm*fm*32, position tile = wn*fn*32; wm*wn < 4: the other waves split K
#define FYN_CONV_TILES(X) \
    X(0, 2, 2, 2, 2)      \
    X(1, 2, 2, 1, 4)      \
    X(2, 2, 1, 2, 2)      \
    X(3, 2, 1, 1, 4)      \
    X(4, 1, 2, 1, 4)      \
    X(5, 1, 1, 1, 4)      \
    X(6, 1, 1, 4, 1)      \
    X(7, 1, 1, 2, 2)      \
    X(8, 1, 2, 4, 1)      \
    X(9, 1, 3, 4, 1)      \
    X(10, 1, 4, 4, 1)     \
    X(11, 1, 2, 2, 2)     \
    X(12, 1, 4, 2, 2)     \
    X(13, 1, 3, 2, 2)     \
    X(14, 1, 4, 1, 4)     \
    X(15, 1, 3, 1, 4)     \
    X(16, 1, 1, 1, 1)     \
    X(17, 1, 1, 2, 1)     \
    X(18, 1, 1, 1, 2)

// (ring depth, unroll) pairs: 2/2 for chunks of 4, 16 and 32 channels; for 32-channel chunks also 4/4, 6/6 and
// 6/18 (a whole 3x3 chunk unrolled: no loop back-edge, hence no conservative wait, inside a chunk); 64- and
// 128-channel chunks (kernels of one to four taps: fewer chunk barriers) use 4/4 and 4/8.
template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN>
static conv_kernel_fn pick_kc(int kc, int pd, int unr) {
    if constexpr (WM * WN < 4) {   // K-split tiles: layers with few positions and many channels; smallest step group only
        if (kc == 32 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 2, 2>;
        if (kc == 64 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 64, 2, 2>;
        if (kc == 128 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 128, 2, 2>;
        // pointwise layers with many input channels: chunks of 256 to 1024 channels, so that a workgroup fetches its
        // whole reduction in one or two memory round trips instead of one per 128 channels
        if (kc == 256 && pd == 4 && unr == 4) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 256, 4, 4>;
        if (kc == 512 && pd == 4 && unr == 4) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 512, 4, 4>;
        if (kc == 1024 && pd == 4 && unr == 4) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 1024, 4, 4>;
        return nullptr;
    } else {
    if (kc == 4 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 4, 2, 2>;
    if (kc == 16 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 16, 2, 2>;
    if (kc == 32 && pd == 2 && unr == 2) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 2, 2>;
    if (kc == 32 && pd == 4 && unr == 4) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 4, 4>;
    if (kc == 32 && pd == 6 && unr == 6) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 6, 6>;
    if (kc == 32 && pd == 6 && unr == 18) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 6, 18>;
    if (kc == 64 && pd == 4 && unr == 4) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 64, 4, 4>;
    if (kc == 128 && pd == 4 && unr == 8) return conv_mfma_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 128, 4, 8>;
    return nullptr;
    }
}

// multi-launch entry points exist for 32-, 64- and 128-channel chunks at their smallest step group
template <typename TIn, typename TOut, bool SPLIT, int FM, int FN, int WM, int WN>
static conv_multi_fn pick_kc_multi(int kc, int pd, int unr) {
    if constexpr (WM * WN < 4) return nullptr;
    else {
    if (kc == 32 && pd == 2 && unr == 2) return conv_mfma_multi_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 32, 2, 2>;
    if (kc == 64 && pd == 4 && unr == 4) return conv_mfma_multi_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 64, 4, 4>;
    if (kc == 128 && pd == 4 && unr == 8) return conv_mfma_multi_kernel<TIn, TOut, SPLIT, FM, FN, WM, WN, 128, 4, 8>;
    return nullptr;
    }
}

#define FYN_CAT2(a, b) a##b
#define FYN_CAT(a, b) FYN_CAT2(a, b)

// lookup among the tiles of one part (a template so that the tiles of other parts are not instantiated)
template <int PART>
static ConvEntry lookup_part(const ConvVariant& v) {
    const bool f16 = v.in_f16 && v.out_f16 && !v.split;
    const bool f32 = !v.in_f16 && !v.out_f16 && v.split;  // split arithmetic is the fp32-storage path
    ConvEntry e;
    if (!f16 && !f32) return e;
#define FYN_TILE(idx_, fm_, fn_, wm_, wn_)                                                                    \
    if constexpr ((idx_) % FYN_CONV_PARTS == PART) {                                                           \
        if (v.fm == fm_ && v.fn == fn_ && v.wm == wm_ && v.wn == wn_) {                                        \
            if (f32) {                                                                                         \
                e.single = pick_kc<float, float, true, fm_, fn_, wm_, wn_>(v.kc, v.pd, v.unr);                 \
                e.multi = pick_kc_multi<float, float, true, fm_, fn_, wm_, wn_>(v.kc, v.pd, v.unr);            \
            } else {                                                                                           \
                e.single = pick_kc<_Float16, _Float16, false, fm_, fn_, wm_, wn_>(v.kc, v.pd, v.unr);          \
                e.multi = pick_kc_multi<_Float16, _Float16, false, fm_, fn_, wm_, wn_>(v.kc, v.pd, v.unr);     \
            }                                                                                                  \
            return e;                                                                                          \
        }                                                                                                      \
    }
    FYN_CONV_TILES(FYN_TILE)
#undef FYN_TILE
    return e;
}

ConvEntry FYN_CAT(conv_mfma_lookup_part, FYN_CONV_PART)(const ConvVariant& v) { return lookup_part<FYN_CONV_PART>(v); }

#if FYN_CONV_PART == 0
#define FYN_DECL(i_) ConvEntry conv_mfma_lookup_part##i_(const ConvVariant& v);
#if FYN_CONV_PARTS > 1
FYN_DECL(1)
#endif
#if FYN_CONV_PARTS > 2
FYN_DECL(2)
#endif
#if FYN_CONV_PARTS > 3
FYN_DECL(3)
#endif
#if FYN_CONV_PARTS > 4
FYN_DECL(4)
FYN_DECL(5)
#endif
#if FYN_CONV_PARTS > 6
FYN_DECL(6)
FYN_DECL(7)
#endif
#undef FYN_DECL

static ConvEntry pick_kernel(const ConvVariant& v) {
    ConvEntry e = conv_mfma_lookup_part0(v);
#if FYN_CONV_PARTS > 1
    if (!e.single) e = conv_mfma_lookup_part1(v);
#endif
#if FYN_CONV_PARTS > 2
    if (!e.single) e = conv_mfma_lookup_part2(v);
#endif
#if FYN_CONV_PARTS > 3
    if (!e.single) e = conv_mfma_lookup_part3(v);
#endif
#if FYN_CONV_PARTS > 4
    if (!e.single) e = conv_mfma_lookup_part4(v);
    if (!e.single) e = conv_mfma_lookup_part5(v);
#endif
#if FYN_CONV_PARTS > 6
    if (!e.single) e = conv_mfma_lookup_part6(v);
    if (!e.single) e = conv_mfma_lookup_part7(v);
#endif
    return e;
}

bool conv_mfma_variant_exists(const ConvVariant& v) { return pick_kernel(v).single != nullptr; }
bool conv_mfma_multi_exists(const ConvVariant& v) { return pick_kernel(v).multi != nullptr; }

// the steps of a chunk divide evenly among the K groups of waves, each taking whole unrolled groups
int conv_mfma_step_multiple(const ConvVariant& v) { return v.unr * (4 / (v.wm * v.wn)); }

int conv_mfma_tile_count() {
    int n = 0;
#define FYN_TILE(idx_, fm_, fn_, wm_, wn_) n++;
    FYN_CONV_TILES(FYN_TILE)
#undef FYN_TILE
    return n;
}

void conv_mfma_tile(int index, int* fm, int* fn, int* wm, int* wn) {
#define FYN_TILE(idx_, fm_, fn_, wm_, wn_) \
    if (index == idx_) { *fm = fm_; *fn = fn_; *wm = wm_; *wn = wn_; }
    FYN_CONV_TILES(FYN_TILE)
#undef FYN_TILE
}

static int blocks_of(const ConvMfmaParams& p) { return p.tiles_x * p.tiles_y * p.cout_blocks * (p.ksplit > 1 ? p.ksplit : 1); }

static int check_params(const ConvVariant& v, const ConvMfmaParams& p) {
    if (p.nsteps < 1 || p.nsteps > 256 || v.unr < 2 || p.nsteps % conv_mfma_step_multiple(v) != 0) return -5;
    if (p.ksplit > 1 && (!p.partial || p.chunks_per_split < 1 || (p.ksplit - 1) * p.chunks_per_split >= p.cin_chunks)) return -7;
    if (p.ksplit <= 1 && p.chunks_per_split < p.cin_chunks) return -7;
    if ((1 << p.tile_w_log2) * v.fm < 8) return -10;   // the epilogue's row mapping needs 8 / FM positions of one tile row
    if (v.kc == 4 && p.nsteps > 64) return -5;         // four table entries per step in the 1 KB table
    // folded kx taps: one cout block of a 32 x (32*FN*4) tile, no split-K, tile wider than the kernel
    if (p.fuse_k && (v.fm != 1 || v.wm != 1 || v.wn != 4 || p.cout_blocks != 1 || p.ksplit > 1 || p.fuse_cout < 1 || p.fuse_cout > 4 ||
                     p.fuse_k * p.fuse_cout > 32 || (1 << p.tile_w_log2) < p.fuse_k || p.out_step != 1 || p.out_cp < 4 ||
                     p.tiles_x * ((1 << p.tile_w_log2) - p.fuse_k + 1) < p.npos_x - (p.fuse_k - 1)))
        return -12;
    // sub-sampled frame: every one of its pixels must be a pixel of the stored frame
    if (p.in_sub && (p.in_sub < 2 || p.in_stride != 1 || p.in_shift != 0 || p.in_y0 != 0 || p.in_x0 != 0 || p.in_oy < 0 || p.in_ox < 0 ||
                     (p.npos_y - 1) * p.in_sub + p.in_oy >= p.in_hp || (p.npos_x - 1) * p.in_sub + p.in_ox >= p.in_wp))
        return -11;
    return 0;
}

// raises a kernel's dynamic LDS limit once per kernel and size (also for the other convolution files: a launch that
// is being captured into a graph then makes no attribute call)
int ensure_lds(const void* fn, size_t lds_bytes) {
    if (lds_bytes <= 48 * 1024) return 0;
    static std::mutex mu;
    static std::map<const void*, size_t> raised;
    std::lock_guard<std::mutex> lk(mu);
    size_t& cur = raised[fn];
    if (cur < lds_bytes) {
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) return -2;
        cur = lds_bytes;
    }
    return 0;
}


int launch_conv_mfma(const ConvVariant& v, const ConvMfmaParams& p_in, size_t lds_bytes, hipStream_t s) {
    conv_kernel_fn fn = pick_kernel(v).single;
    if (!fn) return -1;
    if (int rc = check_params(v, p_in)) return rc;
    if (int rc = ensure_lds(reinterpret_cast<const void*>(fn), lds_bytes)) return rc;
    const int blocks = blocks_of(p_in);
    const dim3 threads(v.fm * v.fn >= 2 ? 512 : 256);
    hipLaunchKernelGGL(fn, dim3(blocks), threads, lds_bytes, s, p_in);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int launch_conv_mfma_multi(const ConvVariant& v, const ConvMfmaMulti& m_in, size_t lds_bytes, hipStream_t s) {
    if (m_in.nsub == 1) return launch_conv_mfma(v, m_in.sub[0], lds_bytes, s);
    conv_multi_fn fn = pick_kernel(v).multi;
    if (!fn) return -1;
    if (m_in.nsub < 1 || m_in.nsub > FYN_CONV_MAX_SUB) return -8;
    int blocks = 0;
    for (int i = 0; i < m_in.nsub; i++) {
        if (int rc = check_params(v, m_in.sub[i])) return rc;
        blocks = blocks_of(m_in.sub[i]) > blocks ? blocks_of(m_in.sub[i]) : blocks;
    }
    if (int rc = ensure_lds(reinterpret_cast<const void*>(fn), lds_bytes)) return rc;
    const dim3 threads(v.fm * v.fn >= 2 ? 512 : 256);
    hipLaunchKernelGGL(fn, dim3(blocks, m_in.nsub), threads, lds_bytes, s, m_in);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
#endif  // FYN_CONV_PART == 0

}  // namespace fynhip
