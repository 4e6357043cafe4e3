// Wide-kernel convolution with at most four output channels (the 9x9 32->3 output layer of a style-transfer net) as
// a row-rolling implicit GEMM on gfx950 matrix cores.
//
// Replaces, for such layers, the render passes of DeepConvLayerNxN::forward (fyusenet/gpu/deep/deepconvlayerNxN.cpp:
// 129-211) and of the shallow ConvLayerNxN::forward (gpu/vanilla/convlayerNxN_vanilla.cpp:72-141).
//
// GEMM view: M = virtual output channels (o, kx), cout*K <= 32 of them: one 32-row fragment; K = (ky, input channel);
// N = the columns x' of one image row of q[y][x'][o*K+kx] = sum_{ky,ci} W[o,ky,kx,ci] * act(in[y+ky-r, x'-r, ci]).
// The output is out[y][x][o] = sum_kx q[y][x+kx][o*K+kx], summed from the accumulators inside the wave.
//
// A workgroup owns a strip of 32*FN columns of q (32*FN - K + 1 output columns) and walks down a block of rows.  The
// input rows of the strip live in an LDS ring of 16 rows (fp16, hi and lo planes with fp32 storage); every input row
// is fetched from memory once per strip, by four staging waves, four rows ahead of the four MFMA waves, each of which
// computes one output row per round (K input rows, K*CS k16-steps).  The weights -- one fragment per step and plane --
// stay in registers for the whole kernel, so the step loop reads nothing but the ring.
//
// fp32 tensors, whose operands are split into fp16 halves: hi*hi runs as fp16 matrix instructions; the two correction
// terms (lo*hi + hi*lo, 2^-11 of the result) run either as two more fp16 passes over the lo planes or -- 32-channel rows
// of an input that carries a value range -- as one v_mfma_f32_32x32x64_f8f6f4 per input row and fragment at twice the
// fp16 rate: the second plane of the ring then holds, per column and eight channels, [8 x fp8(32 lo) | 8 x fp8(hi / 64)]
// and the third weight plane [8 x fp8(hi / 32) | 8 x fp8(64 lo)], so that byte by byte the products are lo*hi and hi*lo
// (p16_common.h; rel-L2 against the fp64 oracle 1e-5 instead of 3e-7).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <type_traits>

#include "kernels.h"
#include "p16_common.h"
#include "range.h"


namespace fynhip {

namespace {
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

constexpr int RING = 16;   // input rows resident per strip: K + 3 in use by a round, 4 being staged (K <= 9)
// Floats per column of a wave's epilogue area [column][virtual channel]: odd, so that the lanes of a wave (one column
// each) fall into distinct banks; cout*K <= 28 virtual channels are kept.
constexpr int ROWS_SCRATCH_PITCH = 29;

// (lds_barrier() orders LDS traffic only: outstanding global loads -- rows fetched two rounds ahead -- and global stores
// -- finished output rows -- stay in flight across it; __syncthreads() would wait for them as well.)
__device__ __forceinline__ float act1r(float x, const Act& a) { return __builtin_amdgcn_fmed3f(x, a.lo, a.hi) + a.leak * fminf(x, 0.f); }

// Eight channels of a staging item as they come from memory; they are converted when the item is written to the ring,
// a round after its load was issued (a conversion at the load would wait for it: one memory round trip per item).
template <typename T>
struct Raw8;
template <>
struct Raw8<float> {
    float4 a, b;
    __device__ __forceinline__ void zero() { a = b = float4{0.f, 0.f, 0.f, 0.f}; }
    __device__ __forceinline__ void load(const float* src) { a = *reinterpret_cast<const float4*>(src); b = *reinterpret_cast<const float4*>(src + 4); }
    __device__ __forceinline__ void get(float* v) const { v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w; }
};
template <>
struct Raw8<_Float16> {
    half8_t h;
    __device__ __forceinline__ void zero() { h = (half8_t)((_Float16)0.f); }
    __device__ __forceinline__ void load(const _Float16* src) { h = *reinterpret_cast<const half8_t*>(src); }
    __device__ __forceinline__ void get(float* v) const {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)h[i];
    }
};

// Staging items in flight in a thread's registers: 8 channels of one column each, and where they go in the ring.
template <typename T, int N>
struct RowBatch {
    Raw8<T> v[N];
    int dst[N];
};

// CS: k16 steps per input row (input channels padded to 16*CS); a column of the ring holds 2*CS chunks of 8 halves.
// The chunk order inside a column is permuted with the column index so that the 16-byte reads of 8 neighbouring lanes
// cover all 32 banks.
template <int CS>
__device__ __forceinline__ int ring_off(int col, int chunk) {
    constexpr int NCH = 2 * CS, CPB = 8 / NCH;   // chunks per column, columns per 128 bytes
    return col * (NCH * 16) + ((chunk ^ ((col / CPB) & (NCH - 1))) * 16);
}

template <typename TIn, typename TOut, bool SPLIT, bool C8, int K, int CS, int FN>
__global__ __launch_bounds__(512) void conv_rows_kernel(const ConvRowsParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    static_assert(!C8 || (SPLIT && CS == 2), "the fp8 form pairs the two k16 steps of a 32-channel row");
    constexpr int NPL = SPLIT ? 2 : 1;
    constexpr int NPLW = SPLIT ? 3 : 1;       // planes of a packed weight fragment
    constexpr int WC = 32 * FN;               // q columns per strip
    constexpr int OW = WC - (K - 1);          // output columns per strip
    constexpr int NCH = 2 * CS;
    constexpr int PLANE = WC * NCH * 16;      // bytes of one plane of one ring row
    constexpr int ROWB = NPL * PLANE;
    constexpr int NSTEPS = K * CS;
    constexpr int ITEMS = WC * NCH;           // staging items (8 channels of one column) per row
    static_assert(K >= 3 && K <= 9 && (K & 1), "kernel sizes 3, 5, 7, 9");
    static_assert(4 * ((K + 2) / 4 + 2) <= RING, "ring too small");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool mfma_wave = wave < 4;
    // Workgroups go to the chip's eight XCDs (one L2 each) in turn: workgroup b runs tile (b % 8) * ceil(tiles / 8) + b / 8,
    // so that an XCD holds neighbouring strips and row blocks, whose input columns and rows overlap.
    const int per_xcd = (p.strips * p.row_blocks + 7) >> 3;
#ifdef FYN_ROWS_PLAIN_MAP
    const int tile = blockIdx.x;
#else
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
#endif
    if (tile >= p.strips * p.row_blocks) return;
    const int strip = tile % p.strips;
    const int rblk = tile / p.strips;
    const int y_begin = rblk * p.rows_per_block;
    const int y_end = min(y_begin + p.rows_per_block, p.out_h);
    const int x0 = strip * OW;                // first q column (= first output column) of the strip
    constexpr int sp = ROWS_SCRATCH_PITCH;    // floats per column of the epilogue area
    unsigned char* ring = lds;
    float* scratch = reinterpret_cast<float*>(lds + RING * ROWB) + (wave & 3) * (WC * sp);

    // value ranges (range.h): clear the words assigned to this launch, read the input tensor's
    __shared__ unsigned range_box[2];   // meeting point of the MFMA waves' output maxima; zero before the first barrier
    if (tid < 2) range_box[tid] = 0u;
    if (blockIdx.x == 0) range_clear(p.reset[0], p.reset[1], p.reset[2], p.reset[3], p.nreset);
    float in_scale = 1.f, inv_in_scale = 1.f;
    if (SPLIT && p.in_amax) in_scale = range_scale(range_after_act(range_reduce(range_load(p.in_amax)), p.act), &inv_in_scale);
    const float acc_mul = p.acc_mul * inv_in_scale;

    // ---- staging: q row j (relative to y_begin) is stored input row in_y0 + y_begin + j ----
    const TIn* in = reinterpret_cast<const TIn*>(p.in);
    const int stid = tid & 255;
    // Four rows at a time: ITEMS items per row dealt to the 256 staging threads.  fetch() issues the loads of a batch
    // into registers, store() converts and writes them into the ring; a batch is fetched one round before it is stored.
    // (The rows of the first round are dealt to all 512 threads: the MFMA waves have nothing else to do until they are in.)
    constexpr int PER = (4 * ITEMS + 255) / 256;   // items per thread and batch
    auto fetch = [&](auto& bt, int j_first, int nrows, int t, int nthreads) {
        constexpr int N = sizeof(bt.dst) / sizeof(int);
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int idx = i * nthreads + t;
            bt.dst[i] = -1;
            bt.v[i].zero();
            if (idx < nrows * ITEMS) {
                const int jr = idx / ITEMS, it = idx - jr * ITEMS;
                const int col = it / NCH, chunk = it - col * NCH;
                const int j = j_first + jr;
                // (coordinates in the frame of repeated pixels, which is the stored frame unless the step is fractional)
                int gy = p.in_y0 + y_begin + j, gx = p.in_x0 + x0 + col;
                const int vhp = p.in_hp << p.in_shift, vwp = p.in_wp << p.in_shift;
                if (p.in_clamp) {
                    gy = min(max(gy, 0), vhp - 1);
                    gx = min(max(gx, 0), vwp - 1);
                }
                bt.dst[i] = (j & (RING - 1)) * ROWB + ring_off<CS>(col, chunk);
                if ((unsigned)gy < (unsigned)vhp && (unsigned)gx < (unsigned)vwp && chunk * 8 < p.in_cp)
                    bt.v[i].load(in + ((size_t)(gy >> p.in_shift) * p.in_wp + (gx >> p.in_shift)) * p.in_cp + chunk * 8);
            }
        }
    };
    // (fp32 tensors: the activation's kind chosen once per call and the hi/lo split in four instructions per pair of values,
    // split8; fp16 tensors: an activation that is exact on halves acts on the packed halves)
    const int act_kind_ = p.act.kind;
    auto store = [&](const auto& bt) {
        constexpr int N = sizeof(bt.dst) / sizeof(int);
        if constexpr (SPLIT) {
            auto split_all = [&](auto kind_) {
                constexpr int KIND = decltype(kind_)::value;
#pragma unroll
                for (int i = 0; i < N; i++) {
                    if (bt.dst[i] < 0) continue;
                    float r[8];
                    bt.v[i].get(r);
                    half8_t hi, lo;
                    split8<KIND>(r, true, p.act, in_scale, hi, lo);
                    *reinterpret_cast<half8_t*>(ring + bt.dst[i]) = hi;
                    *reinterpret_cast<half8_t*>(ring + bt.dst[i] + PLANE) = C8 ? c8_plane(hi, lo) : lo;
                }
            };
            if (act_kind_ == ACT_RELU) split_all(std::integral_constant<int, ACT_RELU>());
            else if (act_kind_ == ACT_NONE) split_all(std::integral_constant<int, ACT_NONE>());
            else split_all(std::integral_constant<int, ACT_LEAKY>());
        } else {
            _Float16 hlo, hhi;
            const bool half_act = act_half_exact(p.act, hlo, hhi);
#pragma unroll
            for (int i = 0; i < N; i++) {
                if (bt.dst[i] < 0) continue;
                half8_t v;
                if (half_act) {
                    v = act_half(bt.v[i].h, hlo, hhi);
                } else {
                    float r[8];
                    bt.v[i].get(r);
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] = (_Float16)act1r(r[e], p.act);
                }
                *reinterpret_cast<half8_t*>(ring + bt.dst[i]) = v;
            }
        }
    };

    const int rows_total = y_end - y_begin + (K - 1);   // q rows this block needs
    // batch b holds q rows [4b, 4b + 4); round g reads batches g .. g + (K + 2) / 4, batch g + 3 is written during round g
    constexpr int NB0 = (K + 2) / 4 + 1;      // batches in the ring before the first round
    const int nbatches = (rows_total + 3) >> 2;
    auto rows_of = [&](int b) { return min(4, rows_total - 4 * b); };
    RowBatch<TIn, PER> nxt;   // the batch in flight (staging waves)
    {
        // the first round's rows, all threads: every load is issued before the first conversion
        constexpr int PER0 = (NB0 * 4 * ITEMS + 511) / 512;
        RowBatch<TIn, PER0> first;
        fetch(first, 0, min(4 * NB0, rows_total), tid, 512);
        store(first);
    }
    // (the batch of the second round is requested once the first round's rows are in: every workgroup of the
    // launch is in this phase at the same time, and it is bound by memory bandwidth)
    if (!mfma_wave) fetch(nxt, 4 * NB0, NB0 < nbatches ? rows_of(NB0) : 0, stid, 256);
    // ---- weights: one fragment per step and plane, in registers from here on (placed behind the staging code so that
    //      the two never hold registers at the same point) ----
    // (fp8 form: the fp16 hi fragment of every step, and per input row the fp8 operands of channels 16g .. 16g + 15 for
    // the lanes of half g = lane / 32: the halves 0 and 1 of the third plane of step sub = g)
    constexpr int NPLA = C8 ? 1 : NPL;
    half8_t a_reg[NSTEPS][NPLA];
    i32x8_t a8[C8 ? K : 1];
    if (mfma_wave) {
        const half8_t* w = reinterpret_cast<const half8_t*>(p.wpack);
#pragma unroll
        for (int t = 0; t < NSTEPS; t++)
#pragma unroll
            for (int pl = 0; pl < NPLA; pl++) a_reg[t][pl] = w[(t * NPLW + pl) * 64 + lane];
        if constexpr (C8) {
            const i32x4_t* w8 = reinterpret_cast<const i32x4_t*>(p.wpack);
#pragma unroll
            for (int ky = 0; ky < K; ky++) {
                const int frag = ((ky * CS + (lane >> 5)) * NPLW + 2) * 64;
                const i32x4_t u = w8[frag + (lane & 31)], v = w8[frag + 32 + (lane & 31)];
                a8[ky] = i32x8_t{u[0], u[1], u[2], u[3], v[0], v[1], v[2], v[3]};
            }
        }
    }
    lds_barrier();

    // per-lane byte offsets of the B fragments inside a ring row: column fn*32 + lane%32, chunk 2*sub + lane/32
    int boff[CS][FN];
#pragma unroll
    for (int sub = 0; sub < CS; sub++)
#pragma unroll
        for (int fn = 0; fn < FN; fn++) boff[sub][fn] = ring_off<CS>(fn * 32 + (lane & 31), 2 * sub + (lane >> 5));
    // fp8 form: the chunks 2g and 2g + 1 of the lane's column in the second plane
    int coff[2][FN];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int fn = 0; fn < FN; fn++) coff[h][fn] = PLANE + ring_off<CS>(fn * 32 + (lane & 31), (2 * (lane >> 5) + h) % NCH);

    float sc4[4], bi4[4];
#pragma unroll
    for (int o = 0; o < 4; o++) {
        sc4[o] = o < p.cout ? p.scale[o] : 0.f;
        bi4[o] = o < p.cout ? p.bias[o] : 0.f;
    }
    TOut* out = reinterpret_cast<TOut*>(p.out);
    const TOut* res = reinterpret_cast<const TOut*>(p.res);

    const int nrounds = (y_end - y_begin + 3) >> 2;
    // One loop per role (the same barriers in both), so that a wave's registers hold either the staged items or the
    // weights, fragments and accumulators.
    if (!mfma_wave) {
        for (int g = 0; g < nrounds; g++) {
            // write batch NB0 + g (fetched a round ago; no round up to g reads its ring slots), fetch the next one
            store(nxt);
            const int b = NB0 + g + 1;
            fetch(nxt, 4 * b, b < nbatches ? rows_of(b) : 0, stid, 256);
            lds_barrier();
        }
        return;
    }
    float vmax = 0.f;   // largest magnitude this lane wrote
    for (int g = 0; g < nrounds; g++) {
        {
            const int yl = 4 * g + wave;          // output row relative to y_begin
            const int y = y_begin + yl;
            if (y < y_end) {
                float16_t acc[FN];
#pragma unroll
                for (int fn = 0; fn < FN; fn++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[fn][r] = 0.f;
                if constexpr (C8) {
                    // Per input row: FN fp16 MFMAs on each of its two k16 steps, then FN fp8 MFMAs on the whole row.  Every
                    // operand buffer is refilled for the next row right behind the MFMA that read it (a memory
                    // instruction issued behind an MFMA runs in its shadow), a row's worth of MFMAs ahead of its use.
                    half8_t bh[CS][FN];
                    i32x8_t bc[FN];
                    auto row_of = [&](int ky) { return ring + ((yl + ky) & (RING - 1)) * ROWB; };
                    auto load_h = [&](int ky, int sub, int fn) { bh[sub][fn] = *reinterpret_cast<const half8_t*>(row_of(ky) + boff[sub][fn]); };
                    auto load_c = [&](int ky, int fn) {
                        const i32x4_t u = *reinterpret_cast<const i32x4_t*>(row_of(ky) + coff[0][fn]);
                        const i32x4_t v = *reinterpret_cast<const i32x4_t*>(row_of(ky) + coff[1][fn]);
                        bc[fn] = i32x8_t{u[0], u[1], u[2], u[3], v[0], v[1], v[2], v[3]};
                    };
#pragma unroll
                    for (int fn = 0; fn < FN; fn++) {
#pragma unroll
                        for (int sub = 0; sub < CS; sub++) load_h(0, sub, fn);
                        load_c(0, fn);
                    }
#pragma unroll
                    for (int ky = 0; ky < K; ky++) {
#pragma unroll
                        for (int sub = 0; sub < CS; sub++)
#pragma unroll
                            for (int fn = 0; fn < FN; fn++) {
                                acc[fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_reg[ky * CS + sub][0], bh[sub][fn], acc[fn], 0, 0, 0);
                                if (ky + 1 < K) load_h(ky + 1, sub, fn);
                                __builtin_amdgcn_sched_barrier(0);
                            }
#pragma unroll
                        for (int fn = 0; fn < FN; fn++) {
                            acc[fn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8[ky], bc[fn], acc[fn], 0, 0, 0, 0, 0, 0);
                            if (ky + 1 < K) load_c(ky + 1, fn);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                } else {
                half8_t b[2][FN][NPL];
                auto load_b = [&](int t, half8_t (&dst)[FN][NPL]) {
                    const int ky = t / CS, sub = t % CS;
                    const unsigned char* row = ring + ((yl + ky) & (RING - 1)) * ROWB;
#pragma unroll
                    for (int pl = 0; pl < NPL; pl++)
#pragma unroll
                        for (int fn = 0; fn < FN; fn++) dst[fn][pl] = *reinterpret_cast<const half8_t*>(row + pl * PLANE + boff[sub][fn]);
                };
                load_b(0, b[0]);
                // one slot per MFMA: the MFMA, then a share of the next step's LDS reads, in this order (a memory
                // instruction issued right behind an MFMA runs in its shadow; one wave cannot queue MFMAs)
                constexpr int NMF = FN * (SPLIT ? 3 : 1), NDS = FN * NPL;
#pragma unroll
                for (int t = 0; t < NSTEPS; t++) {
                    const int kyn = (t + 1) / CS, subn = (t + 1) % CS;
                    const unsigned char* rown = ring + ((yl + kyn) & (RING - 1)) * ROWB;
#pragma unroll
                    for (int i = 0; i < NMF; i++) {
                        const int kind = i / FN, fn = i % FN;
                        const int apl = (kind == 1) ? 1 : 0, bpl = (kind == 2) ? 1 : 0;
                        acc[fn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_reg[t][C8 ? 0 : apl], b[t & 1][fn][bpl], acc[fn], 0, 0, 0);
                        if (t + 1 < NSTEPS) {
#pragma unroll
                            for (int j = i * NDS / NMF; j < (i + 1) * NDS / NMF; j++)
                                b[(t + 1) & 1][j % FN][j / FN] = *reinterpret_cast<const half8_t*>(rown + (j / FN) * PLANE + boff[subn][j % FN]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                }
                // accumulators -> this wave's area [column][virtual channel]: a lane holds column lane%32 of each
                // fragment and rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
                for (int fn = 0; fn < FN; fn++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int rowb = q * 8 + (lane >> 5) * 4;
                        if (rowb < 28) {
                            float* dstp = scratch + (fn * 32 + (lane & 31)) * sp + rowb;
#pragma unroll
                            for (int e = 0; e < 4; e++) dstp[e] = acc[fn][q * 4 + e];
                        }
                    }
                // out[y][x][o] = sum_kx q[x + kx][o*K + kx]: one output column per lane
                for (int x = lane; x < OW; x += 64) {
                    const int gx = x0 + x;
                    if (gx >= p.out_w) break;
                    // all K*4 reads are issued before the first sum (a read under a condition would cost one LDS round
                    // trip each); channels beyond cout read some row of the column and are discarded below
                    float qv[K][4];
#pragma unroll
                    for (int kx = 0; kx < K; kx++) {
                        const float* qp = scratch + (x + kx) * sp;
#pragma unroll
                        for (int o = 0; o < 4; o++) qv[kx][o] = qp[(o * K + kx < 28) ? o * K + kx : 27];
                    }
                    float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kx = 0; kx < K; kx++)
#pragma unroll
                        for (int o = 0; o < 4; o++) a[o] += qv[kx][o];
                    float rv[4] = {0.f, 0.f, 0.f, 0.f};
                    if (res) {
                        const TOut* rp = res + ((size_t)(p.res_off_y + y) * p.res_wp + p.res_off_x + gx) * p.res_cp;
                        if (sizeof(TOut) == 4) {
                            const float4 r4 = *reinterpret_cast<const float4*>(rp);
                            rv[0] = r4.x; rv[1] = r4.y; rv[2] = r4.z; rv[3] = r4.w;
                        } else {
                            const half4_t r4 = *reinterpret_cast<const half4_t*>(rp);
#pragma unroll
                            for (int o = 0; o < 4; o++) rv[o] = (float)r4[o];
                        }
                    }
                    f32x4_t v;
#pragma unroll
                    for (int o = 0; o < 4; o++) {
                        float r = rv[o];
                        if (p.res_relu) r = fmaxf(r, 0.f);
                        if (p.res_scale) r *= sc4[o];
                        v[o] = o < p.cout ? ((a[o] * acc_mul) * sc4[o] + bi4[o]) + r : 0.f;
                        vmax = fmaxf(vmax, fabsf(v[o]));
                    }
                    const size_t oidx = ((size_t)(p.out_off_y + y) * p.out_wp + p.out_off_x + gx) * p.out_cp;
                    if (sizeof(TOut) == 4) {
                        *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + oidx) = v;
                    } else {
                        half4_t hv;
#pragma unroll
                        for (int o = 0; o < 4; o++) hv[o] = (_Float16)v[o];
                        *reinterpret_cast<half4_t*>(reinterpret_cast<_Float16*>(out) + oidx) = hv;
                    }
                }
            }
        }
        lds_barrier();   // the round's rows are consumed, the next round's rows are in the ring
    }
    if (SPLIT && p.out_amax) range_publish_waves(p.out_amax, vmax, range_box, 4);
}

typedef void (*rows_fn)(const ConvRowsParams);

template <typename TIn, typename TOut, bool SPLIT, int FN>
rows_fn pick_rows(int k, int cs, bool c8) {
#define FYN_ROWS(K_, CS_) \
    if (k == K_ && cs == CS_ && !c8) return conv_rows_kernel<TIn, TOut, SPLIT, false, K_, CS_, FN>;
    FYN_ROWS(3, 1) FYN_ROWS(3, 2) FYN_ROWS(5, 1) FYN_ROWS(5, 2) FYN_ROWS(7, 1) FYN_ROWS(7, 2) FYN_ROWS(9, 1) FYN_ROWS(9, 2)
#undef FYN_ROWS
    if constexpr (SPLIT) {
#define FYN_ROWS8(K_) \
    if (k == K_ && cs == 2 && c8) return conv_rows_kernel<TIn, TOut, true, true, K_, 2, FN>;
        FYN_ROWS8(3) FYN_ROWS8(5) FYN_ROWS8(7) FYN_ROWS8(9)
#undef FYN_ROWS8
    }
    return nullptr;
}
}  // namespace

// fp32 tensors, 32-channel rows, an input with a value range (the fp8 operands need its scale), unless the layer asks
// for the three fp16 passes.
bool conv_rows_uses_fp8(const ConvRowsParams& p, bool f16) { return !f16 && p.cs == 2 && p.in_amax != nullptr && !p.exact_split; }

bool conv_rows_supported(int k, int cin_pitch, int cout, bool f16) {
    (void)f16;
    return (k == 3 || k == 5 || k == 7 || k == 9) && cout >= 1 && cout <= 4 && cout * k <= 28 && cin_pitch >= 8 && cin_pitch <= 32 &&
           cin_pitch % 8 == 0;
}

size_t conv_rows_lds_bytes(const ConvRowsParams& p, bool f16) {
    const int wc = 32 * p.fn, nch = 2 * p.cs;
    return (size_t)RING * (f16 ? 1 : 2) * wc * nch * 16 + (size_t)4 * wc * ROWS_SCRATCH_PITCH * sizeof(float);
}

int launch_conv_rows(const ConvRowsParams& p, bool f16, hipStream_t s) {
    if (p.fn != 2) return -1;
    rows_fn fn = f16 ? pick_rows<_Float16, _Float16, false, 2>(p.k, p.cs, false) : pick_rows<float, float, true, 2>(p.k, p.cs, conv_rows_uses_fp8(p, f16));
    if (!fn) return -1;
    // what the kernel's indexing assumes
    if (p.cout * p.k > 28 || p.out_cp != 4 || p.strips < 1 || p.row_blocks < 1 || p.in_shift < 0 || p.in_shift > 8 ||
        p.rows_per_block < 1 || p.rows_per_block % 4 || p.in_cp > 16 * p.cs || p.in_cp % 8 || p.cout * p.k > 32 ||
        (long long)p.strips * (32 * p.fn - (p.k - 1)) < p.out_w || (long long)p.row_blocks * p.rows_per_block < p.out_h)
        return -5;
    const size_t lds_bytes = conv_rows_lds_bytes(p, f16);
    if (lds_bytes > 160 * 1024) return -2;
    if (ensure_lds(reinterpret_cast<const void*>(fn), lds_bytes) != 0) return -2;
    hipLaunchKernelGGL(fn, dim3((p.strips * p.row_blocks + 7) / 8 * 8), dim3(512), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace fynhip
