// Kernel parameter blocks and host-side launchers of the gfx950 layer kernels.
//
// Tensor layout in HBM (all kernels): channel-packed NHWC with a physical zero halo,
//   element (y, x, c) of a tensor with net size HxW, halo `pad`, channel pitch `cp` lives at
//   ((y + pad) * (W + 2*pad) + (x + pad)) * cp + c
// cp = 4 for <= 4 channels, otherwise channels rounded up to a multiple of 8; pad lanes hold 0.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fynhip {

enum ActKind : int { ACT_NONE = 0, ACT_RELU = 1, ACT_LEAKY = 2, ACT_CLIP = 3 };

struct Act {
    int kind;
    float leak, lo, hi;
};

// Output stores that are written through the XCD's L2 as they are issued (sc1: visible at device scope) instead of
// staying dirty there until the write-back at the kernel's end.  A kernel's stores then overlap the work of the
// workgroups that are still computing, and the next launch does not wait behind the write-back of a whole output
// tensor (measured: 1.2 to 3.5 us per launch on outputs of 10 to 40 MB).  The line stays cached as with a plain store
// (no streaming hint: the consumer reads it next).
//
// What such a store does not take part in is the bookkeeping that keeps the eight L2s of the chip consistent for plain
// stores.  Observed: kernels that wrote through pieces of 64 bytes, where two workgroups on two XCDs share a 128-byte
// line, left later launches reading an old half of such lines now and then (whole networks off by O(1), differently
// from pass to pass); a buffer_inv sc1 in every wave of every kernel made the results stable again (and the frames
// 1.7x slower).  A kernel therefore writes through only where (1) every 128-byte line of the output is stored whole by
// one workgroup (a pixel is whole lines, and so is a workgroup's block of its channels), (2) the launch has at least
// eight workgroups, and (3) its workgroups 0..7 -- consecutive workgroups are dealt to consecutive XCDs, so these sit
// on all eight -- drop the clean lines of their L2 once during the launch (the acquire half of device-scope
// visibility: copies of the buffer's earlier contents that other XCDs may hold; nothing in the kernel reads the
// output buffer, so none appears after that).  With (1) and (2) alone no stale read was seen either; (3) costs 1 % of
// the style net's frame and stays.  Everything else stores plainly.  Outputs beyond kStoreThroughMaxBytes do so as
// well: there the L2's write-back of whole lines serves HBM better than 64-byte pieces (measured on 90 and 180 MB
// outputs: 10 to 19 % slower written through).
//
// (The compiler does not look inside the asm statement: a vector instruction that writes a register of a store of more
// than eight bytes must be two wait states ahead of it on this part, which the s_nop provides whatever came before.)
template <class V>
__device__ __forceinline__ void store_through(V* dst, const V v) {
    static_assert(sizeof(V) == 16, "store_through: 16-byte values");
    typedef int wt_i4 __attribute__((ext_vector_type(4)));
    asm volatile("s_nop 1\n\tglobal_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(__builtin_bit_cast(wt_i4, v)) : "memory");
}
template <class V>
__device__ __forceinline__ void store_out(bool through, V* dst, const V v) {
    if (through) store_through(dst, v);
    else *dst = v;
}
constexpr size_t kStoreThroughMaxBytes = size_t(64) << 20;
// the order in which the hardware deals workgroups to the XCDs
__device__ __forceinline__ unsigned hw_block_id() { return blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z); }
// `out`: the tensor's allocation; pixel_bytes: channel pitch in bytes; one_block_per_pixel: a pixel's channels all come
// from one workgroup, or from workgroups that each store whole lines of it; nblocks: workgroups of the launch
__host__ __device__ inline bool store_through_pays(const void* out, int rows, int cols, int pixel_bytes, bool one_block_per_pixel, size_t nblocks) {
    return one_block_per_pixel && (pixel_bytes & 127) == 0 && (reinterpret_cast<size_t>(out) & 127) == 0 &&
           (size_t)rows * cols * pixel_bytes <= kStoreThroughMaxBytes && nblocks >= 8;
}
__device__ __forceinline__ size_t hw_block_count() { return (size_t)gridDim.x * gridDim.y * gridDim.z; }
__device__ __forceinline__ void drop_clean_l2_lines() { asm volatile("buffer_inv sc1" ::: "memory"); }

// View of a device tensor as kernels see it.
struct TView {
    void* ptr;
    int h, w;   // net size
    int pad;    // halo width
    int cp;     // channel pitch (elements)
    int c;      // real channels
    int f16;    // element type: 1 = __half, 0 = float
    __host__ __device__ int wp() const { return w + 2 * pad; }
    __host__ __device__ int hp() const { return h + 2 * pad; }
    size_t elems() const { return (size_t)hp() * wp() * cp; }
    size_t bytes() const { return elems() * (f16 ? 2 : 4); }
};

inline int channel_pitch(int c) { return c <= 4 ? 4 : (c + 7) / 8 * 8; }

// ---------------------------------------------------------------------------------------------
// MFMA implicit-GEMM convolution (conv_mfma.hip)
// ---------------------------------------------------------------------------------------------
struct ConvMfmaParams {
    const void* in;
    void* out;
    const void* res;     // residual tensor or nullptr
    const void* wpack;   // packed A fragments
    const float* scale;  // [cout padded to block tile]
    const float* bias;   // [cout padded to block tile]
    const int* aoff;     // [nsteps] LDS byte offsets of the k16 steps of one channel chunk
    // input tensor (stored frame)
    int in_hp, in_wp, in_cp;
    int in_y0, in_x0;    // stored coordinate sampled by tile-local (0,0) for output position (0,0)
    int in_stride;       // input step per output position
    // Sampling rule of shallow layers.  in_clamp: coordinates outside the frame repeat its edge instead of reading 0.
    // in_shift = s > 0 (fractional-step convolution): in_y0/in_x0 and the taps count in a virtual frame in which
    // every stored pixel is repeated 2^s times in both directions; virtual coordinate v reads stored pixel v >> s.
    int in_clamp, in_shift;
    // in_sub = s > 1 (one-tap layers with stride s): the frame the kernel works in is the sub-sampled grid of the
    // npos_y x npos_x pixels that the layer reads, frame pixel (y, x) being stored pixel (in_oy + y*s, in_ox + x*s);
    // in_stride is 1 then, so a tile stages only the pixels it uses.  0: the stored frame itself.
    int in_sub, in_oy, in_ox;
    // output positions computed by this launch
    int npos_y, npos_x;
    // output tensor addressing: stored y = out_off_y + pos_y * out_step
    int out_wp, out_cp, out_step, out_off_y, out_off_x;
    // residual tensor addressing (same net coordinates as the output)
    int res_wp, res_cp, res_off_y, res_off_x;
    int res_relu, res_scale;
    // tiling
    int tile_w_log2;     // positions per tile row = 1 << tile_w_log2
    int tile_h;          // rows of positions per tile
    int tiles_x, tiles_y;
    int halo_w, halo_h;  // staged input tile size (pixels)
    int pitch;           // LDS bytes per staged pixel (one plane)
    int row_pitch;       // LDS bytes per staged pixel row (>= halo_w * pitch; padded against bank conflicts)
    int plane;           // LDS bytes of one plane (hi); lo plane follows when split
    int cin_chunks, nsteps;
    int mfrags;          // cout fragments (32 each) in wpack
    int cout_blocks;     // grid size along cout
    float acc_mul;       // exact power of two undoing the weight pre-scaling
    // split-K: the grid holds ksplit copies of the (tile, cout block) set; copy ks reduces the channel chunks
    // [ks*chunks_per_split, (ks+1)*chunks_per_split) and writes raw fp32 partial sums, [ks][position][cout_pad],
    // which splitk_reduce sums and finishes (scale, bias, residual).  ksplit == 1: no partials.
    int ksplit, chunks_per_split;
    float* partial;
    int cout_pad;
    // fuse_k = K > 0: a K x K convolution with fuse_cout <= 4 output channels whose kx taps are folded into the GEMM's
    // M dimension (virtual channel o*K + kx, K vertical taps).  Positions are columns of the intermediate
    // q[y][x'][o*K + kx], x' in [0, W + K - 1); the epilogue sums out[y][x][o] = sum_kx q[y][x + kx][o*K + kx] inside
    // the tile, so tiles overlap by K - 1 columns (tile column step tile_w - K + 1) and q never leaves LDS.  scale
    // and bias are indexed by o then; out/res describe the real output.  Tiles with FM = WM = 1, WN = 4 only.
    int fuse_k, fuse_cout;
    // Value ranges (range.h; fp32 storage only, any of them may be null): the word of the input tensor, read at kernel
    // start; the word of the output tensor, raised by the epilogue; up to four words that workgroup 0 clears (tensors
    // that are dead while this kernel runs).
    const unsigned* in_amax;
    unsigned* out_amax;
    unsigned* reset[4];
    int nreset;
    Act act;
};

// Compile-time variant of the conv kernel.
struct ConvVariant {
    int in_f16, out_f16; // storage types
    int split;           // 1: hi/lo fp16 split of both operands (fp32-accurate), 3 MFMAs per pair
    int fm, fn;          // fragments (32 cout / 32 positions) per wave
    int wm, wn;          // waves per block along cout / positions (wm*wn == 4)
    int kc;              // input channels staged per chunk (4 = small-Cin layout with per-tap offsets, 16, 32, 64, 128)
    int pd;              // depth of the weight-fragment prefetch ring in k16 steps (2, 4, 6)
    int unr;             // k16 steps per unrolled group (a multiple of pd; nsteps is a multiple of it)
};

// Up to four (sub-)convolutions that share one kernel variant run as ONE launch (the four output parities
// of a transposed convolution): grid row blockIdx.y works on sub[blockIdx.y].
#define FYN_CONV_MAX_SUB 4
struct ConvMfmaMulti {
    ConvMfmaParams sub[FYN_CONV_MAX_SUB];
    int nsub;
};

// Returns 0 when the variant exists and was launched.
int launch_conv_mfma(const ConvVariant& v, const ConvMfmaParams& p, size_t lds_bytes, hipStream_t s);
int launch_conv_mfma_multi(const ConvVariant& v, const ConvMfmaMulti& m, size_t lds_bytes, hipStream_t s);
bool conv_mfma_variant_exists(const ConvVariant& v);
bool conv_mfma_multi_exists(const ConvVariant& v);   // a multi-launch entry point is compiled for the variant
// The kernel runs its k16 steps in groups of this size: nsteps must be a multiple (pad with zero-weight steps).
int conv_mfma_step_multiple(const ConvVariant& v);
// The compiled tile configurations (fragments per wave fm x fn, waves per block wm x wn).
int conv_mfma_tile_count();
void conv_mfma_tile(int index, int* fm, int* fn, int* wm, int* wn);

// ---------------------------------------------------------------------------------------------
// Row-rolling MFMA convolution for wide kernels with at most four output channels (conv_rows.hip)
// ---------------------------------------------------------------------------------------------
struct ConvRowsParams {
    const void* in;
    void* out;
    const void* res;      // residual tensor or nullptr
    const void* wpack;    // [k*cs steps][plane][lane 0..63][8 halves]: virtual channel o*k+kx = lane%32, input channel 16*sub + 8*(lane/32) + j;
                          // one plane with fp16 tensors, three with fp32 tensors (fp16 hi, fp16 lo, fp8 operands of the correction terms)
    const float* scale;   // [cout]
    const float* bias;    // [cout]
    int k, cs, fn;        // kernel size; k16 steps per input row (input channel pitch <= 16*cs); 32-column fragments per strip
    int in_hp, in_wp, in_cp;   // stored input frame
    int in_y0, in_x0;     // stored row of (output row 0, tap ky 0) and stored column of q column 0 (input padding - radius)
    int in_clamp;         // coordinates outside the stored frame repeat its edge instead of reading 0
    int in_shift;         // fractional-step convolution: in_y0 / in_x0 and the taps count in the frame whose pixels are repeated 2^in_shift times
    int out_h, out_w;
    int out_wp, out_cp, out_off_y, out_off_x;
    int res_wp, res_cp, res_off_y, res_off_x, res_relu, res_scale;
    int strips, row_blocks, rows_per_block;   // grid = strips * row_blocks workgroups; rows_per_block is a multiple of 4
    int cout;
    float acc_mul;
    int exact_split;      // fp32 tensors: three fp16 passes even where the fp8 form of the correction terms would run
    const unsigned* in_amax;   // value-range words as in ConvMfmaParams
    unsigned* out_amax;
    unsigned* reset[4];
    int nreset;
    Act act;
};
int ensure_lds(const void* fn, size_t lds_bytes);   // 0, or -2 when the device refuses the size (conv_mfma.hip)
bool conv_rows_supported(int k, int cin_pitch, int cout, bool f16);
size_t conv_rows_lds_bytes(const ConvRowsParams& p, bool f16);
int launch_conv_rows(const ConvRowsParams& p, bool f16, hipStream_t s);
bool conv_rows_uses_fp8(const ConvRowsParams& p, bool f16);   // the form launch_conv_rows runs

// 3x3 convolution (stride 1 or 2) with fp32 storage on 16-position fragments (conv_p16.hip).  A workgroup's four MFMA
// waves are wm groups of 32 output channels x 4/wm tiles of tile_h x tile_w positions side by side (compiled
// combinations only, see conv_p16_tile).
struct ConvP16Params {
    const void* in;
    void* out;
    const void* res;      // residual tensor or nullptr
    const void* wpack;    // [(chunk*9 + ky*3 + kx)][cout fragment of 16][plane hi, lo (launch_conv_p16, launch_tconv_p16 on fp32 tensors: a third, see launch_pack_fp8_plane)][lane 0..63][8 halves]: output channel
                          // 16*fragment + lane%16, input channel 32*chunk + 8*(lane/16) + j; 6 steps of zeros behind the last
    const float* scale;   // [cout_blocks*32*wm]
    const float* bias;    // [cout_blocks*32*wm]
    int in_hp, in_wp, in_cp;   // stored input frame; in_cp = 32*cin_chunks
    int stride;           // input step per output position
    int in_y0, in_x0;     // stored coordinate of tap (0,0) of output position (0,0) (input padding - 1)
    int in_clamp;         // coordinates outside the stored frame repeat its edge instead of reading 0
    int in_shift;         // launch_conv_p16, fractional-step convolution: in_y0 / in_x0, the taps and the stride count in the frame whose pixels are repeated 2^in_shift times
    int npos_y, npos_x;
    int out_wp, out_cp, out_off_y, out_off_x;
    int res_wp, res_cp, res_off_y, res_off_x, res_relu, res_scale;
    int tile_h, tile_w, wm;    // tiles_x counts workgroup tiles of (4/wm)*tile_w columns
    int tiles_x, tiles_y;
    float rcp_tiles_x;    // 1.0f / tiles_x
    int pos_groups;       // workgroups per block of output channels; workgroup g walks tiles g, g + pos_groups, ...
    int cin_chunks;
    int exact_split;      // launch_conv_p16 on fp32 tensors: three fp16 passes even where the fp8 form of the correction terms would run
    int plain_stores;     // launch_conv_p16, launch_tconv_p16, launch_conv_p16c4: never write the output through (store_through_pays)
    int mfrags;           // cout fragments (16 each) in wpack
    int cout_blocks;      // workgroups along cout (32*wm channels each)
    int f16;              // tensors hold fp16 (wpack then has one plane, and there are no value-range words)
    float acc_mul;
    const unsigned* in_amax;   // value-range words as in ConvMfmaParams
    unsigned* out_amax;
    unsigned* reset[4];
    int nreset;
    Act act;
    // A depthwise 3x3 layer computed inside the staging of a 1x1 launch of the K-resident form (dw_in null: none): the
    // layer's input tensor, its weights [9][dw_cp] and folded scale / bias [dw_cp], the stored coordinate of tap (0,0)
    // of output position (0,0), its step and the activation applied to its input.  `in` is not read then.
    // (launch_conv_e16dw uses the same fields for a depthwise layer BEHIND a 1x1 layer, with its own meaning of dw_hp / dw_wp.)
    const void* dw_in;
    const float* dw_w;
    const float* dw_scale;
    const float* dw_bias;
    int dw_hp, dw_wp, dw_cp, dw_y0, dw_x0, dw_stride;
    Act dw_act;
    // A batch-norm layer in front of the convolution applied while staging (launch_conv_kr16, and launch_conv_d16 on 1x1
    // layers, without a depthwise layer; null: none): x * in_mul[channel] + in_add[channel] before the activation, `in` being the batch-norm layer's input;
    // arrays of at least in_cp floats.  fp16 tensors: rounded to fp16 as the layer would have stored it.
    const float* in_mul;
    const float* in_add;
    // A reduction over two tensors (launch_conv_kr16, 1x1, one round, no depthwise or batch-norm layer in front; in2
    // null: none): chunks from in2_chunk0 on read in2 -- its own pitch, step and origin, the same activation -- at the
    // position's pixel (y, x) * in2_stride + (in2_y0, in2_x0).  A 1x1 layer and the 1x1 projection whose result it
    // adds run as one launch this way.  in2_amax: that tensor's value-range word (both or none are used).
    const void* in2;
    int in2_hp, in2_wp, in2_cp, in2_y0, in2_x0, in2_stride, in2_chunk0;
    const unsigned* in2_amax;
};
// Whether launch_conv_p16 / launch_conv_p16c4 (upsample 1) or launch_tconv_p16 (upsample 2) write their output through
// (the rule the kernels apply, for kernel descriptions).
inline bool conv_p16_stores_through(const ConvP16Params& p, int upsample) {
    const int esz = p.f16 ? 2 : 4;
    return !p.plain_stores && store_through_pays(p.out, upsample * p.npos_y, upsample * p.npos_x, p.out_cp * esz, p.cout_blocks == 1 || (32 * p.wm * esz) % 128 == 0,
                                                 (size_t)p.pos_groups * p.cout_blocks);
}
// Output channel held by row `row` (0..15) of packed weight fragment `mf` when a wave holds groups of `fm` fragments: the
// rows a lane ends up with (four consecutive ones of every fragment) are 4*fm consecutive channels.
inline int p16_row_channel(int mf, int row, int fm) { return (mf / fm) * 16 * fm + 4 * fm * (row / 4) + 4 * (mf % fm) + (row % 4); }
bool conv_p16_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16);
int conv_p16_tile_count();
void conv_p16_tile(int index, int* th, int* tw, int* stride, int* wm);
size_t conv_p16_lds_bytes(const ConvP16Params& p);   // 0: no such compiled combination
// fp32 tensors: wpack of launch_conv_p16 / launch_tconv_p16 has three planes per fragment (fp16 hi, fp16 lo, and
// [8 x fp8(hi / 32) | 8 x fp8(64 lo)] per lane); this fills the third from src = [fragment][lane][those sixteen floats]
int launch_pack_fp8_plane(const float* src, void* wpack, size_t frags, hipStream_t s);
int launch_conv_p16(const ConvP16Params& p, hipStream_t s);
bool conv_p16_uses_fp8(const ConvP16Params& p);   // whether launch_conv_p16 runs the form with the correction terms as fp8 MFMAs
bool conv_p16c4_uses_fp8(const ConvP16Params& p, int k);   // the same for launch_conv_p16c4
// the transposed 3x3 convolution that doubles the image size, on the same parameters: positions (npos_y x npos_x,
// tiles) are input pixels, out_off_* the stored coordinate of output pixel (0, 0), wpack holds the nine taps of a chunk
// in the order of their input shift (conv_p16.hip: TT_KY / TT_KX)
bool tconv_p16_supported(int k, int crop, int in_cp, int in_pad, int cout, int out_cp, bool f16);
int tconv_p16_tile_count();
void tconv_p16_tile(int index, int* th, int* tw, int* wm);
void tconv_p16_tap(int t, int* ky, int* kx);   // kernel tap of step t of a chunk
size_t tconv_p16_lds_bytes(const ConvP16Params& p);
int launch_tconv_p16(const ConvP16Params& p, hipStream_t s);
// the 9x9 convolution on an input of at most four channels, on the same parameters (one chunk, one channel group)
bool conv_p16c4_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16);
int conv_p16c4_tile_count();
void conv_p16c4_tile(int index, int* k, int* th, int* tw, int* steps);
size_t conv_p16c4_lds_bytes(const ConvP16Params& p, int k);
int launch_conv_p16c4(const ConvP16Params& p, int k, hipStream_t s);
// the K-resident form for layers with few positions (k = 1 or 3, stride 1) on the same parameters: tiles of 4x4
// positions, blocks of 16*wm output channels, the whole reduction of a tile in LDS; wpack: [cout block][wave 0..3][step]
// [fragment][plane][lane][8 halves], a wave's steps being (chunk wave + 4*i, tap)
// 1x1 convolution without LDS for many positions and at most 256 input channels (conv_d16.hip), on the same parameters
bool conv_d16_supported(int k, int dil, int in_cp, int chunks, int cout, int out_cp);
int launch_conv_d16(const ConvP16Params& p, hipStream_t s);   // (p.dw_in set: with a depthwise 3x3 layer in front computed by the waves, conv_d16_dw_supported)
bool conv_d16_dw_supported(int chunks, int dw_stride);
// (p.tile_h = 3, 5 or 7: a K x K convolution on an input of at most four channels instead, cin_chunks = steps of eight taps)
bool conv_d16_small_supported(int k, int dil, int in_cp, int cout, int out_cp);
// a 1x1 layer and the depthwise 3x3 layer behind it as one launch (conv_d16.hip: conv_e16dw_kernel)
bool conv_e16dw_supported(int in_cp, int chunks, int dw_stride);
int launch_conv_e16dw(const ConvP16Params& p, hipStream_t s);
int conv_kr16_variant_count();
void conv_kr16_variant(int index, int* taps, int* chunks, int* fm, int* th, int* tw, int* stride);   // compiled combinations: kernel taps, 32-channel chunks, fragments per block, tile
size_t conv_kr16_lds_bytes(const ConvP16Params& p, int k);
int launch_conv_kr16(const ConvP16Params& p, int k, hipStream_t s);
// the K x K convolution (K = 3 or 9, stride 1) between fp16 tensors on the same parameters (conv_h16.hip): 128 output
// channels per workgroup, two tiles of tile_h x tile_w positions side by side; wpack: [(chunk*K + ky)*K + kx][cout
// fragment of 16][lane][8 halves], one plane
bool conv_h16_supported(int k, int stride, int dil, int in_cp, int cout, int out_cp, bool f16);
int conv_h16_tile_count();
void conv_h16_tile(int index, int* k, int* th, int* tw);
size_t conv_h16_lds_bytes(const ConvP16Params& p, int k);
int launch_conv_h16(const ConvP16Params& p, int k, hipStream_t s);

// ---------------------------------------------------------------------------------------------
// Direct (non-MFMA) layer kernels (layers_direct.hip)
// ---------------------------------------------------------------------------------------------
struct ConvDirectParams {
    TView in, out, res;  // res.ptr == nullptr: none
    const float* w;      // [ky][kx][cin][coutp] fp32 (coutp = out.cp)
    const float* scale;
    const float* bias;
    int k, dil, stride;
    int in_y0, in_x0;    // stored coord of tap (0,0) for output (0,0)
    int clamp;           // 1: coordinates clamp to the stored tensor's edge (the sampler's rule for shallow layers: an
                         //    unpadded input repeats its edge, a padded one reads its zero halo)
    int frac_shift;      // 0: ordinary taps.  s > 0 (fractional-step convolution, sourceStep = 2^(1-s)): tap t of output
                         //    x reads stored column pad + floor((2*(stride*x + t) + 1) / 2^s), t = kx + tap_x0 (ky + tap_y0)
    int tap_x0, tap_y0;
    int res_relu, res_scale;
    Act act;
};
void launch_conv_direct(const ConvDirectParams& p, hipStream_t s);

struct DwConvParams {
    TView in, out, res;
    const float* w;      // [9][cp] fp32
    const float* scale;
    const float* bias;
    int dil, stride;
    int res_relu, res_scale;
    int no_strips;       // keep to the one-row kernels (a test switch)
    Act act;
};
void launch_dwconv3x3(const DwConvParams& p, hipStream_t s);

struct PoolParams {
    TView in, out;
    int pool, stride;
    int off;             // window start relative to stored (y*stride, x*stride)
    int is_max;
    Act act;
};
void launch_pool(const PoolParams& p, hipStream_t s);
// partial / splits: for large images, splits x in.cp floats of scratch memory; the pixels are then dealt to `splits`
// workgroups per run of channel groups and a second launch pools their results (null / 1: one launch)
void launch_global_pool(const TView& in, const TView& out, int is_max, const Act& act, hipStream_t s, float* partial = nullptr, int splits = 1);

struct BnParams {
    TView in, out, res;
    const float* scale;
    const float* bias;
    int res_relu, res_bn;
    Act act;
};
void launch_batchnorm(const BnParams& p, hipStream_t s);
void launch_addsub(const TView& a, const TView& b, const TView& out, int sub, const Act& act, hipStream_t s);

// Function-type layers with one input and no weights.  Every output texel (4 channels) is produced from ONE source
// texel picked by `map` and passed through `fn`; the stencil modes (linear scaling, non-maximum suppression,
// blur) have kernels of their own.  Source coordinates beyond the stored input repeat its edge.
enum FuncMap { FMAP_SCALE = 0, FMAP_TRANSPOSE = 1, FMAP_IMGEXTRACT = 2 };
enum FuncFn { FFN_COPY = 0, FFN_SIGMOID = 1, FFN_TANH = 2, FFN_ARITH = 3, FFN_CAST = 4, FFN_BGR = 5 };
struct FuncParams {
    TView in, out;
    Act act;
    int map, fn;
    int op;          // FFN_ARITH: 0 add, 1 sub, 2 mul, 3 div; FFN_CAST: cast target 0..7
    float operand;
    // FMAP_SCALE: source position of output x = ((2x+1)*dx - ox) / (2*ux) texels (floor = nearest)
    int ux, uy, dx, dy, ox, oy;
    int window, in_groups;   // FMAP_IMGEXTRACT
};
void launch_func(const FuncParams& p, hipStream_t s);
void launch_scale_linear(const FuncParams& p, hipStream_t s);
void launch_nonmax(const TView& in, const TView& out, hipStream_t s);
// coef: device array [k*k] floats, taps (-r..last)^2 with coefficients in running order
void launch_blur(const TView& in, const TView& out, const float* coef, int r, int last, hipStream_t s);
// Copies channels [0, in.c) of `in` to channels [c_off, c_off + in.c) of `out` (activated); last: also zeroes the pad
// lanes [c_off + in.c, out.cp).
void launch_concat_part(const TView& in, const TView& out, int c_off, const Act& act, hipStream_t s, bool last);
// out: 2 channels (index as float, max value); idx_out optional int32 [h*w].
void launch_argmax(const TView& in, const TView& out, int32_t* idx_out, const Act& act, hipStream_t s);

// Second stage of a convolution with few output channels and a wide kernel (cout*K <= 32): the MFMA
// stage produced q[y][x'][o*K+kx] = sum_{ky,ci} W[o,ky,kx,ci]*act(in[y+ky-r, x'-r, ci]) for x' in
// [0, W+K-1); this stage forms out[y,x,o] = (sum_kx q[y][x+kx][o*K+kx]) * scale + bias' (+ residual).
struct ShiftReduceParams {
    TView q, out, res;
    int k, cout;
    float acc_mul;
    const float* scale;
    const float* bias;
    int res_relu, res_scale;
    unsigned* out_amax;        // value-range word of the output tensor or null (range.h)
};
void launch_shift_reduce(const ShiftReduceParams& p, hipStream_t s);

// Second pass of a split-K convolution: out = (sum_ks partial[ks]) * acc_mul * scale + bias (+ residual).
struct SplitKReduceParams {
    const float* partial;      // [ksplit][npos_y * npos_x][cout_pad]
    int ksplit, npos_y, npos_x, cout_pad;
    void* out;                 // engine tensor; same addressing fields as ConvMfmaParams
    const void* res;
    int out_f16;
    int out_wp, out_cp, out_step, out_off_y, out_off_x;
    int res_wp, res_cp, res_off_y, res_off_x;
    int res_relu, res_scale;
    float acc_mul;
    const float* scale;
    const float* bias;
    unsigned* out_amax;        // value-range word of the output tensor or null (range.h)
};
void launch_splitk_reduce(const SplitKReduceParams& p, hipStream_t s);

struct GemvParams {
    TView in, out;       // 1x1 spatial
    const void* w;       // [cout][cinp] in storage type (f16) or fp32
    const void* w_split; // launch_fc_mfma on fp32 tensors: [cout][cinp / 8][8 x fp16 hi | 8 x fp16 lo] of the same matrix (null: none)
    int w_f16;
    const float* scale;
    const float* bias;
    Act act;
};
void launch_gemv(const GemvParams& p, hipStream_t s);
// The same layer on the matrix cores (16 output rows per workgroup, the reduction split over its four waves): tensors and
// matrix of one storage type, 32 to 8192 (fp32) or 16384 (fp16) input channels; fp32 tensors: the matrix once more as fp16
// halves (w_split), which asks for weights inside fp16's range (the caller checks).
bool fc_mfma_supported(const GemvParams& p);
int launch_fc_mfma(const GemvParams& p, hipStream_t s);

// Layout conversion between the engine layout and CHW fp32 staging buffers.
// (amax: value-range word of the tensor, raised by what is written, or null; range.h)
void launch_chw_to_tensor(const float* chw, const TView& t, hipStream_t s, unsigned* amax = nullptr);   // net area only
void launch_tensor_to_chw(const TView& t, float* chw, int include_padding, hipStream_t s);
void launch_hwc_to_tensor(const float* hwc, int pc, const TView& t, hipStream_t s, unsigned* amax = nullptr);   // GPU_SHALLOW in
void launch_tensor_to_hwc(const TView& t, float* hwc, int pc, hipStream_t s);             // GPU_SHALLOW out
void launch_fill_zero(void* ptr, size_t bytes, hipStream_t s);
int launch_poison_lds(hipStream_t s);   // debugging aid: all-ones words into every CU's LDS

}  // namespace fynhip
