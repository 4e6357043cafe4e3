// Value-range bookkeeping for the fp32-storage convolution path.
//
// With fp32 storage the matrix-core convolution splits every operand into two fp16 numbers (x = hi + lo).  fp16 covers
// 2^-24 .. 65504, so the split is exact to 22 bits only while the activations of a tensor sit in a window around 1.
// Producers that can do so at no cost (the convolution epilogues and the host-input converters) therefore record the
// largest magnitude they wrote in a per-tensor record (bit patterns of non-negative floats, combined with an integer
// atomic maximum, which is exact and independent of the order of arrival); a consuming convolution reads the record
// at kernel start, multiplies what it stages by a power of two that brings that magnitude to [2^13, 2^14), and folds
// the inverse into the factor it applies to its accumulators.  A record that reads 0 means "not known": scale 1.
// Records are cleared by a convolution kernel that runs between the tensor's last reader and its next producer.
//
// A record is RANGE_SLOTS words, each in a cache line of its own (RANGE_STRIDE words apart), two per XCD.  Device-wide
// atomics are carried out at the memory side, one after the other per address and some 15 ns each (ten thousand waves
// raising one word took longer than the convolution they belonged to; spread over 64 words they still cost a launch
// of 3000 workgroups 2 us).  A workgroup therefore raises a word that belongs to its own XCD, with an atomic of
// workgroup scope, which the XCD's L2 carries out: all workgroups that touch the word share that L2, the kernel's end
// writes the line back, and the reader (a later kernel) takes the maximum over all slots with one load per lane.
#pragma once
#include <hip/hip_runtime.h>

namespace fynhip {

constexpr int RANGE_SLOTS = 16;                                  // 8 XCDs x 2
constexpr int RANGE_STRIDE = 64;                                 // words between slots (256 bytes)
constexpr int RANGE_WORDS = RANGE_SLOTS * RANGE_STRIDE;          // words per record

// Maximum of a wave's 64 values (all lanes active) on the vector ALUs' data-parallel paths: shifts inside rows of 16
// lanes, then the row maxima broadcast into the following rows; lane 63 ends up with the wave's maximum.  Six
// instructions; the same through __shfl_xor is six dependent LDS-crossbar round trips, about 700 cycles, which at the
// end of every workgroup of a launch added up to 0.5-2 us per launch.
__device__ __forceinline__ unsigned range_wave_umax(unsigned v) {
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false));   // row_shr:1
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false));   // row_shr:2
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false));   // row_shr:4
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false));   // row_shr:8
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false));   // row_bcast:15 into rows 1, 3
    v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false));   // row_bcast:31 into rows 2, 3
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}
// (bit patterns of non-negative floats order like the floats)
__device__ __forceinline__ float range_wave_max(float m) { return __uint_as_float(range_wave_umax(__float_as_uint(m))); }

__device__ __forceinline__ unsigned* range_slot(unsigned* record) {
    // XCC_ID: hardware register 20, bits 3:0 (the XCD this wave runs on)
    const unsigned xcc = (unsigned)__builtin_amdgcn_s_getreg((3 << 11) | 20) & 7u;
    return record + (xcc * 2u + ((blockIdx.x + blockIdx.y) & 1u)) * RANGE_STRIDE;
}
__device__ __forceinline__ void range_raise(unsigned* record, float m) {
    if (m > 0.f) (void)__hip_atomic_fetch_max(range_slot(record), __float_as_uint(m), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// Barrier that orders LDS traffic only.  __syncthreads() and __threadfence_block() also wait for the global stores a
// wave has in flight -- at the end of an epilogue that is one memory round trip per workgroup.
__device__ __forceinline__ void range_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Every thread of a workgroup of 256 (all of them alive) calls this with its own maximum (>= 0; NaNs are ignored);
// one device-wide atomic per workgroup.
__device__ __forceinline__ void range_publish_block256(unsigned* record, float m) {
    __shared__ float wave_max[4];
    static_assert(RANGE_SLOTS <= 64, "one slot per lane");
    m = range_wave_max(m);
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    range_lds_barrier();
    if (threadIdx.x == 0) range_raise(record, fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3])));
}

// The same for `nwaves` waves of a workgroup that finish at different times and share no barrier any more: `box` is
// two LDS words that were zero when the first of them arrived; the wave that arrives last publishes.  All 64 lanes
// call.  (The LDS executes one wave's operations in the order of issue; the compiler is kept from reordering them.)
__device__ __forceinline__ void range_publish_waves(unsigned* record, float m, unsigned* box, unsigned nwaves) {
    m = range_wave_max(m);
    if ((threadIdx.x & 63) == 0) {
        atomicMax(&box[0], __float_as_uint(m));
        asm volatile("" ::: "memory");
        if (atomicAdd(&box[1], 1u) == nwaves - 1) {
            asm volatile("" ::: "memory");
            range_raise(record, __uint_as_float(atomicMax(&box[0], 0u)));
        }
    }
}

// The record's maximum in two steps, so that the load can be issued early and waited for late: range_load gives each
// lane its slot (bit patterns of non-negative floats order like the floats), range_reduce the maximum to every lane.
__device__ __forceinline__ unsigned range_load(const unsigned* record) {
    const int lane = threadIdx.x & 63;
    return lane < RANGE_SLOTS ? record[lane * RANGE_STRIDE] : 0u;
}
__device__ __forceinline__ float range_reduce(unsigned v) { return __uint_as_float(range_wave_umax(v)); }

// Workgroup 0 of a kernel (at least 128 threads) clears the up to four records in its care: thread t the slot
// t % RANGE_SLOTS of record t / RANGE_SLOTS.  (The records are named one by one: an array of kernel arguments indexed
// per lane makes the compiler keep the whole argument block in vector registers.)
__device__ __forceinline__ void range_clear(unsigned* r0, unsigned* r1, unsigned* r2, unsigned* r3, int count) {
    static_assert(4 * RANGE_SLOTS <= 128, "one thread per slot");
    const int t = threadIdx.x, which = t / RANGE_SLOTS;
    unsigned* r = which == 0 ? r0 : (which == 1 ? r1 : (which == 2 ? r2 : r3));
    if (which < count && which < 4) atomicExch(r + (t % RANGE_SLOTS) * RANGE_STRIDE, 0u);
}

// Largest magnitude act(x) can take for |x| <= amax, act(x) = min(hi, max(lo, x)) + leak * min(x, 0).
__device__ __forceinline__ float range_after_act(float amax, const Act& a) {
    const float up = fminf(a.hi, fmaxf(a.lo, amax));
    const float dn = fminf(a.hi, fmaxf(a.lo, -amax)) - a.leak * amax;
    return fmaxf(fabsf(up), fabsf(dn));
}

// Power of two s with bound * s in [2^13, 2^14); 1 when the bound is unknown (0), infinite or not a number.  *inv = 1/s.
__device__ __forceinline__ float range_scale(float bound, float* inv) {
    const unsigned bits = __float_as_uint(bound);
    const int e = (int)((bits >> 23) & 0xff);          // biased exponent
    if (e == 0 || e == 0xff) {
        *inv = 1.f;
        return 1.f;
    }
    int k = 13 - (e - 127);                             // bound in [2^(e-127), 2^(e-126))
    k = k < -60 ? -60 : (k > 60 ? 60 : k);
    *inv = __uint_as_float((unsigned)(127 - k) << 23);
    return __uint_as_float((unsigned)(127 + k) << 23);
}

}  // namespace fynhip
