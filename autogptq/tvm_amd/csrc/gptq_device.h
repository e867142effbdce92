// Device-side pieces shared by the GPTQ int3/int4 matmul kernels on gfx950 (CDNA4, wave64).
//
// Common geometry of the matmul kernels
// -------------------------------------
// The product runs on v_mfma_f32_16x16x32_f16.  A wave owns 64 output columns:
// lane (i = lane % 16, q = lane / 16) loads one 128-bit vector of qweight per packed
// row, i.e. the four adjacent columns n0 + 4i .. n0 + 4i + 3, so a wave load is four
// 256-byte runs.  Column set c (0..3) of a wave is {n0 + 4i + c : i = 0..15}; it is the
// N dimension of one MFMA.  The K dimension of an MFMA is 4 lane groups x 8 codes:
// lane group q supplies 8 codes of ITS packed row (int4: one word row = 8 codes;
// int3: one 3-word block = 32 codes = four MFMAs), and the activation operand
// supplies x for the same input channels in the same order.  That order is the
// "slot" order of gptq_unpack.h (codes come out of the magic-number unpack in pairs
// that are not adjacent in k); x reaches the matrix instruction already permuted into slot order
// (in LDS for GROUPED and GATHER, by the pack pass or register permutes for STREAM).
//
// One "step" of a wave is 4 packed rows (int4: 32 input channels, int3: 128).
#pragma once
#include <hip/hip_runtime.h>

#include "gptq_internal.h"
#include "gptq_unpack.h"

namespace gptq {

template <int BITS>
struct Fmt;
template <>
struct Fmt<4> {
    static constexpr int KLANE = 8;    // codes per lane per step
    static constexpr int NB = 1;       // MFMAs along K per column set per step
    static constexpr int WORDS = 1;    // 128-bit loads per lane per step
    static constexpr int KSTEP = 32;   // input channels per wave step
};
template <>
struct Fmt<3> {
    static constexpr int KLANE = 32;
    static constexpr int NB = 4;
    static constexpr int WORDS = 3;
    static constexpr int KSTEP = 128;
};

struct InvTables {
    unsigned char inv4[8];
    unsigned char inv3[32];
    constexpr InvTables() : inv4(), inv3()
    {
        for (int s = 0; s < 8; s++) inv4[SLOT4[s]] = (unsigned char)s;
        for (int s = 0; s < 32; s++) inv3[SLOT3[s]] = (unsigned char)s;
    }
};
static __constant__ InvTables kInv = InvTables();

// The same tables as immediates, for a thread that owns codes 4 q .. 4 q + 3 of a lane block: byte q
// of quad_slots<BITS>(e) is the slot of code 4 q + e.  A lookup in kInv is a load from constant memory
// that nothing else in a kernel has touched yet: it costs a full memory latency at the top of the
// kernel and sits first in the in-order return queue of every later load.
template <int BITS>
__device__ __forceinline__ constexpr uint64_t quad_slots(int e)
{
    constexpr InvTables t = InvTables();
    uint64_t w = 0;
    for (int q = 0; q < Fmt<BITS>::KLANE / 4; q++) {
        w |= (uint64_t)(BITS == 4 ? t.inv4[4 * q + e] : t.inv3[4 * q + e]) << (8 * q);
    }
    return w;
}

// slot (position in the MFMA operand order) of code j of a lane block
template <int BITS>
__device__ __forceinline__ int slot_of_code(int j)
{
    return BITS == 4 ? (int)kInv.inv4[j] : (int)kInv.inv3[j];
}

template <int BITS>
__device__ __forceinline__ int zero_of(const uint32_t *zrow, int n)
{
    if constexpr (BITS == 3) {
        return zero3(zrow, n);
    } else {
        return code_pow2<BITS>(zrow + (n >> 5) * BITS, n & 31) + 1;
    }
}

// The words holding the four zero points of columns n .. n+3 (n % 4 == 0) of the qzeros row
// that starts zrow_off words into qzeros.  32-bit offsets from the uniform base pointer.
template <int BITS>
__device__ __forceinline__ void load_zero_words(const uint32_t *qzeros, uint32_t zrow_off, int n, uint32_t &wa,
                                                uint32_t &wb)
{
    if constexpr (BITS == 4) {
        wa = *(const uint32_t *)((const char *)qzeros + (zrow_off + (uint32_t)(n >> 3)) * 4u);
        wb = 0u;
    } else {
        const uint32_t blk = zrow_off + 3u * (uint32_t)(n >> 5);
        const uint32_t w = (3u * (uint32_t)(n & 31)) >> 5;  // word of the 12-bit field inside the 96-bit block
        wa = *(const uint32_t *)((const char *)qzeros + (blk + w) * 4u);
        wb = *(const uint32_t *)((const char *)qzeros + (blk + (w < 2u ? w + 1u : 2u)) * 4u);
    }
}

template <int BITS>
__device__ __forceinline__ void zeros_from_words(uint32_t wa, uint32_t wb, int n, float z[4])
{
    if constexpr (BITS == 4) {
        const uint32_t f = wa >> (16 * ((n >> 2) & 1));
#pragma unroll
        for (int c = 0; c < 4; c++) z[c] = (float)(int)(((f >> (4 * c)) & 0xfu) + 1u);
    } else {
        const int sh = (3 * (n & 31)) & 31;
        const uint32_t f = (uint32_t)((((uint64_t)wb << 32) | (uint64_t)wa) >> sh);
#pragma unroll
        for (int c = 0; c < 4; c++) z[c] = (float)(int)(((f >> (3 * c)) & 0x7u) + 1u);
    }
}

extern __shared__ __align__(16) unsigned char smem[];

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also carries a memory fence
// that waits for every outstanding global load (s_waitcnt vmcnt(0)), which drains the weight
// prefetch at every barrier and exposes the full HBM latency each time; these kernels only
// exchange data through LDS at their barriers, so waiting for the LDS counter is enough.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0) only (gfx9 encoding: vmcnt and expcnt left at max)
    __builtin_amdgcn_s_barrier();
}

// ---------------------------------------------------------------------------------
// Split-K tail: every workgroup of a column tile writes its fp32 partial tile, the one
// that arrives last adds them in split order (so the sum does not depend on arrival
// order) and writes y.
//
// The partials travel through device-coherent accesses only (write-through stores and
// L2-bypassing loads, the instructions an agent-scope atomic store/load compiles to), so no cache
// writeback or invalidate is needed around the counter: an agent-scope release fence
// here costs a whole-L2 writeback per wave, which serialises the workgroups of an XCD
// and dominated the run time of the first version of these kernels.  Waiting for the
// stores to be acknowledged before the counter is bumped is all the ordering required.
// ---------------------------------------------------------------------------------
// Device-coherent store / load of four floats as two 64-bit relaxed agent-scope atomics
// (global_store_dwordx2 sc1 / global_load_dwordx2 sc1): the widest such access the language
// offers.  (A hand-written 128-bit "sc0 sc1" instruction in inline assembly halves the count
// again, but next to the matrix instructions of the tallest tiles it read one accumulator
// register too early in a few lanes; the compiler does not track hazards into inline assembly.)
__device__ __forceinline__ void store_partial(float *dst, f4 v)
{
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
    __hip_atomic_store((unsigned long long *)dst, __builtin_bit_cast(unsigned long long, lo), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store((unsigned long long *)dst + 1, __builtin_bit_cast(unsigned long long, hi), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ f4 load_partial(const float *src)
{
    typedef float f2 __attribute__((ext_vector_type(2)));
    const unsigned long long a =
        __hip_atomic_load((const unsigned long long *)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long b =
        __hip_atomic_load((const unsigned long long *)src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const f2 lo = __builtin_bit_cast(f2, a), hi = __builtin_bit_cast(f2, b);
    return (f4){lo[0], lo[1], hi[0], hi[1]};
}

// Returns true in the workgroup that must do the final sum.  Every thread calls it.
__device__ __forceinline__ bool arrive_last(int *counter, int split_k, int *lds_flag)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial stores are acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = (old == split_k - 1);
        if (last) {
            // leave the counter at zero for the next launch that uses this workspace
            __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        *lds_flag = last;
    }
    __syncthreads();
    return *lds_flag != 0;
}

}  // namespace gptq
