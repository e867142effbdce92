// Shared by the translation units of the TILED family (gptq_tiled.hip: preparation, pack pass, matmul and its
// transposed form; gptq_tiled_decode.hip and gptq_tiled_decode16.hip: the two decode kernels): how a lane's words of
// a block are addressed and loaded, the magic constants of the register unpack, and what the decode kernels share.
#pragma once
#include <type_traits>
#include <utility>

#include "gptq_device.h"

namespace gptq {

struct alignas(4) W3 {
    uint32_t a, b, c;
};

// Byte offset of lane l's words inside a block, and the lane's load.  Word i of a lane sits at
// l * BITS + i, except for 8 bits: (i / 4) * 256 + l * 4 + i % 4, so that each of the two loads is coalesced.
template <int BITS>
__device__ __forceinline__ constexpr uint32_t tile_lane_bytes(uint32_t l)
{
    return BITS == 8 ? l * 16u : l * (4u * BITS);
}

template <int BITS>
__device__ __forceinline__ void tile_load(const char *src, uint32_t (&wr)[BITS])
{
    if constexpr (BITS == 4) {
        const u4 v = __builtin_nontemporal_load((const u4 *)src);
#pragma unroll
        for (int e = 0; e < 4; e++) wr[e] = v[e];
    } else if constexpr (BITS == 8) {
        const u4 v0 = __builtin_nontemporal_load((const u4 *)src);
        const u4 v1 = __builtin_nontemporal_load((const u4 *)(src + 1024));
#pragma unroll
        for (int e = 0; e < 4; e++) {
            wr[e] = v0[e];
            wr[4 + e] = v1[e];
        }
    } else if constexpr (BITS == 2) {
        const u2 v = __builtin_nontemporal_load((const u2 *)src);
        wr[0] = v[0];
        wr[1] = v[1];
    } else {
        const W3 v = *(const W3 *)src;
        wr[0] = v.a;
        wr[1] = v.b;
        wr[2] = v.c;
    }
}

// The same load through a buffer resource that spans one column tile: the lane's byte offset in a vector register
// that never changes, the block's offset in a scalar register (no per-lane address arithmetic per block).  The
// scalar offset is NOT part of the buffer's range check on this architecture: the caller keeps the block inside
// the tile.
typedef uint32_t u3v __attribute__((ext_vector_type(3)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_buffer(const char *tile, uint32_t bytes)
{
    // (a wave-uniform base; data format word of a raw buffer on this architecture)
    const uint64_t a = (uint64_t)tile;
    // (readfirstlane returns a signed int: through uint32_t, or the low half would sign-extend into the high one)
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
    const uint64_t u = ((uint64_t)hi << 32) | (uint64_t)lo;
    return __builtin_amdgcn_make_buffer_rsrc((void *)u, 0, bytes, 0x00020000);
}

template <int BITS>
__device__ __forceinline__ void tile_load(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_bytes, uint32_t block_bytes,
                                          uint32_t (&wr)[BITS])
{
    constexpr int NT = 2;   // the non-temporal hint the pointer loads above carry
    if constexpr (BITS == 4) {
        const u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, block_bytes, NT);
#pragma unroll
        for (int e = 0; e < 4; e++) wr[e] = v[e];
    } else if constexpr (BITS == 8) {
        const u4 v0 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, block_bytes, NT);
        const u4 v1 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes + 1024u, block_bytes, NT);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            wr[e] = v0[e];
            wr[4 + e] = v1[e];
        }
    } else if constexpr (BITS == 2) {
        const u2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_bytes, block_bytes, NT);
        wr[0] = v[0];
        wr[1] = v[1];
    } else {
        const u3v v = __builtin_amdgcn_raw_buffer_load_b96(rsrc, lane_bytes, block_bytes, 0);
        wr[0] = v[0];
        wr[1] = v[1];
        wr[2] = v[2];
    }
}

// N 16-byte loads issued together and waited for in place, as ONE asm statement: the compiler's own bookkeeping of
// outstanding loads does not see them (a loop of ordinary loads made it put waits for every outstanding load far
// away from the loop, in front of code that every layer runs), and nothing can use a value before it has arrived.
// The wait also covers every older load of the wave: such loops stand before the weight requests.
#define GPTQ_LD(o, i) "global_load_dwordx4 %" #o ", %" #i ", off\n\t"
template <int N>
struct LoadNow;
template <>
struct LoadNow<1> {
    static __device__ __forceinline__ void run(u4 (&v)[1], const void *const (&p)[1])
    {
        asm volatile(GPTQ_LD(0, 1) "s_waitcnt vmcnt(0)" : "=&v"(v[0]) : "v"(p[0]) : "memory");
    }
};
template <>
struct LoadNow<2> {
    static __device__ __forceinline__ void run(u4 (&v)[2], const void *const (&p)[2])
    {
        asm volatile(GPTQ_LD(0, 2) GPTQ_LD(1, 3) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]) : "v"(p[0]), "v"(p[1]) : "memory");
    }
};
template <>
struct LoadNow<3> {
    static __device__ __forceinline__ void run(u4 (&v)[3], const void *const (&p)[3])
    {
        asm volatile(GPTQ_LD(0, 3) GPTQ_LD(1, 4) GPTQ_LD(2, 5) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
    }
};
template <>
struct LoadNow<4> {
    static __device__ __forceinline__ void run(u4 (&v)[4], const void *const (&p)[4])
    {
        asm volatile(GPTQ_LD(0, 4) GPTQ_LD(1, 5) GPTQ_LD(2, 6) GPTQ_LD(3, 7) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
    }
};
template <>
struct LoadNow<5> {
    static __device__ __forceinline__ void run(u4 (&v)[5], const void *const (&p)[5])
    {
        asm volatile(GPTQ_LD(0, 5) GPTQ_LD(1, 6) GPTQ_LD(2, 7) GPTQ_LD(3, 8) GPTQ_LD(4, 9) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]) : "memory");
    }
};
template <>
struct LoadNow<8> {
    static __device__ __forceinline__ void run(u4 (&v)[8], const void *const (&p)[8])
    {
        asm volatile(GPTQ_LD(0, 8) GPTQ_LD(1, 9) GPTQ_LD(2, 10) GPTQ_LD(3, 11) GPTQ_LD(4, 12) GPTQ_LD(5, 13) GPTQ_LD(6, 14) GPTQ_LD(7, 15) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]) : "memory");
    }
};
template <>
struct LoadNow<9> {
    static __device__ __forceinline__ void run(u4 (&v)[9], const void *const (&p)[9])
    {
        asm volatile(GPTQ_LD(0, 9) GPTQ_LD(1, 10) GPTQ_LD(2, 11) GPTQ_LD(3, 12) GPTQ_LD(4, 13) GPTQ_LD(5, 14) GPTQ_LD(6, 15) GPTQ_LD(7, 16) GPTQ_LD(8, 17) "s_waitcnt vmcnt(0)" : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]), "=&v"(v[8]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]), "v"(p[8]) : "memory");
    }
};
#undef GPTQ_LD

// The magic constants of the width's unpack, each held in a vector register.
template <int BITS>
__device__ __forceinline__ void tile_magic(uint32_t (&mg)[TileCodec<BITS>::KINDS])
{
#pragma unroll
    for (int k = 0; k < TileCodec<BITS>::KINDS; k++) mg[k] = opaque_vgpr(TileCodec<BITS>::MAGIC[k]);
}

// ---- shared by the two decode kernels ----
typedef float f2 __attribute__((ext_vector_type(2)));

// 8-bit layers: the decode kernels dequantise every weight as the reference rounds it (fp16(scale * (q - zero)),
// the matmul kernel's arithmetic).  Their weights are sixteen times those of a 4-bit layer, and so is the
// distance between exact products and the reference's rounded ones; the extra packed instructions hide
// behind a stream that is twice as long per weight.
constexpr bool tiled_decode_exact(int bits) { return bits == 8; }

// the sixteen unpacked registers of a lane -> fp16(scale * (q - zero)); sz = fp16 scale | fp16 zero << 16
template <int BITS>
__device__ __forceinline__ void tiled_dequant_exact(u4 (&q)[4], uint32_t sz)
{
    using Codec = TileCodec<BITS>;
    const h2 e = as_h2(sz);
    const h2 s2 = {e[0], e[0]};
    h2 zb[Codec::KINDS];
#pragma unroll
    for (int k = 0; k < Codec::KINDS; k++)
        zb[k] = (h2){e[1], e[1]} + (h2){(_Float16)Codec::base(2 * k), (_Float16)Codec::base(2 * k + 1)};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) q[j][r] = as_u32((as_h2(q[j][r]) - zb[r % Codec::KINDS]) * s2);
}

// v of lane l + N inside its row of 16 lanes (zero past the row's end)
template <int N>
__device__ __forceinline__ float row_shl(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + N, 0xf, 0xf, true));
}

// y = fp16(sum over split of partial[split] (+ bias)): the pass after a product whose K range was cut over
// workgroups (defined in gptq_tiled.hip); out_map: the transposed product's channel map, else nullptr.
int launch_tiled_reduce(const float *partial, const void *bias, void *y, int M, int N, int split_k, const int32_t *out_map,
                        hipStream_t stream);

}  // namespace gptq
