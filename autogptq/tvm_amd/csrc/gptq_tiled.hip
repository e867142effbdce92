// TILED kernel family: the product on a layer that was re-laid once, when it was loaded, into the
// order the matrix instructions consume (gptq_hip_tile_prepare), for any number of rows of x.
//
// The tiled format (also stated in torch ops by pack.tile_layout, which the tests compare with):
//   * the input channels are sorted by group (stable; the identity without an activation order), so
//     position p of the sorted order holds channel xsrc[p] and its group is p / group_size;
//   * qtile is a sequence of blocks, column tile T (32 columns) outermost, then block S (64 positions);
//     block (T, S) is 64 lanes x BITS words, one coalesced wave load (two for 8 bits, whose block is laid
//     out as two halves of 64 lanes x 4 words).  Lane (n = lane % 32, h = lane / 32) holds the 32 codes of
//     column 32 T + n at positions 64 S + 32 h .. + 31, permuted inside the lane so that the register
//     unpack of gptq_unpack.h (TileCodec) yields them in position order: the lane's words are the B
//     operand of four v_mfma_f32_32x32x16_f16 (positions 8 j .. 8 j + 7 of the lane for j = 0..3) with
//     no shuffle;
//   * sz[g][n] = (fp16 scale, fp16 zero point) of group g, column n, one 32-bit word.
//
// tiled_gemm_kernel: a workgroup owns 64 columns (two tiles), 32 * AT rows of x and one K range; its four
// waves (one per SIMD) split that range and never talk until the end.  A wave holds its whole 32 AT x 64
// result in registers (AT = 4: 128 rows, 128 accumulator registers), dequantises every weight of its slice
// exactly once, as the reference does (fp16(scale * (q - zero)), one rounding), and reads x as ready-made A
// fragments that a small pack pass wrote (rows past M and positions past K as zeros).  One wave per SIMD
// overlaps its own vector and matrix instructions (measured: up to six packed-fp16 instructions per
// 32x32x16 matrix instruction are free), so the dequantisation of the next B operand is interleaved with the
// matrix instructions of the current one.  Weights, (scale, zero) words and fragments ride in register
// rings RING blocks deep, requested in the order they are consumed (vector loads return in order on one
// counter, so a wait for a fragment also waits for every older load).
// Measured alternatives that were no faster: an L2 prefetch of the weights through scalar loads (slower: the
// scalar path does not sustain the rate); eight waves per workgroup (two per SIMD, 64-row waves, two row
// halves x four K slices or eight K slices); a wave's whole weight range brought into LDS up front with
// global_load_lds (a CU draws ~35 GB/s from HBM, and those 3.7 us then stand in front of the first matrix
// instruction).  What bounds the 128-row kernel is the A stream (every workgroup reads all of x through its
// CU's L1: 1 MB at ~130 GB/s), the matrix pipes of the 172 CUs that 11008 columns give work to, and the
// fixed costs around the loop.
// The four waves add their tiles through LDS at the end; workgroups along K (split_k > 1) leave fp32 tiles
// in the workspace for tiled_reduce_kernel.
#include <type_traits>
#include <utility>

#include "gptq_device.h"

namespace gptq {

typedef float f16v __attribute__((ext_vector_type(16)));

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

// The magic constants of the width's unpack, each held in a vector register.
template <int BITS>
__device__ __forceinline__ void tile_magic(uint32_t (&mg)[TileCodec<BITS>::KINDS])
{
#pragma unroll
    for (int k = 0; k < TileCodec<BITS>::KINDS; k++) mg[k] = opaque_vgpr(TileCodec<BITS>::MAGIC[k]);
}

// ---------------------------------------------------------------------------------------------------
// Preparation, pass 1: xsrc[p] = the channel at position p of the stable sort by group (the rank of a
// channel inside its group is the number of earlier channels of the same group), -1 for p >= K; and its
// inverse kinv[k] = the position of channel k (positions are below 65536).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void tile_map_kernel(const int32_t *__restrict__ g_idx, int32_t *__restrict__ xsrc,
                                                       uint16_t *__restrict__ kinv, int K, int Kp, int G, int group_size)
{
    __shared__ int tile[256];
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (!g_idx) {
        if (k < Kp) xsrc[k] = k < K ? k : -1;
        if (k < K) kinv[k] = (uint16_t)k;
        return;
    }
    const int g = k < K ? min(max(g_idx[k], 0), G - 1) : -1;
    int rank = 0;
    for (int t0 = 0; t0 <= (int)blockIdx.x * 256; t0 += 256) {
        const int j = t0 + threadIdx.x;
        __syncthreads();
        tile[threadIdx.x] = j < K ? min(max(g_idx[j], 0), G - 1) : -2;
        __syncthreads();
        const int upto = min(256, k - t0);
        for (int i = 0; i < upto; i++) rank += tile[i] == g ? 1 : 0;
    }
    if (k < K) {
        // a group with more than group_size members would leave its range: keep every index in bounds
        const int pos = g * group_size + min(rank, group_size - 1);
        xsrc[pos] = k;
        kinv[k] = (uint16_t)pos;
    } else if (k < Kp) {
        xsrc[k] = -1;
    }
}

// Pass 2: one thread per (column tile, block, lane) gathers its 32 codes through xsrc and writes its words.
template <int BITS>
__global__ __launch_bounds__(256) void tile_retile_kernel(const uint32_t *__restrict__ qweight,
                                                          const int32_t *__restrict__ xsrc, uint32_t *__restrict__ qtile,
                                                          int K, int N, int S_total, int T_total)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const int lane = t & 63;
    const uint32_t blk = t >> 6;  // T * S_total + S
    if (blk >= (uint32_t)T_total * (uint32_t)S_total) return;
    const int T = blk / S_total, S = blk - T * S_total;
    const int n = 32 * T + (lane & 31), h = lane >> 5;
    uint32_t words[BITS];
#pragma unroll
    for (int i = 0; i < BITS; i++) words[i] = 0u;
    for (int s = 0; s < 32; s++) {
        const int src = xsrc[64 * S + 32 * h + s];
        uint32_t q = 0u;
        if (src >= 0 && src < K) {
            const uint32_t *b = qweight + (size_t)(src >> 5) * BITS * N + n;  // the packed block of 32 channels
            const int bit = BITS * (src & 31);
            const int wd = bit >> 5, sh = bit & 31;
            q = b[(size_t)wd * N] >> sh;
            if (sh + BITS > 32) q |= b[(size_t)(wd + 1) * N] << (32 - sh);
            q &= (1u << BITS) - 1u;
        }
        // the stream field that the register unpack hands out as position s
        const int field = TileCodec<BITS>::field(s);
        const int obit = BITS * field;
        const int owd = obit >> 5, osh = obit & 31;
        words[owd] |= q << osh;
        if (osh + BITS > 32) words[owd + 1] |= q >> (32 - osh);
    }
#pragma unroll
    for (int i = 0; i < BITS; i++) {
        const int at = BITS == 8 ? (i >> 2) * 256 + lane * 4 + (i & 3) : lane * BITS + i;
        qtile[(size_t)blk * (64 * BITS) + at] = words[i];
    }
}

// Pass 3: sz[g][n] = fp16 scale | fp16 zero point << 16.
template <int BITS>
__global__ __launch_bounds__(256) void tile_sz_kernel(const uint32_t *__restrict__ qzeros,
                                                      const _Float16 *__restrict__ scales, uint32_t *__restrict__ sz,
                                                      int N, int G)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= (uint32_t)G * (uint32_t)N) return;
    const int g = t / N, n = t - g * N;
    const int z = zero_of<BITS>(qzeros + (size_t)g * (N / 32 * BITS), n);
    const h2 v = {scales[t], (_Float16)(float)z};
    sz[t] = as_u32(v);
}

int launch_tile_prepare(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *g_idx,
                        uint32_t *qtile, uint32_t *sz, int32_t *xsrc, uint16_t *kinv, int K, int N, int G, int bits,
                        int group_size, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const int Kp = (K + 63) / 64 * 64;
    const int S_total = Kp / 64, T_total = N / 32;
    hipLaunchKernelGGL(tile_map_kernel, dim3((Kp + 255) / 256), dim3(256), 0, stream, g_idx, xsrc, kinv, K, Kp, G,
                       group_size);
    const unsigned threads = (unsigned)T_total * (unsigned)S_total * 64u;
    const unsigned szt = (unsigned)G * (unsigned)N;
    auto go = [&](auto bits_c) {
        constexpr int B = decltype(bits_c)::value;
        hipLaunchKernelGGL(tile_retile_kernel<B>, dim3((threads + 255u) / 256u), dim3(256), 0, stream, qweight, xsrc, qtile,
                           K, N, S_total, T_total);
        hipLaunchKernelGGL(tile_sz_kernel<B>, dim3((szt + 255u) / 256u), dim3(256), 0, stream, qzeros,
                           (const _Float16 *)scales, sz, N, G);
    };
    switch (bits) {
        case 2: go(std::integral_constant<int, 2>{}); break;
        case 3: go(std::integral_constant<int, 3>{}); break;
        case 4: go(std::integral_constant<int, 4>{}); break;
        case 8: go(std::integral_constant<int, 8>{}); break;
        default: return GPTQ_HIP_ERR_BAD_ARG;
    }
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------------------------------
// Pack pass: x [M, K] -> A fragments of v_mfma_f32_32x32x16_f16.  Fragment (block S, j, row tile rt) is
// 64 lanes x 16 bytes; lane (m = lane % 32, h = lane / 32) holds x[32 rt + m][xsrc[64 S + 32 h + 8 j + e]],
// e = 0..7.  Rows past M and positions past K are zeros; blocks up to S_pack are written (the kernel's
// waves walk whole ranges, and their refills run a ring past the end).
// One workgroup per row: the row goes to LDS with coalesced loads and the gather through xsrc reads LDS
// (lanes that gather from global memory with one row per lane touch 64 cache lines per instruction).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void tile_pack_x_kernel(const _Float16 *__restrict__ x, const int32_t *__restrict__ xsrc,
                                                          char *__restrict__ xpack, int M, int K, int Kp, int rt_total,
                                                          int S_pack)
{
    const int row = blockIdx.x;
    const int rt = row >> 5, m = row & 31;
    const int tid = threadIdx.x;
    _Float16 *xl = (_Float16 *)smem;
    const bool live = row < M;
    const _Float16 *xr = x + (size_t)row * K;
    const int octets = S_pack * 8;
    int4 ia[2], ib[2];  // the map entries of this thread's first two octets, requested before the row is staged
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int p0 = min(8 * (tid + 256 * i), Kp - 8);
        ia[i] = xsrc ? *(const int4 *)(xsrc + p0) : make_int4(0, 0, 0, 0);
        ib[i] = xsrc ? *(const int4 *)(xsrc + p0 + 4) : make_int4(0, 0, 0, 0);
    }
    if (live && xsrc) {
        for (int i = tid; i < K / 8; i += 256) ((u4 *)xl)[i] = ((const u4 *)xr)[i];
    }
    __syncthreads();
    for (int o = tid, it = 0; o < octets; o += 256, it++) {
        const int p0 = 8 * o;
        const int S = p0 >> 6, h = (p0 >> 5) & 1, j = (p0 >> 3) & 3;
        h8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (live && p0 < Kp) {
            if (xsrc) {
                int4 a, b;
                if (it < 2) {
                    a = ia[it];
                    b = ib[it];
                } else {
                    a = *(const int4 *)(xsrc + p0);
                    b = *(const int4 *)(xsrc + p0 + 4);
                }
                const int idx[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const _Float16 t = xl[min((uint32_t)max(idx[e], 0), (uint32_t)K - 1u)];  // a bad map must not fault
                    v[e] = idx[e] >= 0 ? t : (_Float16)0;
                }
            } else if (p0 < K) {  // K is a multiple of 32: a run of 8 is inside or outside as a whole
                v = *(const h8 *)(xr + p0);
            }
        }
        *(h8 *)(xpack + ((size_t)(4 * S + j) * rt_total + rt) * 1024 + (h * 32 + m) * 16) = v;
    }
}

// ---------------------------------------------------------------------------------------------------
struct TiledParams {
    const char *xpack;     // A fragments, [S_pack * 4][rt_total][64 lanes][16 bytes]
    const char *qtile;     // [T_total][S_total][64 lanes][BITS words]
    const uint32_t *sz;    // [G][N]
    const void *bias;      // fp16 [N] or nullptr
    void *y;               // fp16 [M, N]
    float *partial;        // [split_k][M][N] when split_k > 1
    int M, N, G;
    int S_total, T_total;
    int wave_steps;        // blocks per wave
    int rt_total;          // 32-row tiles over all M blocks
    int split_k;
    int lb_per_group;      // group_size / 32
    // the transposed product only (TRANS): the roles of K and N are swapped, see tiled_gemm_kernel
    const uint32_t *szt;   // [G][S_total][8 octets][8 words]: per octet of columns, (scale, scale) x 4 | (base + zero) x 4
    const int32_t *out_map;  // channel of sorted position p (nullptr = identity): where column p of the result goes
    int tiles_per_group;   // group_size / 32: output tiles (32 positions) per group
};

// One B operand: positions 8 j .. 8 j + 7 of the lane, as fp16(scale * (q - zero)) exactly as the
// reference rounds it: (base + q) - (base + zero) is exact, the product rounds once.
template <int BITS>
__device__ __forceinline__ h8 tiled_bop(const uint32_t (&w)[BITS], int j, h2 s2, const h2 (&zb)[TileCodec<BITS>::KINDS],
                                        const uint32_t (&mg)[TileCodec<BITS>::KINDS])
{
    u4 q;
    TileCodec<BITS>::operand(w, j, q, mg);
    u4 o;
#pragma unroll
    for (int r = 0; r < 4; r++) o[r] = as_u32((as_h2(q[r]) - zb[r % TileCodec<BITS>::KINDS]) * s2);
    return __builtin_bit_cast(h8, o);
}

// The same for the transposed product, where the eight values of an operand are eight COLUMNS of the layer at one
// position: scale and (base + zero) differ per value and come as ready-made register pairs.
template <int BITS>
__device__ __forceinline__ h8 tiled_bop_t(const uint32_t (&w)[BITS], int j, const u4 &s2, const u4 &zb,
                                          const uint32_t (&mg)[TileCodec<BITS>::KINDS])
{
    u4 q;
    TileCodec<BITS>::operand(w, j, q, mg);
    u4 o;
#pragma unroll
    for (int r = 0; r < 4; r++) o[r] = as_u32((as_h2(q[r]) - as_h2(zb[r])) * as_h2(s2[r]));
    return __builtin_bit_cast(h8, o);
}

// AT: 32-row tiles per wave.  RW x KW: waves of the workgroup along M and along K: the workgroup holds
// 32 * AT * RW rows, and its KW waves along K split the workgroup's K range.  CT: 32-column tiles per wave (2, or
// 4 for problems of several row blocks: a fragment of x then feeds four matrix instructions instead of two,
// which halves the fragment traffic per flop, and the 256 accumulator registers fill the wave's second
// register file).
// TRANS: gx = gy @ W^T, the gradient of the product with respect to x.  The kernel is handed the tiled format of the
// TRANSPOSED code matrix (gptq_hip_tile_prepare_transposed): its "positions" are the layer's columns n (the
// reduction runs over them; x here is gy, packed like any x), its "columns" are the layer's sorted positions p, so
// a lane holds 32 columns of one position and a column tile (32 positions) lies in one group.  Scale and zero
// point then differ per value of an operand instead of per lane: the table p.szt holds them as register pairs
// per octet of columns; the workgroup copies the part of its tiles' groups and of its K range into LDS, and
// every operand reads its 32 bytes from there, one operand ahead of the arithmetic.  The weights are formed
// exactly as in the forward product.  The result's column p goes to channel out_map[p].
template <int BITS, int AT, int RW, int KW, int RING, int CT, bool TRANS = false>
__global__ __launch_bounds__(64 * RW * KW) void tiled_gemm_kernel(const TiledParams p)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rw = wave % RW, kw = wave / RW;
    const int n = lane & 31, h = lane >> 5;
    const int T0 = CT * blockIdx.x;
    const int split = blockIdx.y;
    const int rt0 = (blockIdx.z * RW + rw) * AT;
    const int S_begin = (split * KW + kw) * p.wave_steps;
    const int S_last = p.S_total - 1;
    const int lb_last = 2 * p.S_total - 1;

    // per-lane offsets that never change; the block number lives in scalar registers
    uint32_t tile_off[CT], col[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
        const int T = min(T0 + ct, p.T_total - 1);  // a missing tile repeats the last one; it is never stored
        tile_off[ct] = (uint32_t)T * (uint32_t)p.S_total;
        col[ct] = (uint32_t)(32 * T + n);
    }
    const uint32_t b_lane = tile_lane_bytes<BITS>((uint32_t)lane);
    const uint32_t a_lane = (uint32_t)rt0 * 1024u + (uint32_t)lane * 16u;
    const uint32_t a_frag_row = (uint32_t)p.rt_total * 1024u;  // bytes between consecutive (S, j)

    uint32_t w[RING][CT][BITS];
    uint32_t szr[RING][CT];
    h8 a[RING][4][AT];
    auto load_b = [&](int S, uint32_t (&wr)[CT][BITS], uint32_t (&sr)[CT]) {
        const int Sc = min(S, S_last);  // blocks past K repeat the last one (their x is zero)
        const uint32_t lb = (uint32_t)min(2 * S + h, lb_last);
        const uint32_t g = min(lb / (uint32_t)p.lb_per_group, (uint32_t)p.G - 1u);
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            tile_load<BITS>(p.qtile + ((size_t)(tile_off[ct] + (uint32_t)Sc) * (256u * BITS) + b_lane), wr[ct]);
            if constexpr (!TRANS) sr[ct] = p.sz[(size_t)g * p.N + col[ct]];
        }
    };
    auto load_a = [&](int S, int j, h8 (&ar)[AT]) {
        const char *src = p.xpack + (size_t)(4 * S + j) * a_frag_row + a_lane;
#pragma unroll
        for (int rt = 0; rt < AT; rt++) ar[rt] = __builtin_bit_cast(h8, *(const u4 *)(src + rt * 1024));
    };

    // Every workgroup starts its walk at another block of its waves' ranges and wraps around, so that the
    // workgroups, which all read the same A fragments, do not ask the same L2 channels at the same time.
    const int ws_n = p.wave_steps;
    int ahead = (int)((blockIdx.x + 3u * blockIdx.z) % (uint32_t)ws_n);  // block (inside the range) the next request is for
    auto next_block = [&]() {
        const int S = S_begin + ahead;
        ahead = ahead + 1 == ws_n ? 0 : ahead + 1;
        return S;
    };
    // prologue, in consumption order
    int S_of[RING];   // the block each ring slot holds (TRANS: its table entries are looked up by block)
#pragma unroll
    for (int u = 0; u < RING; u++) {
        const int S = next_block();
        S_of[u] = S;
        load_b(S, w[u], szr[u]);
#pragma unroll
        for (int j = 0; j < 4; j++) load_a(S, j, a[u][j]);
    }
    __builtin_amdgcn_sched_barrier(0);
    // TRANS: the (scale, base + zero) pairs of the workgroup's K range for the groups of its CT tiles -> LDS,
    // [ct][block of the range][octet][8 words]
    const int wg_blocks = KW * p.wave_steps;
    const int S_wg0 = split * wg_blocks;
    if constexpr (TRANS) {
        u4 *tbl = (u4 *)smem;
        for (int i = tid; i < CT * wg_blocks * 16; i += 64 * RW * KW) {
            const int ct = i / (wg_blocks * 16), r = i - ct * (wg_blocks * 16);
            const int Sc = min(S_wg0 + (r >> 4), S_last);   // (blocks past K repeat the last one: their x is zero)
            const int g = min(T0 + ct, p.T_total - 1) / p.tiles_per_group;
            tbl[i] = *(const u4 *)(p.szt + ((size_t)g * p.S_total + Sc) * 64 + (r & 15) * 4);
        }
        __syncthreads();
    }

    f16v acc[AT][CT];
#pragma unroll
    for (int rt = 0; rt < AT; rt++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[rt][ct][v] = 0.f;

    using Codec = TileCodec<BITS>;
    constexpr int KINDS = Codec::KINDS;
    uint32_t mg[KINDS];
    tile_magic<BITS>(mg);
    // (base + zero) per register kind: register r of an operand carries the bases of positions 2 r, 2 r + 1
    auto consts_of = [&](uint32_t e, h2 &s2, h2 (&zb)[KINDS]) {
        const h2 v = as_h2(e);
        s2 = (h2){v[0], v[0]};
        const h2 z2 = {v[1], v[1]};
#pragma unroll
        for (int k = 0; k < KINDS; k++)
            zb[k] = z2 + (h2){(_Float16)Codec::base(2 * k), (_Float16)Codec::base(2 * k + 1)};  // exact: small integers
    };

    // TRANS: the table entry of (block S, operand j, tile ct) for this lane's half
    u4 tq_s, tq_z;
    auto tbl_read = [&](int S, int j, int ct) {
        const uint32_t off = (uint32_t)(((ct * wg_blocks + (S - S_wg0)) * 8 + 4 * h + j) * 32);
        tq_s = *(const u4 *)(smem + off);
        tq_z = *(const u4 *)(smem + off + 16);
    };

    // the first operand of the walk
    h2 cs[CT], czb[CT][KINDS];  // (scale, base + zero) of the block being dequantised, per column tile
    h8 bop_next;
    if constexpr (TRANS) {
        tbl_read(S_of[0], 0, 0);
        bop_next = tiled_bop_t<BITS>(w[0][0], 0, tq_s, tq_z, mg);
        tbl_read(S_of[0], CT > 1 ? 0 : 1, CT > 1 ? 1 : 0);   // the entry of the operand after it
    } else {
        consts_of(szr[0][0], cs[0], czb[0]);
        bop_next = tiled_bop<BITS>(w[0][0], 0, cs[0], czb[0], mg);
    }

    // One block of the walk (ring slot u): the 4 CT (j, ct) operands, each multiplied with the AT row tiles
    // while the next operand of the walk is dequantised.  REFILL: the slot's registers are requested again
    // for the block a ring ahead as soon as their last reader is done.
    auto block = [&](auto u_c, auto refill_c) {
        constexpr int u = decltype(u_c)::value;
        constexpr bool REFILL = decltype(refill_c)::value;
        const int S_refill = REFILL ? next_block() : 0;  // the block a ring ahead of this one in the walk
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int ct = 0; ct < CT; ct++) {
                const h8 bop = bop_next;
                {
                    const int jn = ct == CT - 1 ? (j + 1) & 3 : j;
                    const int ctn = ct == CT - 1 ? 0 : ct + 1;
                    constexpr int u1 = (u + 1) % RING;
                    const bool wrap_u = ct == CT - 1 && j == 3;
                    if constexpr (TRANS) {
                        // tq_* hold the entry of the next operand; then the entry of the one after it is requested
                        bop_next = wrap_u ? tiled_bop_t<BITS>(w[u1][ctn], jn, tq_s, tq_z, mg)
                                          : tiled_bop_t<BITS>(w[u][ctn], jn, tq_s, tq_z, mg);
                        const int i2 = j * CT + ct + 2;
                        const bool wrap2 = i2 >= 4 * CT;
                        const int i2w = wrap2 ? i2 - 4 * CT : i2;
                        tbl_read(wrap2 ? S_of[u1] : S_of[u], i2w / CT, i2w % CT);
                    } else {
                        if (jn == 0) consts_of(wrap_u ? szr[u1][ctn] : szr[u][ctn], cs[ctn], czb[ctn]);  // first operand of a block
                        bop_next = wrap_u ? tiled_bop<BITS>(w[u1][ctn], jn, cs[ctn], czb[ctn], mg)
                                          : tiled_bop<BITS>(w[u][ctn], jn, cs[ctn], czb[ctn], mg);
                    }
                }
#pragma unroll
                for (int rt = 0; rt < AT; rt++) {
                    acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[u][j][rt], bop, acc[rt][ct], 0, 0, 0);
                }
                if (REFILL && ct == CT - 1) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (j == 3) {
                        load_b(S_refill, w[u], szr[u]);  // (its last reader, the last operand of the block, is done)
                        S_of[u] = S_refill;
                    }
                    load_a(S_refill, j, a[u][j]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    // whole turns of the ring, then what is left without refills (no load sits behind a branch, and the loop
    // has no early exit: an exit into its latch would make the compiler wait at the head of every turn for
    // almost every load in flight)
    const int full = p.wave_steps / RING * RING;
    for (int i0 = 0; i0 < full; i0 += RING) {
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (block(std::integral_constant<int, U>{}, std::true_type{}), ...);
        }(std::make_integer_sequence<int, RING>{});
    }
    {
        const int rem = p.wave_steps - full;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((U < RING - 1 && U < rem ? block(std::integral_constant<int, U>{}, std::false_type{}) : (void)0), ...);
        }(std::make_integer_sequence<int, RING>{});
    }

    // ---- the waves along K meet in LDS, EP row tiles at a time: [wave][tile rtp * CT + ct][v][lane] floats ----
    constexpr int EP = AT * CT <= 8 ? AT : 8 / CT;   // row tiles per pass (at most eight 4 KB tiles per wave in LDS)
    float *red = (float *)smem;
    const int m0 = 32 * AT * RW * blockIdx.z;
    const _Float16 *bias = (const _Float16 *)p.bias;
    _Float16 *y = (_Float16 *)p.y;
    constexpr int NT = 64 * RW * KW;
    if constexpr (TRANS) __syncthreads();   // the table shares this memory: every wave is done reading it
#pragma unroll
    for (int rp = 0; rp < AT; rp += EP) {
        if (rp > 0) __syncthreads();   // the previous pass has been read
        {
            float *dst = red + (size_t)wave * (EP * CT) * 1024 + lane;
#pragma unroll
            for (int rt = 0; rt < EP; rt++)
#pragma unroll
                for (int ct = 0; ct < CT; ct++)
#pragma unroll
                    for (int v = 0; v < 16; v++) dst[((rt * CT + ct) * 16 + v) * 64] = acc[rp + rt][ct][v];
        }
        __syncthreads();
        // one item = four adjacent columns of one row: element v of lane (n, h) of tile (rt, ct) of a wave in row
        // group rw is row 32 (AT rw + rt) + 8 (v / 4) + 4 h + v % 4, column 32 ct + n
#pragma unroll
        for (int it = 0; it < 32 * EP * RW * 8 * CT / NT; it++) {
            const int item = tid + NT * it;
            const int r = item / (8 * CT), c4 = (item % (8 * CT)) * 4;
            const int ct = c4 >> 5, nn = c4 & 31;
            const int rtw = r >> 5, rr = r & 31;          // 32-row tile of the pass
            const int rwi = rtw / EP, rt = rtw % EP;      // its row group and tile inside the wave's pass
            const int v = 4 * (rr >> 3) + (rr & 3), hh = (rr >> 2) & 1;
            const float *src = red + ((size_t)rwi * (EP * CT) + rt * CT + ct) * 1024 + v * 64 + hh * 32 + nn;
            f4 sum = *(const f4 *)src;
#pragma unroll
            for (int k = 1; k < KW; k++) sum += *(const f4 *)(src + (size_t)k * RW * (EP * CT) * 1024);
            const int row = m0 + 32 * (AT * rwi + rp + rt) + rr;
            const int T = T0 + ct;
            if (row < p.M && T < p.T_total) {
                const size_t o = (size_t)row * p.N + 32 * T + nn;
                if (TRANS && p.split_k == 1 && p.out_map) {
                    // (the reduce pass of a split applies the map itself)
                    const int4 dst = *(const int4 *)(p.out_map + 32 * T + nn);
                    const int d[4] = {dst.x, dst.y, dst.z, dst.w};
#pragma unroll
                    for (int c = 0; c < 4; c++) y[(size_t)row * p.N + min(max(d[c], 0), p.N - 1)] = (_Float16)sum[c];
                } else if (p.split_k == 1) {
                    if (bias) {
                        const h4 b4 = *(const h4 *)(bias + 32 * T + nn);
#pragma unroll
                        for (int c = 0; c < 4; c++) sum[c] += (float)b4[c];
                    }
                    h4 ov;
#pragma unroll
                    for (int c = 0; c < 4; c++) ov[c] = (_Float16)sum[c];
                    *(h4 *)(y + o) = ov;
                } else {
                    *(f4 *)(p.partial + (size_t)split * p.M * p.N + o) = sum;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// tiled_decode_kernel: M <= 4 rows of x on the tiled format.
//
// A workgroup owns ONE column tile (32 columns) and one K range; its KW waves split that range.  With one
// small workgroup per tile every CU gets work whatever N is (11008 columns: 344 workgroups of 4 waves,
// 4096 columns: 128 of 16), and what a wave keeps in flight (PF blocks of 1 KB / 768 B) adds up over the
// many waves of a CU.
// The dots run on v_mfma_f32_4x4x4_16B_f16: sixteen independent 4-lane blocks, lane 4 b + i supplies
// row i of A and column i of B of block b, and result register v of lane 4 b + j is row v of column j.
// A lane of the tiled format holds 32 codes of ONE column, so its unpacked registers are B operands as
// they are (four positions each), the A operand of row i is x[row i] at the same four positions (rows past
// M are zeros), and the four result registers of a lane are the rows of its own column: up to four rows of
// x cost one matrix instruction per four positions.  All 4-lane blocks of a half wave share their positions,
// and the instruction can broadcast the A operand of one block to the others (cbsz / abid): block b of the
// half keeps positions 4 b .. 4 b + 3 in its A registers and the instruction for positions 4 i .. 4 i + 3
// names block i, so x costs one 8-byte LDS read per lane and block.
// Per weight the vector ALU only unpacks (2, 3, 4 bits).
// The codes enter as (base + q) with the bases of the register unpack; per block of 32 positions the
// epilogue takes y += scale * (P - Bsum - zero * Xsum), with Xsum = sum x and Bsum = sum x * base of the
// block computed once per workgroup when x is staged.  Like GROUPED, and unlike the TILED matmul, this
// does not reproduce the fp16 rounding of each dequantised weight: products are exact, sums are fp32.
// 8-bit layers instead dequantise every weight in registers, as the matmul does (tiled_decode_exact), and add
// the products as they are.
// x reaches LDS in position order: a layer with an activation order scatters it through kinv (16-bit
// position per channel, one round trip; every workgroup walks all of x and keeps its K range).
// ---------------------------------------------------------------------------------------------------
struct DecodeParams {
    const _Float16 *x;      // [M, K]
    const uint16_t *kinv;   // [K] position of channel k, or nullptr (identity)
    const char *qtile;
    const uint32_t *sz;     // [G][N]
    const void *bias;
    void *y;                // fp16 [M, N]
    float *partial;         // [split_k][M][N] when split_k > 1
    int M, K, N, G;
    int S_total, T_total;
    int wave_steps;         // blocks (64 positions) per wave
    int split_k;
    int lb_per_group;       // group_size / 32
    uint32_t lbg_magic;     // lane block -> group: umulhi(lb, magic) + (add ? lb : 0)
    int lbg_add;
};

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

// E: blocks of 64 positions that share one epilogue (1, or 2 when the groups are multiples of 128 channels and
// every wave has an even number of blocks: both lane blocks of both blocks then lie in one group).
template <int BITS, int MR, int KW, int E>
__global__ __launch_bounds__(64 * KW) void tiled_decode_kernel(const DecodeParams p)
{
    static_assert(MR <= 4 && (E == 1 || E == 2), "one matrix instruction set per lane block");
    constexpr bool EXACT = tiled_decode_exact(BITS);
    constexpr int NT = 64 * KW;
    constexpr int PF = 2;              // blocks of weights per chunk; two chunks are in flight
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int T = blockIdx.x;
    const int split = blockIdx.y;
    const int wg_steps = p.wave_steps * KW;              // blocks of the workgroup's K range
    const int S_wg = split * wg_steps;                   // its first block
    const int S_begin = S_wg + wave * p.wave_steps;      // this wave's first block
    const int S_last = p.S_total - 1;
    const int span = wg_steps * 64;                      // positions the workgroup stages
    const int p0 = S_wg * 64;                            // its first position

    // LDS: x in position order [MR][span] fp16 | 64 zero bytes | block sums [span / 32][MR] (Xsum, Bsum) |
    //      (scale, zero) words of the range's groups [groups][32] | partial results [KW][MR][32]
    _Float16 *xl = (_Float16 *)smem;
    const uint32_t zero_off = (uint32_t)MR * (uint32_t)span * 2u;
    f2 *xs = (f2 *)(smem + zero_off + 64);
    const int lbs = span / 32;
    const uint32_t g_first = __umulhi((uint32_t)(2 * S_wg), p.lbg_magic) + (p.lbg_add ? (uint32_t)(2 * S_wg) : 0u);
    const uint32_t lb_end = (uint32_t)min(2 * (S_wg + wg_steps), 2 * p.S_total) - 1u;
    const uint32_t g_lastr = min(__umulhi(lb_end, p.lbg_magic) + (p.lbg_add ? lb_end : 0u), (uint32_t)p.G - 1u);
    const int n_groups = (int)(g_lastr - g_first) + 1;
    uint32_t *szl = (uint32_t *)(xs + (size_t)lbs * MR);
    float *red = (float *)(szl + (size_t)n_groups * 32);

    // ---- 1. x and the map first (a wait for them would also wait for every older load: vector loads return
    //         in order), then the first weights of this wave, then the (scale, zero) words ----------------
    // (without a map the channels of the range are the range itself)
    const int k8_lo = p.kinv ? 0 : p0 / 8, k8_hi = p.kinv ? p.K / 8 : min(p0 + span, p.K) / 8;
    constexpr int QP = 2;  // passes over x kept in registers
    u4 kq[QP];
    h8 xq[QP][MR];
#pragma unroll
    for (int ps = 0; ps < QP; ps++) {
        const int k = 8 * min(k8_lo + tid + ps * NT, k8_hi - 1);  // (clamped: the pass is skipped below when outside)
        kq[ps] = p.kinv ? *(const u4 *)(p.kinv + k) : (u4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int m = 0; m < MR; m++) xq[ps][m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
    }
    // the (scale, zero) words of the range's groups for this tile's 32 columns: SZP passes in registers
    constexpr int SZP = 4;
    uint32_t szq[SZP];
#pragma unroll
    for (int ps = 0; ps < SZP; ps++) {
        const int i = min(tid + ps * NT, n_groups * 32 - 1);
        szq[ps] = p.sz[(size_t)(g_first + (uint32_t)(i >> 5)) * p.N + 32 * T + (i & 31)];
    }
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t b_lane = tile_lane_bytes<BITS>((uint32_t)lane);
    const uint32_t tile_off = (uint32_t)T * (uint32_t)p.S_total;
    uint32_t w[2][PF][BITS];
    const int steps = min(p.wave_steps, max(p.S_total - S_begin, 0));  // blocks of this wave that lie inside K
    auto load_w = [&](int i, uint32_t (&wr)[BITS]) {
        // block i of the wave's range; past its end: its first block again (a cache hit that is never multiplied)
        const int Sc = min(S_begin + (i < steps ? i : 0), S_last);
        tile_load<BITS>(p.qtile + ((size_t)(tile_off + (uint32_t)Sc) * (256u * BITS) + b_lane), wr);
    };
    // two chunks of PF blocks are in flight from here on, through the staging of x as well
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(u, w[0][u]);
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(PF + u, w[1][u]);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. stage x in position order ------------------------------------------------------------------
    if (tid < 16) ((uint32_t *)(smem + zero_off))[tid] = 0u;
    {
        // positions of the range that lie past K (the padding of the last block) read as zeros
        const int tail0 = max(p.K - p0, 0);
        for (int i = tail0 + tid; i < span; i += NT)
#pragma unroll
            for (int m = 0; m < MR; m++) xl[m * span + i] = (_Float16)0;
    }
    auto scatter8 = [&](int k, const u4 &kv, const h8 (&xv)[MR]) {
        if (!p.kinv) {   // no activation order: the eight channels are eight consecutive positions, one store
            // (k8_lo .. k8_hi is the workgroup's own range here, a multiple of 8 away from p0)
#pragma unroll
            for (int m = 0; m < MR; m++) *(h8 *)(xl + m * span + (k - p0)) = xv[m];
            return;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int pos = (int)((kv[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            const int pl = pos - p0;
            if ((unsigned)pl < (unsigned)span) {
#pragma unroll
                for (int m = 0; m < MR; m++) xl[m * span + pl] = xv[m][e];
            }
        }
    };
#pragma unroll
    for (int ps = 0; ps < QP; ps++) {
        const int k8 = k8_lo + tid + ps * NT;
        if (k8 < k8_hi) scatter8(8 * k8, kq[ps], xq[ps]);
    }
    for (int k8 = k8_lo + tid + QP * NT; k8 < k8_hi; k8 += NT) {  // long layers: the rest, a pass at a time
        const int k = 8 * k8;
        u4 kv = {0u, 0u, 0u, 0u};
        if (p.kinv) kv = *(const u4 *)(p.kinv + k);
        h8 xv[MR];
#pragma unroll
        for (int m = 0; m < MR; m++) xv[m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
        scatter8(k, kv, xv);
    }
#pragma unroll
    for (int ps = 0; ps < SZP; ps++) {
        const int i = tid + ps * NT;
        if (i < n_groups * 32) szl[i] = szq[ps];
    }
    for (int i = tid + SZP * NT; i < n_groups * 32; i += NT) {  // more groups than the register passes hold
        szl[i] = p.sz[(size_t)(g_first + (uint32_t)(i >> 5)) * p.N + 32 * T + (i & 31)];
    }
    lds_barrier();
    // ---- 3. per epilogue unit (E blocks), half and row: Xsum = sum x, Bsum = sum x * base(position) over the
    //         unit's 32 E positions of that half; every wave for the units of its own slice (LDS serves one
    //         wave's accesses in order: no barrier needed).  Entry ((sb / E) * 2 + h) * MR + m, sb = the unit's
    //         first block inside the workgroup's range ------------------------------------------------------
    if constexpr (!EXACT) {
        // a lane sums 16 consecutive positions; a run of 32 positions (one half of one block) is two lanes,
        // a unit-half 2 E lanes: l, l + 1 (the other half of the run) and, E = 2, l + 4, l + 5 (the other block)
        const int sb0 = S_begin - S_wg;
        for (int q0 = 0; q0 < 4 * p.wave_steps; q0 += 64) {   // 16-position pieces of the wave's range
            const int piece = q0 + lane;
            const int sb = sb0 + (piece >> 2), hh = (piece >> 1) & 1;
            const bool live = piece < 4 * p.wave_steps;
#pragma unroll
            for (int m = 0; m < MR; m++) {
                float X = 0.f, B = 0.f;
                if (live && m < p.M) {
                    const h8 *src = (const h8 *)(xl + m * span + 64 * sb0 + 16 * piece);
#pragma unroll
                    for (int v = 0; v < 2; v++) {
                        const h8 q = src[v];
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            const float xf = (float)q[e];
                            X += xf;
                            B += xf * TileCodec<BITS>::base(e);
                        }
                    }
                }
                // lane l takes l + 1 (and, E = 2, l + 4 and l + 5): the lanes that store (l % 8 in {0, 2}) stay
                // inside their row of 16, so a row shift in the data path does (no LDS round trip)
                X += row_shl<1>(X);
                B += row_shl<1>(B);
                if constexpr (E == 2) {
                    X += row_shl<4>(X);
                    B += row_shl<4>(B);
                }
                if (live && (lane & (E == 2 ? 5 : 1)) == 0) xs[((sb / E) * 2 + hh) * MR + m] = (f2){X, B};
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    // ---- 4. the walk ----------------------------------------------------------------------------------
    uint32_t mg[TileCodec<BITS>::KINDS];
    tile_magic<BITS>(mg);
    const int row_i = lane & 3;  // the row of x this lane supplies to its 4-lane block
    float ysum[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) ysum[m] = 0.f;
    // Per-lane byte offsets that never change; what changes per block is wave-uniform and stays in scalar
    // registers.  A lane whose row lies past M reads the 64 zero bytes whatever the block (stride 0).
    // The matrix instruction broadcasts A: with cbsz = 3 the eight 4-lane blocks of a half wave all take their A
    // operand from block `abid` of the half.  So lane block b of a half holds only positions 4 b .. 4 b + 3 of the
    // half's 32 (one 8-byte read per lane and block instead of 64 bytes), and the instruction for positions
    // 4 i .. 4 i + 3 names abid = i.
    const int lb8 = (lane >> 2) & 7;
    const uint32_t x_base = row_i < p.M ? (uint32_t)(row_i * span + 32 * h + 4 * lb8) * 2u : zero_off;
    const uint32_t x_stride = row_i < p.M ? 128u : 0u;
    const uint32_t xs_lane = zero_off + 64u + (uint32_t)(h * MR) * 8u;   // sums of half h of unit 0
    const uint32_t sz_lane = (uint32_t)((const unsigned char *)szl - smem) + (uint32_t)n * 4u;

    // x of a block: this lane's four positions of row row_i; read one block ahead of its use
    auto load_x = [&](uint32_t sb, u2 &xv) { xv = *(const u2 *)(smem + x_base + x_stride * sb); };
    f4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};  // two chains: a matrix instruction waits for the one it adds to
    uint32_t szw = 0u;   // (scale, zero) word and sums of the unit in flight, read when the unit starts
    f2 xsv[MR];
    auto block = [&](auto uu_c, int S, const uint32_t (&wr)[BITS], const u2 &xc, u2 &xn) {
        constexpr int uu = decltype(uu_c)::value;                 // block inside its unit
        const uint32_t sb = (uint32_t)(S - S_wg);                  // block inside the workgroup's range (wave-uniform)
        if constexpr (uu == 0) {
            // group of the unit's lane blocks (E = 1: the two halves of the wave may differ)
            const uint32_t l0 = 2u * (uint32_t)S;
            const uint32_t g0 = min(__umulhi(l0, p.lbg_magic) + (p.lbg_add ? l0 : 0u), (uint32_t)p.G - 1u) - g_first;
            uint32_t goff = g0 * 128u;
            if constexpr (E == 1) {
                const uint32_t l1 = l0 + 1u;
                const uint32_t g1 = min(__umulhi(l1, p.lbg_magic) + (p.lbg_add ? l1 : 0u), (uint32_t)p.G - 1u) - g_first;
                goff = (h ? g1 : g0) * 128u;
            }
            szw = *(const uint32_t *)(smem + sz_lane + goff);
            if constexpr (!EXACT) {
                const f2 *xb = (const f2 *)(smem + xs_lane + (sb / E) * (uint32_t)(2 * MR * 8));
#pragma unroll
                for (int m = 0; m < MR; m++) xsv[m] = xb[m];
            }
        }
        load_x(sb + 1u, xn);
        // unpack: sixteen registers, positions (2 r, 2 r + 1) of the lane in register r
        u4 q[4];
#pragma unroll
        for (int j = 0; j < 4; j++) TileCodec<BITS>::operand(wr, j, q[j], mg);
        if constexpr (EXACT) tiled_dequant_exact<BITS>(q, szw);
        if constexpr (uu == 0) {
            c0 = (f4){0.f, 0.f, 0.f, 0.f};
            c1 = (f4){0.f, 0.f, 0.f, 0.f};
        }
        const h4 xa = __builtin_bit_cast(h4, xc);
        [&]<int... V>(std::integer_sequence<int, V...>) {
            ((c0 = __builtin_amdgcn_mfma_f32_4x4x4f16(xa, __builtin_bit_cast(h4, (u2){q[V][0], q[V][1]}), c0, 3, 2 * V, 0),
              c1 = __builtin_amdgcn_mfma_f32_4x4x4f16(xa, __builtin_bit_cast(h4, (u2){q[V][2], q[V][3]}), c1, 3, 2 * V + 1, 0)),
             ...);
        }(std::make_integer_sequence<int, 4>{});
        if constexpr (uu == E - 1) {
            if constexpr (EXACT) {
#pragma unroll
                for (int m = 0; m < MR; m++) ysum[m] += c0[m] + c1[m];
            } else {
                const h2 e = as_h2(szw);
                const float sc = (float)e[0], zp = (float)e[1];
#pragma unroll
                for (int m = 0; m < MR; m++) ysum[m] += sc * (((c0[m] + c1[m]) - xsv[m][1]) - zp * xsv[m][0]);
            }
        }
    };

    // Chunks of PF blocks, two in flight; x rides one block ahead in two register sets.  Blocks past the end
    // of K inside a wave's range are harmless (their x and sums are zeros), blocks past the range are skipped.
    u2 xr[2];
    load_x((uint32_t)(S_begin - S_wg), xr[0]);
    auto chunk = [&](int c, uint32_t (&wc)[PF][BITS], auto all_c) {
        constexpr bool ALL = decltype(all_c)::value;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((ALL || c + U < p.wave_steps
                  ? block(std::integral_constant<int, U % E>{}, S_begin + c + U, wc[U], xr[U & 1], xr[(U + 1) & 1])
                  : (void)0),
             ...);
        }(std::make_integer_sequence<int, PF>{});
    };
    int c = 0;
    for (; c + 2 * PF <= p.wave_steps; c += 2 * PF) {
        chunk(c, w[0], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(c + 2 * PF + u, w[0][u]);  // the chunk after the one in flight
        __builtin_amdgcn_sched_barrier(0);
        chunk(c + PF, w[1], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(c + 3 * PF + u, w[1][u]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (c < p.wave_steps) {   // what is left of the range: fewer than two chunks, nothing more to request
        chunk(c, w[0], std::false_type{});
        chunk(c + PF, w[1], std::false_type{});
    }

    // ---- 5. the two halves of a column (lanes n and n + 32), then the waves along K ---------------------
#pragma unroll
    for (int m = 0; m < MR; m++) ysum[m] += __shfl_xor(ysum[m], 32);
    if (h == 0) {
#pragma unroll
        for (int m = 0; m < MR; m++) red[(wave * MR + m) * 32 + n] = ysum[m];
    }
    lds_barrier();
    if (tid < MR * 32) {
        const int m = tid >> 5, nn = tid & 31;
        if (m < p.M) {
            float sum = 0.f;
            for (int k = 0; k < KW; k++) sum += red[(k * MR + m) * 32 + nn];
            const size_t o = (size_t)m * p.N + 32 * T + nn;
            if (p.split_k == 1) {
                if (p.bias) sum += (float)((const _Float16 *)p.bias)[32 * T + nn];
                ((_Float16 *)p.y)[o] = (_Float16)sum;
            } else {
                p.partial[(size_t)split * p.M * p.N + o] = sum;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// tiled_decode16_kernel: the decode product with ONE workgroup per CU.  The unit of work is 16 columns (half a
// column tile) over all of K; workgroup b of `nwg` takes units [units * b / nwg, units * (b + 1) / nwg), so the
// CUs differ by at most one unit (11008 columns: 688 units, two or three per CU; with one 32-column tile per
// workgroup 88 CUs hold two tiles while 168 hold one).  x is staged once per workgroup for all its units.
//
// A wave reads 16 columns as "virtual blocks" of 128 positions: lane (n = lane % 16, q = lane / 16) takes
// lane (n + 16 c) + 32 (q % 2) of real block 2 V + q / 2 of the tile, i.e. its 32 codes of column
// 32 T + 16 c + n at positions 128 V + 32 q .. + 31 (two 256-byte runs per real block).  Everything per lane
// is as in tiled_decode_kernel: the unpacked registers are B operands of v_mfma_f32_4x4x4_16B_f16, four
// consecutive lanes share their positions, and the epilogue takes scale * (P - Bsum - zero * Xsum) per
// 32 positions.  The workgroup's (unit, virtual block) pairs are dealt out to the sixteen waves as contiguous
// ranges; a wave leaves its partial results per unit in LDS, where all meet at the end.
// G128: groups are multiples of 128 channels, so a virtual block lies in one group (scalar group index).
// ---------------------------------------------------------------------------------------------------
struct Decode16Params {
    const _Float16 *x;      // [M, K]
    const uint16_t *kinv;   // [K] position of channel k, or nullptr (identity)
    const char *qtile;
    const uint32_t *sz;     // [G][N]
    const void *bias;
    void *y;                // fp16 [M, N]
    int M, K, N, G;
    int S_total, T_total;   // blocks of 64 positions, tiles of 32 columns
    int V_total;            // virtual blocks of 128 positions
    int units;              // N / 16
    int lb_per_group;       // group_size / 32
    uint32_t lbg_magic;     // lane block (32 positions) -> group: umulhi(lb, magic) + (add ? lb : 0)
    int lbg_add;
};

template <int BITS, int MR, bool G128, bool CONTIG>
__global__ __launch_bounds__(1024) void tiled_decode16_kernel(const Decode16Params p)
{
    static_assert(MR <= 4, "one matrix instruction set per lane block");
    constexpr bool EXACT = tiled_decode_exact(BITS);
    constexpr int NT = 1024, NW = 16;
    constexpr int PF = 2;               // items of weights per chunk; two chunks are in flight
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n16 = lane & 15, lbv = lane >> 4;
    const int u0 = (int)(((long long)p.units * blockIdx.x) / gridDim.x);
    const int u1 = (int)(((long long)p.units * (blockIdx.x + 1)) / gridDim.x);
    const int n_units = u1 - u0;
    const int span = p.V_total * 128;   // positions staged: all of K, padded to whole virtual blocks
    const int S_last = p.S_total - 1;

    // LDS: x in position order [MR][span] fp16 | 64 zero bytes | sums [span / 32][MR] (Xsum, Bsum) |
    //      (scale, zero) as floats [n_units][G][16] | partial results [n_units][NW][MR][64]
    _Float16 *xl = (_Float16 *)smem;
    const uint32_t zero_off = (uint32_t)MR * (uint32_t)span * 2u;
    f2 *xs = (f2 *)(smem + zero_off + 64);
    f2 *szl = xs + (size_t)(span / 32) * MR;
    float *red = (float *)(szl + (size_t)n_units * p.G * 16);

    // ---- 1. requests: x and the map first (loads return in order), the (scale, zero) words, the weights ----
    const int k8_hi = p.K / 8;
    u4 kq;
    h8 xq[MR];
    {
        const int k = 8 * min(tid, k8_hi - 1);
        kq = p.kinv ? *(const u4 *)(p.kinv + k) : (u4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int m = 0; m < MR; m++) xq[m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
    }
    constexpr int SZP = 2;
    const int sz_words = n_units * p.G * 16;
    uint32_t szq[SZP];
    auto sz_src = [&](int i) {   // word i of the table: unit i / (16 G), group (i / 16) % G, column i % 16
        const int ul = i / (16 * p.G), r = i - ul * 16 * p.G;
        return p.sz + (size_t)(r >> 4) * p.N + 16 * (u0 + ul) + (r & 15);
    };
#pragma unroll
    for (int ps = 0; ps < SZP; ps++) szq[ps] = *sz_src(min(tid + ps * NT, sz_words - 1));
    __builtin_amdgcn_sched_barrier(0);

    // items of the workgroup: (unit, virtual block) pairs, unit after unit.
    // CONTIG: wave w takes the contiguous range [I w / 16, I (w + 1) / 16) of them: consecutive virtual blocks of
    // one unit, with a change of unit once or twice per wave.  Otherwise the waves stride over the virtual blocks
    // of every unit (V = wave, wave + 16, ...), which changes unit after every K / 2048 items: measured 0.2 us
    // ahead for one unit of 32 virtual blocks (4096 x 4096), 0.4 us behind for 86 (11008 x 4096).
    const int items_all = n_units * p.V_total;
    const int i0 = CONTIG ? (int)(((long long)items_all * wave) / NW) : 0;
    const int vpu = (p.V_total - wave + NW - 1) / NW;   // strided: per unit (may be 0 for the last waves of a short K)
    const int n_items = CONTIG ? (int)(((long long)items_all * (wave + 1)) / NW) - i0 : n_units * vpu;
    // lane offset inside a virtual block: its lane of the real block, and the second real block for q >= 2
    // (a last, odd virtual block has no second real block: those lanes repeat the first; their x is zero)
    const uint32_t b_lane = tile_lane_bytes<BITS>((uint32_t)(n16 + 32 * (lbv & 1)));
    const uint32_t b_lane2 = b_lane + (uint32_t)(lbv >> 1) * (256u * BITS);
    // cursors: (unit, V) of the next item to request and of the next item to compute
    const int first_u = CONTIG ? min(i0 / p.V_total, n_units - 1) : 0;
    const int first_v = CONTIG ? (n_items > 0 ? i0 % p.V_total : 0) : min(wave, p.V_total - 1);
    int rq_u = first_u, rq_v = first_v, rq_left = n_items;
    auto unit_base = [&](int ul) {   // the first block of a unit's 16 columns (wave-uniform)
        const int unit = u0 + ul;
        return p.qtile + ((size_t)((uint32_t)(unit >> 1) * (uint32_t)p.S_total) * (256u * BITS) +
                          tile_lane_bytes<BITS>(16u * (uint32_t)(unit & 1)));
    };
    const char *rq_ptr = unit_base(rq_u) + (size_t)rq_v * (512u * BITS);
    uint32_t w[2][PF][BITS];
    auto load_w = [&](uint32_t (&wr)[BITS]) {
        tile_load<BITS>(rq_ptr + (2 * rq_v + 1 <= S_last ? b_lane2 : b_lane), wr);
        // past the wave's items: its last item again (a cache hit that is never multiplied)
        if (rq_left > 1) {
            rq_left--;
            if constexpr (CONTIG) {
                rq_v++;
                rq_ptr += 512u * BITS;
                if (rq_v == p.V_total) {
                    rq_v = 0;
                    rq_u++;
                    rq_ptr = unit_base(rq_u);
                }
            } else {
                rq_v += NW;
                rq_ptr += (size_t)NW * (512u * BITS);
                if (rq_v >= p.V_total) {
                    rq_v = wave;
                    rq_u++;
                    rq_ptr = unit_base(rq_u) + (size_t)wave * (512u * BITS);
                }
            }
        }
    };
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(w[0][u]);
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(w[1][u]);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. stage x in position order, and the (scale, zero) words ------------------------------------------
    if (tid < 16) ((uint32_t *)(smem + zero_off))[tid] = 0u;
    for (int i = p.K + tid; i < span; i += NT)   // the padding of the last virtual block reads as zeros
#pragma unroll
        for (int m = 0; m < MR; m++) xl[m * span + i] = (_Float16)0;
    auto scatter8 = [&](int k, const u4 &kv, const h8 (&xv)[MR]) {
        if (!p.kinv) {   // no activation order: the eight channels are eight consecutive positions, one store
#pragma unroll
            for (int m = 0; m < MR; m++) *(h8 *)(xl + m * span + k) = xv[m];
            return;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int pos = min((int)((kv[e >> 1] >> (16 * (e & 1))) & 0xffffu), span - 1);
#pragma unroll
            for (int m = 0; m < MR; m++) xl[m * span + pos] = xv[m][e];
        }
    };
    if (tid < k8_hi) scatter8(8 * tid, kq, xq);
    for (int k8 = tid + NT; k8 < k8_hi; k8 += NT) {   // long layers: the rest, a pass at a time
        const int k = 8 * k8;
        u4 kv = {0u, 0u, 0u, 0u};
        if (p.kinv) kv = *(const u4 *)(p.kinv + k);
        h8 xv[MR];
#pragma unroll
        for (int m = 0; m < MR; m++) xv[m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
        scatter8(k, kv, xv);
    }
#pragma unroll
    for (int ps = 0; ps < SZP; ps++) {
        const int i = tid + ps * NT;
        if (i < sz_words) {
            const h2 e = as_h2(szq[ps]);
            szl[i] = (f2){(float)e[0], (float)e[1]};
        }
    }
    for (int i = tid + SZP * NT; i < sz_words; i += NT) {
        const h2 e = as_h2(*sz_src(i));
        szl[i] = (f2){(float)e[0], (float)e[1]};
    }
    // CONTIG: a wave writes the partial results of the units it walks: the others read as zeros
    if constexpr (CONTIG)
        for (int i = tid; i < n_units * NW * MR * 64; i += NT) red[i] = 0.f;
    lds_barrier();
    // ---- 3. per 32 positions and row: Xsum = sum x, Bsum = sum x * base(position).  A thread sums 16
    //         positions, the lane next to it the other half of the run -------------------------------------
    for (int q0 = 0; !EXACT && q0 < span / 16; q0 += NT) {
        const int piece = q0 + tid;
        const bool live = piece < span / 16;
#pragma unroll
        for (int m = 0; m < MR; m++) {
            float X = 0.f, B = 0.f;
            if (live && m < p.M) {
                const h8 *src = (const h8 *)(xl + m * span + 16 * piece);
#pragma unroll
                for (int v = 0; v < 2; v++) {
                    const h8 q = src[v];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const float xf = (float)q[e];
                        X += xf;
                        B += xf * TileCodec<BITS>::base(e);
                    }
                }
            }
            X += row_shl<1>(X);
            B += row_shl<1>(B);
            if (live && (lane & 1) == 0) xs[(piece >> 1) * MR + m] = (f2){X, B};
        }
    }
    lds_barrier();

    // ---- 4. the walk ----------------------------------------------------------------------------------
    uint32_t mg[TileCodec<BITS>::KINDS];
    tile_magic<BITS>(mg);
    const int row_i = lane & 3;  // the row of x this lane supplies to its 4-lane block
    float ysum[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) ysum[m] = 0.f;
    // per-lane byte offsets that never change; a lane whose row lies past M reads the 64 zero bytes (stride 0).
    // A is broadcast inside each group of four 4-lane blocks (cbsz = 2), the sixteen lanes that share their 32
    // positions: block b of a group holds positions 4 b .. 4 b + 3 and 16 + 4 b .. 16 + 4 b + 3 (two 8-byte reads
    // per lane and item), and the instruction for positions 4 i .. 4 i + 3 takes register set i / 4 with abid = i % 4.
    const int lb4 = (lane >> 2) & 3;
    const uint32_t x_base = row_i < p.M ? (uint32_t)(row_i * span + 32 * lbv + 4 * lb4) * 2u : zero_off;
    const uint32_t x_stride = row_i < p.M ? 256u : 0u;
    const uint32_t x_second = row_i < p.M ? 32u : 0u;   // bytes to positions 16 ..
    const uint32_t xs_lane = zero_off + 64u + (uint32_t)(lbv * MR) * 8u;
    const uint32_t sz_lane = (uint32_t)((const unsigned char *)szl - smem) + (uint32_t)n16 * 8u;
    const uint32_t red_lane = (uint32_t)((const unsigned char *)red - smem) + (uint32_t)lane * 4u;

    auto load_x = [&](int V, u2 (&xv)[2]) {
        const uint32_t xoff = x_base + x_stride * (uint32_t)V;
        xv[0] = *(const u2 *)(smem + xoff);
        xv[1] = *(const u2 *)(smem + xoff + x_second);
    };
    int cu = first_u, cv = first_v, c_left = n_items;   // (unit, V) of the item being computed, items still to compute
    auto item = [&](const uint32_t (&wr)[BITS], const u2 (&xc)[2], u2 (&xn)[2]) {
        const int V = cv, ul = cu;
        // this item's scale, zero point and sums
        uint32_t goff;
        if constexpr (G128) {
            const uint32_t lb = 4u * (uint32_t)V;
            goff = min(__umulhi(lb, p.lbg_magic) + (p.lbg_add ? lb : 0u), (uint32_t)p.G - 1u) * 128u;
        } else {
            const uint32_t lb = 4u * (uint32_t)V + (uint32_t)lbv;
            goff = min(__umulhi(lb, p.lbg_magic) + (p.lbg_add ? lb : 0u), (uint32_t)p.G - 1u) * 128u;
        }
        const f2 szf = *(const f2 *)(smem + sz_lane + (uint32_t)ul * (uint32_t)p.G * 128u + goff);
        f2 xsv[MR];
        if constexpr (!EXACT) {
            const f2 *xb = (const f2 *)(smem + xs_lane + (uint32_t)V * (uint32_t)(4 * MR * 8));
#pragma unroll
            for (int m = 0; m < MR; m++) xsv[m] = xb[m];
        }
        // advance to the next item and read its x
        c_left--;
        cv += CONTIG ? 1 : NW;
        const bool unit_done = cv >= p.V_total || c_left == 0;   // the wave's share of this unit ends here
        if (cv >= p.V_total) {
            cv = CONTIG ? 0 : wave;
            cu++;
        }
        load_x(cv, xn);
        u4 q[4];
#pragma unroll
        for (int j = 0; j < 4; j++) TileCodec<BITS>::operand(wr, j, q[j], mg);
        if constexpr (EXACT) {   // (both floats came from fp16 values: the conversions back are exact)
            const h2 e = {(_Float16)szf[0], (_Float16)szf[1]};
            tiled_dequant_exact<BITS>(q, as_u32(e));
        }
        f4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};  // two chains
        const h4 xa[2] = {__builtin_bit_cast(h4, xc[0]), __builtin_bit_cast(h4, xc[1])};
        [&]<int... V>(std::integer_sequence<int, V...>) {
            ((c0 = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[V / 2], __builtin_bit_cast(h4, (u2){q[V][0], q[V][1]}), c0, 2, (2 * V) % 4, 0),
              c1 = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[V / 2], __builtin_bit_cast(h4, (u2){q[V][2], q[V][3]}), c1, 2, (2 * V + 1) % 4, 0)),
             ...);
        }(std::make_integer_sequence<int, 4>{});
        if constexpr (EXACT) {
#pragma unroll
            for (int m = 0; m < MR; m++) ysum[m] += c0[m] + c1[m];
        } else {
            const float sc = szf[0], zp = szf[1];
#pragma unroll
            for (int m = 0; m < MR; m++) ysum[m] += sc * (((c0[m] + c1[m]) - xsv[m][1]) - zp * xsv[m][0]);
        }
        if (unit_done) {   // (wave-uniform) the wave's share of this unit is complete
#pragma unroll
            for (int m = 0; m < MR; m++) {
                *(float *)(smem + red_lane + (uint32_t)((ul * NW + wave) * MR + m) * 256u) = ysum[m];
                ysum[m] = 0.f;
            }
        }
    };
    u2 xr[2][2];
    load_x(cv, xr[0]);
    auto chunk = [&](int c, uint32_t (&wc)[PF][BITS], auto all_c) {
        constexpr bool ALL = decltype(all_c)::value;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((ALL || c + U < n_items ? item(wc[U], xr[U & 1], xr[(U + 1) & 1]) : (void)0), ...);
        }(std::make_integer_sequence<int, PF>{});
    };
    int c = 0;
    for (; c + 2 * PF <= n_items; c += 2 * PF) {
        chunk(c, w[0], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(w[0][u]);
        __builtin_amdgcn_sched_barrier(0);
        chunk(c + PF, w[1], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(w[1][u]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (c < n_items) {
        chunk(c, w[0], std::false_type{});
        chunk(c + PF, w[1], std::false_type{});
    }
    if (!CONTIG && vpu == 0) {   // strided: a wave without virtual blocks (K shorter than sixteen of them) adds zeros
        for (int ul = 0; ul < n_units; ul++)
#pragma unroll
            for (int m = 0; m < MR; m++) *(float *)(smem + red_lane + (uint32_t)((ul * NW + wave) * MR + m) * 256u) = 0.f;
    }
    lds_barrier();

    // ---- 5. per (unit, row, column): the sixteen waves and the four lane blocks of each ------------------
    // thread = (output o = tid / 16, wave part = tid % 16): four values, then the sixteen lanes of a row
    for (int o0 = 0; o0 < n_units * MR * 16; o0 += NT / 16) {
        const int o = o0 + (tid >> 4), part = tid & 15;
        const bool live = o < n_units * MR * 16;
        const int ul = o / (MR * 16), r = o - ul * MR * 16, m = r >> 4, nn = r & 15;
        float sum = 0.f;
        if (live) {
            const float *src = red + ((size_t)(ul * NW + part) * MR + m) * 64 + nn;
            sum = (src[0] + src[16]) + (src[32] + src[48]);
        }
        sum += row_shl<8>(sum);
        sum += row_shl<4>(sum);
        sum += row_shl<2>(sum);
        sum += row_shl<1>(sum);
        if (live && part == 0 && m < p.M) {
            const int col = 16 * (u0 + ul) + nn;
            if (p.bias) sum += (float)((const _Float16 *)p.bias)[col];
            ((_Float16 *)p.y)[(size_t)m * p.N + col] = (_Float16)sum;
        }
    }
}

// y = fp16(sum over split of partial[split] (+ bias)), four columns per thread, in split order.
__global__ __launch_bounds__(256) void tiled_reduce_kernel(const float *__restrict__ partial, const _Float16 *bias,
                                                           _Float16 *__restrict__ y, int M, int N, int split_k,
                                                           const int32_t *__restrict__ out_map = nullptr)
{
    const uint32_t q = blockIdx.x * 256u + threadIdx.x;
    const uint32_t nq = (uint32_t)N / 4u;
    if (q >= (uint32_t)M * nq) return;
    const uint32_t row = q / nq;
    const uint32_t c = 4u * (q - row * nq);
    f4 sum = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
        const h4 b4 = *(const h4 *)(bias + c);
        sum = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    for (int s = 0; s < split_k; s++) sum += *(const f4 *)(partial + ((size_t)s * M + row) * N + c);
    if (out_map) {   // the transposed product: column c is a sorted position, its channel is out_map[c]
        const int4 dst = *(const int4 *)(out_map + c);
        const int d[4] = {dst.x, dst.y, dst.z, dst.w};
#pragma unroll
        for (int e = 0; e < 4; e++) y[(size_t)row * N + min(max(d[e], 0), N - 1)] = (_Float16)sum[e];
        return;
    }
    h4 o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = (_Float16)sum[e];
    *(h4 *)(y + (size_t)row * N + c) = o;
}

template <int BITS, int AT, int RW, int KW, int RING, int CT>
static int launch_tiled_one(const TiledParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = tiled_gemm_kernel<BITS, AT, RW, KW, RING, CT>;
    const int lds_bytes = tiled_lds_bytes(AT * RW, KW);
    if (plan.lds_bytes < lds_bytes || plan.waves_k != KW || plan.block != 64 * RW * KW) return GPTQ_HIP_ERR_BAD_ARG;
    if (lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, plan.grid_z), dim3(64 * RW * KW), lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// x is packed into the workspace, the matmul runs, and a reduce pass follows when K is split over workgroups.
int launch_tiled(const void *x, const void *qtile, const uint32_t *sz, const int32_t *xsrc, const void *bias, void *y,
                 char *xpack, float *partial, int M, int K, int N, int G, int bits, int group_size,
                 const gptq_hip_plan &plan, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const int Kp = (K + 63) / 64 * 64;
    TiledParams p;
    p.xpack = xpack;
    p.qtile = (const char *)qtile;
    p.sz = sz;
    p.bias = bias;
    p.y = y;
    p.partial = partial;
    p.M = M;
    p.N = N;
    p.G = G;
    p.S_total = Kp / 64;
    p.T_total = N / 32;
    p.wave_steps = plan.k_chunk;
    p.rt_total = plan.row_tiles * plan.m_blocks;
    p.split_k = plan.split_k;
    p.lb_per_group = group_size / 32;
    p.szt = nullptr;
    p.out_map = nullptr;
    p.tiles_per_group = 1;
    const int S_pack = tiled_pack_blocks(plan.split_k, plan.waves_k, plan.k_chunk);
    const int pack_lds = xsrc ? K * 2 : 0;  // one row of x
    if (pack_lds > 65536) {
        if (hipFuncSetAttribute((const void *)tile_pack_x_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, pack_lds) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(tile_pack_x_kernel, dim3(32 * p.rt_total), dim3(256), pack_lds, stream, (const _Float16 *)x, xsrc,
                       xpack, M, K, Kp, p.rt_total, S_pack);
    if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
#define GPTQ_TILED_CASE(B, A)                                                                  \
    if (bits == B && plan.row_tiles == A && plan.waves_n == 1)                                 \
        rc = launch_tiled_one<B, A, 1, 4, tiled_ring(A), 2>(p, plan, stream)
    GPTQ_TILED_CASE(4, 1);
    GPTQ_TILED_CASE(4, 2);
    GPTQ_TILED_CASE(4, 4);
    GPTQ_TILED_CASE(3, 1);
    GPTQ_TILED_CASE(3, 2);
    GPTQ_TILED_CASE(3, 4);
    GPTQ_TILED_CASE(2, 1);
    GPTQ_TILED_CASE(2, 2);
    GPTQ_TILED_CASE(2, 4);
    GPTQ_TILED_CASE(8, 1);
    GPTQ_TILED_CASE(8, 2);
    GPTQ_TILED_CASE(8, 4);
#undef GPTQ_TILED_CASE
    // 128 x 128 per wave (waves_n = 2): a ring of two blocks
    if (plan.row_tiles == 4 && plan.waves_n == 2) {
        switch (bits) {
            case 2: rc = launch_tiled_one<2, 4, 1, 4, 2, 4>(p, plan, stream); break;
            case 3: rc = launch_tiled_one<3, 4, 1, 4, 2, 4>(p, plan, stream); break;
            case 4: rc = launch_tiled_one<4, 4, 1, 4, 2, 4>(p, plan, stream); break;
            case 8: rc = launch_tiled_one<8, 4, 1, 4, 2, 4>(p, plan, stream); break;
            default: break;
        }
    }
    if (rc != GPTQ_HIP_OK) return rc;
    if (plan.split_k > 1) {
        const uint32_t quads = (uint32_t)M * ((uint32_t)N / 4u);
        hipLaunchKernelGGL(tiled_reduce_kernel, dim3((quads + 255u) / 256u), dim3(256), 0, stream, partial,
                           (const _Float16 *)bias, (_Float16 *)y, M, N, plan.split_k);
        if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    }
    return GPTQ_HIP_OK;
}


// ---------------------------------------------------------------------------------------------------
// The transposed product gx[M, K] = gy[M, N] @ W^T.
// Preparation: the tiled format of the transposed code matrix (a lane holds, for sorted position
// p = 32 T + lane % 32, the codes of columns 64 S + 32 (lane / 32) .. + 31; columns past N are zeros), and the table
// of (scale, base + zero) register pairs per group and octet of columns.
// ---------------------------------------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(256) void tile_retile_t_kernel(const uint32_t *__restrict__ qweight,
                                                            const int32_t *__restrict__ xsrc, uint32_t *__restrict__ qtile,
                                                            int K, int N, int S_total, int T_total)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const int lane = t & 63;
    const uint32_t blk = t >> 6;  // T * S_total + S
    if (blk >= (uint32_t)T_total * (uint32_t)S_total) return;
    const int T = blk / S_total, S = blk - T * S_total;
    const int pos = 32 * T + (lane & 31), h = lane >> 5;
    int src = xsrc ? xsrc[pos] : pos;
    src = min(max(src, 0), K - 1);   // a bad map must not fault
    const uint32_t *b = qweight + (size_t)(src >> 5) * BITS * N;   // the packed block of 32 channels
    const int bit = BITS * (src & 31);
    const int wd = bit >> 5, sh = bit & 31;
    uint32_t words[BITS];
#pragma unroll
    for (int i = 0; i < BITS; i++) words[i] = 0u;
    for (int s = 0; s < 32; s++) {
        const int n = 64 * S + 32 * h + s;
        uint32_t q = 0u;
        if (n < N) {
            q = b[(size_t)wd * N + n] >> sh;
            if (sh + BITS > 32) q |= b[(size_t)(wd + 1) * N + n] << (32 - sh);
            q &= (1u << BITS) - 1u;
        }
        const int obit = BITS * TileCodec<BITS>::field(s);
        const int owd = obit >> 5, osh = obit & 31;
        words[owd] |= q << osh;
        if (osh + BITS > 32) words[owd + 1] |= q >> (32 - osh);
    }
#pragma unroll
    for (int i = 0; i < BITS; i++) {
        const int at = BITS == 8 ? (i >> 2) * 256 + lane * 4 + (i & 3) : lane * BITS + i;
        qtile[(size_t)blk * (64 * BITS) + at] = words[i];
    }
}

// szt[g][o] for octet o of columns (8 o .. 8 o + 7): words 0..3 = (scale, scale) of columns (8 o + 2 r, 8 o + 2 r + 1),
// words 4..7 = (base + zero) of the same, with the bases of the register unpack; columns past N: zeros.
template <int BITS>
__global__ __launch_bounds__(256) void tile_szt_kernel(const uint32_t *__restrict__ qzeros,
                                                       const _Float16 *__restrict__ scales, uint32_t *__restrict__ szt,
                                                       int N, int G, int octets)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= (uint32_t)G * (uint32_t)octets) return;
    const int g = t / octets, o = t - g * octets;
    uint32_t out[8];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        h2 s2 = {(_Float16)0, (_Float16)0}, zb = {(_Float16)0, (_Float16)0};
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int n = 8 * o + 2 * r + e;
            if (n < N) {
                s2[e] = scales[(size_t)g * N + n];
                zb[e] = (_Float16)((float)zero_of<BITS>(qzeros + (size_t)g * (N / 32 * BITS), n) + TileCodec<BITS>::base(2 * r + e));
            }
        }
        out[r] = as_u32(s2);
        out[4 + r] = as_u32(zb);
    }
    u4 *dst = (u4 *)(szt + (size_t)t * 8);
    dst[0] = (u4){out[0], out[1], out[2], out[3]};
    dst[1] = (u4){out[4], out[5], out[6], out[7]};
}

int launch_tile_prepare_t(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *xsrc,
                          uint32_t *qtile_t, uint32_t *szt, int K, int N, int G, int bits, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const int S_total = (N + 63) / 64, T_total = K / 32;
    const unsigned threads = (unsigned)T_total * (unsigned)S_total * 64u;
    const unsigned tbl = (unsigned)G * (unsigned)S_total * 8u;
    auto go = [&](auto bits_c) {
        constexpr int B = decltype(bits_c)::value;
        hipLaunchKernelGGL(tile_retile_t_kernel<B>, dim3((threads + 255u) / 256u), dim3(256), 0, stream, qweight, xsrc,
                           qtile_t, K, N, S_total, T_total);
        hipLaunchKernelGGL(tile_szt_kernel<B>, dim3((tbl + 255u) / 256u), dim3(256), 0, stream, qzeros,
                           (const _Float16 *)scales, szt, N, G, S_total * 8);
    };
    switch (bits) {
        case 2: go(std::integral_constant<int, 2>{}); break;
        case 3: go(std::integral_constant<int, 3>{}); break;
        case 4: go(std::integral_constant<int, 4>{}); break;
        case 8: go(std::integral_constant<int, 8>{}); break;
        default: return GPTQ_HIP_ERR_BAD_ARG;
    }
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, int AT>
static int launch_tiled_t_one(const TiledParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = tiled_gemm_kernel<BITS, AT, 1, 4, tiled_ring(AT), 2, true>;
    if (plan.lds_bytes < tiled_t_lds_bytes(AT, 4, plan.k_chunk) || plan.waves_k != 4 || plan.block != 256) return GPTQ_HIP_ERR_BAD_ARG;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, plan.grid_z), dim3(256), plan.lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// gy is packed into the workspace (as x is for the forward product), the matmul runs on the transposed copy, and a
// reduce pass follows when the reduction over N is split over workgroups.
int launch_tiled_t(const void *gy, const void *qtile_t, const uint32_t *szt, const int32_t *xsrc, void *gx, char *xpack,
                   float *partial, int M, int K, int N, int bits, int group_size, const gptq_hip_plan &plan,
                   void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const int Np = (N + 63) / 64 * 64;
    TiledParams p;
    p.xpack = xpack;
    p.qtile = (const char *)qtile_t;
    p.sz = nullptr;
    p.bias = nullptr;
    p.y = gx;
    p.partial = partial;
    p.M = M;
    p.N = K;                 // the result has K columns
    p.G = K / group_size;
    p.S_total = Np / 64;     // the reduction runs over the layer's N columns
    p.T_total = K / 32;
    p.wave_steps = plan.k_chunk;
    p.rt_total = plan.row_tiles * plan.m_blocks;
    p.split_k = plan.split_k;
    p.lb_per_group = 1;
    p.szt = szt;
    p.out_map = xsrc;
    p.tiles_per_group = group_size / 32;
    const int S_pack = tiled_pack_blocks(plan.split_k, plan.waves_k, plan.k_chunk);
    hipLaunchKernelGGL(tile_pack_x_kernel, dim3(32 * p.rt_total), dim3(256), 0, stream, (const _Float16 *)gy,
                       (const int32_t *)nullptr, xpack, M, N, Np, p.rt_total, S_pack);
    if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
#define GPTQ_TILED_T_CASE(B, A) \
    if (bits == B && plan.row_tiles == A) rc = launch_tiled_t_one<B, A>(p, plan, stream)
    GPTQ_TILED_T_CASE(2, 1);
    GPTQ_TILED_T_CASE(2, 2);
    GPTQ_TILED_T_CASE(2, 4);
    GPTQ_TILED_T_CASE(3, 1);
    GPTQ_TILED_T_CASE(3, 2);
    GPTQ_TILED_T_CASE(3, 4);
    GPTQ_TILED_T_CASE(4, 1);
    GPTQ_TILED_T_CASE(4, 2);
    GPTQ_TILED_T_CASE(4, 4);
    GPTQ_TILED_T_CASE(8, 1);
    GPTQ_TILED_T_CASE(8, 2);
    GPTQ_TILED_T_CASE(8, 4);
#undef GPTQ_TILED_T_CASE
    if (rc != GPTQ_HIP_OK) return rc;
    if (plan.split_k > 1) {
        const uint32_t quads = (uint32_t)M * ((uint32_t)K / 4u);
        hipLaunchKernelGGL(tiled_reduce_kernel, dim3((quads + 255u) / 256u), dim3(256), 0, stream, partial,
                           (const _Float16 *)nullptr, (_Float16 *)gx, M, K, plan.split_k, xsrc);
        if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    }
    return GPTQ_HIP_OK;
}

template <int BITS, int MR, int KW, int E>
static int launch_decode_one(const DecodeParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = tiled_decode_kernel<BITS, MR, KW, E>;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, 1), dim3(64 * KW), plan.lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, int MR, int E>
static int launch_decode_kw(const DecodeParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    switch (plan.waves_k) {
        case 4: return launch_decode_one<BITS, MR, 4, E>(p, plan, stream);
        case 8: return launch_decode_one<BITS, MR, 8, E>(p, plan, stream);
        case 16: return launch_decode_one<BITS, MR, 16, E>(p, plan, stream);
        default: return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

// The decode product on the tiled format: one launch, plus a reduce pass when K is split over workgroups.
int launch_tiled_decode(const void *x, const void *qtile, const uint32_t *sz, const uint16_t *kinv, const void *bias,
                        void *y, float *partial, int M, int K, int N, int G, int bits, int group_size,
                        const gptq_hip_plan &plan, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    DecodeParams p;
    p.x = (const _Float16 *)x;
    p.kinv = kinv;
    p.qtile = (const char *)qtile;
    p.sz = sz;
    p.bias = bias;
    p.y = y;
    p.partial = partial;
    p.M = M;
    p.K = K;
    p.N = N;
    p.G = G;
    p.S_total = (K + 63) / 64;
    p.T_total = N / 32;
    p.wave_steps = plan.k_chunk;
    p.split_k = plan.split_k;
    p.lb_per_group = group_size / 32;
    // lane block -> group as a multiply-high (lane blocks are below 2^16 / 32 * 2)
    p.lbg_add = p.lb_per_group == 1;
    p.lbg_magic = p.lbg_add ? 0u : (uint32_t)((1ull << 32) / (uint32_t)p.lb_per_group) + 1u;
    const int mr = tiled_decode_rows(M);
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
    // two blocks per epilogue where every unit of two blocks lies in one group
    const bool pairs = group_size % 128 == 0 && plan.k_chunk % 2 == 0;
#define GPTQ_DECODE_CASE(B, R) \
    if (bits == B && mr == R) rc = pairs ? launch_decode_kw<B, R, 2>(p, plan, stream) : launch_decode_kw<B, R, 1>(p, plan, stream)
    GPTQ_DECODE_CASE(4, 1);
    GPTQ_DECODE_CASE(4, 2);
    GPTQ_DECODE_CASE(4, 4);
    GPTQ_DECODE_CASE(3, 1);
    GPTQ_DECODE_CASE(3, 2);
    GPTQ_DECODE_CASE(3, 4);
    GPTQ_DECODE_CASE(2, 1);
    GPTQ_DECODE_CASE(2, 2);
    GPTQ_DECODE_CASE(2, 4);
    GPTQ_DECODE_CASE(8, 1);
    GPTQ_DECODE_CASE(8, 2);
    GPTQ_DECODE_CASE(8, 4);
#undef GPTQ_DECODE_CASE
    if (rc != GPTQ_HIP_OK) return rc;
    if (plan.split_k > 1) {
        const uint32_t quads = (uint32_t)M * ((uint32_t)N / 4u);
        hipLaunchKernelGGL(tiled_reduce_kernel, dim3((quads + 255u) / 256u), dim3(256), 0, stream, partial,
                           (const _Float16 *)bias, (_Float16 *)y, M, N, plan.split_k);
        if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    }
    return GPTQ_HIP_OK;
}

template <int BITS, int MR, bool G128, bool CONTIG>
static int launch_decode16_one(const Decode16Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = tiled_decode16_kernel<BITS, MR, G128, CONTIG>;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x), dim3(1024), plan.lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// The decode product with one workgroup per CU and 16-column units (plan.waves_n == 2): one launch.
int launch_tiled_decode16(const void *x, const void *qtile, const uint32_t *sz, const uint16_t *kinv, const void *bias,
                          void *y, int M, int K, int N, int G, int bits, int group_size, const gptq_hip_plan &plan,
                          void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    Decode16Params p;
    p.x = (const _Float16 *)x;
    p.kinv = kinv;
    p.qtile = (const char *)qtile;
    p.sz = sz;
    p.bias = bias;
    p.y = y;
    p.M = M;
    p.K = K;
    p.N = N;
    p.G = G;
    p.S_total = (K + 63) / 64;
    p.T_total = N / 32;
    p.V_total = (p.S_total + 1) / 2;
    p.units = N / 16;
    p.lb_per_group = group_size / 32;
    p.lbg_add = p.lb_per_group == 1;
    p.lbg_magic = p.lbg_add ? 0u : (uint32_t)((1ull << 32) / (uint32_t)p.lb_per_group) + 1u;
    const int mr = tiled_decode_rows(M);
    const bool g128 = group_size % 128 == 0;
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
    // contiguous ranges per wave when a wave has more than two items (a long K, or several units per workgroup)
    const bool contig = (long long)((p.units + plan.grid_x - 1) / plan.grid_x) * p.V_total > 32;
#define GPTQ_DECODE16_CASE(B, R)                                                                              \
    if (bits == B && mr == R)                                                                                 \
        rc = g128 ? (contig ? launch_decode16_one<B, R, true, true>(p, plan, stream)                          \
                            : launch_decode16_one<B, R, true, false>(p, plan, stream))                        \
                  : (contig ? launch_decode16_one<B, R, false, true>(p, plan, stream)                         \
                            : launch_decode16_one<B, R, false, false>(p, plan, stream))
    GPTQ_DECODE16_CASE(4, 1);
    GPTQ_DECODE16_CASE(4, 2);
    GPTQ_DECODE16_CASE(4, 4);
    GPTQ_DECODE16_CASE(3, 1);
    GPTQ_DECODE16_CASE(3, 2);
    GPTQ_DECODE16_CASE(3, 4);
    GPTQ_DECODE16_CASE(2, 1);
    GPTQ_DECODE16_CASE(2, 2);
    GPTQ_DECODE16_CASE(2, 4);
    GPTQ_DECODE16_CASE(8, 1);
    GPTQ_DECODE16_CASE(8, 2);
    GPTQ_DECODE16_CASE(8, 4);
#undef GPTQ_DECODE16_CASE
    return rc;
}

}  // namespace gptq

