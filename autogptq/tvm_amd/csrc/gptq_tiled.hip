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
// (The decode kernels for up to four rows of x are in gptq_tiled_decode.hip and gptq_tiled_decode16.hip.)
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
#include "gptq_tiled_common.h"

namespace gptq {

typedef float f16v __attribute__((ext_vector_type(16)));

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
    // DIRECT: the A fragments are read from x itself (no pack pass)
    const _Float16 *x;     // fp16 [M, K]
    int K;
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
// DIRECT: no pack pass.  Without an activation order position p is channel p, so lane (m, h) of fragment (S, j) finds
// its eight values in row m of x at 64 S + 32 h + 8 j: sixteen bytes of a 128-byte line that the lane's other seven
// fragments of the block share.  Rows past M read row M - 1 (a row of the result depends on its own row of x only,
// and those rows are never stored), so a wave's load touches M lines; the launcher takes this form up to 16 rows
// (4096 x 11008, us with / without the pack pass: 8 rows 14.0 / 10.7, 16 rows 14.5 / 11.5; with 32 distinct rows
// per load 14.8 / 16.2, 64 rows 19 / 29.5: every lane then asks for a line of its own), and only when K is a whole
// number of blocks that the waves' ranges cover exactly: there is no zero padding to read.
// What the kernel needs before its first requests go out arrives as fourteen dwords that the dispatcher preloads
// into scalar registers (this source is built with kernel-argument preloading), so that a wave does not begin by
// waiting ~0.4 us for its argument segment: the source of the A operand (the packed fragments, or x itself for
// DIRECT), the weights, the (scale, zero) words, the extents, and the group arithmetic in one word.  The pointers of
// the epilogue and the transposed product's tables follow in memory.
struct TiledTail {
    const void *bias;
    void *y;
    float *partial;
    const uint32_t *szt;
    const int32_t *out_map;
    int split_k, tiles_per_group;
};

template <int BITS, int AT, int RW, int KW, int RING, int CT, bool TRANS = false, bool DIRECT = false>
__global__ __launch_bounds__(64 * RW * KW) void tiled_gemm_kernel(const char *a_src, const char *a_qtile, const uint32_t *a_sz,
                                                                  int a_wave_steps, int a_S_total, int a_T_total, int a_rt_total,
                                                                  int a_N, int a_M, int a_K, uint32_t a_groups, const TiledTail t)
{
    TiledParams p;
    p.xpack = a_src, p.x = (const _Float16 *)a_src, p.qtile = a_qtile, p.sz = a_sz;
    p.wave_steps = a_wave_steps, p.S_total = a_S_total, p.T_total = a_T_total, p.rt_total = a_rt_total;
    p.N = a_N, p.M = a_M, p.K = a_K, p.lb_per_group = (int)(a_groups & 0xfffu), p.G = (int)(a_groups >> 12);
    p.bias = t.bias, p.y = t.y, p.partial = t.partial, p.szt = t.szt, p.out_map = t.out_map;
    p.split_k = t.split_k, p.tiles_per_group = t.tiles_per_group;
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
    // DIRECT: the lane's rows of x, at its half of a block
    const _Float16 *a_row[AT];
    if constexpr (DIRECT) {
#pragma unroll
        for (int rt = 0; rt < AT; rt++)
            a_row[rt] = p.x + (size_t)min(32 * (rt0 + rt) + n, p.M - 1) * (size_t)p.K + 32 * h;
    }
    auto load_a = [&](int S, int j, h8 (&ar)[AT]) {
        if constexpr (DIRECT) {
            const int off = 64 * S + 8 * j;
#pragma unroll
            for (int rt = 0; rt < AT; rt++) ar[rt] = *(const h8 *)(a_row[rt] + off);
        } else {
            const char *src = p.xpack + (size_t)(4 * S + j) * a_frag_row + a_lane;
#pragma unroll
            for (int rt = 0; rt < AT; rt++) ar[rt] = __builtin_bit_cast(h8, *(const u4 *)(src + rt * 1024));
        }
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
    // prologue, in consumption order.  The weights of the whole ring are asked for here (they come from HBM); the A
    // fragments of the first slot only: those of the other slots (L2, short latency) are asked for while the first
    // block is multiplied (FIRST in block below).  With all of them in the prologue a wave spent 2.8 us putting sixty
    // requests into a queue that drains at the memory's pace before its first matrix instruction.
    // (The transposed product keeps the whole ring in its prologue.)
    int S_of[RING];   // the block each ring slot holds (TRANS: its table entries are looked up by block)
#pragma unroll
    for (int u = 0; u < RING; u++) {
        const int S = next_block();
        S_of[u] = S;
        load_b(S, w[u], szr[u]);
        if (TRANS || u == 0) {
#pragma unroll
            for (int j = 0; j < 4; j++) load_a(S, j, a[u][j]);
        }
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
    auto block = [&](auto u_c, auto refill_c, auto first_c) {
        constexpr int u = decltype(u_c)::value;
        constexpr bool REFILL = decltype(refill_c)::value;
        constexpr bool FIRST = decltype(first_c)::value;   // the first block of the walk: asks for the other slots' A fragments
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
                if (FIRST && ct == CT - 1) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 1; s < RING; s++) load_a(S_of[s], j, a[s][j]);
                    __builtin_amdgcn_sched_barrier(0);
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
    if constexpr (TRANS) {
        const int full = p.wave_steps / RING * RING;
        for (int i0 = 0; i0 < full; i0 += RING) {
            [&]<int... U>(std::integer_sequence<int, U...>) {
                (block(std::integral_constant<int, U>{}, std::true_type{}, std::false_type{}), ...);
            }(std::make_integer_sequence<int, RING>{});
        }
        const int rem = p.wave_steps - full;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((U < RING - 1 && U < rem ? block(std::integral_constant<int, U>{}, std::false_type{}, std::false_type{}) : (void)0), ...);
        }(std::make_integer_sequence<int, RING>{});
    } else {
        // the first block by itself (every wave has one; its refill wraps around inside the wave's range when the
        // range is shorter than the ring, like every refill near the end of the walk), then whole turns of the ring
        // that begin at slot 1, then the rest
        block(std::integral_constant<int, 0>{}, std::true_type{}, std::true_type{});
        const int left = p.wave_steps - 1;
        const int full = left / RING * RING;
        for (int i0 = 0; i0 < full; i0 += RING) {
            [&]<int... U>(std::integer_sequence<int, U...>) {
                (block(std::integral_constant<int, (U + 1) % RING>{}, std::true_type{}, std::false_type{}), ...);
            }(std::make_integer_sequence<int, RING>{});
        }
        const int rem = left - full;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((U < RING - 1 && U < rem ? block(std::integral_constant<int, (U + 1) % RING>{}, std::false_type{}, std::false_type{})
                                      : (void)0),
             ...);
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

int launch_tiled_reduce(const float *partial, const void *bias, void *y, int M, int N, int split_k, const int32_t *out_map,
                        hipStream_t stream)
{
    const uint32_t quads = (uint32_t)M * ((uint32_t)N / 4u);
    hipLaunchKernelGGL(tiled_reduce_kernel, dim3((quads + 255u) / 256u), dim3(256), 0, stream, partial,
                       (const _Float16 *)bias, (_Float16 *)y, M, N, split_k, out_map);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// the kernel's argument list from its parameter struct
template <typename Kern>
static int launch_gemm_kernel(Kern kern, dim3 grid, dim3 block, int lds_bytes, hipStream_t stream, const TiledParams &p,
                              bool direct)
{
    if (p.lb_per_group < 0 || p.lb_per_group > 0xfff || p.G < 0 || p.G >= (1 << 20)) return GPTQ_HIP_ERR_UNSUPPORTED;
    TiledTail t;
    t.bias = p.bias, t.y = p.y, t.partial = p.partial, t.szt = p.szt, t.out_map = p.out_map;
    t.split_k = p.split_k, t.tiles_per_group = p.tiles_per_group;
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, direct ? (const char *)p.x : p.xpack, p.qtile, p.sz, p.wave_steps,
                       p.S_total, p.T_total, p.rt_total, p.N, p.M, p.K, (uint32_t)p.lb_per_group | ((uint32_t)p.G << 12), t);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, int AT, int RW, int KW, int RING, int CT, bool DIRECT = false>
static int launch_tiled_one(const TiledParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = tiled_gemm_kernel<BITS, AT, RW, KW, RING, CT, false, DIRECT>;
    const int lds_bytes = tiled_lds_bytes(AT * RW, KW);
    if (plan.lds_bytes < lds_bytes || plan.waves_k != KW || plan.block != 64 * RW * KW) return GPTQ_HIP_ERR_BAD_ARG;
    if (lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    return launch_gemm_kernel(kern, dim3(plan.grid_x, plan.grid_y, plan.grid_z), dim3(64 * RW * KW), lds_bytes, stream, p, DIRECT);
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
    p.x = (const _Float16 *)x;
    p.K = K;
    const int S_pack = tiled_pack_blocks(plan.split_k, plan.waves_k, plan.k_chunk);
    // without an activation order the fragments can be read from x itself: one launch less
    const bool direct = tiled_reads_x_directly(xsrc != nullptr, M, K, plan);
    if (!direct) {
        const int pack_lds = xsrc ? K * 2 : 0;  // one row of x
        if (pack_lds > 65536) {
            if (hipFuncSetAttribute((const void *)tile_pack_x_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    pack_lds) != hipSuccess) {
                (void)hipGetLastError();
                return GPTQ_HIP_ERR_LAUNCH;
            }
        }
        hipLaunchKernelGGL(tile_pack_x_kernel, dim3(32 * p.rt_total), dim3(256), pack_lds, stream, (const _Float16 *)x,
                           xsrc, xpack, M, K, Kp, p.rt_total, S_pack);
        if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    }
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
#define GPTQ_TILED_CASE(B, A)                                                                  \
    if (bits == B && plan.row_tiles == A && plan.waves_n == 1)                                 \
        rc = launch_tiled_one<B, A, 1, 4, tiled_ring(A), 2>(p, plan, stream)
    if (direct) {
        switch (bits) {
            case 2: rc = launch_tiled_one<2, 1, 1, 4, tiled_ring(1), 2, true>(p, plan, stream); break;
            case 3: rc = launch_tiled_one<3, 1, 1, 4, tiled_ring(1), 2, true>(p, plan, stream); break;
            case 4: rc = launch_tiled_one<4, 1, 1, 4, tiled_ring(1), 2, true>(p, plan, stream); break;
            case 8: rc = launch_tiled_one<8, 1, 1, 4, tiled_ring(1), 2, true>(p, plan, stream); break;
            default: break;
        }
    } else {
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
    }
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
    return launch_gemm_kernel(kern, dim3(plan.grid_x, plan.grid_y, plan.grid_z), dim3(256), plan.lds_bytes, stream, p, false);
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
    p.x = nullptr;           // (the forward product's direct read of x: not used here)
    p.K = K;
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

}  // namespace gptq

