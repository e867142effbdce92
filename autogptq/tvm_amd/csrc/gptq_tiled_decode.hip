// TILED family, the decode kernel with a workgroup per 32-column tile: up to four rows of x on the tiled format
// (the format, its preparation and the matmul kernel for more rows are in gptq_tiled.hip; the decode kernel with
// one workgroup per CU in gptq_tiled_decode16.hip).
#include "gptq_tiled_common.h"

namespace gptq {

// ---------------------------------------------------------------------------------------------------
// tiled_decode_kernel: M <= 4 rows of x on the tiled format.
//
// A workgroup owns ONE column tile (32 columns) and one K range; its KW waves split that range.  With one
// small workgroup per tile every CU gets work whatever N is (11008 columns: 344 workgroups of 4 waves,
// 4096 columns: 128 of 16), and what a wave keeps in flight (eight blocks of 1 KB / 768 B) adds up over the
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
    unsigned long long *slots;  // halved tiles (grid_x > T_total): [tile - first halved][MR][32] (tag << 32 | fp32 bits), zero between launches
    int split_k;
    int lb_per_group;       // group_size / 32
    uint32_t lbg_magic;     // lane block -> group: umulhi(lb, magic) + (add ? lb : 0)
    int lbg_add;
    int grid_x, grid_y;     // the launch's grid (from here: the dispatch packet is one more cold line to read)
};

// Everything the kernel needs before its results are stored travels as its first fourteen dwords of arguments,
// which the dispatcher hands over in scalar registers (this source is built with kernel-argument preloading; fourteen
// is what the user registers leave room for): a wave otherwise begins by waiting ~0.4 us for its argument segment to
// arrive from memory.  Hence the packing: M and the blocks per wave in one word, the group arithmetic's flag and the
// number of K ranges in another, and what follows from these (N = 32 tiles, blocks = ceil(K / 64), the number of
// groups) worked out in the kernel.  The pointers of the epilogue follow as a struct, read while the walk runs.
struct DecodeTail {
    const void *bias;
    void *y;
    float *partial;
    unsigned long long *slots;
};

// E: blocks of 64 positions that share one epilogue (1, or 2 when the groups are multiples of 128 channels and
// every wave has an even number of blocks: both lane blocks of both blocks then lie in one group).
template <int BITS, int MR, int KW, int E>
__global__ __launch_bounds__(64 * KW) void tiled_decode_kernel(const _Float16 *a_x, const uint16_t *a_kinv, const char *a_qtile,
                                                               const uint32_t *a_sz, int a_K, uint32_t a_m_steps, int a_T_total,
                                                               int a_grid_x, uint32_t a_lbg_magic, uint32_t a_flags,
                                                               const DecodeTail t)
{
    DecodeParams p;
    p.x = a_x, p.kinv = a_kinv, p.qtile = a_qtile, p.sz = a_sz;
    p.K = a_K, p.M = (int)(a_m_steps & 0xffu), p.wave_steps = (int)(a_m_steps >> 8);
    p.T_total = a_T_total, p.N = 32 * a_T_total, p.S_total = (a_K + 63) >> 6, p.grid_x = a_grid_x;
    p.lbg_magic = a_lbg_magic, p.lbg_add = (int)(a_flags & 1u), p.split_k = (int)(a_flags >> 1), p.grid_y = p.split_k;
    // groups = (K / 32) / (lane blocks per group), by the same multiply-high that maps a lane block to its group
    p.G = (int)(__umulhi((uint32_t)a_K >> 5, a_lbg_magic) + (p.lbg_add ? (uint32_t)a_K >> 5 : 0u));
    p.bias = t.bias, p.y = t.y, p.partial = t.partial, p.slots = t.slots;
    static_assert((MR == 1 || MR == 2 || MR == 4 || MR == 8) && (E == 1 || E == 2), "one or two sets of four rows");
    constexpr int RS = (MR + 3) / 4;   // sets of four rows: a matrix instruction takes four rows of x
    constexpr bool EXACT = tiled_decode_exact(BITS);
    constexpr int NT = 64 * KW;
    constexpr int PF = 2;              // blocks of weights per chunk
    // chunks in flight per wave.  A wave asks for a chunk when it has consumed one, so its walk is a chain of
    // round trips to HBM (0.9-1 us each under load), one per NCH chunks: with two chunks in flight a wave of 16
    // blocks makes four of them, and the walk, not the staging of x, sets the length of the kernel.  Four chunks
    // for the workgroups of four waves (wide layers with K up to 4096: 16 or 8 blocks per wave), one or two rows:
    // 4096 x 11008 int4 7.5 -> 7.0 us with an activation order, 7.5 -> 6.8 without (int3 6.55 either way).  The
    // longer waves of eight and sixteen keep two: four cost them occupancy (100 registers against 60) and more
    // than they gain (9216 x 9216 int3 9.4 -> 10.5 us, 9216 x 36864 24.9 -> 27.9), four rows and 8 bits as well.
    constexpr int NCH = (KW == 4 && MR <= 2 && !EXACT) ? 4 : 2;
    constexpr int RING = NCH * PF;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    // The e tiles past a whole number per CU (the planner: when e is at most half the CUs) are HALVED along K
    // (grid_x = tiles + e): the first tiles - e workgroups take a whole tile each and the 2 e workgroups after
    // them half a tile, so that the fullest CU holds half a tile more than the others instead of a whole one
    // (two whole tiles on 88 of the 256 CUs bound both the memory and the instruction path of 11008 columns).
    // The two halves of a tile meet through one 64-bit exchange per output (see the end of the kernel).
    const int n_halved = p.grid_x - p.T_total;           // e (0: no tile is halved)
    const int n_whole = p.T_total - n_halved;
    const bool is_half = (int)blockIdx.x >= n_whole;
    const int half_i = (int)blockIdx.x - n_whole;        // (halved tile, half) = (half_i / 2, half_i % 2)
    const int T = is_half ? n_whole + (half_i >> 1) : (int)blockIdx.x;
    const int split = is_half ? (half_i & 1) : (int)blockIdx.y;
    // blocks per wave: all of them, or the first half's share (rounded up, to an even count where blocks pair
    // up) and the rest for the second half
    const int ws_first = tiled_decode_first_half(p.wave_steps, E == 2);
    const int ws = is_half ? (split ? p.wave_steps - ws_first : ws_first) : p.wave_steps;
    const int wg_steps = ws * KW;                        // blocks of the workgroup's K range
    const int S_wg = is_half ? split * ws_first * KW : split * wg_steps;   // its first block
    const int S_begin = S_wg + wave * ws;                // this wave's first block
    const int span = wg_steps * 64;                      // positions the workgroup stages
    const int p0 = S_wg * 64;                            // its first position

    // LDS: x in position order [MR][span] fp16 | 64 zero bytes | block sums [span / 32][MR] (Xsum, Bsum) |
    //      partial results [KW][MR][32]
    _Float16 *xl = (_Float16 *)smem;
    const uint32_t zero_off = (uint32_t)MR * (uint32_t)span * 2u;
    f2 *xs = (f2 *)(smem + zero_off + 64);
    const int lbs = span / 32;
    float *red = (float *)(xs + (size_t)lbs * MR);

    // ---- 1. x and the map first (a wait for them would also wait for every older load: vector loads return
    //         in order), then the first weights of this wave, each unit's (scale, zero) word in front of them.
    //         (The words are cold in HBM and belong to one tile: staged through LDS they kept every wave of the
    //         workgroup at the barrier until the last of them had arrived, 0.6-0.9 us after x; a wave now asks
    //         for the word of a unit when it asks for the unit's weights and finds it when they are there.) -----
    // (without a map the channels of the range are the range itself)
    const int k8_lo = p.kinv ? 0 : p0 / 8, k8_hi = p.kinv ? p.K / 8 : min(p0 + span, p.K) / 8;
    constexpr int QP = MR == 8 ? 1 : 2;  // passes over x kept in registers (eight rows: 32 registers a pass)
    u4 kq[QP];
    h8 xq[QP][MR];
#pragma unroll
    for (int ps = 0; ps < QP; ps++) {
        const int k = 8 * min(k8_lo + tid + ps * NT, k8_hi - 1);  // (clamped: the pass is skipped below when outside)
        kq[ps] = p.kinv ? *(const u4 *)(p.kinv + k) : (u4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int m = 0; m < MR; m++) xq[ps][m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
    }
    // (a workgroup with a part of K, a half tile or one of several ranges, keeps the channels of its own range)
    const bool ranged = is_half || p.grid_y > 1;
    auto scatter8 = [&](int k, const u4 &kv, const h8 (&xv)[MR]) {
        if (!p.kinv) {   // no activation order: the eight channels are eight consecutive positions, one store
            // (k8_lo .. k8_hi is the workgroup's own range here, a multiple of 8 away from p0)
#pragma unroll
            for (int m = 0; m < MR; m++) *(h8 *)(xl + m * span + (k - p0)) = xv[m];
            return;
        }
        if (!ranged) {   // the workgroup stages all of K: every position is its own, no test and no branch per channel
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t pos = (kv[e >> 1] >> (16 * (e & 1))) & 0xffffu;
#pragma unroll
                for (int m = 0; m < MR; m++) xl[(uint32_t)(m * span) + pos] = xv[m][e];
            }
            return;
        }
        // a part of K: a channel outside the range goes to a slot of the lane's own in the area of the partial results,
        // which is written again before it is read (no branch per channel: the waves of a half tile are the last of
        // the kernel to finish, and this walk over all of x is what they do first)
        const uint32_t dump = (uint32_t)(((const unsigned char *)red - smem) >> 1) + (uint32_t)lane;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int pos = (int)((kv[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            const int pl = pos - p0;
            const bool mine = (unsigned)pl < (unsigned)span;
#pragma unroll
            for (int m = 0; m < MR; m++) xl[mine ? (uint32_t)(m * span + pl) : dump] = xv[m][e];
        }
    };
    // Long layers: the channels the register passes do not hold, a pass at a time, before the weights are asked for
    // (a wait for a load waits for every older one).  The loads of a pass are issued together and waited for inside one
    // asm statement: left to the compiler's own bookkeeping, a loop with loads in it made it assume their
    // registers still pending wherever the loop may have run, and it put a wait for outstanding loads in front of
    // the weight requests, or, with the loop behind them, a wait for all of them in front of the sums and the walk.
    for (int k8 = k8_lo + tid + QP * NT; k8 < k8_hi; k8 += NT) {
        const int k = 8 * k8;
        u4 kv = {0u, 0u, 0u, 0u};
        h8 xv[MR];
        if (p.kinv) {   // the map and the rows of x, requested together
            const void *ptr[MR + 1];
            u4 v[MR + 1];
            ptr[MR] = p.kinv + k;
#pragma unroll
            for (int m = 0; m < MR; m++) ptr[m] = p.x + (size_t)min(m, p.M - 1) * p.K + k;
            LoadNow<MR + 1>::run(v, ptr);
            kv = v[MR];
#pragma unroll
            for (int m = 0; m < MR; m++) xv[m] = __builtin_bit_cast(h8, v[m]);
        } else {
            const void *ptr[MR];
            u4 v[MR];
#pragma unroll
            for (int m = 0; m < MR; m++) ptr[m] = p.x + (size_t)min(m, p.M - 1) * p.K + k;
            LoadNow<MR>::run(v, ptr);
#pragma unroll
            for (int m = 0; m < MR; m++) xv[m] = __builtin_bit_cast(h8, v[m]);
        }
        scatter8(k, kv, xv);
    }
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t b_lane = tile_lane_bytes<BITS>((uint32_t)lane);
    constexpr uint32_t BLOCK_BYTES = 256u * BITS;
    // the tile as a buffer: the lane's offset in a vector register, the block's in a scalar one.  Blocks requested
    // past the wave's range (ahead of the walk, never multiplied) are the next wave's; past the end of the tile:
    // its last block again (the padding of K past the wave's range: multiplied by zeros of x)
    const __amdgpu_buffer_rsrc_t tile = tile_buffer(p.qtile + (size_t)T * (size_t)p.S_total * BLOCK_BYTES,
                                                    (uint32_t)p.S_total * BLOCK_BYTES);
    const int S_last = p.S_total - 1;
    // the (scale, zero) words of the tile's 32 columns as a buffer: lane n (both halves) reads column n of the
    // group of its lane block, the group's row in a scalar register
    const __amdgpu_buffer_rsrc_t szb = tile_buffer((const char *)(p.sz + 32 * T), (uint32_t)(((size_t)p.G * p.N - 32 * T) * 4));
    const uint32_t sz_lane = (uint32_t)n * 4u;
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    auto group_of = [&](uint32_t lb) { return min(__umulhi(lb, p.lbg_magic) + (p.lbg_add ? lb : 0u), (uint32_t)p.G - 1u); };
    constexpr int UPC = PF / E;        // units per chunk
    uint32_t w[NCH][PF][BITS], szr[NCH][UPC];
    auto load_w = [&](int i, uint32_t (&wr)[BITS]) {
        tile_load<BITS>(tile, b_lane, (uint32_t)min(S_begin + i, S_last) * BLOCK_BYTES, wr);
    };
    auto load_s = [&](int i, uint32_t &sr) {   // the unit that starts with block i of the wave's range
        const uint32_t l0 = 2u * (uint32_t)min(S_begin + i, S_last);
        const uint32_t g0 = group_of(l0);
        uint32_t off = sz_lane;
        if constexpr (E == 1) off += h ? (group_of(l0 + 1u) - g0) * row_bytes : 0u;   // the two halves of a block may differ
        sr = __builtin_amdgcn_raw_buffer_load_b32(szb, off, g0 * row_bytes, 0);
    };
    auto load_chunk = [&](int i, uint32_t (&wc)[PF][BITS], uint32_t (&sc)[UPC]) {
#pragma unroll
        for (int u = 0; u < UPC; u++) load_s(i + u * E, sc[u]);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(i + u, wc[u]);
    };
    // NCH chunks of PF blocks are in flight from here on, through the staging of x as well
#pragma unroll
    for (int j = 0; j < NCH; j++) load_chunk(j * PF, w[j], szr[j]);
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
#pragma unroll
    for (int ps = 0; ps < QP; ps++) {
        const int k8 = k8_lo + tid + ps * NT;
        if (k8 < k8_hi) scatter8(8 * k8, kq[ps], xq[ps]);
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
        for (int q0 = 0; q0 < 4 * ws; q0 += 64) {   // 16-position pieces of the wave's range
            const int piece = q0 + lane;
            const int sb = sb0 + (piece >> 2), hh = (piece >> 1) & 1;
            const bool live = piece < 4 * ws;
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
    // registers.
    // The matrix instruction broadcasts A: with cbsz = 3 the eight 4-lane blocks of a half wave all take their A
    // operand from block `abid` of the half.  So lane block b of a half holds only positions 4 b .. 4 b + 3 of the
    // half's 32 (one 8-byte read per lane and block instead of 64 bytes), and the instruction for positions
    // 4 i .. 4 i + 3 names abid = i.
    const int lb8 = (lane >> 2) & 7;
    // (a lane whose row lies past M supplies the last row again: row i of A only reaches result register i, and
    // the registers past M are never stored; one stride for all lanes keeps the block's offset an immediate)
    uint32_t x_base[RS];
#pragma unroll
    for (int rs = 0; rs < RS; rs++) x_base[rs] = (uint32_t)(min(4 * rs + row_i, p.M - 1) * span + 32 * h + 4 * lb8) * 2u;
    constexpr uint32_t x_stride = 128u;
    const uint32_t xs_lane = zero_off + 64u + (uint32_t)(h * MR) * 8u;   // sums of half h of unit 0

    // x of a block: this lane's four positions of row row_i; read one block ahead of its use
    auto load_x = [&](uint32_t sb, u2 (&xv)[RS]) {
#pragma unroll
        for (int rs = 0; rs < RS; rs++) xv[rs] = *(const u2 *)(smem + x_base[rs] + x_stride * sb);
    };
    f4 c0[RS], c1[RS];  // two chains per set of rows: a matrix instruction waits for the one it adds to
#pragma unroll
    for (int rs = 0; rs < RS; rs++) c0[rs] = c1[rs] = (f4){0.f, 0.f, 0.f, 0.f};
    uint32_t szw = 0u;   // (scale, zero) word and sums of the unit in flight, read when the unit starts
    f2 xsv[MR];
    auto block = [&](auto uu_c, int S, const uint32_t (&wr)[BITS], uint32_t sr, const u2 (&xc)[RS], u2 (&xn)[RS]) {
        constexpr int uu = decltype(uu_c)::value;                 // block inside its unit
        const uint32_t sb = (uint32_t)(S - S_wg);                  // block inside the workgroup's range (wave-uniform)
        if constexpr (uu == 0) {
            szw = sr;   // the unit's (scale, zero) word, requested with its weights
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
#pragma unroll
        for (int rs = 0; rs < RS; rs++) {
            if constexpr (uu == 0) {
                c0[rs] = (f4){0.f, 0.f, 0.f, 0.f};
                c1[rs] = (f4){0.f, 0.f, 0.f, 0.f};
            }
            const h4 xa = __builtin_bit_cast(h4, xc[rs]);
            [&]<int... V>(std::integer_sequence<int, V...>) {
                ((c0[rs] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa, __builtin_bit_cast(h4, (u2){q[V][0], q[V][1]}), c0[rs], 3, 2 * V, 0),
                  c1[rs] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa, __builtin_bit_cast(h4, (u2){q[V][2], q[V][3]}), c1[rs], 3, 2 * V + 1, 0)),
                 ...);
            }(std::make_integer_sequence<int, 4>{});
        }
        if constexpr (uu == E - 1) {
            if constexpr (EXACT) {
#pragma unroll
                for (int m = 0; m < MR; m++) ysum[m] += c0[m / 4][m % 4] + c1[m / 4][m % 4];
            } else {
                const h2 e = as_h2(szw);
                const float sc = (float)e[0], zp = (float)e[1];
#pragma unroll
                for (int m = 0; m < MR; m++)
                    ysum[m] += sc * (((c0[m / 4][m % 4] + c1[m / 4][m % 4]) - xsv[m][1]) - zp * xsv[m][0]);
            }
        }
    };

    // Chunks of PF blocks, NCH in flight; x rides one block ahead in two register sets.  Blocks past the end
    // of K inside a wave's range are harmless (their x and sums are zeros), blocks past the range are skipped.
    u2 xr[2][RS];
    load_x((uint32_t)(S_begin - S_wg), xr[0]);
    auto chunk = [&](int c, uint32_t (&wc)[PF][BITS], const uint32_t (&sc)[UPC], auto all_c) {
        constexpr bool ALL = decltype(all_c)::value;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((ALL || c + U < ws
                  ? block(std::integral_constant<int, U % E>{}, S_begin + c + U, wc[U], sc[U / E], xr[U & 1], xr[(U + 1) & 1])
                  : (void)0),
             ...);
        }(std::make_integer_sequence<int, PF>{});
    };
    int c = 0;
    // steady state: every chunk consumed is replaced by the one a ring further on, which lies inside the range
    for (; c + 2 * RING <= ws; c += RING) {
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            chunk(c + j * PF, w[j], szr[j], std::true_type{});
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(c + RING + j * PF, w[j], szr[j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (ws - c == RING) {   // exactly what is in flight is left: no more requests, no tests
#pragma unroll
        for (int j = 0; j < NCH; j++) chunk(c + j * PF, w[j], szr[j], std::true_type{});
    } else {
        // less than two rings left: the blocks in flight, then the rest, requested as registers come free.  No load
        // stands behind a test (the compiler would no longer know how many are outstanding, and wait for all of them
        // at every chunk): a chunk past the end of the range asks for the range's last chunk again, which the
        // cache has, and is not multiplied.
        const int last_chunk = max((ws - 1) / PF * PF, 0);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            chunk(c + j * PF, w[j], szr[j], std::false_type{});
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(min(c + RING + j * PF, last_chunk), w[j], szr[j]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NCH; j++) chunk(c + RING + j * PF, w[j], szr[j], std::false_type{});
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
            if (is_half) {
                // One 64-bit exchange per output carries the half's sum and a tag: the half that finds the slot
                // empty leaves its sum there; the other finds it, adds (a + b = b + a: the result does not depend on
                // which half came first), writes y and empties the slot for the next launch.  The payload travels
                // inside the atomic itself, so no other ordering is needed.
                unsigned long long *slot = p.slots + ((size_t)(T - n_whole) * MR + m) * 32 + nn;
                const unsigned long long mine = (1ull << 32) | (unsigned long long)__builtin_bit_cast(uint32_t, sum);
                const unsigned long long old = __hip_atomic_exchange(slot, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((old >> 32) != 0ull) {
                    float total = sum + __builtin_bit_cast(float, (uint32_t)old);
                    if (p.bias) total += (float)((const _Float16 *)p.bias)[32 * T + nn];
                    ((_Float16 *)p.y)[o] = (_Float16)total;
                    __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else if (p.split_k == 1) {
                if (p.bias) sum += (float)((const _Float16 *)p.bias)[32 * T + nn];
                ((_Float16 *)p.y)[o] = (_Float16)sum;
            } else {
                p.partial[(size_t)split * p.M * p.N + o] = sum;
            }
        }
    }
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
    if (plan.split_k != plan.grid_y || p.M > 255 || p.wave_steps >= (1 << 24)) return GPTQ_HIP_ERR_BAD_ARG;
    DecodeTail t;
    t.bias = p.bias, t.y = p.y, t.partial = p.partial, t.slots = p.slots;
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, 1), dim3(64 * KW), plan.lds_bytes, stream, p.x, p.kinv, p.qtile, p.sz,
                       p.K, (uint32_t)p.M | ((uint32_t)p.wave_steps << 8), p.T_total, plan.grid_x, p.lbg_magic,
                       (uint32_t)p.lbg_add | ((uint32_t)p.split_k << 1), t);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, int MR, int E>
static int launch_decode_kw(const DecodeParams &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    switch (plan.waves_k) {
        case 4: return launch_decode_one<BITS, MR, 4, E>(p, plan, stream);
        case 8: return launch_decode_one<BITS, MR, 8, E>(p, plan, stream);
        case 16:
            if constexpr (MR == 8) return GPTQ_HIP_ERR_UNSUPPORTED;   // (128 registers per lane do not hold two sets of rows)
            else return launch_decode_one<BITS, MR, 16, E>(p, plan, stream);
        default: return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

// The decode product on the tiled format: one launch, plus a reduce pass when K is split over workgroups.
int launch_tiled_decode(const void *x, const void *qtile, const uint32_t *sz, const uint16_t *kinv, const void *bias,
                        void *y, float *partial, unsigned long long *slots, int M, int K, int N, int G, int bits,
                        int group_size, const gptq_hip_plan &plan, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    if ((unsigned long long)G * (unsigned long long)N >= (1ull << 30)) return GPTQ_HIP_ERR_UNSUPPORTED;   // 32-bit offsets into sz
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
    p.slots = slots;
    p.split_k = plan.split_k;
    p.lb_per_group = group_size / 32;
    // lane block -> group as a multiply-high (lane blocks are below 2^16 / 32 * 2)
    p.lbg_add = p.lb_per_group == 1;
    p.lbg_magic = p.lbg_add ? 0u : (uint32_t)((1ull << 32) / (uint32_t)p.lb_per_group) + 1u;
    {   // the kernel works the number of groups and of columns out from what it is handed: they must come out as given
        const uint32_t lbs = (uint32_t)K >> 5;
        const uint32_t groups = (uint32_t)(((unsigned long long)lbs * p.lbg_magic) >> 32) + (p.lbg_add ? lbs : 0u);
        if ((int)groups != G || N % 32 != 0) return GPTQ_HIP_ERR_UNSUPPORTED;
    }
    const int mr = tiled_decode_rows(M);
    int rc = GPTQ_HIP_ERR_UNSUPPORTED;
    // two blocks per epilogue where every unit of two blocks lies in one group
    // (halved tiles, grid_x > tiles: their waves walk the two even shares of k_chunk that the planner checked)
    const bool pairs = tiled_decode_pairs(group_size, plan.k_chunk);
#define GPTQ_DECODE_CASE(B, R) \
    if (bits == B && mr == R) rc = pairs ? launch_decode_kw<B, R, 2>(p, plan, stream) : launch_decode_kw<B, R, 1>(p, plan, stream)
    GPTQ_DECODE_CASE(4, 1);
    GPTQ_DECODE_CASE(4, 2);
    GPTQ_DECODE_CASE(4, 4);
    GPTQ_DECODE_CASE(4, 8);
    GPTQ_DECODE_CASE(3, 1);
    GPTQ_DECODE_CASE(3, 2);
    GPTQ_DECODE_CASE(3, 4);
    GPTQ_DECODE_CASE(3, 8);
    GPTQ_DECODE_CASE(2, 1);
    GPTQ_DECODE_CASE(2, 2);
    GPTQ_DECODE_CASE(2, 4);
    GPTQ_DECODE_CASE(2, 8);
    GPTQ_DECODE_CASE(8, 1);
    GPTQ_DECODE_CASE(8, 2);
    GPTQ_DECODE_CASE(8, 4);
    GPTQ_DECODE_CASE(8, 8);
#undef GPTQ_DECODE_CASE
    if (rc != GPTQ_HIP_OK) return rc;
    if (plan.split_k > 1) {
        if (launch_tiled_reduce(partial, bias, y, M, N, plan.split_k, nullptr, stream) != GPTQ_HIP_OK)
            return GPTQ_HIP_ERR_LAUNCH;
    }
    return GPTQ_HIP_OK;
}

}  // namespace gptq
