// TILED family, the decode kernel with one workgroup per CU and 16-column units (the kernel with a workgroup per
// 32-column tile is in gptq_tiled_decode.hip; the format, its preparation and the matmul kernel in gptq_tiled.hip).
#include "gptq_tiled_common.h"

namespace gptq {

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
    int grid_x;             // workgroups of the launch
};

// The arguments arrive as fourteen dwords that the dispatcher preloads into scalar registers (this source is built
// with kernel-argument preloading), so that a wave does not begin by waiting ~0.4 us for its argument segment: the
// four input pointers, K, N, one word of (M, the group arithmetic's flag, the grid), the multiplier of the group
// arithmetic, and y.  What follows from these (blocks, tiles, units, groups) is worked out here; the bias pointer,
// needed at the very end, follows in memory.
template <int BITS, int MR, bool G128, bool CONTIG>
__global__ __launch_bounds__(1024) void tiled_decode16_kernel(const _Float16 *a_x, const uint16_t *a_kinv, const char *a_qtile,
                                                              const uint32_t *a_sz, int a_K, int a_N, uint32_t a_packed,
                                                              uint32_t a_lbg_magic, void *a_y, const void *a_bias)
{
    Decode16Params p;
    p.x = a_x, p.kinv = a_kinv, p.qtile = a_qtile, p.sz = a_sz, p.y = a_y, p.bias = a_bias;
    p.K = a_K, p.N = a_N, p.M = (int)(a_packed & 0xffu), p.lbg_add = (int)((a_packed >> 8) & 1u), p.grid_x = (int)(a_packed >> 9);
    p.lbg_magic = a_lbg_magic;
    p.S_total = (a_K + 63) >> 6, p.T_total = a_N >> 5, p.V_total = (p.S_total + 1) >> 1, p.units = a_N >> 4;
    p.G = (int)(__umulhi((uint32_t)a_K >> 5, a_lbg_magic) + (p.lbg_add ? (uint32_t)a_K >> 5 : 0u));
    static_assert(MR <= 4, "one matrix instruction set per lane block");
    constexpr bool EXACT = tiled_decode_exact(BITS);
    constexpr int NT = 1024, NW = 16;
    constexpr int PF = 2;               // items of weights per chunk; two chunks are in flight
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n16 = lane & 15, lbv = lane >> 4;
    // (32-bit: units <= 2^16 and at most 2^15 workgroups, checked at launch; a 64-bit division is ~100 instructions)
    const int u0 = (int)((uint32_t)p.units * blockIdx.x / (uint32_t)p.grid_x);
    const int u1 = (int)((uint32_t)p.units * (blockIdx.x + 1u) / (uint32_t)p.grid_x);
    const int n_units = u1 - u0;
    const int span = p.V_total * 128;   // positions staged: all of K, padded to whole virtual blocks
    const int S_last = p.S_total - 1;

    // LDS: x in position order [MR][span] fp16 | 64 zero bytes | sums [span / 32][MR] (Xsum, Bsum) |
    //      partial results [n_units][NW][MR][64]
    _Float16 *xl = (_Float16 *)smem;
    const uint32_t zero_off = (uint32_t)MR * (uint32_t)span * 2u;
    f2 *xs = (f2 *)(smem + zero_off + 64);
    float *red = (float *)(xs + (size_t)(span / 32) * MR);

    // ---- 1. requests: x and the map first (loads return in order), then the weights, each item's (scale, zero)
    //         word in front of it (the words are cold in HBM: staged through LDS they held every wave at the
    //         barrier until the last of them had arrived, well after x) ---------------------------------------
    const int k8_hi = p.K / 8;
    u4 kq;
    h8 xq[MR];
    {
        const int k = 8 * min(tid, k8_hi - 1);
        kq = p.kinv ? *(const u4 *)(p.kinv + k) : (u4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int m = 0; m < MR; m++) xq[m] = *(const h8 *)(p.x + (size_t)min(m, p.M - 1) * p.K + k);
    }
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
    // Long layers: the channels past the register pass, a pass at a time, before the weights are asked for (a wait
    // for a load waits for every older one).  The loads of a pass are issued together and waited for inside one asm statement: with
    // ordinary loads in a loop behind the weight requests the compiler put a wait for every outstanding load, the
    // weights included, in front of the barrier, the sums and the walk of every layer.
    for (int k8 = tid + NT; k8 < k8_hi; k8 += NT) {
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
    // the (scale, zero) table as a buffer: lane (column n16, lane block lbv) reads the word of its column and of
    // the group of its 32 positions; what is wave-uniform of that (the unit's columns, and the group where all
    // four lane blocks share it) travels in the scalar offset
    const __amdgpu_buffer_rsrc_t szb = tile_buffer((const char *)p.sz, (uint32_t)((size_t)p.G * p.N * 4));
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    auto group_of = [&](uint32_t lb) { return min(__umulhi(lb, p.lbg_magic) + (p.lbg_add ? lb : 0u), (uint32_t)p.G - 1u); };
    uint32_t w[2][PF][BITS], szr[2][PF];
    auto load_w = [&](uint32_t (&wr)[BITS], uint32_t &sr) {
        {
            const uint32_t cols = (uint32_t)(16 * (u0 + rq_u)) * 4u;
            if constexpr (G128) {
                sr = __builtin_amdgcn_raw_buffer_load_b32(szb, (uint32_t)n16 * 4u, group_of(4u * (uint32_t)rq_v) * row_bytes + cols, 0);
            } else {
                sr = __builtin_amdgcn_raw_buffer_load_b32(
                    szb, group_of(4u * (uint32_t)rq_v + (uint32_t)lbv) * row_bytes + (uint32_t)n16 * 4u, cols, 0);
            }
        }
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
    for (int u = 0; u < PF; u++) load_w(w[0][u], szr[0][u]);
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(w[1][u], szr[1][u]);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. stage x in position order -----------------------------------------------------------------------
    if (tid < 16) ((uint32_t *)(smem + zero_off))[tid] = 0u;
    for (int i = p.K + tid; i < span; i += NT)   // the padding of the last virtual block reads as zeros
#pragma unroll
        for (int m = 0; m < MR; m++) xl[m * span + i] = (_Float16)0;
    if (tid < k8_hi) scatter8(8 * tid, kq, xq);
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
    const uint32_t red_lane = (uint32_t)((const unsigned char *)red - smem) + (uint32_t)lane * 4u;

    auto load_x = [&](int V, u2 (&xv)[2]) {
        const uint32_t xoff = x_base + x_stride * (uint32_t)V;
        xv[0] = *(const u2 *)(smem + xoff);
        xv[1] = *(const u2 *)(smem + xoff + x_second);
    };
    int cu = first_u, cv = first_v, c_left = n_items;   // (unit, V) of the item being computed, items still to compute
    auto item = [&](const uint32_t (&wr)[BITS], uint32_t sr, const u2 (&xc)[2], u2 (&xn)[2]) {
        const int V = cv, ul = cu;
        // this item's scale and zero point (the word that came with its weights) and sums
        const h2 sze = as_h2(sr);
        const f2 szf = {(float)sze[0], (float)sze[1]};
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
        if constexpr (EXACT) tiled_dequant_exact<BITS>(q, sr);
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
    auto chunk = [&](int c, uint32_t (&wc)[PF][BITS], const uint32_t (&sc)[PF], auto all_c) {
        constexpr bool ALL = decltype(all_c)::value;
        [&]<int... U>(std::integer_sequence<int, U...>) {
            ((ALL || c + U < n_items ? item(wc[U], sc[U], xr[U & 1], xr[(U + 1) & 1]) : (void)0), ...);
        }(std::make_integer_sequence<int, PF>{});
    };
    int c = 0;
    for (; c + 2 * PF <= n_items; c += 2 * PF) {
        chunk(c, w[0], szr[0], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(w[0][u], szr[0][u]);
        __builtin_amdgcn_sched_barrier(0);
        chunk(c + PF, w[1], szr[1], std::true_type{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; u++) load_w(w[1][u], szr[1][u]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (c < n_items) {
        chunk(c, w[0], szr[0], std::false_type{});
        chunk(c + PF, w[1], szr[1], std::false_type{});
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
    {   // the kernel works the number of groups out from what it is handed: it must come out as given
        const uint32_t lbs = (uint32_t)p.K >> 5;
        const uint32_t groups = (uint32_t)(((unsigned long long)lbs * p.lbg_magic) >> 32) + (p.lbg_add ? lbs : 0u);
        if ((int)groups != p.G || p.M > 255 || plan.grid_x < 1 || plan.grid_x >= (1 << 15) || p.units > (1 << 16))
            return GPTQ_HIP_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x), dim3(1024), plan.lds_bytes, stream, p.x, p.kinv, p.qtile, p.sz, p.K, p.N,
                       (uint32_t)p.M | ((uint32_t)p.lbg_add << 8) | ((uint32_t)plan.grid_x << 9), p.lbg_magic, p.y, p.bias);
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
