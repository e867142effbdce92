// STREAM kernel family: the matmul for M >= 2 (batched decoding and prompt processing).
//
// Up to three launches per call.
//
// 1. pack_kernel (M > 16) rewrites x [M, K] into the order the matrix instruction wants it: for
//    every block of 32 input channels and every 16-row tile, the 64 x 16 bytes that the 64 lanes
//    of a wave hand to v_mfma_f32_16x16x32_f16 as its A operand, lane after lane (1 KiB per
//    fragment), with the 8 values of a lane already in the slot order in which the weight
//    codes leave the unpack.  Rows past M and channels past K are written as zeros, and the
//    channel range is padded to what the matmul waves walk.  It also writes, per block and
//    lane group, the byte offsets of the (scale, zero) table rows of those channels.
//    x is tiny next to the weights, so this pass is cheap; what it buys is that the matmul
//    reads its activations with plain, fully coalesced 16-byte loads: no LDS staging, no
//    barriers in the main loop, no address arithmetic per row, and no L2 channel camping
//    (rows of x are K * 2 bytes apart, which maps a tall narrow tile onto few channels).
//
// 2. stream_kernel: a workgroup owns 64 columns and one block of 16 * RT rows; its waves split
//    the workgroup's K range and never talk to each other until the end, where they add
//    their tiles through LDS in a fixed tree.  A wave unpacks every weight of its range
//    exactly once, dequantises it exactly as the reference does (fp16(scale * (q - zero)), one
//    rounding) into the B operand, and multiplies it with the RT A fragments of the block.
//    Weights, group offsets and A fragments arrive through register rings that are refilled
//    right after use; two waves per SIMD cover what latency is left.
//    The (scale, zero) pairs of the 64 columns live in LDS, [groups][64] + padding.
//    stream_direct_kernel is the same walk for one row tile (M <= 16) without the pack pass:
//    its lanes read x and g_idx themselves.
//
// 3. reduce_kernel (split_k > 1): the workgroups along K leave fp32 tiles in the workspace; this
//    pass adds them in split order, adds the bias and writes y.
// grid of the matmul = (column tiles, split_k, m blocks), block = 64 * waves_k.
#include "gptq_device.h"

namespace gptq {

namespace {

// code of slot s of a lane block, as compile-time tables (SLOT4 / SLOT3 of gptq_unpack.h)
template <int BITS>
__device__ __forceinline__ constexpr int code_of_slot(int s)
{
    return BITS == 4 ? SLOT4[s] : SLOT3[s];
}

}  // namespace

template <int BITS>
__global__ __launch_bounds__(256) void pack_kernel(const Params p)
{
    using F = Fmt<BITS>;
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    const int lane = gid & 63;
    const uint32_t frag = gid >> 6;  // (step, row tile)
    if (frag >= (uint32_t)p.steps_pad * (uint32_t)p.rt_total) return;
    const int s = frag / p.rt_total;
    const int rtg = frag - s * p.rt_total;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int row = 16 * rtg + li;
    const int k0 = F::KSTEP * s + F::KLANE * lq;  // the lane block is whole: K is a multiple of 32
    const bool live = row < p.M && k0 < p.K;

    _Float16 in[F::KLANE];
#pragma unroll
    for (int v = 0; v < F::KLANE / 8; v++) {
        u4 raw = {0u, 0u, 0u, 0u};
        if (live) raw = *(const u4 *)((const _Float16 *)p.x + (size_t)row * p.K + k0 + 8 * v);
        const h8 h = __builtin_bit_cast(h8, raw);
#pragma unroll
        for (int e = 0; e < 8; e++) in[8 * v + e] = h[e];
    }
#pragma unroll
    for (int nb = 0; nb < F::NB; nb++) {
        h8 o;
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = in[code_of_slot<BITS>(8 * nb + j)];
        const size_t f = ((size_t)(s * F::NB + nb) * p.rt_total + rtg) * 64 + lane;
        *(h8 *)((char *)p.xpack + f * 16) = o;
    }

    if (rtg == 0 && li == 0) {
        if (p.act_table) {
            // one table row offset per weight, in slot order
#pragma unroll
            for (int nb = 0; nb < F::NB; nb++) {
                int o[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int k = min(k0 + code_of_slot<BITS>(8 * nb + j), p.K - 1);
                    int g = p.g_idx ? p.g_idx[k] : k / p.group_size;
                    g = min(max(g, 0), p.G - 1);
                    o[j] = g * kStreamTableRow;
                }
                int *dst = p.gpack + ((size_t)(s * F::NB + nb) * 4 + lq) * 8;
                *(int4 *)dst = make_int4(o[0], o[1], o[2], o[3]);
                *(int4 *)(dst + 4) = make_int4(o[4], o[5], o[6], o[7]);
            }
        } else {
            // contiguous groups no narrower than a lane block: one row per lane block
            p.gpack[s * 4 + lq] = (min(k0, p.K - 1) / p.group_size) * kStreamTableRow;
        }
    }
}


// ---- pieces shared by the two matmul kernels of this file ---------------------------------------

// Stages (scale, zero) of groups g_lo .. g_hi x the 64 columns from n_blk on into LDS rows of
// kStreamTableRow bytes (row 0 = g_lo).  Four items per thread at a time so their loads overlap.
template <int BITS>
__device__ __forceinline__ void stage_table(const Params &p, int g_lo, int g_hi, int n_blk, int tid)
{
    constexpr int TROW = kStreamTableRow;
    const _Float16 *scales = (const _Float16 *)p.scales;
    const int zwords = p.N / 32 * BITS;
    const int tab_items = (g_hi - g_lo + 1) * 16;  // four columns of one group each
    for (int base = tid; base < tab_items; base += 4 * (int)blockDim.x) {
        h4 s4[4];
        uint32_t za[4], zb[4];
        int nn[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx = min(base + u * (int)blockDim.x, tab_items - 1);
            const int gr = idx >> 4;
            nn[u] = min(n_blk + 4 * (idx & 15), p.N - 4);
            const uint32_t g = (uint32_t)(g_lo + gr);
            s4[u] = *(const h4 *)((const char *)scales + (g * (uint32_t)p.N + (uint32_t)nn[u]) * 2u);
            load_zero_words<BITS>(p.qzeros, g * (uint32_t)zwords, nn[u], za[u], zb[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx = base + u * (int)blockDim.x;
            if (idx < tab_items) {
                float z[4];
                zeros_from_words<BITS>(za[u], zb[u], nn[u], z);
                u4 e;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const h2 sz = {s4[u][c], (_Float16)z[c]};
                    e[c] = as_u32(sz);
                }
                *(u4 *)(smem + (size_t)(idx >> 4) * TROW + (idx & 15) * 16) = e;
            }
        }
    }
}

// B operands of one block: the reference's weights fp16(scale * (q - zero)) of 8 slots x 4 column
// sets from the biased codes bqn[c] (base + q).  (base + q) - (base + zero) is exact, so the one
// rounding is the product's.  eoff[s]: LDS byte offset of the (scale, zero) entries of slot s
// (ACT); erow[c]: the entry shared by all slots.
template <int BITS, bool ACT>
__device__ __forceinline__ void dequant_block(const u4 (&bqn)[4], const uint32_t (&eoff)[8], const u4 &erow,
                                              h8 (&bop)[4])
{
    // int3 tiles are the ones short of registers: they take the table in two rounds of four slots
    constexpr int ROUNDS = BITS == 3 ? 2 : 1;
    constexpr int SPR = 8 / ROUNDS;  // slots per round
    u4 wv[4];
#pragma unroll
    for (int round = 0; round < ROUNDS; round++) {
        u4 ent[SPR];
        if constexpr (ACT) {
#pragma unroll
            for (int s = 0; s < SPR; s++) ent[s] = *(const u4 *)(smem + eoff[SPR * round + s]);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) {
#pragma unroll
            for (int rr = 0; rr < SPR / 2; rr++) {
                const int r = (SPR / 2) * round + rr;
                // (scale, zero) of the two slots of register r: low halves / high halves
                const uint32_t ea = ACT ? ent[2 * rr][c] : erow[c];
                const uint32_t eb = ACT ? ent[2 * rr + 1][c] : erow[c];
                const h2 s2 = as_h2(__builtin_amdgcn_perm(eb, ea, 0x05040100u));
                const h2 z2 = as_h2(__builtin_amdgcn_perm(eb, ea, 0x07060302u));
                const float ba = BITS == 4 ? BASE4[2 * r] : BASE3[2 * r];
                const float bb = BITS == 4 ? BASE4[2 * r + 1] : BASE3[2 * r + 1];
                const h2 zb = z2 + (h2){(_Float16)ba, (_Float16)bb};  // exact: small integers
                wv[c][r] = as_u32((as_h2(bqn[c][r]) - zb) * s2);
            }
        }
        // keeps the next round's table reads below this point (everything else may cross)
        if constexpr (ACT && ROUNDS > 1) __builtin_amdgcn_sched_barrier(0x067f);
    }
#pragma unroll
    for (int c = 0; c < 4; c++) bop[c] = __builtin_bit_cast(h8, wv[c]);
}

// The waves of the workgroup add their tiles through LDS in a fixed tree; wave 0 ends up with the sum.
template <int RT>
__device__ __forceinline__ void reduce_waves(f4 (&acc)[RT][4], int wave, int WK, int lane)
{
    f4 *red = (f4 *)smem;  // [WK / 2][RT * 4 tiles][64 lanes] of f4, reuses the table's bytes
    for (int stride = WK >> 1; stride >= 1; stride >>= 1) {
        lds_barrier();  // the table, or the previous round, is no longer read
        if (wave >= stride && wave < 2 * stride) {
            f4 *dst = red + (size_t)(wave - stride) * (RT * 4) * 64 + lane;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int c = 0; c < 4; c++) dst[(rt * 4 + c) * 64] = acc[rt][c];
        }
        lds_barrier();
        if (wave < stride) {
            const f4 *src = red + (size_t)wave * (RT * 4) * 64 + lane;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int c = 0; c < 4; c++) acc[rt][c] += src[(rt * 4 + c) * 64];
        }
    }
}

// Epilogue of wave 0: acc[rt][c][v] is y[m0 + 16 rt + 4 q + v][n0 + c]; bias and fp16, or, when K
// is split over workgroups, the fp32 tile into the workspace.
template <int RT>
__device__ __forceinline__ void write_out(const Params &p, f4 (&acc)[RT][4], bool owner, int m0, int rows_here,
                                          int n0, int lq, int split)
{
    const _Float16 *bias = (const _Float16 *)p.bias;
    f4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias && owner) {
        const h4 b4 = *(const h4 *)(bias + n0);
        bv = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    _Float16 *y = (_Float16 *)p.y;
    if (p.split_k == 1) {
        if (owner) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int row = 16 * rt + 4 * lq + v;
                    if (row < rows_here) {
                        h4 o;
#pragma unroll
                        for (int c = 0; c < 4; c++) o[c] = (_Float16)(acc[rt][c][v] + bv[c]);
                        *(h4 *)(y + (size_t)(m0 + row) * p.N + n0) = o;
                    }
                }
            }
        }
        return;
    }
    // split_k > 1: the fp32 tile goes to the workspace with plain stores; reduce_kernel, launched
    // right behind this kernel on the same stream, adds the split_k tiles in order and writes y.
    // (The in-kernel alternative, a counter and the last workgroup summing, costs three dependent
    // round trips to device-coherent memory and slow 64-bit coherent stores for tall tiles.)
    if (owner) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * rt + 4 * lq + v;
                if (row < rows_here) {
                    const f4 o = {acc[rt][0][v], acc[rt][1][v], acc[rt][2][v], acc[rt][3][v]};
                    *(f4 *)(p.partial + ((size_t)split * p.M + (m0 + row)) * p.N + n0) = o;
                }
            }
        }
    }
}

// y = fp16(sum over split of partial[split] (+ bias)), four columns per thread, in split order.
__global__ __launch_bounds__(256) void reduce_kernel(const Params p)
{
    const uint32_t q = blockIdx.x * 256u + threadIdx.x;
    const uint32_t nq = (uint32_t)p.N / 4u;
    if (q >= (uint32_t)p.M * nq) return;
    const uint32_t row = q / nq;
    const uint32_t col = 4u * (q - row * nq);
    f4 sum = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
        const h4 b4 = *(const h4 *)((const _Float16 *)p.bias + col);
        sum = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    for (int s = 0; s < p.split_k; s++) sum += *(const f4 *)(p.partial + ((size_t)s * p.M + row) * p.N + col);
    h4 o;
#pragma unroll
    for (int c = 0; c < 4; c++) o[c] = (_Float16)sum[c];
    *(h4 *)((_Float16 *)p.y + (size_t)row * p.N + col) = o;
}

// Global loads return in order (one counter), so a wait for any load also waits for every older
// one.  The main loop therefore issues its loads in the order it consumes them and keeps all of
// them the same distance ahead: in step s the weights of step s + PF are requested first, then,
// tile by tile as the matrix instructions retire them, the A fragments AD blocks ahead.  Nothing
// is ever waited for that was requested less than a whole ring ago, which is what keeps
// dozens of loads in flight per wave and covers the HBM latency.  The barriers below stop the
// compiler from moving loads across those points (everything else may cross).
#define STREAM_PIN_LOADS() __builtin_amdgcn_sched_barrier(0x07cf)

template <int BITS, int RT, bool ACT>
__global__ __launch_bounds__(512) void stream_kernel(const Params p)
{
    using F = Fmt<BITS>;
    constexpr int PF = stream_pf(BITS);  // steps the weight loads run ahead
    constexpr int AD = kStreamRingBlocks;  // blocks the A fragments (and table offsets) run ahead
    static_assert((PF * F::NB) % AD == 0, "the unrolled group must be whole turns of the A ring");
    constexpr int TROW = kStreamTableRow;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps the K walk in scalar registers
    const int WK = p.waves_k;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int n_blk = blockIdx.x * 64;
    const int col_l = 4 * li;
    const int n0 = n_blk + col_l;
    const bool n_ok = n0 < p.N;
    const int rt0 = blockIdx.z * RT;
    const int m0 = 16 * rt0;
    const int rows_here = min(16 * RT, p.M - m0);
    const int split = blockIdx.y;
    // every wave walks exactly wave_steps steps of the padded step range; past K the packed x is zero
    const int s_begin = split * WK * p.wave_steps;
    const int ws = s_begin + wave * p.wave_steps;
    const int prows = p.K / (BITS == 4 ? 8 : 32);

    // ---- register rings --------------------------------------------------------------------
    // Addresses are a wave-uniform base (step or block number, in scalar registers) plus a
    // per-lane offset that never changes, so the loop spends no vector instructions on them.
    // The packed buffers are padded past their end by the depth of the rings, which lets the
    // refills at the end of a wave's range run unclamped (what they fetch is never used).
    const uint32_t n_ld = (uint32_t)min(n0, p.N - 4);
    u4 w[PF][F::WORDS];
    int grow[PF];
    const uint32_t w_step_bytes = 4u * F::WORDS * (uint32_t)p.N * 4u;  // four packed rows (int3: 3-word blocks)
    const uint32_t w_lane = ((uint32_t)lq * F::WORDS * (uint32_t)p.N + n_ld) * 4u;
    const int last_step = p.steps_total - 1;
    auto load_w = [&](int st, u4 (&wr)[F::WORDS], int &gr) {
        const int st_c = min(st, last_step);  // scalar: steps past K read the last step (their x is zero)
        const char *base = (const char *)p.qweight + (size_t)st_c * w_step_bytes;
        uint32_t voff = w_lane;
        if constexpr (BITS == 3) {
            // K need not be a multiple of 128: lane groups past the last 3-word block repeat it
            const int lq_c = min(lq, prows - 1 - 4 * st_c);
            voff = ((uint32_t)lq_c * F::WORDS * (uint32_t)p.N + n_ld) * 4u;
        }
#pragma unroll
        for (int wd = 0; wd < F::WORDS; wd++) {
            wr[wd] = __builtin_nontemporal_load((const u4 *)(base + (voff + (uint32_t)wd * (uint32_t)p.N * 4u)));
        }
        if constexpr (!ACT) gr = *(const int *)((const char *)p.gpack + (size_t)st * 16 + (uint32_t)lq * 4u);
    };
    const uint32_t a_block_bytes = (uint32_t)p.rt_total * 1024u;
    const uint32_t a_lane = (uint32_t)rt0 * 1024u + (uint32_t)lane * 16u;
    auto load_a = [&](int b, int rt) -> h8 {
        const char *base = (const char *)p.xpack + (size_t)b * a_block_bytes;
        return __builtin_bit_cast(h8, *(const u4 *)(base + (a_lane + (uint32_t)rt * 1024u)));
    };
    auto load_go = [&](int b, u4 (&g)[2]) {
        const char *base = (const char *)p.gpack + (size_t)b * 128;
        g[0] = *(const u4 *)(base + (uint32_t)lq * 32u);
        g[1] = *(const u4 *)(base + ((uint32_t)lq * 32u + 16u));
    };
    h8 a[AD][RT];
    u4 go[ACT ? AD : 1][2];
    const int b_begin = ws * F::NB;
    // prologue in consumption order: step by step, weights first, then that step's blocks
#pragma unroll
    for (int u = 0; u < PF; u++) {
        load_w(ws + u, w[u], grow[u]);
#pragma unroll
        for (int nb = 0; nb < F::NB; nb++) {
            const int bi = u * F::NB + nb;
            if (bi < AD) {
                if constexpr (ACT) load_go(b_begin + bi, go[bi]);
#pragma unroll
                for (int rt = 0; rt < RT; rt++) a[bi][rt] = load_a(b_begin + bi, rt);
            }
        }
    }
    STREAM_PIN_LOADS();

    // ---- (scale, zero) table of the 64 columns: all groups under a g_idx, else those of the
    //      workgroup's K range (row 0 = the first of them) ---------------------------------
    const int k_lo = min(s_begin * F::KSTEP, p.K - 1);
    const int k_hi = min((s_begin + WK * p.wave_steps) * F::KSTEP, p.K) - 1;
    const int g_lo = ACT ? 0 : k_lo / p.group_size;
    const int g_hi = ACT ? p.G - 1 : min(p.G - 1, max(k_hi, k_lo) / p.group_size);
    stage_table<BITS>(p, g_lo, g_hi, n_blk, tid);
    const int tab_bias = col_l * 4 - g_lo * TROW;  // this lane's four columns, rows counted from g_lo

    f4 acc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[rt][c] = (f4){0.f, 0.f, 0.f, 0.f};

    const uint32_t magic_a = opaque_vgpr(BITS == 4 ? MAGIC4_LO : MAGIC3_EVEN);
    const uint32_t magic_b = opaque_vgpr(BITS == 4 ? MAGIC4_HI : MAGIC3_ODD);

    lds_barrier();  // the table is complete

    // ---- main loop: nothing in it is conditional -------------------------------------------
    for (int i0 = 0; i0 < p.wave_steps; i0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const int st = ws + i0 + u;
            u4 bq[4][F::NB];
            if constexpr (BITS == 4) {
#pragma unroll
                for (int c = 0; c < 4; c++) biased4(w[u][0][c], bq[c], magic_a, magic_b);
            }
            u4 erow = {0u, 0u, 0u, 0u};
            if constexpr (!ACT) erow = *(const u4 *)(smem + (uint32_t)(grow[u] + tab_bias));
            if constexpr (BITS == 4) {
                __builtin_amdgcn_sched_barrier(0);
                load_w(st + PF, w[u], grow[u]);  // refill this ring slot
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int nb = 0; nb < F::NB; nb++) {
                const int b = st * F::NB + nb;
                const int slot = (u * F::NB + nb) % AD;  // compile-time after unrolling
                if constexpr (BITS == 3) {
                    // unpacked block by block: all sixteen registers per column at once do not fit
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        biased3_block(w[u][0][c], w[u][1][c], w[u][2][c], nb, bq[c][nb], magic_a, magic_b);
                }
                h8 bop[4];
                {
                    uint32_t eoff[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
                    if constexpr (ACT) {
#pragma unroll
                        for (int s = 0; s < 8; s++) {
                            eoff[s] = (s < 4 ? go[slot][0][s & 3] : go[slot][1][s & 3]) + (uint32_t)tab_bias;
                        }
                    }
                    // refill with the offsets of the block AD ahead; where the request is issued
                    // relative to the table reads is measured per width (int3 before, int4 after)
                    if constexpr (ACT && BITS == 3) load_go(b + AD, go[slot]);
                    u4 bqn[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) bqn[c] = bq[c][nb];
                    dequant_block<BITS, ACT>(bqn, eoff, erow, bop);
                    if constexpr (ACT && BITS == 4) load_go(b + AD, go[slot]);
                }
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        acc[rt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[slot][rt], bop[c], acc[rt][c], 0, 0, 0);
                    }
                    a[slot][rt] = load_a(b + AD, rt);  // refill: this tile of the block AD ahead
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (BITS == 3) {
                load_w(st + PF, w[u], grow[u]);  // refill this ring slot (its words were needed until here)
                STREAM_PIN_LOADS();
            }
        }
    }

    reduce_waves<RT>(acc, wave, WK, lane);
    write_out<RT>(p, acc, wave == 0 && n_ok, m0, rows_here, n0, lq, split);
}


// ---- M <= 16 without the pack pass ------------------------------------------------------------
// One row tile: lane (i, q) reads the 8 (int4) / 32 (int3) channels of ITS lane block straight
// from row min(i, M - 1) of x, and the g_idx entries of the same channels, in natural order, and
// sorts them into slot order in registers (byte permutes for x, plain renaming for the 32-bit
// group numbers).  Both ride in rings of the same depth as the weights, requested right after
// them, so the in-order rule of the loads above holds.  Rows past M compute values nobody
// stores; lane blocks past K are zeroed.
template <int N>
__device__ __forceinline__ uint32_t pick_halves(const uint32_t (&r)[N], int ha, int hb)
{
    const uint32_t sel = ((ha & 1) ? 0x0302u : 0x0100u) | (((hb & 1) ? 0x0706u : 0x0504u) << 16);
    return __builtin_amdgcn_perm(r[hb >> 1], r[ha >> 1], sel);
}

template <int BITS, bool ACT>
__global__ __launch_bounds__(512) void stream_direct_kernel(const Params p)
{
    using F = Fmt<BITS>;
    constexpr int PF = stream_pf(BITS);
    constexpr int TROW = kStreamTableRow;
    constexpr int XV = F::KLANE / 8;  // 16-byte vectors of x per lane block
    constexpr int GV = F::KLANE / 4;  // 16-byte vectors of g_idx per lane block
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int WK = p.waves_k;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int n_blk = blockIdx.x * 64;
    const int col_l = 4 * li;
    const int n0 = n_blk + col_l;
    const bool n_ok = n0 < p.N;
    const int split = blockIdx.y;
    const int s_begin = split * WK * p.wave_steps;
    const int ws = s_begin + wave * p.wave_steps;
    const int prows = p.K / F::KLANE;  // lane blocks along K
    const int last_step = p.steps_total - 1;

    const uint32_t n_ld = (uint32_t)min(n0, p.N - 4);
    const uint32_t x_row = (uint32_t)min(li, p.M - 1) * (uint32_t)p.K * 2u;
    u4 w[PF][F::WORDS];
    u4 xr[PF][XV];
    u4 gr[ACT ? PF : 1][ACT ? GV : 1];
    auto load_step = [&](int st, u4 (&wr)[F::WORDS], u4 (&xv)[XV], u4 (&gv)[ACT ? GV : 1]) {
        const int st_c = min(st, last_step);
        const int lq_c = min(lq, prows - 1 - 4 * st_c);  // lane blocks past K repeat the last one
        const uint32_t blk = (uint32_t)(4 * st_c + lq_c);
        const char *wbase = (const char *)p.qweight + (size_t)st_c * (4u * F::WORDS * (uint32_t)p.N * 4u);
        const uint32_t woff = ((uint32_t)lq_c * F::WORDS * (uint32_t)p.N + n_ld) * 4u;
#pragma unroll
        for (int wd = 0; wd < F::WORDS; wd++) {
            wr[wd] = __builtin_nontemporal_load((const u4 *)(wbase + (woff + (uint32_t)wd * (uint32_t)p.N * 4u)));
        }
        const uint32_t k0 = blk * F::KLANE;
#pragma unroll
        for (int v = 0; v < XV; v++) xv[v] = *(const u4 *)((const char *)p.x + (x_row + (k0 + 8u * v) * 2u));
        if constexpr (ACT) {
#pragma unroll
            for (int v = 0; v < GV; v++) gv[v] = *(const u4 *)((const char *)p.g_idx + (k0 + 4u * v) * 4u);
        }
    };
#pragma unroll
    for (int u = 0; u < PF; u++) load_step(ws + u, w[u], xr[u], gr[ACT ? u : 0]);
    STREAM_PIN_LOADS();

    const int k_lo = min(s_begin * F::KSTEP, p.K - 1);
    const int k_hi = min((s_begin + WK * p.wave_steps) * F::KSTEP, p.K) - 1;
    const int g_lo = ACT ? 0 : k_lo / p.group_size;
    const int g_hi = ACT ? p.G - 1 : min(p.G - 1, max(k_hi, k_lo) / p.group_size);
    stage_table<BITS>(p, g_lo, g_hi, n_blk, tid);
    const int tab_bias = col_l * 4 - g_lo * TROW;

    f4 acc[1][4];
#pragma unroll
    for (int c = 0; c < 4; c++) acc[0][c] = (f4){0.f, 0.f, 0.f, 0.f};
    const uint32_t magic_a = opaque_vgpr(BITS == 4 ? MAGIC4_LO : MAGIC3_EVEN);
    const uint32_t magic_b = opaque_vgpr(BITS == 4 ? MAGIC4_HI : MAGIC3_ODD);
    lds_barrier();  // the table is complete

    for (int i0 = 0; i0 < p.wave_steps; i0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const int st = ws + i0 + u;
            const bool live = 4 * st + lq < prows;  // this lane's block lies inside K
            // everything that reads the ring slot comes first, then the slot is refilled
            u4 bq[4][F::NB];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                if constexpr (BITS == 4) {
                    biased4(w[u][0][c], bq[c], magic_a, magic_b);
                } else {
                    biased3(w[u][0][c], w[u][1][c], w[u][2][c], bq[c], magic_a, magic_b);
                }
            }
            uint32_t xs[F::KLANE / 2];  // natural order, two channels per register
#pragma unroll
            for (int v = 0; v < XV; v++)
#pragma unroll
                for (int e = 0; e < 4; e++) xs[4 * v + e] = live ? xr[u][v][e] : 0u;
            h8 a[F::NB];
#pragma unroll
            for (int nb = 0; nb < F::NB; nb++) {
                u4 f;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    f[r] = pick_halves(xs, code_of_slot<BITS>(8 * nb + 2 * r), code_of_slot<BITS>(8 * nb + 2 * r + 1));
                }
                a[nb] = __builtin_bit_cast(h8, f);
            }
            uint32_t go[ACT ? F::KLANE : 1];  // table row offsets in slot order
            u4 erow = {0u, 0u, 0u, 0u};
            if constexpr (ACT) {
#pragma unroll
                for (int s = 0; s < F::KLANE; s++) {
                    const int cd = code_of_slot<BITS>(s);
                    const int g = (int)gr[u][cd >> 2][cd & 3];
                    go[s] = (uint32_t)(min(max(g, 0), p.G - 1) * TROW + tab_bias);
                }
            } else {
                const uint32_t r = (uint32_t)min(4 * st + lq, prows - 1);
                const uint32_t g = __umulhi(r, p.gdiv_magic) + (p.gdiv_add ? r : 0u);
                erow = *(const u4 *)(smem + (g * TROW + (uint32_t)tab_bias));
            }
            // Nothing may cross these two points: with only the loads pinned the scheduler hoists the
            // ring reads (and with them the waits) of all PF steps above the first refill, so every
            // group of PF steps waits for its loads, computes, and only then requests the next group.
            // (int3 under an activation order keeps the looser pin: with the order fixed it spills 41
            // registers and runs 18 -> 25 us at M = 8.)
            if constexpr (BITS == 3 && ACT) {
                STREAM_PIN_LOADS();
            } else {
                __builtin_amdgcn_sched_barrier(0);
            }
            load_step(st + PF, w[u], xr[u], gr[ACT ? u : 0]);
            if constexpr (BITS == 3 && ACT) {
                STREAM_PIN_LOADS();
            } else {
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int nb = 0; nb < F::NB; nb++) {
                uint32_t eoff[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
                if constexpr (ACT) {
#pragma unroll
                    for (int s = 0; s < 8; s++) eoff[s] = go[8 * nb + s];
                }
                u4 bqn[4];
#pragma unroll
                for (int c = 0; c < 4; c++) bqn[c] = bq[c][nb];
                h8 bop[4];
                dequant_block<BITS, ACT>(bqn, eoff, erow, bop);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    acc[0][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[nb], bop[c], acc[0][c], 0, 0, 0);
                }
            }
        }
    }
    reduce_waves<1>(acc, wave, WK, lane);
    write_out<1>(p, acc, wave == 0 && n_ok, 0, min(16, p.M), n0, lq, split);
}

static int launch_reduce(const Params &p, hipStream_t stream)
{
    if (p.split_k == 1) return GPTQ_HIP_OK;
    const uint32_t quads = (uint32_t)p.M * ((uint32_t)p.N / 4u);
    hipLaunchKernelGGL(reduce_kernel, dim3((quads + 255u) / 256u), dim3(256), 0, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, int RT, bool ACT>
static int launch_stream_one(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = stream_kernel<BITS, RT, ACT>;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    const dim3 grid_d(plan.grid_x, plan.grid_y, plan.grid_z);
    if (p.direct) {
        if constexpr (RT == 1) {
            auto kd = stream_direct_kernel<BITS, ACT>;
            hipLaunchKernelGGL(kd, grid_d, dim3(plan.block), plan.lds_bytes, stream, p);
            if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
            return launch_reduce(p, stream);
        } else {
            return GPTQ_HIP_ERR_BAD_ARG;
        }
    }
    const uint32_t pack_threads = (uint32_t)p.steps_pad * (uint32_t)p.rt_total * 64u;
    hipLaunchKernelGGL(pack_kernel<BITS>, dim3((pack_threads + 255u) / 256u), dim3(256), 0, stream, p);
    if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    const dim3 grid(plan.grid_x, plan.grid_y, plan.grid_z);
    hipLaunchKernelGGL(kern, grid, dim3(plan.block), plan.lds_bytes, stream, p);
    if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ERR_LAUNCH;
    return launch_reduce(p, stream);
}

template <int BITS, bool ACT>
static int launch_stream_rt(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    switch (plan.row_tiles) {
        case 1: return launch_stream_one<BITS, 1, ACT>(p, plan, stream);
        case 2: return launch_stream_one<BITS, 2, ACT>(p, plan, stream);
        case 4: return launch_stream_one<BITS, 4, ACT>(p, plan, stream);
        default: return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

int launch_stream(const Params &p, int bits, const gptq_hip_plan &plan, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    if (bits == 4) {
        return p.act_table ? launch_stream_rt<4, true>(p, plan, stream) : launch_stream_rt<4, false>(p, plan, stream);
    }
    return p.act_table ? launch_stream_rt<3, true>(p, plan, stream) : launch_stream_rt<3, false>(p, plan, stream);
}

}  // namespace gptq
