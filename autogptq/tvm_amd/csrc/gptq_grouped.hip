// GROUPED kernel family: decode-size products (M of 1 or 2 for any g_idx; 3 or 4 with contiguous groups).
//
// Instead of looking a scale and zero up for every weight, the rows of the MFMA are
// expanded by group:  row (m, g) of the activation operand holds x[m, k] where
// g_idx[k] == g and 0 elsewhere.  The MFMA then yields, per group,
//     P[m, g, n] = sum_{k in g} x[m, k] * q[k, n]        (q = the raw integer code)
// and an extra MFMA against a column of ones yields X[m, g] = sum_{k in g} x[m, k].
// The scales and zero points are applied once per group at the end:
//     y[m, n] = sum_g scales[g, n] * (P[m, g, n] - zero[g, n] * X[m, g]).
// Per weight the vector ALU only unpacks the code; nothing is gathered, whatever the
// order of g_idx.  The fp16 rounding of each dequantised weight that the reference
// performs is not reproduced here (products are exact, sums are fp32), so y differs
// from the reference by its rounding noise, far inside the 1e-2 tolerance.
//
// Work split: a workgroup owns 64 * waves_n columns and one K range (all of K when
// split_k == 1); its waves_k waves along K each take a share of that range, keep their
// weight loads one (int3), four (int4, lean operand) or eight (int4, tiles) steps ahead of the matrix
// instructions, and meet in LDS for the reduction.  With split_k == 1 nothing crosses workgroups.
//
// LDS holds the expanded activation operand of the workgroup's K range, laid out as
// the MFMA wants it: a tile is 16 rows x 8 slots of fp16 = 256 bytes, lane i reads its
// 16 bytes at i*16.  It is zero-filled and then scattered into, one 2-byte store per
// (m, k).  Two layouts:
//   dense   : one tile per 16 groups (row = g - first group of the consuming wave), M * TPM tiles per 8 slots;
//   compact : for 17..32 groups, ONE tile per m with row = g % 16, plus a 16-byte mask
//             per 8 slots saying which slots belong to groups < 16.  The two row tiles
//             are that tile AND mask / AND NOT mask: half the LDS, so K = 4096 with 32
//             groups fits one workgroup.
//
// LITE: with contiguous groups that are whole lane blocks (8 channels int4, 32 int3) all 8 slots
// of an operand tile belong to one group, so the tile is "x in row r, zeros elsewhere".  LDS then
// holds just x in unpack order (2 bytes per channel instead of 32) plus 16 zero bytes: a lane reads
// x when its row is the block's group and the zeros otherwise.  Nothing but the positions past the end
// of K is zero-filled (instead of 128 KB of tiles at K = 4096), which the scatter never writes, so one
// barrier (after the scatter) suffices; the scatter's 2-byte stores spread over the banks instead of
// hitting the two banks of one tile row.  Used for int3, and for int4 where one workgroup holds all
// of K (grouped_lite in gptq_internal.h).
//
// Sorted layers: when the loader has sorted the channels of an activation-order layer by
// group (qweight rows permuted, p.kmap saying where each original channel went), the groups
// are contiguous for the weight stream and only the scatter of x follows the map: every
// workgroup walks all of x and keeps the channels whose sorted position falls in its K range
// (p.kmap: one memory round trip), or looks up where the x of each of its positions comes from
// (p.xsrc: two dependent round trips, but no scatter work on channels of other K ranges; the
// host picks it when K is split and long).
//
// Wave-private staging (WAVEX: lean operand, no channel map, at most 512 channels per wave): every
// wave loads and stages the x of its own K range, so the prologue has no workgroup barrier at all.
// Packed rows (PACK, on top of WAVEX, at most four groups per wave): row 4 m + g of an operand tile
// holds activation row m for group g, so up to four activation rows cost the matrix instructions of
// one, up to eight those of two.
#include "gptq_device.h"

namespace gptq {

__device__ __forceinline__ h8 and_h8(h8 a, u4 m)
{
    u4 v = __builtin_bit_cast(u4, a);
    v &= m;
    return __builtin_bit_cast(h8, v);
}

// TPM = row tiles (of 16 groups) per activation row; COMPACT needs TPM == 2.
// WAVEX (lean operand without a channel map, a wave's K range of at most 512 channels): every wave
// stages the x of its own K range itself, so nothing crosses waves before the reduction.
// PACK (WAVEX, at most four groups in a wave's K range, M = 4 rows of which p.M are real): row 4 m + g of
// the ONE operand tile holds x[m] for group g of the wave, so three or four activation rows cost the
// matrix instructions of one; lane group q of the result is activation row q, register v its group v.
template <int BITS, int M, int TPM, bool COMPACT, int NSTEP, bool LITE, bool WAVEX = false, bool PACK = false>
__global__ __launch_bounds__(512) void grouped_kernel(const Params p)
{
    using F = Fmt<BITS>;
    constexpr int ST = COMPACT ? M : M * TPM;    // tiles stored in LDS per 8 slots
    static_assert(!COMPACT || TPM == 2, "compact layout is for two row tiles");
    static_assert(!LITE || (TPM == 1 && !COMPACT), "the lite operand is one row tile of contiguous groups");
    static_assert(!WAVEX || LITE, "wave-private staging is for the lean operand");
    static_assert(!PACK || (WAVEX && (M == 4 || M == 8)), "packed rows: four activation rows x four groups per tile");
    constexpr int MA = PACK ? M / 4 : M;  // operand tiles (and accumulator sets) per row tile
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int WN = p.waves_n;  // 1, 2 or 4
    const int WK = p.waves_k;
    const int nthreads = 64 * WN * WK;  // the block size, without a second trip to the kernel arguments
    const int wn = wave & (WN - 1);
    const int wk = wave >> (WN >> 1);  // log2 of 1, 2, 4
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int BN = 64 * WN;
    const int n0 = blockIdx.x * BN + wn * 64 + 4 * li;
    const bool n_ok = n0 < p.N;
    const int split = blockIdx.y;
    // every wave owns wave_steps consecutive steps (the host made the partition uniform, so no
    // division happens here); ranges past the end of K are cut by s_end
    const int wg_steps = p.wave_steps * WK;
    const int s_begin = split * wg_steps;
    const int s_end = min(s_begin + wg_steps, p.steps_total);
    const int ws = s_begin + wk * p.wave_steps;  // this wave's steps
    const int we = min(ws + p.wave_steps, s_end);
    const int k_base = s_begin * F::KSTEP;
    const int kspan = wg_steps * F::KSTEP;
    const int prows = p.K / (BITS == 4 ? 8 : 32);  // packed rows (int4) or 3-word blocks (int3)
    // contiguous groups: only those inside this K range need rows, counted from the first one
    // (rows are counted per wave: a wave's K range meets few groups, so one row tile usually holds them)
    const int wave_k = p.wave_steps * F::KSTEP;  // channels per wave
    // (the lean operand comes with the lane-block-to-group multiplier, which spares a division here)
    const uint32_t lb0 = (uint32_t)(ws * (F::KSTEP / F::KLANE));  // first lane block of the wave
    const int g_base = LITE ? (int)(__umulhi(lb0, p.gdiv_magic) + (p.gdiv_add ? lb0 : 0u))
                            : (p.g_idx ? 0 : (ws * F::KSTEP) / p.group_size);
    __shared__ int last_flag;
    __shared__ int wave_gb[8];  // sorted layers: first group of each wave along K
    const int32_t *kmap = p.kmap;
    const int32_t *xsrc = p.xsrc;
    auto src_ok = [&](int c) { return (int)min((uint32_t)c, (uint32_t)p.K - 1u); };  // a bad map must not fault
    if constexpr (!LITE) {
        if (kmap && tid < WK) wave_gb[tid] = (k_base + tid * wave_k) / p.group_size;
    }

    const _Float16 *x = (const _Float16 *)p.x;
    const _Float16 *scales = (const _Float16 *)p.scales;
    const int zwords = p.N / 32 * BITS;

    const int nblk8 = kspan / 8;  // 8-slot blocks in the K range
    unsigned char *tiles = smem;
    unsigned char *masks = smem + (size_t)nblk8 * ST * 256;
    float *red = (float *)(masks + (COMPACT ? (size_t)nblk8 * 16 : 0));
    // LITE: x of the K range in unpack order, [M][kspan] fp16, then 16 zero bytes
    _Float16 *xlds = (_Float16 *)smem;
    const uint32_t zero_off = (uint32_t)M * (uint32_t)kspan * 2u;
    if constexpr (LITE) {
        red = (float *)(smem + zero_off + 16);
        if (WAVEX ? lane < 4 : tid < 4) ((uint32_t *)(smem + zero_off))[lane & 3] = 0u;  // WAVEX: every wave writes them
    }

    int qslot[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        constexpr uint64_t words[4] = {quad_slots<BITS>(0), quad_slots<BITS>(1), quad_slots<BITS>(2),
                                       quad_slots<BITS>(3)};
        qslot[e] = (int)((words[e] >> (8 * (tid % (F::KLANE / 4)))) & 0xffu);
    }
    // ---- 1. x and g_idx of the K range: four channels per thread per pass ---------------
    constexpr int QP = 2;  // passes kept in registers so that their loads are the first to return
    const int scan_base = kmap ? 0 : k_base;     // a sorted layer's channels may sit anywhere in x
    const int qpr = (kmap ? p.K : kspan) / 4;    // quads per activation row
    const int nquads = qpr * M;
    // Every load below is unconditional (clamped addresses, results masked where they are used): a
    // load inside a branch makes the number of loads in flight unknown at the next wait, and the
    // compiler then waits for all of them (vmcnt(0)), which serialises x, map and weight latencies.
    // A layer without a map still loads "map" entries (from the packed weights: any readable memory)
    // and ignores them.
    int gq[QP][4];
    h4 xq[QP];
    int4 sq[QP];   // raw map entries (xsrc: the channels of x this thread's positions take)
    bool qv[QP];   // the quad lies inside the rows and channels walked
    const int32_t *mapsrc = xsrc ? xsrc : (kmap ? kmap : (p.g_idx ? p.g_idx : (const int32_t *)p.qweight));
    const bool has_map = kmap != nullptr || p.g_idx != nullptr;
#pragma unroll
    for (int ps = 0; ps < (WAVEX ? 0 : QP); ps++) {
        const int idx = tid + ps * nthreads;
        const int idc = min(idx, nquads - 1);
        const int m = M == 1 ? 0 : idc / qpr;
        const int k = scan_base + 4 * (idc - m * qpr);
        qv[ps] = idx < nquads && k < p.K;  // K % 4 == 0: a quad is inside or outside as a whole
        const int kl = min(k, p.K - 4);
        xq[ps] = *(const h4 *)(x + (size_t)m * p.K + kl);
        sq[ps] = *(const int4 *)(mapsrc + kl);
        // groups of a layer without a map; the choice between these and the loaded entries is made
        // where they are used, so that nothing here waits for a load
#pragma unroll
        for (int e = 0; e < 4; e++) gq[ps][e] = (k + e) / p.group_size;
    }

    // ---- 1w. WAVEX: the wave requests the x of its own K range: at most 512 channels per activation
    //          row, 64 quads per pass ------------------------------------------------------------
    constexpr int XP = 2 * M;
    h4 wxq[XP];
    bool wqv[XP];  // the quad is inside the wave's range and inside K
    int wpos[XP];  // where the quad's lane block starts in xlds
    if constexpr (WAVEX) {
        const int wq = wave_k / 4;  // quads per activation row in this wave's range
        // q / wq as a multiply: exact for q < 8192 and wq <= 128 (the error term q * (wq - 1) stays below 2^20)
        const uint32_t wq_inv = M == 1 ? 0u : ((1u << 20) + (uint32_t)wq - 1u) / (uint32_t)wq;
#pragma unroll
        for (int ps = 0; ps < XP; ps++) {
            const int q = lane + 64 * ps;
            const int m = M == 1 ? 0 : min((int)(((uint32_t)q * wq_inv) >> 20), M - 1);
            const int kc = wk * wave_k + 4 * (q - m * wq);  // position inside the workgroup's K range
            const int k = k_base + kc;
            wqv[ps] = q < M * wq && k < p.K && (!PACK || m < p.M);  // PACK: rows past p.M stay zero
            const int kl = min(max(k, 0), p.K - 4);
            wpos[ps] = m * kspan + (kc / F::KLANE) * F::KLANE;
            wxq[ps] = *(const h4 *)(x + (size_t)(PACK ? min(m, p.M - 1) : m) * p.K + kl);
        }
    }

    // ---- 2. zero the expanded activation operand in LDS while those loads fly ---------
    if constexpr (!WAVEX && !LITE) {
        u4 *z = (u4 *)tiles;
        const int n16 = nblk8 * ST * 16;
        for (int i = tid; i < n16; i += nthreads) z[i] = (u4){0u, 0u, 0u, 0u};
    }
    if constexpr (!WAVEX && LITE) {
        // only positions past the end of K must read as zero; the scatter writes every other one, so
        // the two never touch the same bytes and no barrier is needed between them
        const int tail0 = max(p.K - k_base, 0) / 8;  // K % 32 == 0
        for (int m = 0; m < M; m++)
            for (int i = tail0 + tid; i < kspan / 8; i += nthreads) ((u4 *)(xlds + m * kspan))[i] = (u4){0u, 0u, 0u, 0u};
    }
    // ---- 3. weight loads, software-pipelined: a wave blocks while it issues loads into a full
    //         memory pipeline, so only the first PF steps go out now (they cover the LDS work
    //         below); step s + PF is issued right before step s is consumed ---------------
    // Steps requested ahead.  The lean-operand kernels do best with about 4-5 KB in flight per wave beyond the
    // step being consumed (int4, 1 KB steps, 4096 x 11008: 1 ahead 9.4 us, 2: 7.9, 3: 7.5, 4: 7.45, 5: 7.6, 6: 7.8,
    // 8: 8.1, 12: 8.8, 16: 9.4; int3, 3 KB steps: 1 ahead 6.85 us, 2: 7.3, 3: 7.7, 4: 8.1): deeper queues delay
    // every wave's next request behind the others' and the waves of a workgroup drift apart.
    constexpr int PF = BITS == 4 ? (LITE ? 4 : 8) : 1;
    u4 w[NSTEP][F::WORDS];
    auto load_step = [&](int s, int st) {  // register slot s <- step st
        const int prow = 4 * st + lq;
        const bool ok = n_ok && st < we && prow < prows;
#pragma unroll
        for (int wd = 0; wd < F::WORDS; wd++) {
            // 32-bit byte offset from a uniform base: one VALU op per load instead of 64-bit math.
            // Steps past the wave's range, rows past K and columns past N read the first words of
            // qweight instead (one hot line): whatever they yield meets zeros of x, is skipped, or is
            // never stored.
            const uint32_t off = ok ? ((uint32_t)(prow * F::WORDS + wd) * (uint32_t)p.N + (uint32_t)n0) * 4u : 0u;
            w[s][wd] = __builtin_nontemporal_load((const u4 *)((const char *)p.qweight + off));
        }
    };
#pragma unroll
    for (int s = 0; s < (WAVEX ? 0 : PF) && s < NSTEP; s++) load_step(s, ws + s);
    __builtin_amdgcn_sched_barrier(0);
    if (!WAVEX && xsrc) {  // the x values of this thread's positions, now that their source channels are known
#pragma unroll
        for (int ps = 0; ps < QP; ps++) {
            const int idc = min(tid + ps * nthreads, nquads - 1);
            const _Float16 *xr = x + (size_t)(M == 1 ? 0 : idc / qpr) * p.K;
            xq[ps] = (h4){xr[src_ok(sq[ps].x)], xr[src_ok(sq[ps].y)], xr[src_ok(sq[ps].z)], xr[src_ok(sq[ps].w)]};
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- 4. scales / zero words this lane needs in the epilogue (rows g = 16 t + 4 q + v);
    //         requested behind the scatter of x: ahead of it they delay x and the first weights
    //         (measured 7.4 -> 7.7 us at int3 4096 x 11008) ---------------------------------
    h4 sc[TPM][4];
    uint32_t zwa[TPM][4], zwb[TPM][4];
    // Rows past the last group and lanes past the last column load clamped addresses: their
    // products are zero (no x was scattered there) or never stored, so no branch is needed.
    const int n_ld = min(n0, p.N - 4);
    auto load_epilogue_operands = [&]() {
#pragma unroll
        for (int t = 0; t < TPM; t++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const uint32_t g = (uint32_t)min(g_base + (PACK ? v : 16 * t + 4 * lq + v), p.G - 1);
                const uint32_t soff = (g * (uint32_t)p.N + (uint32_t)n_ld) * 2u;
                sc[t][v] = *(const h4 *)((const char *)scales + soff);
                load_zero_words<BITS>(p.qzeros, g * (uint32_t)zwords, n_ld, zwa[t][v], zwb[t][v]);
            }
        }
    };

    // The epilogue's scales and zero points as floats.  The lean-operand kernels convert them after the
    // first step of the main loop, while the wave waits for weights anyway, instead of after the last.
    float zf[TPM][4][4], sf[TPM][4][4];
    auto prep_epilogue = [&]() {
#pragma unroll
        for (int t = 0; t < TPM; t++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                zeros_from_words<BITS>(zwa[t][v], zwb[t][v], n_ld, zf[t][v]);
#pragma unroll
                for (int c = 0; c < 4; c++) sf[t][v][c] = (float)sc[t][v][c];
            }
    };

    // ---- 4w. WAVEX: the first weight requests, the epilogue operands, and only then the wait for x ----
    if constexpr (WAVEX) {
#pragma unroll
        for (int s = 0; s < PF && s < NSTEP; s++) load_step(s, ws + s);
        __builtin_amdgcn_sched_barrier(0);
        load_epilogue_operands();
        __builtin_amdgcn_sched_barrier(0);
        // x into this wave's part of LDS in unpack order, channels past the end of K as zeros
#pragma unroll
        for (int ps = 0; ps < XP; ps++) {
            if (lane + 64 * ps < M * (wave_k / 4)) {
#pragma unroll
                for (int e = 0; e < 4; e++) xlds[wpos[ps] + qslot[e]] = wqv[ps] ? wxq[ps][e] : (_Float16)0;
            }
        }
        // LDS serves the accesses of one wave in order; the fences only keep the compiler from moving
        // the main loop's reads above these writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if constexpr (!WAVEX) {
    if constexpr (!LITE) lds_barrier();  // the zero fill is complete
    // ---- 5. scatter x into the operand tiles (waits for x / g_idx only) -------------------
    // A thread always owns quads with the same position inside a lane block (kc % KLANE is
    // 4 * (tid % (KLANE / 4)) in every pass because the block size is a multiple of 8), so the
    // four slots of its quad are fixed: qslot[e], looked up once at the top of the kernel.
    // gb: first group of the wave that will consume channel kc (0 under a g_idx)
    auto scatter = [&](int m, int kc, int slot, int g, int gb, _Float16 xv) {
        if constexpr (LITE) {
            xlds[m * kspan + (kc / F::KLANE) * F::KLANE + slot] = xv;
            return;
        }
        const int r = min(max(g, 0), p.G - 1) - gb;  // row of this group
        const int rr = min(max(r, 0), 16 * TPM - 1);
        const int b8 = (kc / F::KLANE) * F::NB + (slot >> 3);
        if constexpr (COMPACT) {
            ((_Float16 *)tiles)[((b8 * ST + m) * 16 + (rr & 15)) * 8 + (slot & 7)] = xv;
            if (m == 0) ((unsigned short *)masks)[b8 * 8 + (slot & 7)] = rr < 16 ? 0xffffu : 0u;
        } else {
            ((_Float16 *)tiles)[((b8 * ST + m * TPM + (rr >> 4)) * 16 + (rr & 15)) * 8 + (slot & 7)] = xv;
        }
    };
    // sorted layer: the map gives position (already in unpack order) and group; channels of other
    // K ranges are dropped
    auto scatter_mapped = [&](int m, int entry, _Float16 xv) {
        const int kc = (entry & 0xffff) - k_base;
        if ((unsigned)kc < (unsigned)kspan) {
            if constexpr (LITE) {
                xlds[m * kspan + kc] = xv;
            } else {
                const int gb = wave_gb[__umulhi((uint32_t)kc, p.wave_div_magic)];
                scatter(m, kc, kc % F::KLANE, entry >> 16, gb, xv);
            }
        }
    };
#pragma unroll
    for (int ps = 0; ps < QP; ps++) {
        const int idx = tid + ps * nthreads;
        if (qv[ps]) {
            const int m = M == 1 ? 0 : idx / qpr;
            const int kc = 4 * (idx - m * qpr);
            const int gm[4] = {sq[ps].x, sq[ps].y, sq[ps].z, sq[ps].w};
            if (kmap) {
#pragma unroll
                for (int e = 0; e < 4; e++) scatter_mapped(m, gm[e], xq[ps][e]);
            } else {
                const int gb = p.g_idx ? 0 : (k_base + (kc / wave_k) * wave_k) / p.group_size;
#pragma unroll
                for (int e = 0; e < 4; e++) scatter(m, kc + e, qslot[e], has_map ? gm[e] : gq[ps][e], gb, xq[ps][e]);
            }
        }
    }
    // long K ranges (and sorted layers, whose workgroups walk all of x): LP passes per trip, all
    // loads of a trip issued before its first scatter
    constexpr int LP = 4;
    for (int base = tid + QP * nthreads; base < nquads; base += LP * nthreads) {
        h4 xl[LP];
        int4 gl[LP];
#pragma unroll
        for (int u = 0; u < LP; u++) {
            const int idx = base + u * nthreads;
            xl[u] = (h4){0, 0, 0, 0};
            gl[u] = make_int4(0, 0, 0, 0);
            if (idx < nquads) {
                const int m = M == 1 ? 0 : idx / qpr;
                const int k = scan_base + 4 * (idx - m * qpr);
                if (k < p.K) {
                    if (xsrc) {
                        gl[u] = *(const int4 *)(xsrc + k);
                    } else {
                        xl[u] = *(const h4 *)(x + (size_t)m * p.K + k);
                        if (p.g_idx || kmap) gl[u] = *(const int4 *)((kmap ? kmap : p.g_idx) + k);
                    }
                }
            }
        }
        if (xsrc) {
#pragma unroll
            for (int u = 0; u < LP; u++) {
                const int idx = base + u * nthreads;
                const int m = M == 1 ? 0 : min(idx, nquads - 1) / qpr;
                const _Float16 *xr = x + (size_t)m * p.K;  // sources of skipped quads are 0: a valid channel
                xl[u] = (h4){xr[src_ok(gl[u].x)], xr[src_ok(gl[u].y)], xr[src_ok(gl[u].z)], xr[src_ok(gl[u].w)]};
            }
        }
#pragma unroll
        for (int u = 0; u < LP; u++) {
            const int idx = base + u * nthreads;
            if (idx >= nquads) continue;
            const int m = M == 1 ? 0 : idx / qpr;
            const int kc = 4 * (idx - m * qpr);
            const int k = scan_base + kc;
            if (k >= p.K) continue;
            const int gv[4] = {gl[u].x, gl[u].y, gl[u].z, gl[u].w};
            if (kmap) {
#pragma unroll
                for (int e = 0; e < 4; e++) scatter_mapped(m, gv[e], xl[u][e]);
            } else {
                const int gb = p.g_idx ? 0 : (k_base + (kc / wave_k) * wave_k) / p.group_size;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int g = p.g_idx ? gv[e] : (k + e) / p.group_size;
                    scatter(m, kc + e, qslot[e], g, gb, xl[u][e]);
                }
            }
        }
    }
    lds_barrier();
    load_epilogue_operands();
    }  // !WAVEX

    // ---- 6. main loop -----------------------------------------------------------------
    // acc[m][t][c] collects sum x * (base + code); accx[m][t] is the same operand against the
    // constant columns "all ones" (column 0 -> X) and "the slot bases" (column 1 -> the base
    // part to subtract).  In the compact layout t = 0 is the masked tile (groups < 16) and
    // t = 1 the unmasked one (all groups): groups >= 16 are their difference.
    f4 acc[MA][TPM][4];
    f4 accx[MA][TPM];
#pragma unroll
    for (int m = 0; m < MA; m++)
#pragma unroll
        for (int t = 0; t < TPM; t++) {
            accx[m][t] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; c++) acc[m][t][c] = (f4){0.f, 0.f, 0.f, 0.f};
        }
    h8 cb;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float base = BITS == 4 ? BASE4[e] : BASE3[e];
        cb[e] = (_Float16)(li == 0 ? 1.0f : (li == 1 ? base : 0.0f));
    }
    const uint32_t magic_a = opaque_vgpr(BITS == 4 ? MAGIC4_LO : MAGIC3_EVEN);
    const uint32_t magic_b = opaque_vgpr(BITS == 4 ? MAGIC4_HI : MAGIC3_ODD);

    for (int st0 = ws; st0 < we; st0 += NSTEP) {
        if (st0 != ws) {
#pragma unroll
            for (int s = 0; s < PF && s < NSTEP; s++) load_step(s, st0 + s);
        }
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            if (st0 + s >= we) break;  // a short range ends the chunk early (no load sits behind this branch)
            if (s + PF < NSTEP) load_step(s + PF, st0 + s + PF);  // past the wave's range: one hot line
            __builtin_amdgcn_sched_barrier(0);
            {
                const int b = (st0 + s - s_begin) * 4 + lq;
                u4 bq[4][F::NB];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    if constexpr (BITS == 4) {
                        biased4(w[s][0][c], bq[c], magic_a, magic_b);
                    } else {
                        biased3(w[s][0][c], w[s][1][c], w[s][2][c], bq[c], magic_a, magic_b);
                    }
                }
#pragma unroll
                for (int nb = 0; nb < F::NB; nb++) {
                    const int b8 = b * F::NB + nb;
                    h8 a[MA][TPM];
                    if constexpr (PACK) {
                        // lane i feeds row i of the tile: activation row i / 4, group i % 4 of the wave
                        const uint32_t lb = (uint32_t)((st0 + s) * 4 + lq);
                        const int row = (int)(__umulhi(lb, p.gdiv_magic) + (p.gdiv_add ? lb : 0u)) - g_base;
#pragma unroll
                        for (int j = 0; j < MA; j++) {  // tile j: activation rows 4 j .. 4 j + 3
                            const uint32_t off =
                                row == (li & 3) ? (uint32_t)((4 * j + (li >> 2)) * kspan + b8 * 8) * 2u : zero_off;
                            a[j][0] = *(const h8 *)(smem + off);
                        }
                    } else if constexpr (LITE) {
                        // the group of this lane block, as a row of the wave's tile
                        const uint32_t lb = (uint32_t)((st0 + s) * 4 + lq);
                        const int row = (int)(__umulhi(lb, p.gdiv_magic) + (p.gdiv_add ? lb : 0u)) - g_base;
#pragma unroll
                        for (int m = 0; m < M; m++) {
                            const uint32_t off = row == li ? (uint32_t)(m * kspan + b8 * 8) * 2u : zero_off;
                            a[m][0] = *(const h8 *)(smem + off);
                        }
                    } else if constexpr (COMPACT) {
                        const u4 mk = *(const u4 *)(masks + (size_t)b8 * 16);
#pragma unroll
                        for (int m = 0; m < M; m++) {
                            a[m][1] = *(const h8 *)(tiles + ((size_t)(b8 * ST + m) * 16 + li) * 16);
                            a[m][0] = and_h8(a[m][1], mk);
                        }
                    } else {
#pragma unroll
                        for (int m = 0; m < M; m++)
#pragma unroll
                            for (int t = 0; t < TPM; t++) {
                                a[m][t] = *(const h8 *)(tiles + ((size_t)(b8 * ST + m * TPM + t) * 16 + li) * 16);
                            }
                    }
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const h8 bop = __builtin_bit_cast(h8, bq[c][nb]);
#pragma unroll
                        for (int m = 0; m < MA; m++)
#pragma unroll
                            for (int t = 0; t < TPM; t++) {
                                acc[m][t][c] =
                                    __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m][t], bop, acc[m][t][c], 0, 0, 0);
                            }
                    }
#pragma unroll
                    for (int m = 0; m < MA; m++)
#pragma unroll
                        for (int t = 0; t < TPM; t++) {
                            accx[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m][t], cb, accx[m][t], 0, 0, 0);
                        }
                }
            }
            if constexpr (LITE) {
                if (s == 0) prep_epilogue();
            }
        }
    }
    if (!LITE || ws >= we) prep_epilogue();  // (a wave without steps still multiplies its zero sums by finite numbers)

    // ---- 7. scales and zero points once per group, then sum over groups ------------------
    // row v of tile t in lane group q is group g_base + 16 t + 4 q + v
    float tot[MA][4];
#pragma unroll
    for (int m = 0; m < MA; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) tot[m][c] = 0.f;
#pragma unroll
    for (int m = 0; m < MA; m++) {
        float xs_prev[4] = {0.f, 0.f, 0.f, 0.f}, bs_prev[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < TPM; t++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float xsum = __shfl(accx[m][t][v], lane & 48);        // column 0: sum of x
                float bsum = __shfl(accx[m][t][v], (lane & 48) | 1);  // column 1: sum of x * base
                float pv[4];
#pragma unroll
                for (int c = 0; c < 4; c++) pv[c] = acc[m][t][c][v];
                if constexpr (COMPACT) {
                    if (t == 0) {
                        xs_prev[v] = xsum;
                        bs_prev[v] = bsum;
                    } else {
                        xsum -= xs_prev[v];
                        bsum -= bs_prev[v];
#pragma unroll
                        for (int c = 0; c < 4; c++) pv[c] -= acc[m][0][c][v];
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    tot[m][c] += sf[t][v][c] * ((pv[c] - bsum) - zf[t][v][c] * xsum);
                }
            }
        }
    }
    if constexpr (!PACK) {  // (PACK: a lane group's rows are the groups of ITS activation row)
#pragma unroll
        for (int m = 0; m < M; m++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                tot[m][c] += __shfl_xor(tot[m][c], 16);
                tot[m][c] += __shfl_xor(tot[m][c], 32);
            }
        }
    }

    // ---- 8. waves along K meet in LDS; one thread per four output columns finishes --------
    if constexpr (PACK) {
#pragma unroll
        for (int j = 0; j < MA; j++) {
            *(f4 *)(red + (((size_t)wk * WN + wn) * M + 4 * j + lq) * 64 + 4 * li) =
                (f4){tot[j][0], tot[j][1], tot[j][2], tot[j][3]};
        }
    } else if (lq == 0) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            *(f4 *)(red + (((size_t)wk * WN + wn) * M + m) * 64 + 4 * li) =
                (f4){tot[m][0], tot[m][1], tot[m][2], tot[m][3]};
        }
    }
    lds_barrier();
    const bool fin = tid < WN * M * 16;
    const int f_wn = tid / (M * 16);
    const int f_m = (tid >> 4) % M;
    const int f_n = blockIdx.x * BN + f_wn * 64 + 4 * (tid & 15);
    const bool writer = fin && f_n < p.N && (!PACK || f_m < p.M);
    f4 sum = {0.f, 0.f, 0.f, 0.f};
    if (writer) {
        for (int k = 0; k < WK; k++) {
            sum += *(const f4 *)(red + (((size_t)k * WN + f_wn) * M + f_m) * 64 + 4 * (tid & 15));
        }
    }
    const _Float16 *bias = (const _Float16 *)p.bias;
    f4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias && writer) {
        const h4 b4 = *(const h4 *)(bias + f_n);
        bv = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    _Float16 *y = (_Float16 *)p.y;
    if (p.split_k == 1) {
        if (writer) {
            h4 o;
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = (_Float16)(sum[c] + bv[c]);
            *(h4 *)(y + (size_t)f_m * p.N + f_n) = o;
        }
        return;
    }
    if (writer) store_partial(p.partial + ((size_t)split * M + f_m) * p.N + f_n, sum);
    if (!arrive_last(p.counters + blockIdx.x, p.split_k, &last_flag)) return;
    if (writer) {
        f4 total = bv;
        for (int s = 0; s < p.split_k; s++) total += load_partial(p.partial + ((size_t)s * M + f_m) * p.N + f_n);
        h4 o;
#pragma unroll
        for (int c = 0; c < 4; c++) o[c] = (_Float16)total[c];
        *(h4 *)(y + (size_t)f_m * p.N + f_n) = o;
    }
}

template <int BITS, int M, int TPM, bool COMPACT, bool LITE = false, bool WAVEX = false>
static int launch_grouped_one(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    constexpr int NSTEP = BITS == 4 ? 16 : 4;
    if constexpr (TPM == 1 && !COMPACT && !LITE) {
        // contiguous groups made of whole lane blocks: the lean operand (the same rule sized the plan's LDS)
        if (grouped_lite(BITS, p.K, p.group_size, p.g_idx != nullptr, TPM, M, plan.k_chunk, plan.waves_n, plan.waves_k,
                         plan.split_k))
            return launch_grouped_one<BITS, M, TPM, COMPACT, true>(p, plan, stream);
    }
    if constexpr (LITE && !WAVEX) {
        // short K ranges per wave and x in the order of the weights: every wave stages its own x
        if (grouped_wavex(true, p.wave_steps * Fmt<BITS>::KSTEP) && !p.kmap && !p.xsrc)
            return launch_grouped_one<BITS, M, TPM, COMPACT, true, true>(p, plan, stream);
    }
    auto kern = grouped_kernel<BITS, M, TPM, COMPACT, NSTEP, LITE, WAVEX>;
    const int lds_bytes = plan.lds_bytes;  // sized by the dispatcher for the operand layout in use
    if (lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, 1), dim3(plan.block), lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// two to four activation rows packed into one operand tile (ROWS = 4), five to eight into two (ROWS = 8)
template <int BITS, int ROWS>
static int launch_grouped_packed(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    constexpr int NSTEP = BITS == 4 ? 16 : 4;
    if (p.kmap || p.xsrc || plan.row_tiles != ROWS ||
        !grouped_packable(BITS, p.K, p.group_size, p.g_idx != nullptr, p.M, plan.k_chunk, plan.waves_k))
        return GPTQ_HIP_ERR_UNSUPPORTED;
    auto kern = grouped_kernel<BITS, ROWS, 1, false, NSTEP, true, true, true>;
    const int lds_bytes = plan.lds_bytes;
    if (lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, 1), dim3(plan.block), lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS>
static int launch_grouped_bits(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    const int tpm = p.gpad / 16;
    if (p.M > 4) return tpm == 1 ? launch_grouped_packed<BITS, 8>(p, plan, stream) : GPTQ_HIP_ERR_UNSUPPORTED;
    if (p.M > 2) return tpm == 1 ? launch_grouped_packed<BITS, 4>(p, plan, stream) : GPTQ_HIP_ERR_UNSUPPORTED;
    if (p.M == 2 && plan.row_tiles == packed_rows_of(2) &&
        grouped_packable(BITS, p.K, p.group_size, p.g_idx != nullptr, p.M, plan.k_chunk, plan.waves_k))
        return launch_grouped_packed<BITS, 4>(p, plan, stream);
    if (p.M == 1) {
        switch (tpm) {
            case 1: return launch_grouped_one<BITS, 1, 1, false>(p, plan, stream);
            case 2: return launch_grouped_one<BITS, 1, 2, true>(p, plan, stream);
            case 3: return launch_grouped_one<BITS, 1, 3, false>(p, plan, stream);
            case 4: return launch_grouped_one<BITS, 1, 4, false>(p, plan, stream);
            default: return GPTQ_HIP_ERR_UNSUPPORTED;
        }
    }
    if (p.M == 2) {
        switch (tpm) {
            case 1: return launch_grouped_one<BITS, 2, 1, false>(p, plan, stream);
            case 2: return launch_grouped_one<BITS, 2, 2, true>(p, plan, stream);
            default: return GPTQ_HIP_ERR_UNSUPPORTED;
        }
    }
    return GPTQ_HIP_ERR_UNSUPPORTED;
}

int launch_grouped(const Params &p, int bits, const gptq_hip_plan &plan, void *stream)
{
    return bits == 4 ? launch_grouped_bits<4>(p, plan, (hipStream_t)stream)
                     : launch_grouped_bits<3>(p, plan, (hipStream_t)stream);
}

}  // namespace gptq
