// GATHER kernel family: see the geometry notes in gptq_device.h.
//
// The weights are dequantised exactly as the reference does (fp16(scale * (q - zero)), one
// rounding) in registers, straight into the B operand of the MFMA; x goes through LDS.
// It covers every g_idx (activation order included) and every M; the dispatcher uses it
// for M >= 3 and as the fallback of the GROUPED family.
//
// Workgroup = waves_n x waves_k waves.  A wave owns 64 columns and all 16 * RT rows of its
// M block, so a weight is unpacked once per workgroup column tile; the waves along K split
// the workgroup's K range and meet in LDS at the end.  split_k > 1 adds workgroups along K
// whose partial tiles meet through the workspace.
//
// LDS: (scale, zero) of every group x the tile's columns [G][BN]; per K wave, double-buffered,
// the group offsets of a chunk of input channels and the x rows of that chunk, both in slot
// order.  The global loads of chunk i+1 are issued before chunk i is multiplied and written
// to the other buffer afterwards: one barrier per chunk, no exposed load latency.
// ACT = false (contiguous groups no narrower than a lane's packed row) reads one table entry
// per packed row instead of one per weight.
// grid = (column tiles, split_k, m blocks).
#include "gptq_device.h"

namespace gptq {

template <int BITS, int RT, bool ACT>
__global__ __launch_bounds__(256) void gather_kernel(const Params p)
{
    using F = Fmt<BITS>;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int WN = p.waves_n;
    const int WK = p.waves_k;
    const int wn = wave % WN;
    const int wk = wave / WN;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int BN = 64 * WN;
    const int GT = 64 * WN;  // threads of one K wave group
    const int gtid = wn * 64 + lane;
    const int n_blk = blockIdx.x * BN;
    const int col_l = wn * 64 + 4 * li;
    const int n0 = n_blk + col_l;
    const bool n_ok = n0 < p.N;
    const int m0 = blockIdx.z * (16 * RT);
    const int rows_here = min(16 * RT, p.M - m0);
    const int split = blockIdx.y;
    // uniform partition made by the host: wave_steps steps per K wave
    const int wg_steps = p.wave_steps * WK;
    const int s_begin = split * wg_steps;
    const int s_end = min(s_begin + wg_steps, p.steps_total);
    const int ws = s_begin + wk * p.wave_steps;
    const int we = min(ws + p.wave_steps, s_end);
    // groups whose (scale, zero) this workgroup can meet: all of them under a g_idx, else those of
    // its K range
    const int g_lo = p.g_idx ? 0 : (s_begin * F::KSTEP) / p.group_size;
    const int g_hi = p.g_idx ? p.G - 1 : min(p.G - 1, (min(s_end * F::KSTEP, p.K) - 1) / p.group_size);

    constexpr int KC = gather_kc(BITS, RT);  // channels staged per chunk (a power of two)
    constexpr int CS = KC / F::KSTEP;        // steps per chunk; divides PF
    const int XS = KC + 8;
    // per K wave group: two buffers (double buffering) of [KC] group offsets + [16 RT][XS] x
    const size_t buf_bytes = (size_t)KC * 4 + (size_t)(16 * RT) * XS * 2;
    // (scale, zero) table: h2 [G][BN], rows padded by 16 bytes so that the four lane groups, which
    // read rows of different groups, do not all land on the same LDS banks
    const int TROW = BN * 4 + 16;
    unsigned char *tab_b = smem;
    unsigned char *stage = smem + (size_t)p.G * TROW + (size_t)wk * 2 * buf_bytes;
    __shared__ int last_flag;

    const _Float16 *x = (const _Float16 *)p.x;
    const _Float16 *scales = (const _Float16 *)p.scales;
    const int zwords = p.N / 32 * BITS;
    const int prows = p.K / (BITS == 4 ? 8 : 32);

    // Everything in the main loop is branch-free per lane: addresses are clamped into bounds and
    // what must not count is multiplied by a zero x (rows past M, channels past K) or never
    // stored (columns past N).  Per-lane branches here cost more than the matrix work.
    const uint32_t n_ld = (uint32_t)min(n0, p.N - 4);
    auto load_w = [&](int st, u4 (&w)[F::WORDS]) {
        const uint32_t prow = (uint32_t)min(4 * st + lq, prows - 1);  // packed row (int4) / 3-word block (int3)
#pragma unroll
        for (int wd = 0; wd < F::WORDS; wd++) {
            const uint32_t off = ((prow * F::WORDS + wd) * (uint32_t)p.N + n_ld) * 4u;
            w[wd] = __builtin_nontemporal_load((const u4 *)((const char *)p.qweight + off));
        }
    };
    // Weight loads run PF steps ahead of their use in a ring of registers: with one wave per
    // SIMD the cache-cold HBM latency must be covered by loads in flight, not by other waves.
    constexpr int PF = BITS == 4 ? 8 : 4;
    static_assert(PF % CS == 0, "a chunk must divide the prefetch ring");
    u4 w[PF][F::WORDS];
#pragma unroll
    for (int u = 0; u < PF; u++) load_w(ws + u, w[u]);

    // ---- staging of one chunk, split into "global -> registers" and "registers -> LDS" so that
    //      the loads of chunk i+1 fly while chunk i is being multiplied ---------------------
    constexpr int XV = gather_xv(BITS, RT);  // 16-byte vectors of x per thread per chunk, at most
    constexpr int GV = gather_gv();          // group indices per thread per chunk, at most
    const int vshift = __builtin_ctz(KC / 8);          // log2(vectors per row)
    const int xve = ((16 * RT) << vshift) / GT;        // vectors this thread stages (uniform)
    const int gve = (KC + GT - 1) / GT;
    h8 xreg[XV];
    int greg[GV];
    auto fetch_chunk = [&](int ch) {
        const int c0 = ws + ch * CS;
        const int c1 = min(c0 + CS, we);
        const int k0 = c0 * F::KSTEP;
        const int kspan = max(c1 - c0, 0) * F::KSTEP;
#pragma unroll
        for (int i = 0; i < XV; i++) {
            if (i < xve) {
                const int v = gtid + i * GT;
                const int r = v >> vshift;
                const int kc = 8 * (v & ((1 << vshift) - 1));
                const bool ok = r < rows_here && kc < kspan && k0 + kc < p.K;
                const uint32_t off =
                    ((uint32_t)(m0 + min(r, rows_here - 1)) * (uint32_t)p.K + (uint32_t)min(k0 + kc, p.K - 8)) * 2u;
                const u4 raw = *(const u4 *)((const char *)x + off);
                const u4 zero = {0u, 0u, 0u, 0u};
                xreg[i] = __builtin_bit_cast(h8, ok ? raw : zero);
            }
        }
#pragma unroll
        for (int i = 0; i < GV; i++) {
            if (i < gve) {
                const int kc = min(gtid + i * GT, KC - 1);  // threads past the chunk repeat its last entry
                const int k = min(k0 + kc, p.K - 1);
                greg[i] = p.g_idx ? p.g_idx[k] : k / p.group_size;
            }
        }
    };
    auto store_chunk = [&](int buf) {
        int *gl = (int *)(stage + (size_t)buf * buf_bytes);
        _Float16 *xs = (_Float16 *)(gl + KC);
#pragma unroll
        for (int i = 0; i < XV; i++) {
            if (i < xve) {
                const int v = gtid + i * GT;
                const int r = v >> vshift;
                const int kc = 8 * (v & ((1 << vshift) - 1));
                _Float16 *dst = xs + r * XS + (kc / F::KLANE) * F::KLANE;
                if constexpr (BITS == 4) {
                    h8 o;  // all eight land in one lane block: one 16-byte store in slot order
#pragma unroll
                    for (int s = 0; s < 8; s++) o[s] = xreg[i][SLOT4[s]];
                    *(h8 *)dst = o;
                } else {
                    const int jb = kc % F::KLANE;
#pragma unroll
                    for (int e = 0; e < 8; e++) dst[slot_of_code<BITS>(jb + e)] = xreg[i][e];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < GV; i++) {
            if (i < gve) {
                const int kc = min(gtid + i * GT, KC - 1);
                const int g = min(max(greg[i], g_lo), g_hi) - g_lo;
                gl[(kc / F::KLANE) * F::KLANE + slot_of_code<BITS>(kc % F::KLANE)] = g * TROW;
            }
        }
    };

    const int nchunks = (p.wave_steps + CS - 1) / CS;
    fetch_chunk(0);

    // (scale, zero) table: four columns of one group per thread and item.  With contiguous groups
    // only the groups of this workgroup's K range are staged (row 0 = the first of them).  Items
    // go four at a time so that their global loads overlap.
    const int tab_rows = g_hi - g_lo + 1;
    const int tab_items = tab_rows * (BN / 4);
    for (int base = tid; base < tab_items; base += 4 * (int)blockDim.x) {
        h4 s4[4];
        uint32_t za[4], zb[4];
        int nn[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx = base + u * (int)blockDim.x;
            const int gr = min(idx, tab_items - 1) / (BN / 4);
            const int c4 = 4 * (min(idx, tab_items - 1) - gr * (BN / 4));
            nn[u] = min(n_blk + c4, p.N - 4);
            const uint32_t g = (uint32_t)(g_lo + gr);
            s4[u] = *(const h4 *)((const char *)scales + (g * (uint32_t)p.N + (uint32_t)nn[u]) * 2u);
            load_zero_words<BITS>(p.qzeros, g * (uint32_t)zwords, nn[u], za[u], zb[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx = base + u * (int)blockDim.x;
            if (idx < tab_items) {
                const int gr = idx / (BN / 4);
                const int c4 = 4 * (idx - gr * (BN / 4));
                float z[4];
                zeros_from_words<BITS>(za[u], zb[u], nn[u], z);
                u4 e;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const h2 sz = {s4[u][c], (_Float16)z[c]};
                    e[c] = as_u32(sz);
                }
                *(u4 *)(tab_b + (size_t)gr * TROW + c4 * 4) = e;
            }
        }
    }

    f4 acc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[rt][c] = (f4){0.f, 0.f, 0.f, 0.f};

    const uint32_t magic_a = opaque_vgpr(BITS == 4 ? MAGIC4_LO : MAGIC3_EVEN);
    const uint32_t magic_b = opaque_vgpr(BITS == 4 ? MAGIC4_HI : MAGIC3_ODD);

    store_chunk(0);
    lds_barrier();
    // steps every wave of the workgroup walks: whole chunks, rounded up to the prefetch ring
    const int total = (nchunks * CS + PF - 1) / PF * PF;
    const int walk_chunks = (total + CS - 1) / CS;  // chunks past the wave's range are staged as zeros
    int ch = 0;  // chunk being multiplied
    for (int i0 = 0; i0 < total; i0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            // No condition guards the matrix work: steps past the wave's range (the host rounds the
            // walk up to whole chunks and to a multiple of PF) multiply x rows that were staged
            // as zeros.  Guarding them makes the compiler shuttle all accumulators between
            // register files at every merge point.
            {
                const int st = ws + i0 + u;
                const int ci = u % CS;  // step inside the chunk: known at compile time
                if ((u % CS) == 0 && ch + 1 < walk_chunks) fetch_chunk(ch + 1);
                const int *gl = (const int *)(stage + (size_t)(ch & 1) * buf_bytes);
                const _Float16 *xs = (const _Float16 *)(gl + KC);
                {
                    const int b = ci * 4 + lq;  // this lane's block inside the chunk
                    u4 bq[4][F::NB];
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        if constexpr (BITS == 4) {
                            biased4(w[u][0][c], bq[c], magic_a, magic_b);
                        } else {
                            biased3(w[u][0][c], w[u][1][c], w[u][2][c], bq[c], magic_a, magic_b);
                        }
                    }
                    // contiguous groups: the (scale, zero) of this lane's packed row, four columns
                    u4 erow = {0u, 0u, 0u, 0u};
                    if constexpr (!ACT) {
                        erow = *(const u4 *)(tab_b + (uint32_t)gl[b * F::KLANE] + (uint32_t)col_l * 4u);
                    }
#pragma unroll
                    for (int nb = 0; nb < F::NB; nb++) {
                        h8 bop[4];
                        if constexpr (ACT) {
                            // (scale, zero) of the 8 slots x 4 columns
                            const u4 go0 = *(const u4 *)(gl + b * F::KLANE + nb * 8);
                            const u4 go1 = *(const u4 *)(gl + b * F::KLANE + nb * 8 + 4);
                            u4 ent[8];
#pragma unroll
                            for (int s = 0; s < 8; s++) {
                                const uint32_t off = (s < 4 ? go0[s & 3] : go1[s & 3]) + (uint32_t)col_l * 4u;
                                ent[s] = *(const u4 *)(tab_b + off);
                            }
#pragma unroll
                            for (int c = 0; c < 4; c++) {
                                u4 wv;
#pragma unroll
                                for (int r = 0; r < 4; r++) {
                                    const uint32_t ea = ent[2 * r][c];
                                    const uint32_t eb = ent[2 * r + 1][c];
                                    const h2 s2 = as_h2((ea & 0xffffu) | (eb << 16));
                                    const h2 z2 = as_h2((ea >> 16) | (eb & 0xffff0000u));
                                    const float ba = BITS == 4 ? BASE4[2 * r] : BASE3[2 * r];
                                    const float bb = BITS == 4 ? BASE4[2 * r + 1] : BASE3[2 * r + 1];
                                    const h2 zb = z2 + (h2){(_Float16)ba, (_Float16)bb};  // exact: small integers
                                    wv[r] = as_u32((as_h2(bq[c][nb][r]) - zb) * s2);      // exact difference, one rounding
                                }
                                bop[c] = __builtin_bit_cast(h8, wv);
                            }
                        } else {
#pragma unroll
                            for (int c = 0; c < 4; c++) {
                                const uint32_t e = erow[c];
                                const h2 s2 = as_h2((e & 0xffffu) | (e << 16));
                                const h2 z2 = as_h2((e >> 16) | (e & 0xffff0000u));
                                u4 wv;
#pragma unroll
                                for (int r = 0; r < 4; r++) {
                                    const float ba = BITS == 4 ? BASE4[2 * r] : BASE3[2 * r];
                                    const float bb = BITS == 4 ? BASE4[2 * r + 1] : BASE3[2 * r + 1];
                                    const h2 zb = z2 + (h2){(_Float16)ba, (_Float16)bb};
                                    wv[r] = as_u32((as_h2(bq[c][nb][r]) - zb) * s2);
                                }
                                bop[c] = __builtin_bit_cast(h8, wv);
                            }
                        }
#pragma unroll
                        for (int rt = 0; rt < RT; rt++) {
                            const h8 a = *(const h8 *)(xs + (16 * rt + li) * XS + b * F::KLANE + nb * 8);
#pragma unroll
                            for (int c = 0; c < 4; c++) {
                                acc[rt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bop[c], acc[rt][c], 0, 0, 0);
                            }
                        }
                    }
                }
                load_w(st + PF, w[u]);  // refill this ring slot
                if ((u % CS) == CS - 1) {
                    if (ch + 1 < walk_chunks) store_chunk((ch + 1) & 1);
                    lds_barrier();  // chunk ch+1 is in LDS, and chunk ch's buffer may be overwritten next time
                    ch++;
                }
            }
        }
    }

    // ---- waves along K meet in LDS: wave (wn, 0) adds the others' tiles in order ------------
    if (WK > 1) {
        float *red = (float *)smem;  // [WK - 1][WN][RT * 16][64], reuses the staging area
        lds_barrier();
        if (wk > 0) {
            float *dst = red + ((size_t)((wk - 1) * WN + wn) * (RT * 16)) * 64 + lane;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int c = 0; c < 4; c++)
#pragma unroll
                    for (int v = 0; v < 4; v++) dst[((rt * 4 + c) * 4 + v) * 64] = acc[rt][c][v];
        }
        lds_barrier();
        if (wk == 0) {
            for (int k = 1; k < WK; k++) {
                const float *src = red + ((size_t)((k - 1) * WN + wn) * (RT * 16)) * 64 + lane;
#pragma unroll
                for (int rt = 0; rt < RT; rt++)
#pragma unroll
                    for (int c = 0; c < 4; c++)
#pragma unroll
                        for (int v = 0; v < 4; v++) acc[rt][c][v] += src[((rt * 4 + c) * 4 + v) * 64];
            }
        }
    }
    const bool owner = wk == 0 && n_ok;

    // ---- epilogue: acc[rt][c][v] is y[m0 + 16 rt + 4 q + v][n0 + c] ----
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

    if (owner) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * rt + 4 * lq + v;
                if (row < rows_here) {
                    const f4 o = {acc[rt][0][v], acc[rt][1][v], acc[rt][2][v], acc[rt][3][v]};
                    store_partial(p.partial + ((size_t)split * p.M + (m0 + row)) * p.N + n0, o);
                }
            }
        }
    }
    int *counter = p.counters + blockIdx.z * gridDim.x + blockIdx.x;
    if (!arrive_last(counter, p.split_k, &last_flag)) {
        return;
    }
    if (owner) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * rt + 4 * lq + v;
                if (row < rows_here) {
                    f4 sum = bv;
                    for (int s = 0; s < p.split_k; s++) {
                        sum += load_partial(p.partial + ((size_t)s * p.M + (m0 + row)) * p.N + n0);
                    }
                    h4 o;
#pragma unroll
                    for (int c = 0; c < 4; c++) o[c] = (_Float16)sum[c];
                    *(h4 *)(y + (size_t)(m0 + row) * p.N + n0) = o;
                }
            }
        }
    }
}

template <int BITS, int RT, bool ACT>
static int launch_gather_one(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = gather_kernel<BITS, RT, ACT>;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    const dim3 grid(plan.grid_x, plan.grid_y, plan.grid_z);
    hipLaunchKernelGGL(kern, grid, dim3(plan.block), plan.lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS, bool ACT>
static int launch_gather_rt(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    switch (plan.row_tiles) {
        case 1: return launch_gather_one<BITS, 1, ACT>(p, plan, stream);
        case 2: return launch_gather_one<BITS, 2, ACT>(p, plan, stream);
        case 4: return launch_gather_one<BITS, 4, ACT>(p, plan, stream);
        default: return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

int launch_gather(const Params &p, int bits, const gptq_hip_plan &plan, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    // the per-row table read needs every code of a lane's packed row in one group
    const int klane = bits == 4 ? 8 : 32;
    const bool act = p.g_idx != nullptr || (p.group_size % klane) != 0;
    if (bits == 4) {
        return act ? launch_gather_rt<4, true>(p, plan, stream) : launch_gather_rt<4, false>(p, plan, stream);
    }
    return act ? launch_gather_rt<3, true>(p, plan, stream) : launch_gather_rt<3, false>(p, plan, stream);
}

}  // namespace gptq
