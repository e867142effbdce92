// GATHER kernel family: see the geometry notes in gptq_device.h.
#include "gptq_device.h"

namespace gptq {

// ---------------------------------------------------------------------------------
// GATHER kernel: exact fp16 weights, scale/zero looked up per weight through g_idx.
// Covers every g_idx (activation order included) and every M.
// LDS: table of (scale, zero) for all groups x the tile's columns; per chunk of input
// channels the group offsets (slot order) and the x rows (slot order).
// grid = (column tiles, split_k, m blocks), block = 64 * waves (all waves along N).
// ---------------------------------------------------------------------------------
template <int BITS, int RT>
__global__ __launch_bounds__(256) void gather_kernel(const Params p)
{
    using F = Fmt<BITS>;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int BN = (int)blockDim.x;  // 64 columns per wave
    const int n_blk = blockIdx.x * BN;
    const int col_l = wave * 64 + 4 * li;
    const int n0 = n_blk + col_l;
    const bool n_ok = n0 < p.N;
    const int m0 = blockIdx.z * (16 * RT);
    const int rows_here = min(16 * RT, p.M - m0);
    const int split = blockIdx.y;
    const int s_begin = (int)((long long)p.steps_total * split / p.split_k);
    const int s_end = (int)((long long)p.steps_total * (split + 1) / p.split_k);

    const int KC = p.chunk_steps * F::KSTEP;
    const int XS = KC + 8;
    unsigned char *tab_b = smem;                            // h2 [G][BN] = (scale, zero)
    int *gl = (int *)(smem + (size_t)p.G * BN * 4);         // [KC] byte offset of the group's table row
    _Float16 *xs = (_Float16 *)(gl + KC);                   // [xs_rows][XS]
    __shared__ int last_flag;

    const _Float16 *x = (const _Float16 *)p.x;
    const _Float16 *scales = (const _Float16 *)p.scales;
    const int zwords = p.N / 32 * BITS;

    for (int idx = tid; idx < p.G * BN; idx += (int)blockDim.x) {
        const int g = idx / BN;
        const int n = n_blk + idx % BN;
        h2 e = {(_Float16)0.0f, (_Float16)0.0f};
        if (n < p.N) {
            e.x = scales[(size_t)g * p.N + n];
            e.y = (_Float16)(float)zero_of<BITS>(p.qzeros + (size_t)g * zwords, n);
        }
        ((h2 *)tab_b)[idx] = e;
    }

    f4 acc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[rt][c] = (f4){0.f, 0.f, 0.f, 0.f};

    const int rows3 = p.K / 32;  // 3-word blocks (int3) ...
    const int rows4 = p.K / 8;   // ... or word rows (int4) along K

    for (int c0 = s_begin; c0 < s_end; c0 += p.chunk_steps) {
        const int c1 = min(c0 + p.chunk_steps, s_end);
        const int k0 = c0 * F::KSTEP;
        const int kspan = (c1 - c0) * F::KSTEP;
        __syncthreads();  // the previous chunk has been consumed by every wave
        for (int kc = tid; kc < kspan; kc += (int)blockDim.x) {
            const int k = k0 + kc;
            int g = 0;
            if (k < p.K) {
                g = p.g_idx ? p.g_idx[k] : k / p.group_size;
                g = min(max(g, 0), p.G - 1);
            }
            const int b = kc / F::KLANE;
            gl[b * F::KLANE + slot_of_code<BITS>(kc % F::KLANE)] = g * BN * 4;
        }
        const int vec_per_row = kspan / 8;
        for (int v = tid; v < rows_here * vec_per_row; v += (int)blockDim.x) {
            const int r = v / vec_per_row;
            const int kc = 8 * (v % vec_per_row);
            const int k = k0 + kc;
            h8 val = {0, 0, 0, 0, 0, 0, 0, 0};
            if (k < p.K) val = *(const h8 *)(x + (size_t)(m0 + r) * p.K + k);
            _Float16 *dst = xs + r * XS + (kc / F::KLANE) * F::KLANE;
            const int jb = kc % F::KLANE;
#pragma unroll
            for (int e = 0; e < 8; e++) dst[slot_of_code<BITS>(jb + e)] = val[e];
        }
        __syncthreads();

        for (int st = c0; st < c1; ++st) {
            const int b = (st - c0) * 4 + lq;  // this lane's block inside the chunk
            u4 w[F::WORDS];
            {
                const int prow = 4 * st + lq;  // packed row (int4) or 3-word block (int3)
                const bool ok = n_ok && prow < (BITS == 4 ? rows4 : rows3);
#pragma unroll
                for (int wd = 0; wd < F::WORDS; wd++) {
                    w[wd] = (u4){0u, 0u, 0u, 0u};
                    if (ok) w[wd] = *(const u4 *)(p.qweight + (size_t)(prow * F::WORDS + wd) * p.N + n0);
                }
            }
            uint32_t mg[4][4 * F::NB];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                if constexpr (BITS == 4) {
                    magic4(w[0][c], mg[c]);
                } else {
                    magic3(w[0][c], w[1][c], w[2][c], mg[c]);
                }
            }
#pragma unroll
            for (int nb = 0; nb < F::NB; nb++) {
                // (scale, zero) of the 8 slots x 4 columns
                const u4 go0 = *(const u4 *)(gl + b * F::KLANE + nb * 8);
                const u4 go1 = *(const u4 *)(gl + b * F::KLANE + nb * 8 + 4);
                u4 ent[8];
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    const uint32_t off = (s < 4 ? go0[s & 3] : go1[s & 3]) + (uint32_t)col_l * 4u;
                    ent[s] = *(const u4 *)(tab_b + off);
                }
                h8 bop[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const uint32_t ea = ent[2 * r][c];
                        const uint32_t eb = ent[2 * r + 1][c];
                        const h2 s2 = as_h2((ea & 0xffffu) | (eb << 16));
                        const h2 z2 = as_h2((ea >> 16) | (eb & 0xffff0000u));
                        const h2 q2 = BITS == 4 ? code_from_magic4(mg[c][nb * 4 + r], nb * 4 + r)
                                                : code_from_magic3(mg[c][nb * 4 + r], nb * 4 + r);
                        const h2 w2 = (q2 - z2) * s2;
                        bop[c][2 * r] = w2.x;
                        bop[c][2 * r + 1] = w2.y;
                    }
                }
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    h8 a = {0, 0, 0, 0, 0, 0, 0, 0};
                    if (16 * rt + li < rows_here) {
                        a = *(const h8 *)(xs + (16 * rt + li) * XS + b * F::KLANE + nb * 8);
                    }
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        acc[rt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bop[c], acc[rt][c], 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- epilogue: acc[rt][c][v] is y[m0 + 16 rt + 4 q + v][n0 + c] ----
    const _Float16 *bias = (const _Float16 *)p.bias;
    f4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias && n_ok) {
        const h4 b4 = *(const h4 *)(bias + n0);
        bv = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    _Float16 *y = (_Float16 *)p.y;
    if (p.split_k == 1) {
        if (n_ok) {
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

    if (n_ok) {
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
    if (!arrive_last(counter, p.split_k, &last_flag)) return;
    if (n_ok) {
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

template <int BITS, int RT>
static int launch_gather_one(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    auto kern = gather_kernel<BITS, RT>;
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

template <int BITS>
static int launch_gather_rt(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    switch (plan.row_tiles) {
        case 1: return launch_gather_one<BITS, 1>(p, plan, stream);
        case 2: return launch_gather_one<BITS, 2>(p, plan, stream);
        case 4: return launch_gather_one<BITS, 4>(p, plan, stream);
        case 8: return launch_gather_one<BITS, 8>(p, plan, stream);
        default: return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

int launch_gather(const Params &p, int bits, const gptq_hip_plan &plan, void *stream)
{
    return bits == 4 ? launch_gather_rt<4>(p, plan, (hipStream_t)stream)
                     : launch_gather_rt<3>(p, plan, (hipStream_t)stream);
}

}  // namespace gptq
