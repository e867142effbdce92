// GROUPED kernel family: decode-size products (M of 1 or 2) for any g_idx.
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
// LDS holds the expanded activation operand of the workgroup's K range, laid out as
// the MFMA wants it: tile (block b, sub-block nb, row tile rt) is 16 rows x 8 slots of
// fp16 = 256 bytes, lane i reads its 16 bytes at i*16.  It is zero-filled and then
// scattered into: one 2-byte store per (m, k).
//
// grid = (column tiles, split_k), block = 64 * waves, every wave owns 64 columns.
#include "gptq_device.h"

namespace gptq {

// The four zero points (already +1) of columns n .. n+3 (n % 4 == 0) of one qzeros row.
template <int BITS>
__device__ __forceinline__ void load_zero_words(const uint32_t *zrow, int n, uint32_t &wa, uint32_t &wb)
{
    if constexpr (BITS == 4) {
        wa = zrow[n >> 3];
        wb = 0u;
    } else {
        const uint32_t *blk = zrow + 3 * (n >> 5);
        const int o = 3 * (n & 31);  // bit offset inside the 96-bit block: a multiple of 12
        const int w = o >> 5;
        wa = blk[w];
        wb = blk[w < 2 ? w + 1 : 2];
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

// RT = row tiles = M * TPM, TPM = tiles (of 16 groups) per activation row.
template <int BITS, int M, int TPM, int NSTEP>
__global__ __launch_bounds__(256) void grouped_kernel(const Params p)
{
    using F = Fmt<BITS>;
    constexpr int RT = M * TPM;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int lq = lane >> 4;
    const int BN = (int)blockDim.x;
    const int n0 = blockIdx.x * BN + wave * 64 + 4 * li;
    const bool n_ok = n0 < p.N;
    const int split = blockIdx.y;
    const int s_begin = (int)((long long)p.steps_total * split / p.split_k);
    const int s_end = (int)((long long)p.steps_total * (split + 1) / p.split_k);
    const int nsteps = s_end - s_begin;
    const int k_base = s_begin * F::KSTEP;
    const int kspan = nsteps * F::KSTEP;
    const int prows = p.K / (BITS == 4 ? 8 : 32);  // packed rows (int4) or 3-word blocks (int3)
    // contiguous groups: only those inside this K range need rows, counted from the first one
    const int g_base = p.g_idx ? 0 : k_base / p.group_size;
    __shared__ int last_flag;

    const _Float16 *x = (const _Float16 *)p.x;
    const _Float16 *scales = (const _Float16 *)p.scales;
    const int zwords = p.N / 32 * BITS;

    // ---- 1. first batch of weight loads goes out before anything else -----------------
    u4 w[NSTEP][F::WORDS];
    auto load_batch = [&](int st0) {
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            const int prow = 4 * (st0 + s) + lq;
            const bool ok = n_ok && (st0 + s) < s_end && prow < prows;
#pragma unroll
            for (int wd = 0; wd < F::WORDS; wd++) {
                w[s][wd] = (u4){0u, 0u, 0u, 0u};
                if (ok) {
                    w[s][wd] = __builtin_nontemporal_load(
                        (const u4 *)(p.qweight + (size_t)(prow * F::WORDS + wd) * p.N + n0));
                }
            }
        }
    };
    load_batch(s_begin);

    // ---- 2. scales / zero words this lane needs in the epilogue: rows g = 16 t + 4 q + v -
    h4 sc[TPM][4];
    uint32_t zwa[TPM][4], zwb[TPM][4];
#pragma unroll
    for (int t = 0; t < TPM; t++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int g = g_base + 16 * t + 4 * lq + v;
            sc[t][v] = (h4){0, 0, 0, 0};
            zwa[t][v] = 0u;
            zwb[t][v] = 0u;
            if (n_ok && g < p.G) {
                sc[t][v] = *(const h4 *)(scales + (size_t)g * p.N + n0);
                load_zero_words<BITS>(p.qzeros + (size_t)g * zwords, n0, zwa[t][v], zwb[t][v]);
            }
        }
    }

    // ---- 3. expanded activation operand in LDS -----------------------------------------
    const int nblk8 = kspan / 8;  // 8-slot blocks in the K range
    {
        u4 *z = (u4 *)smem;
        const int n16 = nblk8 * RT * 16;
        for (int i = tid; i < n16; i += (int)blockDim.x) z[i] = (u4){0u, 0u, 0u, 0u};
    }
    __syncthreads();
    for (int idx = tid; idx < kspan * M; idx += (int)blockDim.x) {
        const int m = idx / kspan;
        const int kc = idx - m * kspan;
        const int k = k_base + kc;
        if (k < p.K) {
            int g = p.g_idx ? p.g_idx[k] : k / p.group_size;
            g = min(max(g, 0), p.G - 1);
            const _Float16 xv = x[(size_t)m * p.K + k];
            const int r = m * (16 * TPM) + min(g - g_base, 16 * TPM - 1);
            const int b = kc / F::KLANE;
            const int slot = slot_of_code<BITS>(kc % F::KLANE);
            const int tile = ((b * F::NB + (slot >> 3)) * RT + (r >> 4));
            ((_Float16 *)smem)[(tile * 16 + (r & 15)) * 8 + (slot & 7)] = xv;
        }
    }
    __syncthreads();

    // ---- 4. main loop -----------------------------------------------------------------
    f4 acc[RT][4];
    f4 accx[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        accx[rt] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; c++) acc[rt][c] = (f4){0.f, 0.f, 0.f, 0.f};
    }
    const h8 ones = {1, 1, 1, 1, 1, 1, 1, 1};

    for (int st0 = s_begin; st0 < s_end; st0 += NSTEP) {
        if (st0 != s_begin) load_batch(st0);
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            if (st0 + s < s_end) {
                const int b = (st0 + s - s_begin) * 4 + lq;
                uint32_t mg[4][4 * F::NB];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    if constexpr (BITS == 4) {
                        magic4(w[s][0][c], mg[c]);
                    } else {
                        magic3(w[s][0][c], w[s][1][c], w[s][2][c], mg[c]);
                    }
                }
#pragma unroll
                for (int nb = 0; nb < F::NB; nb++) {
                    h8 bop[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const h2 q2 = BITS == 4 ? code_from_magic4(mg[c][nb * 4 + r], nb * 4 + r)
                                                    : code_from_magic3(mg[c][nb * 4 + r], nb * 4 + r);
                            bop[c][2 * r] = q2.x;
                            bop[c][2 * r + 1] = q2.y;
                        }
                    }
#pragma unroll
                    for (int rt = 0; rt < RT; rt++) {
                        const h8 a = *(const h8 *)(smem + ((size_t)((b * F::NB + nb) * RT + rt) * 16 + li) * 16);
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            acc[rt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bop[c], acc[rt][c], 0, 0, 0);
                        }
                        accx[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, ones, accx[rt], 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- 5. epilogue: scales and zero points once per group, then sum over groups -------
    // acc[m*TPM + t][c][v] = P[m][g = g_base + 16 t + 4 q + v][n0 + c];  accx[m*TPM + t][v] = X[m][g]
    float tot[M][4];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) tot[m][c] = 0.f;
#pragma unroll
    for (int t = 0; t < TPM; t++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            float z[4];
            zeros_from_words<BITS>(zwa[t][v], zwb[t][v], n0, z);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float s = (float)sc[t][v][c];
#pragma unroll
                for (int m = 0; m < M; m++) {
                    tot[m][c] += s * (acc[m * TPM + t][c][v] - z[c] * accx[m * TPM + t][v]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < M; m++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            tot[m][c] += __shfl_xor(tot[m][c], 16);
            tot[m][c] += __shfl_xor(tot[m][c], 32);
        }
    }

    const _Float16 *bias = (const _Float16 *)p.bias;
    f4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias && n_ok) {
        const h4 b4 = *(const h4 *)(bias + n0);
        bv = (f4){(float)b4[0], (float)b4[1], (float)b4[2], (float)b4[3]};
    }
    _Float16 *y = (_Float16 *)p.y;
    const bool writer = n_ok && lq == 0;
    if (p.split_k == 1) {
        if (writer) {
#pragma unroll
            for (int m = 0; m < M; m++) {
                h4 o;
#pragma unroll
                for (int c = 0; c < 4; c++) o[c] = (_Float16)(tot[m][c] + bv[c]);
                *(h4 *)(y + (size_t)m * p.N + n0) = o;
            }
        }
        return;
    }
    if (writer) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            const f4 o = {tot[m][0], tot[m][1], tot[m][2], tot[m][3]};
            store_partial(p.partial + ((size_t)split * M + m) * p.N + n0, o);
        }
    }
    if (!arrive_last(p.counters + blockIdx.x, p.split_k, &last_flag)) return;
    if (writer) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            f4 sum = bv;
            for (int s = 0; s < p.split_k; s++) {
                sum += load_partial(p.partial + ((size_t)s * M + m) * p.N + n0);
            }
            h4 o;
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = (_Float16)sum[c];
            *(h4 *)(y + (size_t)m * p.N + n0) = o;
        }
    }
}

template <int BITS, int M, int TPM>
static int launch_grouped_one(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    constexpr int NSTEP = BITS == 4 ? 8 : 4;
    auto kern = grouped_kernel<BITS, M, TPM, NSTEP>;
    if (plan.lds_bytes > 65536) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, plan.grid_y, 1), dim3(plan.block), plan.lds_bytes, stream, p);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

template <int BITS>
static int launch_grouped_bits(const Params &p, const gptq_hip_plan &plan, hipStream_t stream)
{
    const int tpm = p.gpad / 16;
    if (p.M == 1) {
        switch (tpm) {
            case 1: return launch_grouped_one<BITS, 1, 1>(p, plan, stream);
            case 2: return launch_grouped_one<BITS, 1, 2>(p, plan, stream);
            case 3: return launch_grouped_one<BITS, 1, 3>(p, plan, stream);
            case 4: return launch_grouped_one<BITS, 1, 4>(p, plan, stream);
            case 6: return launch_grouped_one<BITS, 1, 6>(p, plan, stream);
            default: return GPTQ_HIP_ERR_UNSUPPORTED;
        }
    }
    if (p.M == 2) {
        switch (tpm) {
            case 1: return launch_grouped_one<BITS, 2, 1>(p, plan, stream);
            case 2: return launch_grouped_one<BITS, 2, 2>(p, plan, stream);
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
