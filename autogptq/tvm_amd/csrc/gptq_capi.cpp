// extern "C" entry points: argument checks, plan lookup, launch.  Nothing here
// allocates, synchronises or throws; see include/gptq_hip.h for the contract.
#include <stdint.h>

#include "gptq_internal.h"

namespace {

bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

// wide: also 2 and 8 bits (the dequant kernel and the tiled format cover them, the kernels on the checkpoint layout do not)
int check_common(const int32_t *qweight, const int32_t *qzeros, const void *scales, int K, int N, int bits,
                 int group_size, bool wide = false)
{
    if (!qweight || !qzeros || !scales) return GPTQ_HIP_ERR_BAD_ARG;
    if (bits != 3 && bits != 4 && !(wide && (bits == 2 || bits == 8))) return GPTQ_HIP_ERR_BAD_ARG;
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if ((long long)K * N * bits / 8 >= (1LL << 31)) return GPTQ_HIP_ERR_UNSUPPORTED;  // kernels use 32-bit byte offsets
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    if (!aligned(qweight, 16) || !aligned(qzeros, 4) || !aligned(scales, 8)) return GPTQ_HIP_ERR_BAD_ARG;
    return GPTQ_HIP_OK;
}

int validate_plan(const gptq_hip_plan &pl, int M, int K, int N, int bits, int G, int gs, int act_order)
{
    const int kstep = gptq::kstep_of(bits);
    const int steps_total = (K + kstep - 1) / kstep;
    if (pl.kernel == GPTQ_HIP_KERNEL_STREAM) {
        if (pl.waves_n != 1 || (pl.waves_k != 1 && pl.waves_k != 2 && pl.waves_k != 4 && pl.waves_k != 8))
            return GPTQ_HIP_ERR_UNSUPPORTED;
        if (pl.row_tiles != 1 && pl.row_tiles != 2 && pl.row_tiles != 4) return GPTQ_HIP_ERR_UNSUPPORTED;
        if (pl.block != 64 * pl.waves_k || pl.split_k < 1 || pl.grid_y != pl.split_k) return GPTQ_HIP_ERR_BAD_ARG;
        if ((long long)pl.grid_x * 64 < N || pl.m_blocks < 1 || pl.grid_z != pl.m_blocks ||
            (long long)pl.m_blocks * 16 * pl.row_tiles < M)
            return GPTQ_HIP_ERR_BAD_ARG;
        if (pl.split_k > 1 && (long long)M * N >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;  // reduce pass indexing
        const int wave_steps = gptq::stream_wave_steps(bits, steps_total, pl.split_k, pl.waves_k);
        // every workgroup along K must start inside K
        if ((long long)(pl.split_k - 1) * pl.waves_k * wave_steps >= steps_total) return GPTQ_HIP_ERR_BAD_ARG;
        const int act_table = gptq::stream_act_table(bits, gs, act_order);
        if (pl.lds_bytes > 160 * 1024 ||
            pl.lds_bytes < gptq::stream_lds_bytes(bits, K, G, gs, act_table, pl.row_tiles, pl.waves_k, wave_steps))
            return GPTQ_HIP_ERR_BAD_ARG;
        return GPTQ_HIP_OK;
    }
    if (pl.waves_n != 1 && pl.waves_n != 2 && pl.waves_n != 4) return GPTQ_HIP_ERR_UNSUPPORTED;
    if (pl.waves_k < 1 || pl.waves_n * pl.waves_k > 8) return GPTQ_HIP_ERR_UNSUPPORTED;
    if (pl.block != 64 * pl.waves_n * pl.waves_k) return GPTQ_HIP_ERR_BAD_ARG;
    if (pl.split_k < 1 || pl.split_k > steps_total) return GPTQ_HIP_ERR_BAD_ARG;
    if (pl.grid_x * 64 * pl.waves_n < N || pl.grid_y != pl.split_k) return GPTQ_HIP_ERR_BAD_ARG;
    if (pl.lds_bytes > 160 * 1024) return GPTQ_HIP_ERR_BAD_ARG;
    if (pl.split_k > 1 && (size_t)pl.grid_x * (pl.grid_z > 0 ? pl.grid_z : 1) * sizeof(int) > gptq::kCounterBytes)
        return GPTQ_HIP_ERR_UNSUPPORTED;
    if (pl.kernel == GPTQ_HIP_KERNEL_GROUPED) {
        if (M > gptq::kPackedRows || pl.grid_z != 1) return GPTQ_HIP_ERR_UNSUPPORTED;
        // k_chunk is the K range of one workgroup: waves_k * wave_steps whole steps
        if (pl.k_chunk < kstep * pl.waves_k || pl.k_chunk % (kstep * pl.waves_k) != 0) return GPTQ_HIP_ERR_BAD_ARG;
        const int kr = pl.k_chunk;
        if ((long long)kr * pl.split_k < (long long)steps_total * kstep) return GPTQ_HIP_ERR_BAD_ARG;
        const bool packed = pl.row_tiles == gptq::packed_rows_of(M) && gptq::grouped_packable(bits, K, gs, act_order != 0, M, kr, pl.waves_k);
        if (M > 2 || packed) {
            // packed rows: one operand tile, LDS and partial sums sized for four rows
            if (!packed) return GPTQ_HIP_ERR_UNSUPPORTED;
            if (pl.lds_bytes < gptq::grouped_lds_bytes(kr, gptq::packed_rows_of(M), 1, pl.waves_n, pl.waves_k, true))
                return GPTQ_HIP_ERR_BAD_ARG;
            return GPTQ_HIP_OK;
        }
        if (pl.row_tiles % M != 0) return GPTQ_HIP_ERR_UNSUPPORTED;
        const int tpm = pl.row_tiles / M;
        const int need_tpm = gptq::grouped_tpm(gptq::grouped_groups(kr / pl.waves_k, gs, G, act_order), M);
        if (need_tpm == 0 || tpm != need_tpm) return GPTQ_HIP_ERR_UNSUPPORTED;
        if (pl.lds_bytes < gptq::grouped_lds_bytes(kr, M, tpm, pl.waves_n, pl.waves_k,
                                                   gptq::grouped_lite(bits, K, gs, act_order != 0, tpm, M, kr,
                                                                      pl.waves_n, pl.waves_k, pl.split_k)))
            return GPTQ_HIP_ERR_BAD_ARG;
        return GPTQ_HIP_OK;
    }
    return GPTQ_HIP_ERR_UNSUPPORTED;
}

}  // namespace

// kmap != nullptr: qweight holds the channels sorted by group (g_idx must then be nullptr)
static int run_gemm(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *g_idx,
             const int32_t *kmap, const void *bias, void *y, void *workspace, size_t workspace_bytes, int M, int K,
             int N, int bits, int group_size, const gptq_hip_plan *plan, void *stream)
{
    if (!x || !y || !plan || M < 1) return GPTQ_HIP_ERR_BAD_ARG;
    int rc = check_common(qweight, qzeros, scales, K, N, bits, group_size);
    if (rc != GPTQ_HIP_OK) return rc;
    if (!aligned(x, 16) || !aligned(y, 8) || (bias && !aligned(bias, 8)) || (g_idx && !aligned(g_idx, 16)))
        return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    const int G = (K + gs - 1) / gs;
    const int act_order = (g_idx != nullptr && G > 1) ? 1 : 0;
    if (G == 1) g_idx = nullptr;  // a single group: the gather has nothing to choose
    rc = validate_plan(*plan, M, K, N, bits, G, gs, act_order);
    if (rc != GPTQ_HIP_OK) return rc;

    gptq::Params p;
    p.x = x;
    p.qweight = (const uint32_t *)qweight;
    p.qzeros = (const uint32_t *)qzeros;
    p.scales = scales;
    p.g_idx = g_idx;
    p.bias = bias;
    p.y = y;
    p.partial = nullptr;
    p.counters = nullptr;
    p.M = M;
    p.K = K;
    p.N = N;
    p.G = G;
    p.group_size = gs;
    const int kstep = gptq::kstep_of(bits);
    p.steps_total = (K + kstep - 1) / kstep;
    p.split_k = plan->split_k;
    p.chunk_steps = plan->k_chunk / kstep;
    p.xs_rows = 16 * plan->row_tiles;
    p.row_tiles = plan->row_tiles;
    p.waves_n = plan->waves_n;
    p.waves_k = plan->waves_k;
    p.wave_steps = plan->kernel == GPTQ_HIP_KERNEL_GROUPED
                       ? plan->k_chunk / kstep / plan->waves_k
                       : (p.steps_total + plan->split_k * plan->waves_k - 1) / (plan->split_k * plan->waves_k);
    const bool packed_rows = plan->kernel == GPTQ_HIP_KERNEL_GROUPED && plan->row_tiles == gptq::packed_rows_of(M) &&
                             gptq::grouped_packable(bits, K, gs, act_order != 0, M, plan->k_chunk, plan->waves_k);
    p.gpad = plan->kernel == GPTQ_HIP_KERNEL_GROUPED ? (packed_rows ? 16 : 16 * (plan->row_tiles / M)) : 0;
    p.xpack = nullptr;
    p.gpack = nullptr;
    p.rt_total = 0;
    p.steps_pad = 0;
    p.act_table = 0;
    p.direct = 0;
    p.gdiv_magic = 0;
    p.gdiv_add = 0;
    p.kmap = nullptr;
    p.xsrc = nullptr;
    p.wave_div_magic = 0;
    if (plan->kernel == GPTQ_HIP_KERNEL_GROUPED && !g_idx && gs % (bits == 4 ? 8 : 32) == 0) {
        // group of lane block r = r / d, d = lane blocks per group, as a multiply-high (r < 65536)
        const uint32_t d = (uint32_t)(gs / (bits == 4 ? 8 : 32));
        if (d == 1) {
            p.gdiv_add = 1;
        } else {
            p.gdiv_magic = (uint32_t)((1ull << 32) / d) + 1u;
        }
    }
    size_t ws_plan = workspace_bytes;  // bytes of the workspace the plan itself may use
    if (kmap && (plan->kernel == GPTQ_HIP_KERNEL_STREAM || packed_rows)) {
        // small batches on a sorted layer: x goes into the sorted channel order first (one small pass
        // into the tail of the workspace), then the kernel for contiguous groups reads it directly
        if (plan->kernel == GPTQ_HIP_KERNEL_STREAM &&
            (M > gptq::kSortedMaxRows || plan->row_tiles != 1 ||
             !gptq::stream_direct(bits, K, 1, gptq::stream_act_table(bits, gs, 0), false)))
            return GPTQ_HIP_ERR_UNSUPPORTED;
        const size_t head = gptq::sorted_x_offset(plan->workspace_bytes);
        const size_t xs_bytes = (size_t)M * K * 2;
        if (!workspace || workspace_bytes < head + xs_bytes || !aligned(workspace, 16)) return GPTQ_HIP_ERR_WORKSPACE;
        void *xs = (char *)workspace + head;
        rc = gptq::launch_permute_x(x, kmap + K, xs, M, K, stream);
        if (rc != GPTQ_HIP_OK) return rc;
        p.x = xs;
        ws_plan = head;
    } else if (kmap) {
        // positions are below 65536 and a wave holds at least one step: the multiply-high is exact
        if (plan->kernel != GPTQ_HIP_KERNEL_GROUPED) return GPTQ_HIP_ERR_UNSUPPORTED;
        // a workgroup that holds all of K, or a short x, walks x once and keeps its channels; with K
        // split and a long x it looks its channels up instead (measured crossover near K = 6000)
        if (plan->split_k == 1 || K <= 6144) {
            p.kmap = kmap;
        } else {
            p.xsrc = kmap + K;
        }
        p.wave_div_magic = (uint32_t)((1ull << 32) / (uint32_t)(p.wave_steps * kstep)) + 1u;
    }
    if (plan->kernel == GPTQ_HIP_KERNEL_STREAM) {
        // workspace: counters | partial tiles (split_k > 1) | packed x | packed table offsets
        p.wave_steps = gptq::stream_wave_steps(bits, p.steps_total, plan->split_k, plan->waves_k);
        p.steps_pad = plan->split_k * plan->waves_k * p.wave_steps;
        p.rt_total = plan->row_tiles * plan->m_blocks;
        p.act_table = gptq::stream_act_table(bits, gs, act_order);
        const size_t part =
            plan->split_k > 1 ? ((size_t)plan->split_k * M * N * sizeof(float) + 255) / 256 * 256 : 0;
        p.direct = gptq::stream_direct(bits, K, plan->row_tiles, p.act_table, g_idx != nullptr);
        // the kernel that reads x itself covers one tile of 16 rows and ignores the grid's M extent
        if (plan->row_tiles == 1 && (M > 16 || plan->m_blocks != 1)) return GPTQ_HIP_ERR_BAD_ARG;
        p.gdiv_magic = 0;
        p.gdiv_add = 0;
        if (p.direct) {
            if (!p.act_table) {
                // group of lane block r = r / d, d = lane blocks per group, as a multiply-high
                const uint32_t d = (uint32_t)(gs / (bits == 4 ? 8 : 32));
                if (d == 1) {
                    p.gdiv_add = 1;
                } else {
                    p.gdiv_magic = (uint32_t)((1ull << 32) / d) + 1u;
                }
            }
            if (plan->split_k > 1) {
                const size_t need = gptq::kCounterBytes + part;
                if (!workspace || ws_plan < need || !aligned(workspace, 16)) return GPTQ_HIP_ERR_WORKSPACE;
                p.counters = (int *)workspace;
                p.partial = (float *)((char *)workspace + gptq::kCounterBytes);
            }
            return gptq::launch_stream(p, bits, *plan, stream);
        }
        const size_t xb = gptq::stream_xpack_bytes(bits, p.steps_pad, p.rt_total);
        const size_t gb = gptq::stream_gpack_bytes(bits, p.steps_pad, p.act_table);
        if (xb >= (1ull << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;  // the kernel uses 32-bit byte offsets
        const size_t need = gptq::kCounterBytes + part + xb + gb;
        if (!workspace || workspace_bytes < need || !aligned(workspace, 16)) return GPTQ_HIP_ERR_WORKSPACE;
        p.counters = (int *)workspace;
        p.partial = (float *)((char *)workspace + gptq::kCounterBytes);
        p.xpack = (char *)workspace + gptq::kCounterBytes + part;
        p.gpack = (int32_t *)((char *)p.xpack + xb);
        return gptq::launch_stream(p, bits, *plan, stream);
    }
    if (plan->split_k > 1) {
        // a packed-row plan indexes its partial sums by the rows it is sized for (4 or 8), not by M
        const size_t part_rows = packed_rows ? (size_t)gptq::packed_rows_of(M) : (size_t)M;
        const size_t need = gptq::kCounterBytes + (size_t)plan->split_k * part_rows * N * sizeof(float);
        if (!workspace || ws_plan < need || !aligned(workspace, 16)) return GPTQ_HIP_ERR_WORKSPACE;
        p.counters = (int *)workspace;
        p.partial = (float *)((char *)workspace + gptq::kCounterBytes);
    }
    if (plan->kernel == GPTQ_HIP_KERNEL_GROUPED) return gptq::launch_grouped(p, bits, *plan, stream);
    return GPTQ_HIP_ERR_UNSUPPORTED;
}

extern "C" int gptq_hip_gemm_plan(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                  const int32_t *g_idx, const void *bias, void *y, void *workspace,
                                  size_t workspace_bytes, int M, int K, int N, int bits, int group_size,
                                  const gptq_hip_plan *plan, void *stream)
{
    return run_gemm(x, qweight, qzeros, scales, g_idx, nullptr, bias, y, workspace, workspace_bytes, M, K, N, bits,
                    group_size, plan, stream);
}

extern "C" int gptq_hip_gemm_sorted(const void *x, const int32_t *qweight_sorted, const int32_t *qzeros,
                                    const void *scales, const int32_t *kmap, const void *bias, void *y,
                                    void *workspace, size_t workspace_bytes, int M, int K, int N, int bits,
                                    int group_size, const gptq_hip_plan *plan, void *stream)
{
    if (!kmap || !aligned(kmap, 16)) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    // the map holds 16-bit positions; a group is a whole number of unpack blocks
    if (K >= 65536 || K % gs != 0 || gs % (bits == 4 ? 8 : 32) != 0) return GPTQ_HIP_ERR_UNSUPPORTED;
    gptq_hip_plan chosen;
    if (!plan) {
        const int rc = gptq_hip_select(M, K, N, bits, group_size, 0, &chosen);
        if (rc != GPTQ_HIP_OK) return rc;
        plan = &chosen;
    }
    if (plan->kernel != GPTQ_HIP_KERNEL_GROUPED && !(plan->kernel == GPTQ_HIP_KERNEL_STREAM && M <= gptq::kSortedMaxRows))
        return GPTQ_HIP_ERR_UNSUPPORTED;
    return run_gemm(x, qweight_sorted, qzeros, scales, nullptr, kmap, bias, y, workspace, workspace_bytes, M, K, N,
                    bits, group_size, plan, stream);
}

extern "C" int gptq_hip_sort_channels(const int32_t *qweight, const int32_t *g_idx, int32_t *qweight_sorted,
                                      int32_t *kmap, int K, int N, int bits, int group_size, void *stream)
{
    if (!qweight || !g_idx || !qweight_sorted || !kmap || qweight == qweight_sorted) return GPTQ_HIP_ERR_BAD_ARG;
    if (bits != 3 && bits != 4) return GPTQ_HIP_ERR_BAD_ARG;
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    if (!aligned(qweight, 16) || !aligned(qweight_sorted, 16) || !aligned(kmap, 16) || !aligned(g_idx, 4))
        return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    if (K >= 65536 || K % gs != 0 || gs % (bits == 4 ? 8 : 32) != 0) return GPTQ_HIP_ERR_UNSUPPORTED;
    return gptq::launch_sort_channels((const uint32_t *)qweight, g_idx, (uint32_t *)qweight_sorted, kmap, K, N, K / gs,
                                      bits, gs, stream);
}

extern "C" size_t gptq_hip_sorted_workspace_bytes(int M, int K, int N, int bits, int group_size)
{
    gptq_hip_plan plan;
    if (gptq_hip_select(M, K, N, bits, group_size, 0, &plan) != GPTQ_HIP_OK) return 0;
    const int gs = group_size == -1 ? K : group_size;
    const bool packed_rows = plan.kernel == GPTQ_HIP_KERNEL_GROUPED && plan.row_tiles == gptq::packed_rows_of(M) &&
                             gptq::grouped_packable(bits, K, gs, false, M, plan.k_chunk, plan.waves_k);
    if ((plan.kernel == GPTQ_HIP_KERNEL_STREAM && M <= gptq::kSortedMaxRows) || packed_rows)
        return gptq::sorted_x_offset(plan.workspace_bytes) + (size_t)M * K * 2;
    return plan.workspace_bytes;
}

extern "C" size_t gptq_hip_tiled_bytes(int K, int N, int bits)
{
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0 || (bits != 2 && bits != 3 && bits != 4 && bits != 8)) return 0;
    return (size_t)((K + 63) / 64 * 64) * (size_t)N * bits / 8;
}

extern "C" int gptq_hip_tile_prepare(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                     const int32_t *g_idx, void *qtile, uint32_t *sz, int32_t *xsrc, uint16_t *kinv,
                                     int K, int N, int bits, int group_size, void *stream)
{
    if (!qtile || !sz || !xsrc || !kinv || (const void *)qweight == qtile) return GPTQ_HIP_ERR_BAD_ARG;
    const int rc = check_common(qweight, qzeros, scales, K, N, bits, group_size, true);
    if (rc != GPTQ_HIP_OK) return rc;
    if (!aligned(qtile, 16) || !aligned(sz, 4) || !aligned(xsrc, 16) || !aligned(kinv, 16) || (g_idx && !aligned(g_idx, 4)))
        return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    if (!gptq::tiled_qualifies(K, N, bits, gs)) return GPTQ_HIP_ERR_UNSUPPORTED;
    return gptq::launch_tile_prepare((const uint32_t *)qweight, (const uint32_t *)qzeros, scales, g_idx, (uint32_t *)qtile,
                                     sz, xsrc, kinv, K, N, K / gs, bits, gs, stream);
}

extern "C" int gptq_hip_gemm_tiled(const void *x, const void *qtile, const uint32_t *sz, const int32_t *xsrc,
                                   const uint16_t *kinv, const void *bias, void *y, void *workspace,
                                   size_t workspace_bytes, int M, int K, int N, int bits, int group_size,
                                   const gptq_hip_plan *plan, void *stream)
{
    if ((xsrc == nullptr) != (kinv == nullptr) || (kinv && !aligned(kinv, 16))) return GPTQ_HIP_ERR_BAD_ARG;
    if (!x || !qtile || !sz || !y || M < 1) return GPTQ_HIP_ERR_BAD_ARG;
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8) return GPTQ_HIP_ERR_BAD_ARG;
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    if (!aligned(x, 16) || !aligned(qtile, 16) || !aligned(sz, 4) || !aligned(y, 8) || (bias && !aligned(bias, 8)) ||
        (xsrc && !aligned(xsrc, 16)))
        return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    if (!gptq::tiled_qualifies(K, N, bits, gs)) return GPTQ_HIP_ERR_UNSUPPORTED;
    if ((long long)((K + 63) / 64 * 64) * N * bits / 8 >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    gptq_hip_plan chosen;
    if (!plan) {
        const int rc = gptq_hip_select_tiled(M, K, N, bits, group_size, &chosen);
        if (rc != GPTQ_HIP_OK) return rc;
        plan = &chosen;
    }
    if (plan->kernel == GPTQ_HIP_KERNEL_TILED_DECODE && plan->waves_n == 2) {
        // one workgroup per CU, 16-column units
        const int mr = plan->row_tiles;
        if (M > gptq::kDecodeMaxRows || mr != gptq::tiled_decode_rows(M)) return GPTQ_HIP_ERR_UNSUPPORTED;
        const int units = N / 16;
        const int V_all = ((K + 63) / 64 + 1) / 2;
        if (plan->block != 1024 || plan->waves_k != 16 || plan->split_k != 1 || plan->grid_x < 1 || plan->grid_x > units ||
            plan->grid_y != 1 || plan->grid_z != 1 || plan->k_chunk != (V_all + 15) / 16)
            return GPTQ_HIP_ERR_BAD_ARG;
        const int upw = (units + plan->grid_x - 1) / plan->grid_x;
        if (plan->lds_bytes < gptq::tiled_decode16_lds_bytes(mr, K, K / gs, upw) || plan->lds_bytes > 160 * 1024)
            return GPTQ_HIP_ERR_BAD_ARG;
        return gptq::launch_tiled_decode16(x, qtile, sz, kinv, bias, y, M, K, N, K / gs, bits, gs, *plan, stream);
    }
    if (plan->kernel == GPTQ_HIP_KERNEL_TILED_DECODE) {
        const int mr = plan->row_tiles, kw = plan->waves_k;
        const int S_all = (K + 63) / 64;
        if (M > gptq::kDecodeMaxRows || mr != gptq::tiled_decode_rows(M)) return GPTQ_HIP_ERR_UNSUPPORTED;
        // grid_x: a workgroup per tile, or the planner's halved tiles on top
        const int halved = plan->grid_x - N / 32;
        if (halved != 0 && halved != gptq::tiled_decode_halved(N / 32, plan->k_chunk, plan->split_k, kw, S_all, gs))
            return GPTQ_HIP_ERR_BAD_ARG;
        // a caller that runs halved tiles has to know what their workspace asks for
        if (halved != 0 && !(plan->flags & GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE)) return GPTQ_HIP_ERR_BAD_ARG;
        // and a plan that says so while it writes partial sums (K cut over workgroups, whole tiles) would leave them in
        // a workspace that has to stay zero
        if (halved == 0 && (plan->flags & GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE)) return GPTQ_HIP_ERR_BAD_ARG;
        if ((kw != 4 && kw != 8 && kw != 16) || plan->block != 64 * kw || plan->split_k < 1 || plan->k_chunk < 1 ||
            plan->grid_y != plan->split_k || plan->grid_z != 1 ||
            (long long)plan->split_k * kw * plan->k_chunk < S_all ||
            (long long)(plan->split_k - 1) * kw * plan->k_chunk >= S_all)  // every workgroup starts inside K
            return GPTQ_HIP_ERR_BAD_ARG;
        const int span = gptq::tiled_decode_span(halved, N / 32, plan->k_chunk, kw, gs);
        const int G_all = K / gs;
        const int groups = (span - 1) / gs + 2 < G_all ? (span - 1) / gs + 2 : G_all;
        if (plan->lds_bytes < gptq::tiled_decode_lds_bytes(mr, span, groups, kw) || plan->lds_bytes > 160 * 1024)
            return GPTQ_HIP_ERR_BAD_ARG;
        float *part = nullptr;
        if (plan->split_k > 1) {
            if ((long long)M * N >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
            const size_t need = gptq::kCounterBytes + (size_t)plan->split_k * M * N * sizeof(float);
            if (!workspace || !aligned(workspace, 16) || workspace_bytes < need) return GPTQ_HIP_ERR_WORKSPACE;
            part = (float *)((char *)workspace + gptq::kCounterBytes);
        }
        unsigned long long *slots = nullptr;
        if (halved > 0) {
            const size_t need = gptq::kCounterBytes + gptq::tiled_decode_slot_bytes(halved, mr);
            if (!workspace || !aligned(workspace, 16) || workspace_bytes < need) return GPTQ_HIP_ERR_WORKSPACE;
            slots = (unsigned long long *)((char *)workspace + gptq::kCounterBytes);
        }
        return gptq::launch_tiled_decode(x, qtile, sz, kinv, bias, y, part, slots, M, K, N, G_all, bits, gs, *plan, stream);
    }
    // the plan must be one this family runs, sized for this problem
    const int rts = plan->row_tiles;  // 32-row tiles per workgroup
    const int S_total = (K + 63) / 64;
    if (plan->kernel != GPTQ_HIP_KERNEL_TILED || (rts != 1 && rts != 2 && rts != 4)) return GPTQ_HIP_ERR_UNSUPPORTED;
    const int kwv = 4;
    const int ct = 2 * plan->waves_n;   // 32-column tiles per wave: 2, or 4 (with four row tiles only)
    if ((ct != 2 && ct != 4) || (ct == 4 && rts != 4)) return GPTQ_HIP_ERR_BAD_ARG;
    if (plan->block != 64 * kwv || plan->waves_k != kwv || plan->split_k < 1 || plan->k_chunk < 1 || plan->m_blocks < 1 ||
        plan->grid_x != (N / 32 + ct - 1) / ct || plan->grid_y != plan->split_k || plan->grid_z != plan->m_blocks ||
        (long long)plan->m_blocks * 32 * rts < M || (long long)plan->split_k * kwv * plan->k_chunk < S_total ||
        plan->lds_bytes < gptq::tiled_lds_bytes(rts, kwv) || plan->lds_bytes > 160 * 1024)
        return GPTQ_HIP_ERR_BAD_ARG;
    if (plan->split_k > 1 && (long long)M * N >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    const size_t part = plan->split_k > 1 ? ((size_t)plan->split_k * M * N * sizeof(float) + 255) / 256 * 256 : 0;
    const size_t xb = (size_t)gptq::tiled_pack_blocks(plan->split_k, kwv, plan->k_chunk) * 4 * (size_t)(rts * plan->m_blocks) * 1024;
    if (!workspace || !aligned(workspace, 16) || workspace_bytes < gptq::kCounterBytes + part + xb) return GPTQ_HIP_ERR_WORKSPACE;
    float *partial = (float *)((char *)workspace + gptq::kCounterBytes);
    char *xpack = (char *)workspace + gptq::kCounterBytes + part;
    return gptq::launch_tiled(x, qtile, sz, xsrc, bias, y, xpack, partial, M, K, N, K / gs, bits, gs, *plan, stream);
}

extern "C" size_t gptq_hip_tiled_transposed_bytes(int K, int N, int bits)
{
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0 || (bits != 2 && bits != 3 && bits != 4 && bits != 8)) return 0;
    return (size_t)K * (size_t)((N + 63) / 64 * 64) * bits / 8;
}

extern "C" size_t gptq_hip_tiled_transposed_table_bytes(int K, int N, int group_size)
{
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0 || group_size == 0 || group_size < -1) return 0;
    const int gs = group_size == -1 ? K : group_size;
    if (K % gs != 0) return 0;
    return (size_t)(K / gs) * (size_t)((N + 63) / 64) * 256;
}

extern "C" int gptq_hip_tile_prepare_transposed(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                                const int32_t *xsrc, void *qtile_t, uint32_t *szt, int K, int N, int bits,
                                                int group_size, void *stream)
{
    if (!qtile_t || !szt || (const void *)qweight == qtile_t) return GPTQ_HIP_ERR_BAD_ARG;
    const int rc = check_common(qweight, qzeros, scales, K, N, bits, group_size, true);
    if (rc != GPTQ_HIP_OK) return rc;
    if (!aligned(qtile_t, 16) || !aligned(szt, 16) || (xsrc && !aligned(xsrc, 16))) return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    if (!gptq::tiled_qualifies(K, N, bits, gs)) return GPTQ_HIP_ERR_UNSUPPORTED;
    if ((long long)K * ((N + 63) / 64 * 64) * bits / 8 >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    return gptq::launch_tile_prepare_t((const uint32_t *)qweight, (const uint32_t *)qzeros, scales, xsrc,
                                       (uint32_t *)qtile_t, szt, K, N, K / gs, bits, stream);
}

extern "C" int gptq_hip_gemm_tiled_transposed(const void *gy, const void *qtile_t, const uint32_t *szt,
                                              const int32_t *xsrc, void *gx, void *workspace, size_t workspace_bytes,
                                              int M, int K, int N, int bits, int group_size, const gptq_hip_plan *plan,
                                              void *stream)
{
    if (!gy || !qtile_t || !szt || !gx || M < 1) return GPTQ_HIP_ERR_BAD_ARG;
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8) return GPTQ_HIP_ERR_BAD_ARG;
    if (K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    if (!aligned(gy, 16) || !aligned(qtile_t, 16) || !aligned(szt, 16) || !aligned(gx, 8) || (xsrc && !aligned(xsrc, 16)))
        return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    if (!gptq::tiled_qualifies(K, N, bits, gs)) return GPTQ_HIP_ERR_UNSUPPORTED;
    if ((long long)K * ((N + 63) / 64 * 64) * bits / 8 >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    gptq_hip_plan chosen;
    if (!plan) {
        const int rc = gptq_hip_select_tiled_transposed(M, K, N, bits, group_size, &chosen);
        if (rc != GPTQ_HIP_OK) return rc;
        plan = &chosen;
    }
    // the plan must be one this product runs, sized for this problem
    const int rts = plan->row_tiles, kwv = 4;
    const int S_total = (N + 63) / 64;
    if (plan->kernel != GPTQ_HIP_KERNEL_TILED || (rts != 1 && rts != 2 && rts != 4) || plan->waves_n != 1)
        return GPTQ_HIP_ERR_UNSUPPORTED;
    if (plan->block != 64 * kwv || plan->waves_k != kwv || plan->split_k < 1 || plan->k_chunk < 1 || plan->m_blocks < 1 ||
        plan->grid_x != (K / 32 + 1) / 2 || plan->grid_y != plan->split_k || plan->grid_z != plan->m_blocks ||
        (long long)plan->m_blocks * 32 * rts < M || (long long)plan->split_k * kwv * plan->k_chunk < S_total ||
        kwv * plan->k_chunk > gptq::kTiledTMaxBlocks || plan->lds_bytes < gptq::tiled_t_lds_bytes(rts, kwv, plan->k_chunk) ||
        plan->lds_bytes > 160 * 1024)
        return GPTQ_HIP_ERR_BAD_ARG;
    if (plan->split_k > 1 && (long long)M * K >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    const size_t part = plan->split_k > 1 ? ((size_t)plan->split_k * M * K * sizeof(float) + 255) / 256 * 256 : 0;
    const size_t xb = (size_t)gptq::tiled_pack_blocks(plan->split_k, kwv, plan->k_chunk) * 4 * (size_t)(rts * plan->m_blocks) * 1024;
    if (!workspace || !aligned(workspace, 16) || workspace_bytes < gptq::kCounterBytes + part + xb) return GPTQ_HIP_ERR_WORKSPACE;
    float *partial = (float *)((char *)workspace + gptq::kCounterBytes);
    char *xpack = (char *)workspace + gptq::kCounterBytes + part;
    return gptq::launch_tiled_t(gy, qtile_t, szt, xsrc, gx, xpack, partial, M, K, N, bits, gs, *plan, stream);
}

extern "C" int gptq_hip_gemm(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                             const int32_t *g_idx, const void *bias, void *y, void *workspace,
                             size_t workspace_bytes, int M, int K, int N, int bits, int group_size, void *stream)
{
    gptq_hip_plan plan;
    const int rc = gptq_hip_select(M, K, N, bits, group_size, g_idx != nullptr, &plan);
    if (rc != GPTQ_HIP_OK) return rc;
    return gptq_hip_gemm_plan(x, qweight, qzeros, scales, g_idx, bias, y, workspace, workspace_bytes, M, K, N,
                              bits, group_size, &plan, stream);
}

extern "C" int gptq_hip_dequant(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                const int32_t *g_idx, void *w, int K, int N, int bits, int group_size,
                                void *stream)
{
    if (!w) return GPTQ_HIP_ERR_BAD_ARG;
    const int rc = check_common(qweight, qzeros, scales, K, N, bits, group_size, true);
    if (rc != GPTQ_HIP_OK) return rc;
    const int gs = group_size == -1 ? K : group_size;
    const int G = (K + gs - 1) / gs;
    return gptq::launch_dequant((const uint32_t *)qweight, (const uint32_t *)qzeros, scales, g_idx, w, K, N, G, bits,
                                gs, stream);
}

extern "C" int gptq_hip_workspace_init(void *workspace, size_t workspace_bytes, void *stream)
{
    if (workspace_bytes == 0) return GPTQ_HIP_OK;
    if (!workspace || workspace_bytes % 4 != 0 || !aligned(workspace, 4)) return GPTQ_HIP_ERR_BAD_ARG;
    // (most plans only need the counters at the head to start at zero; a decode plan with halved tiles needs all of it)
    return gptq::launch_fill_zero(workspace, workspace_bytes, stream);
}

extern "C" const char *gptq_hip_strerror(int status)
{
    switch (status) {
        case GPTQ_HIP_OK: return "ok";
        case GPTQ_HIP_ERR_BAD_ARG: return "bad argument (null or misaligned pointer, size, bits or group_size)";
        case GPTQ_HIP_ERR_UNSUPPORTED: return "shape or plan not covered by the kernels";
        case GPTQ_HIP_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case GPTQ_HIP_ERR_LAUNCH: return "HIP launch failed";
        default: return "unknown status";
    }
}

extern "C" int gptq_hip_abi_version(void) { return GPTQ_HIP_ABI_VERSION; }

#ifndef GPTQ_HIP_BUILD_ID
#define GPTQ_HIP_BUILD_ID "unknown"
#endif
extern "C" const char *gptq_hip_build_id(void) { return GPTQ_HIP_BUILD_ID; }
