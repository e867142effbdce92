// Shape dispatcher: a pure host function from (M, K, N, bits, group_size, act_order)
// to a launch plan.  It stands where the reference keeps a JSON database of tuned
// kernels per shape and an M-bucket switch
// (auto_gptq/nn_modules/tvm_untils/cache.py:11-62,
//  auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:77-127,138-189).
#include <string.h>

#include "gptq_internal.h"

namespace {

int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace

namespace gptq {

// Row tiles (of 16 groups) per activation row that the GROUPED kernel is built for.
int grouped_tpm(int groups, int M)
{
    const int tpm = ceil_div(groups, 16);
    const int max_tpm = M == 1 ? 4 : 2;  // (a six-tile instantiation spilled 60-70 registers and lost to STREAM)
    return tpm <= max_tpm ? tpm : 0;
}

// Upper bound of the number of distinct groups one K range of `kr` channels can touch.
int grouped_groups(int kr, int gs, int G, int act_order)
{
    int groups = act_order ? G : (kr - 1) / gs + 2;
    return groups > G ? G : groups;
}

// LDS of the STREAM kernel: the (scale, zero) table of 64 columns, or the reduction buffer of the
// waves along K (half of them write at a time), which reuses the same bytes.
int stream_lds_bytes(int bits, int K, int G, int group_size, int act_table, int row_tiles, int waves_k,
                     int wave_steps)
{
    (void)K;
    long long rows = G;
    if (!act_table) {
        const long long span = (long long)waves_k * wave_steps * kstep_of(bits);
        rows = (span - 1) / group_size + 2;
        if (rows > G) rows = G;
    }
    const long long table = rows * kStreamTableRow;
    const long long red = (long long)(waves_k / 2) * row_tiles * 16 * 64 * 4;
    const long long need = table > red ? table : red;
    return need > (1 << 30) ? (1 << 30) : (int)need;
}

size_t stream_xpack_bytes(int bits, int steps_pad, int rt_total)
{
    // + the depth of the kernel's A ring: its refills run past the end unclamped
    const size_t blocks = (size_t)steps_pad * (bits == 4 ? 1 : 4) + kStreamRingBlocks;
    return blocks * (size_t)rt_total * 1024;
}

size_t stream_gpack_bytes(int bits, int steps_pad, int act_table)
{
    const size_t blocks = (size_t)steps_pad * (bits == 4 ? 1 : 4) + kStreamRingBlocks;
    const size_t bytes = act_table ? blocks * 4 * 8 * sizeof(int32_t)
                                   : (size_t)(steps_pad + stream_pf(bits)) * 4 * sizeof(int32_t);
    return (bytes + 255) / 256 * 256;
}

// LDS of the GROUPED kernel for a K range of kr channels: operand tiles (+ slot masks in the
// compact two-tile layout) + the reduction buffer of the waves along K.
int grouped_lds_bytes(int kr, int M, int tpm, int waves_n, int waves_k, bool lite)
{
    const int red = waves_k * waves_n * M * 64 * 4;
    if (lite) return M * kr * 2 + 16 + red;  // x in unpack order, 16 zero bytes
    const int nblk8 = kr / 8;
    const bool compact = tpm == 2;
    const int stored = compact ? M : M * tpm;
    return nblk8 * stored * 256 + (compact ? nblk8 * 16 : 0) + waves_k * waves_n * M * 64 * 4;
}

}  // namespace gptq

namespace {

// GROUPED: rows expanded by group, M of 1 or 2 (one set of operand tiles per activation row; the packed
// layout for up to eight rows is plan_grouped_packed's).  Returns false when the shape does not fit
// (too many groups for the row tiles, or an LDS operand that no split makes small enough).
bool plan_grouped(int M, int K, int N, int bits, int gs, int G, int act_order, int force_split, int force_waves,
                  gptq_hip_plan *plan)
{
    const int kstep = gptq::kstep_of(bits);
    const int steps_total = ceil_div(K, kstep);
    const int waves_n = force_waves > 0 ? force_waves : 1;
    const int col_tiles = ceil_div(N, 64 * waves_n);
    if ((size_t)col_tiles * sizeof(int) > gptq::kCounterBytes) return false;
    const int lds_cap = gptq::kGroupedLdsCap;
    // a column tile per workgroup and no split is best (nothing crosses workgroups) unless
    // that leaves most of the 256 CUs idle; then as many K ranges as keep the workgroups within one per CU: a few
    // past it wait for a second turn of the chip (one row, us in the ranges named: 8192 x 5120, 80 tiles, in 2 / 3 / 4 /
    // 5: 10.8 / 10.3 / 15.3 / 14.9; 8192 x 6144, 96 tiles, in 2 / 3 / 4: 10.8 / 16.2 / 15.5; 8192 x 7168, 112 tiles: 11.1 / 16.4 /
    // 15.9; 13824 x 5120 int3 in 2 / 3 / 4: 12.1 / 11.0 / 13.8; 11008 x 4608, 72 tiles, in 3 / 4 / 5: 11.1 / 16.6 / 16.2)
    int want = force_split > 0 ? force_split : (col_tiles >= 128 ? 1 : 256 / col_tiles);
    // A workgroup's time is a chain of load latencies (~0.85 us per step of a wave) rather than its share of the
    // HBM bandwidth, and the sum across workgroups costs 2-4 us: while a wave's share of an unsplit K stays within
    // 512 channels (K <= 4096) one workgroup per column tile is faster than filling the chip, however few tiles
    // there are (4096 x 4096 on 64 CUs: int3 6.4 us against 7.6 in four ranges, int4 7.0 against 8.2).
    // Under an activation order (operand tiles, two barriers) the same holds up to 256 channels per wave
    // (2048 x 4096 int3: 5.9 us against 7.3 in four ranges; at 4096 x 4096 one range and four are level).
    if (force_split == 0 && ceil_div(steps_total, 8 / waves_n) * kstep <= (act_order ? 256 : 512)) want = 1;
    if (want > steps_total) want = steps_total;
    for (int want_split = want; want_split <= steps_total && want_split <= 256; want_split++) {
        if (force_split > 0 && want_split != want) return false;
        // uniform partition: every wave gets wave_steps steps, every workgroup waves_k of those
        int waves_k = 8 / waves_n;
        if (waves_k * want_split > steps_total) waves_k = steps_total / want_split;
        if (waves_k < 1) waves_k = 1;
        const int wave_steps = ceil_div(steps_total, want_split * waves_k);
        const int wg_steps = wave_steps * waves_k;
        const int split = ceil_div(steps_total, wg_steps);
        const int kr = wg_steps * kstep;
        // rows are counted per wave: the groups one wave's K range can touch
        const int tpm = gptq::grouped_tpm(gptq::grouped_groups(wave_steps * kstep, gs, G, act_order), M);
        if (tpm == 0) {
            if (act_order) return false;  // the group count does not shrink with the K range
            continue;
        }
        // int4 plans are sized for the tile layout and switch to the lean operand only afterwards
        const bool lite = gptq::grouped_lite(bits, K, gs, act_order != 0, tpm, M, kr, waves_n, waves_k, split);
        if (bits == 4 && gptq::grouped_lds_bytes(kr, M, tpm, waves_n, waves_k, false) > lds_cap) continue;
        const int lds = gptq::grouped_lds_bytes(kr, M, tpm, waves_n, waves_k, lite);
        if (lds > lds_cap) continue;
        plan->kernel = GPTQ_HIP_KERNEL_GROUPED;
        plan->row_tiles = M * tpm;
        plan->m_blocks = 1;
        plan->waves_n = waves_n;
        plan->waves_k = waves_k;
        plan->split_k = split;
        plan->k_chunk = kr;
        plan->grid_x = col_tiles;
        plan->grid_y = split;
        plan->grid_z = 1;
        plan->block = 64 * waves_n * waves_k;
        plan->lds_bytes = lds;
        plan->workspace_bytes = split > 1 ? gptq::kCounterBytes + (size_t)split * M * N * sizeof(float) : 0;
        return true;
    }
    return false;
}

// GROUPED with up to four activation rows packed into one operand tile, or up to eight into two
// (contiguous groups only).  The plan is sized for four or eight rows.
bool plan_grouped_packed(int M, int K, int N, int bits, int gs, int force_split, int force_waves, gptq_hip_plan *plan)
{
    const int kstep = gptq::kstep_of(bits);
    const int steps_total = ceil_div(K, kstep);
    const int waves_n = force_waves > 0 ? force_waves : 1;
    const int col_tiles = ceil_div(N, 64 * waves_n);
    if ((size_t)col_tiles * sizeof(int) > gptq::kCounterBytes) return false;
    int want = force_split > 0 ? force_split : (col_tiles >= 128 ? 1 : 256 / col_tiles);   // as in plan_grouped
    if (force_split == 0 && ceil_div(steps_total, 8 / waves_n) * kstep <= 512) want = 1;
    if (want > steps_total) want = steps_total;
    for (int want_split = want; want_split <= steps_total && want_split <= 256; want_split++) {
        if (force_split > 0 && want_split != want) return false;
        int waves_k = 8 / waves_n;
        if (waves_k * want_split > steps_total) waves_k = steps_total / want_split;
        if (waves_k < 1) waves_k = 1;
        const int wave_steps = ceil_div(steps_total, want_split * waves_k);
        const int wg_steps = wave_steps * waves_k;
        const int split = ceil_div(steps_total, wg_steps);
        const int kr = wg_steps * kstep;
        if (!gptq::grouped_packable(bits, K, gs, false, M, kr, waves_k)) continue;
        const int lds = gptq::grouped_lds_bytes(kr, gptq::packed_rows_of(M), 1, waves_n, waves_k, true);
        if (lds > gptq::kGroupedLdsCap) continue;
        plan->kernel = GPTQ_HIP_KERNEL_GROUPED;
        plan->row_tiles = gptq::packed_rows_of(M);
        plan->m_blocks = 1;
        plan->waves_n = waves_n;
        plan->waves_k = waves_k;
        plan->split_k = split;
        plan->k_chunk = kr;
        plan->grid_x = col_tiles;
        plan->grid_y = split;
        plan->grid_z = 1;
        plan->block = 64 * waves_n * waves_k;
        plan->lds_bytes = lds;
        plan->workspace_bytes =
            split > 1 ? gptq::kCounterBytes + (size_t)split * gptq::packed_rows_of(M) * N * sizeof(float) : 0;
        return true;
    }
    return false;
}

// STREAM: exact weights, any g_idx, any M; x pre-packed, waves independent.
// force_waves is the number of waves along K (1, 2, 4 or 8), 0 = choose.
int plan_stream(int M, int K, int N, int bits, int gs, int G, int act_order, int force_split, int force_waves,
                gptq_hip_plan *plan)
{
    const int kstep = gptq::kstep_of(bits);
    const int steps_total = ceil_div(K, kstep);
    const int pf = gptq::stream_pf(bits);
    const int rt = M <= 16 ? 1 : (M <= 32 ? 2 : gptq::stream_max_row_tiles());
    const int m_blocks = ceil_div(M, 16 * rt);
    const int col_tiles = ceil_div(N, 64);
    const long long tiles = (long long)col_tiles * m_blocks;
    const int act_table = gptq::stream_act_table(bits, gs, act_order);
    const bool can_split = (long long)M * N < (1LL << 32);  // indexing of the pass that adds the partial tiles

    // Waves come from column tiles x M blocks x waves along K inside a workgroup (their tiles meet in
    // LDS) x workgroups along K (their fp32 tiles cross the workspace and a reduce pass adds them:
    // ~3-4 us).  64-row tiles run four waves per workgroup (two workgroups share a CU); shorter
    // tiles eight while all workgroups still fit the chip (2048 wave slots at two per SIMD).
    // Workgroups along K bring the count to about one per CU (256); a long K per wave affords more.
    int waves_k = force_waves > 0 ? force_waves : (rt == 4 ? 4 : (tiles * 8 <= 2048 ? 8 : 4));
    while (waves_k > 1 && waves_k * pf > steps_total) waves_k >>= 1;
    int split = (int)((256 + tiles / 2) / tiles);
    // up to 32 rows a few workgroups past one per CU cost a second turn of the chip, as on the tiled kernels (us at 9 /
    // 32 rows in the ranges named: 8192 x 6144, 96 tiles, in 2 / 3: 13.7 / 17.7 and 19.6 / 24.3; 8192 x 5632 with an
    // activation order, 88 tiles: 17.6 / 25.6 and 21.5 / 30.0; 11008 x 4608, 72 tiles, in 3 / 4: 14.2 / 17.6 and 20.2 / 24.5;
    // 9216 x 9216 int3, 144 tiles, in 1 / 2: 33.0 / 44.6 and 33.7 / 46.0; 28672 x 8192, 128 tiles, in 2 / 3: 30.3 / 39.1)
    if (rt <= 2 && tiles <= 256 && tiles * split > 256) split = (int)(256 / tiles);
    if (split < 1) split = 1;
    if (rt == 1 && tiles >= 128 && tiles < 256 && K / waves_k >= 4096) split = ceil_div(384, (int)tiles);
    int cap = (int)((3LL * K * bits) / (128LL * M));
    if (cap < 1) cap = 1;
    if (split > cap) split = cap;
    if (split > 64) split = 64;
    if (force_split > 0) split = force_split;
    if (!can_split) {
        if (force_split > 1) return GPTQ_HIP_ERR_UNSUPPORTED;
        split = 1;
    }
    if (split * waves_k * pf > steps_total) split = steps_total / (waves_k * pf);
    if (split < 1) split = 1;
    int wave_steps = gptq::stream_wave_steps(bits, steps_total, split, waves_k);
    split = ceil_div(steps_total, wave_steps * waves_k);  // the split actually needed
    wave_steps = gptq::stream_wave_steps(bits, steps_total, split, waves_k);
    const int lds = gptq::stream_lds_bytes(bits, K, G, gs, act_table, rt, waves_k, wave_steps);
    if (lds > 150 * 1024) return GPTQ_HIP_ERR_UNSUPPORTED;  // more groups than the LDS table holds

    plan->kernel = GPTQ_HIP_KERNEL_STREAM;
    plan->row_tiles = rt;
    plan->m_blocks = m_blocks;
    plan->waves_n = 1;
    plan->waves_k = waves_k;
    plan->split_k = split;
    plan->k_chunk = kstep;
    plan->grid_x = col_tiles;
    plan->grid_y = split;
    plan->grid_z = m_blocks;
    plan->block = 64 * waves_k;
    plan->lds_bytes = lds;
    const int steps_pad = split * waves_k * wave_steps;
    size_t ws = gptq::kCounterBytes;
    if (split > 1) ws += ((size_t)split * M * N * sizeof(float) + 255) / 256 * 256;
    if (gptq::stream_direct(bits, K, rt, act_table, act_order)) {
        if (split == 1) ws = 0;  // no pack pass, no partial tiles: nothing to hold
    } else {
        ws += gptq::stream_xpack_bytes(bits, steps_pad, rt * m_blocks);
        ws += gptq::stream_gpack_bytes(bits, steps_pad, act_table);
    }
    plan->workspace_bytes = ws;
    return GPTQ_HIP_OK;
}

}  // namespace

extern "C" int gptq_hip_select(int M, int K, int N, int bits, int group_size, int act_order, gptq_hip_plan *plan)
{
    if (!plan) return GPTQ_HIP_ERR_BAD_ARG;
    memset(plan, 0, sizeof(*plan));
    if (bits != 3 && bits != 4) return GPTQ_HIP_ERR_BAD_ARG;
    if (M < 1 || K < 32 || N < 32) return GPTQ_HIP_ERR_BAD_ARG;
    if (K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;  // the packed format needs both
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    const int G = ceil_div(K, gs);
    // one group for the whole matrix: g_idx carries no information
    if (G == 1) act_order = 0;
    // GROUPED for decoding (M = 1); for M = 2 only where a workgroup holds all of K, since its
    // operand in LDS doubles with M and the cross-workgroup sum costs more than STREAM's pack pass.
    // With the lean operand (int3, contiguous groups) two rows also win when K is split (4096 x 4096
    // 9.0 against 9.2 us, 11008 x 4096 12.0 against 13.1).
    // Under an activation order every group a workgroup meets needs a row: past three row tiles
    // (48 groups) the expansion costs more than STREAM's lookup per weight (measured at N = 4096,
    // int3 / int4: K = 5120 16.1 / 11.6 us against 19.1 / 12.8; K = 8192 19.8 / 22.1 against 15.3 / 13.7;
    // K = 11008 79 / 93 against 20.1 / 16.8).
    // Many column tiles: every workgroup stages x for itself, and past 256 workgroups they run in
    // rounds, so a workgroup takes 128 columns (257..512 tiles) or 256 (more) when that does not
    // force a finer split of K (4096 x 22016: int3 14.4 -> 12.4 us, int4 17.7 -> 13.9; 9216 x 36864:
    // int3 35.9 -> 32.8, int4 55.4 -> 33.9; int4 8192 x 28672 35.6 -> 26.8, while int3 there keeps
    // 64 columns: 22.7 against 26.1 with K split in two).
    // A split into many K ranges leaves the sum to a long tail of workgroups: from eight ranges on
    // (int3: past eight) STREAM's own pass is cheaper (int4 36864 x 9216: 52.6 us in nine ranges
    // against 42.1; 4096 x 512: 14.6 / 15.0 us in 32 ranges against 8.3 / 7.1; 4096 x 2048 in eight
    // ranges: int3 8.0 against 8.5, int4 8.7 against 7.7).
    const int tiles64 = ceil_div(N, 64);
    const int wide = tiles64 > 512 ? 4 : (tiles64 > 256 ? 2 : 0);
    bool grouped = false;
    if (M <= 2) {
        gptq_hip_plan narrow;
        memset(&narrow, 0, sizeof(narrow));
        const bool have_narrow = plan_grouped(M, K, N, bits, gs, G, act_order, 0, 0, &narrow);
        const bool have_wide = wide && plan_grouped(M, K, N, bits, gs, G, act_order, 0, wide, plan);
        if (have_wide && (!have_narrow || plan->split_k <= narrow.split_k)) {
            grouped = true;
        } else if (have_narrow) {
            *plan = narrow;
            grouped = true;
        }
    }
    bool packed = false;
    if (M >= 2 && M <= (bits == 3 ? gptq::kPackedRows : 4) && !act_order) {
        // two to four rows for the matrix instructions of one (five to eight: of two; int4 gains nothing from
        // two tiles: 4096 x 11008, M = 8: 11.6 us against 10.6 on STREAM, while int3 takes 9.8 against 10.5) (contiguous groups, short K ranges per wave).
        // Against STREAM, int3 4096 x 11008: 7.9 us against 9.8 for two to four rows; int4: 8.9 against 10.2;
        // int3 9216 x 9216 in three K ranges: 15.7 against 24.  With K cut into four or more ranges the sum
        // across workgroups costs more than the packing saves (int4 4096 x 4096 in four: 9.0 against 8.6;
        // 11008 x 4096 in six: 16.7 against 11.8).
        gptq_hip_plan pn, pw;
        memset(&pn, 0, sizeof(pn));
        memset(&pw, 0, sizeof(pw));
        const bool have_narrow = plan_grouped_packed(M, K, N, bits, gs, 0, 0, &pn);
        const bool have_wide = wide && plan_grouped_packed(M, K, N, bits, gs, 0, wide, &pw);
        const gptq_hip_plan *best = nullptr;
        if (have_wide && (!have_narrow || pw.split_k <= pn.split_k)) {
            best = &pw;
        } else if (have_narrow) {
            best = &pn;
        }
        if (best && best->split_k <= 3) {
            *plan = *best;
            grouped = packed = true;
        }
    }
    if (grouped &&
        (M == 1 || packed || plan->split_k == 1 ||
         gptq::grouped_lite(bits, K, gs, act_order != 0, plan->row_tiles / M, M, plan->k_chunk, plan->waves_n,
                            plan->waves_k, plan->split_k)) &&
        (!act_order || plan->row_tiles / M <= 3)) {
        if (plan->split_k < (bits == 3 ? 9 : 8)) return GPTQ_HIP_OK;
        gptq_hip_plan alt;
        memset(&alt, 0, sizeof(alt));
        if (plan_stream(M, K, N, bits, gs, G, act_order, 0, 0, &alt) != GPTQ_HIP_OK) return GPTQ_HIP_OK;
        *plan = alt;
        return GPTQ_HIP_OK;
    }
    memset(plan, 0, sizeof(*plan));
    if (plan_stream(M, K, N, bits, gs, G, act_order, 0, 0, plan) == GPTQ_HIP_OK) return GPTQ_HIP_OK;
    memset(plan, 0, sizeof(*plan));
    return GPTQ_HIP_ERR_UNSUPPORTED;
}

extern "C" int gptq_hip_plan_for(int kernel, int M, int K, int N, int bits, int group_size, int act_order,
                                 int split_k, int waves_n, gptq_hip_plan *plan)
{
    gptq_hip_plan tmp;
    const int rc = gptq_hip_select(M, K, N, bits, group_size, act_order, &tmp);  // argument checks
    if (rc != GPTQ_HIP_OK) return rc;
    if (!plan || split_k < 0 || (waves_n != 0 && waves_n != 1 && waves_n != 2 && waves_n != 4 && waves_n != 8))
        return GPTQ_HIP_ERR_BAD_ARG;
    if (waves_n == 8 && kernel != GPTQ_HIP_KERNEL_STREAM) return GPTQ_HIP_ERR_BAD_ARG;
    memset(plan, 0, sizeof(*plan));
    const int gs = group_size == -1 ? K : group_size;
    const int G = ceil_div(K, gs);
    if (G == 1) act_order = 0;
    if (kernel == GPTQ_HIP_KERNEL_STREAM) {
        const int rc2 = plan_stream(M, K, N, bits, gs, G, act_order, split_k, waves_n, plan);
        if (rc2 != GPTQ_HIP_OK) memset(plan, 0, sizeof(*plan));
        return rc2;
    }
    if (kernel == GPTQ_HIP_KERNEL_GROUPED) {
        if (M <= 2 && plan_grouped(M, K, N, bits, gs, G, act_order, split_k, waves_n, plan)) return GPTQ_HIP_OK;
        if (M >= 2 && M <= gptq::kPackedRows && !act_order && plan_grouped_packed(M, K, N, bits, gs, split_k, waves_n, plan))
            return GPTQ_HIP_OK;
        memset(plan, 0, sizeof(*plan));
        return GPTQ_HIP_ERR_UNSUPPORTED;
    }
    return GPTQ_HIP_ERR_UNSUPPORTED;
}

// TILED: a workgroup per 64 columns and block of 32 * row_tiles rows, four waves along K; workgroups along K
// when the column tiles alone leave most CUs idle (their fp32 tiles cross the workspace, so the split stays
// within 3x the packed weights of traffic).
static int tiled_args_ok(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan)
{
    if (!plan) return GPTQ_HIP_ERR_BAD_ARG;
    memset(plan, 0, sizeof(*plan));
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8) return GPTQ_HIP_ERR_BAD_ARG;
    if (M < 1 || K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    if (!gptq::tiled_qualifies(K, N, bits, group_size == -1 ? K : group_size)) return GPTQ_HIP_ERR_UNSUPPORTED;
    return GPTQ_HIP_OK;
}

extern "C" int gptq_hip_select_tiled_decode(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan)
{
    const int ok = tiled_args_ok(M, K, N, bits, group_size, plan);
    if (ok != GPTQ_HIP_OK) return ok;
    if (M > gptq::kDecodeMaxRows) return GPTQ_HIP_ERR_UNSUPPORTED;
    const int gs = group_size == -1 ? K : group_size;
    {
        // Layers of up to 16 columns per CU (N <= 4096): one workgroup of sixteen waves per 16-column unit, all of
        // K staged once per workgroup (waves_n = 2 marks this kernel), when that fits LDS.  Every CU then has
        // work (a workgroup per 32-column tile leaves half of them idle): 11008 x 4096, one row, 9.0 / 9.3 us
        // (int4 / int3) against 10.4 / 11.0; 4096 x 4096 5.3 against 5.4-5.5.  Wider layers would give a workgroup
        // several units; there the kernel below is faster (4096 x 11008: 7.7 / 7.8 us against 9.0 / 9.3).
        const int mr = gptq::tiled_decode_rows(M);
        const int units = N / 16;
        const int nwg = units < gptq::kNumCUs ? units : gptq::kNumCUs;
        const int upw = ceil_div(units, nwg);
        const long long lds = gptq::tiled_decode16_lds_bytes(mr, K, K / gs, upw);
        // (long K: the kernel below with every tile halved, see tiled_decode_halves_all)
        if (M <= 4 && upw == 1 && lds <= 128 * 1024 && !gptq::tiled_decode_halves_all(N / 32, ceil_div(K, 64))) {
            plan->kernel = GPTQ_HIP_KERNEL_TILED_DECODE;
            plan->row_tiles = mr;
            plan->m_blocks = 1;
            plan->waves_n = 2;
            plan->waves_k = 16;
            plan->split_k = 1;
            plan->k_chunk = ceil_div(ceil_div(ceil_div(K, 64), 2), 16);  // virtual blocks per unit and wave
            plan->grid_x = nwg;
            plan->grid_y = 1;
            plan->grid_z = 1;
            plan->block = 1024;
            plan->lds_bytes = (int)lds;
            plan->workspace_bytes = 0;
            return GPTQ_HIP_OK;
        }
    }
    {
        // Otherwise: a workgroup per column tile of 32, enough waves along K to give the chip ~1000 waves, K cut
        // over workgroups only when the staged x would not fit LDS.
        const int mr = gptq::tiled_decode_rows(M);
        const int tiles = N / 32;
        const int S_total = ceil_div(K, 64);
        int kw = tiles * 4 >= 1024 ? 4 : (tiles * 8 >= 1024 ? 8 : 16);
        // and enough of them that a wave walks about sixteen blocks at most: a wave issues one instruction per
        // four clocks, so a long K wants more, shorter waves.  One row, us, kw = 4 / 8 / 16: 8192 x 8192
        // 12.1 / 9.4 / 9.5, 5120 x 13824 10.9 / 9.4 / 11.6, 6144 x 16384 12.7 / 11.0 / 12.4, 9216 x 9216
        // 16.3 / 13.6 / 14.6, 11008 x 11008 21.1 / 17.2 / 18.0, 13824 x 5120 19.9 / 12.6 / 10.6 (4096 x 11008
        // keeps four: 8.2 / 8.2 / 10.1; 28672 x 8192 40.0 / 28.0 / 24.7, 17920 x 6656 26.0 / 17.6 / 14.6, 11008 x 8192
        // 17.6 / 13.0 / 12.1): eight whenever four would walk more than sixteen blocks, sixteen only while that
        // keeps a CU at sixteen waves (one tile per CU)
        if (kw == 4 && ceil_div(S_total, 4) > 16) kw = 8;
        if (kw == 8 && ceil_div(S_total, 8) > 16 && tiles <= gptq::kNumCUs) kw = 16;
        // every tile in two halves: eight waves per half (14336 x 4096, one / four rows: 10.1 / 12.7 us with eight,
        // 9.9 / 12.9 with sixteen; 11008 x 4096 int3 8.4 / 11.2 and 8.5 / 11.4)
        const bool halves_all = gptq::tiled_decode_halves_all(tiles, S_total);
        if (halves_all) kw = 8;
        // five to eight rows: at most eight waves (sixteen leave a lane 128 registers, which the two sets of rows
        // do not fit into)
        if (mr == 8 && kw == 16) kw = 8;
        while (kw > 4 && kw > S_total) kw >>= 1;
        // K beyond 32768 channels with more tiles than CUs: cut over workgroups of eight waves so that a wave walks
        // about twelve blocks (36864 x 9216 int3, one group, one row, the pass that adds the ranges included: 34.6 us
        // uncut with 72 blocks per wave, 31.4 in two ranges; with the current kernel 28.4 in three, 27.6 in four,
        // 26.7 in six, 27.9 in nine, 29.1 in twelve; six ranges of four or sixteen waves 27.6 / 28.4; an odd number
        // of blocks per wave loses the paired epilogue: eight ranges 29.9.  Up to 32768 channels every cut measured
        // lost: 9216 x 9216 9.2 -> 11.8-13.3, 28672 x 8192 25.5 -> 29.1, 11008 x 11008 13.1 -> 16.1)
        int first_split = 1;
        if (S_total > 512 && !halves_all) {
            kw = 8;
            first_split = ceil_div(S_total, 8 * 12);
        }
        for (int split = first_split; split <= S_total; split++) {
            int wave_steps = ceil_div(S_total, split * kw);
            // an even number of blocks per wave keeps the paired epilogue (groups that are multiples of 128 channels)
            // (rounding up to a multiple of four, so that halved tiles come out in equal halves, cost more than
            // unequal halves do: 5120 x 13824, 9.7 -> 11.2 us with twelve blocks per wave instead of ten)
            if (gs % 128 == 0 && wave_steps > 1 && (wave_steps & 1) && split == 1) wave_steps++;
            if (ceil_div(S_total, wave_steps * kw) != split) continue;  // (the split this partition really needs)
            const int halved = gptq::tiled_decode_halved(tiles, wave_steps, split, kw, S_total, gs);
            const int span = gptq::tiled_decode_span(halved, tiles, wave_steps, kw, gs);
            const int groups = (span - 1) / gs + 2 < ceil_div(K, gs) ? (span - 1) / gs + 2 : ceil_div(K, gs);
            const int lds = gptq::tiled_decode_lds_bytes(mr, span, groups, kw);
            if (lds > 128 * 1024) continue;
            if (split > 1 && (long long)M * N >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
            plan->kernel = GPTQ_HIP_KERNEL_TILED_DECODE;
            plan->row_tiles = mr;
            plan->m_blocks = 1;
            plan->waves_n = 1;
            plan->waves_k = kw;
            plan->split_k = split;
            plan->k_chunk = wave_steps;
            // up to CUs / 2 tiles past a whole number per CU run as two halves along K, so that the fullest CU
            // holds half a tile more than the others, not a whole one (4096 x 11008: 344 tiles, 88 of them halved);
            // long layers of up to 4096 columns halve every tile
            plan->grid_x = tiles + halved;
            plan->grid_y = split;
            plan->grid_z = 1;
            plan->block = 64 * kw;
            plan->lds_bytes = lds;
            plan->workspace_bytes = split > 1 ? gptq::kCounterBytes + (size_t)split * M * N * sizeof(float)
                                    : (halved ? gptq::kCounterBytes + gptq::tiled_decode_slot_bytes(halved, mr) : 0);
            // (the halves of a tile meet in slots that must be all zero between launches)
            plan->flags = halved ? GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE : 0;
            return GPTQ_HIP_OK;
        }
        return GPTQ_HIP_ERR_UNSUPPORTED;
    }
}

namespace {

// K ranges of a matmul plan.  Workgroups of two or four row tiles hold a CU alone (264 and ~380 registers per lane),
// and two of one row tile on a CU share its vector ALU, which is what they wait for: either way the launch runs in
// turns of 256 workgroups, a turn lasts as long as a wave's walk, and a K that is cut costs a second pass over
// split x M x N floats.  The number of ranges is the one that makes
//     turns x blocks per wave x (us per block) + [split > 1] (2.5 + 0.8 us per MB of partial tiles)
// least (the fewest ranges within 3 % of it), with 0.4 / 0.58 / 0.94 / 1.7 us per block for 32 x 64, 64 x 64, 128 x 64
// and 128 x 128 waves.  Measured at 17 / 32 rows (one row tile; us in the ranges named): 8192 x 5632, 88 tiles, in 1 / 2 /
// 3 / 4: 22.0 / 17.9 / 22.4 / 20.2; 11008 x 6400, 100 tiles: 27.7 / 22.2 / 28.2 / 24.8; 8192 x 3328, 52 tiles, in 2 / 3 / 4 / 5:
// 17.7 / 15.7 / 15.9 / 20.3; 11008 x 4608, 72 tiles, in 2 / 3 / 4: 21.7 / 19.8 / 24.3; 16384 x 6144, 96 tiles, in 1 / 2 / 3 / 5:
// 36.7 / 27.8 / 35.2 / 31.1; 144 tiles at 32 rows in 1 / 2 / 3 / 5: 9216 x 9216 int3 22.1 / 25.9 / 21.9 / 24.1, 18432 x 9216
// 38.7 / -- / 33.6 / 35.2, 36864 x 9216 71.9 / -- / 58.4 / 57.6; 4096 x 11008 at 16 rows, 172 tiles, in 1 / 2: 13.4 / 19.1.
// Measured at more rows (us; tiles = workgroups per range): 9216 x 9216 int3, 144 tiles, 128 rows in 1 / 2 / 3 ranges 45.9 /
// 52.0 / 43.7, 256 rows (128 x 128 waves) 64.3 / 79.6 / 68.3; 36864 x 9216, 64 / 128 rows: 109 / 115 / 80 and 208 / 187 / 129
// (three ranges are 432 workgroups: two turns of a third of K instead of one turn of all of it, where two ranges
// are two turns of half); 18432 x 9216 at 128 rows 83.9 / 96.0 / 68.7; 8192 x 8192 at 256 rows, 128 tiles: 57.3 / 50.2 /
// 66.6; at 64 rows 8192 x 6144, 96 tiles: 28.3 / 24.1 / 30.2, 11008 x 4608, 72 tiles, in 2 / 3 / 4: 28.0 / 24.8 / 32.0,
// 8192 x 3328, 52 tiles, in 3 / 4 / 5: 19.8 / 18.7 / 24.7; 64-row blocks of narrow layers at 128 rows: 4096 x 4096 in
// 1 / 2 ranges 17.1 / 17.6, 2048 x 4096 11.5 / 13.2, 8192 x 4096 29.5 / 26.5.
int tiled_ranges(int at, bool wide, long long tiles, int S_total, int kwv, double out_elems, int cap)
{
    // One row tile: the count of turns holds for plans of one turn (above); two such workgroups on a CU also hide each
    // other's waits, so past one turn the count is too strict: plans of up to 128 tiles take the best plan of one turn,
    // wider ones are not cut, but for 129 to 160 tiles over a K of 9216 and more, which three ranges put on the chip
    // at once (432 to 480 workgroups: the 144-tile figures above; five ranges at 18432 x 9216 and 9 rows 41.8 against
    // 38.6 in three; 12288 x 12288, 192 tiles, in 1 / 4: 30.3 / 32.2; 6656 x 17920, 280 tiles, without an activation order at
    // 9 rows in 1 / 3: 26.8 / 30.5)
    const bool one_turn = at == 1;
    if (one_turn && tiles > 128) return tiles * 3 <= 480 && S_total >= 144 && cap >= 3 ? 3 : 1;
    const double us_per_block = at == 1 ? 0.4 : (at == 2 ? 0.58 : (wide ? 1.7 : 0.94));
    const int ring = gptq::tiled_ring(at);
    const int most = cap < 64 ? cap : 64;
    double cost[65];
    double best = 1e30;
    for (int s = 1; s <= most; s++) {
        cost[s] = 1e30;
        const int steps = ceil_div(S_total, s * kwv);
        if (s > 1 && (S_total / (s * kwv) < ring || ceil_div(S_total, steps * kwv) != s)) continue;
        if (s > 1 && one_turn && tiles * s > 256) continue;
        const double turns = (double)((tiles * s + 255) / 256);
        cost[s] = turns * steps * us_per_block + (s > 1 ? 2.5 + 0.8e-6 * 4.0 * s * out_elems : 0.0);
        if (cost[s] < best) best = cost[s];
    }
    for (int s = 1; s <= most; s++)
        if (cost[s] <= 1.03 * best) return s;
    return 1;
}

}  // namespace

extern "C" int gptq_hip_select_tiled(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan)
{
    // Up to four rows the decode kernels (one 4-row matrix instruction set per lane block); five to eight rows the
    // workgroup-per-tile decode kernel with two sets, for K up to 11008 (us at 5 / 8 rows, int4, against the matmul
    // kernel with one 32-row tile: 4096 x 11008 9.0 / 9.4 against 9.6 / 9.7, with an activation order 12.7 / 13.2
    // against 14.0 / 14.2; 11008 x 4096 9.9 / 10.3 against 16.7 / 17.2, with an activation order 15.1 / 15.8 against
    // 18.9 / 19.4; 4096 x 4096 7.2 / 7.8 against 9.4 / 9.5; longer K was not measured: eight staged rows of x).
    if (M >= 1 && (M <= gptq::kDecodeSelectRows || (M <= gptq::kDecodeMaxRows && K <= 11008))) {
        const int rc = gptq_hip_select_tiled_decode(M, K, N, bits, group_size, plan);
        if (rc != GPTQ_HIP_ERR_UNSUPPORTED || !plan) return rc;
    }
    const int ok = tiled_args_ok(M, K, N, bits, group_size, plan);
    if (ok != GPTQ_HIP_OK) return ok;
    int at = gptq::tiled_row_tiles(M);
    const int rw = 1, kwv = 4;
    // Narrow layers above 64 rows: where row blocks of 64 rows still find a CU each, they replace the 128-row blocks,
    // whose few workgroups had to cut K (partial tiles and a pass that adds them) to fill the chip (us at 96 / 128 /
    // 256 rows against 128-row blocks, int4 with an activation order: 4096 x 4096 16.8 / 17.1 / 21.7 against 20.1 /
    // 21.2 / 25.1, 2048 x 4096 11.4 / 11.5 / 13.0 against 15.2 / 15.5 / 16.0, 4096 x 2048 16.0 / 16.5 / 17.4 against
    // 17.4 / 18.6 / 24.5, 5120 x 5120 21.0 / 21.4 against 23.5 / 25.1, 6656 x 6656 27.1 / 27.5 against 29.4 / 30.8,
    // 4096 x 8192 18.9 / 19.5 against 22.9 / 24.5, 8192 x 8192 34.3 / 35.0 against 36.7 / 38.3; with more such blocks than
    // CUs they lose: 5120 x 5120 at 256 rows 36.6 against 31.0, 4096 x 11008 at 128 rows 31.1 against 24.8)
    // The same one step down, 33 to 64 rows as two blocks of 32, for K up to 4096 (48 / 64 rows: 4096 x 4096 13.2 / 13.5
    // against 14.4 / 14.9, 4096 x 8192 14.7 / 15.0 against 16.5 / 17.3, 2048 x 4096 9.6 / 9.8 against 11.4 / 11.8, 5120 x 5120
    // and 4096 x 2048 level; 8192 x 4096 21.1 / 20.9 against 19.2 / 19.8 and 11008 x 4096 24.1 / 24.3 against 22.9 / 23.8 stay)
    if (at == 4 && K <= 8192 && (long long)ceil_div(N / 32, 2) * ceil_div(M, 64) <= 256)
        at = 2;
    else if (at == 2 && K <= 4096 && (long long)ceil_div(N / 32, 2) * ceil_div(M, 32) <= 256)
        at = 1;
    const int rows = 32 * at * rw;
    const int m_blocks = ceil_div(M, rows);
    // several row blocks: 128 columns per wave (waves_n = 2), which halves the x fragments a matrix instruction
    // needs; one row block keeps 64 columns, for more workgroups
    // (when that still leaves a workgroup for two of three CUs, or when K is long: the fragments of a row block
    // then need the larger share of L2 that fewer, wider workgroups leave them.  4096 x 11008: 256 rows 49.6 ->
    // 41.9 us, 1024 rows 142 -> 123; 11008 x 4096, 512 rows: 127 -> 88; 4096 x 4096, 512 rows, 128 workgroups:
    // 33.5 -> 40.4, so not there)
    const bool wide = at == 4 && m_blocks >= 2 && ((long long)ceil_div(N / 32, 4) * m_blocks >= 172 || K > 8192);
    const int ct = wide ? 4 : 2;
    const int col_pairs = ceil_div(N / 32, ct);
    const int S_total = ceil_div(K, 64);
    const long long tiles = (long long)col_pairs * m_blocks;
    int cap = (int)((3LL * K * bits) / (128LL * M));
    if (cap < 1) cap = 1;
    int split = tiled_ranges(at, wide, tiles, S_total, kwv, (double)M * N, cap);
    if (split < 1) split = 1;
    if (split > cap) split = cap;
    if ((long long)M * N >= (1LL << 32)) split = 1;  // indexing of the pass that adds the partial tiles
    // every wave gets at least a ring of blocks
    while (split > 1 && S_total / (split * kwv) < gptq::tiled_ring(at)) split--;
    // the partial tiles of all ranges together stay within 10 MB where fewer ranges still give two of three CUs a
    // workgroup (11008 x 4096 at 256 rows, 128 x 128 waves, us in 2 / 3 / 4 ranges: int4 49.9 / 45.3 / 52.3, int3 50.9 /
    // 46.5 / 53.3: the fourth range adds 4 MB of fp32 tiles to write and to read again)
    // (plans of one turn only: in a plan of two turns one range less is one and a half times the walk)
    while (split > 1 && tiles * split <= 256 && (long long)split * M * N * 4 > (10LL << 20) && tiles * (split - 1) >= 172)
        split--;
    const int wave_steps = ceil_div(S_total, split * kwv);
    split = ceil_div(S_total, wave_steps * kwv);
    plan->kernel = GPTQ_HIP_KERNEL_TILED;
    plan->row_tiles = at * rw;
    plan->m_blocks = m_blocks;
    plan->waves_n = ct / 2;
    plan->waves_k = kwv;
    plan->split_k = split;
    plan->k_chunk = wave_steps;  // blocks of 64 positions per wave
    plan->grid_x = col_pairs;
    plan->grid_y = split;
    plan->grid_z = m_blocks;
    plan->block = 64 * rw * kwv;
    plan->lds_bytes = gptq::tiled_lds_bytes(at * rw, kwv);
    size_t ws = gptq::kCounterBytes;
    if (split > 1) ws += ((size_t)split * M * N * sizeof(float) + 255) / 256 * 256;
    ws += (size_t)gptq::tiled_pack_blocks(split, kwv, wave_steps) * 4 * (size_t)(at * rw * m_blocks) * 1024;
    plan->workspace_bytes = ws;
    return GPTQ_HIP_OK;
}

// The transposed product gx[M, K] = gy[M, N] @ W^T on the matmul kernel: the reduction runs over the layer's N
// columns (blocks of 64), the result has K columns (tiles of 32 positions, two per workgroup).
extern "C" int gptq_hip_select_tiled_transposed(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan)
{
    const int ok = tiled_args_ok(M, K, N, bits, group_size, plan);
    if (ok != GPTQ_HIP_OK) return ok;
    int at = gptq::tiled_row_tiles(M);
    const int kwv = 4, ct = 2;
    const int col_pairs = ceil_div(K / 32, ct);
    const int S_total = ceil_div(N, 64);
    // shorter row blocks where they still find a CU each, as in the forward plan (the result has K columns here and
    // the reduction runs over N; us at 64 / 128 / 256 rows against the taller blocks, int4: 4096 x 4096 17.8 / 22.5 / 27.9
    // against 17.7 / 25.6 / 33.0, 8192 x 4096 20.7 / 26.6 against 22.2 / 31.1, 4096 x 2048 13.1 / 16.5 / 20.1 against 14.5 /
    // 21.7 / 24.5, 2048 x 4096 14.9 / 18.0 / 23.3 against 15.1 / 21.0 / 30.3, 5120 x 5120 at 128 rows 27.2 against 29.6; a
    // reduction over 8192 keeps the tall blocks: 4096 x 8192 at 128 / 256 rows 30.9 / 48.4 against 29.6 / 45.8)
    if (at == 4 && N < 8192 && (long long)col_pairs * ceil_div(M, 64) <= 256)
        at = 2;
    else if (at == 2 && N <= 4096 && (long long)col_pairs * ceil_div(M, 32) <= 256)
        at = 1;
    const int m_blocks = ceil_div(M, 32 * at);
    const long long tiles = (long long)col_pairs * m_blocks;
    int cap = (int)((3LL * N * bits) / (128LL * M));   // the fp32 tiles of a split stay within 3x the packed weights
    if (cap < 1) cap = 1;
    // (ranges by the same count of turns as the forward plan)
    int split = tiled_ranges(at, false, tiles, S_total, kwv, (double)M * K, cap);
    if (split < 1) split = 1;
    if (split > cap) split = cap;
    if ((long long)M * K >= (1LL << 32)) split = 1;
    while (split > 1 && S_total / (split * kwv) < gptq::tiled_ring(at)) split--;
    // the table of a workgroup's K range must fit its LDS
    while (ceil_div(S_total, split * kwv) * kwv > gptq::kTiledTMaxBlocks) split++;
    if (split > 1 && (long long)M * K >= (1LL << 32)) return GPTQ_HIP_ERR_UNSUPPORTED;
    const int wave_steps = ceil_div(S_total, split * kwv);
    split = ceil_div(S_total, wave_steps * kwv);
    plan->kernel = GPTQ_HIP_KERNEL_TILED;
    plan->row_tiles = at;
    plan->m_blocks = m_blocks;
    plan->waves_n = 1;
    plan->waves_k = kwv;
    plan->split_k = split;
    plan->k_chunk = wave_steps;
    plan->grid_x = col_pairs;
    plan->grid_y = split;
    plan->grid_z = m_blocks;
    plan->block = 64 * kwv;
    plan->lds_bytes = gptq::tiled_t_lds_bytes(at, kwv, wave_steps);
    size_t ws = gptq::kCounterBytes;
    if (split > 1) ws += ((size_t)split * M * K * sizeof(float) + 255) / 256 * 256;
    ws += (size_t)gptq::tiled_pack_blocks(split, kwv, wave_steps) * 4 * (size_t)(at * m_blocks) * 1024;
    plan->workspace_bytes = ws;
    return GPTQ_HIP_OK;
}

namespace {

// Where the tiled kernels were measured faster than the ones that read the checkpoint layout or its channel-sorted
// copy, on MI355X with the weights cold (us per call, graph replay, group size 128 unless said):
//   * up to 4 rows, layers of up to 4096 columns (decode kernel with a workgroup per 16 columns, or every tile in two
//     halves along K from 4096 channels): always.  4096 x 4096: 4.1-4.2 at one row, 5.2 at four, against 6.8-7.5
//     and 7.8-10.5; 11008 x 4096: int4 9.0-9.4 / 11.5 against 13.5 / 15.3, int3 8.7 / 11.1 against 10.9 / 15.2;
//   * up to 4 rows, wider layers (a workgroup per 32 columns): K = 4096: one and two rows always, three and four up
//     to 16384 columns (4096 x 11008 with an activation order, one / two / four rows: int4 7.8 / 8.1 / 9.8 against
//     8.1 / 11.0 / 11.1, int3 7.3 / 7.7 / 9.7 against 7.7 / 10.2 / 10.3; 4096 x 22016 one row 9.7 / 10.3 against
//     11.4 / 12.8).  Longer K, one and two rows: always (8192 x 8192 9.7 / 9.9 against 14.0 / 13.3, 8192 x 28672
//     24.6 / 26.4 against 32.3 / 30.2, 28672 x 8192 25.1 / 31.7 against 50.1 / 39.2; 36864 x 9216 int3 with one
//     group, K cut in six ranges: 26.7 against 37.3); three and four rows: K up to 6656, and
//     up to 11008 for layers of up to 8192 columns (beyond, the four staged rows of x cost more than they save:
//     8192 x 28672 41.9 against 30.4);
//   * 5 to 8 rows, K up to 11008: the decode kernel with two sets of four rows (5 / 8 rows, int4 / int3, against the
//     better of the other copies: 4096 x 11008 with an activation order 12.7 / 13.2 and 12.8 / 13.3 against 13.4 / 13.6
//     and 12.5 / 12.6 on the sorted copy, without one 9.0 / 9.4 against 9.6 / 9.7 on the matmul kernel; 11008 x 4096 with
//     an activation order 15.1 / 15.8 and 15.3 / 16.1 against 15.8 / 16.0 and 16.4 / 16.9, without one 9.9 / 10.3 against
//     13.1; 4096 x 4096 7.2 / 7.8 against 9.9, with an activation order 9.5 / 10.2 against 10.9 (int3 12.3));
//   * 5 to 16 rows otherwise: only layers without an activation order, K up to 4096 and more than 4096 columns (the matmul
//     kernel then reads x itself, one launch: 4096 x 11008 int4, 5 / 8 / 16 rows: 10.6 / 10.7 / 11.5 against 11.2 /
//     11.3 / 12.5; int3 from nine rows); with an activation order the pack pass makes it 14.6 against 13.4 at 8 rows;
//   * 17 to 128 rows: almost everywhere (4096 x 11008 with an activation order, 32 / 64 / 128 rows: 14.8 / 19.2 /
//     26.6 against 18.1 / 22.1 / 34.1), but for K of 8192 and more where the checkpoint-layout STREAM kernel has
//     nothing to look up per weight: 4-bit layers without an activation order up to 64 rows, of 8192 columns and more
//     (17 / 32 / 64 rows: 8192 x 8192 22.0 / 22.5 / 26.0 against 19.9 / 20.7 / 24.5, 8192 x 28672 43.6 / 43.2 / 54.8 against 40.9 /
//     41.2 / 54.4, 28672 x 8192 level at 42.1 / 42.8 / 56.7 against 43.2 / 44.0 / 55.7; narrower ones keep the tiled copy, whose
//     K ranges fill one turn of the chip: 13824 x 5120 18.7 / 19.5 / 26.7 against 22.8 / 23.1 / 26.9, 17920 x 6656 27.7 / 27.9 /
//     38.8 against 31.1 / 31.2 / 39.3, 8192 x 6144 19.3 / 19.2 / 22.7 against 23.8 / 24.5 / 30.0, 11008 x 4608 17.4 / 17.9 / 22.8
//     against 24.1 / 24.4 / 30.6) and layers of
//     one group beyond 16384 columns (9216 x 36864, 32 / 128 rows: 53.4 / 134 against 52.9 / 126; up to 16384 columns
//     they keep the tiled copy, whose K ranges are cut by turns of the chip: 36864 x 9216, 17 / 32 rows: 57.1 / 57.6
//     against 70.2 / 72.4, 64 / 128 / 256 rows in three ranges 80.2 / 129 / 223 against 98.1 / 172 / 255; 18432 x 9216 33.2 /
//     33.8 against 45.0 / 45.9, 64 / 128 / 256 rows 47.0 / 68.7 / 114 against 56.5 / 90.3 / 134; 9216 x 9216 21.6 / 22.0 against
//     31.4 / 32.0, 64 / 128 / 256 rows 30.2 / 45.9 / 64.3 against 36.2 / 48.4 / 72.6; 12288 x 12288 level at 28); with an activation order also
//     beyond 20480 channels (28672 x 8192 at 17 / 32 rows, int4 48.4 / 48.4 against 47.9 / 49.0, int3 48.4 / 49.0 against
//     49.6 / 50.7; 64 rows 61.6 / 65.5 against 64.9 / 67.9);
//   * above 128 rows: K up to 8192 (4096 x 11008, 512 rows: 75 against 95; 11008 x 4096: 127 against 81), and up to
//     256 rows the longer layers named in the function.
bool tiled_wins(int M, int K, int N, bool act_order, int bits, bool one_group)
{
    if (M <= 4) {
        if (N <= 4096) return true;
        if (K <= 4096) return M <= 2 || N < 16384;
        if (M <= 2) return true;
        if (K > 32768) return false;
        return K <= 6656 || (K <= 11008 && N <= 8192);
    }
    if (M <= 8 && K <= 11008) return true;   // the decode kernel with two sets of rows (below)
    if (M <= 16) {
        // (without an activation order and K beyond 4096, against the STREAM kernel that reads x itself, 9 / 16 rows:
        // 13824 x 5120 12.4 / 15.2 against 15.9 / 18.1, 5120 x 13824 10.0 / 14.1 against 13.1 / 15.1, 11008 x 11008 19.3 / 24.9
        // against 22.0 / 25.9, 6656 x 6656 11.2 / 12.8 against 13.7 / 15.2, 28672 x 8192 level at 31.3 / 35.5; up to 4096
        // columns level or behind: 11008 x 4096 16.1 / 16.1 against 13.1 / 14.2, 8192 x 4096 11.1 / 12.6 against 11.5 / 12.5;
        // and behind at 8192 channels: 8192 x 6144 14.6 / 16.8 against 13.6 / 15.2, 8192 x 8192 17.6 / 19.0 against 14.1 / 15.5)
        if (!act_order && K > 4096) return N > 4096 && !(K > 6656 && K < 11008);
        if (!act_order) return K <= 4096 && N > 4096 && (M >= 9 || bits == 4);
        // with an activation order (9 to 16 rows; pack pass + matmul against the sorted copy, whose time grows with the
        // rows): 4096 x 11008 from twelve rows (9 / 12 / 16 rows, int4: 13.5 / 13.5 / 13.5 against 13.1 / 13.8 / 14.6; int3
        // 13.6 / 13.5 / 13.5 against 13.5 / 13.9 / 15.2), 3-bit layers of up to 4096 columns always (4096 x 4096: 12.3 / 12.4 /
        // 12.4 against 13.0 / 13.2 / 13.8; 4-bit there stays on the checkpoint tensors: 12.7 against 11.1); 11008 x 4096 stays
        // on the sorted copy (18.3-18.9 against 15.9-18.7)
        return K <= 4096 && ((N > 4096 && M >= 12) || (bits == 3 && N <= 4096));
    }
    if (M <= 128) {
        if (one_group && K > 8192 && N > 16384) return false;
        if (M <= 64 && K >= 8192 && N >= 8192 && bits == 4 && !act_order) return false;
        return true;
    }
    // up to 256 rows also K up to 11008, and any K with an activation order (192 / 256 rows against the checkpoint
    // tensors: 11008 x 4096 with an activation order at 256 rows, K in three ranges, 3-bit 46.5 against 51.2, 4-bit 45.3
    // against 48.5; 11008 x 11008 4-bit 85.9 against 109.6 at 256 rows; with an activation order 17920 x 6656 96.4 / 99.6
    // against 112 / 116, 28672 x 8192 4-bit 169 / 172 against 178 / 192, 3-bit 165 / 166 against 169 / 192; without one
    // the longer layers are level or behind: 28672 x 8192 167 / 169 against 164 / 169, 13824 x 5120 at 192 rows 54.7
    // against 46.3)
    return K <= 8192 || (M <= 256 && (K <= 11008 || act_order || (one_group && N <= 16384)));
}

// The plan gptq_hip_gemm_sorted runs for M rows of a layer whose channels were sorted by group, if that path covers
// the problem: the GROUPED family, or up to kSortedMaxRows rows on the STREAM kernel that reads x itself behind the
// pass that reorders x (that pass costs a launch, ~2 us: int3 gains 2-4 us over the per-weight lookups of the
// unsorted kernel at every size measured, int4 1-2 us at 4096 x 11008 and 11008 x 4096 but loses 0.7 us at
// 4096 x 4096).
bool sorted_plan(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan)
{
    const int gs = group_size == -1 ? K : group_size;
    if ((bits != 3 && bits != 4) || K >= 65536 || K % gs != 0 || gs % (bits == 4 ? 8 : 32) != 0) return false;
    if (gptq_hip_select(M, K, N, bits, group_size, 0, plan) != GPTQ_HIP_OK) return false;
    if (plan->kernel == GPTQ_HIP_KERNEL_GROUPED) return true;
    if (plan->kernel == GPTQ_HIP_KERNEL_STREAM && M <= gptq::kSortedMaxRows && plan->row_tiles == 1)
        return bits == 3 || (long long)K * N >= (1LL << 25);
    return false;
}

}  // namespace

extern "C" int gptq_hip_select_route(int M, int K, int N, int bits, int group_size, int act_order, unsigned copies,
                                     const int *switch_rows, gptq_hip_route *route)
{
    if (!route) return GPTQ_HIP_ERR_BAD_ARG;
    memset(route, 0, sizeof(*route));
    route->copy = GPTQ_HIP_ROUTE_LIBRARY;
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8) return GPTQ_HIP_ERR_BAD_ARG;
    if (M < 1 || K < 32 || N < 32 || K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    const unsigned all = GPTQ_HIP_COPY_CHECKPOINT | GPTQ_HIP_COPY_SORTED | GPTQ_HIP_COPY_TILED;
    if (copies == 0 || (copies & ~all)) return GPTQ_HIP_ERR_BAD_ARG;
    static const int kDefaultSwitch[3] = {1152, 1024, 640};
    const int *sw = switch_rows ? switch_rows : kDefaultSwitch;
    if (sw[0] < 0 || sw[1] < 0 || sw[2] < 0) return GPTQ_HIP_ERR_BAD_ARG;
    const int gs = group_size == -1 ? K : group_size;
    const bool one_group = gs >= K;
    const bool act = act_order && !one_group;
    const bool fused_bits = bits == 3 || bits == 4;   // the widths the kernels on the checkpoint layout take
    const bool tiled_ok = (copies & GPTQ_HIP_COPY_TILED) && gptq::tiled_qualifies(K, N, bits, gs);
    auto take_tiled = [&]() {
        if (gptq_hip_select_tiled(M, K, N, bits, group_size, &route->plan) != GPTQ_HIP_OK) {
            memset(&route->plan, 0, sizeof(route->plan));
            return false;
        }
        route->copy = GPTQ_HIP_ROUTE_TILED;
        return true;
    };
    if (copies == GPTQ_HIP_COPY_TILED) {
        // the tiled copy is all the layer has: every M runs there
        if (tiled_ok && take_tiled()) return GPTQ_HIP_OK;
        return GPTQ_HIP_ERR_UNSUPPORTED;
    }
    bool tiled = false;
    if (!fused_bits) {
        if (!tiled_ok) return GPTQ_HIP_OK;   // 2 and 8 bits have no other fused kernels: the library
        tiled = true;
    } else if (tiled_ok && tiled_wins(M, K, N, act, bits, one_group)) {
        tiled = true;
    }
    int threshold = sw[0];
    if (threshold && !tiled) {   // off the tiled copy the library GEMM wins earlier
        if (sw[1] && sw[1] < threshold) threshold = sw[1];
        if (act && sw[2] && sw[2] < threshold) threshold = sw[2];
    }
    if (threshold && M >= threshold) return GPTQ_HIP_OK;
    if (tiled && take_tiled()) return GPTQ_HIP_OK;
    if (!fused_bits) return GPTQ_HIP_OK;
    if ((copies & GPTQ_HIP_COPY_SORTED) && act && M <= gptq::kSortedMaxRows &&
        sorted_plan(M, K, N, bits, group_size, &route->plan)) {
        route->copy = GPTQ_HIP_ROUTE_SORTED;
        return GPTQ_HIP_OK;
    }
    memset(&route->plan, 0, sizeof(route->plan));
    if (copies & GPTQ_HIP_COPY_CHECKPOINT) {
        const int rc = gptq_hip_select(M, K, N, bits, group_size, act ? 1 : 0, &route->plan);
        if (rc == GPTQ_HIP_OK) {
            route->copy = GPTQ_HIP_ROUTE_CHECKPOINT;
            return GPTQ_HIP_OK;
        }
        memset(&route->plan, 0, sizeof(route->plan));
        if (rc != GPTQ_HIP_ERR_UNSUPPORTED) return rc;
    }
    return GPTQ_HIP_OK;   // no fused kernel covers the call: dequant + library GEMM
}

extern "C" size_t gptq_hip_workspace_bytes(int M, int K, int N, int bits, int group_size, int act_order)
{
    gptq_hip_plan plan;
    if (gptq_hip_select(M, K, N, bits, group_size, act_order, &plan) != GPTQ_HIP_OK) return 0;
    return plan.workspace_bytes;
}
