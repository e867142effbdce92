// Internal declarations shared by the dispatcher, the launchers and the C ABI.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "../../../include/gptq_hip.h"

namespace gptq {

// Arguments common to all matmul kernels (device pointers are borrowed for the launch).
struct Params {
    const void *x;           // fp16 [M, K]
    const uint32_t *qweight; // [K/32*bits, N]
    const uint32_t *qzeros;  // [G, N/32*bits]
    const void *scales;      // fp16 [G, N]
    const int32_t *g_idx;    // [K] or nullptr (k / group_size)
    const void *bias;        // fp16 [N] or nullptr
    void *y;                 // fp16 [M, N]
    float *partial;          // [split_k, M, N] when split_k > 1
    int *counters;           // one per (m block, column tile) when split_k > 1; zero between calls
    int M, K, N, G, group_size;
    int steps_total;   // ceil(K / KSTEP): KSTEP = 32 (int4) or 128 (int3)
    int split_k;       // workgroups per column tile
    int chunk_steps;   // steps staged in LDS at a time
    int xs_rows;       // rows of x kept in LDS per workgroup
    int row_tiles;     // 16-row tiles per wave
    int gpad;          // GROUPED kernel: rows per activation row = groups rounded up to 16
    int waves_n;       // waves of the workgroup along N
    int waves_k;       // waves of the workgroup along K
    int wave_steps;    // steps per wave along K (uniform partition of K made by the host)
    // STREAM kernel: x re-laid into matrix-instruction fragment order by its pack pass
    void *xpack;       // [steps_pad * NB][rt_total][64 lanes][8] fp16
    int32_t *gpack;    // table row byte offsets: per weight [steps_pad * NB][4][8], or per lane block [steps_pad][4]
    int rt_total;      // 16-row tiles over all M blocks
    int steps_pad;     // steps walked by all waves of a column tile together (>= steps_total)
    int act_table;     // 1: one (scale, zero) lookup per weight; 0: one per lane block
    int direct;        // 1: no pack pass, the kernel reads x and g_idx itself (M <= 16)
    uint32_t gdiv_magic;  // direct, contiguous groups: group of lane block r = umulhi(r, magic) + (add ? r : 0)
    int gdiv_add;
    // GROUPED kernel on a layer whose channels were sorted by group when it was loaded
    const int32_t *kmap;  // [K] or nullptr: channel k sits at position (kmap[k] & 0xffff) of the sorted
                          // qweight, counted in the order the unpack yields codes; kmap[k] >> 16 = its group
    const int32_t *xsrc;  // [K] or nullptr: xsrc[j] = the channel of x whose codes are j-th along K in the sorted qweight; the
                          // kernel follows kmap when a workgroup holds all of K and xsrc when K is split
    uint32_t wave_div_magic;  // position / channels per wave = umulhi(position, magic), positions < 65536
};

// k handled by one wave step: 4 lane groups x (8 | 32) codes
inline int kstep_of(int bits) { return bits == 4 ? 32 : 128; }

// byte size of the head of the workspace that holds the split-K counters
static const size_t kCounterBytes = 16384;

// GROUPED kernel sizing, shared by the dispatcher and the plan check
int grouped_tpm(int groups, int M);
int grouped_groups(int kr, int gs, int G, int act_order);
int grouped_lds_bytes(int kr, int M, int tpm, int waves_n, int waves_k, bool lite);
// LDS the GROUPED plans may use
static const int kGroupedLdsCap = 144 * 1024;
// The lean operand (x itself in LDS instead of operand tiles) needs groups that are contiguous for the
// weight stream and made of whole lane blocks, and one row tile.  int3 always takes it.  int4 takes it
// only where the tile layout would also hold all of K in one workgroup: there it saves the zero fill
// and the bank conflicts of the scatter (4096 x 11008 9.1 -> 8.3 us); with K split over workgroups
// it is a little slower than the tiles (4096 x 4096 8.4 -> 8.6 us), and a plan that no longer needs to
// split K for LDS loses the workgroups that filled the chip (9216 x 36864 33.9 -> 37.5 us).
inline bool grouped_lite(int bits, int K, int gs, bool has_g_idx, int tpm, int M, int kr, int waves_n, int waves_k,
                         int split_k)
{
    const int klane = bits == 4 ? 8 : 32;
    if (has_g_idx || tpm != 1 || gs % klane != 0 || K / klane >= 65536) return false;
    if (bits == 3) return true;
    return split_k == 1 && grouped_lds_bytes(kr, M, tpm, waves_n, waves_k, false) <= kGroupedLdsCap;
}
// Wave-private staging of x in the lean-operand GROUPED kernel: on a layer whose x needs no reordering,
// a wave whose K range is at most 512 channels loads and stages its own x, which takes the workgroup
// barriers out of the prologue (int3 4096 x 11008: 7.4 -> 6.8 us, int4: 9.4 -> 8.0 us).  Looking the
// channels of a sorted layer up per wave instead (two dependent round trips) loses to the shared
// scatter with its one barrier (7.9 against 7.6 us).
inline bool grouped_wavex(bool lite, int wave_channels) { return lite && wave_channels <= 512; }
// Packed rows in the GROUPED kernel (two to four activation rows for the matrix instructions of one, five
// to eight for those of two):
// the lean operand with wave-private staging, and at most four groups in a wave's K range, counted
// exactly (a wave's range starts at a multiple of its length).  Such plans are sized for four or eight rows and
// say so in row_tiles; a two-row plan of the unpacked kind with four row tiles meets more than 16 groups
// per wave and is therefore never packable, so the two cannot be mistaken for each other.
static const int kPackedRows = 8;  // the most rows a packed plan holds
// rows a packed plan for M activation rows is sized for (its row_tiles): one tile of four, or two
inline int packed_rows_of(int M) { return M <= 4 ? 4 : 8; }
inline int wave_groups_exact(int wave_channels, int gs)
{
    if (gs % wave_channels == 0) return 1;
    return wave_channels % gs == 0 ? wave_channels / gs : 0;  // 0: not a whole number
}
inline bool grouped_packable(int bits, int K, int gs, bool has_g_idx, int M, int kr, int waves_k)
{
    const int klane = bits == 4 ? 8 : 32;
    if (M < 2 || M > kPackedRows || has_g_idx || gs % klane != 0 || K / klane >= 65536) return false;
    if (M > 4 && waves_k < 2) return false;  // the last stage has a thread per 4 outputs of 64 columns: 128 for 8 rows
    const int groups = wave_groups_exact(kr / waves_k, gs);
    return grouped_wavex(true, kr / waves_k) && groups >= 1 && groups <= 4;
}
// STREAM kernel sizing.  A row of its (scale, zero) table: 64 columns x (fp16 scale, fp16 zero),
// padded by 16 bytes so that lane groups reading rows of different groups spread over the banks.
static const int kStreamTableRow = 64 * 4 + 16;
// blocks of 32 channels the A fragments and table offsets run ahead
static const int kStreamRingBlocks = 4;
// steps the weight loads run ahead; every wave walks a multiple of it
constexpr int stream_pf(int bits) { return bits == 4 ? 4 : 2; }
inline int stream_wave_steps(int bits, int steps_total, int split_k, int waves_k)
{
    const int pf = stream_pf(bits);
    const int per_wave = (steps_total + split_k * waves_k - 1) / (split_k * waves_k);
    return (per_wave + pf - 1) / pf * pf;
}
// tallest tile of a STREAM wave in 16-row tiles: 64 rows keep a wave under 256 registers, so two
// waves share a SIMD; taller problems take more M blocks
constexpr int stream_max_row_tiles() { return 4; }
// one lookup per weight unless groups are contiguous and no narrower than a lane block
inline int stream_act_table(int bits, int group_size, int act_order)
{
    return (act_order || group_size % (bits == 4 ? 8 : 32) != 0) ? 1 : 0;
}
// The pack pass can be skipped for one row tile (M <= 16): the kernel then reads x rows and g_idx
// itself.  Needs a g_idx whenever the lookup is per weight, and lane-block numbers below 2^16
// (exactness of its multiply-high division).
inline int stream_direct(int bits, int K, int row_tiles, int act_table, int has_g_idx)
{
    return row_tiles == 1 && (!act_table || has_g_idx) && K / (bits == 4 ? 8 : 32) < 65536;
}
int stream_lds_bytes(int bits, int K, int G, int group_size, int act_table, int row_tiles, int waves_k,
                     int wave_steps);
// bytes of the packed x and of the packed table offsets, each rounded up to 256
size_t stream_xpack_bytes(int bits, int steps_pad, int rt_total);
size_t stream_gpack_bytes(int bits, int steps_pad, int act_table);

int launch_stream(const Params &p, int bits, const gptq_hip_plan &plan, void *stream);
int launch_grouped(const Params &p, int bits, const gptq_hip_plan &plan, void *stream);
int launch_dequant(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *g_idx,
                   void *w, int K, int N, int G, int bits, int group_size, void *stream);
int launch_fill_zero(void *ptr, size_t bytes, void *stream);
int launch_sort_channels(const uint32_t *qweight, const int32_t *g_idx, uint32_t *qweight_sorted, int32_t *kmap, int K,
                         int N, int G, int bits, int group_size, void *stream);
int launch_permute_x(const void *x, const int32_t *src, void *xs, int M, int K, void *stream);
// Rows of x up to which the sorted entry point covers small batches (the STREAM kernel that reads x
// itself, behind a pass that puts x into the sorted channel order)
static const int kSortedMaxRows = 16;
// where that pass puts x in the workspace: behind what the plan itself uses, and never over the
// counters at the head, which every call must leave zero
inline size_t sorted_x_offset(size_t plan_bytes)
{
    const size_t head = plan_bytes > kCounterBytes ? plan_bytes : kCounterBytes;
    return (head + 255) / 256 * 256;
}


// ---- TILED family (a layer re-laid by gptq_hip_tile_prepare) ----------------------------------------
// A workgroup is four waves along K; a wave holds AT 32-row tiles (row_tiles of the plan).
inline int tiled_row_tiles(int M) { return M <= 32 ? 1 : (M <= 64 ? 2 : 4); }
// blocks (64 positions) the register rings of a wave run ahead: the taller the tile, the longer a block
// takes and the fewer of them cover the memory latency (and fit the registers)
constexpr int tiled_ring(int at) { return at >= 4 ? 3 : (at == 2 ? 4 : 6); }
// blocks of x the pack pass writes: what the waves of all K ranges walk
inline int tiled_pack_blocks(int split_k, int waves_k, int wave_steps) { return split_k * waves_k * wave_steps; }
// LDS of a workgroup: the result tiles (32 x 32 floats, two per 32 rows) of its waves
inline int tiled_lds_bytes(int row_tiles, int waves_k) { return waves_k * row_tiles * 2 * 4096; }
// the matmul kernel reads its x fragments from x itself, without the pack pass: up to 16 rows of layers without an
// activation order, when K is a whole number of blocks that the waves' ranges cover exactly (no zero padding is
// read)
constexpr int kTiledDirectRows = 16;
inline bool tiled_reads_x_directly(bool act_order, int M, int K, const gptq_hip_plan &plan)
{
    return !act_order && M <= kTiledDirectRows && plan.kernel == GPTQ_HIP_KERNEL_TILED && plan.row_tiles == 1 &&
           plan.m_blocks == 1 && plan.waves_n == 1 && K % 64 == 0 &&
           plan.split_k * plan.waves_k * plan.k_chunk == K / 64;
}
// the transposed product: the result tiles, or the table of (scale, base + zero) pairs of the workgroup's K range
// for its two column tiles (256 bytes per block and tile), whichever is larger: they share the memory
inline int tiled_t_lds_bytes(int row_tiles, int waves_k, int wave_steps)
{
    const int red = tiled_lds_bytes(row_tiles, waves_k), tbl = 2 * waves_k * wave_steps * 256;
    return red > tbl ? red : tbl;
}
constexpr int kTiledTMaxBlocks = 304;   // blocks of 64 columns a workgroup of the transposed product may walk (LDS)
inline bool tiled_qualifies(int K, int N, int bits, int gs)
{
    // (the pack pass stages one row of x in LDS: K * 2 bytes)
    return (bits == 2 || bits == 3 || bits == 4 || bits == 8) && K % 32 == 0 && N % 32 == 0 && gs % 32 == 0 &&
           K % gs == 0 && K <= 65536;
}
// decode kernel on the tiled format: rows it is built for, and the LDS of a workgroup whose waves cover
// `span` positions of `groups` groups
static const int kDecodeMaxRows = 8;      // rows the decode kernel of the tiled format takes (the 16-column kernel: 4)
constexpr int kDecodeSelectRows = 4;   // rows up to which gptq_hip_select_tiled chooses it
inline int tiled_decode_rows(int M) { return M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 8)); }
inline int tiled_decode_lds_bytes(int mr, int span, int groups, int waves_k)
{
    (void)groups;   // (the (scale, zero) words no longer pass through LDS)
    return mr * span * 2 + 64 + (span / 32) * mr * 8 + waves_k * mr * 128;
}
// decode kernel with one workgroup per CU (16-column units, all of K staged): LDS of a workgroup that takes
// `units_per_wg` units
constexpr int kNumCUs = 256;   // MI355X
inline long long tiled_decode16_lds_bytes(int mr, int K, int groups, int units_per_wg)
{
    const long long span = ((K + 63) / 64 + 1) / 2 * 128;
    (void)groups;   // (the (scale, zero) words no longer pass through LDS)
    return mr * span * 2 + 64 + (span / 32) * mr * 8 + (long long)units_per_wg * 16 * mr * 256;
}
int launch_tile_prepare(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *g_idx,
                        uint32_t *qtile, uint32_t *sz, int32_t *xsrc, uint16_t *kinv, int K, int N, int G, int bits,
                        int group_size, void *stream);
int launch_tiled_decode(const void *x, const void *qtile, const uint32_t *sz, const uint16_t *kinv, const void *bias,
                        void *y, float *partial, unsigned long long *slots, int M, int K, int N, int G, int bits,
                        int group_size, const gptq_hip_plan &plan, void *stream);
// the workgroup-per-tile decode kernel pairs the blocks of a wave up (one epilogue per two blocks) when groups
// are multiples of 128 channels and a wave walks an even number of blocks
constexpr bool tiled_decode_pairs(int group_size, int wave_steps) { return group_size % 128 == 0 && wave_steps % 2 == 0; }
// halved tiles: blocks per wave of the first half (the larger one; an even count where blocks pair up), the
// second half takes the rest
constexpr int tiled_decode_first_half(int wave_steps, bool pairs)
{
    return pairs ? 2 * ((wave_steps + 3) / 4) : (wave_steps + 1) / 2;
}
// tiles of the workgroup-per-tile decode kernel that are halved along K: the e tiles past a whole number per
// CU, when their 2 e halves find a CU each (e <= CUs / 2), so that the fullest CU holds half a tile more than
// the others instead of a whole one.  Both halves pair their blocks up where whole tiles do.  (With more
// halves than CUs nothing is gained, and workgroups of eight waves lose: 5120 x 13824, 176 tiles halved,
// 9.9 -> 11.4 us at one row, 12.8 -> 16.2 at four.)
inline bool tiled_decode_can_halve(int wave_steps, int split_k, int waves_k, int S_total, int group_size)
{
    if (split_k != 1) return false;
    const bool pairs = tiled_decode_pairs(group_size, wave_steps);
    const int first = tiled_decode_first_half(wave_steps, pairs);
    if (wave_steps - first < (pairs ? 2 : 1)) return false;    // nothing left for the second half
    return waves_k * first < S_total;                          // the second half must start inside K
}
// Layers of so few tiles that two workgroups per tile still find a CU each (N <= 4096), with K long enough for
// two ranges (4096 channels): EVERY tile is halved, which gives every CU work like the 16-column kernel does, at
// the lower cost per weight of this one (one / four / eight rows, us, against the 16-column kernel, which has no
// eight-row form: there the comparison is with whole tiles.  4096 x 4096 int4 4.11 / 5.20 / 6.42 against 4.43 / 5.86 /
// 7.29, int3 with an activation order 4.05 / 5.96 / 9.21 against 4.40 / 6.47 / 10.0; 4096 x 2048 3.59 / 4.81 / 6.32 against
// 4.13 / 5.58 / 7.10; 4096 x 1024 3.48 / 4.70 / 6.23 against 4.04 / 5.49 / 7.06; 6144 x 4096 4.79 / 6.04 / 7.87 against 5.45 /
// 7.21 / 8.52; 11008 x 4096 int3 8.4 / 11.2 against 9.6 / 13.6 at one / four rows.  At 2048 channels the halves are four
// blocks per wave: 2048 x 4096 3.93 / 5.17 / 6.31 against 3.98 / 5.33 / 5.72, 2048 x 2048 3.78 / 5.03 / 6.25 against
// 3.79 / 5.19 / 5.66: level up to four rows, a loss at eight, so shorter layers stay with the 16-column kernel).
inline bool tiled_decode_halves_all(int tiles, int S_total) { return 2 * tiles <= kNumCUs && S_total >= 64; }
inline int tiled_decode_halved(int tiles, int wave_steps, int split_k, int waves_k, int S_total, int group_size)
{
    if (!tiled_decode_can_halve(wave_steps, split_k, waves_k, S_total, group_size)) return 0;
    if (tiled_decode_halves_all(tiles, S_total)) return tiles;
    const int e = tiles % kNumCUs;
    if (tiles <= kNumCUs || e == 0 || 2 * e > kNumCUs) return 0;
    return e;
}
// positions a workgroup of the plan stages: a whole tile's range, or the larger half's when every tile is halved
inline int tiled_decode_span(int halved, int tiles, int wave_steps, int waves_k, int group_size)
{
    const int ws = halved == tiles ? tiled_decode_first_half(wave_steps, tiled_decode_pairs(group_size, wave_steps))
                                   : wave_steps;
    return ws * waves_k * 64;
}
// workspace of those tiles: one 64-bit slot per output of a halved tile, behind the counters
inline size_t tiled_decode_slot_bytes(int halved, int mr) { return (size_t)halved * mr * 32 * 8; }
int launch_tiled_decode16(const void *x, const void *qtile, const uint32_t *sz, const uint16_t *kinv, const void *bias,
                          void *y, int M, int K, int N, int G, int bits, int group_size, const gptq_hip_plan &plan,
                          void *stream);
int launch_tile_prepare_t(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *xsrc,
                          uint32_t *qtile_t, uint32_t *szt, int K, int N, int G, int bits, void *stream);
int launch_tiled_t(const void *gy, const void *qtile_t, const uint32_t *szt, const int32_t *xsrc, void *gx, char *xpack,
                   float *partial, int M, int K, int N, int bits, int group_size, const gptq_hip_plan &plan,
                   void *stream);
int launch_tiled(const void *x, const void *qtile, const uint32_t *sz, const int32_t *xsrc, const void *bias, void *y,
                 char *xpack, float *partial, int M, int K, int N, int G, int bits, int group_size,
                 const gptq_hip_plan &plan, void *stream);

}  // namespace gptq
