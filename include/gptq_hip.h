/*
 * C ABI of the MI355X (gfx950) GPTQ int3/int4 QuantLinear kernels.
 *
 * Every pointer except `plan` outputs is a DEVICE pointer owned by the caller.
 * Nothing here allocates, frees or synchronises; launches go to `stream`
 * (a hipStream_t passed as void*, NULL = the default stream).  Functions
 * return GPTQ_HIP_OK or a negative gptq_hip_status and never throw.
 *
 * Tensor formats are those of the reference's standard QuantLinear
 * (auto_gptq/nn_modules/qlinear.py:40-59):
 *   qweight int32 [K/32*bits, N]   codes packed along K, little-endian bit stream
 *   qzeros  int32 [G, N/32*bits]   (zero point - 1) packed along N the same way
 *   scales  fp16  [G, N]
 *   g_idx   int32 [K]              group of input channel k; NULL means k / group_size (16-byte aligned)
 *   bias    fp16  [N] or NULL
 *   x       fp16  [M, K] row-major, y fp16 [M, N] row-major
 * with G = ceil(K / group_size) and group_size = -1 meaning K.
 */
#ifndef GPTQ_HIP_H
#define GPTQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum gptq_hip_status {
    GPTQ_HIP_OK = 0,
    GPTQ_HIP_ERR_BAD_ARG = -1,     /* null pointer, non-positive size, a width the entry point does not take, misaligned */
    GPTQ_HIP_ERR_UNSUPPORTED = -2, /* shape outside what the kernels cover (see gptq_hip_select) */
    GPTQ_HIP_ERR_WORKSPACE = -3,   /* workspace missing or smaller than the plan needs */
    GPTQ_HIP_ERR_LAUNCH = -4       /* the HIP runtime refused the launch */
} gptq_hip_status;

/* kernel families the dispatcher chooses between */
enum {
    /* 1: a retired family; no plan names it */
    GPTQ_HIP_KERNEL_GROUPED = 2, /* rows expanded by group, scales applied once per group; M <= 2 with few groups,
                                    or M <= 8 with contiguous groups (activation rows packed into the
                                    operand tile: such plans have row_tiles = 4 or 8) */
    GPTQ_HIP_KERNEL_STREAM = 3, /* exact fp16 weights, independent waves along K; any g_idx, any M.  M > 16: x is
                                   pre-packed into matrix-instruction fragment order (needs the workspace);
                                   M <= 16: the kernel reads x itself.  split_k > 1 adds a reduce launch. */
    GPTQ_HIP_KERNEL_TILED = 4,  /* a layer re-laid by gptq_hip_tile_prepare: exact fp16 weights, 32 * row_tiles rows
                                   (row_tiles = 1, 2 or 4: the least that covers M up to 128 rows, one step less on
                                   narrow layers whose shorter row blocks still find a compute unit each) x 64 waves_n
                                   columns (waves_n = 1, or 2 with four row tiles: chosen for several row blocks) per
                                   workgroup of waves_k = 4 waves along K, m_blocks row blocks along grid_z
                                   (k_chunk = blocks of 64 channels per wave); x is pre-packed into the
                                   workspace; split_k > 1 adds a reduce launch */
    GPTQ_HIP_KERNEL_TILED_DECODE = 5 /* the same layer for M <= 8 rows, x staged in LDS in the layer's sorted order,
                                   scales applied per 32 or 64 channels; row_tiles = the rows the kernel is built
                                   for (1, 2, 4 or 8; 8 with waves_n = 1 and at most 8 waves only).  waves_n = 1: a workgroup per 32 columns, waves_k (4, 8 or 16)
                                   waves along K with k_chunk blocks of 64 channels each; split_k > 1 (an x that
                                   does not fit LDS) adds a reduce launch.  waves_n = 2: units of 16 columns dealt
                                   out evenly over grid_x workgroups of 16 waves, all of K staged per workgroup
                                   (k_chunk = blocks of 128 channels per unit and wave); chosen for layers of up to
                                   4096 columns and fewer than 4096 channels */
};

/* What the dispatcher decided for one problem; filled by gptq_hip_select. */
typedef struct gptq_hip_plan {
    int kernel;             /* GPTQ_HIP_KERNEL_* */
    int row_tiles;          /* 16-row MFMA tiles held per wave (GROUPED with packed activation rows, M = 2..8 on
                               contiguous groups: the rows the plan is sized for, 4 or 8) */
    int m_blocks;           /* grid extent along M */
    int waves_n;            /* waves of a workgroup laid along N (64 columns each) */
    int waves_k;            /* waves of a workgroup laid along K */
    int split_k;            /* workgroups sharing one column tile; >1 uses the workspace */
    int k_chunk;            /* input channels staged in LDS at a time (STREAM: per wave step) */
    int grid_x, grid_y, grid_z;
    int block;              /* threads per workgroup */
    int lds_bytes;          /* dynamic LDS per workgroup */
    int flags;              /* GPTQ_HIP_PLAN_* bits */
    size_t workspace_bytes; /* 0 when the plan needs none (e.g. GROUPED with split_k == 1) */
} gptq_hip_plan;

/* gptq_hip_plan.flags */
/* The plan's workspace must be ALL zero at the first call, is left all zero by every call, and must not be shared
 * with plans that lack this flag (they write theirs): give such plans a buffer of their own.  Set by the decode
 * plans of the tiled family whose tiles are halved along K (the halves meet in 64-bit slots of the workspace). */
#define GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE 1

/*
 * Shape dispatcher: a pure host function (no GPU needed).  Takes the place of
 * the reference's handler database and M-bucket dispatch
 * (auto_gptq/nn_modules/tvm_untils/cache.py:11-62,
 *  auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:77-127,138-189).
 * act_order != 0 means a g_idx array will be passed.
 */
int gptq_hip_select(int M, int K, int N, int bits, int group_size, int act_order, gptq_hip_plan *plan);

/*
 * The plan of one kernel family with split_k and waves_n forced (0 = let the dispatcher
 * choose; for GPTQ_HIP_KERNEL_STREAM waves_n is the number of waves along K: 1, 2, 4 or 8);
 * GPTQ_HIP_ERR_UNSUPPORTED when that family does not cover the problem.  For benchmarks and
 * tests of single kernels; the reference's counterpart is editing the tile parameters of one
 * handler-database entry (pycuda_warpper.py:77-127).
 */
int gptq_hip_plan_for(int kernel, int M, int K, int N, int bits, int group_size, int act_order, int split_k,
                      int waves_n, gptq_hip_plan *plan);

/* Bytes of workspace gptq_hip_gemm needs for this problem (0 if none): split-K counters and
 * partial tiles, and for M > 16 the pre-packed activations. */
size_t gptq_hip_workspace_bytes(int M, int K, int N, int bits, int group_size, int act_order);

/*
 * Zero-fills a workspace with a fill kernel.  A workspace must be zero before
 * its first use; gptq_hip_gemm leaves it ready for the next call on the same
 * stream.  Calls that share a workspace must not overlap.
 */
int gptq_hip_workspace_init(void *workspace, size_t workspace_bytes, void *stream);

/*
 * y = x @ dequant(qweight, qzeros, scales, g_idx) (+ bias), fp32 accumulate.
 * Replaces the reference's handler call
 *   handler(x, qweight, y, scales, zeros)   (pycuda_warpper.py:138, qlinear_tvm.py:123,150)
 * and computes what qlinear.py:198-245 computes.  Unlike the reference, y is
 * written for exactly M rows (no padded rows) and need not be pre-zeroed.  One to three kernel
 * launches on `stream` (pack pass for M > 16, matmul, reduce pass when the plan splits K).
 */
int gptq_hip_gemm(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                  const int32_t *g_idx, const void *bias, void *y, void *workspace, size_t workspace_bytes,
                  int M, int K, int N, int bits, int group_size, void *stream);

/* Same, with the plan forced by the caller (benchmarks and tests of single kernels). */
int gptq_hip_gemm_plan(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                       const int32_t *g_idx, const void *bias, void *y, void *workspace, size_t workspace_bytes,
                       int M, int K, int N, int bits, int group_size, const gptq_hip_plan *plan, void *stream);

/*
 * gptq_hip_gemm without a workspace argument and without any allocation.  No counterpart in the reference:
 * it is for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The workspace is an array of gptq_hip_static_workspace_limit() bytes
 * (16 MiB) inside the library, one copy per GPU, held until the process ends.  A problem whose plan needs more
 * returns GPTQ_HIP_ERR_WORKSPACE (use gptq_hip_gemm with a workspace of your own).  Every call on a GPU uses that
 * GPU's one array: calls that overlap on the same GPU (different streams or threads) race; calls on one
 * stream, or otherwise ordered, are fine.  The first use on a device looks the array's address up (no launch, no
 * fill: the array starts out zero and every call leaves its counters zero); the runtime may load the code object for
 * that, so make the first call, or gptq_hip_static_init() with the device current, before a stream capture begins.
 */
int gptq_hip_gemm_static(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                         const int32_t *g_idx, const void *bias, void *y, int M, int K, int N, int bits,
                         int group_size, void *stream);
size_t gptq_hip_static_workspace_limit(void);
/* Looks up the current device's array (nothing is launched); GPTQ_HIP_OK, or GPTQ_HIP_ERR_LAUNCH if the runtime
 * refuses.  Optional: gptq_hip_gemm_static does the same on its first call on a device. */
int gptq_hip_static_init(void);

/*
 * The decode product (one row, or a batch of up to 16) for a layer prepared when it was loaded: an activation-order g_idx makes
 * every weight look its group up (qlinear.py:200-242 gathers scales and zeros by g_idx), so the
 * loader sorts the input channels by group once; qweight_sorted holds the same codes with groups
 * contiguous along K and
 *   kmap int32 [2K] (16-byte aligned): kmap[k] & 0xffff = where channel k went, as a position in the
 *                                      order the kernels unpack codes; kmap[k] >> 16 = g_idx[k];
 *                                      kmap[K + j] = the channel whose codes are j-th along K in qweight_sorted
 * tells the kernel where each x[m, k] belongs.  x and y are in the layer's original channel order.
 * qzeros and scales are unchanged.  plan: NULL lets the dispatcher choose, else a plan for
 * (M, K, N, bits, group_size, act_order = 0) of the GROUPED family (M <= 2 without packed rows: one
 * launch, the scatter of x into LDS follows the map) or, for M <= 16, of the STREAM family with one row
 * tile or of the GROUPED family with packed rows (a small pass first writes x in the sorted order into
 * the tail of the workspace, then the kernel for contiguous groups runs: two or three launches).  workspace: gptq_hip_sorted_workspace_bytes, zeroed like any other.
 * Needs K < 65536, equal groups and group_size a multiple of 8 (int4) or 32 (int3);
 * GPTQ_HIP_ERR_UNSUPPORTED otherwise, or for larger batches (they run on the checkpoint's own
 * tensors through gptq_hip_gemm).
 */
int gptq_hip_gemm_sorted(const void *x, const int32_t *qweight_sorted, const int32_t *qzeros, const void *scales,
                         const int32_t *kmap, const void *bias, void *y, void *workspace, size_t workspace_bytes,
                         int M, int K, int N, int bits, int group_size, const gptq_hip_plan *plan, void *stream);

/*
 * The one-time preparation gptq_hip_gemm_sorted asks for, on the GPU: from a layer's qweight and g_idx
 * writes qweight_sorted int32 [K/32*bits, N] (a separate buffer) and kmap int32 [2K], both 16-byte
 * aligned.  The sort is stable (channels of a group keep their order).  g_idx must give every group
 * exactly group_size channels (what GPTQ's activation order produces); other contents give a map
 * that stays in bounds but does not describe the layer.  Same limits as gptq_hip_gemm_sorted
 * (GPTQ_HIP_ERR_UNSUPPORTED beyond them).  Two launches on `stream`; K*K/2 compares, so tens of
 * microseconds at K = 4096 and milliseconds at K = 65535.  The reference's counterpart is the weight
 * re-layout of its TVM module's constructor (qlinear_tvm.py:25-40).
 */
int gptq_hip_sort_channels(const int32_t *qweight, const int32_t *g_idx, int32_t *qweight_sorted, int32_t *kmap,
                           int K, int N, int bits, int group_size, void *stream);

/* Bytes of workspace gptq_hip_gemm_sorted needs with plan = NULL (0 if none): what the plan for contiguous
 * groups needs and, when that plan is a STREAM one, M*K*2 bytes for x in the sorted order behind it (at
 * max(plan bytes, 16 KiB) rounded up to 256: the counters at the head of a workspace stay untouched). */
size_t gptq_hip_sorted_workspace_bytes(int M, int K, int N, int bits, int group_size);

/*
 * The tiled format: a layer re-laid once, when it is loaded, into the order the matrix instructions consume,
 * for any number of rows of x (the reference's TVM module likewise keeps only its own re-laid copy of the
 * weights, auto_gptq/nn_modules/qlinear_tvm.py:25-40,105-107).  With Kp = K rounded up to 64:
 *   qtile  gptq_hip_tiled_bytes(K, N, bits) bytes, 16-byte aligned: blocks of 64 lanes x `bits` words, column tile
 *          (32 columns) outermost, then block of 64 sorted positions; lane (n = lane % 32, h = lane / 32) holds the 32
 *          codes of column 32 T + n at positions 64 S + 32 h .. + 31, permuted inside the lane into the order in
 *          which the kernels' register unpack hands them to the matrix instruction (word i of lane l at
 *          l * bits + i of the block; 8 bits: at (i / 4) * 256 + l * 4 + i % 4)
 *   sz     uint32 [G, N]: fp16 scale | fp16 (zero point) << 16
 *   xsrc   int32 [Kp], 16-byte aligned: the channel of x at sorted position p (stable sort of the channels by
 *          group; the identity without an activation order), -1 for p >= K
 *   kinv   uint16 [K], 16-byte aligned: its inverse, the position of channel k (K <= 65536)
 * gptq_hip_tile_prepare writes the three from the checkpoint tensors (g_idx may be NULL = contiguous groups); it
 * needs whole groups of equal size that are multiples of 32 channels (GPTQ_HIP_ERR_UNSUPPORTED otherwise) and
 * a g_idx that gives every group exactly group_size channels (other contents stay in bounds but do not describe
 * the layer).  Three launches; the sort costs K * K / 2 compares.
 * bits: 2, 3, 4 or 8, every width of the format (qlinear.py:31-32): the tiled entry points are the fused path
 * of 2- and 8-bit layers, which the entry points on the checkpoint layout above do not take.
 */
size_t gptq_hip_tiled_bytes(int K, int N, int bits);
int gptq_hip_tile_prepare(const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *g_idx,
                          void *qtile, uint32_t *sz, int32_t *xsrc, uint16_t *kinv, int K, int N, int bits,
                          int group_size, void *stream);

/* The plan of the TILED family for a problem (workspace_bytes included); takes the place of the reference's
 * tile table per M bucket (pycuda_warpper.py:77-127,150-189). */
int gptq_hip_select_tiled(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan);

/* The plan of the family's decode kernel (GPTQ_HIP_KERNEL_TILED_DECODE), M <= 8 rows (GPTQ_HIP_ERR_UNSUPPORTED
 * above); gptq_hip_select_tiled chooses it by itself up to 4 rows, and up to 8 for K <= 11008, the matmul kernel above.  No counterpart in the reference, whose
 * GEMV handler takes one row (pycuda_warpper.py:150-152).  Plans with halved tiles carry
 * GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE. */
int gptq_hip_select_tiled_decode(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan);

/*
 * y = x @ W (+ bias) on a layer in the tiled format, any M; replaces the same handler call as gptq_hip_gemm
 * (pycuda_warpper.py:138, qlinear_tvm.py:123,150).  x and y are in the layer's own channel order (xsrc = kinv =
 * NULL means no activation order; pass both or neither).  plan: NULL = gptq_hip_select_tiled.  workspace:
 * plan.workspace_bytes (none for most decode plans).  Decode plans: one launch; matmul plans: two
 * (pack pass, matmul); one more when the plan splits K.  A plan whose flags hold
 * GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE wants ALL bytes of its workspace zero at the first call and leaves them zero
 * (the two halves of a tile that is halved along K meet in 64-bit slots behind the counters): give such plans a
 * workspace of their own, which no other entry point writes between the calls.
 */
int gptq_hip_gemm_tiled(const void *x, const void *qtile, const uint32_t *sz, const int32_t *xsrc, const uint16_t *kinv,
                        const void *bias, void *y, void *workspace, size_t workspace_bytes, int M, int K, int N,
                        int bits, int group_size, const gptq_hip_plan *plan, void *stream);

/*
 * The transposed product gx[M, K] = gy[M, N] @ W^T: the gradient of y = x @ W with respect to x, for training on
 * top of frozen quantised layers (the reference's Triton back end: transpose_matmul_248_kernel and
 * transpose_matmul248, auto_gptq/nn_modules/qlinear_triton.py:195-273,298-317, used by its backward, :329-336).  It
 * runs the matmul kernel on a
 * second prepared copy, the tiled format of the transposed code matrix:
 *   qtile_t  gptq_hip_tiled_transposed_bytes(K, N, bits) bytes, 16-byte aligned: blocks of 64 lanes x `bits` words, tile
 *            of 32 sorted positions outermost, then block of 64 columns; lane (lane % 32, h = lane / 32) holds, for
 *            position 32 T + lane % 32, the codes of columns 64 S + 32 h .. + 31 (zeros past N)
 *   szt      gptq_hip_tiled_transposed_table_bytes(K, N, group_size) bytes, 16-byte aligned: per group and octet of
 *            columns, four (scale, scale) and four (base + zero) fp16 pairs in the order of the register unpack
 * gptq_hip_tile_prepare_transposed writes both (two launches).  xsrc: the map of gptq_hip_tile_prepare (the channel at
 * each sorted position), NULL without an activation order; gy and gx are in the layer's own channel order.  The
 * weights are formed exactly as in the forward product (fp16(scale * (q - zero)), one rounding), sums are fp32.
 * plan: NULL = gptq_hip_select_tiled_transposed.  workspace: plan.workspace_bytes, zeroed once.
 */
size_t gptq_hip_tiled_transposed_bytes(int K, int N, int bits);
size_t gptq_hip_tiled_transposed_table_bytes(int K, int N, int group_size);
int gptq_hip_tile_prepare_transposed(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                     const int32_t *xsrc, void *qtile_t, uint32_t *szt, int K, int N, int bits,
                                     int group_size, void *stream);
int gptq_hip_select_tiled_transposed(int M, int K, int N, int bits, int group_size, gptq_hip_plan *plan);
int gptq_hip_gemm_tiled_transposed(const void *gy, const void *qtile_t, const uint32_t *szt, const int32_t *xsrc,
                                   void *gx, void *workspace, size_t workspace_bytes, int M, int K, int N, int bits,
                                   int group_size, const gptq_hip_plan *plan, void *stream);

/*
 * Which copy of a layer a call with M rows runs on, and the plan there: the whole decision the reference's handler
 * makes in one place, from the row count to a kernel and its launch geometry (TVMHandler.__call__,
 * auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:138-189).  A pure host function.
 *   copies       the copies of the layer the caller holds or is willing to prepare (GPTQ_HIP_COPY_* bits):
 *                CHECKPOINT = qweight / qzeros / scales / g_idx as loaded (gptq_hip_gemm_plan), SORTED = the
 *                channel-sorted copy (gptq_hip_sort_channels, gptq_hip_gemm_sorted), TILED = the tiled format
 *                (gptq_hip_tile_prepare, gptq_hip_gemm_tiled).  TILED alone describes a layer that keeps only its
 *                tiled copy: every M then runs there.
 *   switch_rows  rows of x from which the caller prefers W from gptq_hip_dequant and its own fp16 GEMM (what the
 *                reference does from kernel_switch_threshold rows, auto_gptq/nn_modules/qlinear.py:25,198): three
 *                values, for calls on the tiled copy, on the checkpoint tensors, and on the checkpoint tensors of a
 *                layer with an activation order; 0 = never.  NULL = the measured defaults {1152, 1024, 640}.
 * route->copy names the entry point (GPTQ_HIP_ROUTE_LIBRARY: no fused kernel; dequant + library GEMM) and
 * route->plan is the plan to hand to it (zeroed for LIBRARY).  A SORTED or TILED answer for a copy that turns out not
 * to exist (gptq_hip_sort_channels / gptq_hip_tile_prepare refused the layer's contents) is retried with that bit
 * cleared.
 */
enum { GPTQ_HIP_COPY_CHECKPOINT = 1, GPTQ_HIP_COPY_SORTED = 2, GPTQ_HIP_COPY_TILED = 4 };
enum { GPTQ_HIP_ROUTE_CHECKPOINT = 0, GPTQ_HIP_ROUTE_SORTED = 1, GPTQ_HIP_ROUTE_TILED = 2, GPTQ_HIP_ROUTE_LIBRARY = 3 };
typedef struct gptq_hip_route {
    int copy;           /* GPTQ_HIP_ROUTE_* */
    int reserved;
    gptq_hip_plan plan;
} gptq_hip_route;
int gptq_hip_select_route(int M, int K, int N, int bits, int group_size, int act_order, unsigned copies,
                          const int *switch_rows, gptq_hip_route *route);

/*
 * W fp16 [K, N] = scales[g] * (q - (zq[g] + 1)), one rounding per element:
 * the materialised weight of qlinear.py:198-242, for the bit-exact check.  bits may also be 2 or 8
 * here (the other widths of the format, qlinear.py:31-32,211-215): without a tiled copy those layers run as
 * this kernel followed by a library GEMM.
 */
int gptq_hip_dequant(const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *g_idx,
                     void *w, int K, int N, int bits, int group_size, void *stream);

/*
 * Measurement aids, not on the product path and without a counterpart in the reference: small kernels that measure
 * what the GPU gives the product kernels (bench.py --machine times them), so that the floors the kernels are judged
 * against can be re-measured with committed code.  One launch on `stream`, nothing allocated.
 *   GPTQ_HIP_PROBE_EMPTY   `workgroups` x 256 threads that do nothing (the cost of a launch in a chain of launches)
 *   GPTQ_HIP_PROBE_STREAM  `workgroups` workgroups read `bytes` at `buf` once, 16 bytes per lane and request
 *   GPTQ_HIP_PROBE_MIXED   per workgroup, waves 0 and 1 read the `hot_bytes` (>= 64 KiB, small enough to stay in L2)
 *                          at `hot`, `iters` rounds of eight 1 KiB requests, while waves 2 and 3 are idle (mode 0),
 *                          do the same (mode 1) or stream `bytes` at `buf` from HBM with `depth` (1..8) requests in
 *                          flight (mode 2); ticks[4 * workgroup + wave] (device memory, uint64) = wall-clock ticks of
 *                          each reading wave (hipDeviceAttributeWallClockRate gives their rate)
 * `scratch`: 16 bytes of device memory that are never written (they keep the loads alive).
 */
enum { GPTQ_HIP_PROBE_EMPTY = 0, GPTQ_HIP_PROBE_STREAM = 1, GPTQ_HIP_PROBE_MIXED = 2 };
int gptq_hip_probe(int kind, const void *buf, size_t bytes, const void *hot, size_t hot_bytes, int workgroups, int iters,
                   int mode, int depth, unsigned long long *ticks, void *scratch, void *stream);

/* Human-readable text for a gptq_hip_status. */
const char *gptq_hip_strerror(int status);

/* ABI version of this library (bumped when a signature or gptq_hip_plan changes). */
#define GPTQ_HIP_ABI_VERSION 4
int gptq_hip_abi_version(void);

/* Digest of the sources this library was built from (set by the build script; "unknown" otherwise), so that a
 * loader can tell a library that is older than the sources beside it. */
const char *gptq_hip_build_id(void);

#ifdef __cplusplus
}
#endif
#endif /* GPTQ_HIP_H */
