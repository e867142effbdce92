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
};

// k handled by one wave step: 4 lane groups x (8 | 32) codes
inline int kstep_of(int bits) { return bits == 4 ? 32 : 128; }

// byte size of the head of the workspace that holds the split-K counters
static const size_t kCounterBytes = 16384;

// GROUPED kernel sizing, shared by the dispatcher and the plan check
int grouped_tpm(int groups, int M);
int grouped_groups(int kr, int gs, int G, int act_order);
int grouped_lds_bytes(int kr, int M, int tpm, int waves_n, int waves_k);
// Input channels of x the GATHER kernel stages per K wave at a time: fixed per (bits, row tiles) so
// that the kernel's unrolled step loop knows its chunk boundaries at compile time.  The chunk is a
// whole number of steps that divides the weight prefetch depth (8 steps int4, 4 steps int3).
constexpr int gather_kc(int bits, int row_tiles)
{
    return bits == 4 ? (row_tiles >= 8 ? 64 : (row_tiles == 4 ? 128 : 256))
                     : (row_tiles >= 4 ? 128 : (row_tiles == 2 ? 256 : 512));
}
// 16-byte vectors of x one thread of the GATHER kernel can stage per chunk
constexpr int gather_xv(int bits, int row_tiles) { return (bits == 3 && row_tiles != 2) ? 16 : 8; }
// group indices one thread can stage per chunk
constexpr int gather_gv() { return 8; }
int gather_lds_bytes(int G, int kc, int xs_rows, int row_tiles, int waves_n, int waves_k);

int launch_gather(const Params &p, int bits, const gptq_hip_plan &plan, void *stream);
int launch_grouped(const Params &p, int bits, const gptq_hip_plan &plan, void *stream);
int launch_dequant(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *g_idx,
                   void *w, int K, int N, int G, int bits, int group_size, void *stream);
int launch_fill_zero(void *ptr, size_t bytes, void *stream);

}  // namespace gptq
