// Shape dispatcher: a pure host function from (M, K, N, bits, group_size, act_order)
// to a launch plan.  It stands where the reference keeps a JSON database of tuned
// kernels per shape and an M-bucket switch
// (auto_gptq/nn_modules/tvm_untils/cache.py:11-62,
//  auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:77-127,138-189).
#include <string.h>

#include "gptq_internal.h"

namespace {

const int kLdsBudget = 120 * 1024;  // of the 160 KB a gfx950 CU has
const int kTargetWorkgroups = 512;  // two per CU keeps every XCD fed at M = 1

int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace

extern "C" int gptq_hip_select(int M, int K, int N, int bits, int group_size, int act_order, gptq_hip_plan *plan)
{
    if (!plan) return GPTQ_HIP_ERR_BAD_ARG;
    memset(plan, 0, sizeof(*plan));
    if (bits != 3 && bits != 4) return GPTQ_HIP_ERR_BAD_ARG;
    if (M < 1 || K < 32 || N < 32) return GPTQ_HIP_ERR_BAD_ARG;
    if (K % 32 != 0 || N % 32 != 0) return GPTQ_HIP_ERR_BAD_ARG;  // the packed format needs both
    if (group_size == 0 || group_size < -1) return GPTQ_HIP_ERR_BAD_ARG;
    (void)act_order;
    const int gs = group_size == -1 ? K : group_size;
    const int G = ceil_div(K, gs);
    const int kstep = gptq::kstep_of(bits);
    const int steps_total = ceil_div(K, kstep);

    plan->kernel = GPTQ_HIP_KERNEL_GATHER;
    plan->row_tiles = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 64 ? 4 : 8));
    plan->m_blocks = ceil_div(M, 16 * plan->row_tiles);
    const int xs_rows = M < 16 * plan->row_tiles ? M : 16 * plan->row_tiles;
    int kc = xs_rows <= 16 ? 512 : (xs_rows <= 32 ? 256 : 128);
    if (kc > steps_total * kstep) kc = steps_total * kstep;
    plan->k_chunk = kc;
    const int chunk_steps = kc / kstep;

    int waves = 4;
    int lds = 0;
    for (; waves >= 1; waves >>= 1) {
        const int bn = 64 * waves;
        lds = G * bn * 4 + kc * 4 + xs_rows * (kc + 8) * 2;
        if (lds <= kLdsBudget) break;
    }
    if (waves < 1) return GPTQ_HIP_ERR_UNSUPPORTED;  // more groups than the LDS table holds
    plan->waves_n = waves;
    plan->waves_k = 1;
    plan->lds_bytes = lds;
    plan->block = 64 * waves;
    const int col_tiles = ceil_div(N, 64 * waves);

    int split = ceil_div(kTargetWorkgroups, col_tiles * plan->m_blocks);
    // partial sums cost split*M*N*4 bytes each way; keep them well under the packed weights
    int cap = (int)(((long long)K * bits) / (128LL * M));
    if (cap < 1) cap = 1;
    if (split > cap) split = cap;
    const int max_split = steps_total / (chunk_steps > 0 ? 1 : 1);
    if (split > max_split) split = max_split;
    if (split > 64) split = 64;
    if (split < 1) split = 1;
    if ((size_t)col_tiles * plan->m_blocks * sizeof(int) > gptq::kCounterBytes) split = 1;
    plan->split_k = split;
    plan->grid_x = col_tiles;
    plan->grid_y = split;
    plan->grid_z = plan->m_blocks;
    plan->workspace_bytes = split > 1 ? gptq::kCounterBytes + (size_t)split * M * N * sizeof(float) : 0;
    return GPTQ_HIP_OK;
}

extern "C" size_t gptq_hip_workspace_bytes(int M, int K, int N, int bits, int group_size, int act_order)
{
    gptq_hip_plan plan;
    if (gptq_hip_select(M, K, N, bits, group_size, act_order, &plan) != GPTQ_HIP_OK) return 0;
    return plan.workspace_bytes;
}
