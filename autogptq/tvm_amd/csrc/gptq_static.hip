// gptq_hip_gemm_static: gptq_hip_gemm for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The workspace the kernels
// need (split-K counters and partial tiles, activations re-laid for the matrix instructions) is a
// file-scope array in device memory, one copy per GPU, that lives as long as the process.
//
// In host code the array's name is only a handle: its device address is asked for once per device
// with hipGetSymbolAddress and kept; kernels and fills get that address, never the name.
#include <hip/hip_runtime.h>

#include <mutex>

#include "gptq_internal.h"

namespace {

constexpr size_t kStaticScratchBytes = (size_t)16 << 20;  // 16 MiB per GPU

__device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device i, nullptr until first use
std::mutex g_scratch_mutex;

// The address of this device's copy of the array: first use on a device asks the runtime for it.  Nothing is
// launched: an array of static storage duration starts out all zero, which is what the split-K counters at its head
// need before the first call, and every call leaves them zero.
int scratch_of_current_device(void **out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return GPTQ_HIP_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            return GPTQ_HIP_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return GPTQ_HIP_OK;
}

}  // namespace

extern "C" size_t gptq_hip_static_workspace_limit(void) { return kStaticScratchBytes; }

extern "C" int gptq_hip_static_init(void)
{
    void *ws = nullptr;
    return scratch_of_current_device(&ws);
}

extern "C" int gptq_hip_gemm_static(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                                    const int32_t *g_idx, const void *bias, void *y, int M, int K, int N, int bits,
                                    int group_size, void *stream)
{
    gptq_hip_plan plan;
    int rc = gptq_hip_select(M, K, N, bits, group_size, g_idx != nullptr, &plan);
    if (rc != GPTQ_HIP_OK) return rc;
    if (plan.workspace_bytes > kStaticScratchBytes) return GPTQ_HIP_ERR_WORKSPACE;  // beyond the array: use gptq_hip_gemm
    void *ws = nullptr;
    if (plan.workspace_bytes > 0) {
        rc = scratch_of_current_device(&ws);
        if (rc != GPTQ_HIP_OK) return rc;
    }
    return gptq_hip_gemm_plan(x, qweight, qzeros, scales, g_idx, bias, y, ws, ws ? kStaticScratchBytes : 0, M, K, N,
                              bits, group_size, &plan, stream);
}
