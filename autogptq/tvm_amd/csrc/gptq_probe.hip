// Measurement aids: three small kernels that measure what the GPU gives the product kernels, so that the floors the
// kernels are judged against (and sized by) can be re-measured on any box with committed code (bench.py --machine):
//   EMPTY   a kernel that does nothing: the cost of one launch in a chain of dependent launches;
//   STREAM  every workgroup reads its share of a buffer once with 16-byte loads: what a plain read of the same
//           bytes, by the same number of workgroups, costs, launch included (the floor of a decode product);
//   MIXED   in every workgroup two waves read a small buffer that stays in L2 over and over while the other two
//           are idle, do the same, or stream a large buffer from HBM; the two reading waves report how long they
//           took.  A CU's vector-memory pipeline returns data in order across its waves, so loads that hit L2 slow
//           down as soon as the same CU also has misses to HBM in flight: that, not the number of bytes, is what
//           the activation fragments of a matmul kernel pay next to its weight stream.
// None of this is on the product path; gptq_hip_probe has no counterpart in the reference.
#include <hip/hip_runtime.h>

#include "gptq_internal.h"
#include "gptq_unpack.h"

namespace gptq {

__global__ __launch_bounds__(256) void probe_empty_kernel() {}

// `vecs` 16-byte vectors at `buf`, dealt to the workgroups in contiguous shares, every thread's loads independent
// of each other; the values are combined and stored only if all of them are all-ones (they are not: the store
// exists so that the loads do)
__global__ __launch_bounds__(256) void probe_stream_kernel(const u4 *__restrict__ buf, uint32_t vecs, uint32_t *sink)
{
    const uint32_t per_wg = (vecs + gridDim.x - 1) / gridDim.x;
    const uint32_t begin = blockIdx.x * per_wg, end = min(begin + per_wg, vecs);
    u4 acc = {~0u, ~0u, ~0u, ~0u};
    for (uint32_t v = begin + threadIdx.x; v < end; v += 256u) acc &= __builtin_nontemporal_load(buf + v);
    if ((acc[0] & acc[1] & acc[2] & acc[3]) == ~0u && vecs == ~0u) sink[0] = acc[0];
}

// mode 0: waves 2, 3 idle; 1: they read the hot buffer too; 2: they stream `cold` (each wave its own region, `depth`
// 1 KB requests issued per round, a round waited for while the next is in flight).  Waves 0, 1: `iters` rounds of
// eight 1 KB requests into the hot buffer, again one round in flight behind the one waited for.  All requests are
// direct loads into LDS (no registers, no use of the data), so that only the memory pipeline is measured.
// ticks[workgroup * 4 + wave] = wall-clock ticks the wave took.
extern __shared__ __align__(16) unsigned char probe_lds[];

__device__ __forceinline__ void probe_load_1kb(const char *p, unsigned char *lds, bool stream)
{
    if (stream)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                         (__attribute__((address_space(3))) void *)lds, 16, 0, 2);
    else
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                         (__attribute__((address_space(3))) void *)lds, 16, 0, 0);
}

__global__ __launch_bounds__(256) void probe_mixed_kernel(const char *__restrict__ hot, uint32_t hot_kb,
                                                          const char *__restrict__ cold, size_t cold_bytes, int iters,
                                                          int mode, int depth, unsigned long long *ticks)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (wave >= 2 && mode == 0) return;
    const bool reads_hot = wave < 2 || mode == 1;
    unsigned char *lds = probe_lds + wave * 8192;
    const unsigned long long t0 = wall_clock64();
    if (reads_hot) {
        const uint32_t first = (uint32_t)((blockIdx.x * 4 + wave) * 37u) % hot_kb;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const uint32_t kb = (first + 20u * (uint32_t)(it * 8 + u)) % hot_kb;
                probe_load_1kb(hot + (size_t)kb * 1024 + lane * 16, lds + u * 1024, false);
            }
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        }
    } else {
        const size_t region = cold_bytes / ((size_t)gridDim.x * 2) / 1024 * 1024;
        const char *base = cold + region * ((size_t)blockIdx.x * 2 + (wave - 2)) + lane * 16;
        const size_t kbs = region / 1024;
        // the same number of bytes as a wave on the hot buffer reads, so that the stream outlasts the hot waves
        const int rounds = iters * 8 / depth;
        for (int it = 0; it < rounds; it++) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (u < depth) probe_load_1kb(base + (((size_t)it * depth + u) % kbs) * 1024, lds + u * 1024, true);
            }
            if (depth >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else if (depth >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else if (depth >= 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned long long t1 = wall_clock64();
    if (lane == 0) ticks[blockIdx.x * 4 + wave] = t1 - t0;
}

}  // namespace gptq

extern "C" int gptq_hip_probe(int kind, const void *buf, size_t bytes, const void *hot, size_t hot_bytes, int workgroups,
                              int iters, int mode, int depth, unsigned long long *ticks, void *scratch, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    if (workgroups < 1 || workgroups > 65536) return GPTQ_HIP_ERR_BAD_ARG;
    if (kind == GPTQ_HIP_PROBE_EMPTY) {
        hipLaunchKernelGGL(gptq::probe_empty_kernel, dim3(workgroups), dim3(256), 0, stream);
    } else if (kind == GPTQ_HIP_PROBE_STREAM) {
        if (!buf || !scratch || bytes < 16 || bytes / 16 >= 0xffffffffull || ((uintptr_t)buf % 16)) return GPTQ_HIP_ERR_BAD_ARG;
        hipLaunchKernelGGL(gptq::probe_stream_kernel, dim3(workgroups), dim3(256), 0, stream, (const gptq::u4 *)buf,
                           (uint32_t)(bytes / 16), (uint32_t *)scratch);
    } else if (kind == GPTQ_HIP_PROBE_MIXED) {
        if (!hot || !ticks || hot_bytes < 65536 || ((uintptr_t)hot % 16) || iters < 1 || mode < 0 || mode > 2 ||
            depth < 1 || depth > 8)
            return GPTQ_HIP_ERR_BAD_ARG;
        if (mode == 2 && (!buf || ((uintptr_t)buf % 16) || bytes / ((size_t)workgroups * 2) < 65536)) return GPTQ_HIP_ERR_BAD_ARG;
        // 64 KiB of LDS per workgroup: at most two workgroups share a CU, and 256 of them get a CU each
        hipLaunchKernelGGL(gptq::probe_mixed_kernel, dim3(workgroups), dim3(256), 65536, stream, (const char *)hot,
                           (uint32_t)(hot_bytes / 1024), (const char *)buf, bytes, iters, mode, depth, ticks);
    } else {
        return GPTQ_HIP_ERR_BAD_ARG;
    }
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}
