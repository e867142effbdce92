// Dequantisation (bit-exact fp16 weight) and workspace fill kernels.
#include "gptq_device.h"

namespace gptq {

// ---------------------------------------------------------------------------------
// DEQUANT kernel: the materialised fp16 weight, bit for bit what the reference
// computes (qlinear.py:198-242).  One thread per (32 input channels, column).
// ---------------------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(256) void dequant_kernel(const uint32_t *__restrict__ qweight,
                                                      const uint32_t *__restrict__ qzeros,
                                                      const _Float16 *__restrict__ scales,
                                                      const int32_t *__restrict__ g_idx, _Float16 *__restrict__ W,
                                                      int K, int N, int G, int group_size)
{
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int kb = blockIdx.y;  // block of 32 input channels
    if (n >= N) return;
    const int zwords = N / 32 * BITS;
    uint32_t w[BITS];
#pragma unroll
    for (int i = 0; i < BITS; i++) w[i] = qweight[(size_t)(kb * BITS + i) * N + n];
    int g_prev = -1;
    _Float16 s = (_Float16)0.0f;
    int z = 0;
    for (int j = 0; j < 32; j++) {
        const int k = kb * 32 + j;
        int g = g_idx ? g_idx[k] : k / group_size;
        g = min(max(g, 0), G - 1);
        if (g != g_prev) {
            s = scales[(size_t)g * N + n];
            z = zero_of<BITS>(qzeros + (size_t)g * zwords, n);
            g_prev = g;
        }
        int q;
        if constexpr (BITS == 3) {
            q = code3(w[0], w[1], w[2], j);
        } else {
            q = code_pow2<BITS>(w, j);
        }
        W[(size_t)k * N + n] = dequant_one(s, q, z);
    }
}

__global__ void fill_zero_kernel(uint32_t *ptr, size_t words)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < words) ptr[i] = 0u;
}

int launch_dequant(const uint32_t *qweight, const uint32_t *qzeros, const void *scales, const int32_t *g_idx,
                   void *w, int K, int N, int G, int bits, int group_size, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 grid((N + 255) / 256, K / 32);
#define GPTQ_LAUNCH_DEQUANT(B)                                                                           \
    hipLaunchKernelGGL(dequant_kernel<B>, grid, dim3(256), 0, stream, qweight, qzeros, (const _Float16 *)scales, \
                       g_idx, (_Float16 *)w, K, N, G, group_size)
    switch (bits) {
        case 2: GPTQ_LAUNCH_DEQUANT(2); break;
        case 3: GPTQ_LAUNCH_DEQUANT(3); break;
        case 4: GPTQ_LAUNCH_DEQUANT(4); break;
        case 8: GPTQ_LAUNCH_DEQUANT(8); break;
        default: return GPTQ_HIP_ERR_BAD_ARG;
    }
#undef GPTQ_LAUNCH_DEQUANT
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------------
// Load-time channel sort of an activation-order layer (see gptq_hip_sort_channels).
// Pass 1: channel k goes to sorted index g * group_size + (number of earlier channels of its
// group): a stable sort by group without a sort.  Every thread counts over the g_idx entries
// before its own, a tile at a time through LDS (K * K / 2 compares: a one-time cost of tens of
// microseconds at K = 4096).  It writes both halves of the channel map.
// ---------------------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(256) void sort_map_kernel(const int32_t *__restrict__ g_idx, int32_t *__restrict__ kmap,
                                                       int K, int G, int group_size)
{
    __shared__ int tile[256];
    constexpr int KLANE = Fmt<BITS>::KLANE;
    const int k = blockIdx.x * 256 + threadIdx.x;
    const int g = k < K ? min(max(g_idx[k], 0), G - 1) : -1;
    int rank = 0;
    for (int t0 = 0; t0 <= (int)blockIdx.x * 256; t0 += 256) {
        const int j = t0 + threadIdx.x;
        __syncthreads();
        tile[threadIdx.x] = j < K ? min(max(g_idx[j], 0), G - 1) : -2;
        __syncthreads();
        const int upto = min(256, k - t0);  // entries of this tile that lie before k
        for (int i = 0; i < upto; i++) rank += tile[i] == g ? 1 : 0;
    }
    if (k >= K) return;
    // a group with more than group_size members would leave its range: keep every index in bounds
    const int inv = g * group_size + min(rank, group_size - 1);
    const int code = inv % KLANE;
    const int slot = BITS == 4 ? (int)kInv.inv4[code] : (int)kInv.inv3[code];
    kmap[k] = ((inv - code) + slot) | (g << 16);
    kmap[K + inv] = k;
}

// Pass 2: qweight_sorted row j = qweight row kmap[K + j], 32 rows (one packed block) and one column per thread.
template <int BITS>
__global__ __launch_bounds__(256) void sort_repack_kernel(const uint32_t *__restrict__ qweight,
                                                          const int32_t *__restrict__ kmap,
                                                          uint32_t *__restrict__ out, int K, int N)
{
    const int n = blockIdx.x * 256 + threadIdx.x;
    const int jb = blockIdx.y;
    if (n >= N) return;
    uint32_t words[BITS];
#pragma unroll
    for (int i = 0; i < BITS; i++) words[i] = 0u;
    for (int i = 0; i < 32; i++) {
        const int src = min(max(kmap[K + 32 * jb + i], 0), K - 1);
        const uint32_t *blk = qweight + (size_t)(src >> 5) * BITS * N + n;  // the packed block of 32 channels
        uint32_t q;
        const int bit = BITS * (src & 31);
        const int wd = bit >> 5, sh = bit & 31;
        q = blk[(size_t)wd * N] >> sh;
        if (sh + BITS > 32) q |= blk[(size_t)(wd + 1) * N] << (32 - sh);
        q &= (1u << BITS) - 1u;
        const int obit = BITS * i;
        const int owd = obit >> 5, osh = obit & 31;
        words[owd] |= q << osh;
        if (osh + BITS > 32) words[owd + 1] |= q >> (32 - osh);
    }
#pragma unroll
    for (int i = 0; i < BITS; i++) out[(size_t)(jb * BITS + i) * N + n] = words[i];
}

int launch_sort_channels(const uint32_t *qweight, const int32_t *g_idx, uint32_t *qweight_sorted, int32_t *kmap, int K,
                         int N, int G, int bits, int group_size, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 g1((K + 255) / 256), g2((N + 255) / 256, K / 32);
    if (bits == 4) {
        hipLaunchKernelGGL(sort_map_kernel<4>, g1, dim3(256), 0, stream, g_idx, kmap, K, G, group_size);
        hipLaunchKernelGGL(sort_repack_kernel<4>, g2, dim3(256), 0, stream, qweight, kmap, qweight_sorted, K, N);
    } else {
        hipLaunchKernelGGL(sort_map_kernel<3>, g1, dim3(256), 0, stream, g_idx, kmap, K, G, group_size);
        hipLaunchKernelGGL(sort_repack_kernel<3>, g2, dim3(256), 0, stream, qweight, kmap, qweight_sorted, K, N);
    }
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

// xs[m][j] = x[m][src[j]]: the activations of a layer whose channels were sorted by group, in the
// sorted order.  Eight outputs per thread: two index vectors, eight 2-byte gathers (x is small and
// stays in L2), one 16-byte store.  K is a multiple of 32.
__global__ __launch_bounds__(256) void permute_x_kernel(const _Float16 *x, const int32_t *src, _Float16 *xs, int M,
                                                        int K)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const uint32_t per_row = (uint32_t)K / 8u;
    if (t >= (uint32_t)M * per_row) return;
    const uint32_t m = t / per_row;
    const uint32_t j = 8u * (t - m * per_row);
    const int4 a = *(const int4 *)(src + j);
    const int4 b = *(const int4 *)(src + j + 4);
    const int idx[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const _Float16 *row = x + (size_t)m * K;
    h8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = row[min((uint32_t)idx[e], (uint32_t)K - 1u)];  // a bad map must not fault
    *(h8 *)(xs + (size_t)m * K + j) = o;
}

int launch_permute_x(const void *x, const int32_t *src, void *xs, int M, int K, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const unsigned threads = (unsigned)M * (unsigned)(K / 8);
    hipLaunchKernelGGL(permute_x_kernel, dim3((threads + 255u) / 256u), dim3(256), 0, stream, (const _Float16 *)x, src,
                       (_Float16 *)xs, M, K);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

int launch_fill_zero(void *ptr, size_t bytes, void *stream_v)
{
    hipStream_t stream = (hipStream_t)stream_v;
    const size_t words = bytes / 4;
    if (words == 0) return GPTQ_HIP_OK;
    const unsigned blocks = (unsigned)((words + 255) / 256);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, stream, (uint32_t *)ptr, words);
    return hipGetLastError() == hipSuccess ? GPTQ_HIP_OK : GPTQ_HIP_ERR_LAUNCH;
}

}  // namespace gptq
