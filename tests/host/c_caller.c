/* A plain C program that uses the library the way a C caller would: device memory from the HIP runtime, the
 * entry points of include/gptq_hip.h, nothing else.  Reads a layer and x from a file written by the test,
 * computes y three ways (gptq_hip_gemm on the checkpoint tensors; gptq_hip_sort_channels + gptq_hip_gemm_sorted;
 * gptq_hip_tile_prepare + gptq_hip_gemm_tiled) and writes the three results back.
 *
 * file: int32 header {M, K, N, bits, group_size, act_order}, then qweight, qzeros, scales, g_idx, x, bias
 * in that order, as raw little-endian arrays. */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "gptq_hip.h"

#define CHECK_HIP(call)                                                                   \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) {                                                           \
            fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));             \
            return 2;                                                                     \
        }                                                                                 \
    } while (0)
#define CHECK_GPTQ(call)                                                                  \
    do {                                                                                  \
        int rc_ = (call);                                                                 \
        if (rc_ != GPTQ_HIP_OK) {                                                         \
            fprintf(stderr, "%s failed: %s\n", #call, gptq_hip_strerror(rc_));            \
            return 3;                                                                     \
        }                                                                                 \
    } while (0)

static void *upload(FILE *f, size_t bytes)
{
    void *host = malloc(bytes), *dev = NULL;
    if (!host || fread(host, 1, bytes, f) != bytes) return NULL;
    if (hipMalloc(&dev, bytes) != hipSuccess) return NULL;
    if (hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice) != hipSuccess) return NULL;
    free(host);
    return dev;
}

static int workspace_for(size_t bytes, void **ws, hipStream_t stream)
{
    *ws = NULL;
    if (!bytes) return 0;
    if (hipMalloc(ws, bytes) != hipSuccess) return 2;
    return gptq_hip_workspace_init(*ws, bytes, stream);
}

int main(int argc, char **argv)
{
    if (argc != 3) {
        fprintf(stderr, "usage: %s input.bin output.bin\n", argv[0]);
        return 1;
    }
    if (gptq_hip_abi_version() != GPTQ_HIP_ABI_VERSION) {
        fprintf(stderr, "library ABI %d, header %d\n", gptq_hip_abi_version(), GPTQ_HIP_ABI_VERSION);
        return 1;
    }
    FILE *f = fopen(argv[1], "rb");
    int32_t h[6];
    if (!f || fread(h, sizeof(int32_t), 6, f) != 6) return 1;
    const int M = h[0], K = h[1], N = h[2], bits = h[3], group_size = h[4], act_order = h[5];
    const int gs = group_size == -1 ? K : group_size, G = (K + gs - 1) / gs;
    int32_t *qweight = upload(f, (size_t)K / 32 * bits * N * 4);
    int32_t *qzeros = upload(f, (size_t)G * (N / 32 * bits) * 4);
    void *scales = upload(f, (size_t)G * N * 2);
    int32_t *g_idx = upload(f, (size_t)K * 4);
    void *x = upload(f, (size_t)M * K * 2);
    void *bias = upload(f, (size_t)N * 2);
    fclose(f);
    if (!qweight || !qzeros || !scales || !g_idx || !x || !bias) return 1;
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    const size_t ybytes = (size_t)M * N * 2;
    void *y[3];
    for (int i = 0; i < 3; i++) {
        CHECK_HIP(hipMalloc(&y[i], ybytes));
        CHECK_HIP(hipMemset(y[i], 0xff, ybytes));
    }
    const int32_t *g = act_order ? g_idx : NULL;

    /* 1. the checkpoint's own tensors */
    gptq_hip_plan plan;
    CHECK_GPTQ(gptq_hip_select(M, K, N, bits, group_size, act_order, &plan));
    void *ws = NULL;
    CHECK_GPTQ(workspace_for(plan.workspace_bytes, &ws, stream));
    CHECK_GPTQ(gptq_hip_gemm(x, qweight, qzeros, scales, g, bias, y[0], ws, plan.workspace_bytes, M, K, N, bits,
                             group_size, stream));

    /* 2. the channel-sorted copy (decode sizes of activation-order layers); otherwise the same call again */
    int sorted_done = 0;
    if (act_order && M <= 16) {
        int32_t *qsorted = NULL, *kmap = NULL;
        CHECK_HIP(hipMalloc((void **)&qsorted, (size_t)K / 32 * bits * N * 4));
        CHECK_HIP(hipMalloc((void **)&kmap, (size_t)2 * K * 4));
        int rc = gptq_hip_sort_channels(qweight, g_idx, qsorted, kmap, K, N, bits, group_size, stream);
        if (rc == GPTQ_HIP_OK) {
            const size_t wsb = gptq_hip_sorted_workspace_bytes(M, K, N, bits, group_size);
            void *ws2 = NULL;
            CHECK_GPTQ(workspace_for(wsb, &ws2, stream));
            rc = gptq_hip_gemm_sorted(x, qsorted, qzeros, scales, kmap, bias, y[1], ws2, wsb, M, K, N, bits, group_size,
                                      NULL, stream);
            if (rc == GPTQ_HIP_OK) sorted_done = 1;
            else if (rc != GPTQ_HIP_ERR_UNSUPPORTED) CHECK_GPTQ(rc);
        } else if (rc != GPTQ_HIP_ERR_UNSUPPORTED) {
            CHECK_GPTQ(rc);
        }
    }
    if (!sorted_done)
        CHECK_GPTQ(gptq_hip_gemm(x, qweight, qzeros, scales, g, bias, y[1], ws, plan.workspace_bytes, M, K, N, bits,
                                 group_size, stream));

    /* 3. the tiled copy */
    const int Kp = (K + 63) / 64 * 64;
    void *qtile = NULL;
    uint32_t *sz = NULL;
    int32_t *xsrc = NULL;
    uint16_t *kinv = NULL;
    CHECK_HIP(hipMalloc(&qtile, gptq_hip_tiled_bytes(K, N, bits)));
    CHECK_HIP(hipMalloc((void **)&sz, (size_t)G * N * 4));
    CHECK_HIP(hipMalloc((void **)&xsrc, (size_t)Kp * 4));
    CHECK_HIP(hipMalloc((void **)&kinv, (size_t)K * 2));
    CHECK_GPTQ(gptq_hip_tile_prepare(qweight, qzeros, scales, g, qtile, sz, xsrc, kinv, K, N, bits, group_size, stream));
    gptq_hip_plan tplan;
    CHECK_GPTQ(gptq_hip_select_tiled(M, K, N, bits, group_size, &tplan));
    void *ws3 = NULL;
    CHECK_GPTQ(workspace_for(tplan.workspace_bytes, &ws3, stream));
    CHECK_GPTQ(gptq_hip_gemm_tiled(x, qtile, sz, g ? xsrc : NULL, g ? kinv : NULL, bias, y[2], ws3, tplan.workspace_bytes, M,
                                   K, N, bits, group_size, &tplan, stream));
    CHECK_HIP(hipStreamSynchronize(stream));

    FILE *o = fopen(argv[2], "wb");
    if (!o) return 1;
    void *host = malloc(ybytes);
    for (int i = 0; i < 3; i++) {
        CHECK_HIP(hipMemcpy(host, y[i], ybytes, hipMemcpyDeviceToHost));
        if (fwrite(host, 1, ybytes, o) != ybytes) return 1;
    }
    fclose(o);
    printf("ok kernels %d %d sorted %d\n", plan.kernel, tplan.kernel, sorted_done);
    return 0;
}
