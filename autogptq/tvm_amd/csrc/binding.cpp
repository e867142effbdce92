// torch.ops.gptq_hip.*: the C ABI of libgptq_hip.so as dispatcher-visible operators, in C++, so that an eager
// call costs one dispatch and one launch instead of a Python front end around ctypes.  Takes the place of the
// reference's per-call launch glue (auto_gptq/nn_modules/tvm_untils/pycuda_warpper.py:29-59: fetch the raw
// pointers, pick the compiled function for M, launch on the current stream).
//
// The operators take what the module holds (checkpoint tensors, the sorted copy, or the tiled copy), check
// devices, dtypes and shapes, allocate y through torch's caching allocator, and launch on the current HIP
// stream of x's device (torch on ROCm presents its HIP devices and streams under the "cuda" device type; the guard
// and stream classes used here are the ones that go with that).  The workspace the kernels need (split-K counters and partial tiles, re-laid x) is one
// zero-initialised tensor per (device, stream), grown on demand; the kernels leave its counters at zero.
// Only the CUDA (= HIP on ROCm) dispatch key gets kernels; the CPU key gets functions that say so and raise.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <atomic>
#include <map>
#include <mutex>
#include <optional>
#include <tuple>

#include "gptq_hip.h"

#ifndef GPTQ_HIP_BUILD_ID
#define GPTQ_HIP_BUILD_ID "unknown"
#endif

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

void need(const Tensor &t, const char *name, at::ScalarType dtype, const Tensor &like)
{
    TORCH_CHECK(t.is_cuda(), name, " is on ", t.device(), ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
    TORCH_CHECK(t.device() == like.device(), name, " is on ", t.device(), ", x on ", like.device());
    TORCH_CHECK(t.scalar_type() == dtype, name, " must be ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

const void *ptr(const OptTensor &t) { return t.has_value() && t->defined() ? t->data_ptr() : nullptr; }
bool has(const OptTensor &t) { return t.has_value() && t->defined(); }

void raise(int rc, const char *what, int64_t M, int64_t K, int64_t N, int64_t bits, int64_t gs)
{
    TORCH_CHECK(rc == GPTQ_HIP_OK, what, "(M=", M, ", K=", K, ", N=", N, ", bits=", bits, ", group_size=", gs,
                ") failed: ", gptq_hip_strerror(rc), " [status ", rc, "]");
}

// One workspace per (device, stream) and kind; a replaced one stays alive until the process ends only if a caller
// still holds it (the allocator keeps it valid for work already queued on its stream).
// kind 1: the decode plans of the tiled family with halved tiles, whose kernel keeps their bytes zero between launches
// (the slots of the halves): nothing else may write there, so they do not share the workspace the other plans pack x
// or partial sums into.
std::mutex g_ws_mutex;
std::map<std::tuple<int, void *, int>, Tensor> g_ws;

int workspace_kind(const gptq_hip_plan &plan)
{
    // (a decode plan that cuts K over workgroups leaves partial sums in its workspace like any other plan)
    return (plan.flags & GPTQ_HIP_PLAN_PRIVATE_ZERO_WORKSPACE) ? 1 : 0;
}

Tensor workspace(const Tensor &like, size_t nbytes, void *stream, int kind = 0)
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Tensor &ws = g_ws[{(int)like.get_device(), stream, kind}];
    if (!ws.defined() || (size_t)ws.numel() < nbytes) {
        const int64_t n = (int64_t)std::max(nbytes, (size_t)1 << 20);
        ws = at::zeros({n}, like.options().dtype(at::kByte));
    }
    return ws;
}

struct Shape {
    int64_t M, K, N, G;
};

// the checks of the Python front end (ops.check_shapes) on the checkpoint layout
Shape check_layer(const Tensor &x, const Tensor &qweight, const Tensor &qzeros, const Tensor &scales, int64_t g_len,
                  const OptTensor &bias, int64_t bits, int64_t group_size, bool fused_only)
{
    TORCH_CHECK(bits == 3 || bits == 4 || (!fused_only && (bits == 2 || bits == 8)), "Only ",
                fused_only ? "3, 4" : "2, 3, 4, 8", " bits are supported here.");
    TORCH_CHECK(qweight.dim() == 2 && qzeros.dim() == 2 && scales.dim() == 2, "qweight, qzeros and scales must be 2-D");
    const int64_t rows = qweight.size(0), N = qweight.size(1);
    TORCH_CHECK(rows * 32 % bits == 0, "qweight has ", rows, " rows, not a multiple of bits=", bits, " words per 32 channels");
    const int64_t K = rows * 32 / bits;
    TORCH_CHECK(group_size == -1 || group_size > 0, "group_size must be -1 or positive, got ", group_size);
    const int64_t gs = group_size == -1 ? K : group_size;
    const int64_t G = (K + gs - 1) / gs;
    TORCH_CHECK(K % 32 == 0 && N % 32 == 0, "infeatures (", K, ") and outfeatures (", N, ") must be multiples of 32");
    TORCH_CHECK(K < (1LL << 31) && N < (1LL << 31), "layer too large");
    TORCH_CHECK(scales.size(0) == G && scales.size(1) == N, "scales must be [", G, ", ", N, "]");
    TORCH_CHECK(qzeros.size(0) == G && qzeros.size(1) == N / 32 * bits, "qzeros must be [", G, ", ", N / 32 * bits, "]");
    TORCH_CHECK(g_len < 0 || g_len == K, "g_idx must be [", K, "]");
    if (has(bias)) TORCH_CHECK(bias->dim() == 1 && bias->size(0) == N, "bias must be [", N, "]");
    int64_t M = 0;
    if (x.defined()) {
        TORCH_CHECK(x.dim() == 2 && x.size(1) == K, "x must be [M, ", K, "]");
        M = x.size(0);
        TORCH_CHECK(M < (1LL << 31), "too many rows");
    }
    return {M, K, N, G};
}

Tensor gemm(const Tensor &x, const Tensor &qweight, const Tensor &qzeros, const Tensor &scales, const OptTensor &g_idx,
            const OptTensor &bias, int64_t bits, int64_t group_size)
{
    TORCH_CHECK(x.is_cuda(), "x is on ", x.device(), ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
    need(x, "x", at::kHalf, x);
    need(qweight, "qweight", at::kInt, x);
    need(qzeros, "qzeros", at::kInt, x);
    need(scales, "scales", at::kHalf, x);
    if (has(g_idx)) need(*g_idx, "g_idx", at::kInt, x);
    if (has(bias)) need(*bias, "bias", at::kHalf, x);
    const Shape s = check_layer(x, qweight, qzeros, scales, has(g_idx) ? g_idx->numel() : -1, bias, bits, group_size, true);
    Tensor y = at::empty({s.M, s.N}, x.options());
    if (s.M == 0) return y;
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.get_device()).stream();
    gptq_hip_plan plan;
    int rc = gptq_hip_select((int)s.M, (int)s.K, (int)s.N, (int)bits, (int)group_size, has(g_idx), &plan);
    raise(rc, "gptq_hip_gemm", s.M, s.K, s.N, bits, group_size);
    Tensor ws;
    if (plan.workspace_bytes) ws = workspace(x, plan.workspace_bytes, stream);
    rc = gptq_hip_gemm_plan(x.data_ptr(), (const int32_t *)qweight.data_ptr(), (const int32_t *)qzeros.data_ptr(),
                            scales.data_ptr(), (const int32_t *)ptr(g_idx), ptr(bias), y.data_ptr(),
                            ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0, (int)s.M,
                            (int)s.K, (int)s.N, (int)bits, (int)group_size, &plan, stream);
    raise(rc, "gptq_hip_gemm", s.M, s.K, s.N, bits, group_size);
    return y;
}

Tensor gemm_sorted(const Tensor &x, const Tensor &qweight_sorted, const Tensor &qzeros, const Tensor &scales,
                   const Tensor &kmap, const OptTensor &bias, int64_t bits, int64_t group_size)
{
    TORCH_CHECK(x.is_cuda(), "x is on ", x.device(), ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
    need(x, "x", at::kHalf, x);
    need(qweight_sorted, "qweight_sorted", at::kInt, x);
    need(qzeros, "qzeros", at::kInt, x);
    need(scales, "scales", at::kHalf, x);
    need(kmap, "kmap", at::kInt, x);
    if (has(bias)) need(*bias, "bias", at::kHalf, x);
    const Shape s = check_layer(x, qweight_sorted, qzeros, scales, -1, bias, bits, group_size, true);
    TORCH_CHECK(kmap.dim() == 1 && kmap.numel() == 2 * s.K, "kmap must be [", 2 * s.K, "]");
    Tensor y = at::empty({s.M, s.N}, x.options());
    if (s.M == 0) return y;
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.get_device()).stream();
    // the plan of contiguous groups; what the entry point needs beyond it (x in the sorted order) it says itself
    gptq_hip_plan plan;
    int rc = gptq_hip_select((int)s.M, (int)s.K, (int)s.N, (int)bits, (int)group_size, 0, &plan);
    raise(rc, "gptq_hip_gemm_sorted", s.M, s.K, s.N, bits, group_size);
    const size_t need_ws = std::max((size_t)plan.workspace_bytes,
                                    gptq_hip_sorted_workspace_bytes((int)s.M, (int)s.K, (int)s.N, (int)bits, (int)group_size));
    Tensor ws;
    if (need_ws) ws = workspace(x, need_ws, stream);
    rc = gptq_hip_gemm_sorted(x.data_ptr(), (const int32_t *)qweight_sorted.data_ptr(), (const int32_t *)qzeros.data_ptr(),
                              scales.data_ptr(), (const int32_t *)kmap.data_ptr(), ptr(bias), y.data_ptr(),
                              ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0, (int)s.M,
                              (int)s.K, (int)s.N, (int)bits, (int)group_size, &plan, stream);
    raise(rc, "gptq_hip_gemm_sorted", s.M, s.K, s.N, bits, group_size);
    return y;
}

Tensor gemm_tiled(const Tensor &x, const Tensor &qtile, const Tensor &sz, const OptTensor &xsrc, const OptTensor &kinv,
                  const OptTensor &bias, int64_t bits, int64_t group_size)
{
    TORCH_CHECK(x.is_cuda(), "x is on ", x.device(), ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
    need(x, "x", at::kHalf, x);
    need(qtile, "qtile", at::kInt, x);
    need(sz, "sz", at::kInt, x);
    TORCH_CHECK(has(xsrc) == has(kinv), "xsrc and kinv go together: pass both (activation order) or neither");
    if (has(xsrc)) {
        need(*xsrc, "xsrc", at::kInt, x);
        need(*kinv, "kinv", at::kShort, x);
    }
    if (has(bias)) need(*bias, "bias", at::kHalf, x);
    TORCH_CHECK(bits == 2 || bits == 3 || bits == 4 || bits == 8, "Only 2, 3, 4, 8 bits are supported.");
    TORCH_CHECK(x.dim() == 2 && sz.dim() == 2, "x must be [M, K] and sz [G, N]");
    const int64_t M = x.size(0), K = x.size(1), N = sz.size(1);
    TORCH_CHECK(M < (1LL << 31) && K <= 65536 && N < (1LL << 31), "layer too large");
    const int64_t Kp = (K + 63) / 64 * 64;
    TORCH_CHECK(qtile.numel() * 4 == Kp * N * bits / 8, "qtile holds ", qtile.numel() * 4, " bytes, a ", K, " x ", N,
                " layer of ", bits, " bits needs ", Kp * N * bits / 8);
    if (has(xsrc))
        TORCH_CHECK(xsrc->dim() == 1 && xsrc->numel() == Kp && kinv->dim() == 1 && kinv->numel() == K, "xsrc must be [", Kp,
                    "] and kinv [", K, "]");
    if (has(bias)) TORCH_CHECK(bias->dim() == 1 && bias->size(0) == N, "bias must be [", N, "]");
    Tensor y = at::empty({M, N}, x.options());
    if (M == 0) return y;
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.get_device()).stream();
    gptq_hip_plan plan;
    int rc = gptq_hip_select_tiled((int)M, (int)K, (int)N, (int)bits, (int)group_size, &plan);
    raise(rc, "gptq_hip_gemm_tiled", M, K, N, bits, group_size);
    TORCH_CHECK(sz.size(0) == (group_size == -1 ? 1 : K / group_size), "sz must have one row per group");
    Tensor ws;
    if (plan.workspace_bytes) ws = workspace(x, plan.workspace_bytes, stream, workspace_kind(plan));
    rc = gptq_hip_gemm_tiled(x.data_ptr(), qtile.data_ptr(), (const uint32_t *)sz.data_ptr(), (const int32_t *)ptr(xsrc),
                             (const uint16_t *)ptr(kinv), ptr(bias), y.data_ptr(), ws.defined() ? ws.data_ptr() : nullptr,
                             ws.defined() ? (size_t)ws.numel() : 0, (int)M, (int)K, (int)N, (int)bits, (int)group_size,
                             &plan, stream);
    raise(rc, "gptq_hip_gemm_tiled", M, K, N, bits, group_size);
    return y;
}

Tensor dequant(const Tensor &qweight, const Tensor &qzeros, const Tensor &scales, const OptTensor &g_idx, int64_t bits,
               int64_t group_size)
{
    TORCH_CHECK(qweight.is_cuda(), "qweight is on ", qweight.device(),
                ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
    need(qweight, "qweight", at::kInt, qweight);
    need(qzeros, "qzeros", at::kInt, qweight);
    need(scales, "scales", at::kHalf, qweight);
    if (has(g_idx)) need(*g_idx, "g_idx", at::kInt, qweight);
    const Shape s = check_layer(Tensor(), qweight, qzeros, scales, has(g_idx) ? g_idx->numel() : -1, OptTensor(), bits,
                                group_size, false);
    Tensor w = at::empty({s.K, s.N}, scales.options());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(qweight.device());
    void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(qweight.get_device()).stream();
    const int rc = gptq_hip_dequant((const int32_t *)qweight.data_ptr(), (const int32_t *)qzeros.data_ptr(), scales.data_ptr(),
                                    (const int32_t *)ptr(g_idx), w.data_ptr(), (int)s.K, (int)s.N, (int)bits, (int)group_size,
                                    stream);
    raise(rc, "gptq_hip_dequant", 0, s.K, s.N, bits, group_size);
    return w;
}

// One layer's constant tensors, bound once: forward(x) then crosses from Python with a single argument (the
// argument handling of an eight-argument operator costs more host time than the launch itself).
// kind: 0 = checkpoint tensors (qweight, qzeros, scales, g_idx?), 1 = sorted copy (qweight_sorted, qzeros,
// scales, kmap), 2 = tiled copy (qtile, sz, -, xsrc?, kinv?).
struct Layer : torch::CustomClassHolder {
    int64_t kind, bits, group_size;
    Tensor a, b, c;
    OptTensor d, e, bias;

    Layer(int64_t kind_, Tensor a_, Tensor b_, OptTensor c_, OptTensor d_, OptTensor e_, OptTensor bias_, int64_t bits_,
          int64_t group_size_)
        : kind(kind_), bits(bits_), group_size(group_size_), a(std::move(a_)), b(std::move(b_)),
          c(has(c_) ? *c_ : Tensor()), d(std::move(d_)), e(std::move(e_)), bias(std::move(bias_))
    {
        TORCH_CHECK(kind >= 0 && kind <= 2, "kind must be 0 (checkpoint tensors), 1 (sorted copy) or 2 (tiled copy)");
        TORCH_CHECK(kind == 2 || c.defined(), "scales are missing");
        TORCH_CHECK(kind != 1 || has(d), "the sorted copy needs its kmap");
    }

    // What the first fully checked call fixed for its row count: later calls with the same M check x only.
    // Written once, under the mutex, before fast_M is published; calls with another M take the checked path.
    std::atomic<int64_t> fast_M{-1};
    int64_t K = 0, N = 0;
    gptq_hip_plan plan{};
    size_t ws_need = 0;
    std::mutex fix_mutex;

    Tensor forward(const Tensor &x)
    {
        const int64_t fast_rows = fast_M.load(std::memory_order_acquire);
        if (x.dim() == 2 && x.size(0) == fast_rows) {
            TORCH_CHECK(x.is_cuda() && x.device() == a.device(), "x is on ", x.device(), ", the layer on ", a.device(),
                        ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
            TORCH_CHECK(x.scalar_type() == at::kHalf && x.is_contiguous() && x.size(1) == K,
                        "x must be a contiguous fp16 [M, ", K, "] matrix");
            Tensor y = at::empty({fast_rows, N}, x.options());
            const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
            void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.get_device()).stream();
            Tensor ws;
            if (ws_need) ws = workspace(x, ws_need, stream, workspace_kind(plan));
            void *wsp = ws.defined() ? ws.data_ptr() : nullptr;
            const size_t wsb = ws.defined() ? (size_t)ws.numel() : 0;
            const int M = (int)fast_rows, bi = (int)bits, gs = (int)group_size;
            int rc;
            if (kind == 0)
                rc = gptq_hip_gemm_plan(x.data_ptr(), (const int32_t *)a.data_ptr(), (const int32_t *)b.data_ptr(), c.data_ptr(),
                                        (const int32_t *)ptr(d), ptr(bias), y.data_ptr(), wsp, wsb, M, (int)K, (int)N, bi, gs,
                                        &plan, stream);
            else if (kind == 1)
                rc = gptq_hip_gemm_sorted(x.data_ptr(), (const int32_t *)a.data_ptr(), (const int32_t *)b.data_ptr(),
                                          c.data_ptr(), (const int32_t *)ptr(d), ptr(bias), y.data_ptr(), wsp, wsb, M, (int)K,
                                          (int)N, bi, gs, &plan, stream);
            else
                rc = gptq_hip_gemm_tiled(x.data_ptr(), a.data_ptr(), (const uint32_t *)b.data_ptr(), (const int32_t *)ptr(d),
                                         (const uint16_t *)ptr(e), ptr(bias), y.data_ptr(), wsp, wsb, M, (int)K, (int)N, bi, gs,
                                         &plan, stream);
            raise(rc, "gptq_hip.Layer.forward", fast_rows, K, N, bits, group_size);
            return y;
        }
        // the checked path; what it selects is what the operators select
        Tensor y;
        switch (kind) {
        case 0:
            y = gemm(x, a, b, c, d, bias, bits, group_size);
            break;
        case 1:
            y = gemm_sorted(x, a, b, c, *d, bias, bits, group_size);
            break;
        default:
            y = gemm_tiled(x, a, b, d, e, bias, bits, group_size);
        }
        if (x.size(0) > 0 && fast_rows < 0) {
            const int M = (int)x.size(0), Ki = (int)x.size(1), Ni = (int)y.size(1), bi = (int)bits, gs = (int)group_size;
            gptq_hip_plan p;
            const int rc = kind == 2 ? gptq_hip_select_tiled(M, Ki, Ni, bi, gs, &p)
                                     : gptq_hip_select(M, Ki, Ni, bi, gs, kind == 0 && has(d), &p);
            const std::lock_guard<std::mutex> lock(fix_mutex);
            if (rc == GPTQ_HIP_OK && fast_M.load(std::memory_order_relaxed) < 0) {
                plan = p;
                ws_need = p.workspace_bytes;
                if (kind == 1) ws_need = std::max(ws_need, gptq_hip_sorted_workspace_bytes(M, Ki, Ni, bi, gs));
                K = Ki;
                N = Ni;
                fast_M.store(M, std::memory_order_release);
            }
        }
        return y;
    }
};

}  // namespace

TORCH_LIBRARY(gptq_hip, m)
{
    m.class_<Layer>("Layer")
        .def(torch::init<int64_t, Tensor, Tensor, OptTensor, OptTensor, OptTensor, OptTensor, int64_t, int64_t>())
        .def("forward", &Layer::forward);
    m.def("gemm(Tensor x, Tensor qweight, Tensor qzeros, Tensor scales, Tensor? g_idx, Tensor? bias, int bits, "
          "int group_size) -> Tensor");
    m.def("gemm_sorted(Tensor x, Tensor qweight_sorted, Tensor qzeros, Tensor scales, Tensor kmap, Tensor? bias, "
          "int bits, int group_size) -> Tensor");
    m.def("gemm_tiled(Tensor x, Tensor qtile, Tensor sz, Tensor? xsrc, Tensor? kinv, Tensor? bias, int bits, "
          "int group_size) -> Tensor");
    m.def("dequant(Tensor qweight, Tensor qzeros, Tensor scales, Tensor? g_idx, int bits, int group_size) -> Tensor");
    m.def("binding_build_id() -> str", []() -> std::string { return GPTQ_HIP_BUILD_ID; });
}

TORCH_LIBRARY_IMPL(gptq_hip, CUDA, m)
{
    m.impl("gemm", &gemm);
    m.impl("gemm_sorted", &gemm_sorted);
    m.impl("gemm_tiled", &gemm_tiled);
    m.impl("dequant", &dequant);
}

// CPU tensors: there is no CPU implementation and none is wanted; say so instead of the dispatcher's list of keys.
namespace {

[[noreturn]] void no_cpu(const char *op, const Tensor &t)
{
    TORCH_CHECK(false, "torch.ops.gptq_hip.", op, ": argument on ", t.device(),
                ": the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback");
}

Tensor gemm_cpu(const Tensor &x, const Tensor &, const Tensor &, const Tensor &, const OptTensor &, const OptTensor &, int64_t,
                int64_t)
{
    no_cpu("gemm", x);
}
Tensor gemm_sorted_cpu(const Tensor &x, const Tensor &, const Tensor &, const Tensor &, const Tensor &, const OptTensor &,
                       int64_t, int64_t)
{
    no_cpu("gemm_sorted", x);
}
Tensor gemm_tiled_cpu(const Tensor &x, const Tensor &, const Tensor &, const OptTensor &, const OptTensor &, const OptTensor &,
                      int64_t, int64_t)
{
    no_cpu("gemm_tiled", x);
}
Tensor dequant_cpu(const Tensor &qweight, const Tensor &, const Tensor &, const OptTensor &, int64_t, int64_t)
{
    no_cpu("dequant", qweight);
}

}  // namespace

TORCH_LIBRARY_IMPL(gptq_hip, CPU, m)
{
    m.impl("gemm", &gemm_cpu);
    m.impl("gemm_sorted", &gemm_sorted_cpu);
    m.impl("gemm_tiled", &gemm_tiled_cpu);
    m.impl("dequant", &dequant_cpu);
}
