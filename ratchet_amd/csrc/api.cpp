// C ABI of libratchet_hip (see include/ratchet_hip.h).  Every entry point
// catches C++ exceptions and reports a status; nothing here computes on the
// host: a missing device is an error, never a fallback.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <string>

#include "device_common.h"
#include "spec.h"

struct rt_gguf;
namespace rt {
rt_status gguf_load_tensor(const rt_gguf *g, const void *image, uint64_t size, uint64_t index, int32_t dst_dtype,
                           void *staging, void *dst, hipStream_t stream, std::string &why, hipError_t &herr);
}

// Library-owned scratch for rt_matmul_enqueue_static: the f32 partial sums of a product whose K is
// shared among workgroups.  Every GPU the library runs on holds its own copy of the array at its
// own address for the life of the process.  A split keeps tiles x shares within the compute-unit
// count, so on a device of up to 256 compute units no split needs more than 256 tiles of
// 160 x 128 floats, which is this size.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels are given the address that call returns.
constexpr uint64_t kStaticScratchBytes = RT_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct rt_ctx {
    rt::DeviceInfo dev;
    std::mutex mu;
    std::string last_error;
    int last_hip = 0;
    void *static_scratch = nullptr;   // device address of `scratch` on this context's GPU
    hipError_t static_scratch_err = hipSuccess;
    // Checked mode (the environment variable RATCHET_CHECKED, as in the reference's
    // gpu/pools/kernel_module_pool.rs:62-67, read when the context is created): before a matmul is
    // enqueued every operand's device allocation is looked up and must hold the bytes the descriptor
    // implies.  Costs a runtime query per pointer and call; off by default.
    bool checked = false;
};

namespace {

rt_status fail(rt_ctx *ctx, rt_status st, const std::string &msg, hipError_t herr = hipSuccess) {
    if (ctx) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        ctx->last_error = msg;
        if (herr != hipSuccess) {
            ctx->last_hip = (int)herr;
            ctx->last_error += std::string(": ") + hipGetErrorString(herr);
        }
    }
    return st;
}

// Checked mode: `ptr` must lie in a device allocation that extends at least `need` bytes past it.
rt_status check_extent(rt_ctx *ctx, const void *ptr, uint64_t need, const char *what) {
    if (!ptr || need == 0) return RT_OK;
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    const hipError_t e = hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(ctx, RT_ERR_INVALID_ARG, std::string("checked: ") + what + " is not a device allocation");
    }
    const uint64_t off = (uint64_t)((const uint8_t *)ptr - (const uint8_t *)base);
    if (off > size || size - off < need)
        return fail(ctx, RT_ERR_INVALID_ARG, std::string("checked: ") + what + " holds " + std::to_string(size - off) +
                                                 " bytes from the pointer on, the descriptor needs " + std::to_string(need));
    return RT_OK;
}

uint64_t shape_numel(const int64_t *shape, int32_t rank) {
    uint64_t n = 1;
    for (int32_t i = 0; i < rank; i++) n *= (uint64_t)shape[i];
    return n;
}

rt_status hip_fail(rt_ctx *ctx, const char *what, hipError_t e) {
    return fail(ctx, e == hipErrorOutOfMemory ? RT_ERR_OOM : RT_ERR_HIP, what, e);
}

struct DeviceGuard {
    int prev = -1;
    bool ok = false;
    explicit DeviceGuard(int ordinal) {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        ok = hipSetDevice(ordinal) == hipSuccess;
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

#define RT_GUARD_BEGIN try {
#define RT_GUARD_END(ctx)                                                                          \
    }                                                                                              \
    catch (const std::bad_alloc &) { return fail(ctx, RT_ERR_OOM, "host allocation failed"); }     \
    catch (const std::exception &e) { return fail(ctx, RT_ERR_INVALID_ARG, e.what()); }            \
    catch (...) { return fail(ctx, RT_ERR_INVALID_ARG, "unknown exception"); }


// A descriptor lowered once: the strided problem with its kernel family, and what checked mode compares
// the operands' allocations with.
struct Lowered {
    rt::Problem p;
    bool has_bias = false;
    uint64_t lhs_bytes = 0, rhs_bytes = 0, bias_bytes = 0, out_bytes = 0;
};

rt_status lower_matmul(rt_ctx *ctx, const rt_matmul_desc &desc, int32_t activation, Lowered &low) {
    if (activation != RT_ACT_NONE && activation != RT_ACT_GELU && activation != RT_ACT_SILU)
        return fail(ctx, RT_ERR_INVALID_ARG, "unknown activation");
    rt_gemm_spec spec;
    std::string why;
    const rt_status st = rt::make_spec(desc, spec, low.p, &why);
    if (st != RT_OK) return fail(ctx, st, why);
    low.p.act = activation;
    low.has_bias = desc.has_bias != 0;
    if (ctx->checked &&
        (rt_tensor_nbytes(desc.lhs_dt, shape_numel(desc.lhs_shape, desc.lhs_rank), &low.lhs_bytes) != RT_OK ||
         rt_tensor_nbytes(desc.rhs_dt, shape_numel(desc.rhs_shape, desc.rhs_rank), &low.rhs_bytes) != RT_OK ||
         (desc.has_bias && rt_tensor_nbytes(desc.bias_dt, shape_numel(desc.bias_shape, desc.bias_rank), &low.bias_bytes) != RT_OK)))
        return fail(ctx, RT_ERR_INVALID_ARG, "checked: operand sizes");
    low.out_bytes = (uint64_t)low.p.stacks * (uint64_t)low.p.M * (uint64_t)low.p.N * (low.p.act_dt == RT_F16 ? 2u : 4u);
    return RT_OK;
}

// The kernel families in the order they are offered a problem; each declines (hipErrorNotSupported) what it
// does not take.  The first two see the streaming kernel kinds make_spec chose; from the third on the problem is
// a tiled one.
using Launcher = hipError_t (*)(const rt::Problem &, const void *, const void *, const void *, void *, hipStream_t,
                                const rt::DeviceInfo &);
constexpr Launcher kLaunchers[] = {rt::launch_gemv,          // streaming kernels
                                   rt::launch_gemv_chunked,  // Q8_0H / Q4_K weights against a few vectors more than one streaming launch takes
                                   rt::launch_gemm_stream,   // f16 / Q8_0H weights against a few dozen activation rows: one pass over the weight
                                   rt::launch_gemm_nt,       // K-contiguous f16 / Q8_0H problems: the large-tile kernel
                                   rt::launch_gemm_nn_smalln, // f16 products with an untransposed narrow rhs (attention P.V)
                                   rt::launch_gemm_f32,      // f32 products whose operands each have a contiguous axis
                                   rt::launch_gemm_q4k,      // Q4_K weights against many activation rows
                                   rt::launch_gemm};         // anything
constexpr int kNumLaunchers = (int)(sizeof(kLaunchers) / sizeof(kLaunchers[0])), kFirstTiled = 2;

// `hint` (a plan's memory): the family that took this problem last time is offered it first.
rt_status run_matmul(rt_ctx *ctx, const Lowered &low, const void *lhs, const void *rhs, const void *bias, void *out,
                     void *workspace, uint64_t workspace_bytes, void *stream, std::atomic<int> *hint) {
    rt::Problem p = low.p;
    p.workspace = workspace_bytes ? workspace : nullptr, p.workspace_bytes = workspace ? workspace_bytes : 0;
    if (p.kernel == RT_KERNEL_NONE) return RT_OK; // empty output
    if (!lhs || !rhs || !out || (low.has_bias && !bias)) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    const void *A = p.swapped ? rhs : lhs, *B = p.swapped ? lhs : rhs;
    const void *bp = low.has_bias ? bias : nullptr;
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    if (ctx->checked) {
        rt_status st;
        if ((st = check_extent(ctx, lhs, low.lhs_bytes, "lhs")) != RT_OK || (st = check_extent(ctx, rhs, low.rhs_bytes, "rhs")) != RT_OK ||
            (st = check_extent(ctx, bp, low.bias_bytes, "bias")) != RT_OK || (st = check_extent(ctx, out, low.out_bytes, "out")) != RT_OK ||
            // the library's own static scratch is a device symbol of known size, not an allocation to look up
            (p.workspace != ctx->static_scratch &&
             (st = check_extent(ctx, p.workspace, p.workspace_bytes, "workspace")) != RT_OK))
            return st;
    }
    const bool streaming = p.kernel == RT_KERNEL_GEMV_Q8 || p.kernel == RT_KERNEL_GEMV_Q4K || p.kernel == RT_KERNEL_GEMV_FLOAT;
    const int tiled_kind = p.act_dt == RT_F16 ? RT_KERNEL_GEMM_F16 : RT_KERNEL_GEMM_F32;
    hipError_t e = hipErrorNotSupported;
    const int first = hint ? hint->load(std::memory_order_relaxed) : -1;
    if (first >= 0) {
        if (first >= kFirstTiled) p.kernel = tiled_kind;
        e = kLaunchers[first](p, A, B, bp, out, (hipStream_t)stream, ctx->dev);
        if (e == hipErrorNotSupported) p.kernel = low.p.kernel; // other pointers than last time: ask everyone again
    }
    for (int i = streaming ? 0 : 1; i < kNumLaunchers && e == hipErrorNotSupported; i++) {
        if (i == first) continue;
        // operands that miss the streaming kernels' alignment take the tiled kernels
        if (i >= kFirstTiled) p.kernel = tiled_kind;
        e = kLaunchers[i](p, A, B, bp, out, (hipStream_t)stream, ctx->dev);
        if (e == hipSuccess && hint) hint->store(i, std::memory_order_relaxed);
    }
    // no kernel takes the shape (more than 65535 stacks or row tiles of the generic kernel, a misaligned
    // quantized operand): a limit of this library, not a failure of the runtime
    if (e == hipErrorNotSupported)
        return fail(ctx, RT_ERR_UNSUPPORTED, "matmul: no kernel takes this shape (over 65535 stacks or 65535 row tiles, or a "
                                             "quantized operand that is not 16-byte aligned)");
    if (e != hipSuccess) return hip_fail(ctx, "matmul launch", e);
    return RT_OK;
}

} // namespace

// What rt_matmul_plan_create keeps: the lowered problem, and which kernel family took it last time.
struct rt_matmul_plan {
    rt_ctx *ctx = nullptr;
    Lowered low;
    std::atomic<int> launcher{-1};
};

extern "C" {

const char *rt_status_string(rt_status s) {
    switch (s) {
    case RT_OK: return "RT_OK";
    case RT_ERR_INVALID_ARG: return "RT_ERR_INVALID_ARG";
    case RT_ERR_INVALID_SHAPE: return "RT_ERR_INVALID_SHAPE";
    case RT_ERR_DTYPE_MISMATCH: return "RT_ERR_DTYPE_MISMATCH";
    case RT_ERR_UNSUPPORTED: return "RT_ERR_UNSUPPORTED";
    case RT_ERR_NO_DEVICE: return "RT_ERR_NO_DEVICE";
    case RT_ERR_HIP: return "RT_ERR_HIP";
    case RT_ERR_OOM: return "RT_ERR_OOM";
    }
    return "RT_ERR_UNKNOWN";
}

const char *rt_kernel_string(int32_t k) {
    switch (k) {
    case RT_KERNEL_NONE: return "none";
    case RT_KERNEL_GEMV_Q8: return "gemv_q8";
    case RT_KERNEL_GEMV_Q4K: return "gemv_q4k";
    case RT_KERNEL_GEMV_FLOAT: return "gemv_float";
    case RT_KERNEL_GEMM_F16: return "gemm_f16";
    case RT_KERNEL_GEMM_F32: return "gemm_f32";
    }
    return "unknown";
}

rt_status rt_matmul_infer(const rt_matmul_desc *desc, int64_t *out_shape, int32_t *out_rank, int32_t *out_dt) {
    if (!desc || !out_shape || !out_rank || !out_dt) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    rt::Shape out;
    int dt = 0;
    rt_status st = rt::infer(*desc, out, dt);
    if (st != RT_OK) return st;
    if (out.size() > RT_MAX_RANK) return RT_ERR_INVALID_ARG;
    *out_rank = (int32_t)out.size();
    for (size_t i = 0; i < out.size(); i++) out_shape[i] = out[i];
    *out_dt = dt;
    return RT_OK;
    RT_GUARD_END(nullptr)
}

rt_status rt_matmul_validate(const rt_matmul_desc *desc) {
    if (!desc) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    return rt::validate(*desc);
    RT_GUARD_END(nullptr)
}

rt_status rt_matmul_spec(const rt_matmul_desc *desc, rt_gemm_spec *spec) {
    if (!desc || !spec) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    rt::Problem p;
    return rt::make_spec(*desc, *spec, p);
    RT_GUARD_END(nullptr)
}

uint64_t rt_q8_0_scale_offset(uint64_t numel) { return (numel + 255u) & ~(uint64_t)255u; }

rt_status rt_tensor_nbytes(int32_t dtype, uint64_t numel, uint64_t *nbytes) {
    if (!nbytes) return RT_ERR_INVALID_ARG;
    auto a256 = [](uint64_t n) { return (n + 255u) & ~(uint64_t)255u; };
    switch (dtype) {
    case RT_F32: *nbytes = numel * 4; return RT_OK;
    case RT_F16: *nbytes = numel * 2; return RT_OK;
    case RT_Q8_0F:
    case RT_Q8_0H:
        if (numel % 32) return RT_ERR_UNSUPPORTED;
        *nbytes = a256(numel) + a256((numel / 32) * (dtype == RT_Q8_0H ? 2 : 4));
        return RT_OK;
    case RT_Q4_K:
        if (numel % 256) return RT_ERR_UNSUPPORTED;
        *nbytes = (numel / 256) * 144;
        return RT_OK;
    }
    return RT_ERR_INVALID_ARG;
}

rt_status rt_ctx_create(int32_t device_ordinal, rt_ctx **ctx) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    *ctx = nullptr;
    RT_GUARD_BEGIN
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return RT_ERR_NO_DEVICE;
    }
    if (device_ordinal < 0 || device_ordinal >= count) return RT_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_ordinal) != hipSuccess) return RT_ERR_NO_DEVICE;
    rt_ctx *c = new rt_ctx();
    c->dev.ordinal = device_ordinal;
    c->dev.num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    {
        // the address of the static scratch array on this GPU (each device has its own copy)
        DeviceGuard dg(device_ordinal);
        void *ptr = nullptr;
        c->static_scratch_err = dg.ok ? hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) : hipErrorInvalidDevice;
        if (c->static_scratch_err == hipSuccess) c->static_scratch = ptr;
        else (void)hipGetLastError();
    }
    if (const char *env = std::getenv("RATCHET_CHECKED")) c->checked = env[0] != '\0' && !(env[0] == '0' && env[1] == '\0');
    *ctx = c;
    return RT_OK;
    RT_GUARD_END(nullptr)
}

rt_status rt_ctx_destroy(rt_ctx *ctx) {
    delete ctx;
    return RT_OK;
}

const char *rt_last_error(const rt_ctx *ctx) { return ctx ? ctx->last_error.c_str() : ""; }
int32_t rt_last_hip_error(const rt_ctx *ctx) { return ctx ? ctx->last_hip : 0; }

rt_status rt_buf_alloc(rt_ctx *ctx, uint64_t nbytes, void **dptr) {
    if (!ctx || !dptr) return RT_ERR_INVALID_ARG;
    DeviceGuard dg(ctx->dev.ordinal);
    *dptr = nullptr;
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = hipMalloc(dptr, nbytes ? nbytes : 4);
    if (e != hipSuccess) return hip_fail(ctx, "hipMalloc", e);
    return RT_OK;
}

rt_status rt_buf_free(rt_ctx *ctx, void *dptr) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    if (!dptr) return RT_OK;
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = hipFree(dptr);
    if (e != hipSuccess) return hip_fail(ctx, "hipFree", e);
    return RT_OK;
}

rt_status rt_buf_upload(rt_ctx *ctx, void *dst_dev, const void *src_host, uint64_t nbytes, void *stream) {
    if (!ctx || (nbytes && (!dst_dev || !src_host))) return RT_ERR_INVALID_ARG;
    if (!nbytes) return RT_OK;
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "hipMemcpyAsync(H2D)", e);
    return RT_OK;
}

rt_status rt_buf_download(rt_ctx *ctx, void *dst_host, const void *src_dev, uint64_t nbytes, void *stream) {
    if (!ctx || (nbytes && (!dst_host || !src_dev))) return RT_ERR_INVALID_ARG;
    if (!nbytes) return RT_OK;
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "hipMemcpyAsync(D2H)", e);
    return RT_OK;
}

rt_status rt_sync(rt_ctx *ctx, void *stream) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "hipStreamSynchronize", e);
    return RT_OK;
}

rt_status rt_matmul_enqueue(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                            const void *bias, void *out, void *stream) {
    return rt_matmul_enqueue_fused(ctx, desc, lhs, rhs, bias, out, RT_ACT_NONE, stream);
}

rt_status rt_matmul_enqueue_fused(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                                  const void *bias, void *out, int32_t activation, void *stream) {
    return rt_matmul_enqueue_ws(ctx, desc, lhs, rhs, bias, out, activation, nullptr, 0, stream);
}

rt_status rt_matmul_workspace_bytes(rt_ctx *ctx, const rt_matmul_desc *desc, uint64_t *bytes) {
    if (!ctx || !desc || !bytes) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    *bytes = 0;
    rt_gemm_spec spec;
    rt::Problem p;
    std::string why;
    rt_status st = rt::make_spec(*desc, spec, p, &why);
    if (st != RT_OK) return fail(ctx, st, why);
    // only the large-tile GEMM shares a problem among workgroups; the streaming kernels take M <= 16
    if (p.kernel == RT_KERNEL_GEMM_F16) *bytes = rt::gemm_nt_workspace_bytes(p, ctx->dev);
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_matmul_enqueue_ws(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                               const void *bias, void *out, int32_t activation, void *workspace,
                               uint64_t workspace_bytes, void *stream) {
    if (!ctx || !desc) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    Lowered low;
    const rt_status st = lower_matmul(ctx, *desc, activation, low);
    if (st != RT_OK) return st;
    return run_matmul(ctx, low, lhs, rhs, bias, out, workspace, workspace_bytes, stream, nullptr);
    RT_GUARD_END(ctx)
}

rt_status rt_matmul_plan_create(rt_ctx *ctx, const rt_matmul_desc *desc, int32_t activation, rt_matmul_plan **plan) {
    if (!ctx || !desc || !plan) return RT_ERR_INVALID_ARG;
    *plan = nullptr;
    RT_GUARD_BEGIN
    std::unique_ptr<rt_matmul_plan> pl(new rt_matmul_plan);
    pl->ctx = ctx;
    const rt_status st = lower_matmul(ctx, *desc, activation, pl->low);
    if (st != RT_OK) return st;
    *plan = pl.release();
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_matmul_plan_enqueue(rt_matmul_plan *plan, const void *lhs, const void *rhs, const void *bias, void *out,
                                 void *workspace, uint64_t workspace_bytes, void *stream) {
    if (!plan) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    return run_matmul(plan->ctx, plan->low, lhs, rhs, bias, out, workspace, workspace_bytes, stream, &plan->launcher);
    RT_GUARD_END(plan->ctx)
}

rt_status rt_matmul_plan_destroy(rt_matmul_plan *plan) {
    delete plan;
    return RT_OK;
}

rt_status rt_matmul_enqueue_static(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                                   const void *bias, void *out, int32_t activation, void *stream) {
    if (!ctx || !desc) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    uint64_t need = 0;
    const rt_status st = rt_matmul_workspace_bytes(ctx, desc, &need);
    if (st != RT_OK) return st;
    if (need == 0) // this product is not split: no scratch is touched
        return rt_matmul_enqueue_ws(ctx, desc, lhs, rhs, bias, out, activation, nullptr, 0, stream);
    if (need > kStaticScratchBytes)
        return fail(ctx, RT_ERR_UNSUPPORTED,
                    "rt_matmul_enqueue_static: the split of this product needs " + std::to_string(need) +
                        " bytes of scratch, the static buffer holds " + std::to_string(kStaticScratchBytes));
    if (!ctx->static_scratch)
        return hip_fail(ctx, "rt_matmul_enqueue_static: hipGetSymbolAddress of the static scratch failed", ctx->static_scratch_err);
    // every share's sums are written before the second kernel reads them, so nothing needs clearing
    return rt_matmul_enqueue_ws(ctx, desc, lhs, rhs, bias, out, activation, ctx->static_scratch, kStaticScratchBytes, stream);
    RT_GUARD_END(ctx)
}

rt_status rt_quantize_q8_0(rt_ctx *ctx, const void *src_f32, uint64_t numel, void *dst, void *stream) {
    if (!ctx || (numel && (!src_f32 || !dst))) return RT_ERR_INVALID_ARG;
    if (numel % 32) return fail(ctx, RT_ERR_UNSUPPORTED, "numel must be a multiple of 32");
    if (((uintptr_t)src_f32 | (uintptr_t)dst) & 15u) return fail(ctx, RT_ERR_INVALID_ARG, "buffers must be 16-byte aligned");
    DeviceGuard dg(ctx->dev.ordinal);
    hipError_t e = rt::launch_quantize_q8_0((const float *)src_f32, numel, dst, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "quantize_q8_0 launch", e);
    return RT_OK;
}

rt_status rt_dequantize(rt_ctx *ctx, int32_t dtype, const void *src, uint64_t numel, void *dst_f32, void *stream) {
    if (!ctx || (numel && (!src || !dst_f32))) return RT_ERR_INVALID_ARG;
    if (!rt::is_quantized(dtype)) return fail(ctx, RT_ERR_DTYPE_MISMATCH, "not a quantized dtype");
    if (numel % rt::block_numel(dtype)) return fail(ctx, RT_ERR_UNSUPPORTED, "numel must be a multiple of the block size");
    if (((uintptr_t)src | (uintptr_t)dst_f32) & 15u) return fail(ctx, RT_ERR_INVALID_ARG, "buffers must be 16-byte aligned");
    DeviceGuard dg(ctx->dev.ordinal);
    hipError_t e = rt::launch_dequantize(dtype, src, numel, (float *)dst_f32, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "dequantize launch", e);
    return RT_OK;
}

rt_status rt_transcode_gguf_q8_0(rt_ctx *ctx, const void *blocks, uint64_t n_blocks, int32_t dst_dtype, void *dst,
                                 void *stream) {
    if (!ctx || (n_blocks && (!blocks || !dst))) return RT_ERR_INVALID_ARG;
    if (dst_dtype != RT_Q8_0F && dst_dtype != RT_Q8_0H) return fail(ctx, RT_ERR_DTYPE_MISMATCH, "dst must be Q8_0F or Q8_0H");
    if (((uintptr_t)blocks & 1u) || ((uintptr_t)dst & 15u)) return fail(ctx, RT_ERR_INVALID_ARG, "misaligned buffer");
    DeviceGuard dg(ctx->dev.ordinal);
    hipError_t e = rt::launch_transcode_gguf_q8_0(blocks, n_blocks, dst_dtype, dst, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "transcode launch", e);
    return RT_OK;
}

rt_status rt_softmax_validate(int32_t dtype, int32_t rank, const int64_t *shape, int32_t dim) {
    if (!shape || rank < 0 || rank > RT_MAX_RANK) return RT_ERR_INVALID_ARG;
    if (rank < 2 || dim < 0 || dim >= rank) return RT_ERR_INVALID_SHAPE; // softmax.rs:28-33
    for (int i = 0; i < rank; i++)
        if (shape[i] < 0) return RT_ERR_INVALID_SHAPE;
    if (dtype != RT_F32 && dtype != RT_F16) return RT_ERR_DTYPE_MISMATCH; // softmax.rs:36-39
    if (dim != rank - 1) return RT_ERR_UNSUPPORTED;
    return RT_OK;
}

rt_status rt_softmax_enqueue(rt_ctx *ctx, int32_t dtype, void *x, int32_t rank, const int64_t *shape, int32_t dim,
                             void *stream) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    const rt_status st = rt_softmax_validate(dtype, rank, shape, dim);
    if (st != RT_OK) return fail(ctx, st, "softmax: invalid tensor or dimension");
    int64_t rows = 1;
    for (int i = 0; i < rank - 1; i++) rows *= shape[i];
    const int64_t n = shape[rank - 1];
    if (rows == 0 || n == 0) return RT_OK;
    if (!x) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = rt::launch_softmax(dtype, x, rows, n, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "softmax launch", e);
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_unary_enqueue(rt_ctx *ctx, int32_t activation, int32_t dtype, const void *src, void *dst, uint64_t numel,
                           void *stream) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    if (activation != RT_ACT_GELU && activation != RT_ACT_SILU) return fail(ctx, RT_ERR_INVALID_ARG, "unknown activation");
    if (dtype != RT_F32 && dtype != RT_F16) return fail(ctx, RT_ERR_DTYPE_MISMATCH, "unary operators take F32 or F16");
    if (numel == 0) return RT_OK;
    if (!src || !dst) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    if (((uintptr_t)src | (uintptr_t)dst) & 15u) return fail(ctx, RT_ERR_INVALID_ARG, "buffers must be 16-byte aligned");
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = rt::launch_unary(activation, dtype, src, dst, numel, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "unary launch", e);
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_cast_enqueue(rt_ctx *ctx, int32_t src_dtype, int32_t dst_dtype, const void *src, void *dst, uint64_t numel,
                          void *stream) {
    if (!ctx) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    const bool ok = (src_dtype == RT_F32 && dst_dtype == RT_F16) || (src_dtype == RT_F16 && dst_dtype == RT_F32);
    if (!ok) return fail(ctx, RT_ERR_DTYPE_MISMATCH, "cast is between F32 and F16");
    if (numel == 0) return RT_OK;
    if (!src || !dst) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    if (src == dst) return fail(ctx, RT_ERR_INVALID_ARG, "cast cannot run in place");
    if (((uintptr_t)src | (uintptr_t)dst) & 15u) return fail(ctx, RT_ERR_INVALID_ARG, "buffers must be 16-byte aligned");
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = rt::launch_cast(src_dtype, dst_dtype, src, dst, numel, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "cast launch", e);
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_attention_validate(const rt_attention_desc *d) {
    if (!d) return RT_ERR_INVALID_ARG;
    if (d->dtype != RT_F16) return RT_ERR_DTYPE_MISMATCH;
    if (d->batch < 0 || d->heads < 0 || d->q_len < 0 || d->kv_len < 0) return RT_ERR_INVALID_SHAPE;
    if (d->head_dim < 8 || d->head_dim > 128 || d->head_dim % 8) return RT_ERR_INVALID_SHAPE;
    const int64_t *strides[4] = {d->q_strides, d->k_strides, d->v_strides, d->o_strides};
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 3; j++) {
            if (strides[i][j] < 0) return RT_ERR_INVALID_SHAPE;
            // q, k, v rows are read as 16-byte vectors, out rows are written as 8-byte groups
            if (strides[i][j] % (i < 3 ? 8 : 4)) return RT_ERR_UNSUPPORTED;
        }
    if (d->causal != 0 && d->causal != 1) return RT_ERR_INVALID_ARG;
    if (!(d->scale == d->scale)) return RT_ERR_INVALID_ARG;
    return RT_OK;
}

rt_status rt_attention_workspace_bytes(const rt_attention_desc *desc, uint64_t *bytes) {
    if (!desc || !bytes) return RT_ERR_INVALID_ARG;
    const rt_status st = rt_attention_validate(desc);
    if (st != RT_OK) return st;
    *bytes = rt::attention_workspace_bytes(*desc);
    return RT_OK;
}

rt_status rt_attention_enqueue(rt_ctx *ctx, const rt_attention_desc *desc, const void *q, const void *k, const void *v,
                               const void *mask, void *out, void *workspace, uint64_t workspace_bytes, void *stream) {
    if (!ctx || !desc) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    const rt_status st = rt_attention_validate(desc);
    if (st != RT_OK) return fail(ctx, st, "attention: invalid descriptor");
    if (mask && desc->mask_dtype != RT_F32 && desc->mask_dtype != RT_F16)
        return fail(ctx, RT_ERR_DTYPE_MISMATCH, "attention: the mask is F32 or F16");
    if (mask && desc->mask_row_stride < desc->kv_len) return fail(ctx, RT_ERR_INVALID_SHAPE, "attention: mask rows overlap");
    if ((int64_t)desc->batch * desc->heads == 0 || desc->q_len == 0) return RT_OK; // empty output
    if (!q || !out || (desc->kv_len > 0 && (!k || !v))) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15u) || ((uintptr_t)out & 7u))
        return fail(ctx, RT_ERR_INVALID_ARG, "attention: q, k, v must be 16-byte aligned, out 8-byte aligned");
    if ((int64_t)desc->batch * desc->heads > 65535) return fail(ctx, RT_ERR_UNSUPPORTED, "attention: batch * heads above 65535");
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = rt::launch_attention(*desc, q, k, v, mask, out, workspace, workspace_bytes, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return fail(ctx, RT_ERR_UNSUPPORTED, "attention: a head's keys or values span 2^31 elements or more");
    if (e != hipSuccess) return hip_fail(ctx, "attention launch", e);
    return RT_OK;
    RT_GUARD_END(ctx)
}

// cache write of one tensor (cache2 == NULL, dst optional) or of a key / value pair (dst == NULL)
static rt_status cache_write(rt_ctx *ctx, int32_t dtype, void *cache, const void *src, void *cache2, const void *src2,
                             const int64_t *src_strides, void *dst, int32_t batch, int32_t heads, int32_t capacity, int32_t offset,
                             int32_t len, int32_t head_dim, bool pair, void *stream) {
    if (!ctx || !src_strides) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    if (dtype != RT_F32 && dtype != RT_F16) return fail(ctx, RT_ERR_DTYPE_MISMATCH, "cache: F32 or F16");
    if (batch < 0 || heads < 0 || capacity < 0 || offset < 0 || len < 0 || head_dim < 0)
        return fail(ctx, RT_ERR_INVALID_SHAPE, "cache: negative size");
    if (offset > capacity || (int64_t)offset + len > capacity)
        return fail(ctx, RT_ERR_INVALID_SHAPE, "cache: offset + len exceeds the capacity");
    const int64_t esz = dtype == RT_F32 ? 4 : 2, row_bytes = (int64_t)head_dim * esz;
    if (row_bytes % 16) return fail(ctx, RT_ERR_UNSUPPORTED, "cache: rows must be a multiple of 16 bytes");
    for (int i = 0; i < 3; i++)
        if (src_strides[i] < 0 || (src_strides[i] * esz) % 16) return fail(ctx, RT_ERR_UNSUPPORTED, "cache: source strides must keep rows 16-byte aligned");
    if ((int64_t)batch * heads == 0 || head_dim == 0 || (len == 0 && (!dst || offset == 0))) return RT_OK;
    if (!cache || (len && !src) || (pair && (!cache2 || (len && !src2)))) return fail(ctx, RT_ERR_INVALID_ARG, "null device pointer");
    if (((uintptr_t)cache | (uintptr_t)src | (uintptr_t)cache2 | (uintptr_t)src2 | (uintptr_t)dst) & 15u)
        return fail(ctx, RT_ERR_INVALID_ARG, "cache: buffers must be 16-byte aligned");
    if ((int64_t)batch * heads > 65535) return fail(ctx, RT_ERR_UNSUPPORTED, "cache: batch * heads above 65535");
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    hipError_t e = rt::launch_cache_write(cache, src, pair ? cache2 : nullptr, pair ? src2 : nullptr, dst,
                                          (int64_t)heads * capacity * row_bytes, (int64_t)capacity * row_bytes,
                                          src_strides[0] * esz, src_strides[1] * esz, src_strides[2] * esz, batch, heads,
                                          offset, len, row_bytes, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(ctx, "cache write launch", e);
    return RT_OK;
    RT_GUARD_END(ctx)
}

rt_status rt_cache_write_enqueue(rt_ctx *ctx, int32_t dtype, void *cache, const void *src, const int64_t *src_strides, void *dst,
                                 int32_t batch, int32_t heads, int32_t capacity, int32_t offset, int32_t len, int32_t head_dim,
                                 void *stream) {
    return cache_write(ctx, dtype, cache, src, nullptr, nullptr, src_strides, dst, batch, heads, capacity, offset, len, head_dim,
                       false, stream);
}

rt_status rt_cache_write_kv_enqueue(rt_ctx *ctx, int32_t dtype, void *k_cache, const void *k_src, void *v_cache, const void *v_src,
                                    const int64_t *src_strides, int32_t batch, int32_t heads, int32_t capacity, int32_t offset,
                                    int32_t len, int32_t head_dim, void *stream) {
    return cache_write(ctx, dtype, k_cache, k_src, v_cache, v_src, src_strides, nullptr, batch, heads, capacity, offset, len,
                       head_dim, true, stream);
}

rt_status rt_gguf_load_tensor(rt_ctx *ctx, const rt_gguf *g, const void *image, uint64_t size, uint64_t index,
                              int32_t dst_dtype, void *staging, void *dst, void *stream) {
    if (!ctx || !g || !image) return RT_ERR_INVALID_ARG;
    RT_GUARD_BEGIN
    DeviceGuard dg(ctx->dev.ordinal);
    if (!dg.ok) return fail(ctx, RT_ERR_NO_DEVICE, "hipSetDevice failed");
    std::string why;
    hipError_t herr = hipSuccess;
    const rt_status st = rt::gguf_load_tensor(g, image, size, index, dst_dtype, staging, dst, (hipStream_t)stream, why, herr);
    if (st != RT_OK) return st == RT_ERR_HIP ? hip_fail(ctx, why.c_str(), herr) : fail(ctx, st, why);
    return RT_OK;
    RT_GUARD_END(ctx)
}

} // extern "C"
