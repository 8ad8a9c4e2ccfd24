// Device context: error bookkeeping and creation/destruction.
#include "ctx.h"

#include <cstdlib>

namespace altius {

namespace {
thread_local std::string g_error;
}

void set_global_error(const std::string &msg) { g_error = msg; }
const char *global_error() { return g_error.c_str(); }

int DeviceCtx::fail(int code, const std::string &msg) {
    last_error = msg;
    return code;
}

int DeviceCtx::check(hipError_t e, const char *what) {
    if (e == hipSuccess) return AHIP_OK;
    last_error = std::string(what) + ": " + hipGetErrorString(e);
    return e == hipErrorOutOfMemory ? AHIP_ERR_OOM : AHIP_ERR_HIP;
}

int create_device_ctx(int device, hipStream_t stream, bool own_stream, DeviceCtx *ctx, std::string *error) {
    auto fail = [&](hipError_t e, const char *what) {
        if (error) *error = std::string(what) + ": " + hipGetErrorString(e);
        return e == hipErrorOutOfMemory ? AHIP_ERR_OOM : AHIP_ERR_HIP;
    };
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return fail(e, "hipGetDeviceCount");
    if (device < 0 || device >= n) {
        if (error) *error = "no such device: " + std::to_string(device);
        return AHIP_ERR_ARG;
    }
    e = hipSetDevice(device);
    if (e != hipSuccess) return fail(e, "hipSetDevice");
    ctx->device = device;
    // Only ahip_reduce_static needs the fixed array's address: without it that entry point reports the failure, and
    // everything else works.
    (void)reduce_static_setup(device);
    // AHIP_GEMM_SPLIT_K=0 keeps the bf16 GEMM from cutting an XCD's partly filled last round of tiles along k
    // (for measurements).
    if (const char *e = getenv("AHIP_GEMM_SPLIT_K")) ctx->gemm_split_k = atoi(e) != 0;
    // AHIP_STREAMING_THRESHOLD_MIB: the tensor size from which accesses are non-temporal (for measurements; see
    // ahip_set_streaming_threshold).
    if (const char *e = getenv("AHIP_STREAMING_THRESHOLD_MIB")) ctx->nt_threshold_bytes = (size_t)atol(e) << 20;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus >= 8) ctx->cus_per_xcd = cus / 8;
    if (own_stream) {
        // Default priority; non-blocking with respect to the legacy default stream.
        e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) return fail(e, "hipStreamCreate");
        ctx->owns_stream = true;
    } else {
        ctx->stream = stream;
        ctx->owns_stream = false;
    }
    void *scratch = nullptr;
    e = hipMalloc(&scratch, SCRATCH_FLOATS * sizeof(float));
    if (e != hipSuccess) {
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
        ctx->stream = nullptr;
        return fail(e, "hipMalloc(scratch)");
    }
    ctx->scratch = static_cast<float *>(scratch);
    ctx->scratch_floats = SCRATCH_FLOATS;
    void *flags = nullptr;
    e = hipMalloc(&flags, 256);
    if (e == hipSuccess) e = hipMemset(flags, 0, 256);
    if (e != hipSuccess) {
        if (flags) (void)hipFree(flags);
        (void)hipFree(scratch);
        ctx->scratch = nullptr;
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
        ctx->stream = nullptr;
        return fail(e, "hipMalloc(flags)");
    }
    ctx->flags = static_cast<int *>(flags);
    ctx->flags_armed = false;
    // Where do blocks run?  Decides whether the bf16 GEMM may combine the slices of a tile inside one XCD's L2.
    // A probe that cannot run leaves the answer at "not shown", which only switches that cut off.
    // On a stream of the library's own: a caller's stream may be capturing, or busy with work the probe's
    // synchronisation would wait for.
    hipStream_t given = ctx->stream, probe_stream = nullptr;
    if (!ctx->owns_stream && hipStreamCreateWithFlags(&probe_stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        ctx->xcd_round_robin = false;
        return AHIP_OK;
    }
    if (probe_stream) ctx->stream = probe_stream;
    if (probe_xcd_placement(*ctx, cus) != AHIP_OK) ctx->xcd_round_robin = false;
    ctx->stream = given;
    if (probe_stream) (void)hipStreamDestroy(probe_stream);
    return AHIP_OK;
}

int check_device_flags(DeviceCtx &ctx) {
    if (!ctx.flags_armed) return AHIP_OK;
    ctx.flags_armed = false;
    int raised[2] = {0, 0};
    int rc = ctx.check(hipMemcpy(raised, ctx.flags, sizeof(raised), hipMemcpyDeviceToHost), "hipMemcpy(flags)");
    if (rc) return rc;
    if (!raised[0] && !raised[1]) return AHIP_OK;
    rc = ctx.check(hipMemset(ctx.flags, 0, sizeof(raised)), "hipMemset(flags)");
    if (rc) return rc;
    if (raised[1]) {
        // The placement the probe measured did not hold for a launch: the product just computed is not to be
        // trusted, and the cut stays off for the rest of this context's life.
        ctx.xcd_round_robin = false;
        return ctx.fail(AHIP_ERR_HIP, "MatMul: the slices of a tile cut along k ran on different XCDs, so their partial sums could not be "
                                      "combined; the in-kernel cut is now switched off for this context, run the product again");
    }
    return ctx.fail(AHIP_ERR_ARG, "Gather: an index is outside the gathered axis");
}

void destroy_device_ctx(DeviceCtx *ctx) {
    if (hipSetDevice(ctx->device) != hipSuccess) return;
    (void)hipStreamSynchronize(ctx->stream);
    reduce_static_forget_stream(ctx->device, ctx->stream);
    gemm_release_all(*ctx);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    ctx->scratch = nullptr;
    if (ctx->flags) (void)hipFree(ctx->flags);
    ctx->flags = nullptr;
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    ctx->stream = nullptr;
}

}  // namespace altius
