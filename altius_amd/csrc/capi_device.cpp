// C ABI: device shim, host index math and operator entry points.
#include <hip/hip_runtime.h>

#include <cstring>
#include <new>
#include <string>
#include <unordered_map>

#include "core/fixed_dim.h"
#include "capi_guard.h"
#include "device/ctx.h"

using altius::DeviceCtx;
using altius::FixedDimensions;

struct ahip_ctx {
    DeviceCtx d;
};

namespace {

int global_fail(int code, const std::string &msg) {
    altius::set_global_error(msg);
    return code;
}

int global_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return AHIP_OK;
    altius::set_global_error(std::string(what) + ": " + hipGetErrorString(e));
    return e == hipErrorOutOfMemory ? AHIP_ERR_OOM : AHIP_ERR_HIP;
}

int create_ctx(int device, hipStream_t stream, bool own_stream, ahip_ctx **out) {
    if (!out) return global_fail(AHIP_ERR_ARG, "ahip_init: null output pointer");
    *out = nullptr;
    ahip_ctx *c = new (std::nothrow) ahip_ctx();
    if (!c) return global_fail(AHIP_ERR_OOM, "ahip_init: out of host memory");
    std::string err;
    const int rc = altius::create_device_ctx(device, stream, own_stream, &c->d, &err);
    if (rc) {
        delete c;
        return global_fail(rc, "ahip_init: " + err);
    }
    *out = c;
    return AHIP_OK;
}

}  // namespace

#define REQUIRE_CTX(ctx, name)                                                       \
    do {                                                                             \
        if (!(ctx)) return global_fail(AHIP_ERR_ARG, name ": null context");         \
        if (hipSetDevice((ctx)->d.device) != hipSuccess)                             \
            return (ctx)->d.fail(AHIP_ERR_HIP, name ": hipSetDevice failed");        \
    } while (0)

extern "C" {

int ahip_init(int device, ahip_ctx **ctx) { return create_ctx(device, nullptr, true, ctx); }

int ahip_init_on_stream(int device, void *hip_stream, ahip_ctx **ctx) try {
    return create_ctx(device, static_cast<hipStream_t>(hip_stream), false, ctx);
} catch (...) {
    return altius::caught_at_boundary("ahip_init_on_stream");
}

int ahip_destroy(ahip_ctx *ctx) try {
    if (!ctx) return AHIP_OK;
    altius::destroy_device_ctx(&ctx->d);
    delete ctx;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_destroy");
}

const char *ahip_last_error(ahip_ctx *ctx) { return ctx ? ctx->d.last_error.c_str() : altius::global_error(); }

int ahip_device_count(void) try {
    int n = 0;
    int rc = global_check(hipGetDeviceCount(&n), "hipGetDeviceCount");
    return rc ? -rc : n;
} catch (...) {
    return altius::caught_at_boundary("ahip_device_count");
}

int ahip_malloc(ahip_ctx *ctx, size_t bytes, void **dptr) try {
    REQUIRE_CTX(ctx, "ahip_malloc");
    if (!dptr) return ctx->d.fail(AHIP_ERR_ARG, "ahip_malloc: null output pointer");
    *dptr = nullptr;
    if (bytes == 0) return AHIP_OK;
    return ctx->d.check(hipMalloc(dptr, bytes), "hipMalloc");
} catch (...) {
    return altius::caught_at_boundary("ahip_malloc");
}

int ahip_free(ahip_ctx *ctx, void *dptr) try {
    REQUIRE_CTX(ctx, "ahip_free");
    if (!dptr) return AHIP_OK;
    return ctx->d.check(hipFree(dptr), "hipFree");
} catch (...) {
    return altius::caught_at_boundary("ahip_free");
}

int ahip_h2d_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_h2d_async");
    if (bytes == 0) return AHIP_OK;
    if (!dst || !src) return ctx->d.fail(AHIP_ERR_ARG, "ahip_h2d_async: null pointer");
    return ctx->d.check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->d.stream), "hipMemcpyAsync(H2D)");
} catch (...) {
    return altius::caught_at_boundary("ahip_h2d_async");
}

int ahip_d2h_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_d2h_async");
    if (bytes == 0) return AHIP_OK;
    if (!dst || !src) return ctx->d.fail(AHIP_ERR_ARG, "ahip_d2h_async: null pointer");
    return ctx->d.check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->d.stream), "hipMemcpyAsync(D2H)");
} catch (...) {
    return altius::caught_at_boundary("ahip_d2h_async");
}

int ahip_d2d_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_d2d_async");
    if (bytes == 0) return AHIP_OK;
    if (!dst || !src) return ctx->d.fail(AHIP_ERR_ARG, "ahip_d2d_async: null pointer");
    return ctx->d.check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->d.stream), "hipMemcpyAsync(D2D)");
} catch (...) {
    return altius::caught_at_boundary("ahip_d2d_async");
}

int ahip_memset_async(ahip_ctx *ctx, void *dst, int byte_value, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_memset_async");
    if (bytes == 0) return AHIP_OK;
    if (!dst) return ctx->d.fail(AHIP_ERR_ARG, "ahip_memset_async: null pointer");
    return ctx->d.check(hipMemsetAsync(dst, byte_value, bytes, ctx->d.stream), "hipMemsetAsync");
} catch (...) {
    return altius::caught_at_boundary("ahip_memset_async");
}

int ahip_sync(ahip_ctx *ctx) try {
    REQUIRE_CTX(ctx, "ahip_sync");
    const int rc = ctx->d.check(hipStreamSynchronize(ctx->d.stream), "hipStreamSynchronize");
    return rc ? rc : altius::check_device_flags(ctx->d);
} catch (...) {
    return altius::caught_at_boundary("ahip_sync");
}

int ahip_host_alloc(ahip_ctx *ctx, size_t bytes, void **hptr) try {
    REQUIRE_CTX(ctx, "ahip_host_alloc");
    if (!hptr) return ctx->d.fail(AHIP_ERR_ARG, "ahip_host_alloc: null output pointer");
    *hptr = nullptr;
    if (bytes == 0) return AHIP_OK;
    return ctx->d.check(hipHostMalloc(hptr, bytes, hipHostMallocDefault), "hipHostMalloc");
} catch (...) {
    return altius::caught_at_boundary("ahip_host_alloc");
}

int ahip_host_free(ahip_ctx *ctx, void *hptr) try {
    REQUIRE_CTX(ctx, "ahip_host_free");
    if (!hptr) return AHIP_OK;
    return ctx->d.check(hipHostFree(hptr), "hipHostFree");
} catch (...) {
    return altius::caught_at_boundary("ahip_host_free");
}

int ahip_event_create(ahip_ctx *ctx, void **event) try {
    REQUIRE_CTX(ctx, "ahip_event_create");
    if (!event) return ctx->d.fail(AHIP_ERR_ARG, "ahip_event_create: null output pointer");
    hipEvent_t e;
    int rc = ctx->d.check(hipEventCreate(&e), "hipEventCreate");
    if (rc) return rc;
    *event = e;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_event_create");
}

int ahip_event_record(ahip_ctx *ctx, void *event) try {
    REQUIRE_CTX(ctx, "ahip_event_record");
    if (!event) return ctx->d.fail(AHIP_ERR_ARG, "ahip_event_record: null event");
    return ctx->d.check(hipEventRecord(static_cast<hipEvent_t>(event), ctx->d.stream), "hipEventRecord");
} catch (...) {
    return altius::caught_at_boundary("ahip_event_record");
}

int ahip_event_synchronize(ahip_ctx *ctx, void *event) try {
    REQUIRE_CTX(ctx, "ahip_event_synchronize");
    if (!event) return ctx->d.fail(AHIP_ERR_ARG, "ahip_event_synchronize: null event");
    return ctx->d.check(hipEventSynchronize(static_cast<hipEvent_t>(event)), "hipEventSynchronize");
} catch (...) {
    return altius::caught_at_boundary("ahip_event_synchronize");
}

int ahip_event_elapsed_ms(ahip_ctx *ctx, void *start, void *stop, float *ms) try {
    REQUIRE_CTX(ctx, "ahip_event_elapsed_ms");
    if (!start || !stop || !ms) return ctx->d.fail(AHIP_ERR_ARG, "ahip_event_elapsed_ms: null argument");
    return ctx->d.check(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)),
                        "hipEventElapsedTime");
} catch (...) {
    return altius::caught_at_boundary("ahip_event_elapsed_ms");
}

int ahip_event_destroy(ahip_ctx *ctx, void *event) try {
    REQUIRE_CTX(ctx, "ahip_event_destroy");
    if (!event) return AHIP_OK;
    return ctx->d.check(hipEventDestroy(static_cast<hipEvent_t>(event)), "hipEventDestroy");
} catch (...) {
    return altius::caught_at_boundary("ahip_event_destroy");
}

// ---- code objects loaded at run time -----------------------------------------

struct ahip_module {
    hipModule_t mod = nullptr;
    int device = 0;
    std::unordered_map<std::string, hipFunction_t> functions;
};

int ahip_module_load(ahip_ctx *ctx, const void *image, size_t bytes, ahip_module **module) try {
    REQUIRE_CTX(ctx, "ahip_module_load");
    if (!module) return ctx->d.fail(AHIP_ERR_ARG, "ahip_module_load: null output pointer");
    *module = nullptr;
    if (!image || bytes < 8) return ctx->d.fail(AHIP_ERR_ARG, "ahip_module_load: empty image");
    const unsigned char *p = static_cast<const unsigned char *>(image);
    const bool elf = p[0] == 0x7f && p[1] == 'E' && p[2] == 'L' && p[3] == 'F';
    const bool bundle = bytes >= 24 && std::memcmp(p, "__CLANG_OFFLOAD_BUNDLE__", 24) == 0;
    if (!elf && !bundle)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_module_load: image is neither an ELF code object nor an offload bundle");
    ahip_module *m = new (std::nothrow) ahip_module();
    if (!m) return ctx->d.fail(AHIP_ERR_OOM, "ahip_module_load: out of host memory");
    m->device = ctx->d.device;
    // The runtime reads the image through the pointer only during this call.
    const int rc = ctx->d.check(hipModuleLoadData(&m->mod, image), "hipModuleLoadData");
    if (rc) {
        delete m;
        return rc;
    }
    *module = m;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_module_load");
}

int ahip_module_unload(ahip_ctx *ctx, ahip_module *module) try {
    REQUIRE_CTX(ctx, "ahip_module_unload");
    if (!module) return AHIP_OK;
    if (module->device != ctx->d.device)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_module_unload: module belongs to another device");
    // Kernels of the module may still be queued on the stream.
    int rc = ctx->d.check(hipStreamSynchronize(ctx->d.stream), "hipStreamSynchronize");
    const int rc2 = ctx->d.check(hipModuleUnload(module->mod), "hipModuleUnload");
    delete module;
    return rc ? rc : rc2;
} catch (...) {
    return altius::caught_at_boundary("ahip_module_unload");
}

int ahip_launch(ahip_ctx *ctx, ahip_module *module, const char *kernel, const uint32_t grid[3],
                const uint32_t block[3], uint32_t shared_bytes, void **args) try {
    REQUIRE_CTX(ctx, "ahip_launch");
    if (!module || !kernel || !grid || !block)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_launch: null module, kernel name, grid or block");
    if (module->device != ctx->d.device)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_launch: module belongs to another device");
    const uint64_t threads = (uint64_t)block[0] * block[1] * block[2];
    if (threads == 0 || threads > 1024 || block[0] > 1024 || block[1] > 1024 || block[2] > 1024)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_launch: a block holds 1 to 1024 threads");
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0 || grid[1] > 65535u || grid[2] > 65535u ||
        (uint64_t)grid[0] * block[0] > 0xffffffffull)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_launch: grid extent out of range");
    if (shared_bytes > 160u * 1024u)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_launch: more than 160 KiB of shared memory per block");
    hipFunction_t fn = nullptr;
    auto it = module->functions.find(kernel);
    if (it != module->functions.end()) {
        fn = it->second;
    } else {
        const hipError_t e = hipModuleGetFunction(&fn, module->mod, kernel);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return ctx->d.fail(AHIP_ERR_ARG, std::string("ahip_launch: no kernel named '") + kernel +
                                                 "' in the module (" + hipGetErrorString(e) + ")");
        }
        module->functions.emplace(kernel, fn);
    }
    return ctx->d.check(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                              shared_bytes, ctx->d.stream, args, nullptr),
                        "hipModuleLaunchKernel");
} catch (...) {
    return altius::caught_at_boundary("ahip_launch");
}

// ---- host index math -------------------------------------------------------

int ahip_broadcast_shape(int a_rank, const int64_t *a_dims, int b_rank, const int64_t *b_dims, int *out_rank,
                         int64_t *out_dims) try {
    if (a_rank < 0 || b_rank < 0 || (a_rank && !a_dims) || (b_rank && !b_dims) || !out_rank || !out_dims)
        return global_fail(AHIP_ERR_ARG, "ahip_broadcast_shape: invalid argument");
    FixedDimensions a = FixedDimensions::from_i64(a_dims, (size_t)a_rank);
    FixedDimensions b = FixedDimensions::from_i64(b_dims, (size_t)b_rank);
    auto r = a.broadcast(b);
    if (!r)
        return global_fail(AHIP_ERR_SHAPE, "cannot broadcast " + a.to_string() + " with " + b.to_string());
    *out_rank = (int)r->len();
    for (size_t i = 0; i < r->len(); i++) out_dims[i] = (int64_t)(*r)[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_broadcast_shape");
}

int ahip_strides_for_broadcasting(int from_rank, const int64_t *from_dims, int to_rank, const int64_t *to_dims,
                                  int64_t *out_strides) try {
    if (from_rank < 0 || to_rank < 0 || (from_rank && !from_dims) || (to_rank && (!to_dims || !out_strides)))
        return global_fail(AHIP_ERR_ARG, "ahip_strides_for_broadcasting: invalid argument");
    FixedDimensions from = FixedDimensions::from_i64(from_dims, (size_t)from_rank);
    FixedDimensions to = FixedDimensions::from_i64(to_dims, (size_t)to_rank);
    auto r = from.strides_for_broadcasting_to(to);
    if (!r)
        return global_fail(AHIP_ERR_SHAPE, "cannot broadcast " + from.to_string() + " to " + to.to_string());
    for (size_t i = 0; i < r->len(); i++) out_strides[i] = (int64_t)(*r)[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_strides_for_broadcasting");
}

// ---- operators --------------------------------------------------------------

int ahip_binary(ahip_ctx *ctx, int op, float *out, const float *a, const float *b, int rank,
                const int64_t *out_dims, const int64_t *a_strides, const int64_t *b_strides) try {
    REQUIRE_CTX(ctx, "ahip_binary");
    return altius::launch_binary(ctx->d, op, out, a, b, rank, out_dims, a_strides, b_strides);
} catch (...) {
    return altius::caught_at_boundary("ahip_binary");
}

int ahip_unary(ahip_ctx *ctx, int op, float *out, const float *in, size_t n, float alpha, float beta) try {
    REQUIRE_CTX(ctx, "ahip_unary");
    return altius::launch_unary(ctx->d, op, out, in, n, alpha, beta);
} catch (...) {
    return altius::caught_at_boundary("ahip_unary");
}

int ahip_fused_elemwise(ahip_ctx *ctx, float *out, int rank, const int64_t *out_dims, int n_inputs, const float *const *inputs,
                        const int64_t *const *input_strides, int n_steps, const ahip_fused_step *steps) try {
    REQUIRE_CTX(ctx, "ahip_fused_elemwise");
    return altius::launch_fused_elemwise(ctx->d, out, rank, out_dims, n_inputs, inputs, input_strides, n_steps, steps);
} catch (...) {
    return altius::caught_at_boundary("ahip_fused_elemwise");
}

int ahip_fused_use_compiled_chains(ahip_ctx *ctx, int enable) try {
    REQUIRE_CTX(ctx, "ahip_fused_use_compiled_chains");
    ctx->d.fused_static_chains = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_fused_use_compiled_chains");
}

int ahip_softmax_lastaxis(ahip_ctx *ctx, float *out, const float *in, size_t rows, size_t len) try {
    REQUIRE_CTX(ctx, "ahip_softmax_lastaxis");
    return altius::launch_softmax(ctx->d, out, in, rows, len);
} catch (...) {
    return altius::caught_at_boundary("ahip_softmax_lastaxis");
}

int ahip_softmax_lastaxis_prologue(ahip_ctx *ctx, float *out, const float *in, size_t rows, size_t len, int scale_op, float scale,
                                   const float *mask, size_t rows_per_mask) try {
    REQUIRE_CTX(ctx, "ahip_softmax_lastaxis_prologue");
    return altius::launch_softmax_prologue(ctx->d, out, in, rows, len, scale_op, scale, mask, rows_per_mask);
} catch (...) {
    return altius::caught_at_boundary("ahip_softmax_lastaxis_prologue");
}

int ahip_layernorm_lastaxis(ahip_ctx *ctx, float *out, const float *in, const float *gamma, const float *beta,
                            size_t rows, size_t len, float eps) try {
    REQUIRE_CTX(ctx, "ahip_layernorm_lastaxis");
    return altius::launch_layernorm(ctx->d, out, in, gamma, beta, rows, len, eps);
} catch (...) {
    return altius::caught_at_boundary("ahip_layernorm_lastaxis");
}

int ahip_reduce(ahip_ctx *ctx, int kind, float *out, const float *in, size_t outer, size_t reduce, size_t inner) try {
    REQUIRE_CTX(ctx, "ahip_reduce");
    return altius::launch_reduce(ctx->d, kind, out, in, outer, reduce, inner);
} catch (...) {
    return altius::caught_at_boundary("ahip_reduce");
}

int ahip_set_streaming_threshold(ahip_ctx *ctx, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_set_streaming_threshold");
    ctx->d.nt_threshold_bytes = bytes;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_set_streaming_threshold");
}

int ahip_set_load_streaming_threshold(ahip_ctx *ctx, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_set_load_streaming_threshold");
    ctx->d.nt_load_threshold_bytes = bytes;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_set_load_streaming_threshold");
}

int ahip_xcd_round_robin_holds(int cu_count, const uint32_t *xcc_of_block, size_t n_blocks) try {
    return altius::xcd_round_robin_holds(cu_count, xcc_of_block, n_blocks) ? 1 : 0;
} catch (...) {
    return altius::caught_at_boundary("ahip_xcd_round_robin_holds");
}

int ahip_gemm_in_kernel_k_cut(ahip_ctx *ctx, int *placement_shown, int *enabled) try {
    REQUIRE_CTX(ctx, "ahip_gemm_in_kernel_k_cut");
    if (placement_shown) *placement_shown = ctx->d.xcd_round_robin ? 1 : 0;
    if (enabled) *enabled = (ctx->d.gemm_in_kernel_k_cut && ctx->d.gemm_split_k) ? 1 : 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_in_kernel_k_cut");
}

int ahip_gemm_set_in_kernel_k_cut(ahip_ctx *ctx, int enable) try {
    REQUIRE_CTX(ctx, "ahip_gemm_set_in_kernel_k_cut");
    ctx->d.gemm_in_kernel_k_cut = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_set_in_kernel_k_cut");
}

int ahip_reduce_static(ahip_ctx *ctx, int kind, float *out, const float *in, size_t outer, size_t reduce, size_t inner) try {
    REQUIRE_CTX(ctx, "ahip_reduce_static");
    return altius::launch_reduce_static(ctx->d, kind, out, in, outer, reduce, inner);
} catch (...) {
    return altius::caught_at_boundary("ahip_reduce_static");
}

size_t ahip_reduce_static_capacity(void) { return altius::reduce_static_capacity_floats(); }

int ahip_copy_strided(ahip_ctx *ctx, void *out, const void *in, int elem_size, int rank, const int64_t *dims,
                      const int64_t *out_strides, const int64_t *in_strides) try {
    REQUIRE_CTX(ctx, "ahip_copy_strided");
    if (rank > 0 && (!dims || !out_strides || !in_strides)) return ctx->d.fail(AHIP_ERR_ARG, "ahip_copy_strided: null shape");
    return altius::launch_copy_strided(ctx->d, out, in, elem_size, rank, dims, out_strides, in_strides);
} catch (...) {
    return altius::caught_at_boundary("ahip_copy_strided");
}

int ahip_transpose(ahip_ctx *ctx, void *out, const void *in, int elem_size, int rank, const int64_t *in_dims,
                   const int64_t *perm) try {
    REQUIRE_CTX(ctx, "ahip_transpose");
    if (rank > 0 && (!in_dims || !perm)) return ctx->d.fail(AHIP_ERR_ARG, "ahip_transpose: null shape");
    return altius::launch_transpose(ctx->d, out, in, elem_size, rank, in_dims, perm);
} catch (...) {
    return altius::caught_at_boundary("ahip_transpose");
}

int ahip_gather(ahip_ctx *ctx, void *out, const void *data, const void *indices, int index_size, int elem_size,
                size_t outer, size_t axis_len, size_t n_indices, size_t inner) try {
    REQUIRE_CTX(ctx, "ahip_gather");
    ctx->d.flags_armed = true;
    return altius::launch_gather(ctx->d, out, data, indices, index_size, elem_size, outer, axis_len, n_indices, inner,
                                 ctx->d.flags);
} catch (...) {
    return altius::caught_at_boundary("ahip_gather");
}

int ahip_where(ahip_ctx *ctx, void *out, const void *cond, const void *x, const void *y, int elem_size, int rank,
               const int64_t *dims, const int64_t *cond_strides, const int64_t *x_strides, const int64_t *y_strides) try {
    REQUIRE_CTX(ctx, "ahip_where");
    if (rank > 0 && (!dims || !cond_strides || !x_strides || !y_strides)) return ctx->d.fail(AHIP_ERR_ARG, "ahip_where: null shape");
    return altius::launch_where(ctx->d, out, cond, x, y, elem_size, rank, dims, cond_strides, x_strides, y_strides);
} catch (...) {
    return altius::caught_at_boundary("ahip_where");
}

int ahip_greater(ahip_ctx *ctx, void *out, const float *a, const float *b, int rank, const int64_t *dims,
                 const int64_t *a_strides, const int64_t *b_strides) try {
    REQUIRE_CTX(ctx, "ahip_greater");
    if (rank > 0 && (!dims || !a_strides || !b_strides)) return ctx->d.fail(AHIP_ERR_ARG, "ahip_greater: null shape");
    return altius::launch_greater(ctx->d, static_cast<uint8_t *>(out), a, b, rank, dims, a_strides, b_strides);
} catch (...) {
    return altius::caught_at_boundary("ahip_greater");
}

int ahip_cast(ahip_ctx *ctx, void *out, const void *in, int from_elem_type, int to_elem_type, size_t n) try {
    REQUIRE_CTX(ctx, "ahip_cast");
    return altius::launch_cast(ctx->d, out, in, from_elem_type, to_elem_type, n);
} catch (...) {
    return altius::caught_at_boundary("ahip_cast");
}

int ahip_batchnorm(ahip_ctx *ctx, float *out, const float *x, const float *scale, const float *bias, const float *mean,
                   const float *var, size_t n, size_t c, size_t hw, float epsilon) try {
    REQUIRE_CTX(ctx, "ahip_batchnorm");
    return altius::launch_batchnorm(ctx->d, out, x, scale, bias, mean, var, n, c, hw, epsilon);
} catch (...) {
    return altius::caught_at_boundary("ahip_batchnorm");
}

int ahip_gemm(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t batch, size_t m, size_t n,
              size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t a_batch_stride,
              size_t b_batch_stride, size_t c_batch_stride, size_t c0_row_stride, size_t c0_col_stride, float alpha,
              float beta) try {
    REQUIRE_CTX(ctx, "ahip_gemm");
    return altius::launch_gemm(ctx->d, c, a, b, c0, batch, m, n, k, trans_a, trans_b, lda, ldb, ldc, a_batch_stride,
                               b_batch_stride, c_batch_stride, c0_row_stride, c0_col_stride, alpha, beta);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm");
}

int ahip_gemm_batch2(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t batch_outer,
                     size_t batch_inner, size_t m, size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb,
                     size_t ldc, const size_t a_batch_strides[2], const size_t b_batch_strides[2],
                     const size_t c_batch_strides[2], size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta) try {
    REQUIRE_CTX(ctx, "ahip_gemm_batch2");
    if (!a_batch_strides || !b_batch_strides || !c_batch_strides) return ctx->d.fail(AHIP_ERR_ARG, "ahip_gemm_batch2: null strides");
    if (batch_inner == 0) return ctx->d.fail(AHIP_ERR_ARG, "ahip_gemm_batch2: batch_inner is 0");
    return altius::launch_gemm_batch2(ctx->d, c, a, b, c0, batch_outer, batch_inner, m, n, k, trans_a, trans_b, lda, ldb, ldc,
                                      a_batch_strides, b_batch_strides, c_batch_strides, c0_row_stride, c0_col_stride, alpha, beta);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_batch2");
}

int ahip_gemm_activated(ahip_ctx *ctx, int a_op, float *c, const float *a, const float *b, const float *c0, size_t m,
                        size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc,
                        size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta) try {
    REQUIRE_CTX(ctx, "ahip_gemm_activated");
    if (a_op != AHIP_GELU && a_op != AHIP_RELU) return ctx->d.fail(AHIP_ERR_ARG, "ahip_gemm_activated: a_op must be AHIP_GELU or AHIP_RELU");
    if (!altius::gemm_takes_split(ctx->d, m, n, k))
        return ctx->d.fail(AHIP_ERR_UNSUPPORTED, "ahip_gemm_activated: this product does not take the bf16 route");
    return altius::launch_gemm_split(ctx->d, c, a, b, c0, m, n, k, trans_a, trans_b, lda, ldb, ldc, c0_row_stride, c0_col_stride,
                                     alpha, beta, a_op);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_activated");
}

int ahip_gemm_post(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t m, size_t n, size_t k,
                   int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t c0_row_stride, size_t c0_col_stride,
                   float alpha, float beta, int act, const float *residual) try {
    REQUIRE_CTX(ctx, "ahip_gemm_post");
    if (act != 0 && act != AHIP_GELU && act != AHIP_RELU) return ctx->d.fail(AHIP_ERR_ARG, "ahip_gemm_post: act must be 0, AHIP_GELU or AHIP_RELU");
    altius::GemmPost post;
    post.act = act;
    post.residual = residual;
    const size_t none[2] = {0, 0};
    return altius::launch_gemm_batch2(ctx->d, c, a, b, c0, 1, 1, m, n, k, trans_a, trans_b, lda, ldb, ldc, none, none, none, c0_row_stride,
                                      c0_col_stride, alpha, beta, &post);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_post");
}

int ahip_attention(ahip_ctx *ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer,
                   size_t batch_inner, size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo,
                   const size_t q_batch_strides[2], const size_t k_batch_strides[2], const size_t v_batch_strides[2],
                   const size_t o_batch_strides[2], int scale_op, float scale, const float *mask, size_t mask_outer_stride) try {
    REQUIRE_CTX(ctx, "ahip_attention");
    if (!q_batch_strides || !k_batch_strides || !v_batch_strides || !o_batch_strides)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_attention: null strides");
    if (batch_inner == 0) return ctx->d.fail(AHIP_ERR_ARG, "ahip_attention: batch_inner is 0");
    return altius::launch_attention(ctx->d, o, q, k, v, batch_outer, batch_inner, tq, tk, d, ldq, ldk, ldv, ldo, q_batch_strides,
                                    k_batch_strides, v_batch_strides, o_batch_strides, scale_op, scale, mask, mask_outer_stride);
} catch (...) {
    return altius::caught_at_boundary("ahip_attention");
}

int ahip_gemm_set_algorithm(ahip_ctx *ctx, int algorithm) try {
    REQUIRE_CTX(ctx, "ahip_gemm_set_algorithm");
    if (algorithm != AHIP_GEMM_AUTO && algorithm != AHIP_GEMM_FP32 && algorithm != AHIP_GEMM_BF16X3)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_gemm_set_algorithm: unknown algorithm");
    ctx->d.gemm_algorithm = algorithm;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_set_algorithm");
}

int ahip_gemm_register_constant(ahip_ctx *ctx, const void *ptr, size_t bytes) try {
    REQUIRE_CTX(ctx, "ahip_gemm_register_constant");
    return altius::gemm_register_constant(ctx->d, ptr, bytes);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_register_constant");
}

int ahip_gemm_unregister_constant(ahip_ctx *ctx, const void *ptr) try {
    REQUIRE_CTX(ctx, "ahip_gemm_unregister_constant");
    return altius::gemm_unregister_constant(ctx->d, ptr);
} catch (...) {
    return altius::caught_at_boundary("ahip_gemm_unregister_constant");
}

int ahip_conv2d(ahip_ctx *ctx, float *out, const float *x, const float *w, const float *bias, float *col, size_t batch,
                size_t c, size_t ih, size_t iw, size_t oc, size_t oh, size_t ow, size_t kh, size_t kw, size_t stride_h,
                size_t stride_w, size_t dilation_h, size_t dilation_w, size_t pad_top, size_t pad_left, size_t group) try {
    REQUIRE_CTX(ctx, "ahip_conv2d");
    if (!kh || !kw || !stride_h || !stride_w || !dilation_h || !dilation_w)
        return ctx->d.fail(AHIP_ERR_ARG, "ahip_conv2d: kernel, stride and dilation must be positive");
    return altius::launch_conv2d(ctx->d, out, x, w, bias, col, batch, c, ih, iw, oc, oh, ow, kh, kw, stride_h, stride_w,
                                 dilation_h, dilation_w, pad_top, pad_left, group);
} catch (...) {
    return altius::caught_at_boundary("ahip_conv2d");
}

int ahip_maxpool(ahip_ctx *ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                 size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_top, size_t pad_left) try {
    REQUIRE_CTX(ctx, "ahip_maxpool");
    if (!kh || !kw || !stride_h || !stride_w) return ctx->d.fail(AHIP_ERR_ARG, "ahip_maxpool: kernel and stride must be positive");
    return altius::launch_maxpool(ctx->d, out, x, planes, ih, iw, oh, ow, kh, kw, stride_h, stride_w, pad_top, pad_left);
} catch (...) {
    return altius::caught_at_boundary("ahip_maxpool");
}

int ahip_resize(ahip_ctx *ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                int nearest) try {
    REQUIRE_CTX(ctx, "ahip_resize");
    return altius::launch_resize(ctx->d, out, x, planes, ih, iw, oh, ow, nearest);
} catch (...) {
    return altius::caught_at_boundary("ahip_resize");
}

}  // extern "C"
