// Device context and the launcher entry points shared by the C ABI and the
// session.  Everything here is host code; kernels live in the .hip files.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "../../../include/altius_hip.h"

namespace altius {

// One context = one device + one stream.  All work issued through a context is
// ordered on that stream.  A context is not thread-safe; use one per thread.
struct DeviceCtx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    // Partial results of two-stage reductions (device memory, owned).
    float *scratch = nullptr;
    size_t scratch_floats = 0;
    // Tensors of at least this many bytes are streamed with non-temporal accesses.
    size_t nt_threshold_bytes = (size_t)128 << 20;
    std::string last_error;

    bool streaming(size_t bytes) const { return bytes >= nt_threshold_bytes; }

    int fail(int code, const std::string &msg);
    int check(hipError_t e, const char *what);
};

// Sets the calling thread's "no context" error text (ahip_last_error(NULL)).
void set_global_error(const std::string &msg);
const char *global_error();

// Creates / tears down a context (stream + scratch buffer) on `device`.
int create_device_ctx(int device, hipStream_t stream, bool own_stream, DeviceCtx *ctx, std::string *error);
void destroy_device_ctx(DeviceCtx *ctx);

constexpr int MAX_RANK = 8;
constexpr size_t SCRATCH_FLOATS = 1u << 20;  // 4 MiB

int launch_binary(DeviceCtx &ctx, int op, float *out, const float *a, const float *b, int rank,
                  const int64_t *out_dims, const int64_t *a_strides, const int64_t *b_strides);
int launch_unary(DeviceCtx &ctx, int op, float *out, const float *in, size_t n, float alpha,
                 float beta);
int launch_softmax(DeviceCtx &ctx, float *out, const float *in, size_t rows, size_t len);
int launch_layernorm(DeviceCtx &ctx, float *out, const float *in, const float *gamma,
                     const float *beta, size_t rows, size_t len, float eps);
int launch_reduce(DeviceCtx &ctx, int kind, float *out, const float *in, size_t outer, size_t red,
                  size_t inner);

}  // namespace altius
