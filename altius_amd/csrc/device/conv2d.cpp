// Conv2d as the reference computes it (crates/session_interpreter/src/conv2d.rs:26-211): the input is
// unfolded into col[b][c][fy][fx][oh][ow], and for every image and group
//   out[b, g] (oc/g x oh*ow) = W[g] (oc/g x K) * col[b, g] (K x oh*ow) + bias,   K = c/g * kh * kw,
// which is one batched GEMM per group here (weights shared over the batch, bias as a column added
// through the GEMM's C0 operand).
#include "ctx.h"

namespace altius {

int launch_conv2d(DeviceCtx &ctx, float *out, const float *x, const float *w, const float *bias, float *col, size_t batch,
                  size_t c, size_t ih, size_t iw, size_t oc, size_t oh, size_t ow, size_t kh, size_t kw, size_t sh, size_t sw,
                  size_t dh, size_t dw, size_t pad_t, size_t pad_l, size_t group) {
    if (batch == 0 || oc == 0 || oh == 0 || ow == 0) return AHIP_OK;
    if (group == 0 || c % group || oc % group) return ctx.fail(AHIP_ERR_SHAPE, "conv2d: channels do not divide into the groups");
    if (!out || !x || !w || !col) return ctx.fail(AHIP_ERR_ARG, "conv2d: null pointer");
    int rc = launch_im2col(ctx, col, x, batch, c, ih, iw, oh, ow, kh, kw, sh, sw, dh, dw, pad_t, pad_l);
    if (rc) return rc;
    const size_t cg = c / group, ocg = oc / group, ohw = oh * ow, k = cg * kh * kw;
    for (size_t g = 0; g < group; g++) {
        rc = launch_gemm(ctx, out + g * ocg * ohw, w + g * ocg * k, col + g * k * ohw, bias ? bias + g * ocg : nullptr, batch, ocg,
                         ohw, k, 0, 0, k, ohw, ohw, 0, c * kh * kw * ohw, oc * ohw, 1, 0, 1.0f, 1.0f);
        if (rc) return rc;
    }
    return AHIP_OK;
}

}  // namespace altius
