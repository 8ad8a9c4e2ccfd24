// Where blocks run: which of the chip's XCDs (each with its own L2) gets block i of a launch.
//
// The split GEMM cuts the tiles of an XCD's partly filled last round along k and lets the slice that
// finishes last add the others' partial sums up straight out of that XCD's L2 (gemm_split.hip).  That is
// only correct if all slices of a tile really run on one XCD, which the kernel arranges by block id: all
// slices of a tile have the same block id mod 8, and consecutive block ids go to the eight XCDs in turn.
// Measured on the part: the turn does not start at XCD 0 -- a launch carries on where the previous launch
// of its queue stopped, so block 0 may land on any XCD -- but within a launch block i and block i + 8
// always share an XCD, also while other queues dispatch.  Nothing in the programming model promises that
// (another partition mode, another dispatcher), so a context measures it once when it is created: a
// launch of PROBE_BLOCKS blocks records each block's XCC id, and the in-kernel cut is used only if blocks
// 0..7 ran on eight different XCDs, every block i ran where block i mod 8 did, and the CU count is a
// multiple of eight.  The kernel checks the same thing per tile on every launch (the XCC ids of a tile's
// slices must agree) and raises the context's error flag otherwise.
#include <hip/hip_runtime.h>

#include <vector>

#include "ctx.h"

namespace altius {

namespace {

constexpr unsigned PROBE_BLOCKS = 4096;  // sixteen blocks per CU of a 256-CU part: several rounds of dispatch
constexpr unsigned PROBE_THREADS = 512;  // the split GEMM's block size

__global__ __launch_bounds__(PROBE_THREADS) void record_xcc(uint32_t *__restrict__ xcc_of_block) {
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    if (threadIdx.x == 0) xcc_of_block[blockIdx.x] = xcc & 0xfu;
}

}  // namespace

bool xcd_round_robin_holds(int cu_count, const uint32_t *xcc_of_block, size_t n_blocks) {
    if (cu_count < 8 || cu_count % 8 != 0) return false;
    if (!xcc_of_block || n_blocks < 16) return false;  // fewer than two rounds of eight say nothing
    uint32_t seen = 0;
    for (size_t i = 0; i < 8; i++) {
        if (xcc_of_block[i] >= 8) return false;  // not an XCD of an eight-XCD part (or a block that never ran)
        seen |= 1u << xcc_of_block[i];
    }
    if (seen != 0xffu) return false;  // blocks 0..7 did not reach eight different XCDs
    for (size_t i = 8; i < n_blocks; i++)
        if (xcc_of_block[i] != xcc_of_block[i % 8]) return false;
    return true;
}

int probe_xcd_placement(DeviceCtx &ctx, int cu_count) {
    ctx.xcd_round_robin = false;
    if (!ctx.scratch || ctx.scratch_floats < PROBE_BLOCKS) return ctx.fail(AHIP_ERR_ARG, "placement probe: no scratch buffer");
    uint32_t *dev = reinterpret_cast<uint32_t *>(ctx.scratch);
    // 0xff everywhere first: a block that did not run leaves a value no XCD has.
    int rc = ctx.check(hipMemsetAsync(dev, 0xff, PROBE_BLOCKS * sizeof(uint32_t), ctx.stream), "hipMemsetAsync(placement probe)");
    if (rc) return rc;
    hipLaunchKernelGGL(record_xcc, dim3(PROBE_BLOCKS), dim3(PROBE_THREADS), 0, ctx.stream, dev);
    rc = ctx.check(hipGetLastError(), "placement probe launch");
    if (rc) return rc;
    std::vector<uint32_t> host(PROBE_BLOCKS);
    rc = ctx.check(hipMemcpyAsync(host.data(), dev, PROBE_BLOCKS * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx.stream), "hipMemcpyAsync(placement probe)");
    if (rc) return rc;
    rc = ctx.check(hipStreamSynchronize(ctx.stream), "hipStreamSynchronize(placement probe)");
    if (rc) return rc;
    ctx.xcd_round_robin = xcd_round_robin_holds(cu_count, host.data(), host.size());
    return AHIP_OK;
}

}  // namespace altius
