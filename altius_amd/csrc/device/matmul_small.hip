// Many small fp32 products at once: attention's Q K^T ([197, 64] x [64, 197] per head) and P V
// ([197, 197] x [197, 64]) of a session that runs the three operators apart, as the reference does
// (compute_mat_mul, crates/session_interpreter/src/session.rs:621-684, one sgemm per batch entry).
//
// The 128 x 128 tiles of matmul.hip fit such matrices badly: four tiles per head of which 59 % is
// padding, every operand fetched twice.  Here one block takes one whole matrix product, cut into
// 16 x 16 tiles of v_mfma_f32_16x16x4_f32 (197 rows pad to 208, where 32 x 32 tiles pad to 224):
// wavefront w owns rows 16 w .. 16 w + 15 of C, thirteen wavefronts for 197 rows.
//
// The instruction adds four values of k per step, one from each quarter of the wavefront (lane / 16),
// and a sum does not care which four: both kernels hand the quarters the values of k that make their
// loads cheap, the same way for A and B and whichever way round B is stored, so that a product and the
// same product through a view of its second operand add the same numbers in the same order.
//
//   k <= 64 (Q K^T), gemm_small_k64: quarter q takes k = 16 q .. 16 q + 15.  A lane's 16 values of A lie
//     next to each other in memory and go from there to registers; all of B goes through LDS once per
//     block, stored the way it lies in memory, and every wavefront meets its column tiles one after the
//     other and stores a finished 16 x 16 tile of C per column tile.
//   n <= 64 (P V), gemm_small_n64: up to four column tiles, whose accumulators stay in registers while k
//     goes by in chunks of 32; in a chunk step s gives quarter q the value k = 4 s + q.  Per chunk a
//     wavefront stages its own rows of A (lanes along k, so that its loads are whole runs of a row) and
//     the block stages the chunk's part of B.
// C = A B only (no alpha, beta or third operand), A with unit stride along k; B either way round.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.h"
#include "ctx.h"

namespace altius {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;
constexpr int TILE = 16;        // rows / columns of an MFMA tile
constexpr int CHUNK = 64;       // values of k in a chunk: 16 steps of 4
constexpr int STEPS = CHUNK / 4;
constexpr int MAX_WAVES = 16;   // wavefronts per block: up to 256 rows of C
constexpr int MIN_WAVES = 4;    // at least four, so that the staging of B is shared by enough threads
constexpr int N64_CHUNK = 32;       // gemm_small_n64 takes k 32 at a time: two groups of four steps
constexpr int N64_K_PITCH = N64_CHUNK + 4;
constexpr int J_PITCH_N64 = 64 + 16; // floats per LDS row of a chunk of B stored [k][column], columns <= 64: quarters
                                     // q and q + 1 of a wavefront land on different halves of the banks

struct SmallGemm {
    const float *a, *b;
    float *c;
    uint32_t m, n, k;
    uint32_t lda, ldb, ldc;  // A(i, kk) = a[i * lda + kk]; B(kk, j) = b[j * ldb + kk] (k contiguous) or b[kk * ldb + j]
    uint64_t a_bs, b_bs, c_bs, a_bs2, b_bs2, c_bs2;
    uint32_t batch_inner;
    uint32_t batch;  // gemm_small_k64: heads
};

__device__ __forceinline__ void batch_offsets(const SmallGemm &g, const float *&a, const float *&b, float *&c) {
    const uint32_t z = blockIdx.x, zo = z / g.batch_inner, zi = z - zo * g.batch_inner;
    a = g.a + zo * g.a_bs + zi * g.a_bs2;
    b = g.b + zo * g.b_bs + zi * g.b_bs2;
    c = g.c + zo * g.c_bs + zi * g.c_bs2;
}

// The tiles are computed transposed (B's fragment as the instruction's first operand), so that a lane's four results
// lie next to each other in a row of C: element r of a lane's accumulator is C(row0 + lane % 16, col0 + 4 (lane / 16) + r).
__device__ __forceinline__ void store_tile(const floatx4 &acc, uint32_t m, uint32_t n, uint32_t ldc, float *c, uint32_t row0, uint32_t col0, uint32_t lane) {
    const uint32_t row = row0 + (lane & 15), col = col0 + 4 * (lane >> 4);
    if (row >= m) return;
    float *p = c + (size_t)row * ldc + col;
    if (col + 3 < n) {
        *reinterpret_cast<floatx4 *>(p) = acc;  // 16 bytes at a 4-byte boundary: global stores take that
        return;
    }
#pragma unroll
    for (int r = 0; r < 4; r++)
        if (col + r < n) p[r] = acc[r];
}

// k <= 64, m and n <= 208.  One block of 16 wavefronts per compute unit walks the heads blockIdx.x, blockIdx.x + gridDim.x, ...
//
// LDS (160 KB): all of A as [208][64] and all of B, [208][64] when B's k axis is contiguous (both with the 16-byte pieces of a
// row exchanged by piece ^= row % 16, which spreads a column of pieces over the banks without padding) or [64][209] when
// B's columns are.
//
// Twelve wavefronts multiply (three per SIMD) and four fetch (one per SIMD).  B is in LDS twice: while the multipliers
// read one copy the fetchers fill the other with the next head's; the next head's A waits in the fetchers' registers (52
// per lane) and is written between two barriers when the multipliers are done.  The two kinds of work are kept in different wavefronts because the hardware
// counts a wavefront's loads and stores in one counter: a wavefront that waits for a load it issued before storing results
// waits for the stores too, and the head's last stores take several microseconds to drain.
//
// A multiplier sweeps a row of tiles of C from left to right, so that the 64-byte pieces it stores complete each other's
// cache lines while those are still on their way out (pieces that meet a half-written line much later cost twice the
// time), and the wavefronts keep to rows of their own where the shape allows: 197 rows are twelve rows of tiles, one
// per multiplier, and a thirteenth of five rows whose tiles are dealt out one by one (14 or 15 tiles per wavefront).
constexpr int PB_WAVES = 16;
constexpr int FETCHERS = 4, MULTIPLIERS = PB_WAVES - FETCHERS;
constexpr int MAX_MN = 208;                                  // rows of A and columns of B
constexpr int J_PITCH = MAX_MN + 1;                          // floats per LDS row of B stored [k][column]
constexpr int VEC_PIECES = MAX_MN * (CHUNK / 4) / (FETCHERS * WAVE);   // float4s per fetching lane and operand: 13
constexpr int PIECES = MAX_MN * CHUNK / (FETCHERS * WAVE);   // single values per fetching lane and operand: 52

// The float offset of k (a multiple of 4 for float4s) in row `row` of an operand stored [row][64] with exchanged pieces.
__device__ __forceinline__ uint32_t swizzled(uint32_t row, uint32_t k) { return row * CHUNK + ((((k >> 2) ^ row) & 15) << 2) + (k & 3); }

// The fetchers address an operand of a head as a buffer of its own: a thread's pieces differ by a multiple of the row
// stride that is the same for all threads (the instruction's scalar offset), so that one vector register of offsets
// serves them all, and pieces past the operand's last value read as zero without a test.
typedef float f32x4_raw __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_raw __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t operand_buffer(const float *p, uint32_t floats) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0, (int)(floats * 4u), 0x00020000);  // raw buffer of 32-bit words
}

// Pieces FIRST .. FIRST + COUNT - 1 of a [rows][k <= 64] operand -> registers of the 256 fetching threads (ftid).  A
// thread's pieces are 16 (float4s) or 4 (single values) rows apart at the same k; k past `k` reads as zero.
template <int FIRST, int COUNT>
__device__ __forceinline__ void load_rows(float4 (&v)[COUNT], __amdgpu_buffer_rsrc_t src, uint32_t ld, uint32_t k, uint32_t ftid) {
    const uint32_t q = ftid & 15, offset = ((ftid >> 4) * ld + 4 * q) * 4;
    const bool in = 4 * q < k;
#pragma unroll
    for (int u = 0; u < COUNT; u++) {
        const f32x4_raw f = __builtin_bit_cast(f32x4_raw, __builtin_amdgcn_raw_buffer_load_b128(src, offset, 16 * (FIRST + u) * ld * 4, 0));
        v[u] = in ? make_float4(f.x, f.y, f.z, f.w) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}
template <int FIRST, int COUNT>
__device__ __forceinline__ void load_rows(float (&v)[COUNT], __amdgpu_buffer_rsrc_t src, uint32_t ld, uint32_t k, uint32_t ftid) {
    const uint32_t kk = ftid & 63, offset = ((ftid >> 6) * ld + kk) * 4;
    const bool in = kk < k;
#pragma unroll
    for (int u = 0; u < COUNT; u++) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(src, offset, 4 * (FIRST + u) * ld * 4, 0));
        v[u] = in ? f : 0.0f;
    }
}
// ... and from there into LDS, [row][64] with exchanged pieces.
template <int FIRST, int COUNT>
__device__ __forceinline__ void write_rows(const float4 (&v)[COUNT], float *dst, uint32_t ftid) {
#pragma unroll
    for (int u = 0; u < COUNT; u++) *reinterpret_cast<float4 *>(dst + swizzled((ftid >> 4) + 16 * (FIRST + u), 4 * (ftid & 15))) = v[u];
}
template <int FIRST, int COUNT>
__device__ __forceinline__ void write_rows(const float (&v)[COUNT], float *dst, uint32_t ftid) {
#pragma unroll
    for (int u = 0; u < COUNT; u++) dst[swizzled((ftid >> 6) + 4 * (FIRST + u), ftid & 63)] = v[u];
}
// A [k <= 64][columns <= 208] operand: thread ftid < 208 takes column ftid of rows FIRST .. FIRST + COUNT - 1.
template <int FIRST, int COUNT>
__device__ __forceinline__ void load_columns(float (&v)[COUNT], __amdgpu_buffer_rsrc_t src, uint32_t ld, uint32_t cols, uint32_t ftid) {
    const bool in = ftid < cols;
#pragma unroll
    for (int u = 0; u < COUNT; u++) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(src, ftid * 4, (FIRST + u) * ld * 4, 0));
        v[u] = in ? f : 0.0f;
    }
}
template <int FIRST, int COUNT>
__device__ __forceinline__ void write_columns(const float (&v)[COUNT], float *dst, uint32_t ftid) {
    if (ftid >= MAX_MN) return;
#pragma unroll
    for (int u = 0; u < COUNT; u++) dst[(FIRST + u) * J_PITCH + ftid] = v[u];
}
// One operand of a head, global memory -> LDS, in two rounds of loads that are all asked for before the first is
// written (the rounds of the float4 kind hold 7 and 6 pieces, of the others 26 and 26 or 32 and 32).  `extent` is the
// operand's number of rows (ROWS) or columns.
template <bool ROWS, bool VEC>
__device__ __forceinline__ void copy_operand(float *dst, const float *src, uint32_t ld, uint32_t extent, uint32_t k, uint32_t ftid) {
    if constexpr (ROWS && VEC) {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (extent - 1) * ld + k);
        constexpr int H = (VEC_PIECES + 1) / 2;
        float4 v0[H], v1[VEC_PIECES - H];
        load_rows<0, H>(v0, buf, ld, k, ftid);
        write_rows<0, H>(v0, dst, ftid);
        load_rows<H, VEC_PIECES - H>(v1, buf, ld, k, ftid);
        write_rows<H, VEC_PIECES - H>(v1, dst, ftid);
    } else if constexpr (ROWS) {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (extent - 1) * ld + k);
        constexpr int H = PIECES / 2;
        float v0[H], v1[PIECES - H];
        load_rows<0, H>(v0, buf, ld, k, ftid);
        write_rows<0, H>(v0, dst, ftid);
        load_rows<H, PIECES - H>(v1, buf, ld, k, ftid);
        write_rows<H, PIECES - H>(v1, dst, ftid);
    } else {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (k - 1) * ld + extent);
        constexpr int H = CHUNK / 2;
        float v0[H], v1[CHUNK - H];
        load_columns<0, H>(v0, buf, ld, extent, ftid);
        write_columns<0, H>(v0, dst, ftid);
        load_columns<H, CHUNK - H>(v1, buf, ld, extent, ftid);
        write_columns<H, CHUNK - H>(v1, dst, ftid);
    }
}

template <bool B_K_CONTIGUOUS, bool A_VEC, bool B_VEC>
__global__ __launch_bounds__(PB_WAVES * WAVE) void gemm_small_k64(SmallGemm args) {
    extern __shared__ __align__(16) float lds[];
    const uint32_t tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid >> 6;
    constexpr uint32_t b_floats = B_K_CONTIGUOUS ? MAX_MN * CHUNK : CHUNK * J_PITCH;  // B is there twice, for this head and the next
    float *lds_a = lds, *lds_b = lds + MAX_MN * CHUNK;
    const uint32_t batch = args.batch, batch_inner = args.batch_inner;
    const uint32_t head0 = blockIdx.x, head_step = gridDim.x;  // the grid has at most as many blocks as there are heads

    if (wave >= MULTIPLIERS) {
        // ---- a fetching wavefront: B goes straight to the buffer the multipliers are not reading, A waits in registers
        const uint32_t ftid = tid - MULTIPLIERS * WAVE;
        const uint32_t m = args.m, n = args.n, k = args.k, lda = args.lda, ldb = args.ldb;
        using PieceA = typename std::conditional<A_VEC, float4, float>::type;
        constexpr int NA = A_VEC ? VEC_PIECES : PIECES;
        PieceA pa[NA];
        auto operands = [&](uint32_t head, const float *&A, const float *&B) {
            const uint32_t zo = head / batch_inner, zi = head - zo * batch_inner;
            A = args.a + zo * args.a_bs + zi * args.a_bs2, B = args.b + zo * args.b_bs + zi * args.b_bs2;
        };
        const float *A, *B;
        operands(head0, A, B);
        load_rows<0, NA>(pa, operand_buffer(A, (m - 1) * lda + k), lda, k, ftid);
        copy_operand<B_K_CONTIGUOUS, B_VEC>(lds_b, B, ldb, n, k, ftid);
        uint32_t parity = 0;
        for (uint32_t head = head0; head < batch; head += head_step) {
            write_rows<0, NA>(pa, lds_a, ftid);
            __syncthreads();  // this head's A and B are in LDS
            parity ^= 1;
            if (head + head_step < batch) {
                operands(head + head_step, A, B);
                copy_operand<B_K_CONTIGUOUS, B_VEC>(lds_b + parity * b_floats, B, ldb, n, k, ftid);
                load_rows<0, NA>(pa, operand_buffer(A, (m - 1) * lda + k), lda, k, ftid);
            }
            __syncthreads();  // the multipliers are done with this head's A
        }
        return;
    }

    // ---- a multiplying wavefront
    const uint32_t m = args.m, n = args.n, ldc = args.ldc;
    const uint32_t j = lane & 15, quarter = lane >> 4;
    // Which tiles of C, numbered in row-major order, this wavefront takes: count_1 consecutive ones from first_1 on,
    // then every twelfth of the rest.  With 12 or 13 rows of tiles a wavefront owns a whole row and the thirteenth row
    // is dealt out tile by tile; with fewer rows the tiles are cut into twelve runs of consecutive ones.
    const uint32_t col_tiles = (n + TILE - 1) / TILE, row_tiles = (m + TILE - 1) / TILE, tiles = row_tiles * col_tiles;
    uint32_t first_1, count_1, rest_at;
    if (row_tiles >= MULTIPLIERS) {
        first_1 = wave * col_tiles, count_1 = col_tiles, rest_at = MULTIPLIERS * col_tiles;
    } else {
        first_1 = wave * tiles / MULTIPLIERS, count_1 = (wave + 1) * tiles / MULTIPLIERS - first_1, rest_at = tiles;
    }
    const uint32_t rest = tiles - rest_at, count = count_1 + (rest > wave ? (rest - wave + MULTIPLIERS - 1) / MULTIPLIERS : 0);
    auto tile_at = [&](uint32_t i) { return i < count_1 ? first_1 + i : rest_at + wave + (i - count_1) * MULTIPLIERS; };
    const float *b_now = lds_b;
    // this lane's values of a tile's operand: row 16 tile + j of the operand, k = 16 quarter + s
    auto fragment = [&](float (&f)[STEPS], const float *operand, uint32_t tile) {
#pragma unroll
        for (int i = 0; i < STEPS / 4; i++) {
            const float4 v = *reinterpret_cast<const float4 *>(operand + swizzled(tile * TILE + j, STEPS * quarter + 4 * i));
            f[4 * i] = v.x, f[4 * i + 1] = v.y, f[4 * i + 2] = v.z, f[4 * i + 3] = v.w;
        }
    };
    auto fragment_b = [&](float (&f)[STEPS], uint32_t jt) {
        if constexpr (B_K_CONTIGUOUS) {
            fragment(f, b_now, jt);
        } else {
            const float *p = b_now + STEPS * quarter * J_PITCH + jt * TILE + j;
#pragma unroll
            for (int s = 0; s < STEPS; s++) f[s] = p[s * J_PITCH];
        }
    };
    for (uint32_t head = head0; head < batch; head += head_step) {
        __syncthreads();  // this head's A and B are in LDS
        const uint32_t zo = head / batch_inner, zi = head - zo * batch_inner;
        float *C = args.c + zo * args.c_bs + zi * args.c_bs2;
        float a[STEPS], b[STEPS];
        uint32_t it = 0, jt = 0;
        if (count) {
            const uint32_t t = tile_at(0);
            it = t / col_tiles, jt = t - it * col_tiles;
            fragment(a, lds_a, it);
            fragment_b(b, jt);
        }
        for (uint32_t i = 0; i < count; i++) {
            // transposed (B's fragment first): a lane's four results are C(16 it + j, 16 jt + 4 quarter + r)
            floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < STEPS; s++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b[s], a[s], acc, 0, 0, 0);
            const uint32_t row0 = it * TILE, col0 = jt * TILE;
            // the next tile's operands, while the matrix unit is busy
            if (i + 1 < count) {
                const uint32_t t = tile_at(i + 1), it_next = t / col_tiles;
                jt = t - it_next * col_tiles;
                if (it_next != it) fragment(a, lds_a, it_next);
                it = it_next;
                fragment_b(b, jt);
            }
            store_tile(acc, m, n, ldc, C, row0, col0, lane);
        }
        __syncthreads();  // done with this head's A and B
        b_now = b_now == lds_b ? lds_b + b_floats : lds_b;
    }
}

// n <= 16 NT, k in chunks of 32.  LDS: [16][N64_K_PITCH] per wavefront for its rows of A, then the chunk's part of B,
// [k][J_PITCH_N64] when B's columns are contiguous and [column][N64_K_PITCH] when its k axis is.
// B_VEC (columns contiguous only): B's rows are whole, 16-byte aligned float4s.
template <bool B_K_CONTIGUOUS, bool B_VEC, int NT>
__global__ __launch_bounds__(MAX_WAVES * WAVE) void gemm_small_n64(SmallGemm g) {
    extern __shared__ __align__(16) float lds[];
    const uint32_t tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid >> 6, nthreads = blockDim.x, nwaves = nthreads >> 6;
    const uint32_t j = lane & 15, quarter = lane >> 4;
    const uint32_t half = lane >> 5, kk32 = lane & 31;  // staging: two rows of 32 values of k per wavefront and load
    float *a_tile = lds + wave * (TILE * N64_K_PITCH);
    float *b_tile = lds + nwaves * (TILE * N64_K_PITCH);
    const float *A, *B;
    float *C;
    batch_offsets(g, A, B, C);
    const uint32_t row0 = wave * TILE;
    const bool active = row0 < g.m;
    floatx4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (uint32_t k0 = 0; k0 < g.k; k0 += N64_CHUNK) {
        if (k0) __syncthreads();  // everyone has read the previous chunk's part of B
        const bool in = k0 + kk32 < g.k;
        if (active) {
#pragma unroll
            for (int r = 0; r < TILE; r += 2)
                a_tile[(r + half) * N64_K_PITCH + kk32] = in ? A[(size_t)min(row0 + r + half, g.m - 1) * g.lda + k0 + kk32] : 0.0f;
        }
        if (B_K_CONTIGUOUS) {
            for (uint32_t jj = 2 * wave + half; jj < g.n; jj += 2 * nwaves) b_tile[jj * N64_K_PITCH + kk32] = in ? B[(size_t)jj * g.ldb + k0 + kk32] : 0.0f;
        } else if (B_VEC) {
            const uint32_t q = tid & 15;
            if (4 * q < g.n)
                for (uint32_t kk = tid >> 4; kk < N64_CHUNK; kk += nthreads >> 4)
                    *reinterpret_cast<float4 *>(b_tile + kk * J_PITCH_N64 + 4 * q) =
                        k0 + kk < g.k ? *reinterpret_cast<const float4 *>(B + (size_t)(k0 + kk) * g.ldb + 4 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            if (lane < g.n)
                for (uint32_t kk = wave; kk < N64_CHUNK; kk += nwaves) b_tile[kk * J_PITCH_N64 + lane] = k0 + kk < g.k ? B[(size_t)(k0 + kk) * g.ldb + lane] : 0.0f;
        }
        __syncthreads();
        if (!active) continue;
        // four steps (16 values of k) at a time, as many as the chunk holds
        const uint32_t groups = (min((uint32_t)N64_CHUNK, g.k - k0) + 15) / 16;
        const float *ap = a_tile + j * N64_K_PITCH + quarter;
        const float *bp = B_K_CONTIGUOUS ? b_tile + j * N64_K_PITCH + quarter : b_tile + quarter * J_PITCH_N64 + j;
        for (uint32_t grp = 0; grp < groups; grp++) {
            float a4[4], b4[NT][4];
#pragma unroll
            for (int s = 0; s < 4; s++) a4[s] = ap[16 * grp + 4 * s];
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int s = 0; s < 4; s++)
                    b4[t][s] = B_K_CONTIGUOUS ? bp[t * TILE * N64_K_PITCH + 16 * grp + 4 * s] : bp[(16 * grp + 4 * s) * J_PITCH_N64 + t * TILE];
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int t = 0; t < NT; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b4[t][s], a4[s], acc[t], 0, 0, 0);
        }
    }
    if (active) {
#pragma unroll
        for (int t = 0; t < NT; t++) store_tile(acc[t], g.m, g.n, g.ldc, C, row0, t * TILE, lane);
    }
}

inline bool float4_rows(const void *p, size_t ld, const size_t bs[2]) {
    return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0 && bs[0] % 4 == 0 && bs[1] % 4 == 0;
}

}  // namespace

// Whether launch_gemm_small_batched takes this product; decided by the shape alone, so that a product and the same
// product with an operand stored the other way round (a view of K against a materialised K^T) run the same arithmetic.
bool gemm_small_batched_fits(size_t batch, size_t m, size_t n, size_t k) {
    return batch >= 64 && batch < ((size_t)1 << 31) && m >= 1 && m <= (size_t)MAX_WAVES * TILE && k >= 1 &&
           ((k <= CHUNK && n <= (size_t)MAX_MN && m <= (size_t)MAX_MN) || (n <= 64 && k <= 4096));
}

int launch_gemm_small_batched(DeviceCtx &ctx, float *c, const float *a, const float *b, size_t batch_outer, size_t batch_inner, size_t m, size_t n,
                              size_t k, int trans_b, size_t lda, size_t ldb, size_t ldc, const size_t a_bs[2], const size_t b_bs[2],
                              const size_t c_bs[2]) {
    SmallGemm g;
    g.a = a, g.b = b, g.c = c;
    g.m = (uint32_t)m, g.n = (uint32_t)n, g.k = (uint32_t)k;
    g.lda = (uint32_t)lda, g.ldb = (uint32_t)ldb, g.ldc = (uint32_t)ldc;
    g.a_bs = a_bs[0], g.b_bs = b_bs[0], g.c_bs = c_bs[0], g.a_bs2 = a_bs[1], g.b_bs2 = b_bs[1], g.c_bs2 = c_bs[1];
    g.batch_inner = (uint32_t)batch_inner;
    const dim3 grid((unsigned)(batch_outer * batch_inner));
    const size_t waves = std::max<size_t>(MIN_WAVES, (m + TILE - 1) / TILE);
    const dim3 block((unsigned)(waves * WAVE));
    if (k <= CHUNK) {
        const bool a_vec = k % 4 == 0 && float4_rows(a, lda, a_bs);
        const bool b_vec = trans_b && k % 4 == 0 && float4_rows(b, ldb, b_bs);
        g.batch = (uint32_t)(batch_outer * batch_inner);
        const size_t shmem = ((size_t)MAX_MN * CHUNK + 2 * (trans_b ? (size_t)MAX_MN * CHUNK : (size_t)CHUNK * J_PITCH)) * sizeof(float);
        const size_t cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256;
        const dim3 pgrid((unsigned)std::min<size_t>(g.batch, cus)), pblock(PB_WAVES * WAVE);
#define GO(KC, AV, BV) hipLaunchKernelGGL((gemm_small_k64<KC, AV, BV>), pgrid, pblock, shmem, ctx.stream, g)
        if (trans_b) {
            if (a_vec && b_vec) GO(true, true, true);
            else if (a_vec) GO(true, true, false);
            else if (b_vec) GO(true, false, true);
            else GO(true, false, false);
        } else {
            if (a_vec) GO(false, true, false);
            else GO(false, false, false);
        }
#undef GO
    } else {
        const int nt = n <= 16 ? 1 : n <= 32 ? 2 : 4;
        const bool b_vec = !trans_b && n % 4 == 0 && float4_rows(b, ldb, b_bs);
        const size_t shmem = (waves * TILE * N64_K_PITCH + (trans_b ? (size_t)nt * TILE * N64_K_PITCH : (size_t)N64_CHUNK * J_PITCH_N64)) * sizeof(float);
#define GO(KC, BV, NT) hipLaunchKernelGGL((gemm_small_n64<KC, BV, NT>), grid, block, shmem, ctx.stream, g)
#define GO_NT(KC, BV)          \
    if (nt == 1) GO(KC, BV, 1); \
    else if (nt == 2) GO(KC, BV, 2); \
    else GO(KC, BV, 4)
        if (trans_b) {
            GO_NT(true, false);
        } else if (b_vec) {
            GO_NT(false, true);
        } else {
            GO_NT(false, false);
        }
#undef GO_NT
#undef GO
    }
    return ctx.check(hipGetLastError(), "gemm (small batched) launch");
}

}  // namespace altius
