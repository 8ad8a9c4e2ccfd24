// Many small fp32 products at once: attention's Q K^T ([197, 64] x [64, 197] per head) and P V
// ([197, 197] x [197, 64]) of a session that runs the three operators apart, as the reference does
// (compute_mat_mul, crates/session_interpreter/src/session.rs:621-684, one sgemm per batch entry).
//
// The 128 x 128 tiles of matmul.hip fit such matrices badly: four tiles per head of which 59 % is
// padding, every operand fetched twice.  Here one block of 16 wavefronts per compute unit walks the
// heads blockIdx.x, blockIdx.x + gridDim.x, ... and takes each product whole, cut into 16 x 16 tiles
// of v_mfma_f32_16x16x4_f32 (197 rows pad to 208, where 32 x 32 tiles pad to 224).
//
// Twelve wavefronts multiply (three per SIMD) and four fetch (one per SIMD).  The fetchers bring the
// operands from global memory into LDS a step ahead of the multipliers, which read LDS only and store
// results.  The two kinds of work are kept in different wavefronts because the hardware counts a
// wavefront's loads and stores in one counter: a wavefront that waits for a load it issued before
// storing results waits for those stores too, and stores take microseconds to drain.  (One block per
// matrix, loading and then multiplying, leaves the matrix unit idle while it loads, and two such
// blocks on a compute unit do not fill each other's gaps: loads issued while the other block stores
// queue behind those stores in the compute unit's L1, which serves requests in order.)
//
// The instruction adds four values of k per step, one from each quarter of the wavefront (lane / 16),
// and a sum does not care which four: quarter q takes k = 16 q .. 16 q + 15 of a chunk of 64, so that
// a lane reads its 16 values as four 16-byte pieces of a row of LDS.  The assignment is the same for A
// and B and whichever way round B is stored, so that a product and the same product through a view of
// its second operand add the same numbers in the same order.  Tiles are computed transposed (B's
// fragment as the instruction's first operand), so that a lane's four results lie next to each other
// in a row of C.
//
//   k <= 64 (Q K^T), gemm_small_k64: all of A and all of B of a head in LDS (B twice, for this head and
//     the next); a multiplier keeps its rows of A in registers and sweeps its row of tiles of C from
//     left to right, a tile stored as soon as it is finished.
//   n <= 64 (P V), gemm_small_n64: k goes by in chunks of 64, each chunk of A and of B in LDS twice; a
//     multiplier keeps the (up to five) tiles of C it owns in registers until the head is done.
// C = A B only (no alpha, beta or third operand), A with unit stride along k; B either way round;
// m <= 208.
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

struct SmallGemm {
    const float *a, *b;
    float *c;
    uint32_t m, n, k;
    uint32_t lda, ldb, ldc;  // A(i, kk) = a[i * lda + kk]; B(kk, j) = b[j * ldb + kk] (k contiguous) or b[kk * ldb + j]
    uint64_t a_bs, b_bs, c_bs, a_bs2, b_bs2, c_bs2;
    uint32_t batch_inner;
    uint32_t batch;  // heads
};

// A barrier that orders the block's LDS traffic only.  __syncthreads() also waits for the wavefront's global loads and
// stores (one counter for both), which is what the fetchers' loads in flight and the multipliers' draining stores must
// not be made to do: nothing here hands data from wavefront to wavefront through global memory.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
// LDS (156 KB): all of A as [208][64] and all of B as [column][64], whichever way round B lies in memory, both with the
// 16-byte pieces of a row exchanged by piece ^= row % 16, which spreads a column of pieces over the banks without padding.
//
// Twelve wavefronts multiply (three per SIMD) and four fetch (one per SIMD).  B is in LDS twice: while the multipliers
// read one copy the fetchers fill the other with the next head's; the next head's A waits in the fetchers' registers (52
// per lane) and is written between two barriers when the multipliers are done.  The two kinds of work are kept in
// different wavefronts because the hardware counts a wavefront's loads and stores in one counter: a wavefront that waits
// for a load it issued before storing results waits for the stores too, and the head's last stores take several
// microseconds to drain.
//
// A multiplier sweeps a row of tiles of C from left to right, so that the 64-byte pieces it stores complete each other's
// cache lines while those are still on their way out (pieces that meet a half-written line much later cost twice the
// time), and the wavefronts keep to rows of their own where the shape allows: 197 rows are twelve rows of tiles, one
// per multiplier, and a thirteenth of five rows whose tiles are dealt out one by one (14 or 15 tiles per wavefront).
constexpr int PB_WAVES = 16;
constexpr size_t MIN_PRODUCTS = 128;  // fewer leave too many compute units without a block: the general kernel's tiles spread better
                                      // (197 x 197 x 64: 18 against 20 us at 96 products, 28 against 22 us at 192)
constexpr int FETCHERS = 4, MULTIPLIERS = PB_WAVES - FETCHERS;
constexpr int MAX_MN = 208;                                  // rows of A and columns of B
constexpr int VEC_PIECES = MAX_MN * (CHUNK / 4) / (FETCHERS * WAVE);   // float4s per fetching lane and operand: 13
constexpr int PIECES = MAX_MN * CHUNK / (FETCHERS * WAVE);   // single values per fetching lane and operand: 52

// The float offset of k (a multiple of 4 for float4s) in row `row` of an operand stored [row][64] with exchanged pieces.
__device__ __forceinline__ uint32_t swizzled(uint32_t row, uint32_t k) { return row * CHUNK + ((((k >> 2) ^ row) & 15) << 2) + (k & 3); }

// The fetchers address an operand of a head as a buffer of its own, so that pieces past the operand's last value (rows
// past m, columns past n, values of k past the end in an operand stored [k][column]) read as zero without a test and,
// for the last head of a tensor, without touching memory behind it.  The whole offset of a piece goes into the
// instruction's vector offset: the scalar offset takes no part in the comparison with the buffer's size on this part.
// (The launcher sends operands of 2^29 floats and more per head to the general kernel: offsets are 32 bits.)
// One running offset per thread: without the empty asm the compiler keeps an offset register per piece and spills.
__device__ __forceinline__ uint32_t next_piece(uint32_t offset, uint32_t step) {
    offset += step;
    asm volatile("" : "+v"(offset));
    return offset;
}
typedef float f32x4_raw __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_raw __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t operand_buffer(const float *p, uint32_t floats) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0, (int)(floats * 4u), 0x00020000);  // raw buffer of 32-bit words
}

// Pieces FIRST .. FIRST + COUNT - 1 of a [rows][k <= 64] operand -> registers of the 256 fetching threads (ftid).  A
// thread's pieces are 16 (float4s) or 4 (single values) rows apart at the same k; k past `k` reads as zero.
template <int FIRST, int COUNT>
__device__ __forceinline__ void load_rows(float4 (&v)[COUNT], __amdgpu_buffer_rsrc_t src, uint32_t ld, uint32_t k, uint32_t ftid) {
    const uint32_t q = ftid & 15;
    uint32_t offset = (((ftid >> 4) + 16 * FIRST) * ld + 4 * q) * 4;
    const bool in = 4 * q < k;
#pragma unroll
    for (int u = 0; u < COUNT; u++, offset = next_piece(offset, 16 * ld * 4)) {
        const f32x4_raw f = __builtin_bit_cast(f32x4_raw, __builtin_amdgcn_raw_buffer_load_b128(src, offset, 0, 0));
        v[u] = in ? make_float4(f.x, f.y, f.z, f.w) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}
template <int FIRST, int COUNT>
__device__ __forceinline__ void load_rows(float (&v)[COUNT], __amdgpu_buffer_rsrc_t src, uint32_t ld, uint32_t k, uint32_t ftid) {
    const uint32_t kk = ftid & 63;
    uint32_t offset = (((ftid >> 6) + 4 * FIRST) * ld + kk) * 4;
    const bool in = kk < k;
#pragma unroll
    for (int u = 0; u < COUNT; u++, offset = next_piece(offset, 4 * ld * 4)) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(src, offset, 0, 0));
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
    uint32_t offset = (FIRST * ld + ftid) * 4;
#pragma unroll
    for (int u = 0; u < COUNT; u++, offset = next_piece(offset, ld * 4)) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(src, offset, 0, 0));
        v[u] = in ? f : 0.0f;
    }
}
// ... written as [column][64] with exchanged pieces like an operand stored that way: the multipliers read B the same way
// whichever way round it came (eight lanes of a wavefront meet in a bank here; the fetchers have the time).
template <int FIRST, int COUNT>
__device__ __forceinline__ void write_columns(const float (&v)[COUNT], float *dst, uint32_t ftid) {
    if (ftid >= MAX_MN) return;
#pragma unroll
    for (int u = 0; u < COUNT; u++) dst[swizzled(ftid, FIRST + u)] = v[u];
}
// One operand of a head, global memory -> LDS, in rounds of loads that are all asked for before the first is written
// (two rounds of 7 and 6 float4s; four of 13 single values for rows, two of 32 for columns).  `extent` is the
// operand's number of rows (ROWS) or columns.
template <bool ROWS, bool VEC>
__device__ __forceinline__ void copy_operand(float *dst, const float *src, uint32_t ld, uint32_t extent, uint32_t k, uint32_t ftid) {
    // between rounds: keeps the compiler from asking for the next round before this one is written (registers)
    auto round_done = [] { asm volatile("" ::: "memory"); };
    if constexpr (ROWS && VEC) {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (extent - 1) * ld + k);
        constexpr int H = (VEC_PIECES + 1) / 2;
        float4 v0[H], v1[VEC_PIECES - H];
        load_rows<0, H>(v0, buf, ld, k, ftid);
        write_rows<0, H>(v0, dst, ftid);
        round_done();
        load_rows<H, VEC_PIECES - H>(v1, buf, ld, k, ftid);
        write_rows<H, VEC_PIECES - H>(v1, dst, ftid);
    } else if constexpr (ROWS) {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (extent - 1) * ld + k);
        constexpr int H = PIECES / 4;
        float v0[H], v1[H], v2[H], v3[H];
        load_rows<0, H>(v0, buf, ld, k, ftid);
        write_rows<0, H>(v0, dst, ftid);
        round_done();
        load_rows<H, H>(v1, buf, ld, k, ftid);
        write_rows<H, H>(v1, dst, ftid);
        round_done();
        load_rows<2 * H, H>(v2, buf, ld, k, ftid);
        write_rows<2 * H, H>(v2, dst, ftid);
        round_done();
        load_rows<3 * H, H>(v3, buf, ld, k, ftid);
        write_rows<3 * H, H>(v3, dst, ftid);
    } else {
        const __amdgpu_buffer_rsrc_t buf = operand_buffer(src, (k - 1) * ld + extent);
        constexpr int H = CHUNK / 2;
        float v0[H], v1[CHUNK - H];
        load_columns<0, H>(v0, buf, ld, extent, ftid);
        write_columns<0, H>(v0, dst, ftid);
        round_done();
        load_columns<H, CHUNK - H>(v1, buf, ld, extent, ftid);
        write_columns<H, CHUNK - H>(v1, dst, ftid);
    }
    round_done();
}

template <bool B_K_CONTIGUOUS, bool A_VEC, bool B_VEC>
__global__ __launch_bounds__(PB_WAVES * WAVE) void gemm_small_k64(SmallGemm args) {
    extern __shared__ __align__(16) float lds[];
    const uint32_t tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid >> 6;
    constexpr uint32_t b_floats = MAX_MN * CHUNK;  // B is there twice, for this head and the next
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
            lds_barrier();  // this head's A and B are in LDS
            parity ^= 1;
            if (head + head_step < batch) {
                operands(head + head_step, A, B);
                copy_operand<B_K_CONTIGUOUS, B_VEC>(lds_b + parity * b_floats, B, ldb, n, k, ftid);
                load_rows<0, NA>(pa, operand_buffer(A, (m - 1) * lda + k), lda, k, ftid);
            }
            lds_barrier();  // the multipliers are done with this head's A
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
    auto fragment_b = [&](float (&f)[STEPS], uint32_t jt) { fragment(f, b_now, jt); };
    for (uint32_t head = head0; head < batch; head += head_step) {
        lds_barrier();  // this head's A and B are in LDS
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
        lds_barrier();  // done with this head's A and B
        b_now = b_now == lds_b ? lds_b + b_floats : lds_b;
    }
}

// n <= 64, m <= 208, any k.  LDS: a chunk of A, [208][64] with exchanged pieces, and the same chunk of B as
// [column][64] with exchanged pieces; both twice.  While the
// multipliers work on chunk g out of one copy, the fetchers fill the other with chunk g + 1 (of the same head or the
// first of the next), and one barrier per chunk separates the two.
//
// A multiplier owns a row of 16 rows of C (up to four tiles); with 13 rows of tiles the last row's tiles go to
// wavefronts 0 .. 3 as a fifth tile (13 tiles per SIMD).  A's rows are whole 16-byte pieces only by accident (197
// floats per row of P), so the fetchers read them with buffer loads, which need no more than 4-byte alignment, and
// zero what lies past k themselves: a row's last piece reaches into the next row.
constexpr int N64_B_PIECES = CHUNK * 64 / (FETCHERS * WAVE);  // single values per fetching lane of a [64][64] chunk of B: 16

// What a fetching lane holds of a chunk between asking for it and writing it to LDS.
template <bool B_K_CONTIGUOUS>
struct N64Pieces {
    float4 a[VEC_PIECES];
    typename std::conditional<B_K_CONTIGUOUS, float4, float>::type b[B_K_CONTIGUOUS ? 4 : N64_B_PIECES];
};

// Ask for values k0 .. k0 + 63 of A (13 float4s per lane, 16 rows apart; rows past m lie past the buffer's end and read
// as zero) and of B.
template <bool B_K_CONTIGUOUS>
__device__ __forceinline__ void n64_ask(N64Pieces<B_K_CONTIGUOUS> &v, const float *A, const float *B, uint32_t m, uint32_t n, uint32_t k, uint32_t lda,
                                        uint32_t ldb, uint32_t k0, uint32_t ftid) {
    const uint32_t q = ftid & 15;
    const __amdgpu_buffer_rsrc_t abuf = operand_buffer(A, (m - 1) * lda + k);
    uint32_t a_offset = ((ftid >> 4) * lda + k0 + 4 * q) * 4;
#pragma unroll
    for (int u = 0; u < VEC_PIECES; u++, a_offset = next_piece(a_offset, 16 * lda * 4)) {
        const f32x4_raw f = __builtin_bit_cast(f32x4_raw, __builtin_amdgcn_raw_buffer_load_b128(abuf, a_offset, 0, 0));
        v.a[u] = make_float4(f.x, f.y, f.z, f.w);
    }
    if constexpr (B_K_CONTIGUOUS) {  // B as [column][k]: 4 float4s per lane, 16 columns apart
        const __amdgpu_buffer_rsrc_t bbuf = operand_buffer(B, (n - 1) * ldb + k);
        uint32_t b_offset = ((ftid >> 4) * ldb + k0 + 4 * q) * 4;
#pragma unroll
        for (int u = 0; u < 4; u++, b_offset = next_piece(b_offset, 16 * ldb * 4)) {
            const f32x4_raw f = __builtin_bit_cast(f32x4_raw, __builtin_amdgcn_raw_buffer_load_b128(bbuf, b_offset, 0, 0));
            v.b[u] = make_float4(f.x, f.y, f.z, f.w);
        }
    } else {  // B as [k][column]: 16 values per lane, 4 rows of k apart; rows past k lie past the buffer's end
        const __amdgpu_buffer_rsrc_t bbuf = operand_buffer(B, (k - 1) * ldb + n);
        uint32_t b_offset = ((k0 + (ftid >> 6)) * ldb + (ftid & 63)) * 4;
#pragma unroll
        for (int u = 0; u < N64_B_PIECES; u++, b_offset = next_piece(b_offset, 4 * ldb * 4))
            v.b[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bbuf, b_offset, 0, 0));
    }
}

// ... and write them to LDS; what lies past k (a row's last float4 reaches into the next row) and past n becomes zero.
template <bool B_K_CONTIGUOUS>
__device__ __forceinline__ void n64_write(const N64Pieces<B_K_CONTIGUOUS> &v, float *dst_a, float *dst_b, uint32_t n, uint32_t k, uint32_t k0, uint32_t ftid) {
    const uint32_t q = ftid & 15, kk = k0 + 4 * q;
    auto within_k = [&](float4 f) {
        f.x = kk < k ? f.x : 0.f, f.y = kk + 1 < k ? f.y : 0.f, f.z = kk + 2 < k ? f.z : 0.f, f.w = kk + 3 < k ? f.w : 0.f;
        return f;
    };
#pragma unroll
    for (int u = 0; u < VEC_PIECES; u++) *reinterpret_cast<float4 *>(dst_a + swizzled((ftid >> 4) + 16 * u, 4 * q)) = within_k(v.a[u]);
    if constexpr (B_K_CONTIGUOUS) {
#pragma unroll
        for (int u = 0; u < 4; u++) *reinterpret_cast<float4 *>(dst_b + swizzled((ftid >> 4) + 16 * u, 4 * q)) = within_k(v.b[u]);
    } else {
        const uint32_t jj = ftid & 63;  // [column][64] like an operand stored that way (eight lanes meet in a bank)
#pragma unroll
        for (int u = 0; u < N64_B_PIECES; u++) dst_b[swizzled(jj, (ftid >> 6) + 4 * u)] = jj < n ? v.b[u] : 0.f;
    }
}

template <bool B_K_CONTIGUOUS>
__global__ __launch_bounds__(PB_WAVES * WAVE) void gemm_small_n64(SmallGemm args) {
    extern __shared__ __align__(16) float lds[];
    const uint32_t tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid >> 6;
    constexpr uint32_t a_floats = MAX_MN * CHUNK, b_floats = 64 * CHUNK;
    float *lds_a = lds, *lds_b = lds + 2 * a_floats;
    const uint32_t batch = args.batch, batch_inner = args.batch_inner, k = args.k;
    const uint32_t chunks = (k + CHUNK - 1) / CHUNK;
    const uint32_t my_heads = (batch - blockIdx.x + gridDim.x - 1) / gridDim.x;  // the grid has at most as many blocks as there are heads
    const uint32_t steps_total = my_heads * chunks;

    if (wave >= MULTIPLIERS) {
        // ---- a fetching wavefront: chunk g + 1 is written to LDS while the multipliers work on chunk g, and chunk g + 2 is
        // asked for right after, so that its way from memory has two chunks' time
        const uint32_t ftid = tid - MULTIPLIERS * WAVE;
        const uint32_t m = args.m, n = args.n, lda = args.lda, ldb = args.ldb;
        N64Pieces<B_K_CONTIGUOUS> pieces;
        auto ask = [&](uint32_t g) {  // chunk g of this block's heads
            const uint32_t hi = g / chunks, c = g - hi * chunks, head = blockIdx.x + hi * gridDim.x;
            const uint32_t zo = head / batch_inner, zi = head - zo * batch_inner;
            n64_ask<B_K_CONTIGUOUS>(pieces, args.a + zo * args.a_bs + zi * args.a_bs2, args.b + zo * args.b_bs + zi * args.b_bs2, m, n, k, lda, ldb, c * CHUNK, ftid);
        };
        auto write = [&](uint32_t g) {  // -> copy g % 2
            n64_write<B_K_CONTIGUOUS>(pieces, lds_a + (g & 1) * a_floats, lds_b + (g & 1) * b_floats, n, k, (g % chunks) * CHUNK, ftid);
        };
        ask(0);
        write(0);
        for (uint32_t g = 0; g < steps_total; g++) {
            lds_barrier();  // chunk g is in LDS, and the multipliers are done with chunk g - 1
            if (g + 1 < steps_total) { ask(g + 1); write(g + 1); }
        }
        return;
    }

    // ---- a multiplying wavefront
    const uint32_t m = args.m, n = args.n, ldc = args.ldc;
    const uint32_t j = lane & 15, quarter = lane >> 4;
    const uint32_t col_tiles = (n + TILE - 1) / TILE, row_tiles = (m + TILE - 1) / TILE;
    const bool owner = wave < row_tiles;
    // the tiles of the rows past the twelfth: tile e of them belongs to wavefront e
    const uint32_t extras = row_tiles > (uint32_t)MULTIPLIERS ? (row_tiles - MULTIPLIERS) * col_tiles : 0;
    const bool extra = wave < extras;
    const uint32_t extra_it = MULTIPLIERS + wave / col_tiles, extra_jt = wave % col_tiles;
    auto fragment = [&](float (&f)[STEPS], const float *operand, uint32_t tile) {
#pragma unroll
        for (int i = 0; i < STEPS / 4; i++) {
            const float4 v = *reinterpret_cast<const float4 *>(operand + swizzled(tile * TILE + j, STEPS * quarter + 4 * i));
            f[4 * i] = v.x, f[4 * i + 1] = v.y, f[4 * i + 2] = v.z, f[4 * i + 3] = v.w;
        }
    };
    floatx4 acc[4], acc_x;
    uint32_t head = blockIdx.x, c = 0;
    for (uint32_t g = 0; g < steps_total; g++) {
        lds_barrier();  // chunk g is in LDS
        if (c == 0) {
#pragma unroll
            for (int t = 0; t < 4; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
            acc_x = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        const float *a_now = lds_a + (g & 1) * a_floats, *b_now = lds_b + (g & 1) * b_floats;
        // steps of this chunk that hold values of k at all: quarter 0 has the chunk's first 16
        const uint32_t steps = min((uint32_t)STEPS, k - c * CHUNK);
        float a[STEPS], ax[STEPS];
        if (owner) fragment(a, a_now, wave);
        if (extra) fragment(ax, a_now, extra_it);
        auto fragment_b = [&](float (&f)[STEPS], uint32_t t) { fragment(f, b_now, t); };
        // transposed (B's fragment first): a lane's four results are C(16 row of tiles + j, 16 t + 4 quarter + r)
        auto multiply = [&](auto whole) {  // whole: all 16 steps, without a test per step
            constexpr bool WHOLE = decltype(whole)::value;
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if ((uint32_t)t < col_tiles) {
                    float b[STEPS];
                    fragment_b(b, t);
                    if (owner) {
#pragma unroll
                        for (int s = 0; s < STEPS; s++)
                            if (WHOLE || (uint32_t)s < steps) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[s], a[s], acc[t], 0, 0, 0);
                    }
                    if (extra && extra_jt == (uint32_t)t) {
#pragma unroll
                        for (int s = 0; s < STEPS; s++)
                            if (WHOLE || (uint32_t)s < steps) acc_x = __builtin_amdgcn_mfma_f32_16x16x4f32(b[s], ax[s], acc_x, 0, 0, 0);
                    }
                }
            }
        };
        if (owner || extra) {
            if (steps == STEPS) multiply(std::true_type{});
            else multiply(std::false_type{});
        }
        if (++c == chunks) {
            const uint32_t zo = head / batch_inner, zi = head - zo * batch_inner;
            float *C = args.c + zo * args.c_bs + zi * args.c_bs2;
            if (owner) {
#pragma unroll
                for (int t = 0; t < 4; t++)
                    if ((uint32_t)t < col_tiles) store_tile(acc[t], m, n, ldc, C, wave * TILE, t * TILE, lane);
            }
            if (extra) store_tile(acc_x, m, n, ldc, C, extra_it * TILE, extra_jt * TILE, lane);
            c = 0, head += gridDim.x;
        }
    }
}

inline bool float4_rows(const void *p, size_t ld, const size_t bs[2]) {
    return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0 && bs[0] % 4 == 0 && bs[1] % 4 == 0;
}

}  // namespace

// Whether launch_gemm_small_batched takes this product; decided by the shape alone, so that a product and the same
// product with an operand stored the other way round (a view of K against a materialised K^T) run the same arithmetic.
bool gemm_small_batched_fits(size_t batch, size_t m, size_t n, size_t k) {
    return batch >= MIN_PRODUCTS && batch < ((size_t)1 << 31) && m >= 1 && m <= (size_t)MAX_MN && k >= 1 &&
           ((k <= CHUNK && n <= (size_t)MAX_MN) || (n <= 64 && k <= 4096));
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
    g.batch = (uint32_t)(batch_outer * batch_inner);
    const size_t cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256;
    const dim3 grid((unsigned)std::min<size_t>(g.batch, cus)), block(PB_WAVES * WAVE);
    if (k <= CHUNK) {
        const bool a_vec = k % 4 == 0 && float4_rows(a, lda, a_bs);
        const bool b_vec = trans_b && k % 4 == 0 && float4_rows(b, ldb, b_bs);
        const size_t shmem = 3 * (size_t)MAX_MN * CHUNK * sizeof(float);
#define GO(KC, AV, BV) hipLaunchKernelGGL((gemm_small_k64<KC, AV, BV>), grid, block, shmem, ctx.stream, g)
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
        const size_t shmem = 2 * ((size_t)MAX_MN * CHUNK + (size_t)64 * CHUNK) * sizeof(float);
        if (trans_b) hipLaunchKernelGGL((gemm_small_n64<true>), grid, block, shmem, ctx.stream, g);
        else hipLaunchKernelGGL((gemm_small_n64<false>), grid, block, shmem, ctx.stream, g);
    }
    return ctx.check(hipGetLastError(), "gemm (small batched) launch");
}

}  // namespace altius
