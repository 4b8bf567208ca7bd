// Int8 matmul for at most 32 activation rows (decode and small batches): the op is a single pass over the weights, so
// it is built like the W4A16 decode kernel, as independent weight streams rather than as output tiles.
//
//   * the weight matrix [k, n] is cut into chunks of 64 rows x 128 columns (8 KiB); the chunks, in column-block-major
//     order, are dealt out in equal contiguous runs to 1024 wavefronts (one per SIMD), so every SIMD streams the same
//     number of bytes whatever the shape;
//   * a wavefront moves a chunk and the matching 32 x 64 slice of the activations HBM -> LDS with
//     global_load_lds_dwordx4 into a private ring of three stages (two chunks in flight behind the one being
//     computed), waits with a counted vmcnt and has no barriers; bank-conflict swizzles are applied on the source
//     side (the lane that owns an LDS slot fetches the 16 bytes that belong there);
//   * the weights stay [k][n] in LDS and are transposed into the MFMA B operand by ds_read_b64_tr_b8; 8 MFMAs
//     (v_mfma_i32_32x32x32_i8) per chunk, no VALU work at all in the loop;
//   * when a run leaves a column block (and at its end) the valid rows of the int32 accumulators go to a workspace;
//     a second kernel adds the pieces of a block's streams (integers: exact in any order) and applies the epilogue.
#include "matmul_w8a8.h"

namespace ascq {
namespace {

constexpr int kThreads = 256;        // four independent wavefronts per workgroup
constexpr uint32_t kChunkK = 64;
constexpr uint32_t kChunkN = 128;
constexpr uint32_t kMaxWaves = 1024;  // 256 compute units x 4 SIMDs
constexpr uint32_t kMaxRows = 32;
constexpr int kInstr = 10;            // 1 KiB DMA instructions per chunk: 8 of weights, 2 of activations
constexpr int kStage = kInstr * 1024;

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;

struct StreamParams {
    const int8_t* a;
    const int8_t* b;
    int32_t* partial;  // [waves][max_seg][m][128]
    uint32_t m, n, k;
    uint32_t waves, chunks_per_block, total_chunks, max_seg, per, rem;
    EpiParams epi;
};

// Stream `wave` owns chunks [stream_begin(wave), stream_begin(wave + 1)): the first `rem` streams take per + 1 chunks.
__device__ __forceinline__ uint32_t stream_begin(const StreamParams& p, uint32_t wave)
{
    return wave * p.per + (wave < p.rem ? wave : p.rem);
}

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
#define ASCQ_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
// Explicit LDS reads: they only ever follow the counted wait on the stage's loads, and the compiler's own bookkeeping
// of LDS reads against direct-to-LDS loads in flight (conservative around loops) stays out of the way.
#define ASCQ_DS_READ128(dst, addr, off) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off) : "memory")
#define ASCQ_DS_READ_TR64(dst, addr, off) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off) : "memory")

// One chunk from its LDS stage (byte address sa) into the accumulators: 2 K sub-steps x 4 column blocks of 32.
__device__ __forceinline__ void stream_compute(uint32_t sa, const uint32_t (&a_rel)[2], const uint32_t (&b_rel)[4],
                                               i32x16 (&acc)[4])
{
    i32x4 af[2];
    i32x2_t bl[2][4], bh[2][4];
    const uint32_t aa0 = sa + a_rel[0], aa1 = sa + a_rel[1];
    ASCQ_DS_READ128(af[0], aa0, 0);
    ASCQ_DS_READ128(af[1], aa1, 0);
    const uint32_t ab0 = sa + b_rel[0], ab1 = sa + b_rel[1], ab2 = sa + b_rel[2], ab3 = sa + b_rel[3];
    // K sub-step ks adds 32 rows = 4096 bytes, the upper 8 k another 8 rows = 1024 bytes
    ASCQ_DS_READ_TR64(bl[0][0], ab0, 0);
    ASCQ_DS_READ_TR64(bh[0][0], ab0, 1024);
    ASCQ_DS_READ_TR64(bl[0][1], ab1, 0);
    ASCQ_DS_READ_TR64(bh[0][1], ab1, 1024);
    ASCQ_DS_READ_TR64(bl[0][2], ab2, 0);
    ASCQ_DS_READ_TR64(bh[0][2], ab2, 1024);
    ASCQ_DS_READ_TR64(bl[0][3], ab3, 0);
    ASCQ_DS_READ_TR64(bh[0][3], ab3, 1024);
    ASCQ_DS_READ_TR64(bl[1][0], ab0, 4096);
    ASCQ_DS_READ_TR64(bh[1][0], ab0, 4096 + 1024);
    ASCQ_DS_READ_TR64(bl[1][1], ab1, 4096);
    ASCQ_DS_READ_TR64(bh[1][1], ab1, 4096 + 1024);
    ASCQ_DS_READ_TR64(bl[1][2], ab2, 4096);
    ASCQ_DS_READ_TR64(bh[1][2], ab2, 4096 + 1024);
    ASCQ_DS_READ_TR64(bl[1][3], ab3, 4096);
    ASCQ_DS_READ_TR64(bh[1][3], ab3, 4096 + 1024);
    // every value read above is an in/out operand of the wait, so nothing uses one before it has arrived
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(af[0]), "+v"(af[1]), "+v"(bl[0][0]), "+v"(bh[0][0]), "+v"(bl[0][1]), "+v"(bh[0][1]),
                   "+v"(bl[0][2]), "+v"(bh[0][2]), "+v"(bl[0][3]), "+v"(bh[0][3]), "+v"(bl[1][0]), "+v"(bh[1][0]),
                   "+v"(bl[1][1]), "+v"(bh[1][1]), "+v"(bl[1][2]), "+v"(bh[1][2]), "+v"(bl[1][3]), "+v"(bh[1][3]));
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const i32x4 bf = i32x4{bl[ks][j][0], bl[ks][j][1], bh[ks][j][0], bh[ks][j][1]};
            acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks], bf, acc[j], 0, 0, 0);
        }
    }
}

// The valid rows of the accumulators to a piece [m][128] of the workspace; clears them.  Register r of lane l in a
// 32x32 block is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
__device__ __forceinline__ void stream_flush(int32_t* __restrict__ dst, uint32_t m, uint32_t lane, i32x16 (&acc)[4])
{
    const uint32_t lrow = lane & 31u, g = lane >> 5;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = 8u * (r >> 2) + 4u * g + (r & 3);
            if (row < m) {
                dst[row * kChunkN + j * 32u + lrow] = acc[j][r];
            }
        }
        acc[j] = i32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    }
    // Stores and loads retire out of order with respect to each other, so the counted waits on the load queue are
    // only meaningful while no store is pending: drain here (once per column block and stream).
    ASCQ_WAIT_VMCNT(0);
}

__global__ __launch_bounds__(kThreads) void gemm_stream_kernel(StreamParams p)
{
    __shared__ __attribute__((aligned(1024))) char S0[4 * kStage];
    __shared__ __attribute__((aligned(1024))) char S1[4 * kStage];
    __shared__ __attribute__((aligned(1024))) char S2[4 * kStage];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t gw = blockIdx.x * 4u + wave;
    if (gw >= p.waves) {
        return;  // whole wavefront; the kernel has no barriers
    }
    const uint32_t c_begin = stream_begin(p, gw), c_end = stream_begin(p, gw + 1u);
    if (c_begin == c_end) {
        return;
    }
    const uint32_t K = p.k, N = p.n, M = p.m;
    const uint32_t cb_chunks = p.chunks_per_block, max_seg = p.max_seg;
    const int8_t* __restrict__ const Ap = p.a;
    const int8_t* __restrict__ const Bp = p.b;
    int32_t* __restrict__ const Pp = p.partial;

    // ---- producer side.  Weights: LDS slot s = instr * 64 + lane is row kb = s / 8, position s % 8, and holds piece
    // position ^ (2 * ((kb >> 1) & 3)) of the row's eight 16-byte pieces.  Activations: slot s is row s / 4 (rows past
    // m repeat the last row and are never stored), position s % 4, and holds piece position ^ ((row >> 2) & 3).
    uint32_t bk[8], bq[8], aoff[2];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const uint32_t s = u * 64u + lane;
        bk[u] = s >> 3;
        bq[u] = (s & 7u) ^ (2u * ((bk[u] >> 1) & 3u));
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t s = u * 64u + lane;
        const uint32_t row = s >> 2, piece = (s & 3u) ^ ((row >> 2) & 3u);
        const uint32_t rc = row < M ? row : M - 1u;
        aoff[u] = rc * K + 16u * piece;
    }
    uint32_t ib = c_begin / cb_chunks, ik = c_begin % cb_chunks, issued = c_begin;
    auto issue = [&](char* stage) {
        const uint32_t n0 = ib * kChunkN, k0 = ik * kChunkK;
        const int8_t* bsrc = Bp + static_cast<size_t>(k0) * N;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            uint32_t col = n0 + 16u * bq[u];
            col = col + 16u <= N ? col : N - 16u;  // columns past the end are never stored
            __builtin_amdgcn_global_load_lds((gptr_t)(bsrc + static_cast<size_t>(bk[u]) * N + col),
                                             (lds_ptr_t)(stage + u * 1024), 16, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(Ap + k0 + aoff[u]), (lds_ptr_t)(stage + (8 + u) * 1024), 16, 0,
                                             0);
        }
        // advance, staying on the last chunk once the run is exhausted (harmless repeated fetches at the tail)
        if (issued + 1u < c_end) {
            ++issued;
            if (++ik == cb_chunks) {
                ik = 0;
                ++ib;
            }
        }
    };

    // ---- consumer side
    i32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        acc[j] = i32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    }
    const uint32_t lrow = lane & 31u, g = lane >> 5;
    const uint32_t grp16 = (lane >> 4) & 1u, bsub = (lane & 15u) >> 1, psub = lane & 1u;
    // A fragment of K sub-step ks: row lrow, piece 2 ks + g; B fragment of column block j: rows 32 ks + 16 g + bsub
    // (+ 8), pieces 2 j + grp16, byte half psub -- the transposing read hands every lane 8 consecutive k of one column
    uint32_t a_rel[2], b_rel[4];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        a_rel[ks] = 8192u + lrow * 64u + (((2u * ks + g) ^ ((lrow >> 2) & 3u)) << 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        b_rel[j] = (16u * g + bsub) * 128u + (((2u * j + grp16) ^ (2u * ((bsub >> 1) & 3u))) << 4) + 8u * psub;
    }
    uint32_t seg = 0, done_in_block = c_begin % cb_chunks;

    char* s0 = S0 + wave * kStage;
    char* s1 = S1 + wave * kStage;
    char* s2 = S2 + wave * kStage;
    issue(s0);
    issue(s1);
    issue(s2);
    uint32_t c = c_begin;
    // One step: wait until everything but the two newest chunks has landed, compute, hand the piece over when the run
    // leaves its column block, refill the stage.
#define ASCQ_STREAM_STEP(stage)                                                                                   \
    {                                                                                                             \
        ASCQ_WAIT_VMCNT(2 * kInstr);                                                                              \
        stream_compute(static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)(stage))), a_rel, b_rel, acc); \
        if (++done_in_block == cb_chunks) {                                                                       \
            done_in_block = 0;                                                                                    \
            stream_flush(Pp + (static_cast<size_t>(gw) * max_seg + seg) * M * kChunkN, M, lane, acc);              \
            ++seg;                                                                                                \
        }                                                                                                         \
        if (++c == c_end) break;                                                                                  \
        issue(stage);                                                                                             \
    }
    while (true) {
        ASCQ_STREAM_STEP(s0)
        ASCQ_STREAM_STEP(s1)
        ASCQ_STREAM_STEP(s2)
    }
#undef ASCQ_STREAM_STEP
    ASCQ_WAIT_VMCNT(0);
    if (done_in_block != 0) {
        stream_flush(Pp + (static_cast<size_t>(gw) * max_seg + seg) * M * kChunkN, M, lane, acc);
    }
}

// Second pass: for four adjacent outputs, adds the int32 pieces of all streams that worked on their column block
// (exact in any order) and applies the epilogue.
__global__ __launch_bounds__(kThreads) void gemm_stream_sum_kernel(StreamParams p)
{
    const uint32_t quads_per_row = p.n / 4u;
    const uint32_t total = p.m * quads_per_row;
    const uint32_t idx = blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) {
        return;
    }
    const uint32_t row = idx / quads_per_row, col = (idx % quads_per_row) * 4u;
    const uint32_t blk = col / kChunkN, cl = col % kChunkN;
    const uint32_t first_chunk = blk * p.chunks_per_block, end_chunk = first_chunk + p.chunks_per_block;
    const uint32_t big = p.rem * (p.per + 1u);  // chunks owned by the longer streams
    const uint32_t w0 = first_chunk < big ? first_chunk / (p.per + 1u) : p.rem + (first_chunk - big) / p.per;
    uint32_t w1 = end_chunk <= big ? (end_chunk + p.per) / (p.per + 1u) : p.rem + (end_chunk - big + p.per - 1u) / p.per;
    w1 = w1 < p.waves ? w1 : p.waves;
    const size_t piece = static_cast<size_t>(p.m) * kChunkN;  // int32 per piece
    const size_t stride = static_cast<size_t>(p.max_seg) * piece;
    // the first stream may have begun in an earlier block; all later ones begin inside this block (piece 0)
    const size_t first_extra = static_cast<size_t>(blk - stream_begin(p, w0) / p.chunks_per_block) * piece;
    const int32_t* base = p.partial + static_cast<size_t>(w0) * stride + row * kChunkN + cl;
    i32x4 acc = i32x4{0, 0, 0, 0};
    for (uint32_t w = w0; w < w1; w += 8u) {
        i32x4 v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {  // 8 independent loads in flight
            const uint32_t wu = w + u;
            const size_t off = static_cast<size_t>(wu - w0) * stride + (wu == w0 ? first_extra : 0u);
            v[u] = wu < w1 ? *reinterpret_cast<const i32x4*>(base + off) : i32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) acc += v[u];
    }
    const float tok = p.epi.has_tok ? p.epi.tok_scale[row] : 1.0f;
    dispatch_out(p.epi, [&](auto tag) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int32_t a = acc[c];
            if (p.epi.bias_kind == ASCQ_MM_BIAS_I32_PRE) {
                a += static_cast<const int32_t*>(p.epi.bias)[col + c];
            }
            epilogue_store<decltype(tag)::value>(p.epi, row, col + c, a, load_channel_q(p.epi, col + c), tok,
                                                 load_bias_post(p.epi, col + c));
        }
    });
}

struct StreamPlan {
    uint32_t waves, chunks_per_block, total_chunks, max_seg;
};

StreamPlan make_plan(uint32_t n, uint32_t k)
{
    StreamPlan pl;
    const uint32_t blocks_n = (n + kChunkN - 1u) / kChunkN;
    pl.chunks_per_block = k / kChunkK;
    pl.total_chunks = blocks_n * pl.chunks_per_block;
    pl.waves = pl.total_chunks < kMaxWaves ? pl.total_chunks : kMaxWaves;
    const uint32_t per = (pl.total_chunks + pl.waves - 1u) / pl.waves;  // longest run
    pl.max_seg = (per + pl.chunks_per_block - 2u) / pl.chunks_per_block + 1u;
    return pl;
}

}  // namespace

bool gemm_stream_supported(const GemmParams& p)
{
    return p.m <= kMaxRows && p.k % kChunkK == 0 && p.n % 16 == 0 && p.n >= 16 && aligned16(p.a) && aligned16(p.b) &&
           static_cast<uint64_t>((p.n + kChunkN - 1u) / kChunkN) * (p.k / kChunkK) < (1ull << 31);
}

size_t gemm_stream_workspace(uint32_t m, uint32_t n, uint32_t k)
{
    if (m > kMaxRows || k % kChunkK != 0 || k == 0) {
        return 0;
    }
    const StreamPlan pl = make_plan(n, k);
    return static_cast<size_t>(pl.waves) * pl.max_seg * m * kChunkN * sizeof(int32_t);
}

// The caller has checked gemm_stream_supported; the workspace must hold gemm_stream_workspace bytes, 16-byte aligned.
int launch_gemm_stream(const GemmParams& g, void* workspace, hipStream_t st)
{
    const StreamPlan pl = make_plan(g.n, g.k);
    StreamParams p{};
    p.a = g.a;
    p.b = g.b;
    p.partial = static_cast<int32_t*>(workspace);
    p.m = g.m;
    p.n = g.n;
    p.k = g.k;
    p.waves = pl.waves;
    p.chunks_per_block = pl.chunks_per_block;
    p.total_chunks = pl.total_chunks;
    p.max_seg = pl.max_seg;
    p.per = pl.total_chunks / pl.waves;
    p.rem = pl.total_chunks % pl.waves;
    p.epi = g.epi;
    if (plan_recording()) {
        // at most this many streams work on one column block: the partial results the second kernel adds
        const uint32_t pieces = p.per ? (pl.chunks_per_block + p.per - 1u) / p.per + 1u : pl.chunks_per_block;
        plan_note(ASCQ_MM_KERNEL_STREAM, kMaxRows, kChunkN, kChunkK, (pl.waves + 3u) / 4u, pieces, 3u * 4u * kStage,
                  gemm_stream_workspace(g.m, g.n, g.k));
        plan_note(0, 0, 0, 0, 0, 0, 0, 0);  // the kernel that adds the pieces and applies the epilogue
        return ASCQ_OK;
    }
    gemm_stream_kernel<<<(pl.waves + 3u) / 4u, kThreads, 0, st>>>(p);
    int rc = launch_status("ascq_matmul_w8a8 (stream)");
    if (rc != ASCQ_OK) {
        return rc;
    }
    const uint32_t quads = g.m * (g.n / 4u);
    gemm_stream_sum_kernel<<<(quads + kThreads - 1) / kThreads, kThreads, 0, st>>>(p);
    return launch_status("ascq_matmul_w8a8 (stream epilogue)");
}

}  // namespace ascq
