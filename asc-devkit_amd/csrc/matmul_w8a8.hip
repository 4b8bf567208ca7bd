// int8 x int8 -> int32 matmul with the fused dequant epilogue (Matmul + SetQuantScalar / SetQuantVector) and the
// quantized grouped matmul, for gfx950.
//
// Design (one workgroup = 256 lanes = 4 wavefronts, one per SIMD):
//   * v_mfma_i32_32x32x32_i8; a wavefront owns TM x TN accumulator blocks of 32x32 (4x4 -> 256 accumulator
//     registers for the 256x256 tile), so every 16-byte operand fragment read from LDS feeds 4 MFMAs.
//   * K is walked in steps of 128 bytes: one full 128-byte line per row of A per step.  Global loads of step t+1
//     are issued into registers before the MFMAs of step t and written to the other LDS stage after them
//     (double-buffered LDS, one barrier per step).
//   * A [m, k] rows are K-contiguous, which is the MFMA operand order: 16-byte chunks go to LDS unchanged, with the
//     chunk index XOR-swizzled by the row so that both the 16-byte writes and the 16-byte fragment reads of 16
//     consecutive rows hit 16 different 16-byte bank groups.
//   * B [k, n] is N-contiguous: each lane loads a 16(k) x 8(n) byte patch, transposes it in registers with
//     v_perm_b32 (4x4 byte transposes) and writes one 16-byte K-chunk per column.  B rows in LDS are padded to
//     144 bytes; with lanes ordered (k-block fastest) both these writes and the fragment reads are conflict-free.
//     The MFMA sums over k, so any k order inside a chunk is fine as long as A and B agree (they do: byte b of
//     chunk c is k = 16c + b for both).
//   * Epilogue in registers: int32 -> fp32, x channel scale, x token scale, + bias, activation, one rounding to the
//     output type.  No int32 round trip through memory (the reference hands the accumulator to the vector core
//     through a global-memory workspace).
//   * Tiles are numbered so that the 8 XCDs (workgroup id mod 8) each own a contiguous range of tiles, walking M
//     fastest: the workgroups of one XCD share B column panels in that XCD's L2.
//   * Small M is weight-bandwidth bound: 32-row tiles with split-K; partial sums are added with int32 atomics
//     (exact and order-independent) into a caller workspace and a second kernel applies the epilogue.
//   * Grouped matmul: same tile body; each workgroup finds its (group, row range) from the device-side group list,
//     so no host synchronisation is needed and empty groups cost nothing.
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "matmul_w8a8.h"

namespace ascq {
namespace {

constexpr int kThreads = 256;
constexpr int kBK = 128;          // bytes of K per pipeline step
constexpr int kAStride = 128;     // LDS row stride of a K-contiguous operand (XOR swizzle)
constexpr int kBStride = 144;     // LDS row stride of the transposed B operand (padding instead of swizzle)

// 4x4 byte transpose: r[i] holds bytes (n0..n3) of row i; c[j] receives (row0..row3) of column j.
__device__ __forceinline__ void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t& c0,
                                             uint32_t& c1, uint32_t& c2, uint32_t& c3)
{
    // v_perm_b32(s0, s1, sel): selector values 0-3 pick bytes of s1, 4-7 bytes of s0
    const uint32_t lo01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t hi01 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t lo23 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t hi23 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c0 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    c1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    c2 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    c3 = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

__device__ __forceinline__ uint32_t swz_off(uint32_t row, uint32_t chunk)
{
    return row * kAStride + ((chunk ^ ((row >> 1) & 7u)) << 4);
}

template <int TM, int TN, int WGM, int WGN, bool kTransB, int STAGES = 2, int MINBLOCKS = 1>
struct Tile {
    static constexpr int kStages = STAGES;
    static constexpr int kMinBlocks = MINBLOCKS;
    static constexpr int BM = WGM * TM * 32;
    static constexpr int BN = WGN * TN * 32;
    static constexpr int kWGM = WGM, kWGN = WGN, kWTM = TM, kWTN = TN;
    static constexpr int kBRow = kTransB ? kAStride : kBStride;
    static constexpr int kABytes = BM * kAStride;
    static constexpr int kBBytes = BN * kBRow;
    static constexpr int kStage = kABytes + kBBytes;
    static constexpr int kLds = STAGES * kStage;
    static constexpr int kAChunks = BM * (kBK / 16) / kThreads;  // 16-byte chunks of A per lane per step
    static constexpr int kBChunksT = BN * (kBK / 16) / kThreads; // same for a K-contiguous B
    static constexpr int kCols = BN / 32;                        // columns per lane of an N-contiguous B (8 or 4)
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    static_assert(kCols == 8 || kCols == 4, "BN must be 256 or 128");
};

// One output tile: rows [row0, row_end) x columns [n0, n0 + BN), K range [k_begin, k_end).
template <class T, bool kTransB, bool kSplitK>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const int8_t* __restrict__ A,
                                          const int8_t* __restrict__ B, const EpiParams& e, uint32_t row0,
                                          uint32_t row_end, uint32_t n0, uint32_t k_begin, uint32_t k_end,
                                          size_t chan_off, char* smem)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t K = p.k, N = p.n;

    // ---------------- staging registers
    u32x4 areg[T::kAChunks];
    u32x4 bregT[kTransB ? T::kBChunksT : 1];
    uint32_t breg[kTransB ? 1 : 16][kTransB ? 1 : (T::kCols / 4)];

    // lane -> patch of the N-contiguous B tile: k-block fastest so that LDS writes spread over all banks
    const uint32_t kb = tid & 7u;
    const uint32_t nb = tid >> 3;

    // Per-lane source pointers of the first K step (rows / columns past the end are clamped: they are never stored).
    const int8_t* aptr[T::kAChunks];
#pragma unroll
    for (int i = 0; i < T::kAChunks; ++i) {
        const uint32_t c = tid + kThreads * i;
        uint32_t row = row0 + (c >> 3);
        row = row < row_end ? row : row_end - 1;
        aptr[i] = A + static_cast<size_t>(row) * K + ((c & 7u) << 4);
    }
    const int8_t* bptrT[kTransB ? T::kBChunksT : 1];
    const int8_t* bptr = B;
    if constexpr (kTransB) {
#pragma unroll
        for (int i = 0; i < T::kBChunksT; ++i) {
            const uint32_t c = tid + kThreads * i;
            uint32_t col = n0 + (c >> 3);
            col = col < N ? col : N - 1;
            bptrT[i] = B + static_cast<size_t>(col) * K + ((c & 7u) << 4);
        }
    } else {
        uint32_t col = n0 + nb * T::kCols;
        col = col + T::kCols <= N ? col : N - T::kCols;
        bptr = B + static_cast<size_t>(kb * 16u) * N + col;
    }

    // kFull: the whole 128-byte K step is inside [k_begin, k_end): plain loads.  Otherwise loads are clamped to the
    // last valid 16 bytes / row and the out-of-range part is replaced by zeros (selects, no branches).
    auto load_global = [&](uint32_t k0, auto full_tag) {
        constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
        for (int i = 0; i < T::kAChunks; ++i) {
            const uint32_t kk = k0 + (((tid + kThreads * i) & 7u) << 4);
            if constexpr (kFull) {
                areg[i] = *reinterpret_cast<const u32x4*>(aptr[i] + k0);
            } else {
                const bool ok = kk < k_end;
                u32x4 v = *reinterpret_cast<const u32x4*>(aptr[i] + (ok ? k0 : 0u));
                areg[i] = ok ? v : u32x4{0u, 0u, 0u, 0u};
            }
        }
        if constexpr (kTransB) {
#pragma unroll
            for (int i = 0; i < T::kBChunksT; ++i) {
                const uint32_t kk = k0 + (((tid + kThreads * i) & 7u) << 4);
                if constexpr (kFull) {
                    bregT[i] = *reinterpret_cast<const u32x4*>(bptrT[i] + k0);
                } else {
                    const bool ok = kk < k_end;
                    u32x4 v = *reinterpret_cast<const u32x4*>(bptrT[i] + (ok ? k0 : 0u));
                    bregT[i] = ok ? v : u32x4{0u, 0u, 0u, 0u};
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t kk = k0 + kb * 16u + i;
                bool ok = true;
                size_t roff = static_cast<size_t>(k0 + i) * N;
                if constexpr (!kFull) {
                    ok = kk < k_end;
                    roff = ok ? roff : 0;   // row kb*16 of the first step: always valid memory
                }
                const int8_t* src = bptr + roff;
                if constexpr (T::kCols == 8) {
                    u32x2 v = *reinterpret_cast<const u32x2*>(src);
                    breg[i][0] = ok ? v[0] : 0u;
                    breg[i][1] = ok ? v[1] : 0u;
                } else {
                    const uint32_t v = *reinterpret_cast<const uint32_t*>(src);
                    breg[i][0] = ok ? v : 0u;
                }
            }
        }
    };
    auto load_step = [&](uint32_t k0) {
        if (k0 + kBK <= k_end) {
            load_global(k0, std::true_type{});
        } else {
            load_global(k0, std::false_type{});
        }
    };

    auto store_lds = [&](char* stage) {
        char* As = stage;
        char* Bs = stage + T::kABytes;
#pragma unroll
        for (int i = 0; i < T::kAChunks; ++i) {
            const uint32_t c = tid + kThreads * i;
            *reinterpret_cast<u32x4*>(As + swz_off(c >> 3, c & 7u)) = areg[i];
        }
        if constexpr (kTransB) {
#pragma unroll
            for (int i = 0; i < T::kBChunksT; ++i) {
                const uint32_t c = tid + kThreads * i;
                *reinterpret_cast<u32x4*>(Bs + swz_off(c >> 3, c & 7u)) = bregT[i];
            }
        } else {
#pragma unroll
            for (int d = 0; d < T::kCols / 4; ++d) {
                uint32_t t[4][4];  // t[q][c]: rows 4q..4q+3 of column 4d+c
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    transpose4x4(breg[4 * q][d], breg[4 * q + 1][d], breg[4 * q + 2][d], breg[4 * q + 3][d],
                                 t[q][0], t[q][1], t[q][2], t[q][3]);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t col = nb * T::kCols + 4 * d + c;
                    *reinterpret_cast<u32x4*>(Bs + col * kBStride + (kb << 4)) =
                        u32x4{t[0][c], t[1][c], t[2][c], t[3][c]};
                }
            }
        }
    };

    // ---------------- accumulators
    constexpr int kWGN = T::kWGN;  // wavefront grid inside the tile
    constexpr int kWTM = T::kWTM;  // 32x32 blocks per wavefront along M / N
    constexpr int kWTN = T::kWTN;
    const uint32_t wm = wave / kWGN, wn = wave % kWGN;

    i32x16 acc[kWTM][kWTN];
#pragma unroll
    for (int i = 0; i < kWTM; ++i) {
#pragma unroll
        for (int j = 0; j < kWTN; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
        }
    }

    const uint32_t lrow = lane & 31u;
    const uint32_t lgrp = lane >> 5;

    auto compute = [&](const char* stage) {
        const char* As = stage;
        const char* Bs = stage + T::kABytes;
#pragma unroll
        for (int ks = 0; ks < kBK / 32; ++ks) {
            const uint32_t chunk = 2u * ks + lgrp;
            i32x4 af[kWTM], bf[kWTN];
#pragma unroll
            for (int i = 0; i < kWTM; ++i) {
                const uint32_t row = (wm * kWTM + i) * 32u + lrow;
                af[i] = *reinterpret_cast<const i32x4*>(As + swz_off(row, chunk));
            }
#pragma unroll
            for (int j = 0; j < kWTN; ++j) {
                const uint32_t col = (wn * kWTN + j) * 32u + lrow;
                if constexpr (kTransB) {
                    bf[j] = *reinterpret_cast<const i32x4*>(Bs + swz_off(col, chunk));
                } else {
                    bf[j] = *reinterpret_cast<const i32x4*>(Bs + col * kBStride + (chunk << 4));
                }
            }
#pragma unroll
            for (int i = 0; i < kWTM; ++i) {
#pragma unroll
                for (int j = 0; j < kWTN; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
                }
            }
        }
    };

    // ---------------- main loop
    const uint32_t steps = (k_end - k_begin + kBK - 1) / kBK;
    char* stage0 = smem;
    char* stage1 = smem + (T::kStages == 2 ? T::kStage : 0);
    load_step(k_begin);
    store_lds(stage0);
    __syncthreads();
    for (uint32_t t = 0; t < steps; ++t) {
        char* cur = (t & 1u) ? stage1 : stage0;
        char* nxt = (t & 1u) ? stage0 : stage1;
        const bool more = t + 1 < steps;
        if (more) {
            load_step(k_begin + (t + 1) * kBK);
        }
        compute(cur);
        if constexpr (T::kStages == 1) {
            __syncthreads();  // single LDS stage: every wavefront must have read it before it is overwritten
        }
        if (more) {
            store_lds(nxt);
        }
        __syncthreads();
    }

    // ---------------- epilogue (MFMA 32x32 layout: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, col l%32)
    ChannelQ qs[kWTN];
    float bias_post[kWTN];
    int32_t bias_pre[kWTN];
    uint32_t cols[kWTN];
#pragma unroll
    for (int j = 0; j < kWTN; ++j) {
        cols[j] = n0 + (wn * kWTN + j) * 32u + lrow;
        qs[j] = ChannelQ{1.0f, 0, 1};
        bias_post[j] = 0.0f;
        bias_pre[j] = 0;
        if constexpr (!kSplitK) {
            if (cols[j] < N) {
                qs[j] = load_channel_q(e, chan_off + cols[j]);
                bias_post[j] = load_bias_post(e, chan_off + cols[j]);
                if (e.bias_kind == ASCQ_MM_BIAS_I32_PRE) {
                    bias_pre[j] = static_cast<const int32_t*>(e.bias)[chan_off + cols[j]];
                }
            }
        }
    }
    auto run = [&](auto tag) {
        constexpr int kOut = decltype(tag)::value;
#pragma unroll
        for (int i = 0; i < kWTM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = row0 + (wm * kWTM + i) * 32u + 8u * (r >> 2) + 4u * lgrp + (r & 3);
                if (row < row_end) {
                    float tok = 1.0f;
                    if constexpr (!kSplitK) {
                        if (e.has_tok) {
                            tok = e.tok_scale[row];
                        }
                    }
#pragma unroll
                    for (int j = 0; j < kWTN; ++j) {
                        if (cols[j] < N) {
                            if constexpr (kSplitK) {
                                atomicAdd(p.partial + static_cast<size_t>(row) * N + cols[j], acc[i][j][r]);
                            } else {
                                epilogue_store<kOut>(e, row, cols[j], acc[i][j][r] + bias_pre[j], qs[j], tok,
                                                     bias_post[j]);
                            }
                        }
                    }
                }
            }
        }
    };
    if constexpr (kSplitK) {
        run(OutTag<-1>{});
    } else {
        dispatch_out(e, run);
    }
}

template <class T, bool kTransB, bool kSplitK>
__global__ __launch_bounds__(kThreads, T::kMinBlocks) void gemm_kernel(GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t t = xcd_remap(blockIdx.x, total);
    if (t >= total) {
        return;
    }
    const uint32_t tm = t % p.tiles_m, tn = t / p.tiles_m;
    uint32_t k_begin = 0, k_end = p.k;
    if constexpr (kSplitK) {
        k_begin = blockIdx.y * p.k_per_split;
        k_end = min(p.k, k_begin + p.k_per_split);
        if (k_begin >= k_end) {
            return;
        }
    }
    gemm_tile<T, kTransB, kSplitK>(p, p.a, p.b, p.epi, tm * T::BM, p.m, tn * T::BN, k_begin, k_end, 0, smem);
}

// Grouped: tile slot `ms` along M is resolved against the group list by every workgroup (groups is small).
template <class T>
__global__ __launch_bounds__(kThreads) void group_gemm_kernel(GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t t = xcd_remap(blockIdx.x, total);
    if (t >= total) {
        return;
    }
    const uint32_t ms = t % p.tiles_m, tn = t / p.tiles_m;
    // walk the groups: group g owns tile slots [slot, slot + ceil(cnt / BM))
    uint32_t slot = 0;
    int64_t off = 0;
    for (uint32_t g = 0; g < p.groups; ++g) {
        const int64_t v = p.group_list[g];
        const int64_t cnt = p.group_list_kind == ASCQ_GROUP_LIST_PREFIX_SUM ? v - off : v;
        if (cnt <= 0) {
            continue;
        }
        int64_t end = off + cnt;
        if (end > static_cast<int64_t>(p.m)) {
            end = p.m;
        }
        const uint32_t rows = end > off ? static_cast<uint32_t>(end - off) : 0u;
        const uint32_t tiles = (rows + T::BM - 1) / T::BM;
        if (ms < slot + tiles) {
            const uint32_t row0 = static_cast<uint32_t>(off) + (ms - slot) * T::BM;
            gemm_tile<T, false, false>(p, p.a, p.b + static_cast<size_t>(g) * p.k * p.n, p.epi, row0,
                                       static_cast<uint32_t>(end), tn * T::BN, 0, p.k, static_cast<size_t>(g) * p.n,
                                       smem);
            return;
        }
        slot += tiles;
        off += cnt;
    }
}

// Second pass of the split-K path: workspace int32 [m, n] -> output, and leaves the workspace zeroed.
__global__ __launch_bounds__(kThreads) void splitk_epilogue_kernel(GemmParams p)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * kThreads) {
        const size_t row = idx / p.n, col = idx % p.n;
        int32_t acc = p.partial[idx];
        p.partial[idx] = 0;
        if (p.epi.bias_kind == ASCQ_MM_BIAS_I32_PRE) {
            acc += static_cast<const int32_t*>(p.epi.bias)[col];
        }
        const ChannelQ q = load_channel_q(p.epi, col);
        const float tok = p.epi.has_tok ? p.epi.tok_scale[row] : 1.0f;
        const float bp = load_bias_post(p.epi, col);
        dispatch_out(p.epi, [&](auto tag) {
            epilogue_store<decltype(tag)::value>(p.epi, row, col, acc, q, tok, bp);
        });
    }
}

// Shapes the MFMA kernels do not take (odd sizes, unaligned pointers, transposed A): one lane per output.
__global__ __launch_bounds__(kThreads) void gemm_generic_kernel(GemmParams p, int trans_a, int trans_b)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * kThreads) {
        const size_t row = idx / p.n, col = idx % p.n;
        int32_t acc = 0;
        for (uint32_t kk = 0; kk < p.k; ++kk) {
            const int32_t av = trans_a ? p.a[static_cast<size_t>(kk) * p.m + row] : p.a[row * p.k + kk];
            const int32_t bv = trans_b ? p.b[col * p.k + kk] : p.b[static_cast<size_t>(kk) * p.n + col];
            acc += av * bv;
        }
        if (p.epi.bias_kind == ASCQ_MM_BIAS_I32_PRE) {
            acc += static_cast<const int32_t*>(p.epi.bias)[col];
        }
        const ChannelQ q = load_channel_q(p.epi, col);
        const float tok = p.epi.has_tok ? p.epi.tok_scale[row] : 1.0f;
        const float bp = load_bias_post(p.epi, col);
        dispatch_out(p.epi, [&](auto tag) {
            epilogue_store<decltype(tag)::value>(p.epi, row, col, acc, q, tok, bp);
        });
    }
}

typedef Tile<4, 4, 2, 2, false> TileL;   // 256 x 256
typedef Tile<4, 4, 2, 2, true> TileLT;
typedef Tile<2, 4, 2, 2, false> TileM;   // 128 x 256
typedef Tile<2, 4, 2, 2, true> TileMT;
typedef Tile<1, 2, 1, 4, false> TileS;   // 32 x 256, split-K
typedef Tile<1, 2, 1, 4, true> TileST;

template <class K>
int set_lds(K kernel, int bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       bytes);
    if (e != hipSuccess) {
        return fail(ASCQ_EHIP, "hipFuncSetAttribute(%d bytes of LDS): %s", bytes, hipGetErrorString(e));
    }
    return ASCQ_OK;
}

template <class T, bool kTransB, bool kSplitK>
int launch_gemm(GemmParams& p, hipStream_t st)
{
    p.tiles_m = (p.m + T::BM - 1) / T::BM;
    p.tiles_n = (p.n + T::BN - 1) / T::BN;
    auto kernel = gemm_kernel<T, kTransB, kSplitK>;
    const uint32_t total = p.tiles_m * p.tiles_n;
    dim3 grid((total + 7u) / 8u * 8u, kSplitK ? p.k_splits : 1u);
    if (plan_note(ASCQ_MM_KERNEL_STAGED, T::BM, T::BN, kBK, grid.x * grid.y, grid.y, T::kLds,
                  kSplitK ? static_cast<size_t>(p.m) * p.n * sizeof(int32_t) : 0)) {
        return ASCQ_OK;
    }
    int rc = set_lds(kernel, T::kLds);
    if (rc != ASCQ_OK) {
        return rc;
    }
    kernel<<<grid, kThreads, T::kLds, st>>>(p);
    return launch_status("ascq_matmul_w8a8");
}

int validate_mm(const ascq_matmul_desc* d, const char* who, const void* c, const void* a, const void* b,
                const void* bias, const void* qv, const void* tok)
{
    ASCQ_REQUIRE(c && a && b, ASCQ_ENULL, "%s: c / a / b is NULL", who);
    ASCQ_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0, ASCQ_EINVAL, "%s: m, n, k must be greater than 0", who);
    ASCQ_REQUIRE(d->quant_mode >= ASCQ_MM_QUANT_NONE && d->quant_mode <= ASCQ_MM_QUANT_VECTOR, ASCQ_EINVAL,
                 "%s: unknown quant mode %d", who, d->quant_mode);
    ASCQ_REQUIRE(d->scale_format == ASCQ_MM_SCALE_U64 || d->scale_format == ASCQ_MM_SCALE_F32, ASCQ_EINVAL,
                 "%s: unknown scale format %d", who, d->scale_format);
    ASCQ_REQUIRE(d->bias_kind >= ASCQ_MM_BIAS_NONE && d->bias_kind <= ASCQ_MM_BIAS_BF16_POST, ASCQ_EINVAL,
                 "%s: unknown bias kind %d", who, d->bias_kind);
    ASCQ_REQUIRE(d->activation >= ASCQ_MM_ACT_NONE && d->activation <= ASCQ_MM_ACT_SWIGLU, ASCQ_EINVAL,
                 "%s: unknown activation %d", who, d->activation);
    if (d->activation == ASCQ_MM_ACT_SWIGLU) {
        ASCQ_REQUIRE(d->n % 2 == 0, ASCQ_EINVAL, "%s: SwiGLU combines column pairs: n = %u must be even", who, d->n);
        ASCQ_REQUIRE(d->quant_mode != ASCQ_MM_QUANT_NONE &&
                         (d->out_dtype == ASCQ_F16 || d->out_dtype == ASCQ_BF16 || d->out_dtype == ASCQ_F32),
                     ASCQ_EUNSUPPORTED, "%s: SwiGLU needs a dequantising epilogue and a half / bfloat16 / float output", who);
        ASCQ_REQUIRE(d->act_beta == d->act_beta && d->act_beta - d->act_beta == 0.0f, ASCQ_EINVAL,
                     "%s: act_beta must be finite", who);
    }
    ASCQ_REQUIRE(d->b_format == ASCQ_MM_B_ND || d->b_format == ASCQ_MM_B_NZ, ASCQ_EINVAL, "%s: unknown B format %d",
                 who, d->b_format);
    if (d->b_format == ASCQ_MM_B_NZ) {
        ASCQ_REQUIRE(!d->trans_a && !d->trans_b, ASCQ_EUNSUPPORTED, "%s: fractal (NZ) B takes no transposition", who);
        ASCQ_REQUIRE(d->n % 32 == 0 && d->k % 128 == 0, ASCQ_EALIGN,
                     "%s: fractal (NZ) B needs n %% 32 == 0 and k %% 128 == 0 (n=%u, k=%u)", who, d->n, d->k);
        ASCQ_REQUIRE(static_cast<uint64_t>(d->k) * d->n < (1ull << 32), ASCQ_EUNSUPPORTED,
                     "%s: fractal (NZ) B is limited to k * n < 2^32", who);
        ASCQ_REQUIRE(aligned16(a) && aligned16(b), ASCQ_EALIGN, "%s: fractal (NZ) B needs 16-byte aligned a and b",
                     who);
    }
    if (d->quant_mode == ASCQ_MM_QUANT_NONE) {
        ASCQ_REQUIRE(d->out_dtype == ASCQ_I32, ASCQ_EUNSUPPORTED, "%s: without a quant mode the output is int32", who);
        ASCQ_REQUIRE(d->bias_kind <= ASCQ_MM_BIAS_I32_PRE && !d->has_tok_scale && d->activation == ASCQ_MM_ACT_NONE,
                     ASCQ_EUNSUPPORTED, "%s: int32 output takes no fp32 epilogue", who);
    } else {
        const int o = d->out_dtype;
        ASCQ_REQUIRE(o == ASCQ_F16 || o == ASCQ_BF16 || o == ASCQ_F32 || o == ASCQ_I8, ASCQ_EUNSUPPORTED,
                     "%s: output dtype %d is not half / bfloat16 / float / int8", who, o);
        ASCQ_REQUIRE(o != ASCQ_I8 || d->scale_format == ASCQ_MM_SCALE_U64, ASCQ_EUNSUPPORTED,
                     "%s: int8 output (requantisation) needs the uint64 quant parameter format", who);
        if (d->quant_mode == ASCQ_MM_QUANT_VECTOR) {
            ASCQ_REQUIRE(qv != nullptr, ASCQ_ENULL, "%s: quant vector is NULL", who);
        }
    }
    ASCQ_REQUIRE(d->bias_kind == ASCQ_MM_BIAS_NONE || bias != nullptr, ASCQ_ENULL, "%s: bias is NULL", who);
    ASCQ_REQUIRE(!d->has_tok_scale || tok != nullptr, ASCQ_ENULL, "%s: token scale is NULL", who);
    return ASCQ_OK;
}

EpiParams make_epi(const ascq_matmul_desc* d, void* c, const void* bias, const void* qv, const void* tok)
{
    // the SwiGLU epilogue writes one column per column pair
    const uint32_t ldc = d->activation == ASCQ_MM_ACT_SWIGLU && d->quant_mode != ASCQ_MM_QUANT_NONE ? d->n / 2u : d->n;
    return EpiParams{c, bias, qv, static_cast<const float*>(tok), ldc, d->out_dtype, d->quant_mode, d->scale_format,
                     d->bias_kind, d->has_tok_scale, d->activation, d->quant_scalar, d->act_beta};
}

bool fast_path_ok(const ascq_matmul_desc* d, const void* a, const void* b)
{
    if (d->trans_a || d->k % 16 != 0 || !aligned16(a)) {
        return false;
    }
    if (d->trans_b) {
        return aligned16(b);
    }
    return d->n % 8 == 0 && d->n >= 8 && (reinterpret_cast<uintptr_t>(b) & 7u) == 0;
}

// Up to this many rows the 128 x 128 direct-to-LDS kernel (K split over workgroups) is used when the shape allows.
constexpr uint32_t kSkinnyMaxM = 512;

// ascq_matmul_w8a8_packed between 129 and 512 rows: true when the 128 x 128 tiles (no K split: the call has no
// workspace) are expected to beat the weights-in-registers form.  Both estimates are fits to measurements at
// k = 4096, n = 11008 and k = 11008, n = 4096 (the crossovers there: 256 and about 380 rows).  Registers form: the
// weights once (5 us + 1 us per 4.7 MB), then 0.95 us per 16 rows and 4096 of k, per round of workgroups.  Tiles:
// 6.5 us per 1024 of k for up to one tile per compute unit, 1.45 times that with two (they share the unit), and in
// proportion beyond.  Above 512 rows the 256-row tiles always lead.
bool packed_tiles_faster(const GemmParams& p)
{
    const double kk = p.k / 4096.0;
    const double ws_us = 5.0 + static_cast<double>(p.n) * p.k / 4.7e6 +
                         0.95 * kk * ((p.m + 15u) / 16u) * gemm_ws_rounds(p);
    const double tiles = static_cast<double>((p.m + 127u) / 128u) * ((p.n + 127u) / 128u);
    const double cus = device_compute_units();
    const double load = tiles <= cus ? 1.0 : tiles <= 2.0 * cus ? 1.0 + 0.45 * (tiles - cus) / cus : 1.45 * tiles / (2.0 * cus);
    const double tiles_us = 4.0 + 26.0 * kk * load;
    return tiles_us < ws_us;
}
// Up to this many rows the weight-stream kernel is preferred over those tiles.
constexpr uint32_t kStreamMaxM = 8;

// split-K factor for the small-M kernel: enough workgroups to cover the chip ~3 times
uint32_t pick_k_splits(uint32_t n, uint32_t k)
{
    const uint32_t tiles = (n + 255u) / 256u;
    const uint32_t steps = (k + kBK - 1) / kBK;
    uint32_t s = (768u + tiles - 1) / tiles;
    if (s > steps) s = steps;
    if (s > 32u) s = 32u;
    return s ? s : 1u;
}

// SwiGLU for the shapes the large tile kernel does not take: the matmul leaves its int32 accumulators in the workspace
// ([m][n], pre-dequant bias included) and this kernel applies scale, token scale, bias and the activation to each
// column pair.  One lane = one pair.
__global__ __launch_bounds__(256) void swiglu_epilogue_kernel(GemmParams p)
{
    const EpiParams& e = p.epi;
    const size_t half_n = p.n / 2u, total = static_cast<size_t>(p.m) * half_n;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; i < total;
         i += static_cast<size_t>(gridDim.x) * 256u) {
        const size_t row = i / half_n, jp = i % half_n, col = 2u * jp;
        const int32_t a0 = p.partial[row * p.n + col], a1 = p.partial[row * p.n + col + 1u];
        const float tok = e.has_tok ? e.tok_scale[row] : 1.0f;
        const float v0 = epilogue_value(e, a0, load_channel_q(e, col), tok, load_bias_post(e, col));
        const float v1 = epilogue_value(e, a1, load_channel_q(e, col + 1u), tok, load_bias_post(e, col + 1u));
        store_float_out(e, row * e.ldc + jp, swiglu(v0, v1, e.act_beta));
    }
}

// True when the plain matmul of this descriptor runs on the large direct-to-LDS tile kernel, whose epilogue applies
// SwiGLU in registers (16-bit outputs).
bool swiglu_in_tile_kernel(const ascq_matmul_desc* d, const GemmParams& p, const void* a, const void* b)
{
    if (d->out_dtype != ASCQ_F16 && d->out_dtype != ASCQ_BF16) {
        return false;
    }
    if (d->m <= kSkinnyMaxM || !gemm_dma_supported(p)) {
        return false;
    }
    return d->b_format == ASCQ_MM_B_NZ || fast_path_ok(d, a, b);
}

// True when the plain matmul of this descriptor runs on the decode kernels for [n, k] weights (activations resident
// in LDS, or weights held in registers), whose epilogue pairs the columns of a row through neighbouring lanes.
bool swiglu_in_decode_kernel(const ascq_matmul_desc* d, const GemmParams& p, const void* a, const void* b)
{
    if (!d->trans_b || d->trans_a || d->b_format != ASCQ_MM_B_ND || !fast_path_ok(d, a, b)) {
        return false;
    }
    return (d->m <= gemm_packed_pass_rows(p) && gemm_packed_nk_supported(p)) || gemm_ws_supported(p, true);
}

inline size_t round256(size_t v) { return (v + 255u) & ~static_cast<size_t>(255u); }

// the matmul that leaves raw accumulators: same operands, no quantisation, at most the pre-dequant bias
ascq_matmul_desc raw_accumulator_desc(const ascq_matmul_desc* d)
{
    ascq_matmul_desc r = *d;
    r.quant_mode = ASCQ_MM_QUANT_NONE;
    r.out_dtype = ASCQ_I32;
    r.activation = ASCQ_MM_ACT_NONE;
    r.has_tok_scale = 0;
    r.bias_kind = d->bias_kind == ASCQ_MM_BIAS_I32_PRE ? ASCQ_MM_BIAS_I32_PRE : ASCQ_MM_BIAS_NONE;
    return r;
}

}  // namespace
}  // namespace ascq

using namespace ascq;

extern "C" int ascq_matmul_w8a8_workspace_size(const ascq_matmul_desc* d, size_t* bytes)
{
    ASCQ_REQUIRE(d != nullptr && bytes != nullptr, ASCQ_ENULL, "ascq_matmul_w8a8_workspace_size: NULL argument");
    *bytes = 0;
    // The size is that for operands aligned to 16 bytes; it cannot see the pointers.  (A SwiGLU call whose misaligned
    // operands keep it off the tile kernel names the size it needs in its error.)
    GemmParams shape{};
    shape.a = shape.b = reinterpret_cast<const int8_t*>(uintptr_t{16});
    shape.m = d->m;
    shape.n = d->n;
    shape.k = d->k;
    if (d->activation == ASCQ_MM_ACT_SWIGLU && d->quant_mode != ASCQ_MM_QUANT_NONE &&
        !swiglu_in_tile_kernel(d, shape, shape.a, shape.b) && !swiglu_in_decode_kernel(d, shape, shape.a, shape.b)) {
        // Shapes outside the large tile kernel keep their int32 accumulators [m][n] in the workspace, behind the
        // scratch of the matmul that produces them.
        const ascq_matmul_desc r = raw_accumulator_desc(d);
        size_t inner = 0;
        const int rc = ascq_matmul_w8a8_workspace_size(&r, &inner);
        if (rc != ASCQ_OK) {
            return rc;
        }
        *bytes = round256(inner) + static_cast<size_t>(d->m) * d->n * sizeof(int32_t);
        return ASCQ_OK;
    }
    // [n, k] weights held in registers (17 to 224 rows at k up to 4096, fewer at longer k): no scratch
    const bool ws_nk = d->trans_b && !d->trans_a && d->b_format == ASCQ_MM_B_ND && gemm_ws_supported(shape, true);
    if (ws_nk) {
        return ASCQ_OK;
    }
    if (d->m <= 32 && !d->trans_a && pick_k_splits(d->n, d->k) > 1 && !(d->trans_b && d->k % 128 == 0)) {
        // (few rows on [n, k] weights with k % 128 == 0 run the whole-column kernel, which needs none)
        *bytes = static_cast<size_t>(d->m) * d->n * sizeof(int32_t);
    }
    if (d->m <= kSkinnyMaxM && !d->trans_a && d->k % 128 == 0 && d->n % 16 == 0 && !(d->m <= 32 && d->trans_b)) {
        const size_t need =
            static_cast<size_t>(gemm_dma_skinny_splits(d->m, d->n, d->k)) * d->m * d->n * sizeof(int32_t);
        if (need > *bytes && need > static_cast<size_t>(d->m) * d->n * sizeof(int32_t)) {
            *bytes = need;
        }
    }
    if (!d->trans_a && !d->trans_b && d->n % 16 == 0) {
        const size_t need = gemm_stream_workspace(d->m, d->n, d->k);
        if (need > *bytes) {
            *bytes = need;
        }
    }
    return ASCQ_OK;
}

// ref: include/adv_api/matmul/matmul.h:175-185 (SetQuantScalar / SetQuantVector), IterateAll: matmul_impl.h:65-92
extern "C" int ascq_matmul_w8a8(const ascq_matmul_desc* d, void* c, const void* a, const void* b, const void* bias,
                                const void* quant_vector, const void* tok_scale, void* workspace,
                                size_t workspace_bytes, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w8a8: desc is NULL");
    int rc = validate_mm(d, "ascq_matmul_w8a8", c, a, b, bias, quant_vector, tok_scale);
    if (rc != ASCQ_OK) {
        return rc;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    GemmParams p{};
    p.a = static_cast<const int8_t*>(a);
    p.b = static_cast<const int8_t*>(b);
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.epi = make_epi(d, c, bias, quant_vector, tok_scale);
    if (d->activation == ASCQ_MM_ACT_SWIGLU && !swiglu_in_tile_kernel(d, p, a, b) && !swiglu_in_decode_kernel(d, p, a, b)) {
        // raw accumulators into the workspace, then the pairwise epilogue
        const ascq_matmul_desc r = raw_accumulator_desc(d);
        size_t inner = 0;
        rc = ascq_matmul_w8a8_workspace_size(&r, &inner);
        if (rc != ASCQ_OK) {
            return rc;
        }
        inner = round256(inner);
        const size_t need = inner + static_cast<size_t>(d->m) * d->n * sizeof(int32_t);
        ASCQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, ASCQ_EINVAL,
                     "ascq_matmul_w8a8: SwiGLU at this shape needs a workspace of %zu bytes (see "
                     "ascq_matmul_w8a8_workspace_size)", need);
        ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_matmul_w8a8: workspace must be 16-byte aligned");
        p.partial = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + inner);
        rc = ascq_matmul_w8a8(&r, p.partial, a, b, r.bias_kind == ASCQ_MM_BIAS_I32_PRE ? bias : nullptr, nullptr, nullptr,
                              inner ? workspace : nullptr, inner, stream);
        if (rc != ASCQ_OK) {
            return rc;
        }
        const size_t pairs = static_cast<size_t>(d->m) * (d->n / 2u);
        size_t blocks = (pairs + 255u) / 256u;
        if (blocks > 8192) blocks = 8192;
        if (plan_note(0, 0, 0, 0, 0, 0, 0, 0)) {  // the pairwise epilogue kernel
            return ASCQ_OK;
        }
        swiglu_epilogue_kernel<<<static_cast<uint32_t>(blocks), 256, 0, st>>>(p);
        return launch_status("ascq_matmul_w8a8 (SwiGLU epilogue)");
    }
    if (d->b_format == ASCQ_MM_B_NZ) {
        // only the direct-to-LDS tile kernels address the fractal layout; validate_mm has checked what they need
        p.b_nz = 1;
        return d->m <= kSkinnyMaxM ? launch_gemm_dma_skinny(p, workspace, workspace_bytes, st)
                                   : launch_gemm_dma(p, false, st);
    }
    if (!fast_path_ok(d, a, b)) {
        size_t total = static_cast<size_t>(d->m) * d->n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        if (plan_note(ASCQ_MM_KERNEL_GENERIC, 1, 1, 1, static_cast<uint32_t>(blocks), 1, 0, 0)) {
            return ASCQ_OK;
        }
        gemm_generic_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p, d->trans_a, d->trans_b);
        return launch_status("ascq_matmul_w8a8 (generic)");
    }
    // Up to 8 rows the weight streams; from 9 rows on the split-K tiles below are faster when the shape allows them
    // (k = 4096, n = 11008: 16.8-17.9 against 17.3-17.6 us up to 8 rows, 18.9 / 23.1 against 17.0 / 17.5 us at 16 / 32)
    const bool tiles_instead = d->m > kStreamMaxM && gemm_dma_supported(p) && workspace != nullptr &&
                               aligned16(workspace) &&
                               workspace_bytes >= static_cast<size_t>(gemm_dma_skinny_splits(d->m, d->n, d->k)) * d->m * d->n * sizeof(int32_t);
    if (!tiles_instead && !d->trans_b && gemm_stream_supported(p) && workspace != nullptr && aligned16(workspace) &&
        workspace_bytes >= gemm_stream_workspace(d->m, d->n, d->k)) {
        return launch_gemm_stream(p, workspace, st);
    }
    if (d->trans_b && !d->trans_a && gemm_ws_supported(p, true)) {
        return launch_gemm_ws(p, st, true);  // the weights held in registers, the activations streamed
    }
    if (d->m <= gemm_packed_pass_rows(p) && d->trans_b && !d->trans_a && gemm_packed_nk_supported(p)) {
        return launch_gemm_packed(p, st, true);  // activations resident in LDS, nothing but weights in the load queue
    }
    if (d->m <= 32 && d->trans_b && !d->trans_a && gemm_nk_supported(p)) {
        return launch_gemm_nk(p, st);
    }
    if (d->m <= kSkinnyMaxM && !d->trans_a && gemm_dma_supported(p)) {
        return launch_gemm_dma_skinny(p, workspace, workspace_bytes, st, d->trans_b != 0);
    }
    if (d->m <= 32) {
        const uint32_t splits = pick_k_splits(d->n, d->k);
        size_t need = static_cast<size_t>(d->m) * d->n * sizeof(int32_t);
        if (splits > 1 && workspace != nullptr && workspace_bytes >= need &&
            (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0) {
            p.k_splits = splits;
            const uint32_t steps = (d->k + kBK - 1) / kBK;
            p.k_per_split = (steps + splits - 1) / splits * kBK;
            p.partial = static_cast<int32_t*>(workspace);
            if (!plan_recording()) {
                rc = ascq_zero_fill(workspace, need, stream);
                if (rc != ASCQ_OK) {
                    return rc;
                }
            }
            rc = d->trans_b ? launch_gemm<TileST, true, true>(p, st) : launch_gemm<TileS, false, true>(p, st);
            if (rc != ASCQ_OK) {
                return rc;
            }
            if (plan_note(0, 0, 0, 0, 0, 0, 0, 0)) {   // the zero fill ...
                plan_note(0, 0, 0, 0, 0, 0, 0, 0);     // ... and the epilogue kernel
                return ASCQ_OK;
            }
            size_t total = static_cast<size_t>(d->m) * d->n;
            size_t blocks = (total + kThreads - 1) / kThreads;
            if (blocks > 4096) blocks = 4096;
            splitk_epilogue_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
            return launch_status("ascq_matmul_w8a8 (split-K epilogue)");
        }
        return d->trans_b ? launch_gemm<TileST, true, false>(p, st) : launch_gemm<TileS, false, false>(p, st);
    }
    if (d->m > 128 && !d->trans_b && gemm_dma_supported(p)) {
        return launch_gemm_dma(p, false, st);
    }
    if (d->m > 512 && d->trans_b && !d->trans_a && gemm_dma_supported(p)) {
        return launch_gemm_dma(p, false, st, true);  // B as [n][k]: its tiles are staged and read like A's
    }
    if (d->m <= 1024) {
        return d->trans_b ? launch_gemm<TileMT, true, false>(p, st) : launch_gemm<TileM, false, false>(p, st);
    }
    return d->trans_b ? launch_gemm<TileLT, true, false>(p, st) : launch_gemm<TileL, false, false>(p, st);
}

// ref: include/adv_api/matmul/matmul.h:175-185 (the same Matmul with SetQuantScalar / SetQuantVector); the weights in the
// layout of ascq_pack_weight_w8, the counterpart of the packing the reference does offline for its own L1 / L0 layout
// (examples/.../quant_group_matmul_high_performance/scripts/gen_data.py:62-64)
extern "C" int ascq_matmul_w8a8_packed(const ascq_matmul_desc* d, void* c, const void* a, const void* w_packed,
                                       const void* bias, const void* quant_vector, const void* tok_scale, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w8a8_packed: desc is NULL");
    int rc = validate_mm(d, "ascq_matmul_w8a8_packed", c, a, w_packed, bias, quant_vector, tok_scale);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(!d->trans_a && d->b_format == ASCQ_MM_B_ND, ASCQ_EUNSUPPORTED,
                 "ascq_matmul_w8a8_packed: a is [m, k] and the weights are in the packed layout (no trans_a, no NZ)");
    GemmParams p{};
    p.a = static_cast<const int8_t*>(a);
    p.b = static_cast<const int8_t*>(w_packed);
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.epi = make_epi(d, c, bias, quant_vector, tok_scale);
    ASCQ_REQUIRE(d->k % 64u == 0, ASCQ_EUNSUPPORTED, "ascq_matmul_w8a8_packed: k = %u must be a multiple of 64", d->k);
    ASCQ_REQUIRE(aligned16(a) && aligned16(w_packed), ASCQ_EALIGN, "ascq_matmul_w8a8_packed: a and w_packed must be 16-byte aligned");
    ASCQ_REQUIRE(gemm_packed_supported(p), ASCQ_EUNSUPPORTED, "ascq_matmul_w8a8_packed: the packed weights must stay below 2 GiB");
    // Many rows: the direct-to-LDS tile kernels read the packed tiles as they lie (one tile per load instruction), so a
    // caller that packed its weights for decode needs no second copy of them for prefill.  (SwiGLU in those kernels'
    // epilogue exists for 16-bit outputs.)
    const bool tiles_ok = gemm_dma_supported(p) &&
                          (d->activation != ASCQ_MM_ACT_SWIGLU || d->out_dtype == ASCQ_F16 || d->out_dtype == ASCQ_BF16);
    if (tiles_ok && (d->m > kSkinnyMaxM || (d->m > 128u && packed_tiles_faster(p)))) {
        return d->m <= kSkinnyMaxM ? launch_gemm_dma_skinny(p, nullptr, 0, static_cast<hipStream_t>(stream), 2)
                                   : launch_gemm_dma(p, false, static_cast<hipStream_t>(stream), 2);
    }
    if (gemm_ws_supported(p, false)) {
        return launch_gemm_ws(p, static_cast<hipStream_t>(stream), false);
    }
    return launch_gemm_packed(p, static_cast<hipStream_t>(stream));
}

// ref: include/adv_api/matmul/matmul_tilingdata.h:21-72 (TCubeTiling, the reference's host-side plan of a matmul)
extern "C" int ascq_matmul_w8a8_plan(const ascq_matmul_desc* d, const void* c, const void* a, const void* b,
                                     const void* bias, const void* quant_vector, const void* tok_scale,
                                     const void* workspace, size_t workspace_bytes, ascq_matmul_plan* plan)
{
    ASCQ_REQUIRE(plan != nullptr, ASCQ_ENULL, "ascq_matmul_w8a8_plan: plan is NULL");
    // the call itself, with every launch site describing its launch instead of making it
    plan_begin(plan);
    const int rc = ascq_matmul_w8a8(d, const_cast<void*>(c), a, b, bias, quant_vector, tok_scale,
                                    const_cast<void*>(workspace), workspace_bytes, nullptr);
    plan_end();
    return rc;
}

// ---------------------------------------------------------------------------- fused dynamic quantisation + matmul
extern "C" int ascq_linear_w8a8_dynamic_workspace_size(const ascq_matmul_desc* d, size_t* bytes)
{
    ASCQ_REQUIRE(d != nullptr && bytes != nullptr, ASCQ_ENULL, "ascq_linear_w8a8_dynamic_workspace_size: NULL argument");
    size_t mm = 0;
    ascq_matmul_desc dd = *d;
    dd.has_tok_scale = 1;
    int rc = ascq_matmul_w8a8_workspace_size(&dd, &mm);
    if (rc != ASCQ_OK) {
        return rc;
    }
    // q [m, k] int8, token scales [m], then the matmul's own scratch
    *bytes = round256(static_cast<size_t>(d->m) * d->k) + round256(static_cast<size_t>(d->m) * sizeof(float)) + mm;
    return ASCQ_OK;
}

// The activation quantiser of a W8A8 linear and the matmul in one call: q, tok = dynamic per-token quantisation of x
// (ascq_dynamic_quant_per_token), c = matmul(q, b) with the token scales in the epilogue; q and tok live in the
// caller's workspace.  Up to 8 rows of half / bfloat16 x on weights kept as [n, k] run as one launch instead: the
// decode kernel quantises x inside every workgroup on its way into LDS (gemm_packed_dyn_kernel; the same bits, about
// 12 us against 15.5 us per step at k = 4096, n = 11008 and one row, 15.4 against 15.8 us at 8; from 9 rows on the 256
// redundant quantisations cost more than the separate kernel's launch).  The reference composes this
// from ReduceMax / AscendQuant PER_TOKEN and Matmul (impl/adv_api/detail/quantization/quant/
// ascend_quant_per_group_3510_impl.h:142-178, include/adv_api/matmul/matmul.h:175-185).
extern "C" int ascq_linear_w8a8_dynamic(const ascq_matmul_desc* d, int32_t x_dtype, void* c, const void* x,
                                        const void* b, const void* bias, const void* quant_vector, void* workspace,
                                        size_t workspace_bytes, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_linear_w8a8_dynamic: desc is NULL");
    ASCQ_REQUIRE(x_dtype == ASCQ_F16 || x_dtype == ASCQ_BF16 || x_dtype == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_linear_w8a8_dynamic: x dtype %d is not half / bfloat16 / float", x_dtype);
    ASCQ_REQUIRE(!d->trans_a, ASCQ_EUNSUPPORTED, "ascq_linear_w8a8_dynamic: x is [m, k] row-major");
    ASCQ_REQUIRE(d->quant_mode != ASCQ_MM_QUANT_NONE && d->out_dtype != ASCQ_I8, ASCQ_EUNSUPPORTED,
                 "ascq_linear_w8a8_dynamic: the token scales need a floating-point dequantising epilogue");
    ascq_matmul_desc dd = *d;
    dd.has_tok_scale = 1;
    ASCQ_REQUIRE(workspace != nullptr, ASCQ_ENULL, "ascq_linear_w8a8_dynamic: workspace is NULL");
    ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_linear_w8a8_dynamic: workspace must be 16-byte aligned");
    size_t need = 0;
    int rc = ascq_linear_w8a8_dynamic_workspace_size(d, &need);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_linear_w8a8_dynamic: workspace of %zu bytes required (see ascq_linear_w8a8_dynamic_workspace_size)",
                 need);
    char* ws = static_cast<char*>(workspace);
    // validate with a stand-in for the quantised activations (the checks only look at NULL-ness)
    rc = validate_mm(&dd, "ascq_linear_w8a8_dynamic", c, x, b, bias, quant_vector, ws);
    if (rc != ASCQ_OK) {
        return rc;
    }
    if ((x_dtype == ASCQ_F16 || x_dtype == ASCQ_BF16) && d->trans_b && d->b_format == ASCQ_MM_B_ND && aligned16(x) &&
        gemm_packed_dyn_fits(d->m, d->k, true)) {
        // decode on [n, k] weights: the quantisation happens inside the weight-streaming kernel (same bits, one launch)
        GemmParams p{};
        p.a = static_cast<const int8_t*>(x);  // only its alignment is looked at
        p.b = static_cast<const int8_t*>(b);
        p.m = d->m;
        p.n = d->n;
        p.k = d->k;
        p.epi = make_epi(&dd, c, bias, quant_vector, reinterpret_cast<const float*>(ws));
        if (gemm_packed_nk_supported(p)) {
            return launch_gemm_packed_dyn(p, x, x_dtype == ASCQ_BF16, static_cast<hipStream_t>(stream), true);
        }
    }
    int8_t* q = reinterpret_cast<int8_t*>(ws);
    float* tok = reinterpret_cast<float*>(ws + round256(static_cast<size_t>(d->m) * d->k));
    char* rest = reinterpret_cast<char*>(tok) + round256(static_cast<size_t>(d->m) * sizeof(float));
    rc = ascq_dynamic_quant_per_token(x_dtype, d->m, d->k, q, tok, x, stream);
    if (rc != ASCQ_OK) {
        return rc;
    }
    return ascq_matmul_w8a8(&dd, c, q, b, bias, quant_vector, tok, rest,
                            workspace_bytes - static_cast<size_t>(rest - ws), stream);
}

// The same linear on weights packed by ascq_pack_weight_w8: up to 8 rows of half / bfloat16 x are one launch of the
// packed decode kernel with the quantiser inside; anything else is the quantiser kernel followed by
// ascq_matmul_w8a8_packed, with q and the token scales in the workspace.  The results are those of
// ascq_linear_w8a8_dynamic on the unpacked weights, bit for bit.
extern "C" int ascq_linear_w8a8_dynamic_packed(const ascq_matmul_desc* d, int32_t x_dtype, void* c, const void* x,
                                               const void* w_packed, const void* bias, const void* quant_vector,
                                               void* workspace, size_t workspace_bytes, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_linear_w8a8_dynamic_packed: desc is NULL");
    ASCQ_REQUIRE(x_dtype == ASCQ_F16 || x_dtype == ASCQ_BF16 || x_dtype == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_linear_w8a8_dynamic_packed: x dtype %d is not half / bfloat16 / float", x_dtype);
    ASCQ_REQUIRE(d->quant_mode != ASCQ_MM_QUANT_NONE && d->out_dtype != ASCQ_I8, ASCQ_EUNSUPPORTED,
                 "ascq_linear_w8a8_dynamic_packed: the token scales need a floating-point dequantising epilogue");
    ASCQ_REQUIRE(!d->trans_a && d->b_format == ASCQ_MM_B_ND, ASCQ_EUNSUPPORTED,
                 "ascq_linear_w8a8_dynamic_packed: x is [m, k] and the weights are in the packed layout (no trans_a, no NZ)");
    ASCQ_REQUIRE(d->k % 64u == 0, ASCQ_EUNSUPPORTED, "ascq_linear_w8a8_dynamic_packed: k = %u must be a multiple of 64", d->k);
    ascq_matmul_desc dd = *d;
    dd.has_tok_scale = 1;
    dd.trans_b = 0;
    ASCQ_REQUIRE(workspace != nullptr, ASCQ_ENULL, "ascq_linear_w8a8_dynamic_packed: workspace is NULL");
    ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_linear_w8a8_dynamic_packed: workspace must be 16-byte aligned");
    const size_t q_bytes = round256(static_cast<size_t>(d->m) * d->k);
    const size_t need = q_bytes + round256(static_cast<size_t>(d->m) * sizeof(float));
    ASCQ_REQUIRE(workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_linear_w8a8_dynamic_packed: workspace of %zu bytes required (ascq_linear_w8a8_dynamic_workspace_size "
                 "covers it)", need);
    char* ws = static_cast<char*>(workspace);
    int rc = validate_mm(&dd, "ascq_linear_w8a8_dynamic_packed", c, x, w_packed, bias, quant_vector, ws);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(aligned16(w_packed), ASCQ_EALIGN, "ascq_linear_w8a8_dynamic_packed: w_packed must be 16-byte aligned");
    if ((x_dtype == ASCQ_F16 || x_dtype == ASCQ_BF16) && aligned16(x) && gemm_packed_dyn_fits(d->m, d->k, false)) {
        GemmParams p{};
        p.a = static_cast<const int8_t*>(x);  // only its alignment is looked at
        p.b = static_cast<const int8_t*>(w_packed);
        p.m = d->m;
        p.n = d->n;
        p.k = d->k;
        p.epi = make_epi(&dd, c, bias, quant_vector, reinterpret_cast<const float*>(ws));
        ASCQ_REQUIRE(gemm_packed_supported(p), ASCQ_EUNSUPPORTED,
                     "ascq_linear_w8a8_dynamic_packed: the packed weights must stay below 2 GiB");
        return launch_gemm_packed_dyn(p, x, x_dtype == ASCQ_BF16, static_cast<hipStream_t>(stream), false);
    }
    int8_t* q = reinterpret_cast<int8_t*>(ws);
    float* tok = reinterpret_cast<float*>(ws + q_bytes);
    rc = ascq_dynamic_quant_per_token(x_dtype, d->m, d->k, q, tok, x, stream);
    if (rc != ASCQ_OK) {
        return rc;
    }
    return ascq_matmul_w8a8_packed(&dd, c, q, w_packed, bias, quant_vector, tok, stream);
}

// ------------------------------------------------------------------------------- the same call without a workspace
// For callers that cannot allocate (code under stream capture, serving loops, harnesses that forbid hipMalloc): the
// scratch of ascq_linear_w8a8_dynamic (quantised activations, token scales, partial sums of the small-m kernels) lives
// in a device array that is part of this library's code object.  Each GPU the library runs on holds its own copy at
// its own address until the process ends; the address is looked up once per device.  The array keeps the last call's
// contents, which is harmless: every kernel writes what it later reads (nothing is expected to start at zero).
namespace {
constexpr size_t kStaticScratchBytes = ASCQ_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device (in host code the array's name is only a handle for the lookup).
static int static_scratch(void** out)
{
    static std::mutex lock;
    static void* address[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    ASCQ_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, ASCQ_EHIP,
                 "ascq_linear_w8a8_dynamic_noalloc: hipGetDevice failed or device index %d is not below %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> guard(lock);
    if (address[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        ASCQ_REQUIRE(e == hipSuccess && ptr != nullptr, ASCQ_EHIP,
                     "ascq_linear_w8a8_dynamic_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        address[dev] = ptr;
    }
    *out = address[dev];
    return ASCQ_OK;
}

// No counterpart in the reference (its operators take a sharedTmpBuffer or pop one from the TPipe): this entry point
// exists for callers that cannot allocate device memory.
extern "C" int ascq_linear_w8a8_dynamic_noalloc(const ascq_matmul_desc* d, int32_t x_dtype, void* c, const void* x,
                                                const void* b, const void* bias, const void* quant_vector, void* stream)
{
    size_t need = 0;
    int rc = ascq_linear_w8a8_dynamic_workspace_size(d, &need);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(need <= kStaticScratchBytes, ASCQ_EINVAL,
                 "ascq_linear_w8a8_dynamic_noalloc: this shape needs %zu bytes of scratch, the built-in buffer holds %zu "
                 "(use ascq_linear_w8a8_dynamic with a workspace)", need, kStaticScratchBytes);
    void* ptr = nullptr;
    rc = static_scratch(&ptr);
    if (rc != ASCQ_OK) {
        return rc;
    }
    return ascq_linear_w8a8_dynamic(d, x_dtype, c, x, b, bias, quant_vector, ptr, kStaticScratchBytes, stream);
}

// ------------------------------------------------------------------------------------------ int4 x int4 matmul
namespace {
// 16 source bytes (32 nibbles, even element in the low nibble) -> 32 sign-extended int8 per lane and step
__global__ __launch_bounds__(256) void unpack_i4_kernel(uint8_t* dst, const uint8_t* src, size_t bytes)
{
    const size_t quads = bytes / 16u;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; i < quads;
         i += static_cast<size_t>(gridDim.x) * 256u) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(src + i * 16u);
        u32x4 lo8, hi8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // per byte: nibble u -> ((u ^ 8) | 0x80) - 8 has no borrow between bytes, and flipping bit 7 afterwards
            // leaves the two's complement value of the nibble
            const uint32_t lo = ((((w[j] & 0x0F0F0F0Fu) ^ 0x08080808u) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
            const uint32_t hi = (((((w[j] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
            const uint32_t e0123 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
            const uint32_t e4567 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
            if (j < 2) {
                lo8[2 * j] = e0123;
                lo8[2 * j + 1] = e4567;
            } else {
                hi8[2 * (j - 2)] = e0123;
                hi8[2 * (j - 2) + 1] = e4567;
            }
        }
        *reinterpret_cast<u32x4*>(dst + i * 32u) = lo8;
        *reinterpret_cast<u32x4*>(dst + i * 32u + 16u) = hi8;
    }
    // the last bytes of a buffer that is not a multiple of 16 bytes
    const size_t tail = quads * 16u;
    for (size_t i = tail + static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; i < bytes;
         i += static_cast<size_t>(gridDim.x) * 256u) {
        const uint32_t b = src[i];
        dst[2u * i] = static_cast<uint8_t>(static_cast<int>((b & 15u) ^ 8u) - 8);
        dst[2u * i + 1u] = static_cast<uint8_t>(static_cast<int>((b >> 4) ^ 8u) - 8);
    }
}
}  // namespace

// ref: AscendC::int4b_t tensors are two values per byte, even element in the low nibble
// (examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_int4/scripts/gen_data.py:32-42)
extern "C" int ascq_unpack_int4(void* dst, const void* src, size_t elements, void* stream)
{
    ASCQ_REQUIRE(elements == 0 || (dst && src), ASCQ_ENULL, "ascq_unpack_int4: dst / src is NULL");
    ASCQ_REQUIRE(elements % 2 == 0, ASCQ_EINVAL, "ascq_unpack_int4: an even number of int4 elements is required");
    ASCQ_REQUIRE(aligned16(dst) && aligned16(src), ASCQ_EALIGN, "ascq_unpack_int4: dst and src must be 16-byte aligned");
    if (elements == 0) {
        return ASCQ_OK;
    }
    const size_t bytes = elements / 2u;
    size_t blocks = (bytes / 16u + 255u) / 256u;
    blocks = blocks < 1u ? 1u : (blocks > 8192u ? 8192u : blocks);
    unpack_i4_kernel<<<static_cast<uint32_t>(blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), bytes);
    return launch_status("ascq_unpack_int4");
}

static int validate_w4a4(const ascq_matmul_desc* d)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w4a4: desc is NULL");
    // README of the reference example: "When the left matrix A is of int4 data type, transpose is not supported."
    ASCQ_REQUIRE(!d->trans_a, ASCQ_EUNSUPPORTED, "ascq_matmul_w4a4: an int4 A cannot be transposed");
    ASCQ_REQUIRE(d->b_format == ASCQ_MM_B_ND, ASCQ_EUNSUPPORTED, "ascq_matmul_w4a4: int4 B is row-major (ND) only");
    ASCQ_REQUIRE(d->k % 2 == 0, ASCQ_EINVAL, "ascq_matmul_w4a4: k %u must be even (two int4 per byte)", d->k);
    ASCQ_REQUIRE(d->trans_b || d->n % 2 == 0, ASCQ_EINVAL, "ascq_matmul_w4a4: n %u must be even (two int4 per byte)",
                 d->n);
    return ASCQ_OK;
}

extern "C" int ascq_matmul_w4a4_workspace_size(const ascq_matmul_desc* d, size_t* bytes)
{
    int rc = validate_w4a4(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_matmul_w4a4_workspace_size: bytes is NULL");
    size_t mm = 0;
    rc = ascq_matmul_w8a8_workspace_size(d, &mm);
    if (rc != ASCQ_OK) {
        return rc;
    }
    // A and B as int8, then the int8 matmul's own scratch
    *bytes = round256(static_cast<size_t>(d->m) * d->k) + round256(static_cast<size_t>(d->k) * d->n) + mm;
    return ASCQ_OK;
}

// Matmul<int4b_t, int4b_t, C>: both operands are widened to int8 in the caller's workspace (exact) and the int8
// matmul with its epilogues does the rest.  The matrix core of this GPU has no int4 operand format, so the widening is
// what any kernel would do on the way into the MFMA; weights that are used more than once can be widened once with
// ascq_unpack_int4 and given to ascq_matmul_w8a8.
// ref: examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_int4/matmul_int4.asc:52-58, 155
extern "C" int ascq_matmul_w4a4(const ascq_matmul_desc* d, void* c, const void* a, const void* b, const void* bias,
                                const void* quant_vector, const void* tok_scale, void* workspace,
                                size_t workspace_bytes, void* stream)
{
    int rc = validate_w4a4(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    rc = validate_mm(d, "ascq_matmul_w4a4", c, a, b, bias, quant_vector, tok_scale);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(workspace != nullptr, ASCQ_ENULL, "ascq_matmul_w4a4: workspace is NULL");
    ASCQ_REQUIRE(aligned16(workspace) && aligned16(a) && aligned16(b), ASCQ_EALIGN,
                 "ascq_matmul_w4a4: a, b and workspace must be 16-byte aligned");
    size_t need = 0;
    rc = ascq_matmul_w4a4_workspace_size(d, &need);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_matmul_w4a4: workspace of %zu bytes required (see ascq_matmul_w4a4_workspace_size)", need);
    char* ws = static_cast<char*>(workspace);
    char* a8 = ws;
    char* b8 = a8 + round256(static_cast<size_t>(d->m) * d->k);
    char* rest = b8 + round256(static_cast<size_t>(d->k) * d->n);
    rc = ascq_unpack_int4(a8, a, static_cast<size_t>(d->m) * d->k, stream);
    if (rc != ASCQ_OK) {
        return rc;
    }
    rc = ascq_unpack_int4(b8, b, static_cast<size_t>(d->k) * d->n, stream);
    if (rc != ASCQ_OK) {
        return rc;
    }
    return ascq_matmul_w8a8(d, c, a8, b8, bias, quant_vector, tok_scale, rest,
                            workspace_bytes - static_cast<size_t>(rest - ws), stream);
}

// ref: examples/.../quant_group_matmul_high_performance/quant_group_matmul_custom.asc:255-454
extern "C" int ascq_group_matmul_w8a8(const ascq_group_matmul_desc* g, void* y, const void* x, const void* w,
                                      const void* bias, const void* scale, const void* tok_scale,
                                      const int64_t* group_list, void* stream)
{
    ASCQ_REQUIRE(g != nullptr, ASCQ_ENULL, "ascq_group_matmul_w8a8: desc is NULL");
    const ascq_matmul_desc* d = &g->mm;
    int rc = validate_mm(d, "ascq_group_matmul_w8a8", y, x, w, bias, scale, tok_scale);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(group_list != nullptr, ASCQ_ENULL, "ascq_group_matmul_w8a8: group list is NULL");
    ASCQ_REQUIRE(g->groups > 0, ASCQ_EINVAL, "ascq_group_matmul_w8a8: groups must be greater than 0");
    ASCQ_REQUIRE(g->group_list_kind == ASCQ_GROUP_LIST_COUNTS || g->group_list_kind == ASCQ_GROUP_LIST_PREFIX_SUM,
                 ASCQ_EINVAL, "ascq_group_matmul_w8a8: unknown group list kind %d", g->group_list_kind);
    ASCQ_REQUIRE(d->quant_mode == ASCQ_MM_QUANT_VECTOR && d->scale_format == ASCQ_MM_SCALE_F32, ASCQ_EUNSUPPORTED,
                 "ascq_group_matmul_w8a8: the per-group channel scale is an fp32 vector");
    ASCQ_REQUIRE(!d->trans_a && !d->trans_b, ASCQ_EUNSUPPORTED, "ascq_group_matmul_w8a8: transposed operands");
    ASCQ_REQUIRE(d->bias_kind != ASCQ_MM_BIAS_I32_PRE, ASCQ_EUNSUPPORTED,
                 "ascq_group_matmul_w8a8: bias is applied after dequantisation");
    ASCQ_REQUIRE(d->k % 16 == 0 && d->n % 8 == 0 && aligned16(x) && aligned16(w), ASCQ_EALIGN,
                 "ascq_group_matmul_w8a8: k must be a multiple of 16, n of 8, x and w 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    GemmParams p{};
    p.a = static_cast<const int8_t*>(x);
    p.b = static_cast<const int8_t*>(w);
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.group_list = group_list;
    p.groups = g->groups;
    p.group_list_kind = g->group_list_kind;
    p.epi = make_epi(d, y, bias, scale, tok_scale);
    p.b_nz = d->b_format == ASCQ_MM_B_NZ ? 1u : 0u;
    ASCQ_REQUIRE(d->activation != ASCQ_MM_ACT_SWIGLU || d->out_dtype == ASCQ_F16 || d->out_dtype == ASCQ_BF16,
                 ASCQ_EUNSUPPORTED, "ascq_group_matmul_w8a8: SwiGLU writes half or bfloat16 here");
    if (gemm_dma_supported(p)) {
        return launch_gemm_dma(p, true, st);
    }
    ASCQ_REQUIRE(!p.b_nz, ASCQ_EUNSUPPORTED, "ascq_group_matmul_w8a8: fractal (NZ) weights need the tile kernel's shape");
    ASCQ_REQUIRE(d->activation != ASCQ_MM_ACT_SWIGLU, ASCQ_EUNSUPPORTED,
                 "ascq_group_matmul_w8a8: SwiGLU needs the tile kernel's shape (k %% 128 == 0, n %% 16 == 0)");
    typedef TileM T;  // 128 x 256: the 256-row tile spills here (the group bookkeeping on top of 256 accumulator registers)
    // every group adds at most one partial tile along M
    p.tiles_m = (d->m + T::BM - 1) / T::BM + g->groups;
    p.tiles_n = (d->n + T::BN - 1) / T::BN;
    auto kernel = group_gemm_kernel<T>;
    rc = set_lds(kernel, T::kLds);
    if (rc != ASCQ_OK) {
        return rc;
    }
    const uint32_t total = p.tiles_m * p.tiles_n;
    kernel<<<(total + 7u) / 8u * 8u, kThreads, T::kLds, st>>>(p);
    return launch_status("ascq_group_matmul_w8a8");
}
