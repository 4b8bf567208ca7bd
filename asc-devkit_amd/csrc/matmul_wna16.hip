// Weight-only linears for decode: y[m, n] = sum_k x[m, k] * antiquant(w[k, n]) with int4 (W4A16, per-group
// parameters) or int8 (W8A16, per-channel / per-tensor parameters: the Matmul anti-quant path) weights de-quantised in
// registers, never materialised in memory.  The description below is the int4 kernels'; the int8 kernel at the end of
// the file follows the same design.
//
// The kernel is bound by the HBM read of the packed weights (k * n / 2 bytes), so it is built as a set of independent
// streams, one per wavefront, each with its own deep queue of loads:
//   * the weight matrix is cut into chunks of 32 rows x 512 columns (8 KiB); the chunks, in column-block-major order,
//     are dealt out in equal contiguous runs to 1024 wavefronts (one per SIMD of the chip), so every SIMD streams the
//     same number of bytes whatever the shape;
//   * a wavefront moves a chunk HBM -> LDS with global_load_lds_dwordx4 (no registers, tracked by vmcnt) into a private
//     ring of three stages: two chunks (plus the matching scale / offset rows and activations) are always in flight
//     behind the one being computed, independent of register pressure and of where the compiler places its waits;
//     a lane reads back from LDS exactly the bytes it fetched, so there are no bank conflicts and no barriers at all;
//   * a lane owns 16 bytes = 32 adjacent columns of a weight row; the 16 lanes of a quarter-wavefront cover the 512
//     columns and the four quarters take 4 x 8 rows;
//   * de-quantisation follows AscendAntiQuant<int4b_t, half> exactly: the nibble becomes an exact half via the
//     0x6400 exponent trick (1024 + u, or 1024 + 16 u for the nibbles read 4 bits up, which saves the shift), one
//     exact packed add / fma turns it into w, then one rounded half add of the offset and one rounded half multiply by
//     the scale;
//   * the multiply-accumulate runs on the matrix core (v_mfma_f32_16x16x32_f16, fp32 sums).  For up to four
//     activation rows the 8 de-quantised halves of one dword are the B operand as they are; the A operand of output
//     row i carries x[k_g] in slot i and zeros elsewhere, so row i of the result is the running dot product of column
//     i of the dword (rows 0-7 serve one activation row, rows 8-15 a second one).  From five rows on, the halves are
//     regrouped so that a B operand is 8 consecutive k of one column and 16 activation rows fill the A operand (two
//     such row tiles per pass when more than 16 rows remain);
//   * when a wavefront's run leaves a column block (and at its end) the accumulators go to a workspace as they lie in
//     registers; a second kernel adds, for every output, the pieces of all wavefronts that worked on its column block
//     in ascending k order and rounds once to half, so results are deterministic.
#include <type_traits>

#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

constexpr int kThreads = 256;          // four independent wavefronts per workgroup
constexpr uint32_t kColsPerBlock = 512;    // int4: 16 lanes x 32 columns
constexpr uint32_t kW8ColsPerBlock = 256;  // int8: 16 lanes x 16 columns
constexpr uint32_t kChunkRows = 32;
constexpr uint32_t kMaxWaves = 1024;   // 256 compute units x 4 SIMDs
constexpr uint32_t kTileRows = 16;     // activation rows per pass over the weights

// cache policy of the weight loads of the GEMV and W8A16 kernels: 2 = non-temporal (the weights are read once per call
// and should not displace the activations and parameters in the caches): 54 -> 48 us for W8A16 at M = 1, 34.1 ->
// 32.6 us for the int4 GEMV.  The 16-row int4 tile kernel measured no better with it (52-57 us against 51-53 us) and
// keeps the default policy.
constexpr int kWeightAux = 2;
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;

struct WnParams {
    const uint16_t* x;
    const uint8_t* w;
    const uint16_t* scale;
    const uint16_t* offset;
    float* partial;  // [waves][max_seg][row pairs, or 8 slices of a 16-row tile][16 registers][64 lanes]
    uint16_t* y;
    uint32_t m, n, k, group_size, has_offset;
    uint32_t m0;                // first activation row of this pass
    uint32_t waves;             // streams
    uint32_t chunks_per_block;  // k / 32
    uint32_t total_chunks;      // column blocks * chunks_per_block
    uint32_t max_seg;           // column blocks one stream can touch
    uint32_t per, rem;          // total_chunks = waves * per + rem
    // W8A16 only
    uint32_t out_f32;                  // y is float instead of half
    uint32_t scale_bits, offset_bits;  // per-tensor parameters as half bits, used when scale == nullptr
    uint32_t w_nk;                     // the weights are [n, k] (generic kernel only)
};

__device__ __forceinline__ f16x2 bits_to_h2(uint32_t b)
{
    f16x2 r;
    __builtin_memcpy(&r, &b, 4);
    return r;
}

// (c0,c1),(c4,c5) -> (c0,c4) and (c1,c5): the order in which the nibble trick yields column pairs
__device__ __forceinline__ void pair_up(u32x4 v, f16x2 (&out)[4])
{
    out[0] = bits_to_h2(__builtin_amdgcn_perm(v[2], v[0], 0x05040100u));
    out[1] = bits_to_h2(__builtin_amdgcn_perm(v[2], v[0], 0x07060302u));
    out[2] = bits_to_h2(__builtin_amdgcn_perm(v[3], v[1], 0x05040100u));
    out[3] = bits_to_h2(__builtin_amdgcn_perm(v[3], v[1], 0x07060302u));
}

// Stream `wave` owns chunks [stream_begin(wave), stream_begin(wave + 1)): the first `rem` streams take per + 1 chunks.
__device__ __forceinline__ uint32_t stream_begin(const WnParams& p, uint32_t wave)
{
    return wave * p.per + (wave < p.rem ? wave : p.rem);
}

// De-quantises one dword (8 nibbles = 8 adjacent columns of one weight row) into 4 packed half pairs; pair c2 holds
// columns (c2, c2 + 4).  kFold: ofc holds offset - 1032 (even pairs) / offset - 72 (odd pairs), which is exact for
// integer offsets, so that w + offset is one exact operation; otherwise ofc is the offset itself.
template <bool kHasOffset, bool kFold>
__device__ __forceinline__ void w4_dequant_dword(uint32_t word, const f16x2 (&sc)[4], const f16x2 (&ofc)[4],
                                                 f16x2 (&h)[4])
{
    const f16x2 k1032 = {static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};
    const f16x2 k72 = {static_cast<half_t>(72.0f), static_cast<half_t>(72.0f)};
    const f16x2 k16th = {static_cast<half_t>(0.0625f), static_cast<half_t>(0.0625f)};
    const uint32_t qd = word ^ 0x88888888u;  // two's complement nibble -> offset binary u = w + 8
    const uint32_t qh = qd >> 8;
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) {
        // (nibble c2, nibble c2 + 4) -> two exact halves: 1024 + u read in place (c2 even), 1024 + 16 u read
        // 4 bits up (c2 odd, saves the shift)
        uint32_t bits;
        if (c2 & 1) {
            asm("v_and_or_b32 %0, %1, %2, %3"
                : "=v"(bits)
                : "v"(c2 == 1 ? qd : qh), "s"(0x00F000F0u), "v"(0x64006400u));
        } else {
            asm("v_and_or_b32 %0, %1, %2, %3"
                : "=v"(bits)
                : "v"(c2 == 0 ? qd : qh), "s"(0x000F000Fu), "v"(0x64006400u));
        }
        if constexpr (kFold && kHasOffset) {
            // w + offset in one exact operation
            h[c2] = (c2 & 1) ? __builtin_elementwise_fma(bits_to_h2(bits), k16th, ofc[c2])
                             : bits_to_h2(bits) + ofc[c2];
        } else {
            h[c2] = (c2 & 1) ? __builtin_elementwise_fma(bits_to_h2(bits), k16th, -k72)
                             : bits_to_h2(bits) - k1032;  // w, exact
            if constexpr (kHasOffset) {
                h[c2] = h[c2] + ofc[c2];  // one rounding
            }
        }
        h[c2] = sc[c2] * h[c2];  // one rounding
    }
}

// De-quantises the 32 x 32 weights a lane holds of one chunk (8 rows x 4 dwords) and accumulates them against one or
// two pairs of activation rows on the matrix core: the 8 halves of a dword are the B operand as they are, and the A
// operand of output row i carries x[k_g] in slot i and zeros elsewhere.
template <int MP, bool kHasOffset, bool kFold>
__device__ __forceinline__ void w4_accumulate(const u32x4 (&wd)[8], const u32x4 (&xc)[MP], const f16x2 (&sc)[4][4],
                                              const f16x2 (&ofc)[4][4], const uint32_t (&amask)[4],
                                              f32x4 (&acc)[MP][4])
{
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        f16x8 a[MP];
#pragma unroll
        for (int q = 0; q < MP; ++q) {
            const uint32_t xw = xc[q][u >> 1];
            const uint32_t xx =
                (u & 1) ? __builtin_amdgcn_perm(xw, xw, 0x03020302u) : __builtin_amdgcn_perm(xw, xw, 0x01000100u);
            u32x4 av = u32x4{xx & amask[0], xx & amask[1], xx & amask[2], xx & amask[3]};
            __builtin_memcpy(&a[q], &av, 16);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            f16x2 h[4];
            w4_dequant_dword<kHasOffset, kFold>(wd[u][d], sc[d], ofc[d], h);
            f16x8 b;
            __builtin_memcpy(&b, h, 16);
#pragma unroll
            for (int q = 0; q < MP; ++q) {
                acc[q][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[q], b, acc[q][d], 0, 0, 0);
            }
        }
    }
}

// The same weights against a tile of 16 activation rows.  Over the 8 rows a lane holds, column c of dword d is the
// 8 consecutive k the B operand of v_mfma_f32_16x16x32_f16 wants for one column, so the de-quantised halves only
// have to be regrouped (one byte permute per operand dword) and x[16 rows][32 k] is the A operand as it lies in
// memory.  Accumulator e = 8 d + 2 c2 + hi (kept as acc[e / 4][e % 4]) holds, for the lane's quarter g and column
// group jj, rows 4 g .. 4 g + 3 of column 32 jj + 8 d + c2 + 4 hi.
template <bool kHasOffset, int kRT>
__device__ __forceinline__ void w4_accumulate_tile(const u32x4 (&wd)[8], const u32x4 (&xa)[kRT],
                                                   const f16x2 (&sc)[4][4], const f16x2 (&ofc)[4][4],
                                                   f32x4 (&acc)[kRT * 8][4])
{
    f16x8 a[kRT];
#pragma unroll
    for (int t = 0; t < kRT; ++t) __builtin_memcpy(&a[t], &xa[t], 16);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        f16x2 h[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            w4_dequant_dword<kHasOffset, false>(wd[u][d], sc[d], ofc[d], h[u]);
        }
#pragma unroll
        for (int qh = 0; qh < 2; ++qh) {
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const int c2 = 2 * qh + (dd >> 1), hi = dd & 1;  // accumulator e = 8 d + 4 qh + dd
                u32x4 bv;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t even, odd;
                    __builtin_memcpy(&even, &h[2 * t][c2], 4);
                    __builtin_memcpy(&odd, &h[2 * t + 1][c2], 4);
                    bv[t] = __builtin_amdgcn_perm(odd, even, hi ? 0x07060302u : 0x05040100u);
                }
                f16x8 b;
                __builtin_memcpy(&b, &bv, 16);
#pragma unroll
                for (int t = 0; t < kRT; ++t) {
                    acc[8 * t + 2 * d + qh][dd] =
                        __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t], b, acc[8 * t + 2 * d + qh][dd], 0, 0, 0);
                }
            }
        }
    }
}

// True on every lane iff every offset held by any lane of the wavefront is an integer of magnitude <= 512 (then
// (o + 1536) - 1536 == o exactly).  Uniform over the wavefront on purpose: the matrix instruction ignores the execution
// mask, so the two arithmetic paths must never run in one wavefront.
template <int A, int B>
__device__ __forceinline__ bool all_offsets_integral(const f16x2 (&of)[A][B])
{
    const f16x2 k1536 = {static_cast<half_t>(1536.0f), static_cast<half_t>(1536.0f)};
    uint32_t differ = 0;
#pragma unroll
    for (int d = 0; d < A; ++d) {
#pragma unroll
        for (int c2 = 0; c2 < B; ++c2) {
            const f16x2 t = (of[d][c2] + k1536) - k1536;
            uint32_t tb, ob;
            __builtin_memcpy(&tb, &t, 4);
            __builtin_memcpy(&ob, &of[d][c2], 4);
            differ |= (tb ^ ob) & 0x7FFF7FFFu;  // -0 counts as the integer 0
        }
    }
    return __builtin_amdgcn_ballot_w64(differ != 0) == 0;
}

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
#define ASCQ_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

// Five to 16 kRT activation rows per pass over the weights (rows m0 .. m0 + 16 kRT - 1): one stream per SIMD, the rows
// are the rows of kRT MFMA tiles that share every de-quantised B operand (w4_accumulate_tile).  A piece of the
// workspace is [8 kRT slices][16 registers][64 lanes].  Requires n % 32 == 0, k % 32 == 0, group_size % 32 == 0.
template <bool kHasOffset, int kRT>
__global__ __launch_bounds__(kThreads) void w4a16_tile_kernel(WnParams p)
{
    static_assert(kRT == 1 || kRT == 2, "one or two tiles of 16 activation rows per pass");
    constexpr int kParamInstr = kHasOffset ? 2 : 1;
    constexpr int kInstr = 8 + kParamInstr + kRT;  // 1 KiB DMA instructions per chunk
    constexpr int kStage = kInstr * 1024;         // bytes per wavefront and stage
    __shared__ __attribute__((aligned(1024))) char S0[4 * kStage];
    __shared__ __attribute__((aligned(1024))) char S1[4 * kStage];
    __shared__ __attribute__((aligned(1024))) char S2[4 * kStage];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t gw = blockIdx.x * 4u + wave;
    if (gw >= p.waves) {
        return;  // whole wavefront; the kernel has no barriers
    }
    const uint32_t g = lane >> 4, jj = lane & 15u;
    const uint32_t c_begin = stream_begin(p, gw), c_end = stream_begin(p, gw + 1u);
    if (c_begin == c_end) {
        return;
    }
    const size_t row_bytes = p.n / 2;
    const uint32_t cb_chunks = p.chunks_per_block;

    // ---- producer side: chunk (block ib, k-chunk ik) -> stage
    uint32_t ib = c_begin / cb_chunks, ik = c_begin % cb_chunks, issued = c_begin;
    auto issue = [&](char* stage) {
        // Lanes past the last column work on a duplicate of the last 32 columns (never stored): the MFMA ignores the
        // execution mask, so every lane must hold valid operands.
        uint32_t col0 = ib * kColsPerBlock + jj * 32u;
        col0 = col0 < p.n ? col0 : p.n - 32u;
        const uint32_t krow = ik * kChunkRows;
        const uint8_t* wsrc = p.w + static_cast<size_t>(krow + 8u * g) * row_bytes + col0 / 2;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + static_cast<size_t>(u) * row_bytes),
                                             (lds_ptr_t)(stage + u * 1024), 16, 0, 0);
        }
        // parameters of the chunk's group: lane (g, jj) fetches piece g (8 halves) of the 32 columns of jj
        const size_t prow = static_cast<size_t>(krow / p.group_size) * p.n + col0 + 8u * g;
        __builtin_amdgcn_global_load_lds((gptr_t)(p.scale + prow), (lds_ptr_t)(stage + 8 * 1024), 16, 0, 0);
        if constexpr (kHasOffset) {
            __builtin_amdgcn_global_load_lds((gptr_t)(p.offset + prow), (lds_ptr_t)(stage + 9 * 1024), 16, 0, 0);
        }
        // activations of the chunk's 32 k, 16 rows per instruction: lane l fetches piece (l & 3) of row
        // m0 + 16 t + (l >> 2); rows past m fetch row m - 1 and are zeroed when used
#pragma unroll
        for (int t = 0; t < kRT; ++t) {
            const uint32_t m = p.m0 + 16u * t + (lane >> 2);
            const uint32_t mc = m < p.m ? m : p.m - 1u;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.x + static_cast<size_t>(mc) * p.k + krow + 8u * (lane & 3u)),
                                             (lds_ptr_t)(stage + (8 + kParamInstr + t) * 1024), 16, 0, 0);
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
    f32x4 acc[kRT * 8][4];  // accumulator e of row tile t is acc[8 t + e / 4][e % 4]
#pragma unroll
    for (int q = 0; q < kRT * 8; ++q) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[q][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    uint32_t seg = 0, done_in_block = c_begin % cb_chunks;
    // the accumulators as they lie in registers: [16 registers][64 lanes] per slice of four accumulators
    auto flush = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < kRT * 8; ++q) {
            float* dst = p.partial + ((static_cast<size_t>(gw) * p.max_seg + seg) * (kRT * 8u) + q) * 1024u + lane;
            // register r holds row 16 (q / 8) + 4 g + r; lanes of a missing row hold zeros: not stored
#pragma unroll
            for (int d = 0; d < 4; ++d) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool row_valid = p.m0 + 16u * (q >> 3) + 4u * g + r < p.m;
                    if (row_valid) {
                        dst[(d * 4 + r) * 64] = acc[q][d][r];
                    }
                }
                acc[q][d] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        ++seg;
        // Stores and loads retire out of order with respect to each other, so the counted waits on the load queue
        // are only meaningful while no store is pending: drain here (once per column block and stream).
        ASCQ_WAIT_VMCNT(0);
    };
    // The stages are read back with explicit ds_read instructions and one explicit wait: the reads only ever follow
    // the counted wait on the stage's loads above them, and the compiler's own bookkeeping of LDS reads against
    // direct-to-LDS loads in flight (which is conservative around the loop) stays out of the way.
#define ASCQ_DS_READ128(dst, addr, off) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off) : "memory")
    auto compute = [&](const char* stage) __attribute__((always_inline)) {
        const uint32_t sa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)stage));
        const uint32_t a_own = sa + lane * 16u;                      // what this lane fetched itself
        const uint32_t a_par = sa + jj * 16u;                        // parameter pieces of the lane's 32 columns
        const uint32_t a_x = sa + (jj * 4u + g) * 16u;               // activations: row jj of the tile, piece g
        u32x4 wd[8], sraw[4], oraw[4], xraw[kRT];
        ASCQ_DS_READ128(wd[0], a_own, 0 * 1024);
        ASCQ_DS_READ128(wd[1], a_own, 1 * 1024);
        ASCQ_DS_READ128(wd[2], a_own, 2 * 1024);
        ASCQ_DS_READ128(wd[3], a_own, 3 * 1024);
        ASCQ_DS_READ128(wd[4], a_own, 4 * 1024);
        ASCQ_DS_READ128(wd[5], a_own, 5 * 1024);
        ASCQ_DS_READ128(wd[6], a_own, 6 * 1024);
        ASCQ_DS_READ128(wd[7], a_own, 7 * 1024);
        ASCQ_DS_READ128(sraw[0], a_par, 8 * 1024 + 0 * 256);
        ASCQ_DS_READ128(sraw[1], a_par, 8 * 1024 + 1 * 256);
        ASCQ_DS_READ128(sraw[2], a_par, 8 * 1024 + 2 * 256);
        ASCQ_DS_READ128(sraw[3], a_par, 8 * 1024 + 3 * 256);
        if constexpr (kHasOffset) {
            ASCQ_DS_READ128(oraw[0], a_par, 9 * 1024 + 0 * 256);
            ASCQ_DS_READ128(oraw[1], a_par, 9 * 1024 + 1 * 256);
            ASCQ_DS_READ128(oraw[2], a_par, 9 * 1024 + 2 * 256);
            ASCQ_DS_READ128(oraw[3], a_par, 9 * 1024 + 3 * 256);
        }
        ASCQ_DS_READ128(xraw[0], a_x, (8 + kParamInstr) * 1024);
        if constexpr (kRT > 1) ASCQ_DS_READ128(xraw[1], a_x, (8 + kParamInstr + 1) * 1024);
        // every value read above is an in/out operand of the wait, so nothing uses one before it has arrived
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wd[0]), "+v"(wd[1]), "+v"(wd[2]), "+v"(wd[3]), "+v"(wd[4]), "+v"(wd[5]), "+v"(wd[6]),
                       "+v"(wd[7]), "+v"(sraw[0]), "+v"(sraw[1]), "+v"(sraw[2]), "+v"(sraw[3])
                     :
                     : "memory");
        if constexpr (kHasOffset) {
            asm volatile("" : "+v"(oraw[0]), "+v"(oraw[1]), "+v"(oraw[2]), "+v"(oraw[3]));
        }
#pragma unroll
        for (int t = 0; t < kRT; ++t) asm volatile("" : "+v"(xraw[t]));
        f16x2 sc[4][4], of[4][4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            pair_up(sraw[d], sc[d]);
            if constexpr (kHasOffset) {
                pair_up(oraw[d], of[d]);
            }
        }
        // lane (g, jj) carries x[m0 + 16 t + jj][krow + 8 g .. + 8): the A operand of row tile t
        u32x4 xa[kRT];
#pragma unroll
        for (int t = 0; t < kRT; ++t) {
            xa[t] = p.m0 + 16u * t + jj < p.m ? xraw[t] : u32x4{0u, 0u, 0u, 0u};
        }
        // (the integer-offset fold of the GEMV kernel is left out: two arithmetic paths that merge with 128 or 256 live
        // accumulators cost more in register shuffling, or spills, than the packed operation they save)
        w4_accumulate_tile<kHasOffset, kRT>(wd, xa, sc, of, acc);
        if (++done_in_block == cb_chunks) {  // the run leaves this column block
            done_in_block = 0;
            flush();
        }
    };

    char* s0 = S0 + wave * kStage;
    char* s1 = S1 + wave * kStage;
    char* s2 = S2 + wave * kStage;
    issue(s0);
    issue(s1);
    issue(s2);
    uint32_t c = c_begin;
    while (true) {
        ASCQ_WAIT_VMCNT(2 * kInstr);  // everything but the two newest chunks has landed
        compute(s0);
        if (++c == c_end) break;
        issue(s0);
        ASCQ_WAIT_VMCNT(2 * kInstr);
        compute(s1);
        if (++c == c_end) break;
        issue(s1);
        ASCQ_WAIT_VMCNT(2 * kInstr);
        compute(s2);
        if (++c == c_end) break;
        issue(s2);
    }
    ASCQ_WAIT_VMCNT(0);
    if (done_in_block != 0) {
        flush();
    }
}

// Up to four activation rows (MP = 1 or 2 row pairs; the decode GEMV): the same streams, two per SIMD.  To fit 8
// rings into the LDS the ring has two stages and holds only the weights (8 KiB) and the activations (256 bytes); the scale / offset rows of
// a quantisation group are fetched into registers when a chunk opens a new group, ahead of that chunk's weights, so
// they have landed whenever the weights have.  With two stages one chunk is in flight behind the one being computed
// and the wait before a chunk is simply for everything outstanding; the second wavefront of the SIMD fills the time
// a wavefront spends waiting or stalled on its own dependent instructions.
template <int MP, bool kHasOffset>
__global__ __launch_bounds__(512) void w4a16_gemv_kernel(WnParams p)
{
    constexpr int kStage = 8 * 1024 + 256;  // bytes per wavefront and stage
    __shared__ __attribute__((aligned(1024))) char S0[8 * kStage];
    __shared__ __attribute__((aligned(1024))) char S1[8 * kStage];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t gw = blockIdx.x * 8u + wave;
    if (gw >= p.waves) {
        return;  // whole wavefront; the kernel has no barriers
    }
    const uint32_t g = lane >> 4, jj = lane & 15u;
    const uint32_t c_begin = stream_begin(p, gw), c_end = stream_begin(p, gw + 1u);
    if (c_begin == c_end) {
        return;
    }
    const size_t row_bytes = p.n / 2;
    const uint32_t cb_chunks = p.chunks_per_block;
    const uint32_t chunks_per_group = p.group_size / kChunkRows;

    // ---- producer side: chunk (block ib, k-chunk ik) -> stage; parameters of a new group -> registers
    uint32_t ib = c_begin / cb_chunks, ik = c_begin % cb_chunks;
    u32x4 sraw[4], oraw[4];
    bool params_pending = false;
    auto issue = [&](char* stage, bool first) {
        // Lanes past the last column work on a duplicate of the last 32 columns (never stored): the MFMA ignores the
        // execution mask, so every lane must hold valid operands.
        uint32_t col0 = ib * kColsPerBlock + jj * 32u;
        col0 = col0 < p.n ? col0 : p.n - 32u;
        const uint32_t krow = ik * kChunkRows;
        if (first || ik % chunks_per_group == 0u) {  // the chunk opens the run, a group or a column block
            const size_t prow = static_cast<size_t>(krow / p.group_size) * p.n + col0;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                sraw[d] = *reinterpret_cast<const u32x4*>(p.scale + prow + 8 * d);
                if constexpr (kHasOffset) {
                    oraw[d] = *reinterpret_cast<const u32x4*>(p.offset + prow + 8 * d);
                }
            }
            params_pending = true;
        }
        const uint8_t* wsrc = p.w + static_cast<size_t>(krow + 8u * g) * row_bytes + col0 / 2;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + static_cast<size_t>(u) * row_bytes),
                                             (lds_ptr_t)(stage + u * 1024), 16, 0, kWeightAux);
        }
        // activations of the chunk's 32 k for 2 MP rows, one dword per lane: lane l fetches dword (l & 15) of row
        // m0 + ((l >> 4) & (2 MP - 1)); a missing row fetches the last one and is zeroed when used
        {
            const uint32_t m = p.m0 + ((lane >> 4) & (2u * MP - 1u));
            const uint32_t mc = m < p.m ? m : p.m - 1u;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.x + static_cast<size_t>(mc) * p.k + krow + 2u * (lane & 15u)),
                                             (lds_ptr_t)(stage + 8 * 1024), 4, 0, 0);
        }
        if (++ik == cb_chunks) {
            ik = 0;
            ++ib;
        }
    };

    // ---- consumer side
    f32x4 acc[MP][4];
#pragma unroll
    for (int q = 0; q < MP; ++q) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[q][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const uint32_t slot = jj & 7u;
    uint32_t amask[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        amask[r] = (static_cast<uint32_t>(r) == (slot >> 1)) ? ((slot & 1u) ? 0xFFFF0000u : 0x0000FFFFu) : 0u;
    }
    const f16x2 k1032 = {static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};
    const f16x2 k72 = {static_cast<half_t>(72.0f), static_cast<half_t>(72.0f)};
    f16x2 sc[4][4], ofc[4][4];
    bool folded = false;
    uint32_t seg = 0, done_in_block = c_begin % cb_chunks;
    auto flush = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < MP; ++q) {
            float* dst = p.partial + ((static_cast<size_t>(gw) * p.max_seg + seg) * MP + q) * 1024u + lane;
            const bool row_valid = p.m0 + 2u * q + (g >> 1) < p.m;  // lanes of a missing row hold zeros: not stored
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                if (row_valid) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        dst[(d * 4 + r) * 64] = acc[q][d][r];
                    }
                }
                acc[q][d] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        ++seg;
    };
    // called after the wait: turns freshly landed parameter rows into the packed constants of the group
    auto adopt_params = [&]() {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            pair_up(sraw[d], sc[d]);
            if constexpr (kHasOffset) {
                pair_up(oraw[d], ofc[d]);
            }
        }
        folded = false;
        if constexpr (kHasOffset) {
            folded = all_offsets_integral(ofc);
            if (folded) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
#pragma unroll
                    for (int c2 = 0; c2 < 4; ++c2) {
                        ofc[d][c2] = (c2 & 1) ? ofc[d][c2] - k72 : ofc[d][c2] - k1032;  // exact
                    }
                }
            }
        }
        params_pending = false;
    };
    auto compute = [&](const char* stage) __attribute__((always_inline)) {
        const uint32_t sa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)stage));
        const uint32_t a_own = sa + lane * 16u;                           // what this lane fetched itself
        const uint32_t a_x = sa + 8u * 1024u + (jj >> 3) * 64u + g * 16u;  // row (jj >> 3) of a pair, k 8 g .. 8 g + 7
        u32x4 wd[8], xraw[MP];
        ASCQ_DS_READ128(wd[0], a_own, 0 * 1024);
        ASCQ_DS_READ128(wd[1], a_own, 1 * 1024);
        ASCQ_DS_READ128(wd[2], a_own, 2 * 1024);
        ASCQ_DS_READ128(wd[3], a_own, 3 * 1024);
        ASCQ_DS_READ128(wd[4], a_own, 4 * 1024);
        ASCQ_DS_READ128(wd[5], a_own, 5 * 1024);
        ASCQ_DS_READ128(wd[6], a_own, 6 * 1024);
        ASCQ_DS_READ128(wd[7], a_own, 7 * 1024);
        ASCQ_DS_READ128(xraw[0], a_x, 0);
        if constexpr (MP > 1) ASCQ_DS_READ128(xraw[1], a_x, 128);  // the next pair: two rows of 64 bytes further on
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wd[0]), "+v"(wd[1]), "+v"(wd[2]), "+v"(wd[3]), "+v"(wd[4]), "+v"(wd[5]), "+v"(wd[6]),
                       "+v"(wd[7]), "+v"(xraw[0])
                     :
                     : "memory");
        if constexpr (MP > 1) asm volatile("" : "+v"(xraw[1]));
        u32x4 xc[MP];
#pragma unroll
        for (int q = 0; q < MP; ++q) {
            xc[q] = (p.m0 + 2u * q + (jj >> 3) < p.m) ? xraw[q] : u32x4{0u, 0u, 0u, 0u};
        }
        if (kHasOffset && folded) {
            w4_accumulate<MP, kHasOffset, true>(wd, xc, sc, ofc, amask, acc);
        } else {
            w4_accumulate<MP, kHasOffset, false>(wd, xc, sc, ofc, amask, acc);
        }
        if (++done_in_block == cb_chunks) {  // the run leaves this column block
            done_in_block = 0;
            flush();
        }
    };

    char* s0 = S0 + wave * kStage;
    char* s1 = S1 + wave * kStage;
    issue(s0, true);
    uint32_t c = c_begin;
    while (true) {
        ASCQ_WAIT_VMCNT(0);  // chunk c (and parameter rows fetched ahead of it) has landed
        if (params_pending) adopt_params();
        if (c + 1u < c_end) issue(s1, false);
        compute(s0);
        if (++c == c_end) break;
        ASCQ_WAIT_VMCNT(0);
        if (params_pending) adopt_params();
        if (c + 1u < c_end) issue(s0, false);
        compute(s1);
        if (++c == c_end) break;
    }
    if (done_in_block != 0) {
        flush();
    }
}

// W8A16 (A half, B int8 de-quantised per channel or per tensor while it is read): the same streams, two per SIMD, on
// chunks of 32 rows x 256 columns of int8 (8 KiB).  A lane owns 16 adjacent columns of a weight row; over the 8 rows
// it holds, one column is the 8 consecutive k of a B operand, so up to 16 activation rows fill one MFMA tile per
// column.  A byte becomes an exact half by a byte permute into 0x6400 | (w + 128) = 1152 + w; one exact subtraction
// gives w, then one rounded half add of the offset and one rounded half multiply by the scale, as
// AscendAntiQuant<int8_t, half>.  The scale / offset of a column do not depend on k: they are fetched into registers
// when the stream enters a column block.  Accumulator c (kept as acc[c / 4][c % 4]) holds rows 4 g .. 4 g + 3 of
// column 16 jj + c; a piece of the workspace is [4 slices][16 registers][64 lanes].
// Requires n % 16 == 0, k % 32 == 0.
template <bool kHasOffset, int kRT>
__global__ __launch_bounds__(512) void w8a16_tile_kernel(WnParams p)
{
    static_assert(kRT == 1 || kRT == 2, "one or two tiles of 16 activation rows per pass");
    constexpr int kStage = 8 * 1024 + kRT * 1024;  // bytes per wavefront and stage: weights, activations
    __shared__ __attribute__((aligned(1024))) char S0[8 * kStage];
    __shared__ __attribute__((aligned(1024))) char S1[8 * kStage];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t gw = blockIdx.x * 8u + wave;
    if (gw >= p.waves) {
        return;  // whole wavefront; the kernel has no barriers
    }
    const uint32_t g = lane >> 4, jj = lane & 15u;
    const uint32_t c_begin = stream_begin(p, gw), c_end = stream_begin(p, gw + 1u);
    if (c_begin == c_end) {
        return;
    }
    const size_t row_bytes = p.n;
    const uint32_t cb_chunks = p.chunks_per_block;
    const bool per_tensor = p.scale == nullptr;

    // ---- producer side: chunk (block ib, k-chunk ik) -> stage; parameters of a new column block -> registers
    uint32_t ib = c_begin / cb_chunks, ik = c_begin % cb_chunks;
    u32x4 sraw[2], oraw[2];
    bool params_pending = false;
    auto issue = [&](char* stage, bool first) {
        // Lanes past the last column work on a duplicate of the last 16 columns (never stored): the MFMA ignores the
        // execution mask, so every lane must hold valid operands.
        uint32_t col0 = ib * kW8ColsPerBlock + jj * 16u;
        col0 = col0 < p.n ? col0 : p.n - 16u;
        const uint32_t krow = ik * kChunkRows;
        if (first || ik == 0u) {  // the chunk opens the run or a column block
            if (!per_tensor) {
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    sraw[d] = *reinterpret_cast<const u32x4*>(p.scale + col0 + 8 * d);
                    if constexpr (kHasOffset) {
                        oraw[d] = *reinterpret_cast<const u32x4*>(p.offset + col0 + 8 * d);
                    }
                }
            }
            params_pending = true;
        }
        const uint8_t* wsrc = p.w + static_cast<size_t>(krow + 8u * g) * row_bytes + col0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + static_cast<size_t>(u) * row_bytes),
                                             (lds_ptr_t)(stage + u * 1024), 16, 0, kWeightAux);
        }
        // activations of the chunk's 32 k, 16 rows per instruction: lane l fetches piece (l & 3) of row
        // m0 + 16 t + (l >> 2); rows past m fetch row m - 1 and are zeroed when used
#pragma unroll
        for (int t = 0; t < kRT; ++t) {
            const uint32_t m = p.m0 + 16u * t + (lane >> 2);
            const uint32_t mc = m < p.m ? m : p.m - 1u;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.x + static_cast<size_t>(mc) * p.k + krow + 8u * (lane & 3u)),
                                             (lds_ptr_t)(stage + (8 + t) * 1024), 16, 0, 0);
        }
        if (++ik == cb_chunks) {
            ik = 0;
            ++ib;
        }
    };

    // ---- consumer side
    f32x4 acc[kRT * 4][4];  // row tile t: acc[4 t + c / 4][c % 4]
#pragma unroll
    for (int q = 0; q < kRT * 4; ++q) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[q][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const f16x2 k1152 = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};
    f16x2 sc[2][4], ofc[2][4];  // pair i of dword-half d: columns 8 d + 2 i, 8 d + 2 i + 1
    bool folded = false;
    uint32_t seg = 0, done_in_block = c_begin % cb_chunks;
    auto flush = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < kRT * 4; ++q) {
            float* dst = p.partial + ((static_cast<size_t>(gw) * p.max_seg + seg) * (kRT * 4u) + q) * 1024u + lane;
            // register r holds row 16 (q / 4) + 4 g + r; lanes of a missing row hold zeros: not stored
#pragma unroll
            for (int d = 0; d < 4; ++d) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (p.m0 + 16u * (q >> 2) + 4u * g + r < p.m) {
                        dst[(d * 4 + r) * 64] = acc[q][d][r];
                    }
                }
                acc[q][d] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        ++seg;
    };
    // called after the wait: turns freshly landed parameters into the packed constants of the column block
    auto adopt_params = [&]() {
#pragma unroll
        for (int d = 0; d < 2; ++d) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[d][i] = bits_to_h2(per_tensor ? p.scale_bits * 0x00010001u : sraw[d][i]);
                if constexpr (kHasOffset) {
                    ofc[d][i] = bits_to_h2(per_tensor ? p.offset_bits * 0x00010001u : oraw[d][i]);
                }
            }
        }
        folded = false;
        if constexpr (kHasOffset) {
            // with integer offsets w + offset is exact, and so is (1152 + w) + (offset - 1152)
            folded = all_offsets_integral(ofc);
            if (folded) {
#pragma unroll
                for (int d = 0; d < 2; ++d) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) ofc[d][i] = ofc[d][i] - k1152;  // exact
                }
            }
        }
        params_pending = false;
    };
    auto compute = [&](const char* stage) __attribute__((always_inline)) {
        const uint32_t sa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)stage));
        const uint32_t a_own = sa + lane * 16u;                       // what this lane fetched itself
        const uint32_t a_x = sa + 8u * 1024u + (jj * 4u + g) * 16u;   // activations: row jj of the tile, piece g
        u32x4 wd[8], xraw[kRT];
        ASCQ_DS_READ128(wd[0], a_own, 0 * 1024);
        ASCQ_DS_READ128(wd[1], a_own, 1 * 1024);
        ASCQ_DS_READ128(wd[2], a_own, 2 * 1024);
        ASCQ_DS_READ128(wd[3], a_own, 3 * 1024);
        ASCQ_DS_READ128(wd[4], a_own, 4 * 1024);
        ASCQ_DS_READ128(wd[5], a_own, 5 * 1024);
        ASCQ_DS_READ128(wd[6], a_own, 6 * 1024);
        ASCQ_DS_READ128(wd[7], a_own, 7 * 1024);
        ASCQ_DS_READ128(xraw[0], a_x, 0);
        if constexpr (kRT > 1) ASCQ_DS_READ128(xraw[1], a_x, 1024);
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wd[0]), "+v"(wd[1]), "+v"(wd[2]), "+v"(wd[3]), "+v"(wd[4]), "+v"(wd[5]), "+v"(wd[6]),
                       "+v"(wd[7]), "+v"(xraw[0])
                     :
                     : "memory");
        if constexpr (kRT > 1) asm volatile("" : "+v"(xraw[1]));
        // lane (g, jj) carries x[m0 + 16 t + jj][krow + 8 g .. + 8): the A operand of row tile t
        f16x8 a[kRT];
#pragma unroll
        for (int t = 0; t < kRT; ++t) {
            const u32x4 xa = p.m0 + 16u * t + jj < p.m ? xraw[t] : u32x4{0u, 0u, 0u, 0u};
            __builtin_memcpy(&a[t], &xa, 16);
        }
#pragma unroll
        for (int d = 0; d < 2; ++d) {  // columns 8 d .. 8 d + 7 of the lane's 16
            f16x2 h[8][4];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t word = wd[u][2 * d + (i >> 1)] ^ 0x80808080u;  // two's complement -> w + 128
                    // bytes (2 (i & 1), 2 (i & 1) + 1) of the word -> two exact halves 1024 + (w + 128)
                    const uint32_t bits = __builtin_amdgcn_perm(0x64646464u, word, (i & 1) ? 0x04030402u : 0x04010400u);
                    f16x2 v;
                    if (kHasOffset && folded) {
                        v = bits_to_h2(bits) + ofc[d][i];  // w + offset, exact
                    } else {
                        v = bits_to_h2(bits) - k1152;  // w, exact
                        if constexpr (kHasOffset) {
                            v = v + ofc[d][i];  // one rounding
                        }
                    }
                    h[u][i] = sc[d][i] * v;  // one rounding
                }
            }
#pragma unroll
            for (int qh = 0; qh < 2; ++qh) {
#pragma unroll
                for (int dd = 0; dd < 4; ++dd) {
                    const int i = 2 * qh + (dd >> 1), hi = dd & 1;  // column 8 d + 4 qh + dd
                    u32x4 bv;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        uint32_t even, odd;
                        __builtin_memcpy(&even, &h[2 * t][i], 4);
                        __builtin_memcpy(&odd, &h[2 * t + 1][i], 4);
                        bv[t] = __builtin_amdgcn_perm(odd, even, hi ? 0x07060302u : 0x05040100u);
                    }
                    f16x8 b;
                    __builtin_memcpy(&b, &bv, 16);
#pragma unroll
                    for (int t = 0; t < kRT; ++t) {
                        acc[4 * t + 2 * d + qh][dd] =
                            __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t], b, acc[4 * t + 2 * d + qh][dd], 0, 0, 0);
                    }
                }
            }
        }
        if (++done_in_block == cb_chunks) {  // the run leaves this column block
            done_in_block = 0;
            flush();
        }
    };

    char* s0 = S0 + wave * kStage;
    char* s1 = S1 + wave * kStage;
    issue(s0, true);
    uint32_t c = c_begin;
    while (true) {
        ASCQ_WAIT_VMCNT(0);  // chunk c (and parameters fetched ahead of it) has landed
        if (params_pending) adopt_params();
        if (c + 1u < c_end) issue(s1, false);
        compute(s0);
        if (++c == c_end) break;
        ASCQ_WAIT_VMCNT(0);
        if (params_pending) adopt_params();
        if (c + 1u < c_end) issue(s0, false);
        compute(s1);
        if (++c == c_end) break;
    }
    if (done_in_block != 0) {
        flush();
    }
}

// Adds the pieces of all streams that worked on a column block and rounds once to half.  A piece is the image of
// the accumulators of a wavefront, [16 registers][64 lanes] = the 2 rows x 512 columns of the block, so the pieces are
// added element by element in that layout with fully coalesced 16-byte loads, and only the final store is scattered.
// One workgroup per (column block, row pair): 4 sub-groups of 256 lanes take the pieces i = sub, sub + 4, ... in
// ascending k order, the four sums are combined as (s0 + s1) + (s2 + s3): deterministic.
enum PieceLayout { kPiecePairs = 0, kPieceTileW4 = 1, kPieceTileW8 = 2 };

template <int MP, int kLayout = kPiecePairs>
__global__ __launch_bounds__(1024) void stream_sum_kernel(WnParams p)
{
    __shared__ f32x4 part[4][256];
    const uint32_t sub = threadIdx.x >> 8, t = threadIdx.x & 255u;
    const uint32_t blk = blockIdx.x, q = blockIdx.y;
    const uint32_t first_chunk = blk * p.chunks_per_block, end_chunk = first_chunk + p.chunks_per_block;
    // the stream that holds first_chunk, and the first one past the block
    const uint32_t big = p.rem * (p.per + 1u);  // chunks owned by the longer streams
    const uint32_t w0 = first_chunk < big ? first_chunk / (p.per + 1u) : p.rem + (first_chunk - big) / p.per;
    uint32_t w1 = end_chunk <= big ? (end_chunk + p.per) / (p.per + 1u) : p.rem + (end_chunk - big + p.per - 1u) / p.per;
    w1 = w1 < p.waves ? w1 : p.waves;
    const size_t stride = static_cast<size_t>(p.max_seg) * MP * 1024u;  // floats between streams
    // the first stream may have begun in an earlier block; all later ones begin inside this block (piece 0)
    const size_t first_extra = static_cast<size_t>(blk - stream_begin(p, w0) / p.chunks_per_block) * MP * 1024u;
    const float* base = p.partial + (static_cast<size_t>(w0) * p.max_seg * MP + q) * 1024u + 4u * t;
    // the four elements of a lane share their register (t >> 4) and quarter g = (t >> 2) & 3, hence their row (g / 2 of
    // the pair, or 4 g + r of a tile); a row past m was never written
    const uint32_t my_row = kLayout == kPieceTileW8   ? 16u * (q >> 2) + 4u * ((t >> 2) & 3u) + ((t >> 4) & 3u)
                            : kLayout == kPieceTileW4 ? 16u * (q >> 3) + 4u * ((t >> 2) & 3u) + ((t >> 4) & 3u)
                                                      : 2u * q + ((t >> 2) & 3u) / 2u;
    const bool row_valid = p.m0 + my_row < p.m;
    f32x4 s = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t w = w0 + sub; row_valid && w < w1; w += 32u) {
        f32x4 v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {  // 8 independent loads in flight, then an ordered sum
            const uint32_t wu = w + 4u * u;
            const size_t off = static_cast<size_t>(wu - w0) * stride + (wu == w0 ? first_extra : 0u);
            v[u] = wu < w1 ? *reinterpret_cast<const f32x4*>(base + off) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) s += v[u];
    }
    part[sub][t] = s;
    __syncthreads();
    if (sub != 0u) {
        return;
    }
    const f32x4 tot = (part[0][t] + part[1][t]) + (part[2][t] + part[3][t]);
    // element e = (d * 4 + r) * 64 + g * 16 + jj: register r of lane (g, jj) in tile d holds row (g >> 1) of the pair
    // and column slot b8 = 4 (g & 1) + r of the dword, with column = (b8 >> 1) + 4 (b8 & 1)
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) {
        const uint32_t e = 4u * t + i;
        const uint32_t jj = e & 15u, g = (e >> 4) & 3u, r = (e >> 6) & 3u, d = e >> 8;
        uint32_t col, m;
        if constexpr (kLayout == kPieceTileW4) {
            // slice q of row tile q / 8 holds accumulators 4 (q % 8) + d of w4_accumulate_tile
            const uint32_t acc_e = 4u * (q & 7u) + d;
            col = blk * kColsPerBlock + jj * 32u + (acc_e >> 3) * 8u + ((acc_e >> 1) & 3u) + 4u * (acc_e & 1u);
            m = p.m0 + 16u * (q >> 3) + 4u * g + r;
        } else if constexpr (kLayout == kPieceTileW8) {
            // slice q of row tile q / 4 holds columns 4 (q % 4) + d of the lane's 16
            col = blk * kW8ColsPerBlock + jj * 16u + 4u * (q & 3u) + d;
            m = p.m0 + 16u * (q >> 2) + 4u * g + r;
        } else {
            const uint32_t b8 = 4u * (g & 1u) + r;
            col = blk * kColsPerBlock + jj * 32u + d * 8u + (b8 >> 1) + 4u * (b8 & 1u);
            m = p.m0 + 2u * q + (g >> 1);
        }
        if (col < p.n && m < p.m) {
            if (kLayout == kPieceTileW8 && p.out_f32) {
                reinterpret_cast<float*>(p.y)[static_cast<size_t>(m) * p.n + col] = tot[i];
            } else {
                p.y[static_cast<size_t>(m) * p.n + col] = static_cast<uint16_t>(f32_to_half_bits(tot[i]));
            }
        }
    }
}

// Any shape: one lane per output element.
__global__ __launch_bounds__(kThreads) void w4a16_generic_kernel(WnParams p)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * kThreads) {
        const size_t row = idx / p.n, col = idx % p.n;
        float s = 0.0f;
        for (uint32_t kk = 0; kk < p.k; ++kk) {
            const size_t e = static_cast<size_t>(kk) * p.n + col;
            const uint32_t b = p.w[e >> 1];
            const uint32_t nib = (e & 1) ? (b >> 4) : (b & 0xFu);
            half_t h = static_cast<half_t>(static_cast<float>(static_cast<int>(nib ^ 8u) - 8));
            const size_t pi = static_cast<size_t>(kk / p.group_size) * p.n + col;
            if (p.has_offset) {
                h = h + static_cast<half_t>(half_bits_to_f32(p.offset[pi]));
            }
            h = static_cast<half_t>(half_bits_to_f32(p.scale[pi])) * h;
            s += half_bits_to_f32(p.x[row * p.k + kk]) * static_cast<float>(h);
        }
        p.y[idx] = static_cast<uint16_t>(f32_to_half_bits(s));
    }
}

// W8A16, any shape: one lane per output element.
__global__ __launch_bounds__(kThreads) void w8a16_generic_kernel(WnParams p)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * kThreads) {
        const size_t row = idx / p.n, col = idx % p.n;
        const half_t scale = static_cast<half_t>(half_bits_to_f32(p.scale ? p.scale[col] : p.scale_bits));
        const half_t offset =
            p.has_offset ? static_cast<half_t>(half_bits_to_f32(p.scale ? p.offset[col] : p.offset_bits)) : half_t(0);
        float s = 0.0f;
        for (uint32_t kk = 0; kk < p.k; ++kk) {
            const size_t at = p.w_nk ? col * p.k + kk : static_cast<size_t>(kk) * p.n + col;
            half_t h = static_cast<half_t>(static_cast<float>(static_cast<int8_t>(p.w[at])));
            if (p.has_offset) {
                h = h + offset;
            }
            h = scale * h;
            s += half_bits_to_f32(p.x[row * p.k + kk]) * static_cast<float>(h);
        }
        if (p.out_f32) {
            reinterpret_cast<float*>(p.y)[idx] = s;
        } else {
            p.y[idx] = static_cast<uint16_t>(f32_to_half_bits(s));
        }
    }
}

struct W4Plan {
    uint32_t waves, chunks_per_block, total_chunks, max_seg;
};

W4Plan make_plan(uint32_t n, uint32_t k, uint32_t max_waves, uint32_t cols_per_block = kColsPerBlock)
{
    W4Plan pl;
    const uint32_t blocks_n = (n + cols_per_block - 1u) / cols_per_block;
    pl.chunks_per_block = k / kChunkRows;
    pl.total_chunks = blocks_n * pl.chunks_per_block;
    pl.waves = pl.total_chunks < max_waves ? pl.total_chunks : max_waves;
    const uint32_t per = (pl.total_chunks + pl.waves - 1u) / pl.waves;  // longest run
    pl.max_seg = (per + pl.chunks_per_block - 2u) / pl.chunks_per_block + 1u;
    return pl;
}

// bytes of workspace: the larger of the two kernels' needs (two streams per SIMD with up to two row pairs, one with
// up to sixteen)
size_t workspace_need(uint32_t n, uint32_t k)
{
    const W4Plan a = make_plan(n, k, kMaxWaves), b = make_plan(n, k, 2u * kMaxWaves);
    const size_t na = static_cast<size_t>(a.waves) * a.max_seg * kTileRows;
    const size_t nb = static_cast<size_t>(b.waves) * b.max_seg * 2u;
    return (na > nb ? na : nb) * 1024u * sizeof(float);
}

bool fast_ok(const ascq_w4a16_desc* d, const void* x, const void* w, const void* scale, const void* offset)
{
    // total_chunks must fit 32 bits with room for the 64-bit products; k % 8 == 0 keeps activation loads aligned
    return d->n % 32 == 0 && d->k % kChunkRows == 0 && d->group_size % kChunkRows == 0 && aligned16(x) &&
           aligned16(w) && aligned16(scale) && (!d->has_offset || aligned16(offset)) &&
           static_cast<uint64_t>((d->n + kColsPerBlock - 1u) / kColsPerBlock) * (d->k / kChunkRows) < (1ull << 31);
}

}  // namespace
}  // namespace ascq

using namespace ascq;

static int validate_w4(const ascq_w4a16_desc* d)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w4a16: desc is NULL");
    ASCQ_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0, ASCQ_EINVAL, "ascq_matmul_w4a16: m, n, k must be greater than 0");
    ASCQ_REQUIRE(d->n % 2 == 0, ASCQ_EINVAL, "ascq_matmul_w4a16: n must be even (two int4 per byte)");
    ASCQ_REQUIRE(d->group_size > 0 && d->k % d->group_size == 0, ASCQ_EINVAL,
                 "ascq_matmul_w4a16: k %u must be a multiple of group_size %u", d->k, d->group_size);
    return ASCQ_OK;
}

extern "C" int ascq_matmul_w4a16_workspace_size(const ascq_w4a16_desc* d, size_t* bytes)
{
    int rc = validate_w4(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_matmul_w4a16_workspace_size: bytes is NULL");
    *bytes = 0;
    if (d->k % kChunkRows == 0) {
        *bytes = workspace_need(d->n, d->k);
    }
    return ASCQ_OK;
}

// ref: include/adv_api/quantization/ascend_antiquant.h:50-54 (AscendAntiQuant<int4b_t, half>, per group along k)
extern "C" int ascq_matmul_w4a16(const ascq_w4a16_desc* d, void* y, const void* x, const void* w, const void* scale,
                                 const void* offset, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = validate_w4(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(y && x && w && scale, ASCQ_ENULL, "ascq_matmul_w4a16: y / x / w / scale is NULL");
    ASCQ_REQUIRE(!d->has_offset || offset, ASCQ_ENULL, "ascq_matmul_w4a16: offset is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    WnParams p{};
    p.x = static_cast<const uint16_t*>(x);
    p.w = static_cast<const uint8_t*>(w);
    p.scale = static_cast<const uint16_t*>(scale);
    p.offset = static_cast<const uint16_t*>(offset);
    p.partial = static_cast<float*>(workspace);
    p.y = static_cast<uint16_t*>(y);
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.group_size = d->group_size;
    p.has_offset = d->has_offset ? 1u : 0u;
    if (!fast_ok(d, x, w, scale, offset)) {
        const size_t total = static_cast<size_t>(d->m) * d->n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        w4a16_generic_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
        return launch_status("ascq_matmul_w4a16 (generic)");
    }
    const size_t need = workspace_need(d->n, d->k);
    ASCQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_matmul_w4a16: workspace of %zu bytes required (see ascq_matmul_w4a16_workspace_size)", need);
    ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_matmul_w4a16: workspace must be 16-byte aligned");
    const uint32_t col_blocks = (d->n + kColsPerBlock - 1u) / kColsPerBlock;
    auto set_plan = [&](uint32_t max_waves) {
        const W4Plan pl = make_plan(d->n, d->k, max_waves);
        p.waves = pl.waves;
        p.chunks_per_block = pl.chunks_per_block;
        p.total_chunks = pl.total_chunks;
        p.max_seg = pl.max_seg;
        p.per = pl.total_chunks / pl.waves;
        p.rem = pl.total_chunks % pl.waves;
    };
    // at most 32 activation rows per pass over the weights
    for (uint32_t m0 = 0; m0 < d->m;) {
        const uint32_t left = d->m - m0;
        p.m0 = m0;
        if (left <= 4) {
            m0 += 4u;
            set_plan(2u * kMaxWaves);  // two streams per SIMD
            const uint32_t grid = (p.waves + 7u) / 8u;
#define ASCQ_W4_GEMV(MPV)                                                           \
    do {                                                                            \
        if (d->has_offset) {                                                        \
            w4a16_gemv_kernel<MPV, true><<<grid, 512, 0, st>>>(p);                  \
        } else {                                                                    \
            w4a16_gemv_kernel<MPV, false><<<grid, 512, 0, st>>>(p);                 \
        }                                                                           \
        stream_sum_kernel<MPV><<<dim3(col_blocks, MPV), 1024, 0, st>>>(p);           \
    } while (0)
            if (left <= 2) {
                ASCQ_W4_GEMV(1);
            } else {
                ASCQ_W4_GEMV(2);
            }
#undef ASCQ_W4_GEMV
            continue;
        }
        set_plan(kMaxWaves);  // one stream per SIMD, one or two tiles of 16 rows
        const uint32_t grid = (p.waves + 3u) / 4u;
        if (left > kTileRows) {
            if (d->has_offset) {
                w4a16_tile_kernel<true, 2><<<grid, kThreads, 0, st>>>(p);
            } else {
                w4a16_tile_kernel<false, 2><<<grid, kThreads, 0, st>>>(p);
            }
            stream_sum_kernel<16, kPieceTileW4><<<dim3(col_blocks, 16), 1024, 0, st>>>(p);
            m0 += 2u * kTileRows;
        } else {
            if (d->has_offset) {
                w4a16_tile_kernel<true, 1><<<grid, kThreads, 0, st>>>(p);
            } else {
                w4a16_tile_kernel<false, 1><<<grid, kThreads, 0, st>>>(p);
            }
            stream_sum_kernel<8, kPieceTileW4><<<dim3(col_blocks, 8), 1024, 0, st>>>(p);
            m0 += kTileRows;
        }
    }
    return launch_status("ascq_matmul_w4a16");
}

// ------------------------------------------------------------------------------------------------------------ W8A16
// matmul_w8a16_nk.hip
namespace ascq {
bool w8a16_nk_supported(uint32_t k, const void* x, const void* w);
int launch_w8a16_nk(const void* x, const void* w, const void* scale, const void* offset, void* y, uint32_t m, uint32_t n,
                    uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits, uint32_t offset_bits, hipStream_t st,
                    bool channel_sum);
bool w8a16_kn_gemm_supported(uint32_t m, uint32_t k, const void* x, const void* w);
int launch_w8a16_kn_via_transpose(const void* x, const void* w, const void* scale, const void* offset, void* y,
                                  uint32_t m, uint32_t n, uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits,
                                  uint32_t offset_bits, void* workspace, hipStream_t st);
}  // namespace ascq

static int validate_w8a16(const ascq_w8a16_desc* d)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w8a16: desc is NULL");
    ASCQ_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0, ASCQ_EINVAL, "ascq_matmul_w8a16: m, n, k must be greater than 0");
    ASCQ_REQUIRE(d->out_dtype == ASCQ_F16 || d->out_dtype == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_matmul_w8a16: out_dtype must be ASCQ_F16 or ASCQ_F32");
    ASCQ_REQUIRE(d->mode == ASCQ_W8A16_PER_WEIGHT || d->mode == ASCQ_W8A16_CHANNEL_SUM, ASCQ_EINVAL,
                 "ascq_matmul_w8a16: unknown mode %d", d->mode);
    return ASCQ_OK;
}

static bool w8a16_fast_ok(const ascq_w8a16_desc* d, const void* x, const void* w, const void* scale, const void* offset)
{
    return d->n % 16 == 0 && d->k % kChunkRows == 0 && aligned16(x) && aligned16(w) &&
           (d->per_tensor || (aligned16(scale) && (!d->has_offset || aligned16(offset)))) &&
           static_cast<uint64_t>((d->n + kW8ColsPerBlock - 1u) / kW8ColsPerBlock) * (d->k / kChunkRows) < (1ull << 31);
}

static size_t w8a16_workspace_need(uint32_t n, uint32_t k)
{
    const W4Plan pl = make_plan(n, k, 2u * kMaxWaves, kW8ColsPerBlock);
    return static_cast<size_t>(pl.waves) * pl.max_seg * 8u * 1024u * sizeof(float);  // two row tiles of 4 slices
}

extern "C" int ascq_matmul_w8a16_workspace_size(const ascq_w8a16_desc* d, size_t* bytes)
{
    int rc = validate_w8a16(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_matmul_w8a16_workspace_size: bytes is NULL");
    if (d->trans_b) {
        *bytes = 0;  // whole columns per workgroup: nothing to add across workgroups
        return ASCQ_OK;
    }
    *bytes = (d->n % 16 == 0 && d->k % kChunkRows == 0) ? w8a16_workspace_need(d->n, d->k) : 0;
    if (d->m > 96u && d->k % 64u == 0) {
        // many rows: the weights are transposed into the workspace once and a tile GEMM runs on them (a smaller
        // workspace is accepted and the weight-stream kernel then passes over the weights once per 32 rows)
        const size_t need = static_cast<size_t>(d->k) * d->n;
        if (need > *bytes) {
            *bytes = need;
        }
    }
    return ASCQ_OK;
}

// ref: include/adv_api/matmul/matmul.h:161-168 (SetAntiQuantScalar / SetAntiQuantVector);
// impl/adv_api/detail/matmul/stage/copy_cube_in/antiquant/antiquant_processor_using_ub.h:53-130 (AscendAntiQuant of B)
extern "C" int ascq_matmul_w8a16(const ascq_w8a16_desc* d, void* y, const void* x, const void* w, const void* offset,
                                 const void* scale, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = validate_w8a16(d);
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(y && x && w, ASCQ_ENULL, "ascq_matmul_w8a16: y / x / w is NULL");
    ASCQ_REQUIRE(d->per_tensor || scale, ASCQ_ENULL, "ascq_matmul_w8a16: scale vector is NULL");
    ASCQ_REQUIRE(d->per_tensor || !d->has_offset || offset, ASCQ_ENULL, "ascq_matmul_w8a16: offset vector is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    WnParams p{};
    p.x = static_cast<const uint16_t*>(x);
    p.w = static_cast<const uint8_t*>(w);
    p.scale = d->per_tensor ? nullptr : static_cast<const uint16_t*>(scale);
    p.offset = d->per_tensor ? nullptr : static_cast<const uint16_t*>(offset);
    // the per-tensor scalars are halves in the reference (SrcT of SetAntiQuantScalar): one rounding here
    const _Float16 scale_h = static_cast<_Float16>(d->scale), offset_h = static_cast<_Float16>(d->offset);
    uint16_t scale_b, offset_b;
    __builtin_memcpy(&scale_b, &scale_h, 2);
    __builtin_memcpy(&offset_b, &offset_h, 2);
    p.scale_bits = scale_b;
    p.offset_bits = offset_b;
    p.partial = static_cast<float*>(workspace);
    p.y = static_cast<uint16_t*>(y);
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.has_offset = d->has_offset ? 1u : 0u;
    p.out_f32 = d->out_dtype == ASCQ_F32 ? 1u : 0u;
    p.w_nk = d->trans_b ? 1u : 0u;
    if (d->trans_b && (d->k % 128u != 0 || !w8a16_nk_supported(d->k, x, w))) {
        // k off the kernels' 128-element steps, or operands off 16-byte alignment: one lane per output element
        const size_t total = static_cast<size_t>(d->m) * d->n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        w8a16_generic_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
        return launch_status("ascq_matmul_w8a16 (generic, [n, k] weights)");
    }
    if (d->trans_b) {
        return launch_w8a16_nk(x, w, p.scale, p.offset, y, d->m, d->n, d->k, d->has_offset != 0, d->out_dtype == ASCQ_F32,
                               p.scale_bits, p.offset_bits, st, d->mode == ASCQ_W8A16_CHANNEL_SUM);
    }
    if (w8a16_kn_gemm_supported(d->m, d->k, x, w) && workspace != nullptr && aligned16(workspace) &&
        workspace_bytes >= static_cast<size_t>(d->k) * d->n) {
        return launch_w8a16_kn_via_transpose(x, w, p.scale, p.offset, y, d->m, d->n, d->k, d->has_offset != 0,
                                             d->out_dtype == ASCQ_F32, p.scale_bits, p.offset_bits, workspace, st);
    }
    if (!w8a16_fast_ok(d, x, w, scale, offset)) {
        const size_t total = static_cast<size_t>(d->m) * d->n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        w8a16_generic_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
        return launch_status("ascq_matmul_w8a16 (generic)");
    }
    const size_t need = w8a16_workspace_need(d->n, d->k);
    ASCQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_matmul_w8a16: workspace of %zu bytes required (see ascq_matmul_w8a16_workspace_size)", need);
    ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_matmul_w8a16: workspace must be 16-byte aligned");
    const W4Plan pl = make_plan(d->n, d->k, 2u * kMaxWaves, kW8ColsPerBlock);
    p.waves = pl.waves;
    p.chunks_per_block = pl.chunks_per_block;
    p.total_chunks = pl.total_chunks;
    p.max_seg = pl.max_seg;
    p.per = pl.total_chunks / pl.waves;
    p.rem = pl.total_chunks % pl.waves;
    const uint32_t col_blocks = (d->n + kW8ColsPerBlock - 1u) / kW8ColsPerBlock;
    const uint32_t grid = (p.waves + 7u) / 8u;
    // 32 activation rows per pass over the weights (16 when no more are left: fewer MFMAs and a smaller ring)
    for (uint32_t m0 = 0; m0 < d->m;) {
        p.m0 = m0;
        if (d->m - m0 > kTileRows) {
            if (d->has_offset) {
                w8a16_tile_kernel<true, 2><<<grid, 512, 0, st>>>(p);
            } else {
                w8a16_tile_kernel<false, 2><<<grid, 512, 0, st>>>(p);
            }
            stream_sum_kernel<8, kPieceTileW8><<<dim3(col_blocks, 8), 1024, 0, st>>>(p);
            m0 += 2u * kTileRows;
        } else {
            if (d->has_offset) {
                w8a16_tile_kernel<true, 1><<<grid, 512, 0, st>>>(p);
            } else {
                w8a16_tile_kernel<false, 1><<<grid, 512, 0, st>>>(p);
            }
            stream_sum_kernel<4, kPieceTileW8><<<dim3(col_blocks, 4), 1024, 0, st>>>(p);
            m0 += kTileRows;
        }
    }
    return launch_status("ascq_matmul_w8a16");
}
