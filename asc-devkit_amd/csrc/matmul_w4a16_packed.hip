// W4A16 decode GEMV / skinny GEMM on pre-packed int4 weights: one launch, one flat sweep over the weights.
//
// Packed layout (ascq_pack_weight_w4): the [k, n] matrix is cut into slabs of 16 columns and tiles of 128 k; a tile of
// a slab is 1 KiB and the tiles of a slab, then the slabs, follow each other in memory, so the 16 columns of a slab
// are one contiguous run of k / 128 KiB.  Inside a tile, lane l of a wavefront owns 16 bytes: column l % 16 of the
// slab, k = 32 (l / 16) .. + 31; dword d of the 16 bytes holds k = 32 (l / 16) + 8 d .. + 7.  A nibble is stored
// as u = w + 8 (offset binary), and the 8 nibbles of a dword sit in the order in which the 0x6400 exponent trick
// yields pairs: k offsets 0 1 2 3 4 5 6 7 live in nibbles 0 4 1 5 2 6 3 7.  Columns past n and k past the end hold
// w = 0.
//
// With that layout one 16-byte load per lane is a fully coalesced 1 KiB read and the only memory instruction a tile
// costs; a lane needs one scale and one offset per tile (a quantisation group is a multiple of 32 k), and the 8
// de-quantised halves of a dword are, as they lie in the registers, the B operand of v_mfma_f32_16x16x32_f16 for
// column l % 16 and k group l / 16: the matrix core does the multiply-accumulate and the reduction over the four k
// groups, for up to 16 activation rows at the cost of one.  Activations and the workgroup's scale / offset columns are
// staged in LDS once per pass over k (coalesced 16-byte loads); operand row i of a lane reads activation row i % m, so
// there are no zero rows to materialise (result rows >= m repeat earlier ones and are not stored).
//
// A workgroup owns whole slabs: its wavefronts split k, every wavefront streams a contiguous piece of each slab in
// batches of 4 tiles, one batch in flight while one is computed (deeper queues were slower: a compute unit keeps about
// 64 KiB of loads in flight whatever is asked of it, and a wavefront that asks for more only waits at the issue of
// its loads with data it could compute on), and the per-wavefront sums meet in LDS, where they are added in wavefront
// order and rounded once to half: no second kernel, no workspace, deterministic.
// De-quantisation follows AscendAntiQuant<int4b_t, half> exactly by default (one rounded half add of the offset, one
// rounded half multiply by the scale per weight); ASCQ_W4A16_GROUP_SUM applies scale and offset to fp32 sums per tile
// instead.  The products and sums are fp32 either way.
#include <type_traits>

#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

constexpr uint32_t kSlabCols = 16, kTileK = 128, kTileBytes = 1024;
constexpr int kBuf = 2;                  // register buffers: one batch in flight while the other is computed
constexpr uint32_t kPadTiles = 16;       // tiles of padding behind the last slab of a packed matrix (a batch may read on)
constexpr uint32_t kMaxSlabs = 8;        // slabs per workgroup
constexpr uint32_t kMaxRows = 16;        // activation rows per launch
constexpr uint32_t kPool = 152 * 1024;   // LDS of a workgroup: staged activations, parameters, per-wavefront sums
constexpr uint32_t kXBytes = 72 * 1024;  // at most this much of it for the activations of one pass over k
constexpr uint32_t kParBytes = 40 * 1024;// and this much for the (scale, offset) pairs of one pass
constexpr uint32_t kPastEnd = 0x7FFFFFF0u;  // a per-lane buffer offset beyond any buffer this kernel accepts (< 2 GiB)
constexpr int kNt = 2;                   // cache policy of the weight loads: non-temporal (read once per call)
constexpr uint32_t kRowPad = 16;         // bytes added to a staged activation row: rows start 4 banks apart

struct NibbleMasks {
    uint32_t even, odd, exp;  // 0x000F000F, 0x00F000F0, 0x64006400
    uint32_t exp_odd;         // 0x54005400: with a nibble in bits 4..7 of its mantissa the half is 64 + u
};

struct W4pParams {
    const uint16_t* x;       // [m, k] halves, first row of this launch
    const u32x4* wp;         // packed weights
    const uint16_t* scale;   // [k / group_size, n]
    const uint16_t* offset;  // same, or nullptr
    uint16_t* y;             // [m, n] halves, first row of this launch
    uint32_t m;              // rows of this launch, 1 .. 16
    uint32_t n, k;
    uint32_t gs_shift;       // log2(group_size / 32)
    uint32_t slabs, ktiles;  // ceil(n / 16), k / 128
    uint32_t slabs_per_wg;   // 1 .. kMaxSlabs
    uint32_t pass_tiles;     // tiles of k staged per pass (multiple of the wavefront count)
    uint32_t m_magic;        // ceil(2^32 / m): i / m = mulhi(i, m_magic) for i < 65536
    uint32_t par_cw;         // log2 of the lanes that share a group row when the parameters are fetched: 2^cw >= 2 slabs_per_wg
    uint32_t xs_wave, par_wave;  // bytes of staged activations / parameters per wavefront
    uint32_t par_pitch;          // entries per column of a wavefront's parameter table (odd)
    uint32_t par_off, red_off;   // byte offsets of the parameter tables and of the sums inside the LDS pool
    NibbleMasks mk;
    uint32_t red_lanes;      // lanes of a result register that hold rows < m: 16 for m <= 4, else 64
    uint32_t sum_off, sum_wave;  // group-sum form: byte offset of the activation sums in the pool, bytes per wavefront
};

__device__ __forceinline__ f16x2 bits_h2(uint32_t b)
{
    f16x2 r;
    __builtin_memcpy(&r, &b, 4);
    return r;
}
__device__ __forceinline__ uint32_t h2_bits(f16x2 h)
{
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;

// Workgroups are dealt to the 8 XCDs round-robin.  In this order the workgroups of an XCD own neighbouring column
// ranges, so the 128-byte lines of the scale / offset rows, which two or three neighbours share, are fetched once into
// that XCD's L2 instead of once per XCD (0.4 us of 24 at k = 8192, n = 28672).
__device__ __forceinline__ uint32_t xcd_order(uint32_t wg, uint32_t wgs)
{
    return (wgs & 7u) == 0u ? (wg & 7u) * (wgs >> 3) + (wg >> 3) : wg;
}

__device__ __forceinline__ uint32_t mod_m(uint32_t i, const W4pParams& p) { return i - __umulhi(i, p.m_magic) * p.m; }

// One dword of packed weights (8 consecutive k of one column, offset binary) -> the 8 de-quantised halves in k order.
// kFold: ofe holds offset - 1032 and ofo offset - 72 (both halves), exact for integer offsets of magnitude <= 512, so
// that conversion and offset are one exact operation; otherwise ofe is the offset itself.
template <bool kHasOffset, bool kFold>
__device__ __forceinline__ f16x8 dequant8(uint32_t qd, f16x2 sc, f16x2 ofe, f16x2 ofo, const NibbleMasks& mk)
{
    const f16x2 k1032 = {static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};
    const f16x2 k72 = {static_cast<half_t>(72.0f), static_cast<half_t>(72.0f)};
    const f16x2 k16th = {static_cast<half_t>(0.0625f), static_cast<half_t>(0.0625f)};
    const uint32_t qh = qd >> 8;
    f16x2 h[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t src = c < 2 ? qd : qh;
        // 1024 + u read in place (even c), 1024 + 16 u read four bits up (odd c).  The masks arrive as kernel arguments:
        // with values it cannot fold the compiler emits one v_and_or_b32 (VOP3 takes no literals) instead of two
        // instructions with literal operands.
        const uint32_t bits = (src & ((c & 1) ? mk.odd : mk.even)) | mk.exp;
        if constexpr (kHasOffset && kFold) {
            h[c] = (c & 1) ? __builtin_elementwise_fma(bits_h2(bits), k16th, ofo) : bits_h2(bits) + ofe;
        } else {
            h[c] = (c & 1) ? __builtin_elementwise_fma(bits_h2(bits), k16th, -k72) : bits_h2(bits) - k1032;  // w, exact
            if constexpr (kHasOffset) {
                h[c] = h[c] + ofe;  // one rounding
            }
        }
        h[c] = sc * h[c];  // one rounding
    }
    f16x8 b;
    __builtin_memcpy(&b, h, 16);
    return b;
}

// One dword of packed weights -> 8 halves in k order that still carry their conversion constants: k offsets 0 1 4 5
// become 1024 + u = 1032 + w, k offsets 2 3 6 7 become 64 + u = 72 + w.  Four v_and_or_b32 and one shift.
__device__ __forceinline__ f16x8 raw8(uint32_t qd, const NibbleMasks& mk)
{
    const uint32_t qh = qd >> 8;
    uint32_t h[4];
    h[0] = (qd & mk.even) | mk.exp;
    h[1] = (qd & mk.odd) | mk.exp_odd;
    h[2] = (qh & mk.even) | mk.exp;
    h[3] = (qh & mk.odd) | mk.exp_odd;
    f16x8 b;
    __builtin_memcpy(&b, h, 16);
    return b;
}
// The same with every nibble moved into bits 4..7 of its half first (three shifts instead of one): all 8 halves are
// 64 + u = 72 + w.
__device__ __forceinline__ f16x8 raw8_72(uint32_t qd, const NibbleMasks& mk)
{
    uint32_t h[4];
    h[0] = ((qd << 4) & mk.odd) | mk.exp_odd;
    h[1] = (qd & mk.odd) | mk.exp_odd;
    h[2] = ((qd >> 4) & mk.odd) | mk.exp_odd;
    h[3] = ((qd >> 8) & mk.odd) | mk.exp_odd;
    f16x8 b;
    __builtin_memcpy(&b, h, 16);
    return b;
}
constexpr float kBiasEven = 1032.0f, kBiasOdd = 72.0f;  // what raw8 adds to w at k offsets 0 1 4 5 / 2 3 6 7

// kSum = 0: every weight is de-quantised as AscendAntiQuant does it (two roundings to half per weight).
// kSum = 4 (the group-sum form; the number of result registers carried, a power of two up to 4; group_size a multiple
// of 128): the matrix core
// multiplies the activations with the raw halves of raw8 and scale and offset are applied once per tile of 128 k to the
// fp32 sum,  y += scale * (sum_k x_k (w_k + c_k) - sum_k x_k c_k + offset * sum_k x_k),  where the two sums over the
// activations alone are formed once per wavefront and tile before the weights arrive.
template <bool kHasOffset, uint32_t kWaves, uint32_t kBatch, uint32_t kSum>
__global__ __launch_bounds__(kWaves * 64) void w4a16_packed_kernel(W4pParams p)
{
    constexpr uint32_t kThreadsWg = kWaves * 64u;
    constexpr uint32_t kParPieces = 3;  // 8-column parameter pieces per lane (the host keeps a wavefront's table within that)
    __shared__ __attribute__((aligned(16))) char POOL[kPool];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j = lane & 15u, g = lane >> 4;
    // every wavefront stages what its own share of k needs and reads nothing another wavefront wrote: no barriers
    // until the final sum
    char* const XS = POOL + wave * p.xs_wave;               // [m][tiles per wavefront * 128 halves + pad]
    char* const PAR = POOL + p.par_off + wave * p.par_wave;  // [column of the workgroup][group of the wavefront's k] (scale | offset << 16)
    float* const RED = reinterpret_cast<float*>(POOL + p.red_off);    // [wave][slab][register][lane < red_lanes]

    const uint32_t spw = p.slabs_per_wg;
    const uint32_t slab0 = xcd_order(blockIdx.x, gridDim.x) * spw;
    const uint32_t nslabs = min(spw, p.slabs - slab0);
    const uint32_t tpw = p.pass_tiles / kWaves;             // tiles of a pass per wavefront
    const uint32_t pitch = tpw * kTileK * 2u + kRowPad;     // bytes of a staged activation row
    const uint32_t x_lane = mod_m(lane & 15u, p) * pitch + g * 64u;  // operand row i reads row i % m; + tile * 256 + d * 16
    const uint32_t row_bytes = p.n * 2u;                          // one row of scale / offset in memory
    const uint32_t par_col = p.par_pitch * 4u;                    // bytes of one column of the table in LDS (odd number of entries)
    // The quantisation group of a lane's 32 k, (4 tile + g) / (group_size / 32) with group_size / 32 = 2^s, splits into
    // a part that is the same for every lane, (4 tile) >> s, and a per-lane constant, g >> s (s <= 2); for s > 2 the
    // lanes of a tile share one group, tile >> (s - 2).
    const uint32_t gsh = p.gs_shift;
    const uint32_t par_lane0 = (gsh <= 2u ? (g >> gsh) * 4u : 0u) + j * par_col;  // + slab * 16 columns

    // Buffer descriptors: a load takes a per-lane 32-bit offset (range-checked: an offset past the end makes the load
    // return zero without moving data) and a scalar offset that moves with the tile (not range-checked), so no vector
    // instruction is spent on weight addresses inside the loop.
    // the exponent constant lives in a vector register so that mask (scalar) and constant fit one v_and_or_b32
    NibbleMasks mk = p.mk;
    asm volatile("" : "+v"(mk.exp));
    if constexpr (kSum != 0u) {
        asm volatile("" : "+v"(mk.exp_odd));
    }
    char* const SUM = POOL + p.sum_off + wave * p.sum_wave;  // [tile of the wavefront's share][sums of rows 0..3 | -weighted sums]
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<u32x4*>(p.wp), 0, static_cast<int>((p.slabs * p.ktiles + kPadTiles) * kTileBytes), 0x00020000);
    const int par_bytes = static_cast<int>(((p.k / 32u) >> gsh) * row_bytes);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.scale), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(kHasOffset ? p.offset : p.scale), 0, par_bytes, 0x00020000);

    // sums of this wavefront per slab, kept in LDS between passes
    const uint32_t rl = p.red_lanes, red_wave = spw * 4u * rl;  // floats per wavefront
    float* red = RED + wave * red_wave;

    for (uint32_t pt0 = 0; pt0 < p.ktiles; pt0 += p.pass_tiles) {
        const uint32_t ptiles = min(p.pass_tiles, p.ktiles - pt0);
        // ---- this wavefront's work of the pass: tiles [ta, tb) (relative to pt0) of each of its slabs, in batches of
        // kBatch tiles that never straddle a slab: batch q = (slab q / nb, tiles ta + (q % nb) kBatch ...)
        const uint32_t ta = min(wave * tpw, ptiles), tb = min(ta + tpw, ptiles);
        const uint32_t cnt = tb - ta;
        const uint32_t nb = (cnt + kBatch - 1u) / kBatch;
        const uint32_t batches = nb * nslabs;
        const uint32_t g_base = ((pt0 + ta) * 4u) >> gsh;                                          // first group of its k
        const uint32_t g_rows = cnt != 0u ? ((((pt0 + tb) * 4u - 1u) >> gsh) - g_base + 1u) : 0u;  // groups it touches

        // Every weight load is unconditional, so the loop body is straight-line as far as memory loads go and the waits
        // the compiler inserts count exactly: one batch stays in flight while the other is computed.  Once every batch
        // has been requested the per-lane offset points past the end of the buffer and the loads of the loop's last
        // rounds are dropped.
        u32x4 wq[kBuf][kBatch];
        uint32_t l_slab = slab0, l_b = 0, l_q = 0;  // load cursor: slab, batch within the slab, batch number
        bool l_done = batches == 0u;               // every batch has been requested
        auto load = [&](int buf) __attribute__((always_inline)) {
            const uint32_t l_w = l_done ? kPastEnd : lane * 16u;
            // tiles past the wavefront's range (a short last batch) read on into the next tiles or the padding behind the
            // last slab: valid memory, not computed
            const uint32_t base = (l_slab * p.ktiles + pt0 + ta + l_b * kBatch) * kTileBytes;  // scalar
#pragma unroll
            for (uint32_t t = 0; t < kBatch; ++t) {
                wq[buf][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, l_w, base + t * kTileBytes, kNt);
            }
            if (l_q + 1u < batches) {  // uniform
                ++l_q;
                if (++l_b == nb) {
                    l_b = 0;
                    ++l_slab;
                }
            } else {
                l_done = true;
            }
        };

        // ---- The wavefront's activations (m rows x its tiles' k) go straight into its part of the LDS, 1 KiB of a row
        // per instruction; its parameters (its groups x the workgroup's columns) travel through registers.  Loads
        // return in order, so the wait for these leaves the two weight batches requested behind them in flight.  (These
        // small loads go first: a compute unit's queue is served in order, and behind the weight batches of eight
        // wavefronts they would arrive microseconds later.)
        {
            const uint32_t row_pieces = cnt * (kTileK / 8u);
            for (uint32_t r = 0; r < p.m; ++r) {
                const uint16_t* src = p.x + static_cast<size_t>(r) * p.k + (pt0 + ta) * kTileK + lane * 8u;
                for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                    if (c0 + lane < row_pieces) {
                        __builtin_amdgcn_global_load_lds((gptr_t)(src + c0 * 8u), (lds_ptr_t)(XS + r * pitch + c0 * 16u), 16, 0, 0);
                    }
                }
            }
        }
        // Parameter piece (8 columns) of lane l in round u: column piece l % 2^cw, group row (l >> cw) + u (64 >> cw),
        // 2^cw >= 2 slabs_per_wg.
        u32x4 sr[kParPieces], orr[kParPieces];
        const uint32_t par_c = lane & ((1u << p.par_cw) - 1u), par_r0 = lane >> p.par_cw, par_rstep = 64u >> p.par_cw;
#pragma unroll
        for (uint32_t u = 0; u < kParPieces; ++u) {
            const uint32_t r = par_r0 + u * par_rstep;
            const uint32_t col = slab0 * kSlabCols + par_c * 8u;
            const uint32_t off = (r < g_rows && par_c < 2u * spw && col < p.n) ? ((g_base + r) * p.n + col) * 2u : kPastEnd;
            sr[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
            if constexpr (kHasOffset) {
                orr[u] = __builtin_amdgcn_raw_buffer_load_b128(ro, off, 0, 0);
            }
        }
#pragma unroll
        for (int b = 0; b < kBuf; ++b) load(b);
        // Loads return in order: once at most the weight loads just issued are outstanding, the activations have landed
        // in LDS.  The compiler does not count direct-to-LDS loads issued in a loop; told here, with a wait it
        // understands, it neither reads the LDS early nor waits for the weights in front of every LDS read.
        __builtin_amdgcn_s_waitcnt(((kBuf * kBatch) & 15u) | (((kBuf * kBatch) >> 4) << 14) | (7u << 4) | (15u << 8));
        asm volatile("" ::: "memory");
        if (pt0 == 0u && lane < rl) {  // sums of this wavefront per slab, kept in LDS between passes
            for (uint32_t s = 0; s < nslabs * 4u; ++s) red[s * rl + lane] = 0.0f;
        }
#pragma unroll
        for (uint32_t u = 0; u < kParPieces; ++u) {
            const uint32_t r = par_r0 + u * par_rstep;
            if (r < g_rows && par_c < 2u * spw) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t o2 = kHasOffset ? orr[u][e] : 0u;
                    char* dst = PAR + (par_c * 8u + 2u * e) * par_col + r * 4u;
                    *reinterpret_cast<uint32_t*>(dst) = __builtin_amdgcn_perm(o2, sr[u][e], 0x05040100u);            // (s, o) of column 2e
                    *reinterpret_cast<uint32_t*>(dst + par_col) = __builtin_amdgcn_perm(o2, sr[u][e], 0x07060302u);  // column 2e + 1
                }
            }
        }
        if (batches == 0u) {
            continue;  // uniform over the wavefront
        }
        if constexpr (kSum != 0u) {
            // Sums of the staged activations per tile: lane = (tile of the round, result register r, one of 8 parts of
            // 16 k), 8 / kSum tiles per round; register r of the lanes that are stored holds row r % m.  Per part the
            // k offsets 0 1 4 5 (mod 8) and 2 3 6 7 are summed apart, the 8 parts are added across lanes, and the table
            // keeps  sum x  and  -(1032 sum_even x + 72 sum_odd x)  per tile and register.
            constexpr uint32_t kTilesRound = 8u / kSum;
            const uint32_t part = lane & 7u, reg = (lane >> 3) & (kSum - 1u);
            const uint32_t srow = kSum == 1u ? 0u : mod_m(reg, p);
            for (uint32_t t2 = 0; t2 < cnt; t2 += kTilesRound) {
                const uint32_t tt = t2 + (lane >> 3) / kSum;
                const char* src = XS + srow * pitch + min(tt, cnt - 1u) * 256u + part * 32u;
                float se = 0.0f, so = 0.0f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const f16x8 v = *reinterpret_cast<const f16x8*>(src + h * 16);
                    se += (static_cast<float>(v[0]) + static_cast<float>(v[1])) + (static_cast<float>(v[4]) + static_cast<float>(v[5]));
                    so += (static_cast<float>(v[2]) + static_cast<float>(v[3])) + (static_cast<float>(v[6]) + static_cast<float>(v[7]));
                }
                // add over the 8 parts: lane ^ 1, lane ^ 2 inside a quad, then the mirrored half row (the other quad)
                se += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(se), 0xB1, 0xF, 0xF, true));
                so += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(so), 0xB1, 0xF, 0xF, true));
                se += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(se), 0x4E, 0xF, 0xF, true));
                so += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(so), 0x4E, 0xF, 0xF, true));
                se += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(se), 0x141, 0xF, 0xF, true));
                so += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(so), 0x141, 0xF, 0xF, true));
                if (part == 0u && tt < cnt) {
                    float* dst = reinterpret_cast<float*>(SUM + tt * 32u);
                    dst[reg] = se + so;
                    dst[4u + reg] = -(kBiasEven * se + kBiasOdd * so);
                }
            }
        }

        f32x4 acc[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
        uint32_t c_slab = 0, c_b = 0, c_q = 0;  // compute cursor (slab relative to slab0)
        auto compute = [&](int buf) __attribute__((always_inline)) {
            // The batch in this buffer has landed once at most the loads of the other buffers, issued behind it, are
            // outstanding.  Said with a wait the compiler understands: left to count across the loop's back edge
            // itself it waits for every load here, the batch just requested included, and half of the overlap between
            // loads and arithmetic is gone (0.5 us of 24 at k = 8192, n = 28672).
            constexpr uint32_t kBehind = (kBuf - 1) * kBatch;
            __builtin_amdgcn_s_waitcnt((kBehind & 15u) | ((kBehind >> 4) << 14) | (7u << 4) | (15u << 8));
            const bool on = c_q < batches;  // uniform; past the last batch nothing but arithmetic is skipped
            const uint32_t t0 = on ? ta + c_b * kBatch : ta;       // first tile of the batch, relative to pt0
            const uint32_t live = on ? min(kBatch, tb - t0) : 0u;  // tiles of the batch inside the range
            const char* xa0 = XS + x_lane + (t0 - ta) * 256u;
            // (scale, offset) of every tile of the batch; whether every offset is an integer of magnitude <= 512 (it
            // survives (o + 1536) - 1536): then conversion and offset are one exact operation.  With group_size 128 the
            // tiles' entries are consecutive, one address serves the batch; a tile past the range reads on into the next
            // column's entries (or, behind the last table, into the sums: still inside the pool) and is not computed.
            const uint32_t tt0 = pt0 + t0;
            const char* pa0 = PAR + par_lane0 + c_slab * (kSlabCols * par_col) +
                              ((gsh <= 2u ? (tt0 * 4u) >> gsh : tt0 >> (gsh - 2u)) - g_base) * 4u;
            uint32_t pp[kBatch];
            uint32_t frac = 0;
            if (gsh == 2u) {
#pragma unroll
                for (uint32_t t = 0; t < kBatch; ++t) pp[t] = *reinterpret_cast<const uint32_t*>(pa0 + t * 4u);
            } else {
#pragma unroll
                for (uint32_t t = 0; t < kBatch; ++t) {
                    const uint32_t tt = tt0 + t;
                    const uint32_t grow = (gsh <= 2u ? (tt * 4u) >> gsh : tt >> (gsh - 2u)) - (gsh <= 2u ? (tt0 * 4u) >> gsh : tt0 >> (gsh - 2u));
                    pp[t] = *reinterpret_cast<const uint32_t*>(pa0 + grow * 4u);
                }
            }
            if constexpr (kHasOffset && kSum == 0u) {
#pragma unroll
                for (uint32_t t = 0; t < kBatch; ++t) {
                    const f16x2 k1536 = {static_cast<half_t>(1536.0f), static_cast<half_t>(1536.0f)};
                    const f16x2 rt = (bits_h2(pp[t]) + k1536) - k1536;
                    frac |= (h2_bits(rt) ^ pp[t]) & 0x7FFF0000u;  // the offset is the high half
                }
            }
            const bool fold = kHasOffset && kSum == 0u && __builtin_amdgcn_ballot_w64(frac != 0u) == 0;  // uniform
            auto tiles = [&](auto folded) __attribute__((always_inline)) {
                constexpr bool kFold = decltype(folded)::value;
#pragma unroll
                for (uint32_t t = 0; t < kBatch; ++t) {
                    if (t < live) {  // uniform; no memory loads inside, so the wait counts stay exact
                        if constexpr (kSum != 0u) {
                            const f16x2 sp = bits_h2(pp[t]);
                            const float scf = static_cast<float>(sp[0]), off = static_cast<float>(sp[1]);
                            const char* sm = SUM + (t0 - ta + t) * 32u;
                            const f32x4 xs = *reinterpret_cast<const f32x4*>(sm);
                            f32x4 part = *reinterpret_cast<const f32x4*>(sm + 16);
#pragma unroll
                            for (int d = 0; d < 4; ++d) {
                                const f16x8 a = *reinterpret_cast<const f16x8*>(xa0 + t * 256u + d * 16);
                                part = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, raw8(wq[buf][t][d], mk), part, 0, 0, 0);
                            }
#pragma unroll
                            for (uint32_t r = 0; r < kSum; ++r) {
                                acc[0][r] = __builtin_fmaf(scf, kHasOffset ? __builtin_fmaf(off, xs[r], part[r]) : part[r], acc[0][r]);
                            }
                            continue;
                        }
                        const f16x2 sp = bits_h2(pp[t]);
                        const f16x2 sc = {sp[0], sp[0]};
                        f16x2 ofe = {sp[1], sp[1]}, ofo = ofe;
                        if constexpr (kFold) {
                            ofo = ofe - f16x2{static_cast<half_t>(72.0f), static_cast<half_t>(72.0f)};    // exact
                            ofe = ofe - f16x2{static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};  // exact
                        }
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const f16x8 a = *reinterpret_cast<const f16x8*>(xa0 + t * 256u + d * 16);
                            const f16x8 b = dequant8<kHasOffset, kFold>(wq[buf][t][d], sc, ofe, ofo, mk);
                            acc[d & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[d & 1], 0, 0, 0);
                        }
                    }
                }
            };
            if (fold) {
                tiles(std::true_type{});
            } else {
                tiles(std::false_type{});
            }
            ++c_q;
            if (on && ++c_b == nb) {  // the slab is done for this pass: add to the wavefront's sums in LDS
                if (lane < rl) {
                    float* dst = red + c_slab * 4u * rl + lane;
#pragma unroll
                    for (int r = 0; r < 4; ++r) dst[r * rl] += acc[0][r] + acc[1][r];
                }
                acc[0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                acc[1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                c_b = 0;
                ++c_slab;
            }
        };

        for (uint32_t q = 0; q < batches; q += kBuf) {
#pragma unroll
            for (int b = 0; b < kBuf; ++b) {
                compute(b);
                load(b);
            }
        }
    }

    // ---- add the wavefronts' sums in wavefront order, round once, store
    __syncthreads();
    const uint32_t outs = nslabs * p.m * kSlabCols;
    for (uint32_t i = tid; i < outs; i += kThreadsWg) {
        const uint32_t s = i / (p.m * kSlabCols), rc = i % (p.m * kSlabCols);
        const uint32_t r = rc / kSlabCols, c = rc % kSlabCols;
        const uint32_t col = (slab0 + s) * kSlabCols + c;
        // result row r of column c: lane 16 (r / 4) + c, register r % 4
        const uint32_t at = (s * 4u + (r & 3u)) * rl + (r >> 2) * 16u + c;
        float sum = 0.0f;
#pragma unroll
        for (uint32_t w = 0; w < kWaves; ++w) sum += RED[w * red_wave + at];
        if (col < p.n) {
            p.y[static_cast<size_t>(r) * p.n + col] = static_cast<uint16_t>(f32_to_half_bits(sum));
        }
    }
}

// 5 to 16 activation rows: the activations of a whole pass over k no longer fit the LDS wavefront by wavefront (the
// kernel above would need several passes, each refetching parameters and restarting its stream), so the roles turn
// round.  A wavefront owns one slab over all of k: its weights are one contiguous run and the sums of its 16 columns
// never leave its registers - no reduction in LDS, no second pass.  The wavefronts of a workgroup walk k together and
// share the activations: chunk c (8 tiles = 1024 k of all m rows) lies in one of two LDS buffers while the next is
// fetched, one barrier per chunk.  The (scale, offset) pairs of a slab for all of k are staged once per wavefront.
constexpr int kRowsBuf = 2;              // weight buffers: one batch in flight while the other is computed
constexpr uint32_t kRowsBatch = 8;          // tiles per batch of weight loads = tiles per activation chunk
constexpr uint32_t kRowsMaxGroups = 128;    // quantisation groups along k this kernel has LDS for
constexpr uint32_t kRowsChunkBytes = kRowsBatch * kTileK * 2u;  // bytes of one activation row per chunk
constexpr uint32_t kRowsPitch = kRowsChunkBytes + kRowPad;

// kSumForm (group_size a multiple of 128): raw weight halves on the matrix core, all of them 72 + w (raw8_72), scale and
// offset applied once per tile to fp32 sums.  The sum of the activations that both the offset and the 72 multiply comes
// from the matrix core as well - a second product of the same activations with an operand of ones:
//   y += scale * (sum_k x_k (w_k + 72) + (offset - 72) * sum_k x_k).
// The rows differ from lane to lane here, so a table of such sums would cost more vector instructions than the
// de-quantisation it replaces, while the matrix pipe has room.
template <bool kHasOffset, uint32_t kW, bool kSumForm>
__global__ __launch_bounds__(kW * 64) void w4a16_packed_rows_kernel(W4pParams p)
{
    constexpr uint32_t kT = kW * 64u;
    constexpr uint32_t kXP = (kMaxRows * kRowsChunkBytes / 16u + kT - 1u) / kT;  // 16-byte pieces per thread and chunk
    constexpr uint32_t kParWave = kSlabCols * (kRowsMaxGroups + 1u) * 4u;
    __shared__ __attribute__((aligned(16))) char XS[2][kMaxRows * kRowsPitch];
    __shared__ __attribute__((aligned(16))) char PARS[kW * kParWave];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j = lane & 15u, g = lane >> 4;
    const uint32_t slab = xcd_order(blockIdx.x, gridDim.x) * kW + wave;
    const bool live = slab < p.slabs;  // a wavefront without a slab still stages activations and meets the barriers
    char* const PAR = PARS + wave * kParWave;  // [column of the slab][group] (scale | offset << 16)
    const uint32_t gsh = p.gs_shift;
    const uint32_t groups = (p.k / 32u) >> gsh;
    const uint32_t par_col = p.par_pitch * 4u;  // bytes of one column of the table (odd number of entries)
    const uint32_t par_lane0 = (gsh <= 2u ? (g >> gsh) * 4u : 0u) + j * par_col;
    const uint32_t x_lane = (j % p.m) * kRowsPitch + g * 64u;  // operand row i reads row i % m; + tile * 256 + d * 16
    const uint32_t nb = (p.ktiles + kRowsBatch - 1u) / kRowsBatch;

    NibbleMasks mk = p.mk;
    asm volatile("" : "+v"(mk.exp));
    f16x8 b_one;  // the constant B operand of the group-sum form, kept in vector registers
    if constexpr (kSumForm) {
        asm volatile("" : "+v"(mk.exp_odd));
        const f16x2 one = {static_cast<half_t>(1.0f), static_cast<half_t>(1.0f)};
        const f16x2 ho[4] = {one, one, one, one};
        __builtin_memcpy(&b_one, ho, 16);
        asm volatile("" : "+v"(b_one));
    }
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<u32x4*>(p.wp), 0, static_cast<int>((p.slabs * p.ktiles + kPadTiles) * kTileBytes), 0x00020000);
    const int par_bytes = static_cast<int>(groups * p.n * 2u);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.scale), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(kHasOffset ? p.offset : p.scale), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.x), 0, static_cast<int>(p.m * p.k * 2u), 0x00020000);

    // ---- the slab's parameters: lane i fetches 8 columns of group row r0 + i / 2
    for (uint32_t r0 = 0; r0 < groups; r0 += 32u) {
        const uint32_t r = r0 + (lane >> 1), c8 = (lane & 1u) * 8u;
        const uint32_t col = slab * kSlabCols + c8;
        const uint32_t off = (live && r < groups && col < p.n) ? (r * p.n + col) * 2u : kPastEnd;
        const u32x4 sr = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
        u32x4 orr = u32x4{0, 0, 0, 0};
        if constexpr (kHasOffset) {
            orr = __builtin_amdgcn_raw_buffer_load_b128(ro, off, 0, 0);
        }
        if (r < groups) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                char* dst = PAR + (c8 + 2u * e) * par_col + r * 4u;
                *reinterpret_cast<uint32_t*>(dst) = __builtin_amdgcn_perm(orr[e], sr[e], 0x05040100u);            // column 2e
                *reinterpret_cast<uint32_t*>(dst + par_col) = __builtin_amdgcn_perm(orr[e], sr[e], 0x07060302u);  // column 2e + 1
            }
        }
    }

    // ---- activations of chunk c: piece i (16 bytes) is piece i % 128 of row i / 128
    u32x4 xr[kXP];
    auto xload = [&](uint32_t c) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t u = 0; u < kXP; ++u) {
            const uint32_t i = tid + u * kT;
            const uint32_t r = i >> 7, kk = c * (kRowsBatch * kTileK) + (i & 127u) * 8u;
            xr[u] = __builtin_amdgcn_raw_buffer_load_b128(rx, (c < nb && r < p.m && kk < p.k) ? (r * p.k + kk) * 2u : kPastEnd, 0, 0);
        }
    };
    auto xstore = [&](uint32_t c) __attribute__((always_inline)) {
        char* dst = XS[c & 1u];
#pragma unroll
        for (uint32_t u = 0; u < kXP; ++u) {
            const uint32_t i = tid + u * kT;
            const uint32_t r = i >> 7;
            if (c < nb && r < p.m) {
                *reinterpret_cast<u32x4*>(dst + r * kRowsPitch + (i & 127u) * 16u) = xr[u];
            }
        }
    };
    // ---- weights of batch q: unconditional loads (a batch past the end, or of a wavefront without a slab, is given an
    // offset beyond the buffer and moves no data; the last batch may read on into the next slab or the padding)
    u32x4 wq[kRowsBuf][kRowsBatch];
    auto wload = [&](int buf, uint32_t q) __attribute__((always_inline)) {
        const uint32_t l_w = (live && q < nb) ? lane * 16u : kPastEnd;
        const uint32_t base = (slab * p.ktiles + q * kRowsBatch) * kTileBytes;  // scalar
#pragma unroll
        for (uint32_t t = 0; t < kRowsBatch; ++t) {
            wq[buf][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, l_w, base + t * kTileBytes, kNt);
        }
    };

    f32x4 acc[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
    auto compute = [&](int buf, uint32_t q) __attribute__((always_inline)) {
        const uint32_t tt0 = q * kRowsBatch;
        const uint32_t live_t = min(kRowsBatch, p.ktiles - tt0);
        const char* xa0 = XS[q & 1u] + x_lane;
        const char* pa0 = PAR + par_lane0 + (gsh <= 2u ? (tt0 * 4u) >> gsh : tt0 >> (gsh - 2u)) * 4u;
        uint32_t pp[kRowsBatch];
        uint32_t frac = 0;
        if (gsh == 2u) {
#pragma unroll
            for (uint32_t t = 0; t < kRowsBatch; ++t) pp[t] = *reinterpret_cast<const uint32_t*>(pa0 + t * 4u);
        } else {
#pragma unroll
            for (uint32_t t = 0; t < kRowsBatch; ++t) {
                const uint32_t tt = tt0 + t;
                const uint32_t grow = (gsh <= 2u ? (tt * 4u) >> gsh : tt >> (gsh - 2u)) - (gsh <= 2u ? (tt0 * 4u) >> gsh : tt0 >> (gsh - 2u));
                pp[t] = *reinterpret_cast<const uint32_t*>(pa0 + grow * 4u);
            }
        }
        if constexpr (kHasOffset && !kSumForm) {
#pragma unroll
            for (uint32_t t = 0; t < kRowsBatch; ++t) {
                const f16x2 k1536 = {static_cast<half_t>(1536.0f), static_cast<half_t>(1536.0f)};
                const f16x2 rt = (bits_h2(pp[t]) + k1536) - k1536;
                frac |= (h2_bits(rt) ^ pp[t]) & 0x7FFF0000u;  // the offset is the high half
            }
        }
        const bool fold = kHasOffset && !kSumForm && __builtin_amdgcn_ballot_w64(frac != 0u) == 0;  // uniform
        auto tiles = [&](auto folded) __attribute__((always_inline)) {
            constexpr bool kFold = decltype(folded)::value;
#pragma unroll
            for (uint32_t t = 0; t < kRowsBatch; ++t) {
                if (t < live_t) {  // uniform
                    if constexpr (kSumForm) {
                        const f16x2 sp = bits_h2(pp[t]);
                        const float scf = static_cast<float>(sp[0]), off = static_cast<float>(sp[1]);
                        const float off72 = (kHasOffset ? off : 0.0f) - kBiasOdd;
                        f32x4 part = {0.0f, 0.0f, 0.0f, 0.0f}, xs = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const f16x8 a = *reinterpret_cast<const f16x8*>(xa0 + t * 256u + d * 16);
                            xs = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_one, xs, 0, 0, 0);
                            part = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, raw8_72(wq[buf][t][d], mk), part, 0, 0, 0);
                        }
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            acc[0][r] = __builtin_fmaf(scf, __builtin_fmaf(off72, xs[r], part[r]), acc[0][r]);
                        }
                        continue;
                    }
                    const f16x2 sp = bits_h2(pp[t]);
                    const f16x2 sc = {sp[0], sp[0]};
                    f16x2 ofe = {sp[1], sp[1]}, ofo = ofe;
                    if constexpr (kFold) {
                        ofo = ofe - f16x2{static_cast<half_t>(72.0f), static_cast<half_t>(72.0f)};      // exact
                        ofe = ofe - f16x2{static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};  // exact
                    }
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const f16x8 a = *reinterpret_cast<const f16x8*>(xa0 + t * 256u + d * 16);
                        const f16x8 b = dequant8<kHasOffset, kFold>(wq[buf][t][d], sc, ofe, ofo, mk);
                        acc[d & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[d & 1], 0, 0, 0);
                    }
                }
            }
        };
        if (fold) {
            tiles(std::true_type{});
        } else {
            tiles(std::false_type{});
        }
    };

    // One step: request the activations of the next chunk, compute, then request the weights of the batch after next
    // into the buffer just computed (one batch in flight while one is computed: deeper queues were slower), hand the
    // activations over - loads return in order, so that wait leaves the batch just requested in flight - and meet the
    // other wavefronts.
    auto step = [&](int buf, uint32_t q) __attribute__((always_inline)) {
        xload(q + 1u);
        if (live && q < nb) {  // uniform over the wavefront
            compute(buf, q);
        }
        wload(buf, q + kRowsBuf);
        xstore(q + 1u);
        __syncthreads();
    };
    xload(0);
#pragma unroll
    for (int b = 0; b < kRowsBuf; ++b) wload(b, b);
    xstore(0);
    __syncthreads();
    for (uint32_t q = 0; q < nb; q += kRowsBuf) {
#pragma unroll
        for (int b = 0; b < kRowsBuf; ++b) step(b, q + b);
    }

    // ---- result row 4 (lane / 16) + r of column lane % 16: one rounding to half
    const uint32_t col = slab * kSlabCols + j;
    if (live && col < p.n) {
#pragma unroll
        for (uint32_t r = 0; r < 4; ++r) {
            const uint32_t row = 4u * g + r;
            if (row < p.m) {
                p.y[static_cast<size_t>(row) * p.n + col] = static_cast<uint16_t>(f32_to_half_bits(acc[0][r] + acc[1][r]));
            }
        }
    }
}

// ND [k, n / 2] (even column in the low nibble, two's complement) -> packed; one thread per lane of a tile.
__global__ __launch_bounds__(256) void pack_w4_kernel(const uint8_t* __restrict__ w, u32x4* __restrict__ out, uint32_t k,
                                                      uint32_t n, uint32_t slabs, uint32_t ktiles)
{
    const size_t total = static_cast<size_t>(slabs) * ktiles * 64u;
    const size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x;
    if (i >= total + kPadTiles * 64u) {
        return;
    }
    if (i >= total) {  // padding behind the last slab: w = 0
        out[i] = u32x4{0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};
        return;
    }
    const uint32_t lane = static_cast<uint32_t>(i & 63u);
    const size_t tile_id = i >> 6;
    const uint32_t slab = static_cast<uint32_t>(tile_id / ktiles), tile = static_cast<uint32_t>(tile_id % ktiles);
    const uint32_t col = slab * kSlabCols + (lane & 15u), g = lane >> 4;
    const size_t row_bytes = n / 2u;
    u32x4 v;
#pragma unroll
    for (uint32_t d = 0; d < 4; ++d) {
        uint32_t word = 0;
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t kk = tile * kTileK + g * 32u + d * 8u + e;
            uint32_t u = 8u;  // w = 0
            if (kk < k && col < n) {
                const uint8_t byte = w[static_cast<size_t>(kk) * row_bytes + col / 2u];
                u = ((col & 1u) ? (byte >> 4) : (byte & 15u)) ^ 8u;
            }
            const uint32_t nib = (e >> 1) + 4u * (e & 1u);  // k offsets 0..7 -> nibbles 0 4 1 5 2 6 3 7
            word |= u << (4u * nib);
        }
        v[d] = word;
    }
    out[i] = v;
}

}  // namespace
}  // namespace ascq

using namespace ascq;

extern "C" int ascq_pack_weight_w4_size(uint32_t k, uint32_t n, size_t* bytes)
{
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_pack_weight_w4_size: bytes is NULL");
    ASCQ_REQUIRE(k > 0 && n > 0 && n % 2 == 0, ASCQ_EINVAL, "ascq_pack_weight_w4_size: k, n must be positive and n even");
    *bytes = (static_cast<size_t>((n + kSlabCols - 1u) / kSlabCols) * ((k + kTileK - 1u) / kTileK) + kPadTiles) * kTileBytes;
    return ASCQ_OK;
}

extern "C" int ascq_pack_weight_w4(const void* w, void* packed, uint32_t k, uint32_t n, void* stream)
{
    ASCQ_REQUIRE(w && packed, ASCQ_ENULL, "ascq_pack_weight_w4: w / packed is NULL");
    ASCQ_REQUIRE(k > 0 && n > 0 && n % 2 == 0, ASCQ_EINVAL, "ascq_pack_weight_w4: k, n must be positive and n even");
    ASCQ_REQUIRE(aligned16(packed), ASCQ_EALIGN, "ascq_pack_weight_w4: packed must be 16-byte aligned");
    const uint32_t slabs = (n + kSlabCols - 1u) / kSlabCols, ktiles = (k + kTileK - 1u) / kTileK;
    const size_t lanes = (static_cast<size_t>(slabs) * ktiles + kPadTiles) * 64u;
    ASCQ_REQUIRE((lanes + 255u) / 256u < (1ull << 31), ASCQ_EINVAL, "ascq_pack_weight_w4: matrix too large");
    pack_w4_kernel<<<static_cast<uint32_t>((lanes + 255u) / 256u), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t*>(w), static_cast<u32x4*>(packed), k, n, slabs, ktiles);
    return launch_status("ascq_pack_weight_w4");
}

// ref: include/adv_api/quantization/ascend_antiquant.h:50-54 (AscendAntiQuant<int4b_t, half>, per group along k)
extern "C" int ascq_matmul_w4a16_packed(const ascq_w4a16_desc* d, void* y, const void* x, const void* w_packed,
                                        const void* scale, const void* offset, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_matmul_w4a16_packed: desc is NULL");
    ASCQ_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0, ASCQ_EINVAL, "ascq_matmul_w4a16_packed: m, n, k must be greater than 0");
    ASCQ_REQUIRE(d->n % 2 == 0, ASCQ_EINVAL, "ascq_matmul_w4a16_packed: n must be even (two int4 per byte)");
    ASCQ_REQUIRE(d->group_size > 0 && d->k % d->group_size == 0, ASCQ_EINVAL,
                 "ascq_matmul_w4a16_packed: k %u must be a multiple of group_size %u", d->k, d->group_size);
    ASCQ_REQUIRE(y && x && w_packed && scale, ASCQ_ENULL, "ascq_matmul_w4a16_packed: y / x / w_packed / scale is NULL");
    ASCQ_REQUIRE(!d->has_offset || offset, ASCQ_ENULL, "ascq_matmul_w4a16_packed: offset is NULL");
    ASCQ_REQUIRE(d->mode == ASCQ_W4A16_PER_WEIGHT || d->mode == ASCQ_W4A16_GROUP_SUM, ASCQ_EINVAL,
                 "ascq_matmul_w4a16_packed: mode %d is neither ASCQ_W4A16_PER_WEIGHT nor ASCQ_W4A16_GROUP_SUM", d->mode);
    const uint32_t g32 = d->group_size / 32u;
    ASCQ_REQUIRE(d->k % kTileK == 0 && d->n % 8u == 0 && d->group_size % 32u == 0 && (g32 & (g32 - 1u)) == 0, ASCQ_EUNSUPPORTED,
                 "ascq_matmul_w4a16_packed: k must be a multiple of 128, n of 8 and group_size 32 times a power of two "
                 "(use ascq_matmul_w4a16 otherwise)");
    ASCQ_REQUIRE((static_cast<uint64_t>((d->n + kSlabCols - 1u) / kSlabCols) * (d->k / kTileK) + kPadTiles) * kTileBytes < (1ull << 31) &&
                     static_cast<uint64_t>(d->k / d->group_size) * d->n * 2u < (1ull << 31) &&
                     static_cast<uint64_t>(kMaxRows) * d->k * 2u < (1ull << 31),
                 ASCQ_EUNSUPPORTED, "ascq_matmul_w4a16_packed: packed weights, parameter tables and 16 activation rows must "
                                    "each stay below 2 GiB");
    ASCQ_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(scale) && (!d->has_offset || aligned16(offset)), ASCQ_EALIGN,
                 "ascq_matmul_w4a16_packed: x, w_packed, scale and offset must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    W4pParams p{};
    p.wp = static_cast<const u32x4*>(w_packed);
    p.scale = static_cast<const uint16_t*>(scale);
    p.offset = d->has_offset ? static_cast<const uint16_t*>(offset) : nullptr;
    p.n = d->n;
    p.k = d->k;
    p.mk = NibbleMasks{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    p.gs_shift = 0;
    while ((1u << p.gs_shift) < g32) ++p.gs_shift;
    p.slabs = (d->n + kSlabCols - 1u) / kSlabCols;
    p.ktiles = d->k / kTileK;
    const uint32_t cus = device_compute_units();
    constexpr uint32_t waves = 8u, batch = 4u;  // 16 wavefronts with batches of 4 tiles measured slower (37 against 30 us)
    for (uint32_t m0 = 0; m0 < d->m; m0 += kMaxRows) {
        p.m = d->m - m0 < kMaxRows ? d->m - m0 : kMaxRows;
        p.m_magic = static_cast<uint32_t>(((1ull << 32) + p.m - 1u) / p.m);
        p.x = static_cast<const uint16_t*>(x) + static_cast<size_t>(m0) * d->k;
        p.y = static_cast<uint16_t*>(y) + static_cast<size_t>(m0) * d->n;
        const uint32_t groups = d->k / d->group_size;
        if (p.m > 4u && groups <= kRowsMaxGroups) {
            // one wavefront per slab, the activations shared chunk by chunk: as many wavefronts per workgroup as give
            // every compute unit a workgroup (7 at n = 28672 on 256 units), between 4 and 8
            uint32_t kw = (p.slabs + cus - 1u) / cus;
            kw = kw < 4u ? 4u : (kw > 8u ? 8u : kw);
            p.par_pitch = groups | 1u;
            const uint32_t grid = (p.slabs + kw - 1u) / kw;
            auto go = [&](auto has_offset, auto sum_form) {
                constexpr bool kOff = decltype(has_offset)::value, kSumF = decltype(sum_form)::value;
                switch (kw) {
                    case 4: w4a16_packed_rows_kernel<kOff, 4, kSumF><<<grid, 4 * 64, 0, st>>>(p); break;
                    case 5: w4a16_packed_rows_kernel<kOff, 5, kSumF><<<grid, 5 * 64, 0, st>>>(p); break;
                    case 6: w4a16_packed_rows_kernel<kOff, 6, kSumF><<<grid, 6 * 64, 0, st>>>(p); break;
                    case 7: w4a16_packed_rows_kernel<kOff, 7, kSumF><<<grid, 7 * 64, 0, st>>>(p); break;
                    default: w4a16_packed_rows_kernel<kOff, 8, kSumF><<<grid, 8 * 64, 0, st>>>(p); break;
                }
            };
            const bool rows_sum = d->mode == ASCQ_W4A16_GROUP_SUM && p.gs_shift >= 2u;
            if (d->has_offset) {
                rows_sum ? go(std::true_type{}, std::true_type{}) : go(std::true_type{}, std::false_type{});
            } else {
                rows_sum ? go(std::false_type{}, std::true_type{}) : go(std::false_type{}, std::false_type{});
            }
            continue;
        }
        p.red_lanes = p.m <= 4u ? 16u : 64u;
        // Whole slabs per workgroup, one workgroup per compute unit when the slabs allow it; then the longest pass over
        // k whose activations and parameters fit their shares of the LDS (a multiple of the wavefront count), and fewer
        // slabs if the per-wavefront sums would not fit beside them.
        uint32_t spw = (p.slabs + cus - 1u) / cus;
        spw = spw < 1u ? 1u : (spw > kMaxSlabs ? kMaxSlabs : spw);
        // the group-sum form needs whole tiles inside one quantisation group; other group sizes keep the per-weight form
        const bool sum_form = d->mode == ASCQ_W4A16_GROUP_SUM && p.gs_shift >= 2u;
        uint32_t pt = 0, xs_wave = 0, par_wave = 0, red_bytes = 0, sum_wave = 0, par_cw = 1;
        // entries per column of a wavefront's table: the groups its tiles can touch, rounded up to an odd number
        auto par_rows = [&](uint32_t tiles) { return ((((tiles * 4u - 1u) >> p.gs_shift) + 2u) | 1u); };
        for (;; --spw) {
            const uint32_t all = (p.ktiles + waves - 1u) / waves * waves;
            pt = ((kXBytes / p.m - waves * kRowPad) / (kTileK * 2u)) / waves * waves;
            pt = pt < all ? pt : all;
            par_cw = 1u;
            while ((1u << par_cw) < 2u * spw) ++par_cw;
            const uint32_t par_max_rows = 3u * (64u >> par_cw);  // three fetch rounds of a wavefront
            while (pt > waves && (waves * par_rows(pt / waves) * spw * kSlabCols * 4u > kParBytes || par_rows(pt / waves) > par_max_rows)) pt -= waves;
            xs_wave = p.m * (pt / waves * kTileK * 2u + kRowPad);
            par_wave = par_rows(pt / waves) * spw * kSlabCols * 4u;
            red_bytes = waves * spw * 4u * p.red_lanes * 4u;
            sum_wave = sum_form ? pt / waves * 32u : 0u;
            if ((waves * par_wave <= kParBytes && par_rows(pt / waves) <= 3u * (64u >> par_cw) && waves * (xs_wave + par_wave + sum_wave) + red_bytes <= kPool) || spw == 1u) break;
        }
        ASCQ_REQUIRE(waves * par_wave <= kParBytes && par_rows(pt / waves) <= 3u * (64u >> par_cw) && waves * (xs_wave + par_wave + sum_wave) + red_bytes <= kPool, ASCQ_EUNSUPPORTED,
                     "ascq_matmul_w4a16_packed: group_size %u too small for this shape", d->group_size);
        p.slabs_per_wg = spw;
        p.pass_tiles = pt;
        p.par_cw = par_cw;
        p.xs_wave = xs_wave;
        p.par_wave = par_wave;
        p.par_pitch = par_rows(pt / waves);
        p.par_off = waves * xs_wave;
        p.red_off = p.par_off + waves * par_wave;
        p.sum_off = p.red_off + red_bytes;
        p.sum_wave = sum_wave;
        const uint32_t grid = (p.slabs + spw - 1u) / spw;
        auto go = [&](auto has_offset) {
            constexpr bool kOff = decltype(has_offset)::value;
            if (!sum_form) {
                w4a16_packed_kernel<kOff, waves, batch, 0><<<grid, waves * 64u, 0, st>>>(p);
            } else {
                // all four result registers whatever m is: instantiations for one and two registers, whose sums cover
                // more tiles per round, measured 0.3 to 0.9 us slower
                w4a16_packed_kernel<kOff, waves, batch, 4><<<grid, waves * 64u, 0, st>>>(p);
            }
        };
        if (d->has_offset) {
            go(std::true_type{});
        } else {
            go(std::false_type{});
        }
    }
    return launch_status("ascq_matmul_w4a16_packed");
}
