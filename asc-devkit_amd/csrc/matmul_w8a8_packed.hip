// int8 matmul for few activation rows (decode, small batches) on weights pre-packed for this GPU: one launch, no
// workspace, one flat sweep over the weights.  Up to 16 rows the activations stay in LDS and the weights stream past
// them (gemm_packed_kernel, and gemm_packed_dyn_kernel with the per-token quantiser inside); more rows turn the roles
// round (gemm_ws_kernel: the weights stay in registers and the activations stream).
//
// Packed layout (ascq_pack_weight_w8): the [k, n] matrix is cut into slabs of 16 columns and tiles of 64 k; a tile of a
// slab is 1 KiB and the tiles of a slab, then the slabs, follow each other in memory.  Inside a tile lane l of a
// wavefront owns 16 bytes: column l % 16 of the slab, k = 16 (l / 16) .. + 15 - the B operand of
// v_mfma_i32_16x16x64_i8 as it lies.  Columns past n and k past the end hold 0; 16 tiles of zeros follow the last
// slab.  So a tile costs one fully coalesced 16-byte load per lane and one matrix instruction, for up to 16 activation
// rows at the cost of one, and nothing else: no vector ALU work in the loop.
//
// A workgroup owns whole slabs (whole columns: nothing is added across workgroups), its eight wavefronts split k.
// A wavefront moves its share of the activations (its k range of every row) into its part of the LDS once, by
// direct-to-LDS loads, and streams its tiles in batches of 4 with one batch in flight while one is computed (a compute
// unit keeps about 64 KiB of loads in flight whatever is asked of it; deeper queues only make wavefronts wait at the
// issue of their loads).  Operand row i of a lane reads activation row i % rows, so there are no zero rows to
// materialise.  The eight partial sums of a column meet in LDS (integers: exact in any order) and go through the
// element-wise epilogue of the int8 matmul.
//
// The same kernel reads weights kept as [n, k] (the reference's isTransposeB) without any packing: there a "tile" of a
// slab is the 64 bytes k = 64 t .. + 63 of each of its 16 columns, lane l fetching bytes 16 (l / 16) .. + 15 of column
// l % 16 - the same operand, gathered from 16 runs of 64 bytes instead of one run of 1 KiB.  Only the addresses differ:
// the lane's offset is column * k + 16 (l / 16), the scalar offset slab * 16 k + 64 t, and columns past n fall outside
// the buffer, whose range check returns zeros for them.
#include "matmul_w8a8.h"

namespace ascq {
namespace {

constexpr uint32_t kPkCols = 16, kPkTileK = 64, kPkTileBytes = 1024;
constexpr uint32_t kPkPadTiles = 16;   // tiles of zeros behind the last slab (a batch may read on)
constexpr uint32_t kPkWaves = 8, kPkBatch = 4, kPkMaxSlabs = 8, kPkMaxRows = 16;
constexpr int kPkBuf = 2;              // register buffers: one batch in flight while the other is computed
constexpr uint32_t kPkRowPad = 16;     // bytes added to a staged activation row: rows start 4 banks apart
constexpr uint32_t kPkPool = 158 * 1024;  // LDS of a workgroup (of 160 KiB): the staged activations, then 8 KiB of partial sums per slab
constexpr uint32_t kPkPastEnd = 0x7FFFFFF0u;
constexpr int kPkNt = 2;               // cache policy of the weight loads: non-temporal (read once per call)

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;

struct PackedParams {
    const int8_t* a;       // [m, k], first row of this pass
    const i32x4* wp;       // packed weights
    uint32_t m0, rows;     // first row and rows of this pass (1 .. 16)
    uint32_t n, k;
    uint32_t slabs, ktiles;
    uint32_t tpw;          // tiles of k per wavefront
    uint32_t rows_magic;   // ceil(2^32 / rows)
    uint32_t red_off;      // gemm_packed_kernel: bytes of LDS in front of the partial sums
    uint32_t red_slabs;    // ... and the slabs a workgroup holds at most
    EpiParams epi;
};

// Workgroups are dealt to the 8 XCDs round-robin; in this order the workgroups of an XCD own neighbouring slabs.
__device__ __forceinline__ uint32_t pk_xcd_order(uint32_t wg, uint32_t wgs)
{
    return (wgs & 7u) == 0u ? (wg & 7u) * (wgs >> 3) + (wg >> 3) : wg;
}

template <bool kNK>
__global__ __launch_bounds__(kPkWaves * 64) void gemm_packed_kernel(PackedParams p)
{
    // the staged activations (rows x 8 wavefronts x pitch bytes), then the partial sums [wavefront][slab][4][64]
    __shared__ __attribute__((aligned(16))) char POOL[kPkPool];
    char* const XS = POOL;
    int32_t* const red = reinterpret_cast<int32_t*>(POOL + p.red_off);
    const uint32_t red_wave = p.red_slabs * 256u;  // words from a wavefront's sums to the next one's
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    // slabs [s0, s1) of this workgroup: the slabs are dealt out as evenly as they divide
    const uint32_t wg = pk_xcd_order(blockIdx.x, gridDim.x);
    const uint32_t s0 = static_cast<uint32_t>(static_cast<uint64_t>(wg) * p.slabs / gridDim.x);
    const uint32_t s1 = static_cast<uint32_t>(static_cast<uint64_t>(wg + 1u) * p.slabs / gridDim.x);
    const uint32_t nslabs = s1 - s0;
    const uint32_t ta = min(wave * p.tpw, p.ktiles), tb = min(ta + p.tpw, p.ktiles), cnt = tb - ta;
    const uint32_t pitch = p.tpw * kPkTileK + kPkRowPad;
    char* const xs = XS + wave * (p.rows * pitch);

    // ---- this wavefront's share of the activations: up to 1 KiB of a row per instruction, straight into LDS
    {
        const uint32_t row_pieces = cnt * (kPkTileK / 16u);
        for (uint32_t r = 0; r < p.rows; ++r) {
            const int8_t* src = p.a + static_cast<size_t>(p.m0 + r) * p.k + ta * kPkTileK + lane * 16u;
            for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                if (c0 + lane < row_pieces) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(src + c0 * 16u), (lds_ptr_t)(xs + r * pitch + c0 * 16u), 16, 0, 0);
                }
            }
        }
    }
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<i32x4*>(p.wp), 0,
        static_cast<int>(kNK ? p.n * p.k : (p.slabs * p.ktiles + kPkPadTiles) * kPkTileBytes), 0x00020000);
    const uint32_t w_lane = kNK ? lc * p.k + lq * 16u : lane * 16u;  // the lane's 16 bytes inside a tile
    // operand row i reads row i % rows; + tile * 64
    const uint32_t x_lane = (lc - __umulhi(lc, p.rows_magic) * p.rows) * pitch + lq * 16u;

    // ---- batches of kPkBatch tiles that never straddle a slab: batch q = (slab q / nb, tiles ta + (q % nb) kPkBatch ...)
    const uint32_t nb = (cnt + kPkBatch - 1u) / kPkBatch;
    const uint32_t batches = nb * nslabs;
    i32x4 wq[kPkBuf][kPkBatch];
    uint32_t l_slab = s0, l_b = 0, l_q = 0;
    bool l_done = batches == 0u;
    auto load = [&](int buf) __attribute__((always_inline)) {
        // every load is issued, so the waits the compiler inserts count exactly; once every batch has been requested the
        // per-lane offset lies past the end of the buffer and the loads move no data.  A short last batch reads on into
        // the next tiles or the padding: valid memory, not computed.
        const uint32_t l_w = l_done ? kPkPastEnd : w_lane;
        constexpr uint32_t kStep = kNK ? kPkTileK : kPkTileBytes;  // bytes from a tile to the next of its slab
        const uint32_t base = kNK ? l_slab * kPkCols * p.k + (ta + l_b * kPkBatch) * kPkTileK
                                  : (l_slab * p.ktiles + ta + l_b * kPkBatch) * kPkTileBytes;  // scalar
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            wq[buf][t] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, l_w, base + t * kStep, kPkNt));
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
#pragma unroll
    for (int b = 0; b < kPkBuf; ++b) load(b);
    // Loads return in order: once at most the weight loads just issued are outstanding, the activations have landed in
    // LDS.  (The compiler does not count direct-to-LDS loads issued in a loop; it is told here, with a wait it
    // understands, so that it neither reads the LDS early nor waits for the weights in front of every LDS read.)
    __builtin_amdgcn_s_waitcnt(((kPkBuf * kPkBatch) & 15) | (((kPkBuf * kPkBatch) >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");

    i32x4 acc = {0, 0, 0, 0};
    uint32_t c_slab = 0, c_b = 0, c_q = 0;
    auto compute = [&](int buf) __attribute__((always_inline)) {
        if (c_q >= batches) {
            return;  // uniform
        }
        const uint32_t t0 = c_b * kPkBatch;             // first tile of the batch, relative to ta
        const uint32_t live = min(kPkBatch, cnt - t0);
        const char* xa0 = xs + x_lane + t0 * kPkTileK;
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            if (t < live) {  // uniform
                const i32x4 a = *reinterpret_cast<const i32x4*>(xa0 + t * kPkTileK);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, wq[buf][t], acc, 0, 0, 0);
            }
        }
        ++c_q;
        if (++c_b == nb) {  // the slab is done: register i of lane l is row 4 (l / 16) + i, column l % 16
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave * red_wave + c_slab * 256u + i * 64u + lane] = acc[i];
            acc = i32x4{0, 0, 0, 0};
            c_b = 0;
            ++c_slab;
        }
    };
    for (uint32_t q = 0; q < batches; q += kPkBuf) {
#pragma unroll
        for (int b = 0; b < kPkBuf; ++b) {
            compute(b);
            load(b);
        }
    }
    if (batches == 0u) {  // a wavefront without tiles (k shorter than 8 tiles) contributes zeros
        for (uint32_t s = 0; s < nslabs; ++s) {
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave * red_wave + s * 256u + i * 64u + lane] = 0;
        }
    }
    __syncthreads();

    // ---- the eight partial sums of every element, then the element-wise epilogue
    const EpiParams& e = p.epi;
    for (uint32_t s = wave; s < nslabs; s += kPkWaves) {
        const uint32_t col = (s0 + s) * kPkCols + lc;
        if (col >= p.n) {
            continue;
        }
        const ChannelQ q = load_channel_q(e, col);
        const float bp = load_bias_post(e, col);
        const int32_t bias_pre = e.bias_kind == ASCQ_MM_BIAS_I32_PRE ? static_cast<const int32_t*>(e.bias)[col] : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t row_in_pass = 4u * lq + static_cast<uint32_t>(i);
            if (row_in_pass >= p.rows) {
                continue;
            }
            const int32_t* part = red + s * 256u + static_cast<uint32_t>(i) * 64u + lane;
            int32_t sum = part[0];
#pragma unroll
            for (uint32_t wv = 1; wv < kPkWaves; ++wv) sum += part[wv * red_wave];
            sum += bias_pre;
            const uint32_t row = p.m0 + row_in_pass;
            const float tok = e.has_tok ? e.tok_scale[row] : 1.0f;
            epilogue_store_lanes(e, row, col, sum, q, tok, bp);
        }
    }
}

// The same kernel for weights kept as [n, k] with the weights going through LDS: read straight into registers as matrix
// operands, a tile of [n, k] weights is 16 runs of 64 bytes per load instruction, which the memory pipeline of a
// compute unit takes at about half the rate of long runs.  Here a load instruction brings four columns' 256 bytes (the
// four tiles of a batch) into a two-slot ring per wavefront, with the 16-byte pieces of column c stored at position
// piece ^ c, so that the 16 lanes that read one piece of 16 different columns fall on 16 different bank groups.  The
// loads are buffer loads (range-checked: a batch that reaches past the matrix reads zeros, and the requests past the
// last batch move no data); the ring is an array of its own, so that the compiler does not make the reads of the
// staged activations wait for the weights in flight, and its reads are written as instructions.
constexpr uint32_t kNlSlot = kPkBatch * kPkCols * kPkTileK;   // 4 KiB: 16 columns x 256 bytes
constexpr uint32_t kNlRing = kPkWaves * 2u * kNlSlot;         // 64 KiB

__global__ __launch_bounds__(kPkWaves * 64) void gemm_nkl_kernel(PackedParams p)
{
    __shared__ __attribute__((aligned(1024))) char RING[kNlRing];
    __shared__ __attribute__((aligned(16))) char POOL[kPkPool - kNlRing];  // staged activations, then the partial sums
    char* const XS = POOL;
    int32_t* const red = reinterpret_cast<int32_t*>(POOL + p.red_off);
    const uint32_t red_wave = p.red_slabs * 256u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t wg = pk_xcd_order(blockIdx.x, gridDim.x);
    const uint32_t s0 = static_cast<uint32_t>(static_cast<uint64_t>(wg) * p.slabs / gridDim.x);
    const uint32_t s1 = static_cast<uint32_t>(static_cast<uint64_t>(wg + 1u) * p.slabs / gridDim.x);
    const uint32_t nslabs = s1 - s0;
    const uint32_t ta = min(wave * p.tpw, p.ktiles), tb = min(ta + p.tpw, p.ktiles), cnt = tb - ta;
    const uint32_t pitch = p.tpw * kPkTileK + kPkRowPad;
    char* const xs = XS + wave * (p.rows * pitch);
    {
        const uint32_t row_pieces = cnt * (kPkTileK / 16u);
        for (uint32_t r = 0; r < p.rows; ++r) {
            const int8_t* src = p.a + static_cast<size_t>(p.m0 + r) * p.k + ta * kPkTileK + lane * 16u;
            for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                if (c0 + lane < row_pieces) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(src + c0 * 16u), (lds_ptr_t)(xs + r * pitch + c0 * 16u), 16, 0, 0);
                }
            }
        }
    }
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<i32x4*>(p.wp), 0, static_cast<int>(p.n * p.k), 0x00020000);
    // instruction u of a batch: columns 4 u .. 4 u + 3 of the slab; the lane's column and its position in the column's
    // 256 bytes; it fetches piece position ^ column
    uint32_t w_off[kPkBatch];
#pragma unroll
    for (uint32_t u = 0; u < kPkBatch; ++u) {
        const uint32_t col = 4u * u + lq, pos = lc;
        w_off[u] = col * p.k + ((pos ^ col) << 4);
    }
    char* const ring = RING + wave * (2u * kNlSlot);
    const uint32_t x_lane = (lc - __umulhi(lc, p.rows_magic) * p.rows) * pitch + lq * 16u;
    const uint32_t nb = (cnt + kPkBatch - 1u) / kPkBatch;
    const uint32_t batches = nb * nslabs;
    uint32_t l_slab = s0, l_b = 0, l_q = 0;
    bool l_done = batches == 0u;
    auto load = [&](char* slot) __attribute__((always_inline)) {
        const uint32_t base = l_slab * kPkCols * p.k + (ta + l_b * kPkBatch) * kPkTileK;  // scalar
#pragma unroll
        for (uint32_t u = 0; u < kPkBatch; ++u) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(slot + u * 1024u), 16, l_done ? kPkPastEnd : w_off[u], base,
                                                     0, kPkNt);
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
    load(ring);
    load(ring + kNlSlot);
    // loads return in order: with at most the two batches outstanding the activations have landed
    __builtin_amdgcn_s_waitcnt(((2 * kPkBatch) & 15) | (((2 * kPkBatch) >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");

    // the lane's fragment of tile t of a slot: column lc, piece 4 t + lq, stored at position piece ^ lc
    const uint32_t ring_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)ring)) + lc * 256u;
    const uint32_t xs_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)xs)) + x_lane;
    const uint32_t red_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)red)) + (wave * red_wave + lane) * 4u;
    i32x4 acc = {0, 0, 0, 0};
    uint32_t c_slab = 0, c_b = 0, c_q = 0;
    auto step = [&](uint32_t slot_off, char* slot) __attribute__((always_inline)) {
        if (c_q >= batches) {
            return;  // uniform
        }
        // everything but the newest batch has landed
        __builtin_amdgcn_s_waitcnt((kPkBatch & 15) | ((kPkBatch >> 4) << 14) | (7 << 4) | (15 << 8));
        // (every LDS access of the loop is written as an instruction: one the compiler knows of makes it wait for
        // all the weights in flight first.  A batch's last tiles may lie past the wavefront's k range: their
        // activations are whatever follows in LDS, and they are not computed.)
        const uint32_t t0 = c_b * kPkBatch;
        const uint32_t live = min(kPkBatch, cnt - t0);
        const uint32_t xa = xs_lane + t0 * kPkTileK;
        i32x4 w[kPkBatch], a[kPkBatch];
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            const uint32_t addr = ring_lane + slot_off + (((4u * t + lq) ^ lc) << 4);
            asm volatile("ds_read_b128 %0, %1" : "=v"(w[t]) : "v"(addr) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[t]) : "v"(xa), "i"(t * kPkTileK) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
        load(slot);  // the slot is free again
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            if (t < live) {  // uniform
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t], w[t], acc, 0, 0, 0);
            }
        }
        ++c_q;
        if (++c_b == nb) {
            const uint32_t ra = red_lane + c_slab * 1024u;
            asm volatile("ds_write_b32 %0, %1\n\tds_write_b32 %0, %2 offset:256\n\t"
                         "ds_write_b32 %0, %3 offset:512\n\tds_write_b32 %0, %4 offset:768"
                         :
                         : "v"(ra), "v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[3])
                         : "memory");
            acc = i32x4{0, 0, 0, 0};
            c_b = 0;
            ++c_slab;
        }
    };
    for (uint32_t q = 0; q < batches; q += 2u) {
        step(0u, ring);
        step(kNlSlot, ring + kNlSlot);
    }
    if (batches == 0u) {
        for (uint32_t s = 0; s < nslabs; ++s) {
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave * red_wave + s * 256u + i * 64u + lane] = 0;
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the requests past the last batch, the sums' stores
    __syncthreads();

    const EpiParams& e = p.epi;
    for (uint32_t s = wave; s < nslabs; s += kPkWaves) {
        const uint32_t col = (s0 + s) * kPkCols + lc;
        if (col >= p.n) {
            continue;
        }
        const ChannelQ q = load_channel_q(e, col);
        const float bp = load_bias_post(e, col);
        const int32_t bias_pre = e.bias_kind == ASCQ_MM_BIAS_I32_PRE ? static_cast<const int32_t*>(e.bias)[col] : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t row_in_pass = 4u * lq + static_cast<uint32_t>(i);
            if (row_in_pass >= p.rows) {
                continue;
            }
            const int32_t* part = red + s * 256u + static_cast<uint32_t>(i) * 64u + lane;
            int32_t sum = part[0];
#pragma unroll
            for (uint32_t wv = 1; wv < kPkWaves; ++wv) sum += part[wv * red_wave];
            sum += bias_pre;
            const uint32_t row = p.m0 + row_in_pass;
            const float tok = e.has_tok ? e.tok_scale[row] : 1.0f;
            epilogue_store_lanes(e, row, col, sum, q, tok, bp);
        }
    }
}

// The decode kernel with the per-token quantisation of the activations inside (up to 8 rows of half or bfloat16 x):
// q = ascq_dynamic_quant_per_token(x); c = matmul(q, w, tok_scale) in one launch, with those two calls' results bit for
// bit.  Every workgroup needs all of x anyway, so every workgroup quantises it: a wavefront stages its k range of
// every row as it is (2 bytes per element), the wavefronts exchange their rows' absolute maxima through LDS, and each
// turns its own range into the int8 image the matrix instructions read, with the arithmetic of dynq_row_kernel:
// inv = 127 / amax, the product rounded to the nearest integer, ties to even, by adding 1.5 * 2^23.  The weight
// batches requested ahead of all this arrive meanwhile.  The quantisation costs every compute unit about 0.4 us per
// row beyond the first, which is why this form stops at 8 rows: from there on the separate quantiser kernel (one pass
// over x by the whole chip) is cheaper than 256 redundant ones.  The wavefronts' tiles are added into one LDS array with atomics.
constexpr uint32_t kPkDynRows = 8;
constexpr uint32_t kPkDynHBytes = 96 * 1024;   // the staged activations as they come (2 bytes per element)
constexpr uint32_t kPkDynQBytes = 48 * 1024;   // their int8 image

// The largest of the 64 lanes' values, none of which is negative or a NaN (so their bit patterns order like integers),
// in every lane's copy of the result: four shifts inside the rows of 16 lanes and two row broadcasts, all in the
// vector ALU, then lane 63 read back.
__device__ __forceinline__ float pk_wave_max_nonneg(float v)
{
    int x = __float_as_int(v);
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false));  // row_shr:1
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false));  // row_shr:2
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false));  // row_shr:4
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false));  // row_shr:8
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false));  // row_bcast:15 into rows 1 and 3
    x = max(x, __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false));  // row_bcast:31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(x, 63));
}

// kRing ([n, k] weights): the weights go through the LDS ring of gemm_nkl_kernel, which takes 64 KiB from the staged
// activations; every LDS read between the first request and the last arrival is then written as an instruction (one
// the compiler knows of makes it wait for all the weights in flight).
constexpr uint32_t kPkDynRingHBytes = 60 * 1024, kPkDynRingQBytes = 30 * 1024;

template <bool kNK, bool kBf16, bool kRing = false>
__global__ __launch_bounds__(kPkWaves * 64) void gemm_packed_dyn_kernel(PackedParams p, const uint16_t* __restrict__ x)
{
    static_assert(kNK || !kRing, "the ring is for [n, k] weights");
    __shared__ __attribute__((aligned(1024))) char RING[kRing ? kNlRing : 1024u];
    __shared__ __attribute__((aligned(16))) char XH[kRing ? kPkDynRingHBytes : kPkDynHBytes];
    __shared__ __attribute__((aligned(16))) char XS[kRing ? kPkDynRingQBytes : kPkDynQBytes];
    __shared__ int32_t OUT[kPkMaxSlabs][kPkDynRows][16];  // [slab][row][column]
    __shared__ float ROWMAX[kPkWaves][kPkDynRows];
    __shared__ float TOK[kPkDynRows];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t wg = pk_xcd_order(blockIdx.x, gridDim.x);
    const uint32_t s0 = static_cast<uint32_t>(static_cast<uint64_t>(wg) * p.slabs / gridDim.x);
    const uint32_t s1 = static_cast<uint32_t>(static_cast<uint64_t>(wg + 1u) * p.slabs / gridDim.x);
    const uint32_t nslabs = s1 - s0;
    const uint32_t ta = min(wave * p.tpw, p.ktiles), tb = min(ta + p.tpw, p.ktiles), cnt = tb - ta;
    const uint32_t pitch = p.tpw * kPkTileK + kPkRowPad;  // of an int8 row; a staged row is twice as long
    char* const xh = XH + wave * (p.rows * 2u * pitch);
    char* const xs = XS + wave * (p.rows * pitch);
    const uint32_t row_pieces = cnt * (kPkTileK * 2u / 16u);  // 16-byte pieces (8 elements) of a staged row

    // ---- this wavefront's k range of every row, as it is, straight into LDS
    for (uint32_t r = 0; r < p.rows; ++r) {
        const uint16_t* src = x + static_cast<size_t>(p.m0 + r) * p.k + ta * kPkTileK + lane * 8u;
        for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
            if (c0 + lane < row_pieces) {
                __builtin_amdgcn_global_load_lds((gptr_t)(src + c0 * 8u), (lds_ptr_t)(xh + r * 2u * pitch + c0 * 16u), 16, 0, 0);
            }
        }
    }
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<i32x4*>(p.wp), 0,
        static_cast<int>(kNK ? p.n * p.k : (p.slabs * p.ktiles + kPkPadTiles) * kPkTileBytes), 0x00020000);
    const uint32_t w_lane = kNK ? lc * p.k + lq * 16u : lane * 16u;
    const uint32_t x_lane = (p.rows == 1u ? 0u : lc - __umulhi(lc, p.rows_magic) * p.rows) * pitch + lq * 16u;

    const uint32_t nb = (cnt + kPkBatch - 1u) / kPkBatch;
    const uint32_t batches = nb * nslabs;
    i32x4 wq[kPkBuf][kPkBatch];
    uint32_t l_slab = s0, l_b = 0, l_q = 0;
    bool l_done = batches == 0u;
    // (ring) instruction u of a batch: the lane's column 4 u + lq, position lc in its 256 bytes, piece position ^ column
    uint32_t w_off[kPkBatch];
#pragma unroll
    for (uint32_t u = 0; u < kPkBatch; ++u) {
        const uint32_t col = 4u * u + lq;
        w_off[u] = col * p.k + ((lc ^ col) << 4);
    }
    char* const ring = RING + (kRing ? wave * (2u * kNlSlot) : 0u);
    auto load = [&](int buf) __attribute__((always_inline)) {
        const uint32_t l_w = l_done ? kPkPastEnd : w_lane;
        constexpr uint32_t kStep = kNK ? kPkTileK : kPkTileBytes;
        const uint32_t base = kNK ? l_slab * kPkCols * p.k + (ta + l_b * kPkBatch) * kPkTileK
                                  : (l_slab * p.ktiles + ta + l_b * kPkBatch) * kPkTileBytes;  // scalar
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            if constexpr (kRing) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(ring + buf * kNlSlot + t * 1024u), 16,
                                                         l_done ? kPkPastEnd : w_off[t], base, 0, kPkNt);
            } else {
                wq[buf][t] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, l_w, base + t * kStep, kPkNt));
            }
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
#pragma unroll
    for (int b = 0; b < kPkBuf; ++b) load(b);
    // the staged activations have landed once at most the weight loads just issued are outstanding
    __builtin_amdgcn_s_waitcnt(((kPkBuf * kPkBatch) & 15) | (((kPkBuf * kPkBatch) >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");

    // ---- absolute maximum of every row over this wavefront's range; the shared sums start at zero
    auto widen = [](uint32_t half_bits) __attribute__((always_inline)) {
        return kBf16 ? bf16_bits_to_f32(half_bits) : half_bits_to_f32(half_bits);
    };
    auto lds_read16 = [](const char* ptr) __attribute__((always_inline)) {
        if constexpr (kRing) {
            u32x4 v;
            asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                         : "=v"(v)
                         : "v"(static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)ptr)))
                         : "memory");
            return v;
        } else {
            return *reinterpret_cast<const u32x4*>(ptr);
        }
    };
    for (uint32_t i = tid; i < kPkMaxSlabs * kPkDynRows * 16u; i += kPkWaves * 64u) (&OUT[0][0][0])[i] = 0;
#pragma unroll
    for (uint32_t r = 0; r < kPkDynRows; ++r) {
        if (r < p.rows) {  // uniform
            float amax = 0.0f;
            for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                if (c0 + lane < row_pieces) {
                    const u32x4 v = lds_read16(xh + r * 2u * pitch + (c0 + lane) * 16u);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        amax = fmaxf(amax, fabsf(widen(v[i] & 0xFFFFu)));
                        amax = fmaxf(amax, fabsf(widen(v[i] >> 16)));
                    }
                }
            }
            const float wave_amax = pk_wave_max_nonneg(amax);
            if (lane == 0u) {
                ROWMAX[wave][r] = wave_amax;
            }
        }
    }
    // a plain barrier: the fence of __syncthreads() would also wait for the weight loads in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // ---- lane r works out row r's factor once; every lane then quantises its pieces of this wavefront's range
    float lane_inv;
    {
        float amax = 0.0f;
        if (lane < p.rows) {
#pragma unroll
            for (uint32_t wv = 0; wv < kPkWaves; ++wv) {
                float other;
                if constexpr (kRing) {
                    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                                 : "=v"(other)
                                 : "v"(static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&ROWMAX[wv][lane])))
                                 : "memory");
                } else {
                    other = ROWMAX[wv][lane];
                }
                amax = fmaxf(amax, other);
            }
        }
        const bool zero = !(amax > 0.0f);
        lane_inv = zero ? 0.0f : 127.0f / amax;
        if (tid < p.rows) {
            TOK[tid] = zero ? 1.0f : amax / 127.0f;
        }
    }
#pragma unroll
    for (uint32_t r = 0; r < kPkDynRows; ++r) {
        if (r < p.rows) {  // uniform
            const float inv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lane_inv), static_cast<int>(r)));
            for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                if (c0 + lane < row_pieces) {
                    const u32x4 v = lds_read16(xh + r * 2u * pitch + (c0 + lane) * 16u);
                    uint32_t u[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float t0 = __builtin_amdgcn_fmed3f(widen(v[i] & 0xFFFFu) * inv, -128.0f, 127.0f);
                        const float t1 = __builtin_amdgcn_fmed3f(widen(v[i] >> 16) * inv, -128.0f, 127.0f);
                        u[2 * i] = __float_as_uint(t0 + 12582912.0f);
                        u[2 * i + 1] = __float_as_uint(t1 + 12582912.0f);
                    }
                    u32x2 out;
                    out[0] = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u) | __builtin_amdgcn_perm(u[3], u[2], 0x04000c0cu);
                    out[1] = __builtin_amdgcn_perm(u[5], u[4], 0x0c0c0400u) | __builtin_amdgcn_perm(u[7], u[6], 0x04000c0cu);
                    *reinterpret_cast<u32x2*>(xs + r * pitch + (c0 + lane) * 8u) = out;
                }
            }
        }
    }
    // (the matrix operands below are read by the wavefront that wrote them: LDS operations of a wavefront stay in order)

    i32x4 acc = {0, 0, 0, 0};
    uint32_t c_slab = 0, c_b = 0, c_q = 0;
    auto compute = [&](int buf) __attribute__((always_inline)) {
        if (c_q >= batches) {
            return;  // uniform
        }
        const uint32_t t0 = c_b * kPkBatch;
        const uint32_t live = min(kPkBatch, cnt - t0);
        const char* xa0 = xs + x_lane + t0 * kPkTileK;
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            if (t < live) {  // uniform
                const i32x4 a = *reinterpret_cast<const i32x4*>(xa0 + t * kPkTileK);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, wq[buf][t], acc, 0, 0, 0);
            }
        }
        ++c_q;
        if (++c_b == nb) {  // the slab is done: register i of lane l is row 4 (l / 16) + i, column l % 16
            if (4u * lq < p.rows) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    __hip_atomic_fetch_add(&OUT[c_slab][4u * lq + i][lc], acc[i], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
            acc = i32x4{0, 0, 0, 0};
            c_b = 0;
            ++c_slab;
        }
    };
    // (ring) a batch's fragments and the activations' from LDS, the slot refilled, then the arithmetic, as in
    // gemm_nkl_kernel; the sums of a finished slab are added with atomic instructions
    const uint32_t ring_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)ring)) + lc * 256u;
    const uint32_t xs_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)xs)) + x_lane;
    const uint32_t out_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&OUT[0][0][0])) + (4u * lq * 16u + lc) * 4u;
    auto ring_step = [&](int buf) __attribute__((always_inline)) {
        if (c_q >= batches) {
            return;  // uniform
        }
        __builtin_amdgcn_s_waitcnt((kPkBatch & 15) | ((kPkBatch >> 4) << 14) | (7 << 4) | (15 << 8));
        const uint32_t t0 = c_b * kPkBatch;
        const uint32_t live = min(kPkBatch, cnt - t0);
        const uint32_t xa = xs_lane + t0 * kPkTileK;
        i32x4 w[kPkBatch], a[kPkBatch];
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            const uint32_t addr = ring_lane + buf * kNlSlot + (((4u * t + lq) ^ lc) << 4);
            asm volatile("ds_read_b128 %0, %1" : "=v"(w[t]) : "v"(addr) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[t]) : "v"(xa), "i"(t * kPkTileK) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
        load(buf);
#pragma unroll
        for (uint32_t t = 0; t < kPkBatch; ++t) {
            if (t < live) {  // uniform
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t], w[t], acc, 0, 0, 0);
            }
        }
        ++c_q;
        if (++c_b == nb) {
            if (4u * lq < p.rows) {
                asm volatile("ds_add_u32 %0, %1\n\tds_add_u32 %0, %2 offset:64\n\t"
                             "ds_add_u32 %0, %3 offset:128\n\tds_add_u32 %0, %4 offset:192"
                             :
                             : "v"(out_lane + c_slab * (kPkDynRows * 16u * 4u)), "v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[3])
                             : "memory");
            }
            acc = i32x4{0, 0, 0, 0};
            c_b = 0;
            ++c_slab;
        }
    };
    for (uint32_t q = 0; q < batches; q += kPkBuf) {
#pragma unroll
        for (int b = 0; b < kPkBuf; ++b) {
            if constexpr (kRing) {
                ring_step(b);
            } else {
                compute(b);
                load(b);
            }
        }
    }
    if constexpr (kRing) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the requests past the last batch, the additions
    }
    __syncthreads();

    // ---- elements (row, column) and (row + 4, column) of slab s are handled by thread s * 64 + row * 16 + column
    const EpiParams& e = p.epi;
    const uint32_t s = tid >> 6;
    const uint32_t col = (s0 + s) * kPkCols + lc;
    if (s < nslabs && col < p.n) {
        const ChannelQ q = load_channel_q(e, col);
        const float bp = load_bias_post(e, col);
        const int32_t bias_pre = e.bias_kind == ASCQ_MM_BIAS_I32_PRE ? static_cast<const int32_t*>(e.bias)[col] : 0;
#pragma unroll
        for (uint32_t half = 0; half < kPkDynRows / 4u; ++half) {
            const uint32_t row_in_pass = 4u * half + lq;
            if (row_in_pass < p.rows) {
                const int32_t sum = OUT[s][row_in_pass][lc] + bias_pre;
                epilogue_store_lanes(e, p.m0 + row_in_pass, col, sum, q, TOK[row_in_pass], bp);
            }
        }
    }
}

// The weight-stationary form, for more rows than the LDS can hold.  Activations that are streamed beside the weights
// share the compute unit's in-order load queue with them (every L2 hit of an activation load then waits behind the
// weights' trips to memory).  So the two are separated in time: a workgroup first requests all the weights of its
// columns (kS slabs, a wavefront's k range of each in kC chunks of 8 tiles: 96 or 128 registers of ready matrix
// operands per lane) in one burst with nothing else in the queue, and then streams the activations, 16 rows and one
// chunk of k at a time, from the L2 through a two-slot LDS ring per wavefront: one matrix instruction per slab and
// tile on operands that are already in registers.  A row tile's sums over the wavefronts' k ranges meet in one LDS
// array (atomic adds of integers: exact in any order); the epilogue runs once per block of 128 rows.
//   <3, 1>: k up to 4096, up to 3 slabs per workgroup      <2, 2>: k up to 8192, up to 2 slabs
//   <1, 4>: k up to 16384, one slab per workgroup
constexpr uint32_t kWsTpw = 8, kWsRows = 128, kWsMaxChunks = 4;
constexpr uint32_t kWsNkMaxRows = 224;  // [n, k] weights: beyond this the tile kernels are level or ahead
constexpr uint32_t kWsRowBytes = kWsTpw * kPkTileK;   // 512: a staged row (one chunk of the wavefront's k range)
constexpr uint32_t kWsSlot = 16u * kWsRowBytes;       // 8 KiB: 16 rows
constexpr int kWsDma = 8;                             // direct-to-LDS instructions per slot (two rows each)

template <bool kNK, uint32_t kS, uint32_t kC>
__global__ __launch_bounds__(kPkWaves * 64) void gemm_ws_kernel(PackedParams p)
{
    __shared__ __attribute__((aligned(1024))) char R0[kPkWaves * kWsSlot];
    __shared__ __attribute__((aligned(1024))) char R1[kPkWaves * kWsSlot];
    __shared__ int32_t OUT[kWsRows][kS * kPkCols];
    __shared__ float TS[kWsRows];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t wg = pk_xcd_order(blockIdx.x, gridDim.x);
    const uint32_t s0 = static_cast<uint32_t>(static_cast<uint64_t>(wg) * p.slabs / gridDim.x);
    const uint32_t s1 = static_cast<uint32_t>(static_cast<uint64_t>(wg + 1u) * p.slabs / gridDim.x);
    const uint32_t nslabs = s1 - s0;  // at most kS: the host has chosen the grid
    // this wavefront's tiles of k: cnt of them, in nchunks chunks of kWsTpw (nchunks <= kC: the host has chosen kC)
    const uint32_t ta = min(wave * p.tpw, p.ktiles), tb = min(ta + p.tpw, p.ktiles), cnt = tb - ta;
    const uint32_t nchunks = (p.tpw + kWsTpw - 1u) / kWsTpw;
    // the sums of a block of kWsRows rows start at zero; the rows' token scales are kept for the epilogue
    auto begin_block = [&](uint32_t b0) __attribute__((always_inline)) {
        for (uint32_t i = tid; i < kWsRows * kS * kPkCols; i += kPkWaves * 64u) (&OUT[0][0])[i] = 0;
        if (tid < kWsRows) {
            TS[tid] = (p.epi.has_tok && b0 + tid < p.rows) ? p.epi.tok_scale[p.m0 + b0 + tid] : 1.0f;
        }
        __syncthreads();  // no direct-to-LDS load is in flight here
    };
    begin_block(0u);

    // ---- the weights of this wavefront's k range, all slabs: one burst, nothing else in the queue yet
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<i32x4*>(p.wp), 0,
        static_cast<int>(kNK ? p.n * p.k : (p.slabs * p.ktiles + kPkPadTiles) * kPkTileBytes), 0x00020000);
    i32x4 wreg[kC][kS][kWsTpw];
    char* const r0w = R0 + wave * kWsSlot;
    char* const r1w = R1 + wave * kWsSlot;
    if constexpr (!kNK) {
        const uint32_t w_lane = lane * 16u;
#pragma unroll
        for (uint32_t kc = 0; kc < kC; ++kc) {
#pragma unroll
            for (uint32_t s = 0; s < kS; ++s) {
#pragma unroll
                for (uint32_t t = 0; t < kWsTpw; ++t) {
                    // a tile this wavefront does not have is requested past the end of the buffer: no data moves, the
                    // instruction count stays what the waits below assume
                    const uint32_t tile = kc * kWsTpw + t;
                    const uint32_t off = (s < nslabs && tile < cnt) ? w_lane : kPkPastEnd;
                    const uint32_t base = ((s0 + s) * p.ktiles + ta + tile) * kPkTileBytes;  // scalar
                    wreg[kc][s][t] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, off, base, kPkNt));
                }
            }
        }
    } else {
        // [n, k] weights reach their registers through the (still idle) activation ring, as in gemm_nkl_kernel: a
        // load instruction brings four columns' 256 bytes, the pieces of column c at position piece ^ c; four slots
        // of a batch (four tiles of one slab) each, three batches in flight while one is read.
        constexpr uint32_t kUnits = kC * kS * 2u;
        uint32_t w_off[kPkBatch];
#pragma unroll
        for (uint32_t u = 0; u < kPkBatch; ++u) {
            const uint32_t col = 4u * u + lq;
            w_off[u] = col * p.k + ((lc ^ col) << 4);
        }
        auto slot_of = [&](uint32_t j) __attribute__((always_inline)) { return ((j & 2u) != 0u ? r1w : r0w) + (j & 1u) * kNlSlot; };
        auto request = [&](uint32_t j) __attribute__((always_inline)) {  // j: compile-time after unrolling
            const uint32_t kc = j / (kS * 2u), s = (j / 2u) % kS, t0 = kc * kWsTpw + (j % 2u) * kPkBatch;
            const bool have = s < nslabs && t0 < cnt;  // uniform; a batch the wavefront lacks moves no data
            const uint32_t base = have ? (s0 + s) * kPkCols * p.k + (ta + t0) * kPkTileK : 0u;
            char* const slot = slot_of(j & 3u);
#pragma unroll
            for (uint32_t u = 0; u < kPkBatch; ++u) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(slot + u * 1024u), 16, have ? w_off[u] : kPkPastEnd, base, 0,
                                                         kPkNt);
            }
        };
#pragma unroll
        for (uint32_t j = 0; j < (kUnits < 4u ? kUnits : 4u); ++j) request(j);
#pragma unroll
        for (uint32_t j = 0; j < kUnits; ++j) {
            constexpr uint32_t kAll = kUnits;
            const uint32_t behind = (kAll - 1u - j < 3u ? kAll - 1u - j : 3u) * kPkBatch;  // loads that may still be out
            // (a constant after unrolling; the builtin wants an immediate)
            switch (behind) {
                case 12: __builtin_amdgcn_s_waitcnt((12 & 15) | (7 << 4) | (15 << 8)); break;
                case 8: __builtin_amdgcn_s_waitcnt((8 & 15) | (7 << 4) | (15 << 8)); break;
                case 4: __builtin_amdgcn_s_waitcnt((4 & 15) | (7 << 4) | (15 << 8)); break;
                default: __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8)); break;
            }
            const uint32_t kc = j / (kS * 2u), s = (j / 2u) % kS, h = (j % 2u) * kPkBatch;
            const uint32_t sa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)slot_of(j & 3u))) + lc * 256u;
#pragma unroll
            for (uint32_t t = 0; t < kPkBatch; ++t) {
                const uint32_t addr = sa + (((4u * t + lq) ^ lc) << 4);
                asm volatile("ds_read_b128 %0, %1" : "=v"(wreg[kc][s][h + t]) : "v"(addr) : "memory");
            }
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(wreg[kc][s][h]), "+v"(wreg[kc][s][h + 1u]), "+v"(wreg[kc][s][h + 2u]), "+v"(wreg[kc][s][h + 3u]));
            if (j + 4u < kUnits) {
                request(j + 4u);
            }
        }
    }

    // ---- activations: slot position (row r, piece q) holds piece q ^ r of the row's share of one chunk (the
    // reader's 16 rows then fall on 16 different bank groups); pieces past the wavefront's range fetch the chunk's
    // piece 0 and are not read
    // A load's address is a wavefront-uniform base (row tile and chunk) plus the lane's 32-bit offset, which the
    // instruction adds itself; the last row tile, where rows past the end repeat the last row, has offsets of its own.
    // (ntiles, the offsets of the last tile and the base belong to the block of rows being worked on)
    const uint32_t l31 = lane & 31u, l5 = lane >> 5;
    uint32_t ntiles = 0, last_row = 0;  // last_row: the last valid row of the block's last row tile, 0 .. 15
    // instruction u of a slot brings rows 2 u and 2 u + 1: the lane's row is r = 2 u + lane / 32, its piece
    // q = (lane % 32) ^ r, its offset from the base r k + 16 q + the start of the wavefront's k range.  The eight
    // offsets of a full chunk in a full row tile are kept.  With one chunk per range (kC == 1) its partial filling
    // is in them, and the block's last row tile has eight offsets of its own.  With more chunks those registers
    // belong to the weights: a last row tile that is not full and a chunk that the range fills only partly redo
    // these few operations per request (the asm statement there keeps the compiler from holding the offsets, or
    // their parts, across the loop all the same).
    const uint32_t a_lane = l5 * p.k + (cnt != 0u ? ta : 0u) * kPkTileK;  // (no tiles: any valid piece)
    uint32_t a_off[kWsDma], a_off_last[kC == 1u ? kWsDma : 1];
#pragma unroll
    for (uint32_t u = 0; u < static_cast<uint32_t>(kWsDma); ++u) {
        const uint32_t q = l31 ^ (2u * u + l5);
        a_off[u] = a_lane + 2u * u * p.k + ((kC == 1u && q >= cnt * 4u) ? 0u : q * 16u);
    }
    const int8_t* a_base = p.a;
    uint32_t i_rt = 0, i_kc = 0;  // the (row tile, chunk) the next request fetches
    auto issue = [&](char* slot) __attribute__((always_inline)) {
        // Past the last row tile the requests go on (the count of loads in flight stays what the waits assume) and
        // fetch something valid that is never read.
        auto base_of = [&](uint32_t tile, uint32_t col) __attribute__((always_inline)) {
            const uint64_t bv = reinterpret_cast<uint64_t>(a_base + static_cast<size_t>(tile) * 16u * p.k + col);
            uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bv));
            uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bv >> 32));
            asm volatile("" : "+s"(lo), "+s"(hi));
            return reinterpret_cast<const int8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
        };
        if constexpr (kC == 1u) {
            const uint32_t tile = i_rt < ntiles ? i_rt : ntiles - 1u;  // (past the end: the last one again)
            const int8_t* base = base_of(tile, 0u);
            if (tile + 1u == ntiles) {  // uniform
#pragma unroll
                for (int u = 0; u < kWsDma; ++u) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(base + a_off_last[u]), (lds_ptr_t)(slot + u * 1024), 16, 0, 0);
                }
            } else {
#pragma unroll
                for (int u = 0; u < kWsDma; ++u) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(base + a_off[u]), (lds_ptr_t)(slot + u * 1024), 16, 0, 0);
                }
            }
            ++i_rt;
        } else {
            const uint32_t t0 = i_kc * kWsTpw;
            const uint32_t live = cnt > t0 ? min(kWsTpw, cnt - t0) : 0u;  // tiles of this chunk the wavefront has
            if (i_rt >= ntiles) {  // uniform; past the end: every lane the first piece of the block's first row
                const int8_t* base = base_of(0u, 0u);
                uint32_t first = (cnt != 0u ? ta : 0u) * kPkTileK;
                asm volatile("" : "+v"(first));
#pragma unroll
                for (int u = 0; u < kWsDma; ++u) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(base + first), (lds_ptr_t)(slot + u * 1024), 16, 0, 0);
                }
            } else {
                const int8_t* base = base_of(i_rt, live != 0u ? t0 * kPkTileK : 0u);
                const uint32_t row_max = i_rt + 1u == ntiles ? last_row : 15u;
                if (live == kWsTpw && row_max == 15u) {  // uniform
#pragma unroll
                    for (int u = 0; u < kWsDma; ++u) {
                        __builtin_amdgcn_global_load_lds((gptr_t)(base + a_off[u]), (lds_ptr_t)(slot + u * 1024), 16, 0, 0);
                    }
                } else {  // rows past the block's last one fetch the last one; pieces past the range fetch piece 0
                    const uint32_t pieces = live * 4u;
                    uint32_t x31 = l31, x5 = l5, xc = (cnt != 0u ? ta : 0u) * kPkTileK;
                    asm volatile("" : "+v"(x31), "+v"(x5), "+v"(xc));
#pragma unroll
                    for (uint32_t u = 0; u < static_cast<uint32_t>(kWsDma); ++u) {
                        const uint32_t r = 2u * u + x5, q = x31 ^ r;  // (both factors below 2^24: k is at most 16384)
                        const uint32_t off = xc + __umul24(min(r, row_max), p.k) + (q < pieces ? q * 16u : 0u);
                        __builtin_amdgcn_global_load_lds((gptr_t)(base + off), (lds_ptr_t)(slot + u * 1024), 16, 0, 0);
                    }
                }
            }
            if (++i_kc == nchunks) {
                i_kc = 0;
                ++i_rt;
            }
        }
    };
    // the lane's fragment of tile t: row lc, pieces 4 t + lq; its four sums of a row tile and slab: rows 4 lq + i
    const uint32_t frag = lc * kWsRowBytes;
    const uint32_t out_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&OUT[0][0])) +
                              (4u * lq * kS * kPkCols + lc) * 4u;
    i32x4 acc[kS];
#pragma unroll
    for (uint32_t s = 0; s < kS; ++s) acc[s] = i32x4{0, 0, 0, 0};
    // a slot's fragments into registers (after which the slot can be refilled), then the arithmetic on them
    auto fetch = [&](i32x4 (&a)[kWsTpw], char* slot) __attribute__((always_inline)) {
        const uint32_t sa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)slot)) + frag;
#pragma unroll
        for (uint32_t t = 0; t < kWsTpw; ++t) {
            const uint32_t addr = sa + (((4u * t + lq) ^ lc) << 4);
            asm volatile("ds_read_b128 %0, %1" : "=v"(a[t]) : "v"(addr) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
    };
    auto compute = [&](const i32x4 (&a)[kWsTpw], uint32_t kc, uint32_t rt) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t t = 0; t < kWsTpw; ++t) {
            if (kc * kWsTpw + t < cnt) {  // uniform
#pragma unroll
                for (uint32_t s = 0; s < kS; ++s) {
                    if (s < nslabs) {  // uniform
                        acc[s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t], wreg[kc][s][t], acc[s], 0, 0, 0);
                    }
                }
            }
        }
        if (kc + 1u != nchunks) {  // uniform: the row tile's sums are complete after its last chunk
            return;
        }
        // Register i of lane l is row 4 (l / 16) + i of the row tile, column l % 16 of the slab.  Rows past the last
        // one (copies of it) are added to rows of OUT that nobody reads.  The additions are written as instructions:
        // an LDS atomic the compiler knows of makes it wait for every direct-to-LDS load in flight first.
        const uint32_t oa = out_lane + rt * (16u * kS * kPkCols * 4u);
#pragma unroll
        for (uint32_t s = 0; s < kS; ++s) {
            if (s < nslabs) {  // uniform
                asm volatile("ds_add_u32 %0, %1 offset:%5\n\tds_add_u32 %0, %2 offset:%6\n\t"
                             "ds_add_u32 %0, %3 offset:%7\n\tds_add_u32 %0, %4 offset:%8"
                             :
                             : "v"(oa), "v"(acc[s][0]), "v"(acc[s][1]), "v"(acc[s][2]), "v"(acc[s][3]),
                               "i"(s * kPkCols * 4u), "i"(s * kPkCols * 4u + kS * kPkCols * 4u),
                               "i"(s * kPkCols * 4u + 2u * kS * kPkCols * 4u),
                               "i"(s * kPkCols * 4u + 3u * kS * kPkCols * 4u)
                             : "memory");
            }
            acc[s] = i32x4{0, 0, 0, 0};
        }
    };
    const EpiParams& e = p.epi;
    uint32_t brows = 0;
    auto set_block = [&](uint32_t b0) __attribute__((always_inline)) {
        brows = min(kWsRows, p.rows - b0);
        ntiles = (brows + 15u) / 16u;
        last_row = brows - (ntiles - 1u) * 16u - 1u;
        if constexpr (kC == 1u) {
#pragma unroll
            for (uint32_t u = 0; u < static_cast<uint32_t>(kWsDma); ++u) {
                const uint32_t r = 2u * u + l5;
                a_off_last[u] = a_off[u] - (r - min(r, last_row)) * p.k;
            }
        }
        a_base = p.a + static_cast<size_t>(p.m0 + b0) * p.k;
        i_rt = 0;
        i_kc = 0;
    };
    // the first block's first two slots are requested right behind the weights
    set_block(0u);
    issue(r0w);
    issue(r1w);
    for (uint32_t b0 = 0; b0 < p.rows; b0 += kWsRows) {  // blocks of kWsRows rows: the weights stay where they are
        // Loads return in order: with at most the newest slot's kWsDma loads outstanding, everything older (the
        // weights, the slot about to be read) has arrived.  A slot is refilled as soon as its fragments are in
        // registers; past the last row tile the refills fetch the last tile again, so that the count never changes.
        // (the wait for the LDS counter alone, which the compiler understands, keeps it from placing one of its own
        // inside the loop for something that was pending in front of it)
        __builtin_amdgcn_s_waitcnt(0xC07F);
        auto step = [&](uint32_t kc, uint32_t rt, char* slot) __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt((kWsDma & 15) | ((kWsDma >> 4) << 14) | (7 << 4) | (15 << 8));
            i32x4 a[kWsTpw];
            fetch(a, slot);
            issue(slot);
            compute(a, kc, rt);
        };
        if constexpr (kC == 1u) {
            for (uint32_t rt = 0; rt < ntiles; rt += 2u) {
                step(0u, rt, r0w);
                if (rt + 1u < ntiles) {
                    step(0u, rt + 1u, r1w);
                }
            }
        } else {
            uint32_t parity = 0;
            for (uint32_t rt = 0; rt < ntiles; ++rt) {
#pragma unroll
                for (uint32_t kc = 0; kc < kC; ++kc) {
                    if (kc < nchunks) {  // uniform
                        step(kc, rt, parity != 0u ? r1w : r0w);
                        parity ^= 1u;
                    }
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // nothing lands in LDS after the barrier
        __syncthreads();

        // ---- a thread keeps one column (its parameters are fetched once) and walks down the rows, eight apart
        const uint32_t c = lane, col = s0 * kPkCols + c;
        if (c < nslabs * kPkCols && col < p.n) {
            const ChannelQ q = load_channel_q(e, col);
            const float bp = load_bias_post(e, col);
            const int32_t bias_pre = e.bias_kind == ASCQ_MM_BIAS_I32_PRE ? static_cast<const int32_t*>(e.bias)[col] : 0;
            if (e.activation == ASCQ_MM_ACT_SWIGLU) {  // uniform: column pairs through neighbouring lanes
                for (uint32_t row = wave; row < brows; row += kPkWaves) {
                    epilogue_store_lanes(e, p.m0 + b0 + row, col, OUT[row][c] + bias_pre, q, TS[row], bp);
                }
            } else {
                dispatch_out(e, [&](auto tag) {
                    for (uint32_t row = wave; row < brows; row += kPkWaves) {
                        epilogue_store<decltype(tag)::value>(e, p.m0 + b0 + row, col, OUT[row][c] + bias_pre, q, TS[row], bp);
                    }
                });
            }
        }
        if (b0 + kWsRows < p.rows) {
            __syncthreads();  // the next block clears what this epilogue read
            begin_block(b0 + kWsRows);
            set_block(b0 + kWsRows);
            issue(r0w);
            issue(r1w);
        }
    }
}

// [k, n] (or [n, k] with trans) -> packed; one thread per lane of a tile.
__global__ __launch_bounds__(256) void pack_w8_kernel(const int8_t* __restrict__ w, i32x4* __restrict__ out, uint32_t k,
                                                      uint32_t n, uint32_t slabs, uint32_t ktiles, int trans)
{
    const size_t total = static_cast<size_t>(slabs) * ktiles * 64u;
    const size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x;
    if (i >= total + kPkPadTiles * 64u) {
        return;
    }
    i32x4 v = {0, 0, 0, 0};
    if (i < total) {
        const uint32_t lane = static_cast<uint32_t>(i & 63u);
        const size_t tile_id = i >> 6;
        const uint32_t slab = static_cast<uint32_t>(tile_id / ktiles), tile = static_cast<uint32_t>(tile_id % ktiles);
        const uint32_t col = slab * kPkCols + (lane & 15u), kq = lane >> 4;
#pragma unroll
        for (uint32_t d = 0; d < 4; ++d) {
            uint32_t word = 0;
#pragma unroll
            for (uint32_t b = 0; b < 4; ++b) {
                const uint32_t kk = tile * kPkTileK + kq * 16u + d * 4u + b;
                uint32_t byte = 0;
                if (kk < k && col < n) {
                    byte = static_cast<uint8_t>(trans ? w[static_cast<size_t>(col) * k + kk] : w[static_cast<size_t>(kk) * n + col]);
                }
                word |= byte << (8u * b);
            }
            v[d] = static_cast<int32_t>(word);
        }
    }
    out[i] = v;
}

}  // namespace

// B as [n, k], read in place by the same kernel (offsets are 32-bit and the range check marks the end at 2 GiB)
bool gemm_packed_nk_supported(const GemmParams& p)
{
    return p.k % kPkTileK == 0 && aligned16(p.a) && aligned16(p.b) &&
           static_cast<uint64_t>(p.n + kPkCols) * p.k < (1ull << 31) - 64u * kPkTileK;
}

bool gemm_packed_supported(const GemmParams& p)
{
    return p.k % kPkTileK == 0 && aligned16(p.a) && aligned16(p.b) &&
           (static_cast<uint64_t>((p.n + kPkCols - 1u) / kPkCols) * (p.k / kPkTileK) + kPkPadTiles) * kPkTileBytes < (1ull << 31);
}

namespace {

// the grid of the resident form: one workgroup per compute unit when the slabs allow it, at most kPkMaxSlabs slabs each
uint32_t packed_grid(uint32_t slabs)
{
    const uint32_t cus = device_compute_units();
    uint32_t grid = slabs < cus ? slabs : cus;
    if ((slabs + grid - 1u) / grid > kPkMaxSlabs) {
        grid = (slabs + kPkMaxSlabs - 1u) / kPkMaxSlabs;
    }
    return grid;
}

}  // namespace

// Rows the resident form takes per pass over the weights: 16, fewer when k is so long that the staged activations of
// 16 rows would not fit the LDS beside the partial sums (8 KiB per slab of a workgroup); 0: k is too long altogether.
uint32_t gemm_packed_pass_rows(const GemmParams& p)
{
    const uint32_t slabs = (p.n + kPkCols - 1u) / kPkCols;
    const uint32_t grid = packed_grid(slabs);
    const uint32_t tpw = (p.k / kPkTileK + kPkWaves - 1u) / kPkWaves;
    const uint32_t red_bytes = (slabs + grid - 1u) / grid * kPkWaves * 1024u;
    const uint32_t rows = (kPkPool - red_bytes) / (kPkWaves * (tpw * kPkTileK + kPkRowPad));
    return rows > kPkMaxRows ? kPkMaxRows : rows;
}

// p.b: the packed weights, or with b_nk the plain [n, k] matrix.  Any m, gemm_packed_pass_rows() rows per pass over
// the weights (the callers send more rows than one pass takes only when k is too long for the weight-stationary form).
int launch_gemm_packed(const GemmParams& p, hipStream_t st, bool b_nk)
{
    PackedParams q{};
    q.wp = reinterpret_cast<const i32x4*>(p.b);
    q.a = p.a;
    q.n = p.n;
    q.k = p.k;
    q.slabs = (p.n + kPkCols - 1u) / kPkCols;
    q.ktiles = p.k / kPkTileK;
    q.tpw = (q.ktiles + kPkWaves - 1u) / kPkWaves;
    q.epi = p.epi;
    const uint32_t grid = packed_grid(q.slabs);
    q.red_slabs = (q.slabs + grid - 1u) / grid;
    const uint32_t row_bytes = kPkWaves * (q.tpw * kPkTileK + kPkRowPad);
    const uint32_t pass_rows = gemm_packed_pass_rows(p);
    q.red_off = pass_rows * row_bytes;
    if (pass_rows == 0u) {
        return fail(ASCQ_EUNSUPPORTED, "ascq_matmul_w8a8_packed: k = %u is too long for the staged activations", p.k);
    }
    // [n, k] weights whose rows' activations leave 64 KiB of the LDS free: the weights go through a ring there
    const uint32_t red_bytes = q.red_slabs * kPkWaves * 1024u;
    if (b_nk && static_cast<uint64_t>(p.m) * row_bytes + red_bytes + kNlRing <= kPkPool) {
        q.m0 = 0;
        q.rows = p.m;
        q.rows_magic = static_cast<uint32_t>(((1ull << 32) + q.rows - 1u) / q.rows);
        q.red_off = p.m * row_bytes;
        if (plan_note(ASCQ_MM_KERNEL_STREAM, 16, 16 * q.red_slabs, kPkTileK, grid, 1, kPkPool, 0)) {
            return ASCQ_OK;
        }
        gemm_nkl_kernel<<<grid, kPkWaves * 64u, 0, st>>>(q);
        return launch_status("ascq_matmul_w8a8 ([n, k] weight stream through LDS)");
    }
    for (uint32_t m0 = 0; m0 < p.m; m0 += q.rows) {
        const uint32_t left = p.m - m0;
        q.m0 = m0;
        q.rows = left < pass_rows ? left : pass_rows;
        q.rows_magic = static_cast<uint32_t>(((1ull << 32) + q.rows - 1u) / q.rows);
        if (plan_note(ASCQ_MM_KERNEL_STREAM, 16, 16 * ((q.slabs + grid - 1u) / grid), kPkTileK, grid, 1,
                      kPkPool, 0)) {
            return ASCQ_OK;
        }
        if (b_nk) {
            gemm_packed_kernel<true><<<grid, kPkWaves * 64u, 0, st>>>(q);
        } else {
            gemm_packed_kernel<false><<<grid, kPkWaves * 64u, 0, st>>>(q);
        }
    }
    return launch_status(b_nk ? "ascq_matmul_w8a8 ([n, k] weight stream)" : "ascq_matmul_w8a8_packed");
}

// The weight-stationary form: any number of rows in one launch (the sums and the epilogue go in blocks of 128 rows), k
// up to 16384 (a wavefront's k range of its slabs fits 96 or 128 tile registers).  At k = 4096, n = 11008 it costs
// 9.5 us (packed weights; 11.5 us for [n, k] weights, whose tiles arrive as 16 runs of 64 bytes) plus about 1 us per
// 16 rows: every workgroup streams all of the activations, 128 MB through the L2s at 128 rows.  It takes the calls
// whose rows the resident form cannot hold in one pass: on packed weights all of them; on [n, k] weights those up to
// 224 rows at k up to 4096, where it leads the K-split tiles (20.4 against 24.4 us at 128 rows), and at longer k
// those up to 64 rows (k up to 8192; 48 beyond) whose slabs one round of workgroups holds (k = 8192, n = 8192, 64
// rows: 21.2 against 23.9 us; k = 11008, n = 4096, 32 rows: 17.0 against 20.9 us; the tile kernels lead from there
// on, and at once where the workgroups need a second round).
namespace {

// chunks of kWsTpw tiles in a wavefront's k range; the slabs a workgroup's registers hold then; the grid: one
// workgroup per compute unit when that leaves it no more slabs than that, otherwise more workgroups
uint32_t ws_chunks(uint32_t k)
{
    const uint32_t tpw = (k / kPkTileK + kPkWaves - 1u) / kPkWaves;
    return (tpw + kWsTpw - 1u) / kWsTpw;
}

uint32_t ws_max_slabs(uint32_t nchunks) { return nchunks == 1u ? 3u : nchunks == 2u ? 2u : 1u; }

uint32_t ws_grid(uint32_t slabs, uint32_t max_slabs)
{
    const uint32_t cus = device_compute_units();
    uint32_t grid = slabs < cus ? slabs : cus;
    if ((slabs + grid - 1u) / grid > max_slabs) {
        grid = (slabs + max_slabs - 1u) / max_slabs;
    }
    return grid;
}

}  // namespace

bool gemm_ws_supported(const GemmParams& p, bool b_nk)
{
    if (p.k % kPkTileK != 0 || p.k / kPkTileK > kPkWaves * kWsTpw * kWsMaxChunks) {
        return false;
    }
    if (p.m <= gemm_packed_pass_rows(p)) {
        return false;  // the activations fit the LDS: the resident form
    }
    if (!b_nk) {
        return gemm_packed_supported(p);
    }
    if (!gemm_packed_nk_supported(p)) {
        return false;
    }
    const uint32_t nchunks = ws_chunks(p.k);
    if (nchunks == 1u) {
        return p.m <= kWsNkMaxRows;
    }
    return p.m <= (nchunks == 2u ? 64u : 48u) && ws_grid((p.n + kPkCols - 1u) / kPkCols, ws_max_slabs(nchunks)) <= device_compute_units();
}

// Rounds of workgroups the weight-stationary form needs on this device (1: every workgroup is resident at once).
uint32_t gemm_ws_rounds(const GemmParams& p)
{
    const uint32_t cus = device_compute_units();
    return (ws_grid((p.n + kPkCols - 1u) / kPkCols, ws_max_slabs(ws_chunks(p.k))) + cus - 1u) / cus;
}

int launch_gemm_ws(const GemmParams& p, hipStream_t st, bool b_nk)
{
    PackedParams q{};
    q.wp = reinterpret_cast<const i32x4*>(p.b);
    q.a = p.a;
    q.n = p.n;
    q.k = p.k;
    q.slabs = (p.n + kPkCols - 1u) / kPkCols;
    q.ktiles = p.k / kPkTileK;
    q.tpw = (q.ktiles + kPkWaves - 1u) / kPkWaves;
    q.epi = p.epi;
    q.rows_magic = 0;
    const uint32_t nchunks = ws_chunks(p.k), max_slabs = ws_max_slabs(nchunks);
    const uint32_t grid = ws_grid(q.slabs, max_slabs);
    q.m0 = 0;
    q.rows = p.m;
    if (plan_note(ASCQ_MM_KERNEL_STREAM, kWsRows, kPkCols * ((q.slabs + grid - 1u) / grid), kPkTileK, grid, 1,
                  2u * kPkWaves * kWsSlot + kWsRows * max_slabs * kPkCols * 4u, 0)) {
        return ASCQ_OK;
    }
    auto go = [&](auto nk) {
        constexpr bool kNK = decltype(nk)::value;
        if (nchunks == 1u) {
            gemm_ws_kernel<kNK, 3, 1><<<grid, kPkWaves * 64u, 0, st>>>(q);
        } else if (nchunks == 2u) {
            gemm_ws_kernel<kNK, 2, 2><<<grid, kPkWaves * 64u, 0, st>>>(q);
        } else {
            gemm_ws_kernel<kNK, 1, 4><<<grid, kPkWaves * 64u, 0, st>>>(q);
        }
    };
    if (b_nk) {
        go(std::true_type{});
    } else {
        go(std::false_type{});
    }
    return launch_status(b_nk ? "ascq_matmul_w8a8 ([n, k] weights held in registers)"
                              : "ascq_matmul_w8a8_packed (weights held in registers)");
}

// The fused form: x [m, k] of halves or bfloat16s is quantised per token inside the kernel (p.epi.has_tok must be set;
// p.a and p.epi.tok_scale are not read).  False when the shape does not fit (the caller then runs the two kernels).
// On [n, k] weights the form runs where the LDS ring for the weights fits beside the rows (7 rows at k = 4096, 4 at
// 7168, 2 at 14848): without the ring the separate quantiser and the ring kernel for the matmul are level or ahead.
bool gemm_packed_dyn_fits(uint32_t m, uint32_t k, bool b_nk)
{
    if (m == 0u || m > kPkDynRows || k % kPkTileK != 0) {
        return false;
    }
    const uint32_t tpw = (k / kPkTileK + kPkWaves - 1u) / kPkWaves;
    // (the staged rows take twice the int8 image's bytes, of twice the space)
    return m * kPkWaves * (tpw * kPkTileK + kPkRowPad) <= (b_nk ? kPkDynRingQBytes : kPkDynQBytes);
}

int launch_gemm_packed_dyn(const GemmParams& p, const void* x, bool x_bf16, hipStream_t st, bool b_nk)
{
    const uint32_t cus = device_compute_units();
    PackedParams q{};
    q.wp = reinterpret_cast<const i32x4*>(p.b);
    q.a = nullptr;
    q.n = p.n;
    q.k = p.k;
    q.slabs = (p.n + kPkCols - 1u) / kPkCols;
    q.ktiles = p.k / kPkTileK;
    q.tpw = (q.ktiles + kPkWaves - 1u) / kPkWaves;
    q.epi = p.epi;
    q.m0 = 0;
    q.rows = p.m;
    q.rows_magic = static_cast<uint32_t>(((1ull << 32) + q.rows - 1u) / q.rows);
    uint32_t grid = q.slabs < cus ? q.slabs : cus;
    if ((q.slabs + grid - 1u) / grid > kPkMaxSlabs) {
        grid = (q.slabs + kPkMaxSlabs - 1u) / kPkMaxSlabs;
    }
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    if (!gemm_packed_dyn_fits(p.m, p.k, b_nk)) {
        return fail(ASCQ_EUNSUPPORTED, "ascq_linear_w8a8_dynamic: %u rows of k = %u do not fit the fused decode kernel", p.m, p.k);
    }
    if (b_nk) {  // [n, k] weights go through the LDS ring
        if (x_bf16) {
            gemm_packed_dyn_kernel<true, true, true><<<grid, kPkWaves * 64u, 0, st>>>(q, xp);
        } else {
            gemm_packed_dyn_kernel<true, false, true><<<grid, kPkWaves * 64u, 0, st>>>(q, xp);
        }
    } else if (x_bf16) {
        gemm_packed_dyn_kernel<false, true><<<grid, kPkWaves * 64u, 0, st>>>(q, xp);
    } else {
        gemm_packed_dyn_kernel<false, false><<<grid, kPkWaves * 64u, 0, st>>>(q, xp);
    }
    return launch_status("ascq_linear_w8a8_dynamic (fused decode kernel)");
}

}  // namespace ascq

using namespace ascq;

extern "C" int ascq_pack_weight_w8_size(uint32_t k, uint32_t n, size_t* bytes)
{
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_pack_weight_w8_size: bytes is NULL");
    ASCQ_REQUIRE(k > 0 && n > 0, ASCQ_EINVAL, "ascq_pack_weight_w8_size: k, n must be positive");
    *bytes = (static_cast<size_t>((n + kPkCols - 1u) / kPkCols) * ((k + kPkTileK - 1u) / kPkTileK) + kPkPadTiles) * kPkTileBytes;
    return ASCQ_OK;
}

extern "C" int ascq_pack_weight_w8(const void* w, void* packed, uint32_t k, uint32_t n, int32_t trans_b, void* stream)
{
    ASCQ_REQUIRE(w && packed, ASCQ_ENULL, "ascq_pack_weight_w8: w / packed is NULL");
    ASCQ_REQUIRE(k > 0 && n > 0, ASCQ_EINVAL, "ascq_pack_weight_w8: k, n must be positive");
    ASCQ_REQUIRE(aligned16(packed), ASCQ_EALIGN, "ascq_pack_weight_w8: packed must be 16-byte aligned");
    ASCQ_REQUIRE(w != packed, ASCQ_EINVAL, "ascq_pack_weight_w8: packed must not be w");
    const uint32_t slabs = (n + kPkCols - 1u) / kPkCols, ktiles = (k + kPkTileK - 1u) / kPkTileK;
    const size_t lanes = (static_cast<size_t>(slabs) * ktiles + kPkPadTiles) * 64u;
    ASCQ_REQUIRE((lanes + 255u) / 256u < (1ull << 31), ASCQ_EINVAL, "ascq_pack_weight_w8: matrix too large");
    pack_w8_kernel<<<static_cast<uint32_t>((lanes + 255u) / 256u), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const int8_t*>(w), static_cast<i32x4*>(packed), k, n, slabs, ktiles, trans_b != 0);
    return launch_status("ascq_pack_weight_w8");
}
