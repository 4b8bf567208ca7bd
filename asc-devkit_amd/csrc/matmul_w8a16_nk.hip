// W8A16 with the weights given as [n, k] (the reference's isTransposeB): y[m, n] = x[m, k] * dequant(w)[n, k]^T.
//
// In this layout a column of the product owns one contiguous run of k bytes, so whole columns can belong to one
// workgroup and nothing has to be added across workgroups: one launch, no workspace, a fixed summation order.
//   * a workgroup of 8 wavefronts owns up to 8 groups of 16 columns; its wavefronts split k into runs of 128;
//   * per 128 k a lane fetches 2 x 16 bytes of one column (lane l: column l % 16, bytes 16 (l / 16) .. + 15 of each
//     64-byte half), which are the B operands of four v_mfma_f32_16x16x32_f16 as they lie: the 8 consecutive k of a
//     B operand are 8 consecutive bytes; the A operand takes x at the same k, straight from global memory (x is small
//     and is read once per wavefront and run, for all column groups of the workgroup);
//   * a byte becomes an exact half by a byte permute into 0x6400 | (w + 128) = 1152 + w, one exact subtraction gives w,
//     then one rounded half add of the column's offset and one rounded half multiply by its scale, as
//     AscendAntiQuant<int8_t, half> (ref: impl/adv_api/detail/matmul/stage/copy_cube_in/antiquant/
//     antiquant_processor_using_ub.h:53-130); scale and offset belong to the lane's column, so they are lane constants;
//   * the 8 partial sums of a column group are added in wavefront order in LDS and rounded once to the output type.
// Up to 16 activation rows per pass; the host loops over more.  Requires k % 128 == 0, x / w 16-byte aligned.
#include <type_traits>
#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

constexpr uint32_t kWaves = 8, kMaxGroups = 8, kRows = 16, kRun = 128;
// up to this many rows the whole-column kernel runs, 16 rows per pass (two passes cost what one pass of the tile GEMM
// over up to 128 rows costs: 120 us at k = 8192, n = 28672)
constexpr uint32_t kDecodeRows = 32;

struct NkParams {
    const uint16_t* x;       // [m, k] halves (this pass's first row)
    const uint8_t* w;        // [n, k] int8
    const uint16_t* scale;   // [n] halves, or nullptr: scale_bits / offset_bits for every column
    const uint16_t* offset;  // [n] halves (only read when has_offset)
    void* y;                 // [m, n] halves or floats (this pass's first row)
    uint32_t m, n, k;        // m: rows of this pass, at most 16
    uint32_t groups;         // column groups per workgroup, 1 .. kMaxGroups (selects the kernel instantiation)
    uint32_t out_f32;
    uint32_t scale_bits, offset_bits;
};

__device__ __forceinline__ f16x2_t h2_from_bits(uint32_t b)
{
    f16x2_t r;
    __builtin_memcpy(&r, &b, 4);
    return r;
}

// four int8 of a dword -> two dwords of packed halves (bytes 0, 1 and bytes 2, 3), de-quantised
template <bool kHasOffset>
__device__ __forceinline__ void dequant4(uint32_t wbytes, f16x2_t scale2, f16x2_t offset2, uint32_t& lo, uint32_t& hi)
{
    const uint32_t flipped = wbytes ^ 0x80808080u;  // w + 128 as an unsigned byte
    // 0x64 in the high byte of each half: selector 0x0c would give 0x00, so the constant comes from the second source
    const uint32_t k64 = 0x64646464u;
    f16x2_t a = h2_from_bits(__builtin_amdgcn_perm(k64, flipped, 0x04010400u));  // (1152 + w0, 1152 + w1)
    f16x2_t b = h2_from_bits(__builtin_amdgcn_perm(k64, flipped, 0x04030402u));  // (1152 + w2, 1152 + w3)
    const f16x2_t bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    a = a - bias;  // exact
    b = b - bias;
    if constexpr (kHasOffset) {
        a = a + offset2;
        b = b + offset2;
    }
    a = scale2 * a;
    b = scale2 * b;
    __builtin_memcpy(&lo, &a, 4);
    __builtin_memcpy(&hi, &b, 4);
}

// G: column groups per workgroup (the same for every workgroup of a launch; the last one may own fewer and then repeats
// its last group, whose duplicate results are not stored).
template <bool kHasOffset, int G>
__global__ __launch_bounds__(kWaves * 64) void w8a16_nk_kernel(NkParams p)
{
    __shared__ float RED[kWaves][G][4][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t n_groups = (p.n + 15u) / 16u;
    const uint32_t g0 = blockIdx.x * G;  // first column group of this workgroup
    if (g0 >= n_groups) {
        return;
    }
    const uint32_t my_groups = n_groups - g0 < G ? n_groups - g0 : G;

    // the lane's column in each group: its weights, scale and offset (columns past n repeat the last one; their
    // results are never stored)
    const uint8_t* wcol[G];
    f16x2_t sc[G], of[G];
#pragma unroll
    for (uint32_t g = 0; g < G; ++g) {
        uint32_t col = (g0 + (g < my_groups ? g : my_groups - 1u)) * 16u + lc;
        col = col < p.n ? col : p.n - 1u;
        wcol[g] = p.w + static_cast<size_t>(col) * p.k + 16u * lq;
        const uint32_t sb = p.scale ? p.scale[col] : p.scale_bits;
        const uint32_t ob = kHasOffset ? (p.scale ? p.offset[col] : p.offset_bits) : 0u;
        sc[g] = h2_from_bits(sb | (sb << 16));
        of[g] = h2_from_bits(ob | (ob << 16));
    }
    // the lane's row of x (rows past m read row 0 and are masked to zero)
    const bool row_ok = lc < p.m;
    const uint16_t* xrow = p.x + static_cast<size_t>(row_ok ? lc : 0u) * p.k + 16u * lq;

    f32x4_t acc[G];
#pragma unroll
    for (uint32_t g = 0; g < G; ++g) acc[g] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // One run = 128 k: per column group two 16-byte weight loads, for x four (halves 16 lq .. + 15 of both 64-k halves:
    // two B-operand-sized pieces of 8 each).  All loads of a run are issued together, unconditionally, one run ahead.
    auto load_run = [&](uint32_t r, u32x4 (&wv)[G][2], u32x4 (&xa)[4]) __attribute__((always_inline)) {
        const uint32_t k0 = r * kRun;
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) {
            wv[g][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wcol[g] + k0));
            wv[g][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wcol[g] + k0 + 64u));
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const u32x4* src = reinterpret_cast<const u32x4*>(xrow + k0 + 64u * h);
            xa[2 * h] = src[0];
            xa[2 * h + 1] = src[1];
        }
    };
    auto compute_run = [&](const u32x4 (&wv)[G][2], const u32x4 (&xraw)[4]) __attribute__((always_inline)) {
        u32x4 xa[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) xa[i] = row_ok ? xraw[i] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int part = 0; part < 2; ++part) {  // bytes 8 part .. 8 part + 7 of the lane's 16
                    uint32_t b0, b1, b2, b3;
                    dequant4<kHasOffset>(wv[g][h][2 * part], sc[g], of[g], b0, b1);
                    dequant4<kHasOffset>(wv[g][h][2 * part + 1], sc[g], of[g], b2, b3);
                    const u32x4 bq = {b0, b1, b2, b3};
                    f16x8_t bop, aop;
                    __builtin_memcpy(&bop, &bq, 16);
                    __builtin_memcpy(&aop, &xa[2 * h + part], 16);
                    // D[row][col] += sum_k A[row][k] B[k][col]: A = x (rows), B = weights (columns)
                    acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, bop, acc[g], 0, 0, 0);
                }
            }
        }
    };

    // runs dealt to the wavefronts in contiguous shares (a share may be empty when k is short)
    const uint32_t runs = p.k / kRun;
    const uint32_t r_begin = runs * wave / kWaves, r_end = runs * (wave + 1u) / kWaves;
    if (r_begin < r_end) {
        u32x4 w0[G][2], w1[G][2], x0[4], x1[4];
        const uint32_t last = r_end - 1u;
        load_run(r_begin, w0, x0);
        for (uint32_t r = r_begin; r < r_end; r += 2) {
            load_run(r + 1u < last ? r + 1u : last, w1, x1);
            compute_run(w0, x0);
            load_run(r + 2u < last ? r + 2u : last, w0, x0);
            if (r + 1u < r_end) {
                compute_run(w1, x1);
            }
        }
    }

    // ---- the wavefronts' partial sums, added in wavefront order; register i of lane l is row 4 (l / 16) + i,
    // column l % 16 of the group
#pragma unroll
    for (uint32_t g = 0; g < G; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) RED[wave][g][i][lane] = acc[g][i];
    }
    __syncthreads();
    if (wave < my_groups) {
        const uint32_t g = wave;
        const uint32_t col = (g0 + g) * 16u + lc;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = RED[0][g][i][lane];
#pragma unroll
            for (uint32_t wv = 1; wv < kWaves; ++wv) s += RED[wv][g][i][lane];
            const uint32_t row = 4u * lq + static_cast<uint32_t>(i);
            if (row < p.m && col < p.n) {
                const size_t idx = static_cast<size_t>(row) * p.n + col;
                if (p.out_f32) {
                    static_cast<float*>(p.y)[idx] = s;
                } else {
                    static_cast<uint16_t*>(p.y)[idx] = static_cast<uint16_t>(f32_to_half_bits(s));
                }
            }
        }
    }
}

template <bool kHasOffset>
void launch_nk(const NkParams& p, uint32_t grid, hipStream_t st)
{
    switch (p.groups) {
        case 1: w8a16_nk_kernel<kHasOffset, 1><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 2: w8a16_nk_kernel<kHasOffset, 2><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 3: w8a16_nk_kernel<kHasOffset, 3><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 4: w8a16_nk_kernel<kHasOffset, 4><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 5: w8a16_nk_kernel<kHasOffset, 5><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 6: w8a16_nk_kernel<kHasOffset, 6><<<grid, kWaves * 64, 0, st>>>(p); break;
        case 7: w8a16_nk_kernel<kHasOffset, 7><<<grid, kWaves * 64, 0, st>>>(p); break;
        default: w8a16_nk_kernel<kHasOffset, 8><<<grid, kWaves * 64, 0, st>>>(p); break;
    }
}

// ---- up to 4 activation rows: one flat sweep over the weights with the activations resident in LDS.
// The kernel above fetches its rows of x from memory run by run, in the same in-order queue of the compute unit as
// the weights; here a wavefront stages its k range of every row once (direct-to-LDS loads) and then has nothing but
// weights in flight: batches of 4 tiles (64 k x 16 columns: the lane's 16 bytes are 16 consecutive k of its column),
// two register buffers, buffer loads whose lane offset is column * k + 16 (l / 16) and whose scalar offset walks the
// tiles, so that columns past n fall outside the buffer and read as zeros.  The workgroups of an XCD own neighbouring
// column groups.
//   kSum = false: the reference's arithmetic per weight (dequant4 above), two MFMAs per tile.
//   kSum = true (ASCQ_W8A16_CHANNEL_SUM): y = scale * (sum_k x w + offset * sum_k x) with the sums in fp32.  The bytes
//   go into the matrix core as the exact halves 1152 + w (one xor and two byte permutes per dword); the bias and the
//   offset are one fma per column group and row, on sum_k x, which the matrix core adds up as well (the same A
//   operands against a B operand of ones, during the wavefront's first column group only).
constexpr uint32_t kSkTileK = 64, kSkBatch = 4, kSkMaxSlabs = 8, kSkMaxRows = 4;
constexpr int kSkBuf = 2;
constexpr uint32_t kSkRowPad = 32;             // bytes added to a staged row of x
constexpr uint32_t kSkXBytes = 96 * 1024;      // LDS for the staged activations of a workgroup
constexpr uint32_t kSkPastEnd = 0x7FFFFFF0u;
// kRing: the weights go through LDS instead of straight into registers.  Read as matrix operands, a tile of [n, k]
// weights is 16 runs of 64 bytes per load instruction, which a compute unit's load path takes at about half the rate
// of long runs; through a two-slot ring per wavefront a load instruction brings four columns' 256 bytes (the four
// tiles of a batch), the 16-byte pieces of column c stored at position piece ^ c so that the 16 lanes reading one
// piece of 16 columns fall on 16 bank groups.  The loads are range-checked buffer loads to LDS; every LDS read of the
// loop is written as an instruction (one the compiler knows of makes it wait for all the weights in flight).
constexpr uint32_t kSkSlot = kSkBatch * 16u * kSkTileK;    // 4 KiB: 16 columns x 256 bytes
constexpr uint32_t kSkRing = kWaves * 2u * kSkSlot;        // 64 KiB
constexpr uint32_t kSkRingXBytes = 76 * 1024;              // what is left for the staged activations beside it
typedef __attribute__((address_space(3))) void* sk_lds_t;

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;

struct SkParams {
    const uint16_t* x;       // [rows, k] halves (this pass's first row)
    const uint8_t* w;        // [n, k] int8
    const uint16_t* scale;   // [n] halves, or nullptr: scale_bits / offset_bits for every column
    const uint16_t* offset;
    void* y;                 // [rows, n] halves or floats (this pass's first row)
    uint32_t rows, n, k;     // rows of this pass, 1 .. 4
    uint32_t slabs, ktiles, tpw;
    uint32_t out_f32;
    uint32_t scale_bits, offset_bits;
};

__device__ __forceinline__ uint32_t sk_xcd_order(uint32_t wg, uint32_t wgs)
{
    return (wgs & 7u) == 0u ? (wg & 7u) * (wgs >> 3) + (wg >> 3) : wg;
}

template <bool kHasOffset, bool kSum, bool kRing>
__global__ __launch_bounds__(kWaves * 64) void w8a16_nk_stream_kernel(SkParams p)
{
    __shared__ __attribute__((aligned(1024))) char RING[kRing ? kSkRing : 1024u];
    __shared__ __attribute__((aligned(16))) char XS[kRing ? kSkRingXBytes : kSkXBytes];
    __shared__ float RED[kWaves][kSkMaxSlabs][4][16];
    __shared__ uint32_t PAR[kSkMaxSlabs][16];  // (scale | offset << 16) of the workgroup's columns
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t wg = sk_xcd_order(blockIdx.x, gridDim.x);
    const uint32_t s0 = static_cast<uint32_t>(static_cast<uint64_t>(wg) * p.slabs / gridDim.x);
    const uint32_t s1 = static_cast<uint32_t>(static_cast<uint64_t>(wg + 1u) * p.slabs / gridDim.x);
    const uint32_t nslabs = s1 - s0;
    const uint32_t ta = min(wave * p.tpw, p.ktiles), tb = min(ta + p.tpw, p.ktiles), cnt = tb - ta;
    const uint32_t pitch = p.tpw * (kSkTileK * 2u) + kSkRowPad;
    char* const xs = XS + wave * (p.rows * pitch);

    // ---- this wavefront's k range of every row, straight into LDS (1 KiB of a row per instruction)
    {
        const uint32_t row_pieces = cnt * (kSkTileK * 2u / 16u);
        for (uint32_t r = 0; r < p.rows; ++r) {
            const uint16_t* src = p.x + static_cast<size_t>(r) * p.k + ta * kSkTileK + lane * 8u;
            for (uint32_t c0 = 0; c0 < row_pieces; c0 += 64u) {
                if (c0 + lane < row_pieces) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(src + c0 * 8u), (lds_ptr_t)(xs + r * pitch + c0 * 16u), 16, 0, 0);
                }
            }
        }
    }
    // ---- the columns' parameters: thread t < 16 nslabs fetches those of column group t / 16, column t % 16
    uint32_t my_par = 0;
    if (tid < nslabs * 16u) {
        uint32_t col = (s0 + (tid >> 4)) * 16u + (tid & 15u);
        col = col < p.n ? col : p.n - 1u;
        const uint32_t sb = p.scale ? p.scale[col] : p.scale_bits;
        const uint32_t ob = kHasOffset ? (p.scale ? p.offset[col] : p.offset_bits) : 0u;
        my_par = sb | (ob << 16);
    }
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.w), 0, static_cast<int>(p.n * p.k), 0x00020000);
    const uint32_t w_lane = lc * p.k + lq * 16u;
    // operand row i reads row i % rows (rows <= 4: a mask or a compare); + tile * 128
    const uint32_t xrow = p.rows == 3u ? (lc % 3u) : (lc & (p.rows - 1u));
    const uint32_t x_lane = xrow * pitch + lq * 32u;

    const uint32_t nb = (cnt + kSkBatch - 1u) / kSkBatch;
    const uint32_t batches = nb * nslabs;
    u32x4 wq[kSkBuf][kSkBatch];
    char* const ring = RING + (kRing ? wave * (2u * kSkSlot) : 0u);
    uint32_t l_slab = s0, l_b = 0, l_q = 0;
    bool l_done = batches == 0u;
    auto load = [&](int buf) __attribute__((always_inline)) {
        // every load is issued, so the waits count exactly; once every batch has been requested the lane offset lies
        // past the end of the buffer and the loads move no data.  A short last batch reads on along its columns (or
        // past the buffer's end, as zeros): not computed.
        const uint32_t l_w = l_done ? kSkPastEnd : w_lane;
        const uint32_t base = l_slab * 16u * p.k + (ta + l_b * kSkBatch) * kSkTileK;  // scalar
#pragma unroll
        for (uint32_t t = 0; t < kSkBatch; ++t) {
            if constexpr (kRing) {  // instruction t: the lane's column 4 t + lq, position lc, piece position ^ column
                const uint32_t col = 4u * t + lq;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (sk_lds_t)(ring + buf * kSkSlot + t * 1024u), 16,
                                                         l_done ? kSkPastEnd : col * p.k + ((lc ^ col) << 4), base, 0, 2);
            } else {
                wq[buf][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, l_w, base + t * kSkTileK, 2);
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
    for (int b = 0; b < kSkBuf; ++b) load(b);
    // Loads return in order: with at most the weight loads just issued outstanding, the activations have landed in LDS
    // and the parameters in their register.  (The compiler does not count direct-to-LDS loads issued in a loop.)
    __builtin_amdgcn_s_waitcnt(((kSkBuf * kSkBatch) & 15) | (((kSkBuf * kSkBatch) >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");
    if (tid < nslabs * 16u) {
        PAR[tid >> 4][tid & 15u] = my_par;
    }
    // a plain barrier: the fence of __syncthreads() would also wait for the weight loads in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f}, xsum = {0.0f, 0.0f, 0.0f, 0.0f};
    f16x2_t sc2 = {}, of2 = {};
    float corr = 0.0f;  // kSum: offset - 1152 of the lane's column
    uint32_t c_slab = 0, c_b = 0, c_q = 0;
    const f16x8_t ones = {1, 1, 1, 1, 1, 1, 1, 1};
    auto compute = [&](int buf) __attribute__((always_inline)) {
        constexpr uint32_t kBehind = (kSkBuf - 1) * kSkBatch;
        __builtin_amdgcn_s_waitcnt((kBehind & 15u) | ((kBehind >> 4) << 14) | (7u << 4) | (15u << 8));
        if (c_q >= batches) {
            return;  // uniform
        }
        if constexpr (kRing) {  // the batch's fragments out of the ring, the slot refilled at once
            const uint32_t wa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((sk_lds_t)ring)) + buf * kSkSlot + lc * 256u;
#pragma unroll
            for (uint32_t t = 0; t < kSkBatch; ++t) {
                const uint32_t addr = wa + (((4u * t + lq) ^ lc) << 4);
                asm volatile("ds_read_b128 %0, %1" : "=v"(wq[buf][t]) : "v"(addr) : "memory");
            }
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wq[buf][0]), "+v"(wq[buf][1]), "+v"(wq[buf][2]), "+v"(wq[buf][3]));
            load(buf);
        }
        if (c_b == 0u) {  // a new column group: the lane's column parameters
            uint32_t pr;
            if constexpr (kRing) {
                asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                             : "=v"(pr)
                             : "v"(static_cast<uint32_t>(reinterpret_cast<uintptr_t>((sk_lds_t)&PAR[c_slab][lc])))
                             : "memory");
            } else {
                pr = PAR[c_slab][lc];
            }
            sc2 = h2_from_bits((pr & 0xFFFFu) | (pr << 16));
            of2 = h2_from_bits((pr >> 16) | (pr & 0xFFFF0000u));
            corr = (kHasOffset ? static_cast<float>(of2[0]) : 0.0f) - 1152.0f;
        }
        const uint32_t t0 = c_b * kSkBatch;
        const uint32_t live = min(kSkBatch, cnt - t0);
        const char* xa0 = xs + x_lane + t0 * (kSkTileK * 2u);
#pragma unroll
        for (uint32_t t = 0; t < kSkBatch; ++t) {
            if (t < live) {  // uniform
                f16x8_t a0, a1;
                if constexpr (kRing) {
                    const uint32_t xa = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((sk_lds_t)xa0));
                    asm volatile("ds_read_b128 %0, %2 offset:%3\n\tds_read_b128 %1, %2 offset:%4\n\ts_waitcnt lgkmcnt(0)"
                                 : "=&v"(a0), "=&v"(a1)
                                 : "v"(xa), "i"(t * (kSkTileK * 2u)), "i"(t * (kSkTileK * 2u) + 16u)
                                 : "memory");
                } else {
                    a0 = *reinterpret_cast<const f16x8_t*>(xa0 + t * (kSkTileK * 2u));
                    a1 = *reinterpret_cast<const f16x8_t*>(xa0 + t * (kSkTileK * 2u) + 16u);
                }
                uint32_t h[8];
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    if constexpr (kSum) {
                        const uint32_t flipped = wq[buf][t][d] ^ 0x80808080u;  // w + 128 as an unsigned byte
                        h[2 * d] = __builtin_amdgcn_perm(0x64646464u, flipped, 0x04010400u);      // (1152 + w0, 1152 + w1)
                        h[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, flipped, 0x04030402u);  // (1152 + w2, 1152 + w3)
                    } else {
                        dequant4<kHasOffset>(wq[buf][t][d], sc2, of2, h[2 * d], h[2 * d + 1]);
                    }
                }
                const u32x4 q0 = {h[0], h[1], h[2], h[3]}, q1 = {h[4], h[5], h[6], h[7]};
                f16x8_t b0, b1;
                __builtin_memcpy(&b0, &q0, 16);
                __builtin_memcpy(&b1, &q1, 16);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc, 0, 0, 0);
                if (kSum && c_slab == 0u) {  // uniform: sum_k x of this wavefront's k range, once
                    xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, ones, xsum, 0, 0, 0);
                    xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, ones, xsum, 0, 0, 0);
                }
            }
        }
        ++c_q;
        if (++c_b == nb) {  // the column group is done: register i of lane l is row 4 (l / 16) + i, column l % 16
            if (lq == 0u) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    RED[wave][c_slab][i][lc] = kSum ? __builtin_fmaf(corr, xsum[i], acc[i]) : acc[i];
                }
            }
            acc = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            c_b = 0;
            ++c_slab;
        }
    };
    for (uint32_t q = 0; q < batches; q += kSkBuf) {
#pragma unroll
        for (int b = 0; b < kSkBuf; ++b) {
            compute(b);
            if constexpr (!kRing) {
                load(b);
            }
        }
    }
    if constexpr (kRing) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the requests past the last batch
    }
    if (batches == 0u && lq == 0u) {  // a wavefront without tiles (k shorter than 8 tiles) contributes zeros
        for (uint32_t s = 0; s < nslabs; ++s) {
#pragma unroll
            for (int i = 0; i < 4; ++i) RED[wave][s][i][lc] = 0.0f;
        }
    }
    __syncthreads();

    // ---- the eight partial sums of every element in wavefront order, one rounding, store
    const uint32_t outs = nslabs * p.rows * 16u;
    for (uint32_t i = tid; i < outs; i += kWaves * 64u) {
        const uint32_t s = i / (p.rows * 16u), rc = i % (p.rows * 16u);
        const uint32_t r = rc >> 4, c = rc & 15u;
        const uint32_t col = (s0 + s) * 16u + c;
        float sum = RED[0][s][r][c];
#pragma unroll
        for (uint32_t wv = 1; wv < kWaves; ++wv) sum += RED[wv][s][r][c];
        if constexpr (kSum) {
            const uint32_t pr = PAR[s][c];
            sum = sum * half_bits_to_f32(pr & 0xFFFFu);
        }
        if (col < p.n) {
            const size_t idx = static_cast<size_t>(r) * p.n + col;
            if (p.out_f32) {
                static_cast<float*>(p.y)[idx] = sum;
            } else {
                static_cast<uint16_t*>(p.y)[idx] = static_cast<uint16_t>(f32_to_half_bits(sum));
            }
        }
    }
}

// ---- many activation rows: a half GEMM whose B-tile loader de-quantises.
// Workgroup = 4 wavefronts (2 x 2) on a 128 x 128 tile, K step 64, two LDS stages of 32 KiB (two workgroups per compute
// unit).  Both tiles sit in LDS as [row or column][64 k] halves, 128 bytes per line in 8 pieces of 16 bytes, piece c of
// line r stored at position c ^ ((r >> 1) & 7): a 16-byte access is served 16 lanes (256 bytes, all 64 banks) at a
// time, two lines fill one 256-byte bank row, so the sixteen neighbouring lines of such a group must put their piece
// into eight different positions per line parity.  A thread stages 32 bytes of one column of B per K step (registers: load, de-quantise exactly as
// the decode kernel does, four 16-byte LDS writes) and two 16-byte pieces of A; the global loads of the next K step are
// issued before the MFMAs of the current one.  v_mfma_f32_32x32x16_f16: lane l holds row (column) l % 32 and the 8
// consecutive k 8 (l / 32) .. + 7 of a K sub-step, i.e. one 16-byte piece of a line.
constexpr uint32_t kGM = 128, kGN = 128, kGK = 64;
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <bool kHasOffset>
__global__ __launch_bounds__(256, 2) void w8a16_nk_gemm_kernel(NkParams p, uint32_t tiles_m)
{
    __shared__ __attribute__((aligned(16))) uint8_t AS[2][kGM * kGK * 2];
    __shared__ __attribute__((aligned(16))) uint8_t BS[2][kGN * kGK * 2];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    // an XCD (workgroup id mod 8) takes a contiguous share of the tiles, ordered in bands of 8 row tiles: the
    // workgroups that run side by side in it share their rows of x and their columns of B in its L2
    const uint32_t tiles_n = (p.n + kGN - 1u) / kGN;
    const uint32_t t = xcd_remap(blockIdx.x, tiles_m * tiles_n);
    if (t == 0xFFFFFFFFu) {
        return;  // whole workgroup (the launch is rounded up to a multiple of 8)
    }
    uint32_t tm, tn;
    band_order(t, tiles_m, tiles_n, tm, tn);
    const uint32_t row0 = tm * kGM, col0 = tn * kGN;

    // ---- staging roles
    // B: thread t stages bytes 32 (t & 1) .. + 31 of column col0 + t / 2 (pieces 4 (t & 1) .. + 3 of its LDS line)
    const uint32_t bcol_l = tid >> 1, bhalf = tid & 1u;
    uint32_t bcol = col0 + bcol_l;
    bcol = bcol < p.n ? bcol : p.n - 1u;
    const uint8_t* bsrc = p.w + static_cast<size_t>(bcol) * p.k + 32u * bhalf;
    const uint32_t sb = p.scale ? p.scale[bcol] : p.scale_bits;
    const uint32_t ob = kHasOffset ? (p.scale ? p.offset[bcol] : p.offset_bits) : 0u;
    const f16x2_t sc2 = h2_from_bits(sb | (sb << 16)), of2 = h2_from_bits(ob | (ob << 16));
    // A: thread t stages pieces (t & 7) of rows t / 8 and t / 8 + 32 .. (four rows, 16 bytes each)
    const uint32_t apiece = tid & 7u, arow_l = tid >> 3;
    const uint16_t* asrc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t r = row0 + arow_l + 32u * j;
        r = r < p.m ? r : p.m - 1u;
        asrc[j] = p.x + static_cast<size_t>(r) * p.k + 8u * apiece;
    }

    // Two register sets for the raw data of the next two K steps: the loads of step s + 2 are issued while step s
    // computes, and the data of step s + 1 is de-quantised and written to the other LDS stage in four parts, one behind
    // the MFMAs of each K sub-step, so that the vector ALU works while the matrix pipe is busy.
    struct Raw {
        u32x4 b[2], a[4];
    };
    auto fetch = [&](Raw& raw, uint32_t step) __attribute__((always_inline)) {
        const uint32_t k0 = step * kGK;
        raw.b[0] = *reinterpret_cast<const u32x4*>(bsrc + k0);
        raw.b[1] = *reinterpret_cast<const u32x4*>(bsrc + k0 + 16u);
#pragma unroll
        for (int j = 0; j < 4; ++j) raw.a[j] = *reinterpret_cast<const u32x4*>(asrc[j] + k0);
    };
    // part q of a step's staging: piece q of the thread's half line of B, piece q of its A pieces
    auto stage_part = [&](const Raw& raw, uint32_t st, int q) __attribute__((always_inline)) {
        uint32_t h0, h1, h2, h3;
        dequant4<kHasOffset>(raw.b[q >> 1][2 * (q & 1)], sc2, of2, h0, h1);
        dequant4<kHasOffset>(raw.b[q >> 1][2 * (q & 1) + 1], sc2, of2, h2, h3);
        const uint32_t piece = 4u * bhalf + static_cast<uint32_t>(q);
        *reinterpret_cast<u32x4*>(&BS[st][bcol_l * 128u + ((piece ^ ((bcol_l >> 1) & 7u)) << 4)]) = u32x4{h0, h1, h2, h3};
        const uint32_t r = arow_l + 32u * static_cast<uint32_t>(q);
        *reinterpret_cast<u32x4*>(&AS[st][r * 128u + ((apiece ^ ((r >> 1) & 7u)) << 4)]) = raw.a[q];
    };

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const uint32_t lrow = lane & 31u, lk = lane >> 5;  // operand line and which 8 k of a sub-step
    // one K step on LDS stage st; `next` (data of the following step) is staged into the other LDS stage when do_stage
    auto step_body = [&](uint32_t st, const Raw& next, auto do_stage) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t piece = 2u * ks + lk;
            f16x8_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t r = wm * 64u + i * 32u + lrow;
                af[i] = *reinterpret_cast<const f16x8_t*>(&AS[st][r * 128u + ((piece ^ ((r >> 1) & 7u)) << 4)]);
                const uint32_t c = wn * 64u + i * 32u + lrow;
                bf[i] = *reinterpret_cast<const f16x8_t*>(&BS[st][c * 128u + ((piece ^ ((c >> 1) & 7u)) << 4)]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
            if constexpr (decltype(do_stage)::value) {  // the other stage was last read before the barrier that ended the previous step
                stage_part(next, st ^ 1u, ks);
            }
        }
    };

    const uint32_t steps = p.k / kGK;
    const uint32_t last = steps - 1u;
    Raw r0, r1;
    fetch(r0, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) stage_part(r0, 0, q);
    fetch(r1, 1u < last ? 1u : last);  // data of step 1 (clamped: a single-step problem re-reads step 0 and drops it)
    __syncthreads();
    // Steps in pairs, an odd last one behind the loop, and nothing in a pair conditional (past the end the fetches
    // repeat the last step's and the staging fills an LDS stage nobody reads): with a second half that can be skipped
    // the compiler sees a path on which the first half's fetch is the newest load at the loop's top and waits there
    // for every load in every pass, which takes the fetches' two-step lead away.
    uint32_t s = 0;
    for (; s + 1u < steps; s += 2) {
        // step s on stage 0: r1 holds step s + 1; fetch step s + 2 into r0
        fetch(r0, s + 2u < last ? s + 2u : last);
        step_body(0u, r1, std::true_type{});
        __syncthreads();
        fetch(r1, s + 3u < last ? s + 3u : last);
        step_body(1u, r0, std::true_type{});
        __syncthreads();
    }
    if (s < steps) {
        step_body(0u, r1, std::false_type{});
        __syncthreads();
    }

    // ---- register r of lane l in a 32 x 32 block: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
    if (!p.out_f32 && p.n % 2u == 0) {
        // half output: after one swap between neighbouring lanes the even lane holds columns (l, l + 1) of the
        // wavefront's first block of 32 and the odd lane columns (l - 1, l) of the second: one dword store per lane,
        // and the 32 lanes of a row write one full 128-byte line
        const bool odd = (lane & 1u) != 0;
        const uint32_t colw = col0 + wn * 64u;
        const uint32_t col = odd ? colw + 32u + (lrow - 1u) : colw + lrow;  // first column of the lane's pair
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = row0 + wm * 64u + i * 32u + 8u * (r >> 2) + 4u * lk + (r & 3);
                const uint32_t h0 = f32_to_half_bits(acc[i][0][r]), h1 = f32_to_half_bits(acc[i][1][r]);
                const uint32_t recv = static_cast<uint32_t>(
                    __builtin_amdgcn_mov_dpp(static_cast<int>(odd ? h0 : h1), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                const uint32_t word = odd ? (recv | (h1 << 16)) : (h0 | (recv << 16));
                if (row < p.m && col < p.n) {
                    __builtin_nontemporal_store(word, reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(p.y) +
                                                                                  static_cast<size_t>(row) * p.n + col));
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t col = col0 + wn * 64u + j * 32u + lrow;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = row0 + wm * 64u + i * 32u + 8u * (r >> 2) + 4u * lk + (r & 3);
                if (row < p.m && col < p.n) {
                    const size_t idx = static_cast<size_t>(row) * p.n + col;
                    if (p.out_f32) {
                        static_cast<float*>(p.y)[idx] = acc[i][j][r];
                    } else {
                        static_cast<uint16_t*>(p.y)[idx] = static_cast<uint16_t>(f32_to_half_bits(acc[i][j][r]));
                    }
                }
            }
        }
    }
}

// int8 [k, n] -> [n, k] through 64 x 64 tiles in LDS (the tile GEMM wants k-contiguous weights).  k % 64 == 0.
// kVec: n % 16 == 0 and src 16-byte aligned, so a thread's 16 columns of a row are one load.
template <bool kVec>
__global__ __launch_bounds__(256) void transpose_i8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                           uint32_t k, uint32_t n)
{
    __shared__ __attribute__((aligned(16))) uint8_t T[64][68];
    const uint32_t tiles_n = (n + 63u) / 64u;
    const uint32_t k0 = (blockIdx.x / tiles_n) * 64u, n0 = (blockIdx.x % tiles_n) * 64u;
    const uint32_t t = threadIdx.x, r = t >> 2, c = (t & 3u) * 16u;
    const uint8_t* row = src + static_cast<size_t>(k0 + r) * n;
    if constexpr (kVec) {
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (n0 + c < n) {
            v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + n0 + c));
        }
#pragma unroll
        for (uint32_t w = 0; w < 4; ++w) *reinterpret_cast<uint32_t*>(&T[r][c + 4u * w]) = v[w];
    } else {
#pragma unroll
        for (uint32_t i = 0; i < 16; ++i) {
            const uint32_t col = n0 + c + i;
            T[r][c + i] = row[col < n ? col : n - 1u];
        }
    }
    __syncthreads();
    if (n0 + r < n) {
        uint32_t out[4];
#pragma unroll
        for (uint32_t w = 0; w < 4; ++w) {
            out[w] = 0;
#pragma unroll
            for (uint32_t b = 0; b < 4; ++b) out[w] |= static_cast<uint32_t>(T[c + 4u * w + b][r]) << (8u * b);
        }
        *reinterpret_cast<u32x4*>(dst + static_cast<size_t>(n0 + r) * k + k0 + c) = u32x4{out[0], out[1], out[2], out[3]};
    }
}

}  // namespace

bool w8a16_nk_supported(uint32_t k, const void* x, const void* w)
{
    return k % kRun == 0 && aligned16(x) && aligned16(w);
}

int launch_w8a16_nk(const void* x, const void* w, const void* scale, const void* offset, void* y, uint32_t m, uint32_t n,
                    uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits, uint32_t offset_bits, hipStream_t st,
                    bool channel_sum);

// Weights given as [k, n] and many rows: transposed once into the caller's workspace (k * n bytes), then the tile GEMM.
bool w8a16_kn_gemm_supported(uint32_t m, uint32_t k, const void* x, const void* w)
{
    return m > 96u && k % kGK == 0 && aligned16(x) && (reinterpret_cast<uintptr_t>(w) & 3u) == 0;
}

int launch_w8a16_kn_via_transpose(const void* x, const void* w, const void* scale, const void* offset, void* y,
                                  uint32_t m, uint32_t n, uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits,
                                  uint32_t offset_bits, void* workspace, hipStream_t st)
{
    const uint32_t tiles = (k / 64u) * ((n + 63u) / 64u);
    if (n % 16u == 0 && aligned16(w)) {
        transpose_i8_kernel<true><<<tiles, 256, 0, st>>>(static_cast<const uint8_t*>(w), static_cast<uint8_t*>(workspace), k, n);
    } else {
        transpose_i8_kernel<false><<<tiles, 256, 0, st>>>(static_cast<const uint8_t*>(w), static_cast<uint8_t*>(workspace), k, n);
    }
    return launch_w8a16_nk(x, workspace, scale, offset, y, m, n, k, has_offset, out_f32, scale_bits, offset_bits, st,
                           false);
}

// x, y: first row of the whole problem; m rows in passes of 16.
int launch_w8a16_nk(const void* x, const void* w, const void* scale, const void* offset, void* y, uint32_t m, uint32_t n,
                    uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits, uint32_t offset_bits, hipStream_t st,
                    bool channel_sum)
{
    // up to 4 rows (k % 64 == 0, offsets that fit the buffer loads' 31 bits, activations that fit the LDS): the stream
    // kernel with the activations resident
    if (m <= kSkMaxRows && k % kSkTileK == 0 && static_cast<uint64_t>(n + 16u) * k < (1ull << 31) - 64u * kSkTileK) {
        SkParams q{};
        q.x = static_cast<const uint16_t*>(x);
        q.w = static_cast<const uint8_t*>(w);
        q.scale = static_cast<const uint16_t*>(scale);
        q.offset = static_cast<const uint16_t*>(offset);
        q.y = y;
        q.rows = m;
        q.n = n;
        q.k = k;
        q.slabs = (n + 15u) / 16u;
        q.ktiles = k / kSkTileK;
        q.tpw = (q.ktiles + kWaves - 1u) / kWaves;
        q.out_f32 = out_f32 ? 1u : 0u;
        q.scale_bits = scale_bits;
        q.offset_bits = offset_bits;
        const uint32_t x_bytes = kWaves * m * (q.tpw * kSkTileK * 2u + kSkRowPad);
        const bool ring = x_bytes <= kSkRingXBytes;
        if (x_bytes <= kSkXBytes) {
            const uint32_t cus = device_compute_units();
            uint32_t grid = q.slabs < cus ? q.slabs : cus;
            if ((q.slabs + grid - 1u) / grid > kSkMaxSlabs) {
                grid = (q.slabs + kSkMaxSlabs - 1u) / kSkMaxSlabs;
            }
            auto go = [&](auto off, auto sum, auto rg) {
                w8a16_nk_stream_kernel<decltype(off)::value, decltype(sum)::value, decltype(rg)::value>
                    <<<grid, kWaves * 64u, 0, st>>>(q);
            };
            auto pick_ring = [&](auto off, auto sum) {
                ring ? go(off, sum, std::true_type{}) : go(off, sum, std::false_type{});
            };
            if (channel_sum) {
                has_offset ? pick_ring(std::true_type{}, std::true_type{}) : pick_ring(std::false_type{}, std::true_type{});
            } else {
                has_offset ? pick_ring(std::true_type{}, std::false_type{}) : pick_ring(std::false_type{}, std::false_type{});
            }
            return launch_status("ascq_matmul_w8a16");
        }
    }
    NkParams p{};
    p.w = static_cast<const uint8_t*>(w);
    p.scale = static_cast<const uint16_t*>(scale);
    p.offset = static_cast<const uint16_t*>(offset);
    p.n = n;
    p.k = k;
    p.out_f32 = out_f32 ? 1u : 0u;
    p.scale_bits = scale_bits;
    p.offset_bits = offset_bits;
    const int cus = static_cast<int>(device_compute_units());
    const uint32_t n_groups = (n + 15u) / 16u;
    // one workgroup per compute unit: two, three or seven times as many smaller ones measured slower at every m
    // (49.7 against 52.7-57.8 us at m = 1, k = 8192, n = 28672)
    uint32_t per = (n_groups + static_cast<uint32_t>(cus) - 1u) / static_cast<uint32_t>(cus);
    per = per > kMaxGroups ? kMaxGroups : per;
    p.groups = per;
    const uint32_t grid = (n_groups + per - 1u) / per;
    if (m > kDecodeRows && k % kGK == 0) {
        // more rows than a few passes of the decode kernel: the tile GEMM reads the weights once per 128 rows
        p.m = m;
        p.x = static_cast<const uint16_t*>(x);
        p.y = y;
        const uint32_t tiles_m = (m + kGM - 1u) / kGM, tiles_n = (n + kGN - 1u) / kGN;
        if (has_offset) {
            w8a16_nk_gemm_kernel<true><<<(tiles_m * tiles_n + 7u) / 8u * 8u, 256, 0, st>>>(p, tiles_m);
        } else {
            w8a16_nk_gemm_kernel<false><<<(tiles_m * tiles_n + 7u) / 8u * 8u, 256, 0, st>>>(p, tiles_m);
        }
        return launch_status("ascq_matmul_w8a16");
    }
    for (uint32_t m0 = 0; m0 < m; m0 += kRows) {
        p.m = m - m0 < kRows ? m - m0 : kRows;
        p.x = static_cast<const uint16_t*>(x) + static_cast<size_t>(m0) * k;
        p.y = out_f32 ? static_cast<void*>(static_cast<float*>(y) + static_cast<size_t>(m0) * n)
                      : static_cast<void*>(static_cast<uint16_t*>(y) + static_cast<size_t>(m0) * n);
        if (has_offset) {
            launch_nk<true>(p, grid, st);
        } else {
            launch_nk<false>(p, grid, st);
        }
    }
    return launch_status("ascq_matmul_w8a16");
}

}  // namespace ascq
