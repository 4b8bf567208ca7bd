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
#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

constexpr uint32_t kWaves = 8, kMaxGroups = 8, kRows = 16, kRun = 128;

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

}  // namespace

bool w8a16_nk_supported(uint32_t k, const void* x, const void* w)
{
    return k % kRun == 0 && aligned16(x) && aligned16(w);
}

// x, y: first row of the whole problem; m rows in passes of 16.
int launch_w8a16_nk(const void* x, const void* w, const void* scale, const void* offset, void* y, uint32_t m, uint32_t n,
                    uint32_t k, bool has_offset, bool out_f32, uint32_t scale_bits, uint32_t offset_bits, hipStream_t st)
{
    NkParams p{};
    p.w = static_cast<const uint8_t*>(w);
    p.scale = static_cast<const uint16_t*>(scale);
    p.offset = static_cast<const uint16_t*>(offset);
    p.n = n;
    p.k = k;
    p.out_f32 = out_f32 ? 1u : 0u;
    p.scale_bits = scale_bits;
    p.offset_bits = offset_bits;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        cus = 256;
    }
    const uint32_t n_groups = (n + 15u) / 16u;
    // one workgroup per compute unit: two, three or seven times as many smaller ones measured slower at every m
    // (49.7 against 52.7-57.8 us at m = 1, k = 8192, n = 28672)
    uint32_t per = (n_groups + static_cast<uint32_t>(cus) - 1u) / static_cast<uint32_t>(cus);
    per = per > kMaxGroups ? kMaxGroups : per;
    p.groups = per;
    const uint32_t grid = (n_groups + per - 1u) / per;
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
