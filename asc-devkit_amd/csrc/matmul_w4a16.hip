// W4A16 weight-only linear for decode: y[m, n] = sum_k x[m, k] * antiquant(w[k, n]) with int4 weights de-quantised in
// registers (never materialised in memory).
//
// The kernel is bound by the HBM read of the packed weights (k * n / 2 bytes).  Layout of the work:
//   * a lane owns 16 bytes = 32 adjacent columns of a weight row; 16 lanes cover 512 columns (256 contiguous bytes);
//   * the 16 lane groups of a workgroup take 8 consecutive k rows each, so a workgroup consumes 128 rows x 512
//     columns per pass with 8 independent 16-byte loads in flight per lane;
//   * K is split over gridDim.y so that (n / 512) * splits workgroups cover the chip several times;
//   * de-quantisation follows AscendAntiQuant<int4b_t, half> exactly: the nibble becomes an exact half via the
//     0x6400 exponent trick (1024 + u) - 1032, then one rounded half add of the offset and one rounded half
//     multiply by the scale (packed v_pk_add_f16 / v_pk_mul_f16 on two columns at a time);
//   * products are accumulated in fp32, reduced across the 16 lane groups through LDS and written as fp32 partial
//     sums; a second small kernel adds the K-splits in a fixed order and rounds once to half, so results are
//     deterministic.
#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

constexpr int kThreads = 256;
constexpr int kColsPerBlock = 512;
constexpr int kRowsPerPass = 128;

struct W4Params {
    const uint16_t* x;
    const uint8_t* w;
    const uint16_t* scale;
    const uint16_t* offset;
    float* partial;  // [splits, m, n]
    uint16_t* y;
    uint32_t m, n, k, group_size, has_offset;
    uint32_t splits, k_per_split;
    uint32_t m0;  // first activation row handled by this launch
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

template <int MT>
__global__ __launch_bounds__(kThreads) void w4a16_partial_kernel(W4Params p)
{
    __shared__ float red[16][kColsPerBlock];
    const uint32_t tid = threadIdx.x;
    const uint32_t ln = tid & 15u;   // 32-column slot inside the 512-column block
    const uint32_t rg = tid >> 4;    // row group: 8 consecutive k rows per pass
    const uint32_t col0 = blockIdx.x * kColsPerBlock + ln * 32u;
    const bool active = col0 < p.n;  // n % 32 == 0
    const uint32_t k_begin = blockIdx.y * p.k_per_split;
    const uint32_t k_end = min(p.k, k_begin + p.k_per_split);
    const size_t row_bytes = p.n / 2;

    float acc[MT][32];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int c = 0; c < 32; ++c) acc[m][c] = 0.0f;
    }
    const f16x2 k1032 = {static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};

    if (active) {
        for (uint32_t kp = k_begin; kp < k_end; kp += kRowsPerPass) {
            const uint32_t k0 = kp + rg * 8u;  // k % 128 == 0 and group_size % 8 == 0: the 8 rows share a group
            u32x4 wv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                wv[i] = *reinterpret_cast<const u32x4*>(p.w + static_cast<size_t>(k0 + i) * row_bytes + col0 / 2);
            }
            const size_t prow = static_cast<size_t>(k0 / p.group_size) * p.n + col0;
            f16x2 sc[4][4], of[4][4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                pair_up(*reinterpret_cast<const u32x4*>(p.scale + prow + 8 * d), sc[d]);
                if (p.has_offset) {
                    pair_up(*reinterpret_cast<const u32x4*>(p.offset + prow + 8 * d), of[d]);
                }
            }
            float xv[MT][8];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                load8<ASCQ_F16>(p.x, static_cast<size_t>(p.m0 + m) * p.k + k0, xv[m]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t q = wv[i][d] ^ 0x88888888u;  // two's complement nibble -> offset binary u = w + 8
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        f16x2 h = bits_to_h2(((q >> (4 * c)) & 0x000F000Fu) | 0x64006400u);  // 1024 + u, exact
                        h = h - k1032;                                                      // w, exact
                        if (p.has_offset) {
                            h = h + of[d][c];  // one rounding
                        }
                        h = sc[d][c] * h;      // one rounding
                        const float w0 = static_cast<float>(h[0]);
                        const float w1 = static_cast<float>(h[1]);
#pragma unroll
                        for (int m = 0; m < MT; ++m) {
                            acc[m][8 * d + c] += xv[m][i] * w0;
                            acc[m][8 * d + c + 4] += xv[m][i] * w1;
                        }
                    }
                }
            }
        }
    }

    // reduce the 16 row groups through LDS, one activation row at a time
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 32; c += 4) {
            *reinterpret_cast<f32x4*>(&red[rg][ln * 32 + c]) =
                f32x4{acc[m][c], acc[m][c + 1], acc[m][c + 2], acc[m][c + 3]};
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t c = tid + h * kThreads;
            const uint32_t col = blockIdx.x * kColsPerBlock + c;
            if (col < p.n) {
                float s = 0.0f;
#pragma unroll
                for (int g = 0; g < 16; ++g) s += red[g][c];
                p.partial[(static_cast<size_t>(blockIdx.y) * p.m + p.m0 + m) * p.n + col] = s;
            }
        }
    }
}

__global__ __launch_bounds__(kThreads) void w4a16_reduce_kernel(W4Params p)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * kThreads) {
        float s = 0.0f;
        for (uint32_t sp = 0; sp < p.splits; ++sp) {
            s += p.partial[static_cast<size_t>(sp) * total + idx];
        }
        p.y[idx] = static_cast<uint16_t>(f32_to_half_bits(s));
    }
}

// Any shape: one lane per output element.
__global__ __launch_bounds__(kThreads) void w4a16_generic_kernel(W4Params p)
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

uint32_t pick_splits(uint32_t n, uint32_t k, uint32_t group_size)
{
    // K range per workgroup: a multiple of 128 rows and of the group size; aim at >= 1536 workgroups
    const uint32_t blocks_n = (n + kColsPerBlock - 1) / kColsPerBlock;
    uint32_t unit = kRowsPerPass;
    while (unit % group_size != 0 && unit < k) unit += kRowsPerPass;
    uint32_t units = k / unit;
    uint32_t want = (1536u + blocks_n - 1) / blocks_n;
    uint32_t splits = units < want ? units : want;
    if (splits == 0) splits = 1;
    while (units % splits != 0) --splits;
    return splits;
}

bool fast_ok(const ascq_w4a16_desc* d, const void* x, const void* w, const void* scale, const void* offset)
{
    return d->n % 32 == 0 && d->k % kRowsPerPass == 0 && d->group_size % 8 == 0 &&
           (kRowsPerPass % d->group_size == 0 || d->group_size % kRowsPerPass == 0) && aligned16(x) && aligned16(w) &&
           aligned16(scale) && (!d->has_offset || aligned16(offset));
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
    const uint32_t splits = pick_splits(d->n, d->k, d->group_size);
    *bytes = static_cast<size_t>(splits) * d->m * d->n * sizeof(float);
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
    W4Params p{static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(scale),
               static_cast<const uint16_t*>(offset), static_cast<float*>(workspace), static_cast<uint16_t*>(y),
               d->m, d->n, d->k, d->group_size, static_cast<uint32_t>(d->has_offset ? 1 : 0), 1, d->k, 0};
    const size_t total = static_cast<size_t>(d->m) * d->n;
    if (!fast_ok(d, x, w, scale, offset)) {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        w4a16_generic_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
        return launch_status("ascq_matmul_w4a16 (generic)");
    }
    p.splits = pick_splits(d->n, d->k, d->group_size);
    p.k_per_split = d->k / p.splits;
    const size_t need = static_cast<size_t>(p.splits) * total * sizeof(float);
    ASCQ_REQUIRE(workspace != nullptr && workspace_bytes >= need, ASCQ_EINVAL,
                 "ascq_matmul_w4a16: workspace of %zu bytes required (see ascq_matmul_w4a16_workspace_size)", need);
    ASCQ_REQUIRE(aligned16(workspace), ASCQ_EALIGN, "ascq_matmul_w4a16: workspace must be 16-byte aligned");
    dim3 grid((d->n + kColsPerBlock - 1) / kColsPerBlock, p.splits);
    for (uint32_t m0 = 0; m0 < d->m;) {
        const uint32_t left = d->m - m0;
        p.m0 = m0;
        if (left >= 4) {
            w4a16_partial_kernel<4><<<grid, kThreads, 0, st>>>(p);
            m0 += 4;
        } else if (left >= 2) {
            w4a16_partial_kernel<2><<<grid, kThreads, 0, st>>>(p);
            m0 += 2;
        } else {
            w4a16_partial_kernel<1><<<grid, kThreads, 0, st>>>(p);
            m0 += 1;
        }
    }
    rc = launch_status("ascq_matmul_w4a16");
    if (rc != ASCQ_OK) {
        return rc;
    }
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 2048) blocks = 2048;
    w4a16_reduce_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
    return launch_status("ascq_matmul_w4a16 (reduce)");
}
