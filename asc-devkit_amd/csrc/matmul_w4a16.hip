// W4A16 weight-only linear for decode: y[m, n] = sum_k x[m, k] * antiquant(w[k, n]) with int4 weights de-quantised in
// registers (never materialised in memory).
//
// The kernel is bound by the HBM read of the packed weights (k * n / 2 bytes).  Layout of the work:
//   * a lane owns 16 bytes = 32 adjacent columns of a weight row; the 16 lanes of a quarter-wavefront cover 512
//     columns (256 contiguous bytes) and the four quarters take four different k rows, so one load instruction of a
//     wavefront reads 4 rows x 256 bytes; 8 such loads are in flight per lane;
//   * the four wavefronts of a workgroup take different k ranges of the same 512 columns, K is further split over
//     gridDim.y, so that about 450 workgroups stream the weights;
//   * de-quantisation follows AscendAntiQuant<int4b_t, half> exactly: the nibble becomes an exact half via the
//     0x6400 exponent trick (1024 + u) - 1032, then one rounded half add of the offset and one rounded half
//     multiply by the scale (packed v_pk_add_f16 / v_pk_mul_f16 on two columns at a time);
//   * the multiply-accumulate runs on the matrix core instead of the VALU: the 8 de-quantised halves of one dword
//     are the B operand of v_mfma_f32_16x16x32_f16 as they are (k slot (g, b) = row of quarter g, column b of the
//     dword); the A operand of output row i carries x[k_g] in slot i and zeros elsewhere, so row i of the result is
//     the running dot product of column i of the dword.  Rows 0-7 serve one activation row, rows 8-15 a second one;
//     more activation rows take more MFMAs on the same de-quantised operand.  Accumulation is fp32;
//   * partial sums are reduced across the wavefronts through LDS and written as fp32; a second small kernel adds
//     the K-splits in a fixed order and rounds once to half, so results are deterministic.
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

// slot b of the de-quantised operand holds column (b >> 1) + 4 * (b & 1) of the dword
__device__ __forceinline__ uint32_t slot_to_col(uint32_t b) { return (b >> 1) + 4u * (b & 1u); }

// MP = number of activation-row pairs handled per pass over the weights (m <= 2 * MP).
// Requires n % 32 == 0, group_size % 32 == 0, k_per_split % 128 == 0.
template <int MP, bool kHasOffset>
__global__ __launch_bounds__(kThreads) void w4a16_mfma_kernel(W4Params p)
{
    __shared__ float red[4][2][kColsPerBlock];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t g = lane >> 4, jj = lane & 15u;
    // Lanes past the last column work on a duplicate of the last 32 columns (their results are never stored): the
    // MFMA ignores the execution mask, so every lane must hold a valid A operand.
    uint32_t col0 = blockIdx.x * kColsPerBlock + jj * 32u;
    col0 = col0 < p.n ? col0 : p.n - 32u;
    const uint32_t rows_per_wave = p.k_per_split / 4u;
    const uint32_t kw0 = blockIdx.y * p.k_per_split + wave * rows_per_wave;
    const size_t row_bytes = p.n / 2;

    f32x4 acc[MP][4];
#pragma unroll
    for (int q = 0; q < MP; ++q) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[q][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    // A operand: lane (g, i) carries x[m][k_g] in half-slot (i & 7) for m = 2 * pair + (i >> 3)
    const uint32_t slot = jj & 7u;
    uint32_t amask[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        amask[r] = (static_cast<uint32_t>(r) == (slot >> 1)) ? ((slot & 1u) ? 0xFFFF0000u : 0x0000FFFFu) : 0u;
    }
    const f16x2 k1032 = {static_cast<half_t>(1032.0f), static_cast<half_t>(1032.0f)};

    // Software pipeline over chunks of 32 rows: the 8 weight loads (and the activations) of chunk c + 1 are issued
    // before chunk c is de-quantised, so a lane always has 8-16 loads of 16 bytes in flight.
    const uint8_t* wbase = p.w + static_cast<size_t>(kw0 + 8u * g) * row_bytes + col0 / 2;
    const uint32_t chunks = rows_per_wave / 32u;
    u32x4 wv[2][8];
    u32x4 xv[2][MP];
    f16x2 sc[4][4], of[4][4];
    uint32_t cur_group = 0xFFFFFFFFu;
    auto load_chunk = [&](uint32_t c, u32x4 (&wd)[8], u32x4 (&xd)[MP]) {
        const uint8_t* src = wbase + static_cast<size_t>(c) * 32u * row_bytes;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            wd[u] = *reinterpret_cast<const u32x4*>(src + static_cast<size_t>(u) * row_bytes);
        }
#pragma unroll
        for (int q = 0; q < MP; ++q) {
            const uint32_t m = p.m0 + 2u * q + (jj >> 3);
            xd[q] = u32x4{0u, 0u, 0u, 0u};
            if (m < p.m) {
                xd[q] = *reinterpret_cast<const u32x4*>(p.x + static_cast<size_t>(m) * p.k + kw0 + c * 32u + 8u * g);
            }
        }
    };
    auto compute_chunk = [&](uint32_t c, const u32x4 (&wd)[8], const u32x4 (&xd)[MP]) {
        const uint32_t grp = (kw0 + c * 32u) / p.group_size;  // the 32 rows of a chunk share a group
        if (grp != cur_group) {
            cur_group = grp;
            const size_t prow = static_cast<size_t>(grp) * p.n + col0;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                pair_up(*reinterpret_cast<const u32x4*>(p.scale + prow + 8 * d), sc[d]);
                if constexpr (kHasOffset) {
                    pair_up(*reinterpret_cast<const u32x4*>(p.offset + prow + 8 * d), of[d]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            f16x8 a[MP];
#pragma unroll
            for (int q = 0; q < MP; ++q) {
                const uint32_t xw = xd[q][u >> 1];
                const uint32_t xx = (u & 1) ? __builtin_amdgcn_perm(xw, xw, 0x03020302u)
                                            : __builtin_amdgcn_perm(xw, xw, 0x01000100u);
                u32x4 av = u32x4{xx & amask[0], xx & amask[1], xx & amask[2], xx & amask[3]};
                __builtin_memcpy(&a[q], &av, 16);
            }
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t qd = wd[u][d] ^ 0x88888888u;  // two's complement nibble -> offset binary u = w + 8
                f16x2 h[4];
#pragma unroll
                for (int c2 = 0; c2 < 4; ++c2) {
                    uint32_t bits;  // (nibble c2, nibble c2 + 4) -> two halves 1024 + u, exact
                    asm("v_and_or_b32 %0, %1, %2, %3"
                        : "=v"(bits)
                        : "v"(qd >> (4 * c2)), "s"(0x000F000Fu), "v"(0x64006400u));
                    h[c2] = bits_to_h2(bits) - k1032;  // w, exact
                    if constexpr (kHasOffset) {
                        h[c2] = h[c2] + of[d][c2];  // one rounding
                    }
                    h[c2] = sc[d][c2] * h[c2];      // one rounding
                }
                f16x8 b;
                __builtin_memcpy(&b, h, 16);
#pragma unroll
                for (int q = 0; q < MP; ++q) {
                    acc[q][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[q], b, acc[q][d], 0, 0, 0);
                }
            }
        }
    };
    load_chunk(0, wv[0], xv[0]);
    for (uint32_t c = 0; c < chunks; c += 2) {
        if (c + 1 < chunks) {
            load_chunk(c + 1, wv[1], xv[1]);
        }
        compute_chunk(c, wv[0], xv[0]);
        if (c + 1 < chunks) {
            if (c + 2 < chunks) {
                load_chunk(c + 2, wv[0], xv[0]);
            }
            compute_chunk(c + 1, wv[1], xv[1]);
        }
    }

    // result tile d of pair q: register r of lane (g, jj) is row 4 g + r -> activation row 2 q + (g >> 1),
    // slot 4 (g & 1) + r -> column jj * 32 + d * 8 + slot_to_col(slot)
#pragma unroll
    for (int q = 0; q < MP; ++q) {
        __syncthreads();
#pragma unroll
        for (int d = 0; d < 4; ++d) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                red[wave][g >> 1][jj * 32 + d * 8 + slot_to_col(4u * (g & 1u) + r)] = acc[q][d][r];
            }
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t idx = tid + e * kThreads;  // 0..1023: (row of the pair, column)
            const uint32_t mr = idx >> 9, c = idx & 511u;
            const uint32_t m = p.m0 + 2u * q + mr;
            const uint32_t col = blockIdx.x * kColsPerBlock + c;
            if (m < p.m && col < p.n) {
                const float s = ((red[0][mr][c] + red[1][mr][c]) + red[2][mr][c]) + red[3][mr][c];
                p.partial[(static_cast<size_t>(blockIdx.y) * p.m + m) * p.n + col] = s;
            }
        }
    }
}

// Adds the K-splits in a fixed order (deterministic) and rounds once to half.  Launched after the partial kernel: the
// kernel boundary makes the partial sums visible, which is far cheaper here than device-scope fences in 900 workgroups.
__global__ __launch_bounds__(kThreads) void w4a16_reduce_kernel(W4Params p)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    const size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= total) {
        return;
    }
    float s = 0.0f;
    uint32_t sp = 0;
    for (; sp + 8 <= p.splits; sp += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p.partial[static_cast<size_t>(sp + u) * total + idx];  // 8 loads in flight
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; sp < p.splits; ++sp) {
        s += p.partial[static_cast<size_t>(sp) * total + idx];
    }
    p.y[idx] = static_cast<uint16_t>(f32_to_half_bits(s));
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
    // K range per workgroup: a multiple of 128 rows (32 per wavefront) and of the group size; aim at ~450 workgroups (measured best on 256 CUs)
    (void)group_size;
    const uint32_t blocks_n = (n + kColsPerBlock - 1) / kColsPerBlock;
    const uint32_t units = k / kRowsPerPass;
    const uint32_t target = 448u;  // workgroups per launch that measured fastest on 256 compute units
    uint32_t want = (target + blocks_n - 1) / blocks_n;
    uint32_t splits = units < want ? units : want;
    if (splits == 0) splits = 1;
    while (units % splits != 0) --splits;
    return splits;
}

bool fast_ok(const ascq_w4a16_desc* d, const void* x, const void* w, const void* scale, const void* offset)
{
    return d->n % 32 == 0 && d->k % kRowsPerPass == 0 && d->group_size % 32 == 0 && aligned16(x) && aligned16(w) &&
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
    for (uint32_t m0 = 0; m0 < d->m; m0 += 16) {
        const uint32_t left = d->m - m0;
        p.m0 = m0;
#define ASCQ_W4_LAUNCH(MPV)                                                  \
    do {                                                                     \
        if (d->has_offset) {                                                 \
            w4a16_mfma_kernel<MPV, true><<<grid, kThreads, 0, st>>>(p);      \
        } else {                                                             \
            w4a16_mfma_kernel<MPV, false><<<grid, kThreads, 0, st>>>(p);     \
        }                                                                    \
    } while (0)
        if (left <= 2) {
            ASCQ_W4_LAUNCH(1);
        } else if (left <= 4) {
            ASCQ_W4_LAUNCH(2);
        } else if (left <= 8) {
            ASCQ_W4_LAUNCH(4);
        } else {
            ASCQ_W4_LAUNCH(8);
        }
#undef ASCQ_W4_LAUNCH
    }
    rc = launch_status("ascq_matmul_w4a16");
    if (rc != ASCQ_OK) {
        return rc;
    }
    const size_t blocks = (total + kThreads - 1) / kThreads;
    w4a16_reduce_kernel<<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(p);
    return launch_status("ascq_matmul_w4a16 (reduce)");
}
