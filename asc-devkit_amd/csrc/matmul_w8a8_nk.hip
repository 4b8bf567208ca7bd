// int8 matmul for few activation rows with B given as [n, k] (the reference's isTransposeB; the layout in which a
// linear layer's weights are usually kept): c[m, n] = epilogue(a[m, k] * b[n, k]^T).
//
// A column of the product owns one contiguous run of k bytes, so whole columns belong to one workgroup and nothing is
// added across workgroups: one launch, no workspace, and integer sums whose order does not matter anyway.
//   * a workgroup of 8 wavefronts owns up to 8 groups of 16 columns; its wavefronts split k into runs of 128;
//   * per run a lane fetches 2 x 16 bytes of one column (lane l: column l % 16, bytes 16 (l / 16) .. + 15 of each
//     64-byte piece): each fetch is the B operand of one v_mfma_i32_16x16x64_i8 as it lies, and the A operand is the
//     same 16 bytes of the lane's row of a, straight from global memory (a is small and read once per wavefront and
//     run for all column groups) - no vector ALU work and no LDS in the loop;
//   * up to 32 rows per pass: two row tiles share every weight fetch;
//   * the 8 partial sums of a column group are added in LDS and go through the element-wise epilogue.
// Requires k % 128 == 0 and a, b 16-byte aligned.
#include "matmul_w8a8.h"

namespace ascq {
namespace {

constexpr uint32_t kNkWaves = 8, kNkMaxGroups = 8, kNkRun = 128;

// G: column groups per workgroup (the last workgroup may own fewer and repeats its last group; the duplicates are not
// stored).  RT: row tiles of 16.
template <int G, int RT>
__global__ __launch_bounds__(kNkWaves * 64) void gemm_nk_kernel(GemmParams p, uint32_t m0)
{
    __shared__ int32_t RED[kNkWaves][RT][G][4][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lc = lane & 15u, lq = lane >> 4;
    const uint32_t n_groups = (p.n + 15u) / 16u;
    const uint32_t g0 = blockIdx.x * G;
    if (g0 >= n_groups) {
        return;
    }
    const uint32_t my_groups = n_groups - g0 < G ? n_groups - g0 : G;
    const uint32_t rows = p.m - m0 < 16u * RT ? p.m - m0 : 16u * RT;  // rows of this pass

    const int8_t* bcol[G];
#pragma unroll
    for (uint32_t g = 0; g < G; ++g) {
        uint32_t col = (g0 + (g < my_groups ? g : my_groups - 1u)) * 16u + lc;
        col = col < p.n ? col : p.n - 1u;
        bcol[g] = p.b + static_cast<size_t>(col) * p.k + 16u * lq;
    }
    // the lane's rows of a (rows past the end read the pass's first row and are masked to zero)
    const int8_t* arow[RT];
    bool row_ok[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        row_ok[t] = 16u * t + lc < rows;
        arow[t] = p.a + static_cast<size_t>(m0 + (row_ok[t] ? 16u * t + lc : 0u)) * p.k + 16u * lq;
    }

    i32x4 acc[RT][G];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) acc[t][g] = i32x4{0, 0, 0, 0};
    }

    // all loads of a run are issued together, unconditionally, one run ahead of the MFMAs that use them
    auto load_run = [&](uint32_t r, i32x4 (&bv)[G][2], i32x4 (&av)[RT][2]) __attribute__((always_inline)) {
        const uint32_t k0 = r * kNkRun;
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                bv[g][h] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(bcol[g] + k0 + 64u * h));
            }
        }
#pragma unroll
        for (int t = 0; t < RT; ++t) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                av[t][h] = *reinterpret_cast<const i32x4*>(arow[t] + k0 + 64u * h);
            }
        }
    };
    auto compute_run = [&](const i32x4 (&bv)[G][2], const i32x4 (&araw)[RT][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            i32x4 av[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) av[h] = row_ok[t] ? araw[t][h] : i32x4{0, 0, 0, 0};
#pragma unroll
            for (uint32_t g = 0; g < G; ++g) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    acc[t][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[h], bv[g][h], acc[t][g], 0, 0, 0);
                }
            }
        }
    };

    const uint32_t runs = p.k / kNkRun;
    const uint32_t r_begin = runs * wave / kNkWaves, r_end = runs * (wave + 1u) / kNkWaves;
    if (r_begin < r_end) {
        i32x4 b0[G][2], b1[G][2], a0[RT][2], a1[RT][2];
        const uint32_t last = r_end - 1u;
        load_run(r_begin, b0, a0);
        for (uint32_t r = r_begin; r < r_end; r += 2) {
            load_run(r + 1u < last ? r + 1u : last, b1, a1);
            compute_run(b0, a0);
            load_run(r + 2u < last ? r + 2u : last, b0, a0);
            if (r + 1u < r_end) {
                compute_run(b1, a1);
            }
        }
    }

    // ---- register i of lane l is row 4 (l / 16) + i, column l % 16 of the tile
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) {
#pragma unroll
            for (int i = 0; i < 4; ++i) RED[wave][t][g][i][lane] = acc[t][g][i];
        }
    }
    __syncthreads();
    const EpiParams& e = p.epi;
    for (uint32_t job = wave; job < RT * my_groups; job += kNkWaves) {
        const uint32_t t = job / my_groups, g = job - t * my_groups;
        const uint32_t col = (g0 + g) * 16u + lc;
        if (col >= p.n) {
            continue;
        }
        const ChannelQ q = load_channel_q(e, col);
        const float bp = load_bias_post(e, col);
        const int32_t bias_pre = e.bias_kind == ASCQ_MM_BIAS_I32_PRE ? static_cast<const int32_t*>(e.bias)[col] : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t row_in_pass = 16u * t + 4u * lq + static_cast<uint32_t>(i);
            if (row_in_pass >= rows) {
                continue;
            }
            int32_t s = RED[0][t][g][i][lane];
#pragma unroll
            for (uint32_t wv = 1; wv < kNkWaves; ++wv) s += RED[wv][t][g][i][lane];
            s += bias_pre;
            const uint32_t row = m0 + row_in_pass;
            const float tok = e.has_tok ? e.tok_scale[row] : 1.0f;
            dispatch_out(e, [&](auto tag) { epilogue_store<decltype(tag)::value>(e, row, col, s, q, tok, bp); });
        }
    }
}

template <int RT>
void launch_nk_rt(const GemmParams& p, uint32_t m0, uint32_t groups, uint32_t grid, hipStream_t st)
{
    switch (groups) {
        case 1: gemm_nk_kernel<1, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 2: gemm_nk_kernel<2, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 3: gemm_nk_kernel<3, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 4: gemm_nk_kernel<4, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 5: gemm_nk_kernel<5, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 6: gemm_nk_kernel<6, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        case 7: gemm_nk_kernel<7, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
        default: gemm_nk_kernel<8, RT><<<grid, kNkWaves * 64, 0, st>>>(p, m0); break;
    }
}

}  // namespace

bool gemm_nk_supported(const GemmParams& p)
{
    return p.k % kNkRun == 0 && aligned16(p.a) && aligned16(p.b);
}

// Any m; 32 rows per pass over the weights (16 in a last pass of at most 16 rows).
int launch_gemm_nk(const GemmParams& p, hipStream_t st)
{
    const int cus = static_cast<int>(device_compute_units());
    const uint32_t n_groups = (p.n + 15u) / 16u;
    // Column groups per workgroup: one workgroup per compute unit when several rows share the weights (every
    // workgroup reads all of a once); with at most 4 rows a is negligible and three times as many, smaller workgroups
    // start and drain faster (13.9 against 15.5 us at m = 1, k = 4096, n = 11008; 19.2 against 17.8 us at m = 16).
    const uint32_t slots = static_cast<uint32_t>(cus) * (p.m <= 4u ? 3u : 1u);
    uint32_t per = (n_groups + slots - 1u) / slots;
    const bool two = p.m > 16u;
    per = per > kNkMaxGroups ? kNkMaxGroups : per;

    const uint32_t grid = (n_groups + per - 1u) / per;
    if (plan_note(ASCQ_MM_KERNEL_STREAM, two ? 32 : 16, 16 * per, kNkRun, grid, 1, kNkWaves * (two ? 2 : 1) * per * 1024u, 0)) {
        return ASCQ_OK;
    }
    for (uint32_t m0 = 0; m0 < p.m;) {
        if (p.m - m0 > 16u) {
            launch_nk_rt<2>(p, m0, per, grid, st);
            m0 += 32u;
        } else {
            launch_nk_rt<1>(p, m0, per, grid, st);
            m0 += 16u;
        }
    }
    return launch_status("ascq_matmul_w8a8");
}

}  // namespace ascq
