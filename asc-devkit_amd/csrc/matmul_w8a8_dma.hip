// Large-M int8 matmul for gfx950 built on the two CDNA4 data-movement instructions that remove all register staging:
//
//   * global_load_lds_dwordx4: every lane names a 16-byte global source, the data lands in LDS at
//     (uniform base + lane * 16) without passing through registers and is tracked by vmcnt.  Because the global
//     address is free per lane, the bank-conflict swizzles are applied on the *source* side: the lane that owns LDS
//     slot s fetches the 16 bytes that belong in that slot.
//   * ds_read_b64_tr_b8: a transposing LDS read.  Within 16 lanes, lane l receives byte (l & 7) of the eight 8-byte
//     rows addressed by lanes 2b + (l >> 3), b = 0..7.  Pointing even lanes at columns [c, c+8) and odd lanes at
//     [c+8, c+16) of eight consecutive k rows gives every lane the 8 consecutive k values of column c + l: exactly
//     the MFMA B operand, read from a B tile that is stored in LDS as it is in memory ([k][n], n contiguous).
//
// So the main loop is: DMA loads for the next K step, LDS reads, MFMAs - no VALU work, no LDS writes, no staging
// registers.  A workgroup is 512 lanes (8 wavefronts, two per SIMD, so that one wavefront's LDS / address
// instructions issue under the other's MFMAs) and owns a 256 x 256 tile; a wavefront owns 128 x 64 (4 x 2 MFMA
// blocks of 32x32x32, 128 accumulator registers).  Two LDS stages of 64 KiB (A 256 x 128 B, B 128 x 256 B) are
// separate arrays so that the compiler can tell that LDS reads of one stage do not depend on DMA writes to the
// other.
//
// LDS layouts (all reads and writes conflict-free, measured at ~220-250 B/clk/CU):
//   A stage: row r = 128 bytes = 8 pieces of 16; piece c is stored at position c ^ ((r >> 1) & 7).
//   B stage: row k = 256 bytes = 16 pieces of 16; piece q is stored at position q ^ (2 * (k & 7)).
#include <type_traits>
#include <utility>

#include "matmul_w8a8.h"

namespace ascq {
namespace {

constexpr int kThreads = 512;
constexpr int BK = 128;

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef i32x2_t __attribute__((address_space(3)))* lds_v2_t;

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression.
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// 16-bit output of two adjacent columns packed into one dword store.
template <int kOut>
__device__ __forceinline__ uint32_t to_bits16(float v)
{
    if constexpr (kOut == ASCQ_BF16) {
        return f32_to_bf16_bits(v);
    } else {
        return f32_to_half_bits_sat(v);
    }
}

template <bool kBiasPost, bool kGelu>
__device__ __forceinline__ float epi_value(int32_t acc, float chan, float tok, float bias_post)
{
    float v = static_cast<float>(acc) * chan;
    v = v * tok;  // tok is 1.0f without a token scale: an exact identity
    if constexpr (kBiasPost) {
        v = v + bias_post;
    }
    if constexpr (kGelu) {
        v = faster_gelu(v);
    }
    return v;
}

// 256 x 256: wavefronts 2 (M) x 4 (N), 128 x 64 each.  256 x 128: wavefronts 4 (M) x 2 (N), 64 x 64 each (used for the
// last, partially filled round of tiles: half-width tiles finish it in half the time).  128 x 128: 32 x 64 per
// wavefront, 64 KiB of LDS so that two workgroups share a CU; with kSplitK the K range is divided over blockIdx.y and
// the int32 partial tiles go to a workspace [split][m][n] that a second kernel sums (small M: the weights are read
// once, by enough workgroups to fill the chip).
// The body of a workgroup: tile number `bid` (before the XCD remapping) of the launch, K split `bidy`.  The LDS arrays
// are declared by the kernels and handed in, so that one kernel can run tiles of two shapes.
// kBT: B is given as [n][k] (transposed operand): its tile is staged and read exactly like A's, with plain 16-byte
// LDS reads instead of the transposing ones.
// Where a tile lies: rows [row0, row_end) of A and C (row_end clips the tile), columns from n0, the weight matrix it
// multiplies with and the offset of that matrix's per-channel parameters (grouped: those of the tile's group).
struct TilePlace {
    uint32_t row0, row_end, n0;
    const int8_t* b;
    size_t chan_off;
};

// kB: how B lies in memory.  0: [k, n] (or the fractal panels); 1: [n, k]; 2: the layout of ascq_pack_weight_w8
// (slabs of 16 columns, each a run of 1 KiB tiles of 64 k: lane l of a tile owns column l % 16, k 16 (l / 16) .. + 15).
template <int BM, int BN, bool kSplitK, bool kGrouped, int kB = 0>
__device__ __forceinline__ void gemm_dma_tile_at(const GemmParams& p, const TilePlace& at, uint32_t bidy, char* A0,
                                                 char* B0, char* A1, char* B1, float* TS)
{
    constexpr bool kBT = kB == 1, kBP = kB == 2;
    constexpr int kWN = BN / 64;            // wavefronts along N
    constexpr int kWM = 8 / kWN;            // wavefronts along M
    constexpr int TI = BM / 32 / kWM;       // 32x32 blocks per wavefront along M
    constexpr int TJ = 2;                   // and along N
    constexpr int kPieces = BN / 16;        // 16-byte pieces per B row
    constexpr int kAInstr = BM * BK / 1024 / 8;  // A DMA instructions per wavefront and K step
    constexpr int kBInstr = BK * BN / 1024 / 8;  // B DMA instructions per wavefront and K step
    constexpr int kKsB = 32 * BN;           // bytes of B per K sub-step of 32 rows
    static_assert(TI >= 1 && TI * 32 * kWM == BM && kAInstr >= 1, "tile shape does not fit eight wavefronts");

    const uint32_t K = p.k, N = p.n;
    const uint32_t row0 = at.row0, row_end = at.row_end, n0 = at.n0;
    const int8_t* Bmat = at.b;
    const size_t chan_off = at.chan_off;
    uint32_t tid = threadIdx.x;
    if constexpr (kGrouped) {
        // The grouped kernel runs tiles in a loop: without this the compiler computes everything that depends only on
        // the lane once, ahead of the loop, and those registers are missing in the tile's main loop.
        asm volatile("" : "+v"(tid));
    }
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / kWN, wn = wave % kWN;
    if (tid < BM) {
        // read by the epilogue only; the barriers of the main loop order this store before those reads
        const uint32_t row = row0 + tid;
        TS[tid] = (p.epi.has_tok && row < row_end) ? p.epi.tok_scale[row] : 1.0f;
    }

    // ---- DMA sources: 4 A and 4 B instructions per wavefront and K step; lane owns LDS slot (instr * 64 + lane)
    uint32_t aoff[kAInstr], boff[kBInstr];
#pragma unroll
    for (int u = 0; u < kAInstr; ++u) {
        const uint32_t s = (wave * kAInstr + u) * 64 + lane;
        const uint32_t r = s >> 3, c = (s & 7u) ^ ((r >> 1) & 7u);
        uint32_t row = row0 + r;
        row = row < row_end ? row : row_end - 1;  // rows past the end are never stored: any valid row will do
        aoff[u] = (row - row0) * K + 16u * c;
    }
#pragma unroll
    for (int u = 0; u < kBInstr; ++u) {
        const uint32_t s = (wave * kBInstr + u) * 64 + lane;
        if constexpr (kBP) {
            // one instruction = one packed tile: piece (slab j of the tile's BN / 16, k tile h of the step's two)
            // lands in LDS as it lies in memory; slabs past the last one are never stored
            const uint32_t piece = wave * kBInstr + u, j = piece >> 1, h = piece & 1u;
            const uint32_t slab0 = n0 >> 4, last = (N + 15u) / 16u - 1u;
            const uint32_t slab = slab0 + j < last ? slab0 + j : last;
            boff[u] = (slab - slab0) * (K * 16u) + h * 1024u + lane * 16u;
            continue;
        }
        if constexpr (kBT) {
            const uint32_t r = s >> 3, c = (s & 7u) ^ ((r >> 1) & 7u);
            uint32_t col = n0 + r;
            col = col < N ? col : N - 1u;  // columns past the end are never stored
            boff[u] = (col - n0) * K + 16u * c;
            continue;
        }
        const uint32_t kb = s / kPieces;
        const uint32_t swz = BN == 256 ? 2u * (kb & 7u) : 2u * ((kb >> 1) & 3u);
        const uint32_t q = (s % kPieces) ^ swz;
        uint32_t col = n0 + 16u * q;
        col = col + 16u <= N ? col : N - 16u;      // columns past the end are never stored
        // fractal B: panels of 32 columns, each a contiguous row-major [K][32] block
        boff[u] = p.b_nz ? ((col >> 5) * K + kb) * 32u + (col & 31u) : kb * N + (col - n0);
    }
    const uint32_t ldb = kBT ? 1u : kBP ? 16u : p.b_nz ? 32u : N;  // bytes from one k to the next
    // K range of this workgroup, in steps of BK
    uint32_t s_begin = 0, steps = K / BK;
    if constexpr (kSplitK) {
        s_begin = steps * bidy / p.k_splits;
        steps = steps * (bidy + 1u) / p.k_splits - s_begin;
    }
    const int8_t* Abase = p.a + static_cast<size_t>(row0) * K + static_cast<size_t>(s_begin) * BK;
    const int8_t* Bbase = Bmat + (kBT ? static_cast<size_t>(n0) * K : kBP ? static_cast<size_t>(n0 >> 4) * K * 16u : p.b_nz ? 0u : n0) +
                          static_cast<size_t>(s_begin) * BK * ldb;
    // A wavefront-uniform address, pinned to scalar registers: a load's address is then this base plus the lane's
    // 32-bit offset, which the load instruction adds itself (otherwise the compiler widens the offsets to 64 bits
    // ahead of the loop and adds the base per load: twice the registers and an addition per load).
    auto uniform = [](const int8_t* q) __attribute__((always_inline)) {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        asm volatile("" : "+s"(lo), "+s"(hi));
        return reinterpret_cast<const int8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
    };
    auto issue = [&](uint32_t k0, char* As, char* Bs) {
        const int8_t* ab = uniform(Abase + k0);
        const int8_t* bb = uniform(Bbase + static_cast<size_t>(k0) * ldb);
#pragma unroll
        for (int u = 0; u < kAInstr; ++u) asm volatile("" : "+v"(aoff[u]));
#pragma unroll
        for (int u = 0; u < kBInstr; ++u) asm volatile("" : "+v"(boff[u]));
#pragma unroll
        for (int u = 0; u < kAInstr; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(ab + aoff[u]), (lds_ptr_t)(As + (wave * kAInstr + u) * 1024), 16,
                                             0, 0);
        }
#pragma unroll
        for (int u = 0; u < kBInstr; ++u) {
            // split-K (few rows): the weights are read once, or by a handful of row tiles at the same time
            __builtin_amdgcn_global_load_lds((gptr_t)(bb + boff[u]), (lds_ptr_t)(Bs + (wave * kBInstr + u) * 1024), 16, 0,
                                             kSplitK ? 2 : 0);
        }
    };

    i32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i) {
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
        }
    }

    // ---- fragment addresses: one base per K sub-step (A) / per column block (B), everything else is an immediate
    const uint32_t lrow = lane & 31u, g = lane >> 5;
    const uint32_t grp16 = (lane >> 4) & 1u, bsub = (lane & 15u) >> 1, psub = lane & 1u;
    uint32_t a_base[4], b_base[2], bt_base[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        a_base[ks] = (wm * (TI * 32) + lrow) * 128 + (((2 * ks + g) ^ ((lrow >> 1) & 7u)) << 4);
        bt_base[ks] = (wn * (TJ * 32) + lrow) * 128 + (((2 * ks + g) ^ ((lrow >> 1) & 7u)) << 4);
        if constexpr (kBP) {
            // column block j of the wavefront: slabs 4 wn + 2 j + lrow / 16 (2 KiB each: the step's two k tiles); sub-step
            // ks is k tile ks / 2, its 16-byte groups 2 (ks % 2) + g; inside a group the 16 columns lie side by side
            bt_base[ks] = wn * 8192u + (lrow >> 4) * 2048u + (ks >> 1) * 1024u + ((ks & 1) * 2u + g) * 256u + (lrow & 15u) * 16u;
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t swz = BN == 256 ? 2u * bsub : 2u * ((bsub >> 1) & 3u);
        b_base[j] = (16 * g + bsub) * BN + (((4 * wn + 2 * j + grp16) ^ swz) << 4) + 8 * psub;
    }
    // In the order the MFMAs of a sub-step want them (they run row block by row block): B0, A0, B1, A1, A2, ...
    auto load_frags = [&](const char* As, const char* Bs, int ks, i32x4 (&af)[TI], i32x4 (&bf)[TJ]) {
        auto load_b = [&](int j) {
            if constexpr (kBT || kBP) {
                bf[j] = *reinterpret_cast<const i32x4*>(Bs + bt_base[ks] + j * 4096);
            } else {
                const i32x2_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2_t)(Bs + b_base[j] + ks * kKsB));
                const i32x2_t hi =
                    __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2_t)(Bs + b_base[j] + ks * kKsB + 8 * BN));
                bf[j] = i32x4{lo[0], lo[1], hi[0], hi[1]};
            }
        };
        load_b(0);
        af[0] = *reinterpret_cast<const i32x4*>(As + a_base[ks]);
        load_b(1);
#pragma unroll
        for (int i = 1; i < TI; ++i) {
            af[i] = *reinterpret_cast<const i32x4*>(As + a_base[ks] + i * 4096);
        }
    };
    // Fragment registers live across K steps: buffer 0 holds sub-steps 0 and 2, buffer 1 sub-steps 1 and 3.
    i32x4 af[2][TI], bf[2][TJ];
    auto mfma_block = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][i], bf[buf][j], acc[i][j], 0, 0, 0);
            }
        }
    };
    // The LDS reads of a sub-step go out behind its first MFMAs (kReadsPerMfma behind each), so that the matrix
    // instructions of its second half run while the last reads are still on their way: the next sub-step starts by
    // waiting for all of them.
    auto interleave = [&]() __attribute__((always_inline)) {
        constexpr int kReads = TI + ((kBT || kBP) ? TJ : 2 * TJ);
        constexpr int kMfmas = TI * TJ;
        constexpr int kFront = (kMfmas + 1) / 2;
        constexpr int kPer = (kReads + kFront - 1) / kFront;
        static_for<kMfmas>([&](auto n) {
            constexpr int kLeft = kReads - decltype(n)::value * kPer;
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (kLeft > 0) {
                __builtin_amdgcn_sched_group_barrier(0x100, kLeft < kPer ? kLeft : kPer, 0);
            }
        });
        __builtin_amdgcn_sched_barrier(0);
    };
    // Sub-steps 0-2 of a K step whose sub-step-0 fragments are already in buffer 0; on return the fragments of
    // sub-step 3 are on their way into buffer 1 and nothing else of the stage will be read.
    auto head = [&](const char* As, const char* Bs) __attribute__((always_inline)) {
        // Re-materialise the bases inside the loop body: the constant parts of every address then fold into the
        // 16-bit offset field of the DS instructions instead of being hoisted into dozens of registers.
#pragma unroll
        for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(a_base[q]));
#pragma unroll
        for (int q = 0; q < 2; ++q) asm volatile("" : "+v"(b_base[q]));
        if constexpr (kBT || kBP) {
#pragma unroll
            for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(bt_base[q]));
        }
#pragma unroll
        for (int ks = 0; ks < 3; ++ks) {
            load_frags(As, Bs, ks + 1, af[(ks + 1) & 1], bf[(ks + 1) & 1]);
            mfma_block(ks & 1);
            interleave();
        }
    };
    // Behind the barrier: the MFMAs of sub-step 3 run while the first fragments of the next K step (stage An, Bn)
    // arrive, so the matrix pipe has work during the burst of LDS reads that follows every barrier.
    auto tail = [&](const char* An, const char* Bn) __attribute__((always_inline)) {
        load_frags(An, Bn, 0, af[0], bf[0]);
        mfma_block(1);
        interleave();
    };

    if (steps != 0) {
        issue(0, A0, B0);
    }
    asm volatile("s_waitcnt vmcnt(0)");
    __syncthreads();
    // A wavefront whose rows all lie past the end of the tile's group (ragged grouped tiles) skips the matrix work and
    // only keeps the loads and barriers going: its SIMD then runs one wavefront's MFMAs per K step instead of two.
    const bool wave_active = !kGrouped || row0 + wm * (TI * 32u) < row_end;
    if (steps > 1) {
        issue(BK, A1, B1);
    }
    if (wave_active && steps != 0) {
        load_frags(A0, B0, 0, af[0], bf[0]);
    }
    // Per K step: sub-steps 0-2, wait for the next stage's DMA, barrier (every wavefront has the last fragments of
    // this stage in registers, so the stage is free), DMA of the step after next into this stage, sub-step 3.
    // The loop body never branches between two ways of updating the accumulators (that would make the compiler
    // shuffle all 256 of them): the steady state always has a next step, the last one or two steps are peeled.
    uint32_t s = 0;
#define ASCQ_WAIT_AND_BARRIER()             \
    do {                                    \
        asm volatile("s_waitcnt vmcnt(0)"); \
        __syncthreads();                    \
    } while (0)
    for (; s + 2 < steps; s += 2) {
        if (wave_active) head(A0, B0);
        ASCQ_WAIT_AND_BARRIER();
        issue((s + 2) * BK, A0, B0);
        if (wave_active) tail(A1, B1);
        if (wave_active) head(A1, B1);
        ASCQ_WAIT_AND_BARRIER();
        if (s + 3 < steps) {
            issue((s + 3) * BK, A1, B1);
        }
        if (wave_active) tail(A0, B0);
    }
    if (s + 1 < steps) {  // two steps left: this one in stage 0, the last one on its way into stage 1
        if (wave_active) head(A0, B0);
        asm volatile("s_waitcnt vmcnt(0)");
        __syncthreads();
        if (wave_active) tail(A1, B1);
        ++s;
    }
    if (s < steps) {  // the last step: stage 0 for an odd number of steps, stage 1 for an even one
        const char* Al = (steps & 1u) ? A0 : A1;
        const char* Bl = (steps & 1u) ? B0 : B1;
        if (wave_active) {
            head(Al, Bl);
            mfma_block(1);
        }
    }

    // ---- epilogue: register r of lane l in a 32x32 block is row 8*(r/4) + 4*(l/32) + r%4, column l%32
    if constexpr (kSplitK) {
        int32_t* part = p.partial + static_cast<size_t>(bidy) * p.m * N;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                const uint32_t col = n0 + (wn * TJ + j) * 32u + lrow;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = row0 + (wm * TI + i) * 32u + 8u * (r >> 2) + 4u * g + (r & 3);
                    if (row < row_end && col < N) {
                        part[static_cast<size_t>(row) * N + col] = acc[i][j][r];
                    }
                }
            }
        }
        return;
    }
    const EpiParams& e = p.epi;
    auto run = [&](auto tag) {
        constexpr int kOut = decltype(tag)::value;
        const uint32_t colw = n0 + wn * (TJ * 32u);  // first column of this wavefront
        ChannelQ q[TJ];
        float bias_post[TJ];
        int32_t bias_pre[TJ];
        bool cvalid[TJ];
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const uint32_t col = colw + j * 32u + lrow;
            cvalid[j] = col < N;
            q[j] = ChannelQ{1.0f, 0, 1};
            bias_post[j] = 0.0f;
            bias_pre[j] = 0;
            if (cvalid[j]) {
                q[j] = load_channel_q(e, chan_off + col);
                bias_post[j] = load_bias_post(e, chan_off + col);
                if (e.bias_kind == ASCQ_MM_BIAS_I32_PRE) {
                    bias_pre[j] = static_cast<const int32_t*>(e.bias)[chan_off + col];
                }
            }
        }
        // The uniform choices (post-dequant bias, activation) are made once, outside the element loops, so that each
        // wavefront runs one compact straight-line epilogue.
        auto store_all = [&](auto bias_tag, auto gelu_tag, auto swiglu_tag) {
            constexpr bool kBiasPost = decltype(bias_tag)::value;
            constexpr bool kGelu = decltype(gelu_tag)::value;
            constexpr bool kSwiGlu = decltype(swiglu_tag)::value;
            (void)kBiasPost;
            (void)kGelu;
            (void)kSwiGlu;
    #pragma unroll
            for (int i = 0; i < TI; ++i) {
                const uint32_t lbase = (wm * TI + i) * 32u + 4u * g;  // row inside the tile of register 0
    #pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    const f32x4 tok4 = *reinterpret_cast<const f32x4*>(&TS[lbase + 8u * rq]);
    #pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const int r = 4 * rq + rr;
                        const uint32_t row = row0 + lbase + 8u * rq + rr;
                        if constexpr (kOut == ASCQ_BF16 || kOut == ASCQ_F16) {
                            // One dword store per lane covers a full 128-byte line per row: even lanes write columns
                            // (l, l+1) of the first 32-column block, odd lanes columns (l-1, l) of the second one.
                            static_assert(TJ == 2, "the paired store assumes two column blocks per wavefront");
                            const bool odd = (lane & 1u) != 0;
                            if constexpr (kSwiGlu) {
                                // Adjacent lanes hold the two columns of a pair.  After one lane swap the even lane
                                // owns the pair of the first 32-column block (src0 its own value, src1 its
                                // neighbour's), the odd lane the pair of the second block (src0 its neighbour's).
                                const float v0 = epi_value<kBiasPost, false>(acc[i][0][r] + bias_pre[0], q[0].s, tok4[rr],
                                                                             bias_post[0]);
                                const float v1 = epi_value<kBiasPost, false>(acc[i][1][r] + bias_pre[1], q[1].s, tok4[rr],
                                                                             bias_post[1]);
                                const float recv = __int_as_float(__builtin_amdgcn_mov_dpp(
                                    __float_as_int(odd ? v0 : v1), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                                const float o = swiglu(odd ? recv : v0, odd ? v1 : recv, e.act_beta);
                                const uint32_t col = odd ? colw + 32u + (lrow - 1u) : colw + lrow;  // first column of the pair
                                if (row < row_end && col < N) {
                                    __builtin_nontemporal_store(
                                        static_cast<uint16_t>(to_bits16<kOut>(o)),
                                        static_cast<uint16_t*>(e.c) + static_cast<size_t>(row) * e.ldc + (col >> 1));
                                }
                                continue;
                            }
                            const uint32_t h0 =
                                to_bits16<kOut>(
                                    epi_value<kBiasPost, kGelu>(acc[i][0][r] + bias_pre[0], q[0].s, tok4[rr], bias_post[0]));
                            const uint32_t h1 =
                                to_bits16<kOut>(
                                    epi_value<kBiasPost, kGelu>(acc[i][1][r] + bias_pre[1], q[1].s, tok4[rr], bias_post[1]));
                            const uint32_t send = odd ? h0 : h1;
                            const uint32_t recv = static_cast<uint32_t>(
                                __builtin_amdgcn_mov_dpp(static_cast<int>(send), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                            const uint32_t word = odd ? (recv | (h1 << 16)) : (h0 | (recv << 16));
                            const uint32_t col = odd ? colw + 32u + (lrow - 1u) : colw + lrow;
                            if (row < row_end && col < N) {
                                __builtin_nontemporal_store(
                                    word, reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(e.c) +
                                                                      static_cast<size_t>(row) * e.ldc + col));
                            }
                        } else {
    #pragma unroll
                            for (int j = 0; j < TJ; ++j) {
                                if (cvalid[j] && row < row_end) {
                                    epilogue_store<kOut>(e, row, colw + j * 32u + lrow, acc[i][j][r] + bias_pre[j], q[j],
                                                         tok4[rr], bias_post[j]);
                                }
                            }
                        }
                    }
                }
            }
        };
        if constexpr (kOut == ASCQ_BF16 || kOut == ASCQ_F16) {
            // Quant words that shift the accumulator first (mode-control bit) are rare: when any column of the
            // wavefront carries one, a compact epilogue that reads every choice at run time serves the whole
            // wavefront, element by element, and the specialised ones below stay as they are.
            if (e.scale_format == ASCQ_MM_SCALE_U64 && e.quant_mode != ASCQ_MM_QUANT_NONE &&
                __builtin_amdgcn_ballot_w64(((q[0].ctl | q[TJ - 1].ctl) & 2) != 0) != 0) {
                const bool odd = (lane & 1u) != 0;
#pragma unroll  // (a run-time index into the accumulators would move them to scratch memory)
                for (int i = 0; i < TI; ++i) {
                    const uint32_t lbase = (wm * TI + i) * 32u + 4u * g;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t lrow_t = lbase + 8u * (r >> 2) + (r & 3);
                        const uint32_t row = row0 + lrow_t;
                        const float tok = TS[lrow_t];
                        float v[TJ];
#pragma unroll
                        for (int j = 0; j < TJ; ++j) {
                            v[j] = epilogue_value(e, acc[i][j][r] + bias_pre[j], q[j], tok, bias_post[j]);
                        }
                        if (e.activation == ASCQ_MM_ACT_SWIGLU) {
                            const float recv = __int_as_float(__builtin_amdgcn_mov_dpp(
                                __float_as_int(odd ? v[0] : v[TJ - 1]), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                            const float o = swiglu(odd ? recv : v[0], odd ? v[TJ - 1] : recv, e.act_beta);
                            const uint32_t col = odd ? colw + 32u + (lrow - 1u) : colw + lrow;
                            if (row < row_end && col < N) {
                                static_cast<uint16_t*>(e.c)[static_cast<size_t>(row) * e.ldc + (col >> 1)] =
                                    static_cast<uint16_t>(to_bits16<kOut>(o));
                            }
                            continue;
                        }
#pragma unroll
                        for (int j = 0; j < TJ; ++j) {
                            if (cvalid[j] && row < row_end) {
                                const float o = e.activation == ASCQ_MM_ACT_FASTER_GELU ? faster_gelu(v[j]) : v[j];
                                static_cast<uint16_t*>(e.c)[static_cast<size_t>(row) * e.ldc + colw + j * 32u + lrow] =
                                    static_cast<uint16_t>(to_bits16<kOut>(o));
                            }
                        }
                    }
                }
                return;
            }
            const bool bias_post_on = e.bias_kind >= ASCQ_MM_BIAS_F32_POST;
            const bool gelu_on = e.activation == ASCQ_MM_ACT_FASTER_GELU;
            if (e.activation == ASCQ_MM_ACT_SWIGLU) {
                if (bias_post_on) {
                    store_all(std::true_type{}, std::false_type{}, std::true_type{});
                } else {
                    store_all(std::false_type{}, std::false_type{}, std::true_type{});
                }
            } else if (gelu_on) {
                if (bias_post_on) {
                    store_all(std::true_type{}, std::true_type{}, std::false_type{});
                } else {
                    store_all(std::false_type{}, std::true_type{}, std::false_type{});
                }
            } else if (bias_post_on) {
                store_all(std::true_type{}, std::false_type{}, std::false_type{});
            } else {
                store_all(std::false_type{}, std::false_type{}, std::false_type{});
            }
        } else {
            // the generic store reads both choices at run time (the host sends SwiGLU with these outputs elsewhere)
            store_all(std::false_type{}, std::false_type{}, std::false_type{});
        }
    };
    dispatch_out(e, run);
}

// The plain matmul: tile number `bid` of the launch (before the XCD remapping), column tiles counted from col_begin,
// row tiles innermost so that the tiles an XCD runs side by side share their B columns.
template <int BM, int BN, bool kSplitK, int kB>
__device__ __forceinline__ void gemm_dma_tile(const GemmParams& p, uint32_t col_begin, uint32_t bid, uint32_t bidy,
                                              char* A0, char* B0, char* A1, char* B1, float* TS)
{
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t t = xcd_remap(bid, total);
    if (t >= total) {
        return;
    }
    // bands of 8 row tiles, inside a band column by column (band_order): an XCD's share stays a block of a few columns
    // by 8 rows whose rows of A and columns of B it reuses from its L2, however many rows the matrix has
    uint32_t ms, tn;
    band_order(t, p.tiles_m, p.tiles_n, ms, tn);
    const TilePlace at{ms * BM, p.m, col_begin + tn * BN, p.b, 0};
    gemm_dma_tile_at<BM, BN, kSplitK, false, kB>(p, at, bidy, A0, B0, A1, B1, TS);
}

// Rows [off, end) of group g (clipped to m); false when the group owns none.  `off` is carried from group to group.
__device__ __forceinline__ bool group_rows(const GemmParams& p, uint32_t g, int64_t& off, uint32_t& first, uint32_t& end)
{
    const int64_t v = p.group_list[g];
    const int64_t cnt = p.group_list_kind == ASCQ_GROUP_LIST_PREFIX_SUM ? v - off : v;
    if (cnt <= 0) {
        return false;
    }
    const int64_t begin = off;
    off += cnt;
    const int64_t stop = off > static_cast<int64_t>(p.m) ? static_cast<int64_t>(p.m) : off;
    first = static_cast<uint32_t>(begin);
    end = static_cast<uint32_t>(stop);
    return stop > begin;
}

// Row tiles of a group: `big` tiles of 256 rows (a remainder of more than 128 rows is one of them) and at most one
// small tile of 128 rows for a shorter remainder.
__device__ __forceinline__ void group_row_tiles(uint32_t rows, uint32_t& big, uint32_t& small)
{
    const uint32_t rem = rows & 255u;
    big = (rows >> 8) + (rem > 128u ? 1u : 0u);
    small = (rem != 0u && rem <= 128u) ? 1u : 0u;
}

// One phase of the grouped kernel's plan (see gemm_dma_group_kernel): the workgroup's ids that fall into it.
template <uint32_t phase>
__device__ __forceinline__ void gemm_dma_group_phase(const GemmParams& p, const uint32_t* PLAN, char* A0, char* B0,
                                                     char* A1, char* B1, float* TS)
{
    for (uint32_t id = blockIdx.x;; id += gridDim.x) {
        const uint32_t tiles_n = p.tiles_n;
        const uint32_t big_tiles = __builtin_amdgcn_readfirstlane(PLAN[0]);
        const uint32_t small_tiles = __builtin_amdgcn_readfirstlane(PLAN[1]);
        const uint32_t wide = __builtin_amdgcn_readfirstlane(PLAN[2]);
        const uint32_t col_narrow = wide * 256u;
        const uint32_t narrow = col_narrow < p.n ? (p.n - col_narrow + 127u) / 128u : 0u;
        const uint32_t count0 = big_tiles * wide, count1 = big_tiles * narrow, count2 = small_tiles * tiles_n;
        const uint32_t first1 = (count0 + 7u) & ~7u, first2 = first1 + ((count1 + 7u) & ~7u);
        const uint32_t first = phase == 0 ? 0u : phase == 1 ? first1 : first2;
        const uint32_t count = phase == 0 ? count0 : phase == 1 ? count1 : count2;
        const uint32_t cols = phase == 0 ? wide : phase == 1 ? narrow : tiles_n;
        if (id < first) {
            continue;  // an id of an earlier phase
        }
        if (id >= first + ((count + 7u) & ~7u)) {
            break;
        }
        const uint32_t t = xcd_remap(id - first, count);
        if (t >= count) {
            continue;  // padding of the phase
        }
        TilePlace at{0, 0, 0, nullptr, 0};
        {
            uint32_t base = 0;
            int64_t off = 0;
            for (uint32_t g = 0; g < p.groups; ++g) {
                uint32_t first, end, big, small;
                if (!group_rows(p, g, off, first, end)) {
                    continue;
                }
                group_row_tiles(end - first, big, small);
                const uint32_t mine = phase == 2 ? small : big;
                if (t >= base + mine * cols) {
                    base += mine * cols;
                    continue;
                }
                const uint32_t local = t - base;
                const uint32_t tn = local / mine, tr = local - tn * mine;
                at.row0 = first + (phase == 2 ? ((end - first) >> 8) * 256u : tr * 256u);
                at.row_end = end;
                at.n0 = phase == 1 ? col_narrow + tn * 128u : tn * 256u;
                at.b = p.b + static_cast<size_t>(g) * p.k * p.n;
                at.chan_off = static_cast<size_t>(g) * p.n;
                break;
            }
        }
        if (at.b == nullptr) {
            continue;
        }
        if constexpr (phase == 0) {
            gemm_dma_tile_at<256, 256, false, true>(p, at, 0u, A0, B0, A1, B1, TS);
        } else if constexpr (phase == 1) {
            gemm_dma_tile_at<256, 128, false, true>(p, at, 0u, A0, B0, A1, B1, TS);
        } else if (at.row_end - at.row0 <= 64u) {  // uniform: a remainder of at most 64 rows
            gemm_dma_tile_at<64, 256, false, true>(p, at, 0u, A0, B0, A1, B1, TS);
        } else {
            gemm_dma_tile_at<128, 256, false, true>(p, at, 0u, A0, B0, A1, B1, TS);
        }
        __syncthreads();  // the next tile's loads and token scales overwrite what slower wavefronts may still read
    }
}

// The grouped matmul in one launch of persistent workgroups, one per compute unit.  Every workgroup reads the group
// list and derives the same plan from it:
//   phase 0: the big row tiles x the first `wide` 256-wide tile columns, as many as fill whole rounds of the chip;
//   phase 1: the big row tiles x the remaining columns as 256 x 128 tiles (the last, partial round in half-size pieces);
//   phase 2: the groups' short remainders (at most 128 rows) as 128 x 256 tiles (64 x 256 up to 64 rows), cheapest last.
// Tile ids run through the phases in this order (each phase padded to a multiple of 8 ids, so that id mod 8 stays the
// XCD of the workgroup that takes it); workgroup w takes ids w, w + gridDim.x, ...  Inside a phase the tiles are
// ordered group by group, column by column, the row tiles of a column adjacent, and an XCD takes a contiguous share:
// about one group per XCD, whose rows of A stay in that L2 while each B tile is fetched once for the row tiles that
// run side by side.  The group sizes are known only on the device, so a launch sized by the host for the worst case
// would consist mostly of workgroups with nothing to do; the loop has none.  gridDim.x must be a multiple of 8;
// p.tiles_n = 256-wide tile columns of the whole matrix.
__global__ __launch_bounds__(kThreads, 1) void gemm_dma_group_kernel(GemmParams p)
{
    __shared__ __attribute__((aligned(1024))) char A0[256 * BK];
    __shared__ __attribute__((aligned(1024))) char B0[BK * 256];
    __shared__ __attribute__((aligned(1024))) char A1[256 * BK];
    __shared__ __attribute__((aligned(1024))) char B1[BK * 256];
    __shared__ __attribute__((aligned(16))) float TS[256];
    uint32_t n_big = 0, n_small = 0;
    {
        int64_t off = 0;
        for (uint32_t g = 0; g < p.groups; ++g) {
            uint32_t first, end, big, small;
            if (group_rows(p, g, off, first, end)) {
                group_row_tiles(end - first, big, small);
                n_big += big;
                n_small += small;
            }
        }
    }
    // The plan is parked in LDS and re-read per tile: held in scalar registers across the tile bodies it would push
    // the compiler into spilling them.
    __shared__ uint32_t PLAN[4];
    {
        const uint32_t units = n_big * p.tiles_n + (n_small * p.tiles_n + 1u) / 2u;  // work in 256 x 256 tiles
        uint32_t wide = n_big ? units / gridDim.x * gridDim.x / n_big : 0u;
        if (wide > p.tiles_n) {
            wide = p.tiles_n;
        }
        if (threadIdx.x == 0) {
            PLAN[0] = n_big;
            PLAN[1] = n_small;
            PLAN[2] = wide;
        }
        __syncthreads();
    }
    // One loop per phase (a workgroup's ids ascend, so it passes through the phases in order anyway): each loop holds
    // one tile shape's code and registers.
    gemm_dma_group_phase<0>(p, PLAN, A0, B0, A1, B1, TS);
    gemm_dma_group_phase<1>(p, PLAN, A0, B0, A1, B1, TS);
    gemm_dma_group_phase<2>(p, PLAN, A0, B0, A1, B1, TS);
}

template <int BM, int BN, bool kSplitK, int kB = 0>
__global__ __launch_bounds__(kThreads, (BM * BK + BK * BN) * 2 <= 65536 ? 2 : 1) void gemm_dma_kernel(
    GemmParams p, uint32_t col_begin)
{
    __shared__ __attribute__((aligned(1024))) char A0[BM * BK];
    __shared__ __attribute__((aligned(1024))) char B0[BK * BN];
    __shared__ __attribute__((aligned(1024))) char A1[BM * BK];
    __shared__ __attribute__((aligned(1024))) char B1[BK * BN];
    __shared__ __attribute__((aligned(16))) float TS[BM];  // token scales of the tile's rows (1.0f when there are none)
    gemm_dma_tile<BM, BN, kSplitK, kB>(p, col_begin, blockIdx.x, blockIdx.y, A0, B0, A1, B1, TS);
}

// One launch for a matrix whose last round of 256 x 256 tiles would be mostly empty: workgroups [0, wide_wgs) run the
// 256 x 256 tiles of the first `p.tiles_n` tile columns, the rest 256 x 128 tiles of the remaining columns.  A compute
// unit that has finished its wide tile takes a narrow one at once, without the drain between two launches.
template <int kB>
__global__ __launch_bounds__(kThreads, 1) void gemm_dma_dual_kernel(GemmParams p, uint32_t wide_wgs,
                                                                    uint32_t narrow_tiles_n, uint32_t col_begin)
{
    __shared__ __attribute__((aligned(1024))) char A0[256 * BK];
    __shared__ __attribute__((aligned(1024))) char B0[BK * 256];
    __shared__ __attribute__((aligned(1024))) char A1[256 * BK];
    __shared__ __attribute__((aligned(1024))) char B1[BK * 256];
    __shared__ __attribute__((aligned(16))) float TS[256];
    if (blockIdx.x < wide_wgs) {
        gemm_dma_tile<256, 256, false, kB>(p, 0u, blockIdx.x, 0u, A0, B0, A1, B1, TS);
    } else {
        GemmParams q = p;
        q.tiles_n = narrow_tiles_n;
        gemm_dma_tile<256, 128, false, kB>(q, col_begin, blockIdx.x - wide_wgs, 0u, A0, B0, A1, B1, TS);
    }
}

// Second pass of the split-K path: sums the int32 partial tiles [split][m][n] in split order (integer addition: exact in
// any order) and applies the epilogue.  One lane = four consecutive columns.
__global__ __launch_bounds__(256) void splitk_sum_epilogue_kernel(GemmParams p)
{
    const size_t quads = static_cast<size_t>(p.m) * p.n / 4u;
    const size_t plane = static_cast<size_t>(p.m) * p.n;
    for (size_t qd = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; qd < quads;
         qd += static_cast<size_t>(gridDim.x) * 256u) {
        const size_t idx = qd * 4u;
        i32x4 acc = *reinterpret_cast<const i32x4*>(p.partial + idx);
        for (uint32_t sp = 1; sp < p.k_splits; ++sp) {
            const i32x4 v = *reinterpret_cast<const i32x4*>(p.partial + sp * plane + idx);
            acc += v;
        }
        const size_t row = idx / p.n, col = idx % p.n;
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
}

}  // namespace

bool gemm_dma_supported(const GemmParams& p)
{
    return p.k % BK == 0 && p.n % 16 == 0 && p.n >= 16 && aligned16(p.a) && aligned16(p.b);
}

namespace {

// calls f with the B layout (0: [k, n], 1: [n, k], 2: packed by ascq_pack_weight_w8) as a compile-time constant
template <class F>
void with_b_layout(int b_layout, F&& f)
{
    if (b_layout == 2) {
        f(std::integral_constant<int, 2>{});
    } else if (b_layout == 1) {
        f(std::integral_constant<int, 1>{});
    } else {
        f(std::integral_constant<int, 0>{});
    }
}

}  // namespace

int launch_gemm_dma(GemmParams& p, bool grouped, hipStream_t st, int b_layout)
{
    uint32_t tiles_n = (p.n + 255u) / 256u;
    if (grouped) {
        // The group sizes are on the device; the kernel plans its tiles there.  One persistent workgroup per compute
        // unit (a multiple of 8, so that a workgroup's id mod 8 is its XCD), fewer when no group list over m rows
        // can need that many tiles: big row tiles hold more than 128 rows each, at most m / 256 + groups of them, and
        // every group adds at most one short remainder.
        const uint32_t big = p.m / 129u < p.m / 256u + p.groups ? p.m / 129u : p.m / 256u + p.groups;
        const uint32_t small = p.groups < p.m ? p.groups : p.m;
        const uint64_t most = static_cast<uint64_t>(big) * 2u * tiles_n + static_cast<uint64_t>(small) * tiles_n + 24u;
        uint32_t wgs = device_compute_units() / 8u * 8u;
        if (wgs == 0u) {
            wgs = 8u;
        }
        if (most < wgs) {
            wgs = static_cast<uint32_t>((most + 7u) / 8u * 8u);
        }
        p.tiles_m = big + small;
        p.tiles_n = tiles_n;
        if (plan_recording()) {
            plan_note(ASCQ_MM_KERNEL_DMA_256, 256, 256, BK, wgs, 1, 2u * (256u * BK + BK * 256u) + 256u * 4u, 0);
            return ASCQ_OK;
        }
        gemm_dma_group_kernel<<<wgs, kThreads, 0, st>>>(p);
        return launch_status("ascq_group_matmul_w8a8");
    }
    p.tiles_m = (p.m + 255u) / 256u;
    // Tile quantisation: when the last round of 256-wide tiles would fill less than half of the 256 CUs, its
    // columns are computed with 128-wide tiles, which finish that round in about half the time.
    uint32_t narrow_cols = 0;  // number of 256-wide column tiles handed to the 128-wide kernel
    const uint32_t total = p.tiles_m * tiles_n;
    const uint32_t rem = total % 256u;
    if (total > 256u && rem != 0 && rem <= 128u) {
        narrow_cols = (rem + p.tiles_m - 1) / p.tiles_m;
        if (narrow_cols > tiles_n) {
            narrow_cols = tiles_n;
        }
    }
    const uint32_t wide_cols = tiles_n - narrow_cols;
    if (plan_recording()) {
        constexpr uint32_t kLdsWide = 2u * (256u * BK + BK * 256u) + 256u * 4u;
        constexpr uint32_t kLdsNarrow = 2u * (256u * BK + BK * 128u) + 256u * 4u;
        const uint32_t wide_wg = (p.tiles_m * wide_cols + 7u) / 8u * 8u;
        const uint32_t narrow_tiles = narrow_cols ? (p.n - wide_cols * 256u + 127u) / 128u : 0u;
        const uint32_t narrow_wg = (p.tiles_m * narrow_tiles + 7u) / 8u * 8u;
        if (wide_cols) {
            plan_note(ASCQ_MM_KERNEL_DMA_256, 256, 256, BK, wide_wg, 1, kLdsWide, 0);
            if (narrow_cols) {
                plan_note_extra(128, narrow_wg);  // workgroups of the same launch
            }
        } else {
            plan_note(ASCQ_MM_KERNEL_DMA_256, 256, 128, BK, narrow_wg, 1, kLdsNarrow, 0);
        }
        return ASCQ_OK;
    }
    if (wide_cols && narrow_cols) {
        // both tile shapes in one launch (narrow_cols is only ever non-zero for the plain matmul)
        const uint32_t col_begin = wide_cols * 256u;
        const uint32_t narrow_tiles_n = (p.n - col_begin + 127u) / 128u;
        const uint32_t wide_wgs = (p.tiles_m * wide_cols + 7u) / 8u * 8u;
        const uint32_t narrow_wgs = (p.tiles_m * narrow_tiles_n + 7u) / 8u * 8u;
        p.tiles_n = wide_cols;
        with_b_layout(b_layout, [&](auto kb) {
            gemm_dma_dual_kernel<decltype(kb)::value><<<wide_wgs + narrow_wgs, kThreads, 0, st>>>(p, wide_wgs, narrow_tiles_n,
                                                                                                  col_begin);
        });
        return launch_status("ascq_matmul_w8a8");
    }
    if (wide_cols) {
        p.tiles_n = wide_cols;
        const uint32_t t = p.tiles_m * p.tiles_n;
        // the wide launch must not touch the narrow region: clip n for its column masks
        GemmParams q = p;
        if (narrow_cols) {
            q.n = p.n;  // row pitch stays n; columns >= wide_cols * 256 are simply not assigned to any tile
        }
        with_b_layout(b_layout, [&](auto kb) {
            gemm_dma_kernel<256, 256, false, decltype(kb)::value><<<(t + 7u) / 8u * 8u, kThreads, 0, st>>>(q, 0u);
        });
    }
    if (narrow_cols) {
        const uint32_t col_begin = wide_cols * 256u;
        p.tiles_n = (p.n - col_begin + 127u) / 128u;
        const uint32_t t = p.tiles_m * p.tiles_n;
        with_b_layout(b_layout, [&](auto kb) {
            gemm_dma_kernel<256, 128, false, decltype(kb)::value><<<(t + 7u) / 8u * 8u, kThreads, 0, st>>>(p, col_begin);
        });
    }
    return launch_status("ascq_matmul_w8a8");
}

// Split factor of the 128 x 128 kernel: two workgroups per CU when the partial tiles are small next to the weights,
// one per CU otherwise; never more splits than K steps.
uint32_t gemm_dma_skinny_splits(uint32_t m, uint32_t n, uint32_t k)
{
    // Measured at k = 4096, n = 11008 (86 column tiles) with the weights coming from HBM: one row tile (m <= 128) is
    // fastest with 4 splits (17-25 us; 2 splits 21-25, 6 splits 25-32, none 30), two or more row tiles are fastest
    // with none (30-32 us for m = 160 .. 384 against 32-55 with 2): once the tiles alone cover most of the compute
    // units the int32 partial tiles, written and read back, cost more than the idle units.  Hence: no split from 160
    // tiles on, otherwise about 1.35 workgroups per compute unit, all resident at once (two fit a unit).
    const uint32_t tiles = ((m + 127u) / 128u) * ((n + 127u) / 128u);
    if (tiles >= 160u) {
        return 1u;
    }
    uint32_t s = 344u / tiles;
    const uint32_t steps = k / BK;
    if (s > steps) s = steps;
    if (s > 16u) s = 16u;
    return s ? s : 1u;
}

// M up to a few hundred rows: 128 x 128 tiles, K split over blockIdx.y when a workspace of
// splits * m * n * 4 bytes (16-byte aligned) is given.  b_layout: 0 [k, n], 1 [n, k], 2 packed (never split: its
// entry point has no workspace).
int launch_gemm_dma_skinny(GemmParams& p, void* workspace, size_t workspace_bytes, hipStream_t st, int b_layout)
{
    p.tiles_m = (p.m + 127u) / 128u;
    p.tiles_n = (p.n + 127u) / 128u;
    const uint32_t t = (p.tiles_m * p.tiles_n + 7u) / 8u * 8u;
    uint32_t splits = gemm_dma_skinny_splits(p.m, p.n, p.k);
    const size_t need = static_cast<size_t>(splits) * p.m * p.n * sizeof(int32_t);
    if (splits > 1 && (workspace == nullptr || workspace_bytes < need || !aligned16(workspace) || b_layout == 2)) {
        splits = 1;
    }
    if (plan_recording()) {
        constexpr uint32_t kLds = 2u * (128u * BK + BK * 128u) + 128u * 4u;
        plan_note(ASCQ_MM_KERNEL_DMA_128, 128, 128, BK, t * splits, splits, kLds, splits > 1 ? need : 0);
        if (splits > 1) {
            plan_note(0, 0, 0, 0, 0, 0, 0, 0);  // the kernel that adds the partial tiles and applies the epilogue
        }
        return ASCQ_OK;
    }
    if (splits == 1) {
        with_b_layout(b_layout, [&](auto kb) {
            gemm_dma_kernel<128, 128, false, decltype(kb)::value><<<t, kThreads, 0, st>>>(p, 0u);
        });
        return launch_status("ascq_matmul_w8a8");
    }
    p.k_splits = splits;
    p.partial = static_cast<int32_t*>(workspace);
    if (b_layout == 1) {
        gemm_dma_kernel<128, 128, true, 1><<<dim3(t, splits), kThreads, 0, st>>>(p, 0u);
    } else {
        gemm_dma_kernel<128, 128, true><<<dim3(t, splits), kThreads, 0, st>>>(p, 0u);
    }
    int rc = launch_status("ascq_matmul_w8a8 (split-K)");
    if (rc != ASCQ_OK) {
        return rc;
    }
    size_t blocks = (static_cast<size_t>(p.m) * p.n / 4u + 255u) / 256u;
    if (blocks > 8192u) blocks = 8192u;
    splitk_sum_epilogue_kernel<<<static_cast<uint32_t>(blocks), 256, 0, st>>>(p);
    return launch_status("ascq_matmul_w8a8 (split-K epilogue)");
}

}  // namespace ascq
