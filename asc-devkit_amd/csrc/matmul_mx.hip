// Block-scaled (MX) matmul: c[m, n] = sum_k a[m, k] 2^(sa[m, k / 32] - 127) * b[n, k] 2^(sb[n, k / 32] - 127) (+ bias).
// a and b are fp8 (e4m3fn, e5m2) or fp4 (e2m1, e1m2; two per byte along k), both k-contiguous; the scales are one
// fp8_e8m0 byte per row and 32 k.
//
// The tile kernel feeds v_mfma_scale_f32_32x32x64_f8f6f4 straight from the given buffers: 256 x 256 tiles, K step of
// 128 bytes of a row (128 fp8 or 256 fp4 values), two LDS stages filled by global_load_lds_dwordx4, 8 wavefronts as
// 2 x 4, each on 128 x 64 of the tile (4 x 2 blocks of 32 x 32, 128 fp32 accumulators).  A tile row is a 128-byte line
// in LDS whose 16-byte pieces are XOR-swizzled by half the row number, applied on the source side of the load.
//   * 8-bit operands: one instruction takes 64 k; registers 0-3 of lane l hold k = 16 (l / 32) .. + 15 and registers
//     4-7 k = 32 + 16 (l / 32) .. + 15 of row l % 32, and the scale of k < 32 comes from lanes 0-31, that of k >= 32
//     from lanes 32-63: two 16-byte LDS reads per operand and instruction.
//   * 4-bit operands: registers 0-3 of lane l hold its row's k = 32 (l / 32) .. + 31 (16 bytes), scaled by the lane's
//     own scale byte: one read per operand and instruction.
//   * 6-bit operands (e2m3 codes, what two e1m2 operands are rewritten as): registers 0-5 of lane l hold its row's
//     k = 32 (l / 32) .. + 31 as little-endian 6-bit fields (24 bytes, padded to 32 in memory), scaled by the lane's
//     own scale byte: a 16-byte and an 8-byte read per operand and instruction.
// In every case lane l needs scale byte 2 j + l / 32 of its row's bytes for this K step in sub-step j; a lane holds
// the bytes of a K step as one dword (8- and 6-bit) or two (4-bit) per row, staged through LDS, and shifts them right
// by 8 (l / 32) where they are used, so that the byte selector of the instruction is the constant 0 or 2.
// The element-wise kernel (one lane per output) takes every other shape; a 4-bit operand beside an 8-bit one, or e1m2
// beside e2m1, is first widened to e4m3, which holds every fp4 value.
#include <type_traits>
#include <utility>

#include "matmul_w8a8.h"

namespace ascq {
namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression.
template <class F, int... I>
__device__ __forceinline__ void mx_static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void mx_static_for(F&& f)
{
    mx_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr uint32_t kMxBM = 256, kMxBN = 256, kMxBK = 128;  // BK in bytes of an operand row
constexpr int kMxThreads = 512;
constexpr uint32_t kMxScaleBuf = (kMxBM + kMxBN) * 16u;  // 16 scale bytes of every row of a tile's a and b

struct MxParams {
    const uint8_t* a;
    const uint8_t* b;
    const uint8_t* sa;
    const uint8_t* sb;
    const float* bias;
    void* c;
    uint32_t m, n, k;       // k in elements
    uint32_t row_bytes;     // bytes of a row of a / b in the tile kernel (both operands have the same width there)
    uint32_t sk;            // bytes of a scale row
    uint32_t tiles_m, tiles_n;
    int32_t a_format, b_format, out_dtype;
};

__device__ __forceinline__ void mx_store(const MxParams& p, size_t idx, float v)
{
    if (p.out_dtype == ASCQ_F32) {
        static_cast<float*>(p.c)[idx] = v;
    } else if (p.out_dtype == ASCQ_BF16) {
        static_cast<uint16_t*>(p.c)[idx] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    } else {
        static_cast<uint16_t*>(p.c)[idx] = static_cast<uint16_t>(f32_to_half_bits_sat(v));
    }
}

// kFour: both operands 4-bit (e2m1); otherwise both a byte per value in memory, with the instruction's format codes
// kCa / kCb (0 = e4m3, 1 = e5m2, 2 = e2m3 as written by mx_widen_e1m2_kernel; 4 = e2m1).
template <bool kFour, int kCa, int kCb>
__global__ __launch_bounds__(kMxThreads, 1) void mx_tile_kernel(MxParams p)
{
    __shared__ __attribute__((aligned(1024))) char A0[kMxBM * kMxBK];
    __shared__ __attribute__((aligned(1024))) char B0[kMxBN * kMxBK];
    __shared__ __attribute__((aligned(1024))) char A1[kMxBM * kMxBK];
    __shared__ __attribute__((aligned(1024))) char B1[kMxBN * kMxBK];
    __shared__ __attribute__((aligned(1024))) char SC[2 * kMxScaleBuf];  // two buffers of scale bytes, see below
    constexpr int TI = 4, TJ = 2;
    constexpr bool kSix = !kFour && kCa == 2;  // e2m3 codes, the 24 bytes of every 32 values padded to 32
    static_assert(!kSix || kCb == 2, "6-bit operands come in pairs");
    constexpr int kSub = kFour ? 4 : 2;       // instructions (64 k each) per K step and block pair
    constexpr int kScaleDw = kFour ? 2 : 1;   // dwords of scale bytes per row and K step

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 2, wn = wave & 3u;
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t t = xcd_remap(blockIdx.x, total);  // every XCD takes a contiguous share
    if (t >= total) {
        return;
    }
    // Tiles run in bands of 8 row tiles, inside a band column by column with the row tiles of a column adjacent: an
    // XCD's share is then a block of about 8 x 16 tiles whose rows of a and b stay in its L2 while they are reused
    // (with all row tiles of a column adjacent and 32 of them, an XCD ran one column at a time and fetched a again
    // for every column: 1177 MB from memory for 67 MB of operands at m = n = k = 8192).
    constexpr uint32_t kBand = 8;
    const uint32_t per_band = kBand * p.tiles_n, full = p.tiles_m / kBand;
    uint32_t tm, tn;
    if (t < full * per_band) {
        const uint32_t r = t % per_band;
        tm = (t / per_band) * kBand + r % kBand;
        tn = r / kBand;
    } else {
        const uint32_t r = t - full * per_band, rows_last = p.tiles_m - full * kBand;
        tm = full * kBand + r % rows_last;
        tn = r / rows_last;
    }
    const uint32_t row0 = tm * kMxBM, n0 = tn * kMxBN;
    const uint32_t RB = p.row_bytes;

    // ---- DMA sources: 4 A and 4 B instructions per wavefront and K step; lane owns LDS slot (instr * 64 + lane) of
    // 16 bytes: row slot / 8, position slot % 8, which holds piece position ^ ((row / 2) % 8) of the row's 128 bytes
    uint32_t aoff[4], boff[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint32_t s = (wave * 4u + u) * 64u + lane;
        const uint32_t r = s >> 3, c = (s & 7u) ^ ((r >> 1) & 7u);
        uint32_t row = row0 + r, col = n0 + r;
        row = row < p.m ? row : p.m - 1u;  // rows and columns past the end are never stored: any valid one will do
        col = col < p.n ? col : p.n - 1u;
        aoff[u] = (row - row0) * RB + 16u * c;
        boff[u] = (col - n0) * RB + 16u * c;
    }
    const uint8_t* Abase = p.a + static_cast<size_t>(row0) * RB;
    const uint8_t* Bbase = p.b + static_cast<size_t>(n0) * RB;
    // A wavefront-uniform address, pinned to scalar registers: a load's address is then this base plus the lane's
    // 32-bit offset, which the load instruction adds itself (otherwise the compiler folds the lane's offset into
    // 64-bit per-lane addresses: twice the registers and an addition per load).
    auto uniform = [](const uint8_t* q) __attribute__((always_inline)) {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        asm volatile("" : "+s"(lo), "+s"(hi));  // opaque: keeps the compiler from re-associating base and lane offset
        return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
    };
    auto issue = [&](uint32_t k0, char* As, char* Bs) __attribute__((always_inline)) {
        const uint8_t* ab = uniform(Abase + k0);
        const uint8_t* bb = uniform(Bbase + k0);
        // (re-materialised here: widened to 64 bits once, ahead of the loop, the offsets would no longer be seen as
        // 32-bit offsets where the loads are selected)
#pragma unroll
        for (int u = 0; u < 4; ++u) asm volatile("" : "+v"(aoff[u]), "+v"(boff[u]));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(ab + aoff[u]), (lds_ptr_t)(As + (wave * 4u + u) * 1024u), 16, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            __builtin_amdgcn_global_load_lds((gptr_t)(bb + boff[u]), (lds_ptr_t)(Bs + (wave * 4u + u) * 1024u), 16, 0, 0);
        }
    };

    // ---- scale bytes.  They come through LDS: a wavefront reading its rows' bytes from memory fetched 32 lines per
    // load for 8 bytes of each, three times the lines of the tile loads themselves, and the kernel took half as
    // long again for it.  Here every second K step one 16-byte load per row (wavefronts 0-3: the 256 rows of a,
    // 4-7: those of b) brings the bytes of the two steps of a "slot" (4-bit form: exactly those 16 bytes; 8-bit form:
    // 8 of them) into buffer slot % 2, as a direct-to-LDS load beside the tile loads; at the row's end the 16 bytes
    // are moved back to stay inside the row.  A lane then reads its rows' bytes of a step with one LDS read per row.
    // The registers hold the bytes as loaded; the shift for the lane's half is applied where they are used.
    const uint32_t lrow = lane & 31u, h = lane >> 5, hshift = 8u * h;
    constexpr uint32_t kBs = 4u * kScaleDw;  // scale bytes per row and K step
    const uint32_t steps = RB / kMxBK, last = steps - 1u, last_slot = last >> 1;
    const bool sc_is_a = wave < 4u;
    const uint8_t* sc_base = sc_is_a ? p.sa : p.sb;
    uint32_t sc_lane;  // the lane's row of scale bytes (m * sk and n * sk stay below 2^32)
    {
        uint32_t r = (sc_is_a ? row0 : n0) + (wave & 3u) * 64u + lane;
        const uint32_t lim = sc_is_a ? p.m : p.n;
        r = r < lim ? r : lim - 1u;
        sc_lane = r * p.sk;
    }
    auto slot_off = [&](uint32_t slot) {  // first of the 16 bytes loaded for a slot
        const uint32_t o = 2u * kBs * slot, cap = p.sk - 16u;
        return o < cap ? o : cap;
    };
    // slot: counted on past the end (it picks the buffer); the bytes are those of the last slot then
    auto issue_scales = [&](uint32_t slot) __attribute__((always_inline)) {
        const uint32_t data = slot < last_slot ? slot : last_slot;
        asm volatile("" : "+v"(sc_lane));
        __builtin_amdgcn_global_load_lds((gptr_t)(uniform(sc_base + slot_off(data)) + sc_lane),
                                         (lds_ptr_t)(SC + (slot & 1u) * kMxScaleBuf + wave * 1024u), 16, 0, 0);
    };
    struct Scales {
        uint32_t a[TI][kScaleDw], b[TJ][kScaleDw];
    };
    const uint32_t sc_va = (wm * (TI * 32u) + lrow) * 16u, sc_vb = kMxBM * 16u + (wn * (TJ * 32u) + lrow) * 16u;
    // the bytes of K step `step` (counted on past the end like the slot) from LDS into registers
    auto read_scales = [&](Scales& sc, uint32_t step) __attribute__((always_inline)) {
        const uint32_t slot = step >> 1, data = slot < last_slot ? slot : last_slot, st = step < last ? step : last;
        const uint32_t off = (slot & 1u) * kMxScaleBuf + kBs * st - slot_off(data);
        const char* pa = SC + sc_va + off;
        const char* pb = SC + sc_vb + off;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            if constexpr (kScaleDw == 2) {
                const u32x2 v = *reinterpret_cast<const u32x2*>(pa + i * 512);
                sc.a[i][0] = v[0];
                sc.a[i][1] = v[1];
            } else {
                sc.a[i][0] = *reinterpret_cast<const uint32_t*>(pa + i * 512);
            }
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            if constexpr (kScaleDw == 2) {
                const u32x2 v = *reinterpret_cast<const u32x2*>(pb + j * 512);
                sc.b[j][0] = v[0];
                sc.b[j][1] = v[1];
            } else {
                sc.b[j][0] = *reinterpret_cast<const uint32_t*>(pb + j * 512);
            }
        }
    };

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i) {
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        }
    }

    // ---- fragments: piece q of tile line r sits at r * 128 + ((q ^ ((r / 2) % 8)) * 16).  A lane reads piece
    // kPieceStep u + h (+ 2 for the upper registers of an 8-bit operand) of a line whose number is lrow + a multiple
    // of 32, i.e. at lrow * 128 + (((kPieceStep u) ^ (h ^ swizzle)) * 16) + constants: one register per u.
    // (6-bit operands, 24 bytes per lane: pieces 4 s + 2 h and the first half of 4 s + 2 h + 1, u = 2 s and 2 s + 1)
    constexpr int kPieceStep = 2;
    constexpr int kPieces = 4;   // u = 0 .. 3: pieces 0 2 4 6 (+ h)
    uint32_t foff[kPieces];
#pragma unroll
    for (int u = 0; u < kPieces; ++u) {
        const uint32_t piece = kSix ? 4u * (u >> 1) + 2u * h + (u & 1) : static_cast<uint32_t>(kPieceStep * u) ^ h;
        foff[u] = lrow * 128u + ((piece ^ ((lrow >> 1) & 7u)) << 4);
        if (kSix && (u & 1)) {
            foff[u] += 8u * (lrow & 1u);  // odd rows keep these 8 bytes in the piece's second half
        }
    }
    auto frag = [&](const char* S, uint32_t line0, int u) __attribute__((always_inline)) {
        return *reinterpret_cast<const i32x4*>(S + line0 * 128u + foff[u]);
    };
    struct Frags {
        v8i a[TI], b[TJ];
    };
    // the operands of sub-step s (64 k) of a stage
    auto load_frags = [&](Frags& f, const char* As, const char* Bs, int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const uint32_t line0 = (wm * TI + i) * 32u;  // (lines 32 apart share the swizzle of lrow)
            if constexpr (kFour) {
                const i32x4 lo = frag(As, line0, s);
                f.a[i] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, -1, -1, -1, -1);  // the instruction reads 4 registers of a 4-bit operand
            } else if constexpr (kSix) {
                const i32x4 lo = frag(As, line0, 2 * s);
                const i32x2_t hi = *reinterpret_cast<const i32x2_t*>(As + line0 * 128u + foff[2 * s + 1]);
                v8i t = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, -1, -1, -1, -1);  // the instruction reads 6 registers
                t[4] = hi[0];
                t[5] = hi[1];
                f.a[i] = t;
            } else {
                const i32x4 lo = frag(As, line0, 2 * s), hi = frag(As, line0, 2 * s + 1);
                f.a[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const uint32_t line0 = (wn * TJ + j) * 32u;
            if constexpr (kFour) {
                const i32x4 lo = frag(Bs, line0, s);
                f.b[j] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, -1, -1, -1, -1);
            } else if constexpr (kSix) {
                const i32x4 lo = frag(Bs, line0, 2 * s);
                const i32x2_t hi = *reinterpret_cast<const i32x2_t*>(Bs + line0 * 128u + foff[2 * s + 1]);
                v8i t = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, -1, -1, -1, -1);  // the instruction reads 6 registers
                t[4] = hi[0];
                t[5] = hi[1];
                f.b[j] = t;
            } else {
                const i32x4 lo = frag(Bs, line0, 2 * s), hi = frag(Bs, line0, 2 * s + 1);
                f.b[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
    };
    // the 8 matrix instructions of sub-step s: scale byte 2 s (+ the lane's half, shifted in) of the step's bytes
    auto mfmas = [&](const Frags& f, const Scales& sc, auto sub) __attribute__((always_inline)) {
        constexpr int s = decltype(sub)::value;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    f.a[i], f.b[j], acc[i][j], kCa, kCb, (s & 1) ? 2 : 0, static_cast<int>(sc.a[i][s >> 1] >> hshift),
                    (s & 1) ? 2 : 0, static_cast<int>(sc.b[j][s >> 1] >> hshift));
            }
        }
    };

    // ---- main loop: the loads of step s + 1 (tiles and, every second step, scale bytes, all direct to LDS) run under
    // the arithmetic of step s; one wait and one barrier per step (the next stage has landed, and everyone has left
    // the stage that the step after next will overwrite).  Behind the barrier a wavefront first reads the next
    // step's scale bytes from LDS, then issues the loads: a load into the scale buffers ahead of those reads would
    // make the compiler wait for it, and with it for the tile loads, before the reads.
    Scales s0, s1;
    Frags f;
    // Nothing between the instructions of a step is conditional (a branch there makes the compiler shuffle the
    // accumulators): past the end the loads repeat the last step's, into a stage and buffers nobody reads again.
    auto next_step = [&](uint32_t s) { return s + 2u < last ? s + 2u : last; };
    issue(0, A0, B0);
    issue_scales(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_scales(s0, 0);
    issue((steps > 1u ? 1u : 0u) * kMxBK, A1, B1);  // a single step is loaded twice: stage 1 is then never read
    if constexpr (kFour) {
        // 4-bit operands are 24 registers a set: two sets.  The LDS reads of a sub-step are spread behind the first
        // matrix instructions of the sub-step before (scheduling groups: one instruction, two reads, ...), so that the
        // LDS works while the matrix pipe does; the first operands of the next step, whose stage has landed, are read
        // behind the barrier under this step's last instructions.
        Frags g;
        auto interleave = [&]() __attribute__((always_inline)) {
            constexpr int kReads = TI + TJ, kMfmas = TI * TJ, kPer = 2;
            mx_static_for<kMfmas>([&](auto n) {
                constexpr int kLeft = kReads - decltype(n)::value * kPer;
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (kLeft > 0) {
                    __builtin_amdgcn_sched_group_barrier(0x100, kLeft < kPer ? kLeft : kPer, 0);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        };
        load_frags(f, A0, B0, 0);
        // step s in stage x; `even` steps also load the scale bytes of the slot after the next
        auto step2 = [&](char* Ax, char* Bx, const char* Ay, const char* By, const Scales& sc, Scales& sc_next, uint32_t s,
                         auto even) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < kPieces; ++u) asm volatile("" : "+v"(foff[u]));
            load_frags(g, Ax, Bx, 1);
            mfmas(f, sc, std::integral_constant<int, 0>{});
            interleave();
            load_frags(f, Ax, Bx, 2);
            mfmas(g, sc, std::integral_constant<int, 1>{});
            interleave();
            load_frags(g, Ax, Bx, 3);
            mfmas(f, sc, std::integral_constant<int, 2>{});
            interleave();
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
            read_scales(sc_next, s + 1u);
            __builtin_amdgcn_sched_barrier(0);
            issue(next_step(s) * kMxBK, Ax, Bx);
            if constexpr (decltype(even)::value) {
                issue_scales((s >> 1) + 1u);
            }
            load_frags(f, Ay, By, 0);
            mfmas(g, sc, std::integral_constant<int, 3>{});
            interleave();
        };
        // Steps in pairs, an odd last one behind the loop: with a second half that can be skipped inside the loop the
        // compiler sees a path on which the tile loads of the first half are the newest at the loop's top, and
        // waits there for all loads before the first LDS reads of every pass.
        uint32_t s = 0;
        for (; s + 1u < steps; s += 2) {
            step2(A0, B0, A1, B1, s0, s1, s, std::true_type{});
            step2(A1, B1, A0, B0, s1, s0, s + 1u, std::false_type{});
        }
        if (s < steps) {
            step2(A0, B0, A1, B1, s0, s1, s, std::true_type{});
        }
    } else {
        // A K step: all sub-steps but the last, then the last one's operands into registers, then the wait and the
        // barrier, and only then the last sub-step's instructions: behind the barrier the matrix pipe has work at once.
        auto step = [&](char* Ax, char* Bx, const Scales& sc, Scales& sc_next, uint32_t s, auto even) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < kPieces; ++u) asm volatile("" : "+v"(foff[u]));
            mx_static_for<kSub - 1>([&](auto sub) {
                load_frags(f, Ax, Bx, decltype(sub)::value);
                mfmas(f, sc, sub);
            });
            load_frags(f, Ax, Bx, kSub - 1);
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
            read_scales(sc_next, s + 1u);
            __builtin_amdgcn_sched_barrier(0);
            issue(next_step(s) * kMxBK, Ax, Bx);
            if constexpr (decltype(even)::value) {
                issue_scales((s >> 1) + 1u);
            }
            mfmas(f, sc, std::integral_constant<int, kSub - 1>{});
        };
        uint32_t s = 0;
        for (; s + 1u < steps; s += 2) {
            step(A0, B0, s0, s1, s, std::true_type{});
            step(A1, B1, s1, s0, s + 1u, std::false_type{});
        }
        if (s < steps) {
            step(A0, B0, s0, s1, s, std::true_type{});
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the repeated loads of the last steps

    // ---- register r of lane l in a 32 x 32 block: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
    float bias[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const uint32_t col = n0 + (wn * TJ + j) * 32u + lrow;
        bias[j] = (p.bias != nullptr && col < p.n) ? p.bias[col] : 0.0f;
    }
    if (p.out_dtype != ASCQ_F32 && p.n % 2u == 0) {
        // 16-bit outputs: after one swap between neighbouring lanes the even lane holds columns (l, l + 1) of the
        // wavefront's first block of 32 and the odd lane columns (l - 1, l) of the second: one dword store per lane,
        // and the 32 lanes of a row write one full 128-byte line
        const bool odd = (lane & 1u) != 0;
        const bool bf = p.out_dtype == ASCQ_BF16;
        const uint32_t colw = n0 + wn * (TJ * 32u);
        const uint32_t col = odd ? colw + 32u + (lrow - 1u) : colw + lrow;  // first column of the lane's pair
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = row0 + (wm * TI + i) * 32u + 8u * (r >> 2) + 4u * h + (r & 3);
                const float v0 = acc[i][0][r] + bias[0], v1 = acc[i][1][r] + bias[1];
                const uint32_t h0 = bf ? f32_to_bf16_bits(v0) : f32_to_half_bits_sat(v0);
                const uint32_t h1 = bf ? f32_to_bf16_bits(v1) : f32_to_half_bits_sat(v1);
                const uint32_t recv = static_cast<uint32_t>(
                    __builtin_amdgcn_mov_dpp(static_cast<int>(odd ? h0 : h1), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                const uint32_t word = odd ? (recv | (h1 << 16)) : (h0 | (recv << 16));
                if (row < p.m && col < p.n) {
                    __builtin_nontemporal_store(word, reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(p.c) +
                                                                                  static_cast<size_t>(row) * p.n + col));
                }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const uint32_t col = n0 + (wn * TJ + j) * 32u + lrow;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = row0 + (wm * TI + i) * 32u + 8u * (r >> 2) + 4u * h + (r & 3);
                if (row < p.m && col < p.n) {
                    mx_store(p, static_cast<size_t>(row) * p.n + col, acc[i][j][r] + bias[j]);
                }
            }
        }
    }
}

// value of an operand element: 8-bit formats by the hardware conversions (exact), 4-bit ones by their tables
__device__ __forceinline__ float mx_value(const uint8_t* row, uint32_t k, int fmt)
{
    if (fmt == ASCQ_QDST_FP8_E4M3FN) {
        return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(row[k]), 0);
    }
    if (fmt == ASCQ_QDST_FP8_E5M2) {
        return __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(row[k]), 0);
    }
    const uint32_t code = (row[k >> 1] >> (4u * (k & 1u))) & 15u;
    const uint32_t mag = code & 7u;
    float v;
    if (fmt == ASCQ_QDST_FP4_E2M1) {
        v = mag < 2u ? 0.5f * static_cast<float>(mag) : static_cast<float>(2u + (mag & 1u)) * static_cast<float>(1u << ((mag >> 1) - 1u)) * 0.5f;
    } else {
        v = 0.25f * static_cast<float>(mag);
    }
    return (code & 8u) ? -v : v;
}

__device__ __forceinline__ float e8m0_value(uint8_t e)
{
    // 2^(e - 127); e = 0 is 2^-127 (a subnormal float), e = 255 (NaN in the format) is passed on as NaN
    return e == 255u ? __uint_as_float(0x7FC00000u) : (e == 0u ? __uint_as_float(0x00400000u) : __uint_as_float(static_cast<uint32_t>(e) << 23));
}

// One lane per output element; the sum of a block of 32 k is formed in fp32, scaled, and added to the total.
__global__ __launch_bounds__(256) void mx_elementwise_kernel(MxParams p, uint32_t a_row_bytes, uint32_t b_row_bytes)
{
    const size_t total = static_cast<size_t>(p.m) * p.n;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * 256u) {
        const uint32_t i = static_cast<uint32_t>(idx / p.n), j = static_cast<uint32_t>(idx % p.n);
        const uint8_t* ar = p.a + static_cast<size_t>(i) * a_row_bytes;
        const uint8_t* br = p.b + static_cast<size_t>(j) * b_row_bytes;
        float sum = 0.0f;
        for (uint32_t k0 = 0; k0 < p.k; k0 += 32u) {
            const uint32_t k1 = k0 + 32u < p.k ? k0 + 32u : p.k;
            float part = 0.0f;
            for (uint32_t k = k0; k < k1; ++k) {
                part = __builtin_fmaf(mx_value(ar, k, p.a_format), mx_value(br, k, p.b_format), part);
            }
            const float sc = e8m0_value(p.sa[static_cast<size_t>(i) * p.sk + (k0 >> 5)]) * e8m0_value(p.sb[static_cast<size_t>(j) * p.sk + (k0 >> 5)]);
            sum = __builtin_fmaf(part, sc, sum);
        }
        if (p.bias != nullptr) {
            sum += p.bias[j];
        }
        mx_store(p, idx, sum);
    }
}

// fp4 [rows, k / 2 bytes] -> e4m3 [rows, k bytes]; every fp4 value of either format is an e4m3 value.
// e2m1 magnitudes 0 .5 1 1.5 2 3 4 6 and e1m2 magnitudes 0 .25 .. 1.75 as e4m3 codes (bias 7, 3 mantissa bits)
__global__ __launch_bounds__(256) void mx_widen_fp4_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                           size_t pieces, int fmt)
{
    // the eight magnitudes' e4m3 codes as a byte table in two registers: a byte permute looks four nibbles up at once
    const uint64_t lut = fmt == ASCQ_QDST_FP4_E2M1 ? 0x4C4844403C383000ull : 0x3E3C3A3834302800ull;
    const uint32_t lut_lo = static_cast<uint32_t>(lut), lut_hi = static_cast<uint32_t>(lut >> 32);
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; i < pieces; i += static_cast<size_t>(gridDim.x) * 256u) {
        const u32x4 q = __builtin_nontemporal_load(src + i);  // 32 values
        u32x4 out[2];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t e = q[d] & 0x0F0F0F0Fu, o = (q[d] >> 4) & 0x0F0F0F0Fu;  // values 0 2 4 6 / 1 3 5 7 of the dword
            const uint32_t ve = __builtin_amdgcn_perm(lut_hi, lut_lo, e & 0x07070707u) | ((e & 0x08080808u) << 4);
            const uint32_t vo = __builtin_amdgcn_perm(lut_hi, lut_lo, o & 0x07070707u) | ((o & 0x08080808u) << 4);
            out[d >> 1][2 * (d & 1)] = __builtin_amdgcn_perm(vo, ve, 0x05010400u);      // values 0 1 2 3
            out[d >> 1][2 * (d & 1) + 1] = __builtin_amdgcn_perm(vo, ve, 0x07030602u);  // values 4 5 6 7
        }
        dst[2 * i] = out[0];
        dst[2 * i + 1] = out[1];
    }
}

// e1m2 [rows, k / 2 bytes] -> e2m3 codes, 32 values as 24 bytes (little-endian 6-bit fields, the layout the matrix
// instruction reads from a lane's six registers) followed by 8 unused bytes, so that a row is k bytes like an 8-bit
// operand's.  An e1m2 value is +-(code / 4), code 0 .. 7, which is the e2m3 value with magnitude bits 2 * code (its
// subnormals run 0, 1/8 .. 7/8 and its first binade 1, 9/8 .. 15/8).
// The last 8 of the 24 bytes sit in the first half of the second 16-byte piece in even rows and in its second half in
// odd rows: an 8-byte LDS read is served 16 lanes at a time, a row and its neighbour keep their pieces at the same
// position of their 128-byte lines, and the two would meet in the same banks.
__global__ __launch_bounds__(256) void mx_widen_e1m2_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                            size_t pieces, uint32_t pieces_per_row)
{
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x; i < pieces; i += static_cast<size_t>(gridDim.x) * 256u) {
        const u32x4 q = __builtin_nontemporal_load(src + i);  // 32 values, value v of a dword in bits 4 v .. 4 v + 3
        uint64_t c[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint64_t t = q[d];
            t = (t & 0xFFFFull) | ((t & 0xFFFF0000ull) << 8);                              // values 0-3 | 4-7, 24 bits each
            t = (t & 0x00000000FF0000FFull) | ((t & 0x000000FF0000FF00ull) << 4);          // pairs, 12 bits each
            t = (t & 0x00000F00F00F00Full) | ((t & 0x0000F00F00F00F0ull) << 2);            // value v in bits 6 v .. 6 v + 3
            c[d] = ((t & 0x0000208208208208ull) << 2) | ((t & 0x00001C71C71C71C7ull) << 1);  // sign to bit 5, magnitude doubled
        }
        const u32x4 lo = {static_cast<uint32_t>(c[0]), static_cast<uint32_t>(c[0] >> 32) | (static_cast<uint32_t>(c[1]) << 16),
                          static_cast<uint32_t>(c[1] >> 16), static_cast<uint32_t>(c[2])};
        const uint32_t w4 = static_cast<uint32_t>(c[2] >> 32) | (static_cast<uint32_t>(c[3]) << 16);
        const uint32_t w5 = static_cast<uint32_t>(c[3] >> 16);
        const bool upper = ((i / pieces_per_row) & 1u) != 0;
        dst[2 * i] = lo;
        dst[2 * i + 1] = upper ? u32x4{0u, 0u, w4, w5} : u32x4{w4, w5, 0u, 0u};
    }
}

inline bool is_fp8(int f) { return f == ASCQ_QDST_FP8_E4M3FN || f == ASCQ_QDST_FP8_E5M2; }
inline bool is_fp4(int f) { return f == ASCQ_QDST_FP4_E2M1 || f == ASCQ_QDST_FP4_E1M2; }

// which operands the tile path widens to e4m3 first: a 4-bit operand unless both are e2m1
inline void mx_widen_plan(const ascq_mx_desc* d, bool& widen_a, bool& widen_b)
{
    const bool both_e2m1 = d->a_format == ASCQ_QDST_FP4_E2M1 && d->b_format == ASCQ_QDST_FP4_E2M1;
    widen_a = is_fp4(d->a_format) && !both_e2m1;
    widen_b = is_fp4(d->b_format) && !both_e2m1;
}

inline bool mx_tile_shape_ok(const ascq_mx_desc* d)
{
    bool wa, wb;
    mx_widen_plan(d, wa, wb);
    const bool four = is_fp4(d->a_format) && !wa;  // both e2m1
    return d->k % (four ? 256u : 128u) == 0 && d->scale_k % 8u == 0 && d->scale_k >= 16u && d->m >= 64u && d->n >= 64u;
}

int mx_validate(const ascq_mx_desc* d, const char* who)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "%s: desc is NULL", who);
    ASCQ_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0, ASCQ_EINVAL, "%s: m, n, k must be greater than 0", who);
    ASCQ_REQUIRE((is_fp8(d->a_format) || is_fp4(d->a_format)) && (is_fp8(d->b_format) || is_fp4(d->b_format)), ASCQ_EINVAL,
                 "%s: a_format / b_format must be one of FP8_E4M3FN, FP8_E5M2, FP4_E2M1, FP4_E1M2", who);
    ASCQ_REQUIRE(!(is_fp4(d->a_format) || is_fp4(d->b_format)) || d->k % 2u == 0, ASCQ_EINVAL,
                 "%s: k %u must be even for a 4-bit operand (two values per byte)", who, d->k);
    ASCQ_REQUIRE(d->scale_k >= (d->k + 31u) / 32u, ASCQ_EINVAL, "%s: scale_k %u is less than ceil(k / 32) = %u", who,
                 d->scale_k, (d->k + 31u) / 32u);
    ASCQ_REQUIRE(d->out_dtype == ASCQ_F32 || d->out_dtype == ASCQ_BF16 || d->out_dtype == ASCQ_F16, ASCQ_EINVAL,
                 "%s: out_dtype must be F32, BF16 or F16", who);
    return ASCQ_OK;
}

}  // namespace
}  // namespace ascq

using namespace ascq;

extern "C" int ascq_matmul_mx_workspace_size(const ascq_mx_desc* d, size_t* bytes)
{
    ASCQ_REQUIRE(bytes != nullptr, ASCQ_ENULL, "ascq_matmul_mx_workspace_size: bytes is NULL");
    const int rc = mx_validate(d, "ascq_matmul_mx_workspace_size");
    if (rc != ASCQ_OK) {
        return rc;
    }
    *bytes = 0;
    bool wa, wb;
    mx_widen_plan(d, wa, wb);
    if ((wa || wb) && mx_tile_shape_ok(d)) {
        *bytes = (wa ? static_cast<size_t>(d->m) * d->k : 0u) + (wb ? static_cast<size_t>(d->n) * d->k : 0u);
    }
    return ASCQ_OK;
}

// ref: include/basic_api/kernel_operator_mm_intf.h:321-340 (MmadMx); golden: examples/01_simd_cpp_api/03_basic_api/
// 03_matrix_compute/mmad_mx/scripts/gen_data.py:52-140
extern "C" int ascq_matmul_mx(const ascq_mx_desc* d, void* c, const void* a, const void* b, const void* a_scale,
                              const void* b_scale, const void* bias, void* workspace, size_t workspace_bytes, void* stream)
{
    const int rc = mx_validate(d, "ascq_matmul_mx");
    if (rc != ASCQ_OK) {
        return rc;
    }
    ASCQ_REQUIRE(c && a && b && a_scale && b_scale, ASCQ_ENULL, "ascq_matmul_mx: c / a / b / a_scale / b_scale is NULL");
    ASCQ_REQUIRE(!d->has_bias || bias, ASCQ_ENULL, "ascq_matmul_mx: bias is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    MxParams p{};
    p.a = static_cast<const uint8_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.sa = static_cast<const uint8_t*>(a_scale);
    p.sb = static_cast<const uint8_t*>(b_scale);
    p.bias = d->has_bias ? static_cast<const float*>(bias) : nullptr;
    p.c = c;
    p.m = d->m;
    p.n = d->n;
    p.k = d->k;
    p.sk = d->scale_k;
    p.a_format = d->a_format;
    p.b_format = d->b_format;
    p.out_dtype = d->out_dtype;

    bool wa, wb;
    mx_widen_plan(d, wa, wb);
    const size_t need = (wa ? static_cast<size_t>(d->m) * d->k : 0u) + (wb ? static_cast<size_t>(d->n) * d->k : 0u);
    const bool tile = mx_tile_shape_ok(d) && aligned16(a) && aligned16(b) && (reinterpret_cast<uintptr_t>(a_scale) & 7u) == 0 &&
                      (reinterpret_cast<uintptr_t>(b_scale) & 7u) == 0 &&
                      (need == 0 || (workspace != nullptr && workspace_bytes >= need && aligned16(workspace)));
    if (!tile) {
        const uint32_t arb = is_fp4(d->a_format) ? d->k / 2u : d->k, brb = is_fp4(d->b_format) ? d->k / 2u : d->k;
        size_t blocks = (static_cast<size_t>(d->m) * d->n + 255u) / 256u;
        if (blocks > 65536u) blocks = 65536u;
        mx_elementwise_kernel<<<static_cast<uint32_t>(blocks), 256, 0, st>>>(p, arb, brb);
        return launch_status("ascq_matmul_mx (element-wise)");
    }
    int fa = d->a_format, fb = d->b_format;
    // two e1m2 operands become e2m3 codes, which the matrix core runs at the 4-bit rate; any other 4-bit operand e4m3
    const bool six = fa == ASCQ_QDST_FP4_E1M2 && fb == ASCQ_QDST_FP4_E1M2;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    auto widen = [&](const uint8_t*& src, int& fmt, size_t rows) {
        const size_t pieces = rows * (d->k / 2u) / 16u;  // k is a multiple of 128 here
        size_t blocks = (pieces + 255u) / 256u;
        if (blocks > 65536u) blocks = 65536u;
        if (six) {
            mx_widen_e1m2_kernel<<<static_cast<uint32_t>(blocks), 256, 0, st>>>(reinterpret_cast<const u32x4*>(src),
                                                                               reinterpret_cast<u32x4*>(ws), pieces, d->k / 32u);
        } else {
            mx_widen_fp4_kernel<<<static_cast<uint32_t>(blocks), 256, 0, st>>>(reinterpret_cast<const u32x4*>(src),
                                                                              reinterpret_cast<u32x4*>(ws), pieces, fmt);
        }
        src = ws;
        ws += rows * d->k;
        fmt = ASCQ_QDST_FP8_E4M3FN;
    };
    if (wa) {
        widen(p.a, fa, d->m);
    }
    if (wb) {
        widen(p.b, fb, d->n);
    }
    const bool four = is_fp4(fa);  // (after the widening: both e2m1)
    p.row_bytes = four ? d->k / 2u : d->k;
    p.tiles_m = (d->m + kMxBM - 1u) / kMxBM;
    p.tiles_n = (d->n + kMxBN - 1u) / kMxBN;
    const uint32_t grid = (p.tiles_m * p.tiles_n + 7u) / 8u * 8u;
    if (four) {
        mx_tile_kernel<true, 4, 4><<<grid, kMxThreads, 0, st>>>(p);
    } else if (six) {
        mx_tile_kernel<false, 2, 2><<<grid, kMxThreads, 0, st>>>(p);
    } else if (fa == ASCQ_QDST_FP8_E4M3FN && fb == ASCQ_QDST_FP8_E4M3FN) {
        mx_tile_kernel<false, 0, 0><<<grid, kMxThreads, 0, st>>>(p);
    } else if (fa == ASCQ_QDST_FP8_E4M3FN) {
        mx_tile_kernel<false, 0, 1><<<grid, kMxThreads, 0, st>>>(p);
    } else if (fb == ASCQ_QDST_FP8_E4M3FN) {
        mx_tile_kernel<false, 1, 0><<<grid, kMxThreads, 0, st>>>(p);
    } else {
        mx_tile_kernel<false, 1, 1><<<grid, kMxThreads, 0, st>>>(p);
    }
    return launch_status("ascq_matmul_mx");
}
