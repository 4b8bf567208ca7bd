// Machine ceilings the kernels of libascq are read against, measured on the GPU this program runs on and printed as
// one JSON object on stdout:
//   * int8 matrix-pipe rate of a register-resident loop of v_mfma_i32_32x32x32_i8 with constant operands and with
//     random int8 operands (same instruction stream: the difference is the clock the power management allows);
//   * the shader clock during each of those loops, from the ratio of the shader-clock counter to the constant
//     100 MHz real-time counter read inside the kernel;
//   * device-to-device copy, read-only sweep and write-only fill of 1 GiB (HBM bandwidth actually reachable);
//   * LDS read bandwidth per compute unit with 16-byte reads;
//   * a small streaming job, 2048 workgroups that each read one 8 KiB row and write 4 KiB (16 MiB in, 8 MiB out, the
//     same buffers every launch): what launch, ramp-up and drain cost a kernel of that size whatever it computes;
//     and the same job on rows that no cache holds.
// Every figure is the mean of the second half of `reps` back-to-back launches (the first half brings the clocks to
// their sustained state).  No input, no dependence on libascq.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                              \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) {                                                            \
            fprintf(stderr, "machine_probe: %s (line %d)\n", hipGetErrorString(e_), __LINE__); \
            return 1;                                                                      \
        }                                                                                  \
    } while (0)

// 16 independent 32x32 accumulators, 4 + 4 operand fragments held in registers: the MFMA stream of a 128 x 128
// register tile without any loads.  clk[0] / clk[1] receive shader-clock and real-time ticks of workgroup 0.
__global__ __launch_bounds__(256) void mfma_loop(int* out, const i32x4* in, int iters, unsigned long long* clk)
{
    i32x16 acc[4][4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    i32x4 af[4], bf[4];
    for (int i = 0; i < 4; ++i) {
        af[i] = in[threadIdx.x + 256 * i];
        bf[i] = in[threadIdx.x + 256 * (i + 4)];
    }
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    int s = 0;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = c1 - c0;
        clk[1] = r1 - r0;
    }
}

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ b, size_t n)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) b[i] = a[i];
}

__global__ __launch_bounds__(256) void read_kernel(const u32x4* __restrict__ a, int* out, size_t n)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    unsigned s = 0;
    for (; i + 3 * stride < n; i += 4 * stride) {
        const u32x4 v0 = __builtin_nontemporal_load(a + i), v1 = __builtin_nontemporal_load(a + i + stride),
                    v2 = __builtin_nontemporal_load(a + i + 2 * stride), v3 = __builtin_nontemporal_load(a + i + 3 * stride);
        s += v0.x ^ v1.y ^ v2.z ^ v3.w;
    }
    if (s == 0x12345678u) out[0] = static_cast<int>(s);
}

__global__ __launch_bounds__(256) void fill_kernel(u32x4* __restrict__ b, size_t n)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    const u32x4 v = {1, 2, 3, 4};
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) __builtin_nontemporal_store(v, b + i);
}

// 8 x 16-byte LDS reads per lane and iteration, rows of 128 bytes with the XOR swizzle of the GEMM's A tile.  The reads
// and the wait for them are one asm statement, so the compiler never sees a register whose load is still in flight.
// One workgroup per row of 8 KiB: two 16-byte loads per lane, the even bytes of each stored as 8 bytes.
__global__ __launch_bounds__(256) void row_2to1_kernel(const u32x4* __restrict__ a, unsigned long long* __restrict__ b)
{
    const size_t base = static_cast<size_t>(blockIdx.x) * 512;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const u32x4 v = a[base + k * 256 + threadIdx.x];
        const unsigned lo = __builtin_amdgcn_perm(v[1], v[0], 0x06040200u);
        const unsigned hi = __builtin_amdgcn_perm(v[3], v[2], 0x06040200u);
        b[base + k * 256 + threadIdx.x] = (static_cast<unsigned long long>(hi) << 32) | lo;
    }
}

__global__ __launch_bounds__(256) void lds_read_loop(int* out, int iters)
{
    __shared__ __attribute__((aligned(16))) char smem[65536];
    for (int i = threadIdx.x; i < 65536 / 4; i += 256) reinterpret_cast<int*>(smem)[i] = i;
    __syncthreads();
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned row = (lane & 31) + wave * 32, piece = lane >> 5;
    unsigned base[4];
    for (int u = 0; u < 4; ++u) {
        base[u] = static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)) + row * 128 + (((piece + 2 * u) ^ ((row >> 1) & 7)) << 4);
    }
    i32x4 s = {0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
        i32x4 v0, v1, v2, v3, v4, v5, v6, v7;
        asm volatile(
            "ds_read_b128 %0, %8\n ds_read_b128 %1, %9\n ds_read_b128 %2, %10\n ds_read_b128 %3, %11\n"
            "ds_read_b128 %4, %8 offset:16384\n ds_read_b128 %5, %9 offset:16384\n ds_read_b128 %6, %10 offset:16384\n"
            "ds_read_b128 %7, %11 offset:16384\n s_waitcnt lgkmcnt(0)"
            : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6), "=&v"(v7)
            : "v"(base[0]), "v"(base[1]), "v"(base[2]), "v"(base[3])
            : "memory");
        s += v0 ^ v1 ^ v2 ^ v3 ^ v4 ^ v5 ^ v6 ^ v7;
    }
    out[blockIdx.x * 256 + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

int main()
{
    int dev = 0;
    CK(hipSetDevice(dev));
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, dev));
    int wall_khz = 0, clock_khz = 0;
    CK(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, dev));
    CK(hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeClockRate, dev));
    const int cus = prop.multiProcessorCount;
    int* out;
    CK(hipMalloc(&out, 4096 * 256 * 4));
    i32x4* in;
    CK(hipMalloc(&in, 256 * 8 * 16));
    unsigned long long* clk;
    CK(hipMalloc(&clk, 16));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int reps = 24;
    float ms = 0;

    printf("{\"device\": \"%s\", \"gcn_arch\": \"%s\", \"compute_units\": %d, \"max_clock_mhz\": %d", prop.name,
           prop.gcnArchName, cus, clock_khz / 1000);

    // ---- MFMA loops: constant operands, then random int8 operands
    const int iters = 4000, blocks = cus * 4;  // one workgroup of four wavefronts per SIMD quadruple, four per CU
    for (int mode = 0; mode < 2; ++mode) {
        std::vector<int> h(256 * 8 * 4);
        srand(3);
        for (auto& v : h) v = mode == 0 ? 0x01010101 : (rand() ^ (rand() << 16));
        CK(hipMemcpy(in, h.data(), h.size() * 4, hipMemcpyHostToDevice));
        for (int r = 0; r < reps / 2; ++r) mfma_loop<<<blocks, 256>>>(out, in, iters, clk);
        CK(hipEventRecord(e0));
        for (int r = 0; r < reps / 2; ++r) mfma_loop<<<blocks, 256>>>(out, in, iters, clk);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        CK(hipEventElapsedTime(&ms, e0, e1));
        unsigned long long hc[2];
        CK(hipMemcpy(hc, clk, 16, hipMemcpyDeviceToHost));
        const double ops = 2.0 * 32 * 32 * 32 * 16.0 * iters * 4 * blocks * (reps / 2);
        const double shader_mhz = hc[1] ? static_cast<double>(hc[0]) / static_cast<double>(hc[1]) * (wall_khz / 1000.0) : 0.0;
        printf(", \"mfma_i8_%s_tops\": %.1f, \"mfma_i8_%s_shader_counter_mhz\": %.0f", mode == 0 ? "constant" : "random",
               ops / (ms * 1e-3) / 1e12, mode == 0 ? "constant" : "random", shader_mhz);
    }

    // ---- HBM: 1 GiB copy, read sweep, fill
    const size_t n = static_cast<size_t>(1) << 30;
    u32x4 *a, *b;
    CK(hipMalloc(&a, n));
    CK(hipMalloc(&b, n));
    CK(hipMemset(a, 1, n));
    const int gb = cus * 32;
    for (int r = 0; r < 4; ++r) copy_kernel<<<gb, 256>>>(a, b, n / 16);
    CK(hipEventRecord(e0));
    for (int r = 0; r < 8; ++r) copy_kernel<<<gb, 256>>>(a, b, n / 16);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"copy_1gib_gbs\": %.0f", 2.0 * n * 8 / (ms * 1e-3) / 1e9);
    for (int r = 0; r < 4; ++r) read_kernel<<<gb, 256>>>(a, out, n / 16);
    CK(hipEventRecord(e0));
    for (int r = 0; r < 8; ++r) read_kernel<<<gb, 256>>>(a, out, n / 16);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"read_1gib_gbs\": %.0f", 1.0 * n * 8 / (ms * 1e-3) / 1e9);
    for (int r = 0; r < 4; ++r) fill_kernel<<<gb, 256>>>(b, n / 16);
    CK(hipEventRecord(e0));
    for (int r = 0; r < 8; ++r) fill_kernel<<<gb, 256>>>(b, n / 16);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"fill_1gib_gbs\": %.0f", 1.0 * n * 8 / (ms * 1e-3) / 1e9);

    // ---- LDS reads
    const int lds_iters = 4000;
    for (int r = 0; r < 4; ++r) lds_read_loop<<<cus * 4, 256>>>(out, lds_iters);
    CK(hipEventRecord(e0));
    for (int r = 0; r < 8; ++r) lds_read_loop<<<cus * 4, 256>>>(out, lds_iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double lds_bytes = 16.0 * 256 * 8 * lds_iters * cus * 4 * 8;
    printf(", \"lds_read_bytes_per_clock_per_cu_at_max_clock\": %.0f",
           lds_bytes / (ms * 1e-3) / (clock_khz * 1e3) / cus);

    // ---- a 24 MiB streaming job
    for (int r = 0; r < 100; ++r) row_2to1_kernel<<<2048, 256>>>(a, reinterpret_cast<unsigned long long*>(b));
    CK(hipEventRecord(e0));
    for (int r = 0; r < 400; ++r) row_2to1_kernel<<<2048, 256>>>(a, reinterpret_cast<unsigned long long*>(b));
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"rows_2048x8kib_read_4kib_written_us\": %.2f", ms * 1e3 / 400);
    // the same job on fresh rows every launch (32 positions of the 1 GiB buffers in turn: 512 MiB in, 256 MiB out,
    // more than the caches hold), as a kernel meets them whose input another kernel produced some launches earlier
    const size_t step_a = static_cast<size_t>(2048) * 512, step_b = step_a / 2;  // in u32x4
    for (int r = 0; r < 100; ++r) {
        row_2to1_kernel<<<2048, 256>>>(a + (r % 32) * step_a, reinterpret_cast<unsigned long long*>(b + (r % 32) * step_b));
    }
    CK(hipEventRecord(e0));
    for (int r = 0; r < 400; ++r) {
        row_2to1_kernel<<<2048, 256>>>(a + (r % 32) * step_a, reinterpret_cast<unsigned long long*>(b + (r % 32) * step_b));
    }
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"rows_2048x8kib_fresh_rows_us\": %.2f}\n", ms * 1e3 / 400);
    return 0;
}
