// Drives the HIP library through the C++ host mirror (include/ascq_ascendc.hpp) the way a reference user drives
// AscendC::AscendQuant / AscendDequant / AscendAntiQuant / Matmul (int8 and anti-quant), and compares every result
// bit-for-bit with the CPU oracle.  Host code only: device memory comes from the HIP runtime, the kernels from libascq.so.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/ascq_ascendc.hpp"
#include "../../oracle/ascq_oracle.h"
#include "../splitmix64.h"

namespace {

int g_failed = 0;

#define HIP_OK(expr)                                                                    \
    do {                                                                                \
        hipError_t e_ = (expr);                                                         \
        if (e_ != hipSuccess) {                                                         \
            std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));      \
            std::exit(2);                                                               \
        }                                                                               \
    } while (0)

struct Rng {  // the generator shared with the Python tests (tests/splitmix64.h)
    splitmix64 g;
    explicit Rng(uint64_t seed) : g{seed} {}
    uint64_t next() { return splitmix64_next(&g); }
    float uniform(float lo, float hi) { return splitmix64_uniform(&g, lo, hi); }
    int integer(int lo, int hi) { return splitmix64_integer(&g, lo, hi); }
};

template <typename T>
class DeviceBuffer {
public:
    explicit DeviceBuffer(size_t count) : count_(count) { HIP_OK(hipMalloc(&ptr_, count * sizeof(T) + 16)); }
    DeviceBuffer(const std::vector<T>& host) : DeviceBuffer(host.size())
    {
        HIP_OK(hipMemcpy(ptr_, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
    }
    ~DeviceBuffer() { (void)hipFree(ptr_); }
    template <typename U>
    ascq::DeviceTensor<U> view(uint32_t size) const
    {
        return ascq::DeviceTensor<U>(static_cast<U*>(ptr_), size);
    }
    void* ptr() const { return ptr_; }
    std::vector<T> download() const
    {
        std::vector<T> h(count_);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(h.data(), ptr_, count_ * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }

private:
    void* ptr_ = nullptr;
    size_t count_;
};

template <typename T>
void expect_equal(const char* what, const std::vector<T>& got, const std::vector<T>& want)
{
    size_t bad = 0;
    for (size_t i = 0; i < want.size(); ++i) bad += got[i] != want[i];
    std::printf("[%s] %s: %zu of %zu elements differ\n", bad ? "FAIL" : " ok ", what, bad, want.size());
    std::fflush(stdout);
    g_failed += bad != 0;
}

std::vector<uint16_t> random_halves(Rng& r, size_t n, float lo, float hi)
{
    std::vector<uint16_t> v(n);
    for (auto& e : v) e = orc_f32_to_f16(r.uniform(lo, hi));
    return v;
}

// The first case's inputs and, with a GPU, its output as checksums: tests/test_gpu_cpp_host.py draws the same inputs
// with the Python generator, runs the same operator through the Python mirror and must arrive at the same numbers.
void test_quant_per_channel(bool inputs_only)
{
    std::printf("[case] AscendQuant<half> per channel 64x256\n");
    Rng r{1};
    const uint32_t m = 64, n = 256;
    auto x = random_halves(r, m * n, -6.0f, 6.0f), s = random_halves(r, n, 5.0f, 40.0f), o = random_halves(r, n, -3.0f, 3.0f);
    std::printf("[inputs] quant_per_channel x=%016llx s=%016llx o=%016llx\n",
                (unsigned long long)fnv1a64(x.data(), x.size() * 2), (unsigned long long)fnv1a64(s.data(), s.size() * 2),
                (unsigned long long)fnv1a64(o.data(), o.size() * 2));
    if (inputs_only) {
        return;
    }
    DeviceBuffer<uint16_t> dx(x), ds(s), dof(o);
    DeviceBuffer<int8_t> dq(m * n);
    ascq::AscendQuant<ascq::half>(dq.view<int8_t>(m * n), dx.view<ascq::half>(m * n), ds.view<ascq::half>(n),
                                  dof.view<ascq::half>(n), n, n, m * n);
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_CHANNEL;
    d.src_dtype = d.scale_dtype = ASCQ_F16;
    d.compute = ASCQ_COMPUTE_F16;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_TENSOR;
    d.m = m;
    d.n = n;
    d.cal_count = m * n;
    std::vector<int8_t> want(m * n);
    orc_quant(&d, want.data(), x.data(), s.data(), o.data());
    expect_equal("AscendQuant per channel", dq.download(), want);
    {
        auto q = dq.download();
        std::printf("[output] quant_per_channel q=%016llx\n", (unsigned long long)fnv1a64(q.data(), q.size()));
    }

    std::printf("[case] AscendQuant<half> per tensor 1024\n");
    ascq::AscendQuant<ascq::half>(dq.view<int8_t>(1024), dx.view<ascq::half>(1024), 2.0f, 0.9f, 1024);
    d = ascq_quant_desc{};
    d.policy = ASCQ_PER_TENSOR;
    d.src_dtype = d.scale_dtype = ASCQ_F16;
    d.compute = ASCQ_COMPUTE_F16;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_SCALAR;
    d.scale = 2.0f;
    d.offset = 0.9f;
    d.m = 1;
    d.n = d.cal_count = 1024;
    want.assign(1024, 0);
    orc_quant(&d, want.data(), x.data(), nullptr, nullptr);
    auto got = dq.download();
    got.resize(1024);
    expect_equal("AscendQuant per tensor", got, want);
}

void test_quant_per_token_fp8()
{
    std::printf("[case] AscendQuant<fp8_e4m3fn_t, half, float> PER_TOKEN 12x256\n");
    Rng r{7};
    const uint32_t m = 12, n = 256;
    auto x = random_halves(r, m * n, -3.0f, 3.0f);
    std::vector<float> sc(m), of(m);
    for (auto& e : sc) e = r.uniform(0.01f, 200.0f);  // the largest products pass 448 and saturate
    for (auto& e : of) e = r.uniform(-1.0f, 1.0f);
    DeviceBuffer<uint16_t> dx(x);
    DeviceBuffer<float> dsc(sc), dof(of);
    DeviceBuffer<uint8_t> dq(m * n);
    ascq::AscendQuantConfig cfg{};
    cfg.hasOffset = true;
    ascq::AscendQuantParam para{};
    para.m = m;
    para.n = n;
    para.calCount = m * n;
    ascq::AscendQuant(dq.view<ascq::fp8_e4m3fn_t>(m * n), dx.view<ascq::half>(m * n), dsc.view<float>(m),
                      dof.view<float>(m), para, cfg, ascq::AscendQuantPolicy::PER_TOKEN);
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_TOKEN;
    d.src_dtype = ASCQ_F16;
    d.scale_dtype = ASCQ_F32;
    d.compute = ASCQ_COMPUTE_SCALE_T;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_TENSOR;
    d.k_dim = 1;
    d.m = m;
    d.n = n;
    d.cal_count = m * n;
    d.dst_format = ASCQ_QDST_FP8_E4M3FN;
    std::vector<uint8_t> want(m * n);
    orc_quant(&d, reinterpret_cast<int8_t*>(want.data()), x.data(), sc.data(), of.data());
    expect_equal("AscendQuant fp8 per token", dq.download(), want);

    // the same call with a hifloat8_t destination (RoundMode::CAST_ROUND, the type's default)
    std::printf("[case] AscendQuant<hifloat8_t, half, float> PER_TOKEN 12x256\n");
    cfg.roundMode = ascq::RoundMode::CAST_ROUND;
    ascq::AscendQuant(dq.view<ascq::hifloat8_t>(m * n), dx.view<ascq::half>(m * n), dsc.view<float>(m),
                      dof.view<float>(m), para, cfg, ascq::AscendQuantPolicy::PER_TOKEN);
    d.round_mode = ASCQ_CAST_ROUND;
    d.dst_format = ASCQ_QDST_HIF8;
    orc_quant(&d, reinterpret_cast<int8_t*>(want.data()), x.data(), sc.data(), of.data());
    expect_equal("AscendQuant hifloat8 per token", dq.download(), want);
}

void test_quant_per_group_fp4()
{
    std::printf("[case] AscendQuant<fp4x2_e2m1_t, half, float> PER_GROUP 12x256, groupSize 64, CAST_FLOOR\n");
    Rng r{9};
    const uint32_t m = 12, n = 256, gs = 64;
    auto x = random_halves(r, m * n, -3.0f, 3.0f);
    std::vector<float> sc(m * n / gs);
    for (auto& e : sc) e = r.uniform(0.05f, 4.0f);  // the largest products pass 6 and saturate
    DeviceBuffer<uint16_t> dx(x);
    DeviceBuffer<float> dsc(sc);
    DeviceBuffer<uint8_t> dq(m * n / 2);
    ascq::AscendQuantConfig cfg{};
    cfg.hasOffset = false;
    cfg.roundMode = ascq::RoundMode::CAST_FLOOR;
    ascq::AscendQuantParam para{};
    para.m = m;
    para.n = n;
    para.calCount = m * n;
    para.groupSize = gs;
    ascq::AscendQuant(dq.view<ascq::fp4x2_e2m1_t>(m * n), dx.view<ascq::half>(m * n), dsc.view<float>(m * n / gs),
                      dsc.view<float>(m * n / gs), para, cfg, ascq::AscendQuantPolicy::PER_GROUP);
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_GROUP;
    d.src_dtype = ASCQ_F16;
    d.scale_dtype = ASCQ_F32;
    d.compute = ASCQ_COMPUTE_SCALE_T;
    d.round_mode = ASCQ_CAST_FLOOR;
    d.offset_kind = ASCQ_OFFSET_NONE;
    d.k_dim = 1;
    d.m = m;
    d.n = n;
    d.cal_count = m * n;
    d.group_size = gs;
    d.dst_format = ASCQ_QDST_FP4_E2M1;
    std::vector<uint8_t> want(m * n / 2);
    orc_quant(&d, reinterpret_cast<int8_t*>(want.data()), x.data(), sc.data(), nullptr);
    expect_equal("AscendQuant fp4 per group", dq.download(), want);
}

void test_dequant()
{
    std::printf("[case] AscendDequant<bfloat16_t, float, MULTI_ROW> 32x40, calCount 36\n");
    Rng r{2};
    const uint32_t m = 32, n = 40, cal = 36;
    std::vector<int32_t> src(m * n);
    for (auto& e : src) e = r.integer(-(1 << 20), 1 << 20);
    std::vector<float> sc(n);
    for (auto& e : sc) e = r.uniform(1e-5f, 1e-3f);
    const uint32_t stride = ascq_dequant_dst_stride(ASCQ_BF16, n);
    DeviceBuffer<int32_t> dsrc(src);
    DeviceBuffer<float> dsc(sc);
    std::vector<uint16_t> init(m * stride, 0x7FC0);
    DeviceBuffer<uint16_t> ddst(init);
    ascq::AscendDequant<ascq::bfloat16_t, float, ascq::DeQuantMode::DEQUANT_WITH_MULTI_ROW>(
        ddst.view<ascq::bfloat16_t>(m * stride), dsrc.view<int32_t>(m * n), dsc.view<float>(n),
        ascq::DequantParams{m, n, cal});
    ascq_dequant_desc d{};
    d.policy = ASCQ_PER_CHANNEL;
    d.src_dtype = ASCQ_I32;
    d.scale_dtype = ASCQ_F32;
    d.dst_dtype = ASCQ_BF16;
    d.mode = ASCQ_DEQUANT_WITH_MULTI_ROW;
    d.m = m;
    d.n = n;
    d.cal_count = cal;
    std::vector<uint16_t> want(init);
    orc_dequant(&d, want.data(), src.data(), sc.data());
    expect_equal("AscendDequant", ddst.download(), want);
}

void test_antiquant()
{
    std::printf("[case] AscendAntiQuant<int8_t, half, false> 64x128, 2 groups\n");
    Rng r{3};
    const uint32_t k = 64, n = 128, groups = 2;
    std::vector<int8_t> w(k * n);
    for (auto& e : w) e = static_cast<int8_t>(r.integer(-128, 127));
    auto sc = random_halves(r, groups * n, 1e-3f, 1e-1f);
    std::vector<uint16_t> of(groups * n);
    for (auto& e : of) e = orc_f32_to_f16(static_cast<float>(r.integer(-8, 8)));
    DeviceBuffer<int8_t> dw(w);
    DeviceBuffer<uint16_t> dsc(sc), dof(of), ddst(k * n);
    ascq::AntiQuantShapeInfo info{groups, n, groups, n};
    ascq::AscendAntiQuant<int8_t, ascq::half, false>(ddst.view<ascq::half>(k * n), dw.view<int8_t>(k * n),
                                                     dof.view<ascq::half>(groups * n), dsc.view<ascq::half>(groups * n),
                                                     k, info);
    ascq_antiquant_desc d{};
    d.src_dtype = ASCQ_I8;
    d.dst_dtype = ASCQ_F16;
    d.has_offset = 1;
    d.k = k;
    d.n = n;
    d.offset_height = d.scale_height = groups;
    d.offset_width = d.scale_width = n;
    std::vector<uint16_t> want(k * n);
    orc_antiquant(&d, want.data(), w.data(), of.data(), sc.data());
    expect_equal("AscendAntiQuant", ddst.download(), want);
}

void test_matmul()
{
    Rng r{4};
    const uint32_t m = 96, n = 160, k = 256;
    std::vector<int8_t> a(m * k), b(k * n);
    for (auto& e : a) e = static_cast<int8_t>(r.integer(-127, 127));
    for (auto& e : b) e = static_cast<int8_t>(r.integer(-127, 127));
    std::vector<float> cs(n), ts(m);
    for (auto& e : cs) e = r.uniform(1e-4f, 1e-2f);
    for (auto& e : ts) e = r.uniform(1e-3f, 1e-1f);
    std::vector<int32_t> bias(n);
    for (auto& e : bias) e = r.integer(-1000, 1000);
    DeviceBuffer<int8_t> da(a), db(b);
    DeviceBuffer<float> dcs(cs), dts(ts);
    DeviceBuffer<int32_t> dbias(bias);

    std::printf("[case] Matmul<bfloat16_t> 96x160x256, SetQuantVector(float) + token scale\n");
    {
        DeviceBuffer<uint16_t> dc(m * n);
        ascq::Matmul<ascq::bfloat16_t> mm(m, n, k);
        mm.SetTensorA(da.view<int8_t>(m * k));
        mm.SetTensorB(db.view<int8_t>(k * n));
        mm.SetQuantVector(dcs.view<float>(n));
        mm.SetTokenScale(dts.view<float>(m));
        // the plan query launches nothing and leaves the object ready for the call: 96 rows without a workspace are
        // one launch of 128 x 128 tiles
        const ascq_matmul_plan plan = mm.GetPlan(dc.view<ascq::bfloat16_t>(m * n));
        if (plan.kernel != ASCQ_MM_KERNEL_DMA_128 || plan.tile_m != 128 || plan.k_splits != 1 || plan.launches != 1) {
            std::printf("FAIL Matmul plan: kernel %d tile_m %u k_splits %u launches %u\n", plan.kernel, plan.tile_m,
                        plan.k_splits, plan.launches);
            ++g_failed;
        }
        mm.IterateAll(dc.view<ascq::bfloat16_t>(m * n));
        std::vector<uint16_t> want(m * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a.data(), b.data(), nullptr, cs.data(), ts.data());
        expect_equal("Matmul bf16 epilogue", dc.download(), want);
    }
    std::printf("[case] Matmul<half> 96x160x256, int32 bias + SetQuantScalar(uint64)\n");
    {
        DeviceBuffer<uint16_t> dc(m * n);
        ascq::Matmul<ascq::half> mm(m, n, k);
        mm.SetTensorA(da.view<int8_t>(m * k));
        mm.SetTensorB(db.view<int8_t>(k * n));
        mm.SetBias(dbias.view<int32_t>(n));
        mm.SetQuantScalar(ascq_pack_quant_param(0.00123f, 0, 0));
        mm.IterateAll(dc.view<ascq::half>(m * n));
        std::vector<uint16_t> want(m * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a.data(), b.data(), bias.data(), nullptr, nullptr);
        expect_equal("Matmul DEQF16 epilogue", dc.download(), want);
    }
    std::printf("[case] Matmul<int32_t> 96x160x256, no quant\n");
    {
        DeviceBuffer<int32_t> dc(m * n);
        ascq::Matmul<int32_t> mm(m, n, k);
        mm.SetTensorA(da.view<int8_t>(m * k));
        mm.SetTensorB(db.view<int8_t>(k * n));
        mm.IterateAll(dc.view<int32_t>(m * n));
        std::vector<int32_t> want(m * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a.data(), b.data(), nullptr, nullptr, nullptr);
        expect_equal("Matmul int32", dc.download(), want);
    }
    std::printf("[case] Matmul<bfloat16_t> 7x160x256 on weights packed by PackWeightInt8 (decode kernel)\n");
    {
        const uint32_t rows = 7;
        DeviceBuffer<uint8_t> dpacked(ascq::PackWeightInt8Size(k, n));
        ascq::PackWeightInt8(db.view<int8_t>(k * n), dpacked.ptr(), k, n);
        DeviceBuffer<uint16_t> dc(rows * n);
        ascq::Matmul<ascq::bfloat16_t> mm(rows, n, k);
        mm.SetTensorA(da.view<int8_t>(rows * k));
        mm.SetTensorBPacked(dpacked.ptr());
        mm.SetQuantVector(dcs.view<float>(n));
        mm.SetTokenScale(dts.view<float>(rows));
        mm.IterateAll(dc.view<ascq::bfloat16_t>(rows * n));
        std::vector<uint16_t> want(rows * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a.data(), b.data(), nullptr, cs.data(), ts.data());
        expect_equal("Matmul on packed int8 weights", dc.download(), want);
    }
    std::printf("[case] Matmul<bfloat16_t> 96x160x256 on packed weights (weights held in registers, activations streamed)\n");
    {
        DeviceBuffer<uint8_t> dpacked(ascq::PackWeightInt8Size(k, n));
        ascq::PackWeightInt8(db.view<int8_t>(k * n), dpacked.ptr(), k, n);
        DeviceBuffer<uint16_t> dc(m * n);
        ascq::Matmul<ascq::bfloat16_t> mm(m, n, k);
        mm.SetTensorA(da.view<int8_t>(m * k));
        mm.SetTensorBPacked(dpacked.ptr());
        mm.SetQuantVector(dcs.view<float>(n));
        mm.SetTokenScale(dts.view<float>(m));
        mm.IterateAll(dc.view<ascq::bfloat16_t>(m * n));
        std::vector<uint16_t> want(m * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a.data(), b.data(), nullptr, cs.data(), ts.data());
        expect_equal("Matmul on packed int8 weights, 96 rows", dc.download(), want);
    }
    std::printf("[case] ascq_linear_w8a8_dynamic_packed 3x160x256: bfloat16 x quantised per token inside the decode kernel\n");
    {
        const uint32_t rows = 3;
        std::vector<uint16_t> x(rows * k);
        for (auto& e : x) e = orc_f32_to_bf16(r.uniform(-4.0f, 4.0f));
        DeviceBuffer<uint16_t> dx(x), dc(rows * n);
        DeviceBuffer<uint8_t> dpacked(ascq::PackWeightInt8Size(k, n));
        ascq::PackWeightInt8(db.view<int8_t>(k * n), dpacked.ptr(), k, n);
        ascq_matmul_desc d{};
        d.m = rows;
        d.n = n;
        d.k = k;
        d.out_dtype = ASCQ_BF16;
        d.quant_mode = ASCQ_MM_QUANT_VECTOR;
        d.scale_format = ASCQ_MM_SCALE_F32;
        size_t need = 0;
        ascq::Check(ascq_linear_w8a8_dynamic_workspace_size(&d, &need));
        DeviceBuffer<uint8_t> dws(need ? need : 16);
        ascq::Check(ascq_linear_w8a8_dynamic_packed(&d, ASCQ_BF16, dc.ptr(), dx.ptr(), dpacked.ptr(), nullptr, dcs.ptr(),
                                                    dws.ptr(), need ? need : 16, nullptr));
        std::vector<int8_t> q(rows * k);
        std::vector<float> tok(rows);
        orc_dynamic_quant_per_token(ASCQ_BF16, rows, k, q.data(), tok.data(), x.data());
        d.has_tok_scale = 1;
        std::vector<uint16_t> want(rows * n);
        orc_matmul_w8a8(&d, want.data(), q.data(), b.data(), nullptr, cs.data(), tok.data());
        expect_equal("one-launch linear on packed weights", dc.download(), want);
    }
    std::printf("[case] Matmul<int32_t, int4b_t> 96x160x256, int32 bias\n");
    {
        // int4 operands, two per byte with the even element in the low nibble; the oracle sees the same values as int8
        std::vector<int8_t> a4v(m * k), b4v(k * n);
        for (auto& e : a4v) e = static_cast<int8_t>(r.integer(-8, 7));
        for (auto& e : b4v) e = static_cast<int8_t>(r.integer(-8, 7));
        auto pack = [](const std::vector<int8_t>& v) {
            std::vector<uint8_t> p(v.size() / 2);
            for (size_t i = 0; i < p.size(); ++i) {
                p[i] = static_cast<uint8_t>((v[2 * i] & 0x0F) | ((v[2 * i + 1] & 0x0F) << 4));
            }
            return p;
        };
        DeviceBuffer<uint8_t> da4(pack(a4v)), db4(pack(b4v));
        DeviceBuffer<int32_t> dc(m * n);
        ascq::Matmul<int32_t, ascq::int4b_t> mm(m, n, k);
        mm.SetTensorA(da4.view<ascq::int4b_t>(m * k));
        mm.SetTensorB(db4.view<ascq::int4b_t>(k * n));
        mm.SetBias(dbias.view<int32_t>(n));
        DeviceBuffer<uint8_t> ws(mm.GetWorkspaceSize());
        mm.SetWorkspace(ws.view<uint8_t>(0).GetPhyAddr(), mm.GetWorkspaceSize());
        mm.IterateAll(dc.view<int32_t>(m * n));
        std::vector<int32_t> want(m * n);
        orc_matmul_w8a8(&mm.Desc(), want.data(), a4v.data(), b4v.data(), bias.data(), nullptr, nullptr);
        expect_equal("Matmul int4 x int4", dc.download(), want);
    }
}

void test_antiquant_matmul()
{
    // small integers, a power-of-two scale and an integer offset: every product and partial sum is exact in fp32, so
    // the result does not depend on the order of accumulation and must equal the oracle's bit for bit
    std::printf("[case] AntiQuantMatmul<float> 5x272x128, SetAntiQuantVector\n");
    Rng r{6};
    const uint32_t m = 5, n = 272, k = 128;
    std::vector<uint16_t> x(m * k), sc(n), of(n);
    std::vector<int8_t> w(k * n);
    for (auto& e : x) e = orc_f32_to_f16(static_cast<float>(r.integer(-4, 4)));
    for (auto& e : w) e = static_cast<int8_t>(r.integer(-128, 127));
    for (auto& e : sc) e = orc_f32_to_f16(r.integer(0, 1) ? 0.5f : 0.25f);
    for (auto& e : of) e = orc_f32_to_f16(static_cast<float>(r.integer(-8, 8)));
    DeviceBuffer<uint16_t> dx(x), dsc(sc), dof(of);
    DeviceBuffer<int8_t> dw(w);
    DeviceBuffer<float> dc(m * n);
    ascq::AntiQuantMatmul<float> mm(m, n, k);
    DeviceBuffer<uint8_t> ws(mm.GetWorkspaceSize() + 16);
    mm.SetTensorA(dx.view<ascq::half>(m * k));
    mm.SetTensorB(dw.view<int8_t>(k * n));
    mm.SetAntiQuantVector(dof.view<ascq::half>(n), dsc.view<ascq::half>(n));
    mm.SetWorkspace(ws.view<uint8_t>(1).GetPhyAddr(), mm.GetWorkspaceSize());
    mm.IterateAll(dc.view<float>(m * n));
    std::vector<float> want(m * n);
    orc_matmul_w8a16(&mm.Desc(), want.data(), x.data(), w.data(), of.data(), sc.data());
    expect_equal("AntiQuantMatmul", dc.download(), want);

    // the same product from weights kept as [n, k] (SetTensorB(b, isTransposeB = true)): no workspace
    std::printf("[case] AntiQuantMatmul<float> 5x272x128, B as [n, k]\n");
    std::vector<int8_t> wt(n * k);
    for (uint32_t j = 0; j < n; ++j)
        for (uint32_t kk = 0; kk < k; ++kk) wt[j * k + kk] = w[kk * n + j];
    DeviceBuffer<int8_t> dwt(wt);
    DeviceBuffer<float> dc2(m * n);
    ascq::AntiQuantMatmul<float> mt(m, n, k);
    mt.SetTensorA(dx.view<ascq::half>(m * k));
    mt.SetTensorB(dwt.view<int8_t>(k * n), true);
    mt.SetAntiQuantVector(dof.view<ascq::half>(n), dsc.view<ascq::half>(n));
    if (mt.GetWorkspaceSize() != 0) {
        std::printf("[FAIL] [n, k] weights asked for a workspace\n");
        ++g_failed;
    }
    mt.IterateAll(dc2.view<float>(m * n));
    expect_equal("AntiQuantMatmul [n, k]", dc2.download(), want);
}

void test_unified_surface()
{
    // Quantize / Dequantize / AntiQuantize with the policy inside the config, each against the oracle entry point of
    // the operator it forwards to
    Rng r{13};
    const uint32_t m = 24, n = 128, gs = 32;
    std::printf("[case] Quantize<PER_GROUP kDim=1, CAST_ROUND, offset> half -> int8 24x128\n");
    {
        auto x = random_halves(r, m * n, -4.0f, 4.0f);
        std::vector<float> sc(m * n / gs), of(m * n / gs);
        for (auto& e : sc) e = r.uniform(5.0f, 40.0f);
        for (auto& e : of) e = r.uniform(-3.0f, 3.0f);
        DeviceBuffer<uint16_t> dx(x);
        DeviceBuffer<float> dsc(sc), dof(of);
        DeviceBuffer<int8_t> dq(m * n);
        ascq::QuantizeConfig cfg{ascq::QuantizePolicy::PER_GROUP, true, ascq::RoundMode::CAST_ROUND, 1};
        ascq::Quantize(dq.view<int8_t>(m * n), dx.view<ascq::half>(m * n), dsc.view<float>(m * n / gs),
                       dof.view<float>(m * n / gs), ascq::QuantizeParams{m, n, gs}, cfg);
        ascq_quant_desc d{};
        d.policy = ASCQ_PER_GROUP;
        d.src_dtype = ASCQ_F16;
        d.scale_dtype = ASCQ_F32;
        d.compute = ASCQ_COMPUTE_F32;
        d.round_mode = ASCQ_CAST_ROUND;
        d.offset_kind = ASCQ_OFFSET_TENSOR;
        d.k_dim = 1;
        d.m = m;
        d.n = n;
        d.cal_count = m * n;
        d.group_size = gs;
        std::vector<int8_t> want(m * n);
        orc_quant(&d, want.data(), x.data(), sc.data(), of.data());
        expect_equal("Quantize per group", dq.download(), want);
    }
    std::printf("[case] Dequantize<PER_TOKEN> int32 -> bfloat16 24x128\n");
    {
        std::vector<int32_t> src(m * n);
        for (auto& e : src) e = r.integer(-(1 << 20), 1 << 20);
        std::vector<float> sc(m);
        for (auto& e : sc) e = r.uniform(1e-5f, 1e-3f);
        DeviceBuffer<int32_t> ds(src);
        DeviceBuffer<float> dsc(sc);
        DeviceBuffer<uint16_t> dd(m * n);
        ascq::DequantizeConfig cfg{ascq::DequantizePolicy::PER_TOKEN, false, 1};
        ascq::Dequantize(dd.view<ascq::bfloat16_t>(m * n), ds.view<int32_t>(m * n), dsc.view<float>(m),
                         dsc.view<float>(m), ascq::DequantizeParams{m, n, 0}, cfg);
        ascq_dequant_desc d{};
        d.policy = ASCQ_PER_TOKEN;
        d.src_dtype = ASCQ_I32;
        d.scale_dtype = ASCQ_F32;
        d.dst_dtype = ASCQ_BF16;
        d.mode = ASCQ_DEQUANT_WITH_MULTI_ROW;
        d.k_dim = 1;
        d.m = m;
        d.n = n;
        d.cal_count = m * n;
        std::vector<uint16_t> want(m * n);
        orc_dequant(&d, want.data(), src.data(), sc.data());
        expect_equal("Dequantize per token", dd.download(), want);
    }
    std::printf("[case] AntiQuantize<PER_TENSOR, offset> fp8_e4m3fn -> half 24x128\n");
    {
        std::vector<uint8_t> codes(m * n);
        for (auto& e : codes) {
            e = static_cast<uint8_t>(r.integer(0, 255));
            if ((e & 0x7F) == 0x7F) e = 0x3C;  // no NaN codes
        }
        DeviceBuffer<uint8_t> dc(codes);
        DeviceBuffer<uint16_t> dd(m * n);
        ascq::AntiQuantizeConfig cfg{ascq::AntiQuantizePolicy::PER_TENSOR, true, 1};
        ascq::AntiQuantize(dd.view<ascq::half>(m * n), dc.view<ascq::fp8_e4m3fn_t>(m * n), 0.37123f, -3.2517f,
                           ascq::AntiQuantizeParams{m, n, 0}, cfg);
        ascq_antiquant_policy_desc d{};
        d.policy = ASCQ_PER_TENSOR;
        d.src_format = ASCQ_QDST_FP8_E4M3FN;
        d.scale_dtype = ASCQ_F16;
        d.dst_dtype = ASCQ_F16;
        d.compute = ASCQ_COMPUTE_F32;
        d.has_offset = 1;
        d.k_dim = 1;
        d.m = m;
        d.n = n;
        d.cal_count = m * n;
        d.scale = 0.37123f;
        d.offset = -3.2517f;
        std::vector<uint16_t> want(m * n);
        orc_antiquant_policy(&d, want.data(), codes.data(), nullptr, nullptr);
        expect_equal("AntiQuantize per tensor", dd.download(), want);
    }
}

void test_antiquant_fp4()
{
    std::printf("[case] AscendAntiQuant<half, fp4x2_e2m1_t, fp8_e8m0_t> PER_GROUP 12x256, groupSize 64\n");
    Rng r{21};
    const uint32_t m = 12, n = 256, gs = 64;
    std::vector<uint8_t> packed(m * n / 2), sc(m * n / gs);
    for (auto& e : packed) e = static_cast<uint8_t>(r.integer(0, 255));
    for (auto& e : sc) e = static_cast<uint8_t>(r.integer(100, 150));  // 2^-27 .. 2^23: part of it past half's range
    DeviceBuffer<uint8_t> dp(packed), dsc(sc);
    DeviceBuffer<uint16_t> dd(m * n);
    ascq::AscendAntiQuantConfig cfg{};
    cfg.hasOffset = false;
    ascq::AscendAntiQuantParam para{};
    para.m = m;
    para.n = n;
    para.calCount = m * n;
    para.groupSize = gs;
    ascq::AscendAntiQuant(dd.view<ascq::half>(m * n), dp.view<ascq::fp4x2_e2m1_t>(m * n),
                          dsc.view<ascq::fp8_e8m0_t>(m * n / gs), dsc.view<ascq::fp8_e8m0_t>(m * n / gs), para, cfg,
                          ascq::AscendAntiQuantPolicy::PER_GROUP);
    ascq_antiquant_policy_desc d{};
    d.policy = ASCQ_PER_GROUP;
    d.src_format = ASCQ_QDST_FP4_E2M1;
    d.scale_dtype = ASCQ_E8M0;
    d.dst_dtype = ASCQ_F16;
    d.compute = ASCQ_COMPUTE_SCALE_T;
    d.k_dim = 1;
    d.m = m;
    d.n = n;
    d.cal_count = m * n;
    d.group_size = gs;
    std::vector<uint16_t> want(m * n);
    orc_antiquant_policy(&d, want.data(), packed.data(), sc.data(), nullptr);
    expect_equal("AscendAntiQuant fp4 per group", dd.download(), want);
}

void test_errors()
{
    std::printf("[case] argument errors surface as ascq::Error\n");
    DeviceBuffer<uint16_t> x(64);
    DeviceBuffer<int8_t> q(64);
    bool threw = false;
    try {
        ascq::AscendQuant<ascq::half>(q.view<int8_t>(64), x.view<ascq::half>(64), x.view<ascq::half>(32),
                                      x.view<ascq::half>(16), 32, 16, 64);
    } catch (const ascq::Error& e) {
        threw = e.status() == ASCQ_EINVAL;
    }
    int ok = threw;
    threw = false;
    try {
        ascq::Matmul<ascq::half> mm(16, 16, 16);  // no tensors set
        mm.SetQuantScalar(ascq_pack_quant_param(1.0f, 0, 0));
        mm.IterateAll(x.view<ascq::half>(64));
    } catch (const ascq::Error& e) {
        threw = e.status() != ASCQ_OK && std::strlen(e.what()) > 0;
    }
    ok += threw;
    std::printf("[%s] error paths: %d of 2 raised\n", ok == 2 ? " ok " : "FAIL", ok);
    g_failed += ok != 2;
}

}  // namespace

int main(int argc, char** argv)
{
    if (argc > 1 && std::strcmp(argv[1], "--inputs") == 0) {  // no GPU needed: the generated inputs only
        test_quant_per_channel(true);
        return 0;
    }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
        std::fprintf(stderr, "no GPU\n");
        return 2;
    }
    std::printf("library: %s\n", ascq_version());
    test_quant_per_channel(false);
    test_quant_per_token_fp8();
    test_quant_per_group_fp4();
    test_dequant();
    test_antiquant();
    test_matmul();
    test_antiquant_matmul();
    test_unified_surface();
    test_antiquant_fp4();
    test_errors();
    std::printf("%s\n", g_failed ? "FAILED" : "ALL PASSED");
    return g_failed ? 1 : 0;
}
