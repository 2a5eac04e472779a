// Tests of the C++ host layer, written the way the reference tests its kernels
// (src/04kernel/test/kernels/*/test_cuda.cpp): Tensor::share -> Collector::filter (or
// Kernel::build) -> lower(res) -> device::init -> malloc / copyFromHost -> routine -> copyToHost
// -> compare with the CPU result.  The CPU result comes from the oracle (oracle/oracle.h).
//
//   rg_host_tests cpu     host logic only (no GPU needed)
//   rg_host_tests gpu     everything that runs a routine on the AMD device
#include "kernel/attributes/broadcaster.h"
#include "kernel/attributes/mat_mul_integer_info.h"
#include "kernel/attributes/softmax_info.h"
#include "kernel/collectors/attention.h"
#include "kernel/collectors/dequantize_linear.h"
#include "kernel/collectors/dynamic_quantize_linear.h"
#include "kernel/collectors/mat_mul_integer.h"
#include "kernel/collectors/rms_normalization.h"
#include "kernel/collectors/rotary_embedding.h"
#include "kernel/collectors/softmax.h"
#include "hardware/device_manager.h"
#include "hardware/mem_pool.h"
#include "rg_mirror/hip_kernels.h"
#include "oracle.h"

#include <cmath>
#include <immintrin.h>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <random>
#include <tuple>

using namespace refactor;
using namespace kernel;
using namespace hardware;

static int g_failed = 0, g_checks = 0;
#define EXPECT(COND)                                                              \
    do {                                                                          \
        ++g_checks;                                                               \
        if (!(COND)) {                                                            \
            ++g_failed;                                                           \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #COND);       \
        }                                                                         \
    } while (0)
#define RUN(NAME)                                  \
    do {                                           \
        std::printf("[ RUN  ] %s\n", #NAME);       \
        std::fflush(stdout);                       \
        NAME();                                    \
    } while (0)
template<class E, class F> static bool throws(F &&f) {
    try { f(); } catch (E const &) { return true; } catch (...) { return false; }
    return false;
}

// IEEE binary16 with round-to-nearest-even (F16C)
static uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }
static float h2f(uint16_t h) { return _cvtsh_ss(h); }

// ------------------------------------------------------------------ host logic (no GPU)

static void broadcasterKnownAnswer() {
    // src/04kernel/test/attributes/test_broadcaster.cpp:7-36
    Broadcaster b({{3, 5, 7}, {5, 7}, {}, {2, 1, 1, 1}});
    EXPECT(b.outputsCount == 210);
    EXPECT((b.strides == std::vector<dim_t>{0, 0, 0, 1, 105, 35, 0, 0, 0, 35, 1, 1, 0, 0, 1}));
    std::vector<dim_t> ans(b.inputsCount);
    b.locate(1, ans.data());
    EXPECT((ans == std::vector<dim_t>{1, 1, 0, 0}));
    b.locate(40, ans.data());
    EXPECT((ans == std::vector<dim_t>{40, 5, 0, 0}));
    Broadcaster same({{2, 3}, {2, 3}});
    EXPECT(!same.needBroadcast() && same.outputsCount == 6);
    same.locate(4, ans.data());
    EXPECT(ans[0] == 4 && ans[1] == 4);
    EXPECT(throws<std::runtime_error>([] { Broadcaster bad({{2, 3}, {4, 3}}); }));
}

static void shapeDigests() {
    auto x = Tensor::share(DataType::F32, Shape{2, 3, 4, 5});
    SoftmaxInfo s(*x, 1);
    EXPECT(s.pre == 2 && s.mid == 3 && s.post == 20 && s.type == DataType::F32);
    EXPECT(x->elementsSize() == 120 && x->bytesSize() == 480 && (x->strides() == Strides{60, 20, 5, 1}));

    // MatMulIntegerInfo: signedness comes from the zero point's dtype, a constant all-zero zero
    // point is elided, one element = scalar, batch dims broadcast
    auto A = Tensor::share(DataType::U8, Shape{2, 1, 4, 8});
    auto B = Tensor::share(DataType::I8, Shape{3, 8, 5});
    auto az = Tensor::share(DataType::U8, Shape{});
    auto bz = Tensor::share(DataType::I8, Shape{1});
    *static_cast<int8_t *>(bz->malloc()) = 0;// constant zero -> no zero point work
    MatMulIntegerInfo info(TensorRefs{*A, *B, *az, *bz});
    EXPECT(info.m == 4 && info.k == 8 && info.n == 5 && info.batch() == 6);
    EXPECT(info.a.withZeroPoint && !info.a.signed_ && info.a.scalar);
    EXPECT(!info.b.withZeroPoint);
    dim_t at[2];
    info.broadcaster.locate(4, at);// output batch (1, 1) -> A matrix 1, B matrix 1
    EXPECT(at[0] == 1 && at[1] == 1);
    auto rowZp = Tensor::share(DataType::I8, Shape{2, 1, 4});
    MatMulIntegerInfo perRow(TensorRefs{*A, *B, *rowZp});
    EXPECT(perRow.a.withZeroPoint && perRow.a.signed_ && !perRow.a.scalar && !perRow.b.withZeroPoint);
}

static void memPoolBestFit() {
    // src/02hardware/test/test_mem_pool.cpp:8-32
    MemPool pool(std::make_shared<CpuMemory>(), 64ul << 20, 8);
    auto a = 2 * 10 * 20 * 30 * sizeof(float), b = 3 * 10 * 20 * 30 * sizeof(float),
         c = 5 * 10 * 20 * 30 * sizeof(float), d = 7 * 10 * 20 * 30 * sizeof(float);
    auto aPtr = pool.malloc(a), bPtr = pool.malloc(b), cPtr = pool.malloc(c), dPtr = pool.malloc(d);
    EXPECT(aPtr != bPtr && bPtr != cPtr && cPtr != dPtr);
    pool.free(bPtr);
    pool.free(cPtr);
    EXPECT(pool.malloc(b + c) == bPtr);// the two freed neighbours were merged
    EXPECT(pool.malloc(0) == nullptr);
    EXPECT(throws<std::runtime_error>([&] { pool.malloc(1ul << 30); }));// out of memory
    int onStack = 0;
    EXPECT(throws<std::runtime_error>([&] { pool.free(&onStack); }));   // invalid ptr
    MemPool aligned(std::make_shared<CpuMemory>(), 1 << 20, 256);
    auto p0 = static_cast<uint8_t *>(aligned.malloc(3)), p1 = static_cast<uint8_t *>(aligned.malloc(300));
    EXPECT((p1 - p0) % 256 == 0 && p1 - p0 >= 256);
}

static void resourcesAndErrors() {
    struct Counter final : runtime::Resource {
        int value = 0;
        static size_t typeId() noexcept { static uint8_t ID = 1; return reinterpret_cast<size_t>(&ID); }
        static runtime::ResourceBox build(int v) { auto r = std::make_unique<Counter>(); r->value = v; return r; }
        size_t resourceTypeId() const noexcept final { return typeId(); }
        std::string_view description() const noexcept final { return "counter"; }
    };
    runtime::Resources res;
    EXPECT(res.fetch<Counter>() == nullptr);
    EXPECT(res.fetchOrStore<Counter>(7)->value == 7);
    EXPECT(res.fetchOrStore<Counter>(9)->value == 7);// already stored: the builder is not run again
    EXPECT(res.fetch<Counter>()->is(Counter::typeId()));

    // the base Kernel::lower throws like the reference's; messages carry " Source file:line"
    struct Stub final : Kernel {
        size_t kernelTypeId() const final { return 0; }
        std::string_view description() const final { return "stub"; }
    } stub;
    EXPECT(throws<UnimplementError>([&] { stub.lower(res); }));
    try {
        RUNTIME_ERROR("boom");
    } catch (std::runtime_error const &e) {
        EXPECT(std::string(e.what()).find("boom Source ") == 0 && std::string(e.what()).find("test_main.cc:") != std::string::npos);
    }
    // CPU blobs: bounded copies
    auto cpu = device::fetch(Device::Type::Cpu);
    EXPECT(cpu && cpu->type() == Device::Type::Cpu && device::fetch(Device::Type::Amd, 5) == nullptr);
    auto blob = cpu->malloc(16);
    char buf[32] = {};
    EXPECT(throws<std::runtime_error>([&] { blob->copyFromHost(buf, 17); }));
    blob->copyFromHost("0123456789abcdef");
    blob->copyToHost(buf, 16);
    EXPECT(std::memcmp(buf, "0123456789abcdef", 16) == 0);
}

static void collectorsSelectOrDecline() {
    using T = Device::Type;
    auto f32 = Tensor::share(DataType::F32, Shape{2, 3, 64});
    auto w = Tensor::share(DataType::F32, Shape{64});
    auto i32 = Tensor::share(DataType::I32, Shape{2, 3, 64});
    auto amd = RmsNormalizationCollector(T::Amd, 1e-5f).filter({*f32, *w}, {*f32});
    EXPECT(amd.size() == 1 && amd[0]->is<RmsNormalizationHip>());
    EXPECT(std::string(amd[0]->description()).find("gfx950") != std::string::npos);
    EXPECT(RmsNormalizationCollector(T::Amd, 1e-5f).filter({*i32, *w}, {*i32}).empty());// not a float type
    EXPECT(RmsNormalizationCollector(T::Cpu, 1e-5f).filter({*f32, *w}, {*f32}).empty());// no CPU kernels in this build
    EXPECT(throws<UnreachableError>([&] { RmsNormalizationCollector(T::Nvidia, 1e-5f).filter({*f32, *w}, {*f32}); }));

    EXPECT(SoftmaxCollector(T::Amd, 2).filter({*f32}, {*f32}).size() == 1);
    EXPECT(SoftmaxCollector(T::Amd, 1, true).filter({*f32}, {*f32}).empty());// causal needs the last axis
    auto sq = Tensor::share(DataType::FP16, Shape{4, 16, 16});
    auto causal = SoftmaxCollector(T::Amd, 2, true).filter({*sq}, {*sq});
    EXPECT(causal.size() == 1 && static_cast<SoftmaxHip const &>(*causal[0]).causalRows == 16);

    // DequantizeLinear: per-tensor (reference) and per-axis; mismatching zero point is declined
    auto x8 = Tensor::share(DataType::I8, Shape{4, 6});
    auto y = Tensor::share(DataType::F32, Shape{4, 6});
    auto s1 = Tensor::share(DataType::F32, Shape{});
    auto s6 = Tensor::share(DataType::F32, Shape{6});
    auto z6u = Tensor::share(DataType::U8, Shape{6});
    auto k1 = DequantizeLinearCollector(T::Amd).filter({*x8, *s1}, {*y});
    EXPECT(k1.size() == 1 && !static_cast<DequantizeLinearHip const &>(*k1[0]).perAxis);
    auto k6 = DequantizeLinearCollector(T::Amd, 1).filter({*x8, *s6}, {*y});
    EXPECT(k6.size() == 1 && static_cast<DequantizeLinearHip const &>(*k6[0]).axisLen == 6);
    EXPECT(DequantizeLinearCollector(T::Amd, 0).filter({*x8, *s6}, {*y}).empty());  // axis 0 has 4 entries
    EXPECT(DequantizeLinearCollector(T::Amd, 1).filter({*x8, *s6, *z6u}, {*y}).empty());

    // DynamicQuantizeLinear: float -> (uint8, float scalar, uint8 scalar); the routine asks for a workspace
    auto xf = Tensor::share(DataType::F32, Shape{4, 6});
    auto yq = Tensor::share(DataType::U8, Shape{4, 6});
    auto zq = Tensor::share(DataType::U8, Shape{});
    auto dq = DynamicQuantizeLinearCollector(T::Amd).filter({*xf}, {*yq, *s1, *zq});
    EXPECT(dq.size() == 1 && static_cast<DynamicQuantizeLinearHip const &>(*dq[0]).size == 24);
    {
        runtime::Resources res_;
        EXPECT(dq[0]->lower(res_).workspaceOffset > 0);
    }
    EXPECT(DynamicQuantizeLinearCollector(T::Amd).filter({*x8}, {*yq, *s1, *zq}).empty());
    EXPECT(DynamicQuantizeLinearCollector(T::Cpu).filter({*xf}, {*yq, *s1, *zq}).empty());

    // MatMul: shapes, transposes and bias strides from the tensors; unsupported types are declined
    {
        auto a = Tensor::share(DataType::F32, Shape{2, 1, 5, 7});
        auto bt = Tensor::share(DataType::F32, Shape{1, 3, 4, 7});
        auto cRow = Tensor::share(DataType::F32, Shape{5, 1});
        auto cFull = Tensor::share(DataType::F32, Shape{2, 3, 5, 4});
        auto cOdd = Tensor::share(DataType::F32, Shape{2, 1, 5, 4});
        MatMulInfo info(*a, *bt, std::cref(*cRow), false, true, 0.5f, 2.f);
        EXPECT(info.m == 5 && info.k == 7 && info.n == 4 && info.batch() == 6 && info.hasBias && info.biasSupported);
        EXPECT(info.biasStrideM == 1 && info.biasStrideN == 0 && info.biasStrideBatch == 0);
        MatMulInfo full(*a, *bt, std::cref(*cFull), false, true, 1.f, 1.f);
        EXPECT(full.biasStrideBatch == 20 && full.biasStrideM == 4 && full.biasStrideN == 1);
        EXPECT(!MatMulInfo(*a, *bt, std::cref(*cOdd), false, true, 1.f, 1.f).biasSupported);
        EXPECT(MatMulCollector(T::Amd, 1, 1, false, true).filter({*a, *bt, *cRow}, {*cFull}).size() == 1);
        EXPECT(MatMulCollector(T::Amd, 1, 1, false, true).filter({*a, *bt, *cOdd}, {*cFull}).empty());
        EXPECT(MatMulCollector(T::Cpu, 1, 1, false, true).filter({*a, *bt}, {*cFull}).empty());
        auto ai = Tensor::share(DataType::I32, Shape{5, 7});
        auto bi = Tensor::share(DataType::I32, Shape{7, 4});
        EXPECT(MatMulCollector(T::Amd, 1, 1, false, false).filter({*ai, *bi}, {*cFull}).empty());
        EXPECT(throws<std::runtime_error>(
            [&] { MatMulInfo bad(*a, *Tensor::share(DataType::F32, Shape{6, 4}), std::nullopt, false, false, 1.f, 1.f); }));
    }

    // Cast: every pair of numeric types has a kernel; strings and complex numbers do not
    auto c8 = Tensor::share(DataType::I8, Shape{4, 6});
    auto ch = Tensor::share(DataType::FP16, Shape{4, 6});
    auto cb = Tensor::share(DataType::Bool, Shape{4, 6});
    auto cs = Tensor::share(DataType::String, Shape{4, 6});
    auto ck = CastCollector(T::Amd).filter({*xf}, {*c8});
    EXPECT(ck.size() == 1 && static_cast<CastHip const &>(*ck[0]).size == 24 &&
           static_cast<CastHip const &>(*ck[0]).from == DataType::F32 && static_cast<CastHip const &>(*ck[0]).to == DataType::I8);
    EXPECT(CastCollector(T::Amd).filter({*ch}, {*cb}).size() == 1);
    EXPECT(CastCollector(T::Amd).filter({*cs}, {*c8}).empty());
    EXPECT(CastCollector(T::Amd).filter({*xf}, {*Tensor::share(DataType::I8, Shape{5})}).empty());
    EXPECT(CastCollector(T::Cpu).filter({*xf}, {*c8}).empty());

    // Attention: parameter block from the tensors; head-count and dtype rules
    auto q = Tensor::share(DataType::FP16, Shape{2, 8, 1, 128});
    auto kv = Tensor::share(DataType::FP16, Shape{2, 2, 1, 128});
    auto past = Tensor::share(DataType::I64, Shape{1});
    auto cache = Tensor::share(DataType::FP16, Shape{2, 2, 64, 128});
    auto at = AttentionCollector(T::Amd, 64).filter({*q, *kv, *kv, *past}, {*q, *cache, *cache});
    EXPECT(at.size() == 1);
    auto const &info = static_cast<AttentionHip const &>(*at[0]).info;
    EXPECT(info.batch == 2 && info.nHead == 8 && info.nKVHead == 2 && info.seqLen == 1 && info.cacheLen == 64 &&
           info.headDim == 128 && info.pastFromInput && info.pastCount == 1 && !info.resetCache);
    auto kv3 = Tensor::share(DataType::FP16, Shape{2, 3, 1, 128});
    EXPECT(AttentionCollector(T::Amd, 64).filter({*q, *kv3, *kv3, *past}, {*q, *cache, *cache}).empty());
    auto q32 = Tensor::share(DataType::F32, Shape{2, 8, 1, 128});
    EXPECT(AttentionCollector(T::Amd, 0).filter({*q32, *q32, *q32}, {*q32}).empty());

    auto xr = Tensor::share(DataType::FP16, Shape{2, 5, 4, 64});
    auto pos = Tensor::share(DataType::I64, Shape{2, 5});
    auto posBad = Tensor::share(DataType::I64, Shape{7});
    EXPECT(RotaryEmbeddingCollector(T::Amd, 10000.f).filter({*xr, *pos}, {*xr}).size() == 1);
    EXPECT(RotaryEmbeddingCollector(T::Amd, 10000.f).filter({*xr, *posBad}, {*xr}).empty());
}

// ------------------------------------------------------------------ routines on the AMD device

static Device &amd() { return *device::init(Device::Type::Amd, 0, "pool=4294967296"); }

static void rmsNormalizationHip() {
    // src/04kernel/test/kernels/rms_normalization/test_cuda.cpp:13-52 (x = 2, w = 3 -> 3), then random
    auto x = Tensor::share(DataType::F32, Shape{2, 3, 4096});
    auto w = Tensor::share(DataType::F32, Shape{4096});
    auto kernels = RmsNormalizationCollector(Device::Type::Amd, 0).filter({*x, *w}, {*x});
    EXPECT(kernels.size() == 1);
    runtime::Resources res;
    auto routine = kernels[0]->lower(res).routine;
    auto &dev = amd();
    auto yGpu = dev.malloc(x->bytesSize()), xGpu = dev.malloc(x->bytesSize()), wGpu = dev.malloc(w->bytesSize());
    std::vector<float> x_(x->elementsSize(), 2), w_(w->elementsSize(), 3), y_(x->elementsSize()), ref(x->elementsSize());
    for (int round = 0; round < 2; ++round) {
        if (round == 1) {
            std::mt19937 rng(1);
            std::normal_distribution<float> n01;
            std::uniform_real_distribution<float> u(0.5f, 1.5f);
            for (auto &v : x_) v = n01(rng);
            for (auto &v : w_) v = u(rng);
            routine = RmsNormalizationHip::build(1e-5f, *x)->lower(res).routine;
        }
        xGpu->copyFromHost(x_.data());
        wGpu->copyFromHost(w_.data());
        void const *inputs[]{*xGpu, *wGpu};
        void *outputs[]{*yGpu};
        routine(res, nullptr, inputs, outputs);
        yGpu->copyToHost(y_.data());
        oracle_rms_norm_f32(ref.data(), x_.data(), w_.data(), 6, 4096, round ? 1e-5f : 0.f, 1);
        bool ok = true;
        for (size_t i = 0; i < y_.size(); ++i) ok &= std::fabs(y_[i] - ref[i]) <= 1e-5f * std::fabs(ref[i]);
        EXPECT(ok);
        if (round == 0) EXPECT(y_[0] == 3.0f && y_.back() == 3.0f);
    }
}

static void softmaxHip() {
    auto x = Tensor::share(DataType::F32, Shape{2, 3, 2, 5});
    runtime::Resources res;
    auto &dev = amd();
    std::mt19937 rng(3);
    std::normal_distribution<float> n(0, 3);
    std::vector<float> x_(x->elementsSize()), y_(x_.size()), ref(x_.size());
    for (auto &v : x_) v = n(rng);
    auto xGpu = dev.malloc(x->bytesSize()), yGpu = dev.malloc(x->bytesSize());
    xGpu->copyFromHost(x_.data());
    for (dim_t axis = 0; axis < 4; ++axis) {// the reference's test uses axis 1 (softmax/test_cpu.cpp:8-31)
        auto kernels = SoftmaxCollector(Device::Type::Amd, axis).filter({*x}, {*x});
        EXPECT(kernels.size() == 1);
        auto routine = kernels[0]->lower(res).routine;
        void const *inputs[]{*xGpu};
        void *outputs[]{*yGpu};
        routine(res, nullptr, inputs, outputs);
        yGpu->copyToHost(y_.data());
        SoftmaxInfo info(*x, axis);
        oracle_softmax_f32(ref.data(), x_.data(), info.pre, info.mid, info.post, 1);
        bool ok = true;
        for (size_t i = 0; i < y_.size(); ++i) ok &= std::fabs(y_[i] - ref[i]) <= 1e-5f * ref[i];
        EXPECT(ok);
    }
    // causal, fp16
    auto h = Tensor::share(DataType::FP16, Shape{3, 32, 32});
    std::vector<uint16_t> h_(h->elementsSize()), hy(h_.size());
    std::vector<float> hf(h_.size()), href(h_.size());
    for (size_t i = 0; i < h_.size(); ++i) { h_[i] = f2h(n(rng)); hf[i] = h2f(h_[i]); }
    auto hGpu = dev.malloc(h->bytesSize()), hyGpu = dev.malloc(h->bytesSize());
    hGpu->copyFromHost(h_.data());
    auto routine = SoftmaxCollector(Device::Type::Amd, 2, true).filter({*h}, {*h})[0]->lower(res).routine;
    void const *inputs[]{*hGpu};
    void *outputs[]{*hyGpu};
    routine(res, nullptr, inputs, outputs);
    hyGpu->copyToHost(hy.data());
    oracle_softmax_causal_f32(href.data(), hf.data(), 3, 32, 32, 1);
    bool ok = true;
    for (size_t i = 0; i < hy.size(); ++i) ok &= std::fabs(h2f(hy[i]) - href[i]) <= 2e-3f;
    EXPECT(ok && h2f(hy[1]) == 0.f && h2f(hy[0]) == 1.f);
}

static void matMulIntegerHip() {
    runtime::Resources res;
    auto &dev = amd();
    {// src/04kernel/test/kernels/mat_mul_integer/test_cublas_kernel.cpp:13-59
        auto A = Tensor::share(DataType::U8, Shape{1, 4});
        auto B = Tensor::share(DataType::U8, Shape{4, 12});
        auto Y = Tensor::share(DataType::I32, Shape{1, 12});
        auto kernels = MatMulIntegerCollector(Device::Type::Amd).filter({*A, *B}, {*Y});
        EXPECT(kernels.size() == 1);
        auto [routine, workspace] = kernels[0]->lower(res);
        EXPECT(workspace == 0);// the reference's kernels need none either when there is no zero point
        std::vector<uint8_t> a(4), b(48);
        std::iota(a.begin(), a.end(), 1);
        for (int r = 0; r < 4; ++r) std::iota(b.begin() + 12 * r, b.begin() + 12 * (r + 1), 1);
        auto ma = dev.malloc(4), mb = dev.malloc(48), my = dev.malloc(48);
        ma->copyFromHost(a.data());
        mb->copyFromHost(b.data());
        void const *inputs[]{*ma, *mb};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        std::vector<int32_t> y(12);
        my->copyToHost(y.data());
        bool ok = true;
        for (int j = 0; j < 12; ++j) ok &= y[j] == 10 * (j + 1);
        EXPECT(ok);
    }
    {// zero points as device tensors, MFMA-sized, broadcast batch; bit-exact against the oracle
        auto A = Tensor::share(DataType::U8, Shape{2, 1, 256, 128});
        auto B = Tensor::share(DataType::I8, Shape{3, 128, 256});
        auto az = Tensor::share(DataType::U8, Shape{});
        auto bz = Tensor::share(DataType::I8, Shape{});
        auto Y = Tensor::share(DataType::I32, Shape{2, 3, 256, 256});
        auto kernels = MatMulIntegerCollector(Device::Type::Amd).filter({*A, *B, *az, *bz}, {*Y});
        auto [routine, workspace] = kernels[0]->lower(res);
        // the CPU kernel of the reference needs batch*(m*k + k*n) bytes here
        EXPECT(workspace <= 6 * (256 * 128 + 128 * 256));
        std::mt19937 rng(5);
        std::vector<uint8_t> a(A->elementsSize()), b(B->elementsSize());
        for (auto &v : a) v = rng();
        for (auto &v : b) v = rng();
        uint8_t azv = 128;
        int8_t bzv = 3;
        auto ma = dev.malloc(a.size()), mb = dev.malloc(b.size()), my = dev.malloc(Y->bytesSize()),
             maz = dev.malloc(1), mbz = dev.malloc(1), ws = dev.malloc(workspace ? workspace : 1);
        ma->copyFromHost(a.data());
        mb->copyFromHost(b.data());
        maz->copyFromHost(&azv);
        mbz->copyFromHost(&bzv);
        void const *inputs[]{*ma, *mb, *maz, *mbz};
        void *outputs[]{*my};
        routine(res, *ws, inputs, outputs);
        std::vector<int32_t> y(Y->elementsSize()), ref(y.size());
        my->copyToHost(y.data());
        uint32_t aOff[6], bOff[6];
        for (dim_t i = 0; i < 6; ++i) { aOff[i] = i / 3; bOff[i] = i % 3; }
        oracle_matmul_integer(ref.data(), a.data(), b.data(), &azv, 0, 1, &bzv, 1, 1, 6, 256, 128, 256, aOff, bOff, 2, 3, 8);
        EXPECT(y == ref);
    }
}

static void dynamicQuantizeLinearHip() {
    runtime::Resources res;
    auto &dev = amd();
    auto run = [&](std::vector<float> const &x_) {
        auto const n = x_.size();
        auto x = Tensor::share(DataType::F32, Shape{static_cast<dim_t>(n)});
        auto y = Tensor::share(DataType::U8, Shape{static_cast<dim_t>(n)});
        auto scale = Tensor::share(DataType::F32, Shape{});
        auto zp = Tensor::share(DataType::U8, Shape{});
        auto kernels = DynamicQuantizeLinearCollector(Device::Type::Amd).filter({*x}, {*y, *scale, *zp});
        EXPECT(kernels.size() == 1);
        auto [routine, workspaceSize] = kernels[0]->lower(res);
        auto mx = dev.malloc(n * 4), my = dev.malloc(n), ms = dev.malloc(4), mz = dev.malloc(1),
             ws = dev.malloc(workspaceSize);
        mx->copyFromHost(x_.data());
        void const *inputs[]{*mx};
        void *outputs[]{*my, *ms, *mz};
        routine(res, *ws, inputs, outputs);
        std::vector<uint8_t> yData(n), ref(n);
        float s, sRef;
        uint8_t z, zRef;
        my->copyToHost(yData.data());
        ms->copyToHost(&s);
        mz->copyToHost(&z);
        oracle_dynamic_quantize_linear(ref.data(), &sRef, &zRef, x_.data(), n);
        EXPECT(yData == ref && s == sRef && z == zRef);
        return std::tuple{yData, s, z};
    };
    {// src/04kernel/test/kernels/dynamic_quantize_linear/test_cpu.cpp:8-39
        auto [y, s, z] = run({0, 2, -3, -2.5, 1.34, 0.5});
        EXPECT(s == (2 + 3) / 255.f && z == 153);
        std::vector<float> x{0, 2, -3, -2.5, 1.34, 0.5};
        for (size_t i = 0; i < x.size(); ++i) EXPECT(y[i] == static_cast<uint8_t>(std::round(x[i] / s) + z));
    }
    {// src/04kernel/test/kernels/dynamic_quantize_linear/test_cuda.cpp:14-73 (device result == CPU result)
        std::vector<float> x(20);
        for (size_t i = 0; i < x.size(); ++i) x[i] = i * 3 + 15;
        run(x);
    }
    {
        std::mt19937 rng(11);
        std::normal_distribution<float> g(0.f, 3.f);
        std::vector<float> x(100003);
        for (auto &v : x) v = g(rng);
        run(x);
    }
    // anything but float -> (uint8, float, uint8) is declined
    auto xh = Tensor::share(DataType::FP16, Shape{8});
    auto y = Tensor::share(DataType::U8, Shape{8});
    auto scale = Tensor::share(DataType::F32, Shape{});
    auto zp = Tensor::share(DataType::U8, Shape{});
    EXPECT(DynamicQuantizeLinearCollector(Device::Type::Amd).filter({*xh}, {*y, *scale, *zp}).empty());
}

static void matMulHip() {
    runtime::Resources res;
    auto &dev = amd();
    auto run = [&](Tensor const &A, Tensor const &B, Tensor const *C, Tensor const &Y, std::vector<float> const &a,
                   std::vector<float> const &b, std::vector<float> const &c) {
        auto kernels = C ? MatMulCollector(Device::Type::Amd, 1, 1, false, false).filter({A, B, *C}, {Y})
                         : MatMulCollector(Device::Type::Amd, 1, 1, false, false).filter({A, B}, {Y});
        EXPECT(kernels.size() == 1);
        auto routine = kernels[0]->lower(res).routine;
        auto ma = dev.malloc(a.size() * 4), mb = dev.malloc(b.size() * 4), mc = dev.malloc(std::max<size_t>(c.size(), 1) * 4),
             my = dev.malloc(Y.elementsSize() * 4);
        ma->copyFromHost(a.data());
        mb->copyFromHost(b.data());
        if (!c.empty()) mc->copyFromHost(c.data());
        void const *inputs[]{*ma, *mb, *mc};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        std::vector<float> y(Y.elementsSize());
        my->copyToHost(y.data());
        return y;
    };
    {// src/04kernel/test/kernels/mat_mul/test_cpu.cpp:24-39 and test_cublas.cpp (same vectors on the device)
        auto A = Tensor::share(DataType::F32, Shape{1, 2, 2});
        auto B = Tensor::share(DataType::F32, Shape{2, 2});
        auto C = Tensor::share(DataType::F32, Shape{});
        auto Y = Tensor::share(DataType::F32, Shape{2, 2});
        auto y = run(*A, *B, C.get(), *Y, {1.0, 2.0, 0.0, 0.5}, {1.0, 2.0, 0.0, 0.5}, {1.0});
        EXPECT((y == std::vector<float>{2, 4, 1, 1.25}));
    }
    {// test_cpu.cpp:57-79: both operands broadcast over the batch, bias [2, 1]
        auto A = Tensor::share(DataType::F32, Shape{2, 1, 2, 2});
        auto B = Tensor::share(DataType::F32, Shape{1, 2, 2, 2});
        auto C = Tensor::share(DataType::F32, Shape{2, 1});
        auto Y = Tensor::share(DataType::F32, Shape{2, 2, 2, 2});
        auto y = run(*A, *B, C.get(), *Y, {1.0, 2.0, 0.0, 0.5, 1.0, 0.0, 0.0, 1.0}, {1.0, 2.0, 0.0, 0.5, 1.0, 0.0, 0.0, 1.0},
                     {1.0, 0.0});
        EXPECT((y == std::vector<float>{2.0, 4.0, 0.0, 0.25, 2.0, 3.0, 0.0, 0.5, 2.0, 3.0, 0.0, 0.5, 2.0, 1.0, 0.0, 1.0}));
    }
    {// against the oracle's serial loop, float, odd sizes, no bias
        std::mt19937 rng(9);
        std::uniform_int_distribution<int> g(-4, 4);  // integer-valued: every partial sum is exact
        dim_t const m = 37, k = 53, n = 29;
        std::vector<float> a(m * k), b(k * n), ref(m * n, 0.f);
        for (auto &v : a) v = static_cast<float>(g(rng));
        for (auto &v : b) v = static_cast<float>(g(rng));
        auto A = Tensor::share(DataType::F32, Shape{m, k});
        auto B = Tensor::share(DataType::F32, Shape{k, n});
        auto Y = Tensor::share(DataType::F32, Shape{m, n});
        auto y = run(*A, *B, nullptr, *Y, a, b, {});
        oracle_matmul_bias_f32(ref.data(), a.data(), b.data(), m, k, n, k, 1, n, 1, 1.f, 0.f);
        EXPECT(y == ref);
    }
}

static void castHip() {
    runtime::Resources res;
    auto &dev = amd();
    {// src/04kernel/test/kernels/cast/test_cpu.cpp:8-33 and test_cuda.cpp: F64 iota [2,3,4,5] -> I8, y[i] == i
        auto x = Tensor::share(DataType::F64, Shape{2, 3, 4, 5});
        auto y = Tensor::share(DataType::I8, Shape{2, 3, 4, 5});
        auto kernels = CastCollector(Device::Type::Amd).filter({*x}, {*y});
        EXPECT(kernels.size() == 1);
        auto routine = kernels[0]->lower(res).routine;
        std::vector<double> x_(x->elementsSize());
        std::iota(x_.begin(), x_.end(), 0);
        auto mx = dev.malloc(x_.size() * 8), my = dev.malloc(x_.size());
        mx->copyFromHost(x_.data());
        void const *inputs[]{*mx};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        std::vector<int8_t> y_(x_.size());
        my->copyToHost(y_.data());
        for (size_t i = 0; i < y_.size(); ++i) EXPECT(y_[i] == static_cast<int8_t>(i));
    }
    {// float -> int32 -> float on values the reference's static_cast defines; odd length
        std::mt19937 rng(5);
        std::uniform_real_distribution<float> g(-1e6f, 1e6f);
        std::vector<float> x_(10007);
        for (auto &v : x_) v = g(rng);
        auto x = Tensor::share(DataType::F32, Shape{10007});
        auto y = Tensor::share(DataType::I32, Shape{10007});
        auto k1 = CastCollector(Device::Type::Amd).filter({*x}, {*y});
        auto k2 = CastCollector(Device::Type::Amd).filter({*y}, {*x});
        EXPECT(k1.size() == 1 && k2.size() == 1);
        auto mx = dev.malloc(x_.size() * 4), my = dev.malloc(x_.size() * 4), mz = dev.malloc(x_.size() * 4);
        mx->copyFromHost(x_.data());
        {
            void const *inputs[]{*mx};
            void *outputs[]{*my};
            k1[0]->lower(res).routine(res, nullptr, inputs, outputs);
        }
        {
            void const *inputs[]{*my};
            void *outputs[]{*mz};
            k2[0]->lower(res).routine(res, nullptr, inputs, outputs);
        }
        std::vector<int32_t> y_(x_.size());
        std::vector<float> z_(x_.size());
        my->copyToHost(y_.data());
        mz->copyToHost(z_.data());
        for (size_t i = 0; i < x_.size(); ++i)
            EXPECT(y_[i] == static_cast<int32_t>(x_[i]) && z_[i] == static_cast<float>(y_[i]));
    }
}

static void dequantizeLinearHip() {
    runtime::Resources res;
    auto &dev = amd();
    {// src/04kernel/test/kernels/dequantize_linear/test_cpu.cpp:8-31
        auto x = Tensor::share(DataType::U8, Shape{4});
        auto scale = Tensor::share(DataType::F32, Shape{});
        auto zp = Tensor::share(DataType::U8, Shape{});
        auto y = Tensor::share(DataType::F32, Shape{4});
        auto kernels = DequantizeLinearCollector(Device::Type::Amd).filter({*x, *scale, *zp}, {*y});
        EXPECT(kernels.size() == 1);
        auto routine = kernels[0]->lower(res).routine;
        uint8_t xData[]{0, 3, 128, 255}, zp_ = 128;
        float scale_ = 2;
        auto mx = dev.malloc(4), ms = dev.malloc(4), mz = dev.malloc(1), my = dev.malloc(16);
        mx->copyFromHost(xData);
        ms->copyFromHost(&scale_);
        mz->copyFromHost(&zp_);
        void const *inputs[]{*mx, *ms, *mz};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        float yData[4];
        my->copyToHost(yData);
        EXPECT(yData[0] == -256 && yData[1] == -250 && yData[2] == 0 && yData[3] == 254);
    }
    {// per-axis scale on axis 1, bit-exact
        auto x = Tensor::share(DataType::I8, Shape{64, 256});
        auto scale = Tensor::share(DataType::F32, Shape{256});
        auto y = Tensor::share(DataType::F32, Shape{64, 256});
        auto routine = DequantizeLinearCollector(Device::Type::Amd, 1).filter({*x, *scale}, {*y})[0]->lower(res).routine;
        std::mt19937 rng(7);
        std::vector<int8_t> x_(x->elementsSize());
        std::vector<float> s_(256), y_(x_.size()), ref(x_.size());
        for (auto &v : x_) v = rng();
        std::uniform_real_distribution<float> u(1e-3f, 1e-2f);
        for (auto &v : s_) v = u(rng);
        auto mx = dev.malloc(x_.size()), ms = dev.malloc(1024), my = dev.malloc(y->bytesSize());
        mx->copyFromHost(x_.data());
        ms->copyFromHost(s_.data());
        void const *inputs[]{*mx, *ms};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        my->copyToHost(y_.data());
        oracle_dequantize_linear(ref.data(), x_.data(), s_.data(), nullptr, 64, 256, 1, ORACLE_I8, 256, 1);
        EXPECT(std::memcmp(y_.data(), ref.data(), y_.size() * 4) == 0);
    }
}

static void attentionHip() {
    // decode with a persistent cache (4 inputs, max_seq_len = S): two consecutive steps through
    // the same Resources, past_seq_len read from device memory each time
    constexpr dim_t N = 2, H = 8, Hkv = 2, D = 128, S = 96;
    auto q = Tensor::share(DataType::FP16, Shape{N, H, 1, D});
    auto kv = Tensor::share(DataType::FP16, Shape{N, Hkv, 1, D});
    auto past = Tensor::share(DataType::I64, Shape{N});
    auto cache = Tensor::share(DataType::FP16, Shape{N, Hkv, S, D});
    auto kernels = AttentionCollector(Device::Type::Amd, S).filter({*q, *kv, *kv, *past}, {*q, *cache, *cache});
    EXPECT(kernels.size() == 1);
    runtime::Resources res;
    auto [routine, workspace] = kernels[0]->lower(res);
    EXPECT(workspace > 0 && res.fetch<HipAttentionState>() != nullptr);
    auto &dev = amd();
    std::mt19937 rng(9);
    std::normal_distribution<float> n01;
    auto randomHalf = [&](size_t n) { std::vector<uint16_t> v(n); for (auto &e : v) e = f2h(n01(rng)); return v; };
    auto kc = randomHalf(cache->elementsSize()), vc = randomHalf(cache->elementsSize());
    auto mq = dev.malloc(q->bytesSize()), mk = dev.malloc(kv->bytesSize()), mv = dev.malloc(kv->bytesSize()),
         mp = dev.malloc(N * 8), mo = dev.malloc(q->bytesSize()), mkc = dev.malloc(cache->bytesSize()),
         mvc = dev.malloc(cache->bytesSize()), ws = dev.malloc(workspace);
    mkc->copyFromHost(kc.data());
    mvc->copyFromHost(vc.data());
    int64_t pastLen[N] = {40, 7};
    float const scale = 1.0f / std::sqrt(static_cast<float>(D));
    for (int step = 0; step < 2; ++step) {
        auto q_ = randomHalf(q->elementsSize()), k_ = randomHalf(kv->elementsSize()), v_ = randomHalf(kv->elementsSize());
        mq->copyFromHost(q_.data());
        mk->copyFromHost(k_.data());
        mv->copyFromHost(v_.data());
        mp->copyFromHost(pastLen);
        void const *inputs[]{*mq, *mk, *mv, *mp};
        void *outputs[]{*mo, *mkc, *mvc};
        routine(res, *ws, inputs, outputs);
        std::vector<uint16_t> o(q->elementsSize()), kcOut(kc.size()), vcOut(vc.size());
        mo->copyToHost(o.data());
        mkc->copyToHost(kcOut.data());
        mvc->copyToHost(vcOut.data());
        // expected caches: the new row appended at past_b
        for (dim_t b = 0; b < N; ++b)
            for (dim_t h = 0; h < Hkv; ++h) {
                std::memcpy(&kc[((b * Hkv + h) * S + pastLen[b]) * D], &k_[(b * Hkv + h) * D], D * 2);
                std::memcpy(&vc[((b * Hkv + h) * S + pastLen[b]) * D], &v_[(b * Hkv + h) * D], D * 2);
            }
        EXPECT(kcOut == kc && vcOut == vc);
        bool ok = true;
        std::vector<float> scratch(2 * S), ref(D), qf(D);
        for (dim_t b = 0; b < N; ++b)
            for (dim_t h = 0; h < H; ++h) {
                dim_t const len = pastLen[b] + 1, kh = h / (H / Hkv);
                std::vector<float> kf(len * D), vf(len * D);
                for (size_t i = 0; i < len * D; ++i) {
                    kf[i] = h2f(kc[(b * Hkv + kh) * S * D + i]);
                    vf[i] = h2f(vc[(b * Hkv + kh) * S * D + i]);
                }
                for (dim_t i = 0; i < D; ++i) qf[i] = h2f(q_[(b * H + h) * D + i]);
                oracle_attention_head_f32(ref.data(), qf.data(), kf.data(), vf.data(), 1, pastLen[b], D, scale, 1, scratch.data());
                for (dim_t i = 0; i < D; ++i) ok &= std::fabs(h2f(o[(b * H + h) * D + i]) - ref[i]) <= 2e-3f;
            }
        EXPECT(ok);
        for (auto &p : pastLen) ++p;
    }
}

static void rotaryEmbeddingHip() {
    constexpr dim_t B = 2, S = 33, H = 4, D = 64;
    auto x = Tensor::share(DataType::FP16, Shape{B, S, H, D});
    auto pos = Tensor::share(DataType::I64, Shape{B, S});
    runtime::Resources res;
    auto routine = RotaryEmbeddingCollector(Device::Type::Amd, 10000.f).filter({*x, *pos}, {*x})[0]->lower(res).routine;
    auto &dev = amd();
    std::mt19937 rng(4);
    std::normal_distribution<float> n01;
    std::vector<uint16_t> x_(x->elementsSize()), y_(x_.size());
    std::vector<float> xf(x_.size()), ref(x_.size());
    for (size_t i = 0; i < x_.size(); ++i) { x_[i] = f2h(n01(rng)); xf[i] = h2f(x_[i]); }
    std::vector<int64_t> p(B * S);
    for (dim_t i = 0; i < B * S; ++i) p[i] = (i % S) * 61 % 2048;
    auto mx = dev.malloc(x->bytesSize()), mp = dev.malloc(p.size() * 8), my = dev.malloc(x->bytesSize());
    mx->copyFromHost(x_.data());
    mp->copyFromHost(p.data());
    void const *inputs[]{*mx, *mp};
    void *outputs[]{*my};
    routine(res, nullptr, inputs, outputs);
    my->copyToHost(y_.data());
    oracle_rope_f32(ref.data(), xf.data(), p.data(), 1, B, S, H, D, 10000.f, 1);
    bool ok = true;
    for (size_t i = 0; i < y_.size(); ++i) ok &= std::fabs(h2f(y_[i]) - ref[i]) <= 2e-3f;
    EXPECT(ok);
}

static void amdDeviceAndPool() {
    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    EXPECT(dev && dev->type() == Device::Type::Amd && device::fetch(Device::Type::Amd) == dev);
    auto a = dev->malloc(1000), b = dev->malloc(1000);
    EXPECT(reinterpret_cast<uintptr_t>(a->get()) % 256 == 0 && reinterpret_cast<uintptr_t>(b->get()) % 256 == 0);
    std::vector<uint8_t> src(1000), dst(1000);
    std::iota(src.begin(), src.end(), 0);
    a->copyFromHost(src.data());
    b->copyFrom(*a);
    b->copyToHost(dst.data());
    EXPECT(src == dst);
    auto onCpu = device::fetch(Device::Type::Cpu)->malloc(1000);
    onCpu->copyFrom(*b);// device -> host blob
    EXPECT(std::memcmp(onCpu->get(), src.data(), 1000) == 0);
    device::sync(Device::Type::Amd);
    EXPECT(throws<std::runtime_error>([&] { dev->malloc(1ul << 40); }));
}

int main(int argc, char **argv) {
    std::string mode = argc > 1 ? argv[1] : "cpu";
    RUN(broadcasterKnownAnswer);
    RUN(shapeDigests);
    RUN(memPoolBestFit);
    RUN(resourcesAndErrors);
    RUN(collectorsSelectOrDecline);
    if (mode == "gpu") {
        RUN(amdDeviceAndPool);
        RUN(rmsNormalizationHip);
        RUN(softmaxHip);
        RUN(matMulIntegerHip);
        RUN(dequantizeLinearHip);
        RUN(dynamicQuantizeLinearHip);
        RUN(castHip);
        RUN(matMulHip);
        RUN(attentionHip);
        RUN(rotaryEmbeddingHip);
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
