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
#include "kernel/attributes/transpose_info.h"
#include "kernel/collectors/transpose.h"
#include "kernel/attributes/expand_info.h"
#include "kernel/attributes/split_info.h"
#include "kernel/collectors/concat.h"
#include "kernel/collectors/expand.h"
#include "kernel/collectors/split.h"
#include "kernel/collectors/where.h"
#include "computation/operators/split.h"
#include "computation/operators/transpose.h"
#include "kernel/collectors/attention.h"
#include "kernel/collectors/dequantize_linear.h"
#include "kernel/collectors/dynamic_quantize_linear.h"
#include "kernel/collectors/mat_mul_integer.h"
#include "kernel/collectors/rms_normalization.h"
#include "kernel/collectors/rotary_embedding.h"
#include "kernel/collectors/softmax.h"
#include "computation/graph.h"
#include "computation/operators/attention.h"
#include "computation/operators/reshape.h"
#include "graph_topo.h"
#include "hardware/device_manager.h"
#include "hardware/mem_offset_calculator.h"
#include "kernel/allocators.h"
#include "kernel/graph.h"
#include "runtime/stream.h"
#include "hardware/mem_pool.h"
#include "rg_mirror/executor.h"
#include "rg_mirror/hip_kernels.h"
#include "oracle.h"

#include <chrono>
#include <cmath>
#include <immintrin.h>
#include <cstdio>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <numeric>
#include <random>
#include <tuple>
#include <unistd.h>

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
// every case prints its name before it starts and its verdict when it returns, so that the
// output of one run of the driver can be split into one result per case
#define RUN(NAME)                                                                   \
    do {                                                                            \
        if (!only.empty() && only != #NAME) break;                                  \
        std::printf("[ RUN  ] %s\n", #NAME);                                        \
        std::fflush(stdout);                                                        \
        int const failedBefore = g_failed;                                          \
        try {                                                                       \
            NAME();                                                                 \
        } catch (std::exception const &e) {                                         \
            ++g_failed;                                                             \
            std::printf("  FAILED %s: exception: %s\n", #NAME, e.what());           \
        }                                                                           \
        std::printf("[ %s ] %s\n", g_failed == failedBefore ? " OK " : "FAIL", #NAME); \
        std::fflush(stdout);                                                        \
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
        // a bias that broadcasts over one batch dimension only is expanded into a workspace first
        MatMulInfo odd(*a, *bt, std::cref(*cOdd), false, true, 1.f, 1.f);
        EXPECT(odd.biasSupported && (odd.biasExpandFrom == std::vector<dim_t>{2, 1, 5, 4}) &&
               (odd.biasExpandTo == std::vector<dim_t>{2, 3, 5, 4}) && odd.biasStrideBatch == 20 && odd.biasStrideM == 4);
        EXPECT(MatMulCollector(T::Amd, 1, 1, false, true).filter({*a, *bt, *cRow}, {*cFull}).size() == 1);
        {
            auto ks = MatMulCollector(T::Amd, 1, 1, false, true).filter({*a, *bt, *cOdd}, {*cFull});
            runtime::Resources res_;
            EXPECT(ks.size() == 1 && ks[0]->lower(res_).workspaceOffset == 2 * 3 * 5 * 4 * 4);
        }
        // one that does not broadcast at all is declined
        auto cBad = Tensor::share(DataType::F32, Shape{3, 1, 5, 4});
        EXPECT(!MatMulInfo(*a, *bt, std::cref(*cBad), false, true, 1.f, 1.f).biasSupported);
        EXPECT(MatMulCollector(T::Amd, 1, 1, false, true).filter({*a, *bt, *cBad}, {*cFull}).empty());
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

// ------------------------------------------------------------------ graph -> stream (host logic)

static void graphTopoAndBuilder() {
    using graph_topo::Builder;
    // keys chosen so that key order ("a" < "b") is the reverse of the order the nodes can run in
    Builder<std::string, int, std::string, int> b;
    b.topology["b"] = {{"x", "w0"}, {"t0"}};
    b.topology["a"] = {{"t0", "w1", "x"}, {"t1", "t2"}};
    b.globalInputs = {"x"};
    b.globalOutputs = {"t2", "t0"};
    b.nodes = {{"a", 11}, {"b", 22}};
    b.edges = {{"x", 100}, {"w0", 101}, {"w1", 103}, {"t0", 102}, {"t2", 105}};
    auto g = b.build();
    auto const &t = g.topology;
    EXPECT(t.nodeCount() == 2 && t.edgeCount() == 6 && t.globalInputsCount() == 1 && t.globalOutputsCount() == 2);
    EXPECT((g.nodes == std::vector<int>{22, 11}));
    // numbering: x | w0 t0 | w1 t1 t2   (t1 has no value of its own: default-constructed)
    EXPECT((g.edges == std::vector<int>{100, 101, 102, 103, 0, 105}));
    std::vector<count_t> conn(t.connections().begin(), t.connections().end());
    EXPECT((conn == std::vector<count_t>{5, 2, 0, 1, 2, 3, 0}));
    EXPECT(t.globalOutputs().size() == 2 && t.globalOutputs()[0] == 5 && t.globalOutputs()[1] == 2);
    size_t seen = 0;
    for (auto [idx, inputs, outputs] : t) {
        if (idx == 0) EXPECT(inputs.size() == 2 && inputs[0] == 0 && inputs[1] == 1 && outputs.size() == 1 && outputs[0] == 2);
        if (idx == 1) EXPECT(inputs.size() == 3 && inputs[0] == 2 && inputs[1] == 3 && inputs[2] == 0 && outputs.size() == 2 && outputs[0] == 4 && outputs[1] == 5);
        ++seen;
    }
    EXPECT(seen == 2);
    EXPECT(t.node(1).outputs.at(1) == 5 && t.firstEdgeOf(1) == 3 && t.localEdgesOf(1) == 1);
    EXPECT(throws<std::runtime_error>([&] { t.node(2); }));
    EXPECT(t.toString().find("node 1: 2 3 0 -> 4 5") != std::string::npos);
    // two nodes that wait for each other cannot be ordered
    Builder<int, int, int, int> cyc;
    cyc.topology[0] = {{1}, {0}};
    cyc.topology[1] = {{0}, {1}};
    cyc.nodes = {{0, 0}, {1, 1}};
    EXPECT(throws<std::runtime_error>([&] { cyc.build(); }));
    // hand-built topology: an edge numbered after the node's own cannot be read
    graph_topo::GraphTopo manual(1, 1);
    EXPECT(manual.pushNode({0}, 0, 1).begin_ == 1);
    EXPECT(throws<std::runtime_error>([&] { manual.pushNode({3}, 0, 1); }));
    manual.setGlobalOutput(0, 1);
    EXPECT(manual.globalOutputs()[0] == 1);
}

static void offsetCalculatorPlan() {
    OffsetCalculator c(8);
    EXPECT(c.alloc(10) == 0 && c.alloc(20) == 16 && c.alloc(8) == 40 && c.peak() == 48);
    c.free(16, 20);                                  // free: [16, 40)
    EXPECT(c.alloc(8) == 16);                        // best (only) fit, split: [24, 40) stays free
    EXPECT(c.alloc(16) == 24 && c.peak() == 48);     // exact fit
    c.free(40, 8);                                   // the free block now touches the end
    EXPECT(c.alloc(32) == 40 && c.peak() == 72);     // too small, grows with the range
    c.free(0, 10);
    c.free(24, 16);
    c.free(16, 8);                                   // merges with both neighbours: [0, 40)
    EXPECT(c.alloc(40) == 0 && c.peak() == 72);
    // best fit prefers the smaller of two free blocks
    OffsetCalculator d(1);
    auto a0 = d.alloc(100), a1 = d.alloc(10), a2 = d.alloc(50), a3 = d.alloc(10);
    d.free(a0, 100);
    d.free(a2, 50);
    EXPECT(d.alloc(40) == a2 && d.alloc(60) == a0 && a1 == 100 && a3 == 160 && d.peak() == 170);
    EXPECT(throws<std::runtime_error>([&] { d.free(a1, 10); d.free(a1, 10); }));
    EXPECT(alignBytes(100, 32) == 128 && alignBytes(128, 32) == 128 && alignBytes(0, 32) == 0);
}

namespace {
    // y[i] = x[i] + addend over `n` floats; with `viaWorkspace` the sum is formed in the workspace first
    class AddKernel final : public Kernel {
        float _addend;
        size_t _n;
        bool _viaWorkspace;

    public:
        AddKernel(float addend, size_t n, bool viaWorkspace) : _addend(addend), _n(n), _viaWorkspace(viaWorkspace) {}
        static size_t typeId() noexcept {
            static uint8_t ID = 1;
            return reinterpret_cast<size_t>(&ID);
        }
        size_t kernelTypeId() const final { return typeId(); }
        std::string_view description() const final { return "test kernel: add a constant on the host"; }
        RoutineWorkspace lower(Resources &) const final {
            auto routine = [addend = _addend, n = _n, ws = _viaWorkspace](Resources &, void *workspace, void const *const *inputs, void *const *outputs) {
                auto x = static_cast<float const *>(inputs[0]);
                auto y = static_cast<float *>(outputs[0]);
                auto t = ws ? static_cast<float *>(workspace) : y;
                for (size_t i = 0; i < n; ++i) t[i] = x[i] + addend;
                if (ws) std::memcpy(y, t, n * sizeof(float));
            };
            return {std::move(routine), _viaWorkspace ? _n * sizeof(float) : 0};
        }
    };
    // y = a + b
    class SumKernel final : public Kernel {
        size_t _n;

    public:
        explicit SumKernel(size_t n) : _n(n) {}
        static size_t typeId() noexcept {
            static uint8_t ID = 1;
            return reinterpret_cast<size_t>(&ID);
        }
        size_t kernelTypeId() const final { return typeId(); }
        std::string_view description() const final { return "test kernel: add two tensors on the host"; }
        RoutineWorkspace lower(Resources &) const final {
            return [n = _n](Resources &, void *, void const *const *inputs, void *const *outputs) {
                auto a = static_cast<float const *>(inputs[0]), b = static_cast<float const *>(inputs[1]);
                auto y = static_cast<float *>(outputs[0]);
                for (size_t i = 0; i < n; ++i) y[i] = a[i] + b[i];
            };
        }
    };
}// namespace

// x -> (+1) -> t0 -> (+2, workspace) -> t1 -> (+ c) -> t2 -> (+4) -> y, with c a constant edge and an
// unused second output nobody reads
static kernel::Graph chainGraph(size_t n, Arc<kernel::Blob> constant) {
    graph_topo::GraphTopo topo(1, 1);
    topo.pushNode({0}, 0, 1);       // edge 1 = t0
    topo.pushNode({1}, 0, 1);       // edge 2 = t1
    topo.pushNode({2, 3}, 1, 1);    // edge 3 = c (local), edge 4 = t2
    topo.pushNode({4}, 0, 1);       // edge 5 = y
    topo.setGlobalOutput(0, 5);
    std::vector<kernel::Node> nodes;
    nodes.push_back({std::make_unique<AddKernel>(1.f, n, false), "n0"});
    nodes.push_back({std::make_unique<AddKernel>(2.f, n, true), "n1"});
    nodes.push_back({std::make_unique<SumKernel>(n), "n2"});
    nodes.push_back({std::make_unique<AddKernel>(4.f, n, false), "n3"});
    auto const bytes = n * sizeof(float);
    std::vector<kernel::Edge> edges{{nullptr, bytes, "x"}, {nullptr, bytes, "t0"}, {nullptr, bytes, "t1"},
                                    {std::move(constant), bytes, "c"}, {nullptr, bytes, "t2"}, {nullptr, bytes, "y"}};
    return kernel::Graph(std::move(topo), std::move(nodes), std::move(edges));
}

static void allocatorsAndStreamOnCpu() {
    constexpr size_t n = 25;// 100 bytes: 128 once aligned to 32
    auto [constant, cPtr] = kernel::Blob::share(n * sizeof(float));
    for (size_t i = 0; i < n; ++i) static_cast<float *>(cPtr)[i] = 10.f * i;
    auto graph = chainGraph(n, constant);
    auto const &topo = graph._internal.topology;

    auto lowerNodes = [&] {
        runtime::Resources res;
        std::vector<runtime::Node> nodes;
        for (auto const &node : graph._internal.nodes) nodes.emplace_back(node.kernel->lower(res));
        return nodes;
    };
    {// flat: t0 | t1, workspace of n1 | t2, nothing is reused
        auto [stack, nodes, edges] = flatAllocate(topo, lowerNodes(), graph._internal.edges, 32);
        EXPECT(stack == 4 * 128);
        EXPECT(edges[0].stackOffset == SIZE_MAX && edges[3].stackOffset == SIZE_MAX && edges[5].stackOffset == SIZE_MAX - 1);
        EXPECT(edges[1].stackOffset == 0 && edges[2].stackOffset == 128 && nodes[1].workspaceOffset == 256 && edges[4].stackOffset == 384);
        EXPECT(nodes[0].workspaceOffset == 0 && nodes[2].workspaceOffset == 0);
    }
    {// reusable: t2 takes the range t0 has given back; the workspace of n1 is free again after n1
        auto [stack, nodes, edges] = reusableAllocate(topo, lowerNodes(), graph._internal.edges, 32);
        EXPECT(stack == 3 * 128);
        EXPECT(edges[1].stackOffset == 0 && edges[2].stackOffset == 128 && nodes[1].workspaceOffset == 256);
        EXPECT(edges[4].stackOffset == 0);
        EXPECT(edges[5].stackOffset == SIZE_MAX - 1 && edges[0].stackOffset == SIZE_MAX);
    }

    for (auto allocator : {flatAllocate, reusableAllocate}) {
        auto stream = graph.lower(device::fetch(Device::Type::Cpu), allocator);
        EXPECT(stream.graph().edges[3].blob && stream.graph().edges[3].name == "c");// the constant was uploaded
        EXPECT(stream.getData(5) && !stream.getData(0) && !stream.getData(1));      // global output has a blob, the input not yet
        std::vector<float> x(n), y(n, -1.f);
        std::iota(x.begin(), x.end(), 0.f);
        stream.setData(0, x.data(), n * sizeof(float));
        stream.run();
        EXPECT(stream.copyData(5, y.data(), n * sizeof(float)));
        bool ok = true;
        for (size_t i = 0; i < n; ++i) ok &= y[i] == x[i] + 7.f + 10.f * i;
        EXPECT(ok);
        EXPECT(!stream.copyData(1, y.data(), n * sizeof(float)));// a stack edge cannot be read back

        // a second run on new data in a caller-provided blob; trace sees every node once, in order,
        // with the addresses the routines were given
        auto blob = stream.setData(0, n * sizeof(float));
        for (auto &v : x) v = -v;
        blob->copyFromHost(x.data(), n * sizeof(float));
        std::vector<count_t> order;
        bool addressesOk = true;
        stream.trace([&](count_t idx, void const *const *inputs, void const *const *outputs) {
            order.push_back(idx);
            if (idx == 0) addressesOk &= inputs[0] == blob->get();
            if (idx == 2) addressesOk &= inputs[1] == stream.getData(3)->get();
            if (idx == 3) addressesOk &= outputs[0] == stream.getData(5)->get();
        });
        EXPECT((order == std::vector<count_t>{0, 1, 2, 3}) && addressesOk);
        stream.copyData(5, y.data(), n * sizeof(float));
        ok = true;
        for (size_t i = 0; i < n; ++i) ok &= y[i] == x[i] + 7.f + 10.f * i;
        EXPECT(ok);
        auto times = stream.bench(nullptr);
        EXPECT(times.size() == 4);
    }
    // the same constant on the same device is uploaded once and shared by the streams that are alive
    auto s1 = graph.lower(device::fetch(Device::Type::Cpu), flatAllocate);
    auto s2 = graph.lower(device::fetch(Device::Type::Cpu), reusableAllocate);
    EXPECT(s1.getData(3) == s2.getData(3));
    {// A constant that is freed while a stream still holds its device copy, then another constant of the
        // same size that lands at the same host address: the second graph must see its own values.
        auto run = [&](runtime::Stream &stream) {
            std::vector<float> x(n, 0.f), y(n, -1.f);
            stream.setData(0, x.data(), n * sizeof(float));
            stream.run();
            stream.copyData(5, y.data(), n * sizeof(float));
            return y;
        };
        auto [cA, pA] = kernel::Blob::share(n * sizeof(float));
        for (size_t i = 0; i < n; ++i) static_cast<float *>(pA)[i] = 1.f;
        auto const addressA = cA.get();
        auto graphA = std::make_unique<kernel::Graph>(chainGraph(n, std::move(cA)));
        auto streamA = graphA->lower(device::fetch(Device::Type::Cpu), flatAllocate);
        graphA.reset();// the host blob of A is gone, its device copy lives on in streamA
        std::vector<Arc<kernel::Blob>> held;
        Arc<kernel::Blob> cB;
        void *pB = nullptr;
        for (int attempt = 0; attempt < 64 && !cB; ++attempt) {
            auto [c, ptr] = kernel::Blob::share(n * sizeof(float));
            if (c.get() == addressA) cB = std::move(c), pB = ptr;
            else held.push_back(std::move(c));
        }
        bool const collided = static_cast<bool>(cB);
        if (!collided) std::tie(cB, pB) = kernel::Blob::share(n * sizeof(float));
        std::printf("  constant cache: host address %s\n", collided ? "reused" : "not reused by this allocator");
        for (size_t i = 0; i < n; ++i) static_cast<float *>(pB)[i] = 100.f;
        auto graphB = chainGraph(n, cB);
        auto streamB = graphB.lower(device::fetch(Device::Type::Cpu), flatAllocate);
        EXPECT(streamB.getData(3) != streamA.getData(3));
        auto const yA = run(streamA), yB = run(streamB);
        EXPECT(yA == std::vector<float>(n, 8.f));
        EXPECT(yB == std::vector<float>(n, 107.f));
    }
    // a node without kernel lowers to the empty routine
    graph_topo::GraphTopo topo1(1, 1);
    topo1.pushNode({0}, 0, 1);
    topo1.setGlobalOutput(0, 1);
    std::vector<kernel::Node> nodes1;
    nodes1.push_back({nullptr, "nothing"});
    kernel::Graph empty(std::move(topo1), std::move(nodes1), {{nullptr, 4, "in"}, {nullptr, 4, "out"}});
    auto s3 = empty.lower(device::fetch(Device::Type::Cpu), flatAllocate);
    s3.setData(0, size_t(4));
    s3.run();
    EXPECT(s3.getData(1) && s3.getData(1)->size() == 4);
}

namespace {
    // an operator with a kernel for the CPU target, so that the executor can be driven without a GPU
    struct AddConstant final : public computation::Operator {
        float addend;
        size_t n;
        AddConstant(float addend_, size_t n_) : addend(addend_), n(n_) {}
        static size_t typeId() noexcept {
            static uint8_t ID = 1;
            return reinterpret_cast<size_t>(&ID);
        }
        size_t opTypeId() const noexcept final { return typeId(); }
        std::string_view name() const noexcept final { return "AddConstant"; }
        kernel::CollectorBox candidateKernels(computation::Target target) const final {
            struct Collector final : public InfoCollector {
                float addend;
                size_t n;
                Collector(Device::Type t, float a, size_t n_) : InfoCollector(t), addend(a), n(n_) {}
                std::vector<KernelBox> filter(TensorRefs, TensorRefs) const final {
                    std::vector<KernelBox> ans;
                    if (_target == Device::Type::Cpu) ans.emplace_back(std::make_unique<AddKernel>(addend, n, false));
                    return ans;
                }
            };
            return std::make_unique<Collector>(target, addend, n);
        }
    };
    std::vector<char> readFile(std::filesystem::path const &p) {
        std::ifstream is(p, std::ios::binary);
        return {std::istreambuf_iterator<char>(is), std::istreambuf_iterator<char>()};
    }
}// namespace

static void executorOnCpu() {
    using namespace python_ffi;
    constexpr dim_t n = 6;
    auto t = Tensor::share(DataType::F32, Shape{2, 3});
    auto build = [&] {
        graph_topo::GraphTopo topo(1, 1);
        auto mid = topo.pushNode({0}, 0, 1).begin_;
        auto out = topo.pushNode({mid}, 0, 1).begin_;
        topo.setGlobalOutput(0, out);
        std::vector<computation::Node> ops;
        ops.push_back({std::make_unique<AddConstant>(1.f, n), "plus1"});
        ops.push_back({std::make_unique<AddConstant>(10.f, n), "plus10"});
        return computation::Graph(std::move(topo), std::move(ops), {{t, "x"}, {t, "mid"}, {t, "y"}});
    };
    EXPECT(findDevice("CPU", 0) == device::fetch(Device::Type::Cpu));
    EXPECT(throws<UnreachableError>([] { findDevice("tpu", 0); }));
    EXPECT(throws<UnreachableError>([&] { compile(build(), "cuda", "flat"); }));
    auto exe = compile(build(), "cpu", "flat");
    float x[n]{0, 1, 2, 3, 4, 5}, y[n]{};
    EXPECT(throws<std::runtime_error>([&] { exe->setInput(0, x, 4); }));// size mismatch
    exe->setInput(0, x, sizeof x);
    exe->run();
    exe->getOutput(0, y, sizeof y);
    EXPECT(y[0] == 11.f && y[5] == 16.f && exe->getOutputBlob(0)->size() == sizeof y);
    auto times = exe->bench(true);
    EXPECT(times.size() == 2 && times[0].first == "plus1" && times[1].first == "plus10");
    // another allocator: the input that was set is carried over
    exe->dispatch(findDevice("cpu", 0), "reuse");
    exe->run();
    std::fill(y, y + n, 0.f);
    exe->getOutput(0, y, sizeof y);
    EXPECT(y[0] == 11.f && y[5] == 16.f);
    // trace: a meta file per node, every tensor as .npy with a parsable header and the right bytes
    auto dir = std::filesystem::temp_directory_path() / ("rg_host_trace_" + std::to_string(::getpid()));
    exe->trace(dir.string(), "npy");
    auto meta = readFile(dir / "node000001.meta");
    std::string metaText(meta.begin(), meta.end());
    EXPECT(metaText.find("input\t0\tmid\t") != std::string::npos && metaText.find("output\t0\ty\t") != std::string::npos);
    auto npy = readFile(dir / "data000003.npy");// node 0: x, mid; node 1: mid, y
    EXPECT(npy.size() == 128 + sizeof y && std::memcmp(npy.data(), "\x93NUMPY\x01\x00", 8) == 0 && npy[127] == '\n');
    std::string header(npy.begin() + 10, npy.begin() + 128);
    EXPECT(header.find("'descr': '<f4'") != std::string::npos && header.find("'shape': (2,3,)") != std::string::npos);
    EXPECT(std::memcmp(npy.data() + 128, y, sizeof y) == 0);
    std::filesystem::remove_all(dir);
}

static void transposeInfoDigest() {
    {// src/04kernel/test/attributes/test_transpose_info.cpp:7-43
        TransposeInfo a(DataType::F32, {1, 2, 3, 2, 1}, {1, 2, 3, 0, 4});
        EXPECT(a.blockSize == 48 && a.blockCount == 1 && a.dims.size() == 1);
        TransposeInfo b(DataType::F32, {1, 1, 2, 1, 1}, {1, 2, 3, 0, 4});
        EXPECT(b.blockSize == 8 && b.blockCount == 1 && b.dims.size() == 1);
        TransposeInfo c(DataType::F32, {1, 2, 3, 4, 5}, {2, 3, 1, 0, 4});
        EXPECT(c.blockSize == 20 && c.blockCount == 24 && c.dims.size() == 2);
        EXPECT(c.dims[1].strideI == 12 && c.dims[1].strideO == 1 && c.dims[0].strideI == 1 && c.dims[0].strideO == 2);
    }
    // random shapes: the digest equals the oracle's, and copying block locate(i) to block i equals its result
    std::mt19937 rng(4);
    bool same = true, moved = true;
    for (int t = 0; t < 500; ++t) {
        auto const rank = 1 + rng() % 6;
        std::vector<dim_t> shape(rank), perm(rank);
        for (auto &d : shape) d = 1 + rng() % 4;
        std::iota(perm.begin(), perm.end(), 0);
        std::shuffle(perm.begin(), perm.end(), rng);
        TransposeInfo info(DataType::I16, shape, perm);
        uint32_t si[8], so[8], block, count;
        auto const dims = oracle_transpose_info(si, so, &block, &count, shape.data(), perm.data(), static_cast<int>(rank), 2);
        same &= static_cast<size_t>(dims) == info.dims.size() && block == info.blockSize && count == info.blockCount;
        for (size_t i = 0; same && i < info.dims.size(); ++i) same &= info.dims[i].strideI == si[i] && info.dims[i].strideO == so[i];
        std::vector<int16_t> x(static_cast<size_t>(info.blockSize) * info.blockCount / 2), y(x.size()), ref(x.size());
        std::iota(x.begin(), x.end(), 0);
        for (dim_t i = 0; i < info.blockCount; ++i)
            std::memcpy(reinterpret_cast<uint8_t *>(y.data()) + i * info.blockSize,
                        reinterpret_cast<uint8_t *>(x.data()) + info.locate(i) * info.blockSize, info.blockSize);
        oracle_transpose(ref.data(), x.data(), shape.data(), perm.data(), static_cast<int>(rank), 2);
        moved &= y == ref;
    }
    EXPECT(same);
    EXPECT(moved);
    EXPECT(throws<std::runtime_error>([] { TransposeInfo(DataType::F32, {2, 3}, {0}); }));
    EXPECT(TransposeCollector(Device::Type::Amd, {1, 0}).filter({*Tensor::share(DataType::FP16, Shape{4, 6})}, {*Tensor::share(DataType::FP16, Shape{6, 4})}).size() == 1);
    EXPECT(computation::Transpose({0, 2, 1, 3}).serialize() == "Transpose([ 0 2 1 3 ])");
}

static void computationGraphLowers() {
    using namespace computation;
    // x -> Identity -> Reshape -> RmsNormalization -> y, y also renamed to the second global output
    constexpr dim_t R = 4, C = 64;
    auto x = Tensor::share(DataType::F32, Shape{R, C});
    auto w = Tensor::share(DataType::F32, Shape{C});
    graph_topo::GraphTopo topo(2, 2);
    topo.pushNode({0}, 0, 1);      // 2 = identity(x)
    topo.pushNode({2}, 0, 1);      // 3 = reshape(2)
    topo.pushNode({3, 1}, 0, 1);   // 4 = rms(3, w)
    topo.pushNode({4}, 0, 1);      // 5 = identity(4)
    topo.setGlobalOutput(0, 4);
    topo.setGlobalOutput(1, 5);
    auto nodes = [] {
        std::vector<computation::Node> n;
        n.push_back({std::make_unique<Identity>(), "id0"});
        n.push_back({std::make_unique<Reshape>(), "reshape"});
        n.push_back({std::make_unique<RmsNormalization>(1e-5f), "norm"});
        n.push_back({std::make_unique<Identity>(), "id1"});
        return n;
    };
    std::vector<computation::Edge> edges{{x, "x"}, {w, "w"}, {x, "x1"}, {x, "x2"}, {x, "y"}, {x, "y1"}};
    computation::Graph g(topo, nodes(), edges);
    EXPECT(g.internal().nodes[2].op->is<RmsNormalization>() && !g.internal().nodes[2].op->is<Softmax>());
    EXPECT(g.internal().nodes[2].op->serialize() == "RmsNormalization(1e-05)");
    EXPECT(MatMul(1, 0, false, true).serialize() == "MatMul(1, 0, N, T)" && Attention(64).serialize() == "Attention(64)");
    auto k = g.lower(Target::Amd);
    auto const &kt = k._internal.topology;
    // the norm reads x itself, both global outputs are the norm's output; renamed edges have no size
    EXPECT(kt.node(2).inputs[0] == 0 && kt.node(2).inputs[1] == 1);
    EXPECT(kt.globalOutputs()[0] == 4 && kt.globalOutputs()[1] == 4);
    EXPECT(k._internal.edges[2].size == 0 && k._internal.edges[3].size == 0 && k._internal.edges[5].size == 0);
    EXPECT(k._internal.edges[4].size == R * C * 4 && k._internal.edges[4].name == "y");
    EXPECT(!k._internal.nodes[0].kernel && !k._internal.nodes[1].kernel && k._internal.nodes[2].kernel && !k._internal.nodes[3].kernel);
    EXPECT(k._internal.nodes[2].name == "norm");
    // planning the stack works with the renamed (empty) edges in place
    runtime::Resources res;
    std::vector<runtime::Node> lowered;
    for (auto const &n : k._internal.nodes) lowered.emplace_back(n.kernel ? n.kernel->lower(res) : runtime::Node(runtime::emptyRoutine));
    auto plan = reusableAllocate(kt, std::move(lowered), k._internal.edges, 256);
    EXPECT(plan.stack == 0 && plan.edges[4].stackOffset == SIZE_MAX - 1);
    // an operator whose collector finds nothing is reported by node name; the base class has no collector
    auto xi = Tensor::share(DataType::I64, Shape{R, C});
    std::vector<computation::Edge> bad{{xi, "x"}, {w, "w"}, {xi, "x1"}, {xi, "x2"}, {xi, "y"}, {xi, "y1"}};
    computation::Graph gBad(topo, nodes(), bad);
    bool named = false;
    try { gBad.lower(Target::Amd); } catch (std::runtime_error const &e) { named = std::string(e.what()).find("No kernel selected for \"norm\"") != std::string::npos; }
    EXPECT(named);
    EXPECT(throws<UnimplementError>([] { Identity().candidateKernels(Target::Amd); }));

    // MatMulInteger -> DequantizeLinear becomes one node only if the scale runs along the last axis (or is one
    // value), there is no zero point, and nothing else reads the sums
    auto quantised = [](int axis, dim_t scales, bool withZeroPoint) {
        auto a = Tensor::share(DataType::U8, Shape{4, 8}), b = Tensor::share(DataType::I8, Shape{8, 4});
        auto acc = Tensor::share(DataType::I32, Shape{4, 4}), out = Tensor::share(DataType::F32, Shape{4, 4});
        auto sc = Tensor::share(DataType::F32, Shape{scales}), zp = Tensor::share(DataType::I32, Shape{scales});
        graph_topo::GraphTopo t(withZeroPoint ? 4 : 3, 1);
        auto accEdge = t.pushNode({0, 1}, 0, 1).begin_;
        std::vector<count_t> in{accEdge, 2};
        if (withZeroPoint) in.push_back(3);
        auto outEdge = t.pushNode(in, 0, 1).begin_;
        t.setGlobalOutput(0, outEdge);
        std::vector<computation::Node> n;
        n.push_back({std::make_unique<MatMulInteger>(), "mm"});
        n.push_back({std::make_unique<DequantizeLinear>(axis), "dq"});
        std::vector<computation::Edge> e{{a, "a"}, {b, "b"}, {sc, "scale"}};
        if (withZeroPoint) e.push_back({zp, "zp"});
        e.push_back({acc, "acc"});
        e.push_back({out, "out"});
        return computation::Graph(std::move(t), std::move(n), std::move(e)).lower(Target::Amd)._internal.nodes.size();
    };
    EXPECT(quantised(1, 4, false) == 1 && quantised(1, 1, false) == 1 && quantised(-1, 4, false) == 1);
    EXPECT(quantised(0, 4, false) == 2 && quantised(1, 4, true) == 2);
}

// Split / Concat / Expand digests against the reference's vectors
// (src/04kernel/test/attributes/test_split_info.cpp:7-30, test_expand_info.cpp:7-18) and the collectors
static void dataMoverDigests() {
    using T = Device::Type;
    std::vector<Arc<Tensor>> parts{
        Tensor::share(DataType::I64, Shape{2, 3, 1, 1, 7, 7}), Tensor::share(DataType::I64, Shape{2, 3, 1, 9, 7, 7}),
        Tensor::share(DataType::I64, Shape{2, 3, 1, 3, 7, 7}), Tensor::share(DataType::I64, Shape{2, 3, 1, 7, 7, 7})};
    TensorRefs refs;
    for (auto const &t : parts) refs.emplace_back(*t);
    SplitInfo info(3, refs);
    dim_t const postfix = 49 * 8;
    EXPECT(info.blockCount == 6 && info.sum == 20 * postfix);
    EXPECT((info.segments == std::vector<dim_t>{1 * postfix, 9 * postfix, 3 * postfix, 7 * postfix}));

    auto in = Tensor::share(DataType::F32, Shape{3, 4, 1, 6}), out = Tensor::share(DataType::F32, Shape{2, 3, 4, 5, 6});
    ExpandInfo e(*in, *out);
    EXPECT(e.blockSize == 24 && e.blockCount == 120);
    EXPECT((e.strides == std::vector<ExpandInfo::Dim>{{0, 60}, {1, 5}, {0, 1}}));
    ExpandInfo same(*out, *out);
    EXPECT(same.strides.empty() && same.blockCount == 1 && same.blockSize == 720 * 4);
    ExpandInfo bias(DataType::F32, {4096}, {512, 4096});
    EXPECT(bias.blockSize == 16384 && bias.blockCount == 512 && (bias.strides == std::vector<ExpandInfo::Dim>{{0, 1}}));

    auto joined = Tensor::share(DataType::I64, Shape{2, 3, 1, 20, 7, 7});
    auto sp = SplitCollector(T::Amd, 3).filter({*joined}, refs);
    EXPECT(sp.size() == 1 && sp[0]->is<SplitHip>() && static_cast<SplitHip const &>(*sp[0]).info.sum == 20 * postfix);
    auto cc = ConcatCollector(T::Amd, 3).filter(refs, {*joined});
    EXPECT(cc.size() == 1 && cc[0]->is<ConcatHip>());
    EXPECT(SplitCollector(T::Cpu, 3).filter({*joined}, refs).empty() && ConcatCollector(T::Cpu, 3).filter(refs, {*joined}).empty());
    EXPECT(SplitCollector(T::Amd, 9).filter({*joined}, refs).empty());// no such axis
    EXPECT(ExpandCollector(T::Amd).filter({*in}, {*out}).size() == 1 && ExpandCollector(T::Amd).filter({*out}, {*in}).empty());
    {// shapes that do not broadcast, a type change and missing tensors give no kernel and throw nothing
        auto odd = Tensor::share(DataType::F32, Shape{3, 4, 2, 6}), other = Tensor::share(DataType::I32, Shape{2, 3, 4, 5, 6});
        bool threw = false;
        try {
            EXPECT(ExpandCollector(T::Amd).filter({*odd}, {*out}).empty());
            EXPECT(ExpandCollector(T::Amd).filter({*in}, {*other}).empty());
            EXPECT(ExpandCollector(T::Amd).filter({}, {*out}).empty() && ExpandCollector(T::Amd).filter({*in}, {}).empty());
        } catch (...) { threw = true; }
        EXPECT(!threw);
    }
    auto c = Tensor::share(DataType::Bool, Shape{2, 5});
    auto x = Tensor::share(DataType::F32, Shape{2, 3, 2, 5}), y = Tensor::share(DataType::F32, Shape{3, 2, 5});
    auto wh = WhereCollector(T::Amd).filter({*c, *x, *y}, {*x});
    EXPECT(wh.size() == 1 && wh[0]->is<WhereHip>() && static_cast<WhereHip const &>(*wh[0]).broadcaster.outputsCount == 60);
    auto yi = Tensor::share(DataType::I32, Shape{3, 2, 5});
    EXPECT(WhereCollector(T::Amd).filter({*c, *x, *yi}, {*x}).empty());// x and y of different types
    EXPECT(throws<UnreachableError>([&] { SplitCollector(T::Nvidia, 3).filter({*joined}, refs); }));
}

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
        auto [routine, workspace] = kernels[0]->lower(res);
        auto ma = dev.malloc(a.size() * 4), mb = dev.malloc(b.size() * 4), mc = dev.malloc(std::max<size_t>(c.size(), 1) * 4),
             my = dev.malloc(Y.elementsSize() * 4), ws = dev.malloc(workspace ? workspace : 1);
        ma->copyFromHost(a.data());
        mb->copyFromHost(b.data());
        if (!c.empty()) mc->copyFromHost(c.data());
        void const *inputs[]{*ma, *mb, *mc};
        void *outputs[]{*my};
        routine(res, *ws, inputs, outputs);
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
    {// a bias that broadcasts over one batch dimension and not the other ([3, 1, m, 1] under [3, 2, m, n]): the
     // reference expands every bias into Y first (src/04kernel/src/kernels/mat_mul/cublas_kernel.cu:26-39); here this
     // one goes through Expand into the workspace.  Shapes of test_cpu.cpp:57-79 with a third matrix; integers: exact
        std::mt19937 rng(13);
        std::uniform_int_distribution<int> g(-3, 3);
        dim_t const m = 5, k = 7, n = 6;
        std::vector<float> a(3 * m * k), b(2 * k * n), c(3 * m);
        for (auto &v : a) v = static_cast<float>(g(rng));
        for (auto &v : b) v = static_cast<float>(g(rng));
        for (auto &v : c) v = static_cast<float>(g(rng));
        auto A = Tensor::share(DataType::F32, Shape{3, 1, m, k});
        auto B = Tensor::share(DataType::F32, Shape{1, 2, k, n});
        auto C = Tensor::share(DataType::F32, Shape{3, 1, m, 1});
        auto Y = Tensor::share(DataType::F32, Shape{3, 2, m, n});
        MatMulInfo info(*A, *B, std::make_optional(std::cref(*C)), false, false, 1, 1);
        EXPECT(info.biasSupported && !info.biasExpandFrom.empty());
        auto y = run(*A, *B, C.get(), *Y, a, b, c);
        bool same = true;
        for (dim_t i = 0; i < 3; ++i)
            for (dim_t j = 0; j < 2; ++j)
                for (dim_t r = 0; r < m; ++r)
                    for (dim_t q = 0; q < n; ++q) {
                        float sum = c[i * m + r];
                        for (dim_t t = 0; t < k; ++t) sum += a[(i * m + r) * k + t] * b[(j * k + t) * n + q];
                        same = same && y[((i * 2 + j) * m + r) * n + q] == sum;
                    }
        EXPECT(same);
        // what does not broadcast is still declined
        auto bad = Tensor::share(DataType::F32, Shape{2, 1, m, 1});
        EXPECT(MatMulCollector(Device::Type::Amd, 1, 1, false, false).filter({*A, *B, *bad}, {*Y}).empty());
    }
    {// few rows of FP16 against weights kept as [k, n]: lower() asks for the library's workspace (shares of k meet
     // there) and the routine hands it on; operands in {-1, 0, 1}, so every sum is an integer FP16 holds exactly.
     // The workspace arrives as the allocator left it: nothing in it needs preparing.
        std::mt19937 rng(17);
        std::uniform_int_distribution<int> g(-1, 1);
        dim_t const k = 1024, n = 1024;
        for (dim_t m : {dim_t(1), dim_t(4), dim_t(20)}) {
            std::vector<int> a(m * k), b(k * n);
            for (auto &v : a) v = g(rng);
            for (auto &v : b) v = g(rng);
            std::vector<uint16_t> ah(a.size()), bh(b.size());
            for (size_t i = 0; i < a.size(); ++i) ah[i] = f2h(static_cast<float>(a[i]));
            for (size_t i = 0; i < b.size(); ++i) bh[i] = f2h(static_cast<float>(b[i]));
            auto A = Tensor::share(DataType::FP16, Shape{m, k});
            auto B = Tensor::share(DataType::FP16, Shape{k, n});
            auto Y = Tensor::share(DataType::FP16, Shape{m, n});
            auto kernels = MatMulCollector(Device::Type::Amd, 1, 1, false, false).filter({*A, *B}, {*Y});
            EXPECT(kernels.size() == 1);
            auto [routine, workspace] = kernels[0]->lower(res);
            EXPECT(workspace > 0);
            auto ma = dev.malloc(ah.size() * 2), mb = dev.malloc(bh.size() * 2), my = dev.malloc(m * n * 2), ws = dev.malloc(workspace);
            std::vector<uint8_t> junk(workspace, 0xa5);
            ws->copyFromHost(junk.data());
            ma->copyFromHost(ah.data());
            mb->copyFromHost(bh.data());
            void const *inputs[]{*ma, *mb};
            void *outputs[]{*my};
            std::vector<uint16_t> y(m * n);
            bool same = true;
            for (int round = 0; round < 2; ++round) {  // the second call finds what the first one left
                routine(res, *ws, inputs, outputs);
                my->copyToHost(y.data());
                for (dim_t i = 0; i < m; ++i)
                    for (dim_t j = 0; j < n; ++j) {
                        int sum = 0;
                        for (dim_t t = 0; t < k; ++t) sum += a[i * k + t] * b[t * n + j];
                        same = same && y[i * n + j] == f2h(static_cast<float>(sum));
                    }
            }
            EXPECT(same);
        }
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

// DynamicQuantizeLinear -> MatMulInteger -> DequantizeLinear lowered as one graph on the AMD device:
// the quantised linear layer y = (q(x) - zp) @ W * scale, every kernel picked by its collector,
// intermediate tensors and workspaces on the stream's stack, W a constant uploaded by lower().
static void quantisedLinearStream() {
    constexpr dim_t M = 96, K = 512, N = 256;
    auto x = Tensor::share(DataType::F32, Shape{M, K});
    auto xq = Tensor::share(DataType::U8, Shape{M, K});
    auto scale = Tensor::share(DataType::F32, Shape{});
    auto zp = Tensor::share(DataType::U8, Shape{});
    auto [wBlob, wPtr] = kernel::Blob::share(K * N);
    auto w = Tensor::share(DataType::I8, Shape{K, N}, LayoutType::Others, wBlob);
    auto acc = Tensor::share(DataType::I32, Shape{M, N});
    auto y = Tensor::share(DataType::F32, Shape{M, N});
    std::mt19937 rng(21);
    std::vector<int8_t> w_(K * N);
    for (auto &v : w_) v = static_cast<int8_t>(rng());
    std::memcpy(wPtr, w_.data(), w_.size());
    std::vector<float> x_(M * K);
    std::normal_distribution<float> g(0.3f, 2.f);
    for (auto &v : x_) v = g(rng);

    // edges: 0 x | 1 xq 2 scale 3 zp | 4 W (local) 5 acc | 6 y
    // With `accIsOutput` the int32 sums are a result of the graph too, which keeps the three operators
    // apart; otherwise lower() folds the dequantisation into the product.
    auto build = [&](bool accIsOutput) {
        graph_topo::GraphTopo topo(1, accIsOutput ? 2 : 1);
        topo.pushNode({0}, 0, 3);
        topo.pushNode({1, 4, 3}, 1, 1);
        topo.pushNode({5, 2}, 0, 1);
        topo.setGlobalOutput(0, 6);
        if (accIsOutput) topo.setGlobalOutput(1, 5);
        std::vector<computation::Node> ops;
        ops.push_back({std::make_unique<computation::DynamicQuantizeLinear>(), "quantise"});
        ops.push_back({std::make_unique<computation::MatMulInteger>(), "matmul"});
        ops.push_back({std::make_unique<computation::DequantizeLinear>(), "dequantise"});
        return computation::Graph(std::move(topo), std::move(ops),
                                  {{x, "x"}, {xq, "xq"}, {scale, "scale"}, {zp, "zp"}, {w, "W"}, {acc, "acc"}, {y, "y"}})
            .lower(computation::Target::Amd);
    };
    auto apart = build(true), fused = build(false);
    EXPECT(apart._internal.nodes.size() == 3 && apart._internal.edges[4].data == wBlob && apart._internal.edges[5].size == acc->bytesSize());
    // fused: x | xq scale zp | W y
    EXPECT(fused._internal.nodes.size() == 2 && fused._internal.edges.size() == 6);
    EXPECT(fused._internal.nodes[1].name == "matmul+dequantise" && fused._internal.nodes[1].kernel->is<MatMulIntegerDequantizeHip>());
    EXPECT(fused._internal.edges[4].data == wBlob && fused._internal.edges[5].name == "y" && fused._internal.topology.globalOutputs()[0] == 5);
    {
        auto node = fused._internal.topology.node(1);
        EXPECT(node.inputs.size() == 4 && node.inputs[0] == 1 && node.inputs[1] == 4 && node.inputs[2] == 3 && node.inputs[3] == 2);
    }

    // oracle chain
    std::vector<uint8_t> q(M * K);
    float s;
    uint8_t z;
    oracle_dynamic_quantize_linear(q.data(), &s, &z, x_.data(), x_.size());
    std::vector<int32_t> accRef(M * N);
    oracle_matmul_integer(accRef.data(), q.data(), w_.data(), &z, 0, 1, nullptr, 1, 1, 1, M, K, N, nullptr, nullptr, 1, 1, 8);
    std::vector<float> ref(M * N), out(M * N);
    oracle_dequantize_linear(ref.data(), accRef.data(), &s, nullptr, 1, 1, M * N, ORACLE_I32, 1, 1);

    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    for (auto const *graph : {&apart, &fused})
        for (auto allocator : {flatAllocate, reusableAllocate}) {
            auto stream = graph->lower(dev, allocator);
            auto const nodeCount = stream.graph().nodes.size();
            auto const yEdge = stream.graph().topology.globalOutputs()[0];
            // every stack offset is 256-byte aligned on this device
            bool aligned = true;
            for (auto const &e : stream.graph().edges)
                if (!e.blob && e.stackOffset < SIZE_MAX - 1) aligned &= e.stackOffset % 256 == 0;
            for (auto const &n : stream.graph().nodes) aligned &= n.workspaceOffset % 256 == 0;
            EXPECT(aligned);
            stream.setData(0, x_.data(), x->bytesSize());
            stream.run();
            device::sync(Device::Type::Amd);
            std::fill(out.begin(), out.end(), -1.f);
            EXPECT(stream.copyData(yEdge, out.data(), y->bytesSize()));
            EXPECT(std::memcmp(out.data(), ref.data(), out.size() * sizeof(float)) == 0);
            if (nodeCount == 3) {// the int32 sums are a result as well
                std::vector<int32_t> accGpu(M * N);
                EXPECT(stream.copyData(stream.graph().topology.globalOutputs()[1], accGpu.data(), accGpu.size() * 4) && accGpu == accRef);
            }
            // bench: one duration per node, each including the wait for the device
            auto times = stream.bench([] { device::sync(Device::Type::Amd); });
            bool positive = times.size() == nodeCount;
            for (auto t : times) positive &= t.count() > 0;
            EXPECT(positive);
            // trace: copy results out node by node (what Executor::trace is for)
            std::vector<uint8_t> qGpu(M * K);
            std::vector<float> last(M * N);
            stream.trace([&](count_t idx, void const *const *, void const *const *outputs) {
                device::sync(Device::Type::Amd);
                if (idx == 0) AmdMemory().copyDH(qGpu.data(), outputs[0], qGpu.size());
                if (idx + 1 == nodeCount) AmdMemory().copyDH(last.data(), outputs[0], last.size() * 4);
            });
            EXPECT(qGpu == q && std::memcmp(last.data(), ref.data(), last.size() * 4) == 0);
        }
}

// The head of a quantised layer as a graph: RmsNormalization -> DynamicQuantizeLinear -> MatMulInteger ->
// DequantizeLinear.  On the AMD target lower() joins the first two (the normalising launch leaves its output's
// extrema, so the normalised tensor is read once) and the last two; the normalised tensor stays an output of the
// joined node (here it is a result of the graph as well).  Checked against the oracle chain: the normalised
// tensor within 1e-5 relative of the reference's serial sum, everything behind it bit for bit on that tensor.
static void normQuantisedLinearStream() {
    constexpr dim_t M = 64, K = 1024, N = 256;
    auto x = Tensor::share(DataType::F32, Shape{M, K});
    auto wn = Tensor::share(DataType::F32, Shape{K});
    auto xn = Tensor::share(DataType::F32, Shape{M, K});
    auto xq = Tensor::share(DataType::U8, Shape{M, K});
    auto scale = Tensor::share(DataType::F32, Shape{});
    auto zp = Tensor::share(DataType::U8, Shape{});
    auto [wBlob, wPtr] = kernel::Blob::share(K * N);
    auto w = Tensor::share(DataType::I8, Shape{K, N}, LayoutType::Others, wBlob);
    auto acc = Tensor::share(DataType::I32, Shape{M, N});
    auto y = Tensor::share(DataType::F32, Shape{M, N});
    std::mt19937 rng(27);
    std::vector<int8_t> w_(K * N);
    for (auto &v : w_) v = static_cast<int8_t>(rng());
    std::memcpy(wPtr, w_.data(), w_.size());
    std::vector<float> x_(M * K), g_(K);
    std::normal_distribution<float> g(0.1f, 1.5f);
    std::uniform_real_distribution<float> u(0.5f, 1.5f);
    for (auto &v : x_) v = g(rng);
    for (auto &v : g_) v = u(rng);

    // edges: 0 x 1 gain | 2 xn | 3 xq 4 scale 5 zp | 6 W (local) 7 acc | 8 y
    graph_topo::GraphTopo topo(2, 2);
    topo.pushNode({0, 1}, 0, 1);
    topo.pushNode({2}, 0, 3);
    topo.pushNode({3, 6, 5}, 1, 1);
    topo.pushNode({7, 4}, 0, 1);
    topo.setGlobalOutput(0, 8);
    topo.setGlobalOutput(1, 2);
    std::vector<computation::Node> ops;
    ops.push_back({std::make_unique<computation::RmsNormalization>(1e-5f), "norm"});
    ops.push_back({std::make_unique<computation::DynamicQuantizeLinear>(), "quantise"});
    ops.push_back({std::make_unique<computation::MatMulInteger>(), "matmul"});
    ops.push_back({std::make_unique<computation::DequantizeLinear>(), "dequantise"});
    auto lowered = computation::Graph(std::move(topo), std::move(ops),
                                      {{x, "x"}, {wn, "gain"}, {xn, "xn"}, {xq, "xq"}, {scale, "scale"}, {zp, "zp"},
                                       {w, "W"}, {acc, "acc"}, {y, "y"}})
                       .lower(computation::Target::Amd);
    EXPECT(lowered._internal.nodes.size() == 2);
    EXPECT(lowered._internal.nodes[0].name == "norm+quantise" && lowered._internal.nodes[0].kernel->is<RmsNormalizationQuantizeHip>());
    EXPECT(lowered._internal.nodes[1].name == "matmul+dequantise" && lowered._internal.nodes[1].kernel->is<MatMulIntegerDequantizeHip>());
    {
        auto node = lowered._internal.topology.node(0);
        EXPECT(node.inputs.size() == 2 && node.outputs.size() == 4);
    }

    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    for (auto allocator : {flatAllocate, reusableAllocate}) {
        auto stream = lowered.lower(dev, allocator);
        stream.setData(0, x_.data(), x->bytesSize());
        stream.setData(1, g_.data(), wn->bytesSize());
        stream.run();
        device::sync(Device::Type::Amd);
        std::vector<float> out(M * N), norm(M * K), normRef(M * K);
        EXPECT(stream.copyData(stream.graph().topology.globalOutputs()[0], out.data(), out.size() * 4));
        EXPECT(stream.copyData(stream.graph().topology.globalOutputs()[1], norm.data(), norm.size() * 4));
        oracle_rms_norm_f32(normRef.data(), x_.data(), g_.data(), M, K, 1e-5f, 1);
        bool close = true;
        for (size_t i = 0; i < norm.size(); ++i) close &= std::fabs(norm[i] - normRef[i]) <= 1e-5f * std::fabs(normRef[i]) + 1e-30f;
        EXPECT(close);
        // the chain behind the normalised tensor, on the tensor the device produced
        std::vector<uint8_t> q(M * K);
        float s;
        uint8_t z;
        oracle_dynamic_quantize_linear(q.data(), &s, &z, norm.data(), norm.size());
        std::vector<int32_t> accRef(M * N);
        oracle_matmul_integer(accRef.data(), q.data(), w_.data(), &z, 0, 1, nullptr, 1, 1, 1, M, K, N, nullptr, nullptr, 1, 1, 8);
        std::vector<float> ref(M * N);
        oracle_dequantize_linear(ref.data(), accRef.data(), &s, nullptr, 1, 1, M * N, ORACLE_I32, 1, 1);
        EXPECT(std::memcmp(out.data(), ref.data(), out.size() * sizeof(float)) == 0);
    }
    // shapes the pair is not joined for keep their two kernels (rows that are no whole vectors)
    {
        auto xo = Tensor::share(DataType::F32, Shape{8, 130});
        auto wo = Tensor::share(DataType::F32, Shape{130});
        auto qo = Tensor::share(DataType::U8, Shape{8, 130});
        graph_topo::GraphTopo t2(2, 3);
        t2.pushNode({0, 1}, 0, 1);
        t2.pushNode({2}, 0, 3);
        for (count_t i = 0; i < 3; ++i) t2.setGlobalOutput(i, 3 + i);
        std::vector<computation::Node> ops2;
        ops2.push_back({std::make_unique<computation::RmsNormalization>(1e-5f), "norm"});
        ops2.push_back({std::make_unique<computation::DynamicQuantizeLinear>(), "quantise"});
        auto apart = computation::Graph(std::move(t2), std::move(ops2),
                                        {{xo, "x"}, {wo, "gain"}, {xo, "xn"}, {qo, "xq"}, {scale, "scale"}, {zp, "zp"}})
                         .lower(computation::Target::Amd);
        EXPECT(apart._internal.nodes.size() == 2 && apart._internal.nodes[0].kernel->is<RmsNormalizationHip>());
    }
}

// One decode step of an attention block as a graph: RotaryEmbedding on q and k ([N, 1, heads, D]),
// Reshape to the attention layout ([N, heads, 1, D]: the same bytes, no kernel), Attention with the
// caches as persistent global outputs.  Two steps enqueued routine by routine, then the graph is
// recorded as one HIP graph and three more steps are replays of it with new contents in the same
// blobs; every step is checked against the oracle in the same way.
static void decodeAttentionStream() {
    using namespace computation;
    constexpr dim_t N = 3, H = 8, Hkv = 2, D = 128, S = 64;
    constexpr float theta = 10000.f;
    auto q = Tensor::share(DataType::FP16, Shape{N, 1, H, D}), qa = Tensor::share(DataType::FP16, Shape{N, H, 1, D});
    auto k = Tensor::share(DataType::FP16, Shape{N, 1, Hkv, D}), ka = Tensor::share(DataType::FP16, Shape{N, Hkv, 1, D});
    auto pos = Tensor::share(DataType::I64, Shape{N, 1}), past = Tensor::share(DataType::I64, Shape{N});
    auto cache = Tensor::share(DataType::FP16, Shape{N, Hkv, S, D});
    // edges: 0 q 1 k 2 v 3 pos 4 past | 5 qr | 6 kr | 7 q' | 8 k' | 9 o 10 kcache 11 vcache
    graph_topo::GraphTopo topo(5, 3);
    topo.pushNode({0, 3}, 0, 1);
    topo.pushNode({1, 3}, 0, 1);
    topo.pushNode({5}, 0, 1);
    topo.pushNode({6}, 0, 1);
    topo.pushNode({7, 8, 2, 4}, 0, 3);
    for (count_t i = 0; i < 3; ++i) topo.setGlobalOutput(i, 9 + i);
    std::vector<computation::Node> ops;
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_q"});
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_k"});
    ops.push_back({std::make_unique<Reshape>(), "q_heads_first"});
    ops.push_back({std::make_unique<Reshape>(), "k_heads_first"});
    ops.push_back({std::make_unique<Attention>(S), "attention"});
    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    auto stream = computation::Graph(std::move(topo), std::move(ops),
                                     {{q, "q"}, {k, "k"}, {ka, "v"}, {pos, "pos"}, {past, "past"}, {q, "qr"}, {k, "kr"},
                                      {qa, "q'"}, {ka, "k'"}, {qa, "o"}, {cache, "k_cache"}, {cache, "v_cache"}})
                      .lower(Target::Amd)
                      .lower(dev, reusableAllocate);

    std::mt19937 rng(33);
    std::normal_distribution<float> n01;
    auto randomHalf = [&](size_t n) { std::vector<uint16_t> v(n); for (auto &e : v) e = f2h(n01(rng)); return v; };
    auto kc = randomHalf(cache->elementsSize()), vc = randomHalf(cache->elementsSize());
    stream.getData(10)->copyFromHost(kc.data());
    stream.getData(11)->copyFromHost(vc.data());
    int64_t pastLen[N] = {17, 0, 40};
    float const scale = 1.0f / std::sqrt(static_cast<float>(D));
    auto rope = [&](std::vector<uint16_t> const &x, dim_t heads) {// oracle on up-cast values, one rounding back
        std::vector<float> xf(x.size()), yf(x.size());
        for (size_t i = 0; i < x.size(); ++i) xf[i] = h2f(x[i]);
        oracle_rope_f32(yf.data(), xf.data(), pastLen, 1, N, 1, heads, D, theta, 1);
        std::vector<uint16_t> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) y[i] = f2h(yf[i]);
        return y;
    };
    EXPECT(throws<std::runtime_error>([&] { stream.replay(); }));// nothing recorded yet
    for (int step = 0; step < 5; ++step) {
        auto q_ = randomHalf(q->elementsSize()), k_ = randomHalf(k->elementsSize()), v_ = randomHalf(k->elementsSize());
        if (step < 2) {
            stream.setData(0, q_.data(), q_.size() * 2);
            stream.setData(1, k_.data(), k_.size() * 2);
            stream.setData(2, v_.data(), v_.size() * 2);
            stream.setData(3, pastLen, sizeof pastLen);
            stream.setData(4, pastLen, sizeof pastLen);
            stream.run();
        } else {
            if (step == 2) {
                stream.record();// runs the previous step once more (same rows, same values) and records
                EXPECT(stream.recorded());
            }
            stream.getData(0)->copyFromHost(q_.data(), q_.size() * 2);
            stream.getData(1)->copyFromHost(k_.data(), k_.size() * 2);
            stream.getData(2)->copyFromHost(v_.data(), v_.size() * 2);
            stream.getData(3)->copyFromHost(pastLen, sizeof pastLen);
            stream.getData(4)->copyFromHost(pastLen, sizeof pastLen);
            stream.replay();
        }
        device::sync(Device::Type::Amd);
        std::vector<uint16_t> o(q_.size()), kcOut(kc.size()), vcOut(vc.size());
        EXPECT(stream.copyData(9, o.data(), o.size() * 2) && stream.copyData(10, kcOut.data(), kc.size() * 2) &&
               stream.copyData(11, vcOut.data(), vc.size() * 2));
        auto qr = rope(q_, H), kr = rope(k_, Hkv);
        // caches: V rows appended bit for bit, K rows within the rotary embedding's tolerance, the rest untouched
        bool rowsOk = true;
        for (dim_t b = 0; b < N; ++b)
            for (dim_t h = 0; h < Hkv; ++h) {
                auto const at = ((b * Hkv + h) * S + pastLen[b]) * D;
                for (dim_t i = 0; i < D; ++i) rowsOk &= std::fabs(h2f(kcOut[at + i]) - h2f(kr[(b * Hkv + h) * D + i])) <= 2e-3f;
                std::memcpy(&kc[at], &kcOut[at], D * 2);// continue from what the device wrote
                std::memcpy(&vc[at], &v_[(b * Hkv + h) * D], D * 2);
            }
        EXPECT(rowsOk && kcOut == kc && vcOut == vc);
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
                for (dim_t i = 0; i < D; ++i) qf[i] = h2f(qr[(b * H + h) * D + i]);
                oracle_attention_head_f32(ref.data(), qf.data(), kf.data(), vf.data(), 1, pastLen[b], D, scale, 1, scratch.data());
                for (dim_t i = 0; i < D; ++i) ok &= std::fabs(h2f(o[(b * H + h) * D + i]) - ref[i]) <= 4e-3f;
            }
        EXPECT(ok);// 2e-3 of the attention on top of q rotated within 2e-3
        for (auto &p : pastLen) ++p;
    }
    {// what the recording saves per step (printed, not asserted): same work enqueued 200 times each way
        auto clock = [] { return std::chrono::steady_clock::now(); };
        device::sync(Device::Type::Amd);
        auto t0 = clock();
        for (int i = 0; i < 200; ++i) stream.run();
        device::sync(Device::Type::Amd);
        auto t1 = clock();
        for (int i = 0; i < 200; ++i) stream.replay();
        device::sync(Device::Type::Amd);
        auto t2 = clock();
        std::printf("  decode block (2 x RotaryEmbedding + Attention): %.1f us per step enqueued routine by routine, %.1f us replayed\n",
                    std::chrono::duration<double, std::micro>(t1 - t0).count() / 200,
                    std::chrono::duration<double, std::micro>(t2 - t1).count() / 200);
    }
    // another blob on an edge discards the recording
    stream.setData(0, q->bytesSize());
    EXPECT(!stream.recorded() && throws<std::runtime_error>([&] { stream.replay(); }));
    // a stream on the CPU device has nothing to record
    graph_topo::GraphTopo topo1(1, 1);
    topo1.pushNode({0}, 0, 1);
    topo1.setGlobalOutput(0, 1);
    std::vector<kernel::Node> nodes1;
    nodes1.push_back({nullptr, "nothing"});
    auto onCpu = kernel::Graph(std::move(topo1), std::move(nodes1), {{nullptr, 4, "in"}, {nullptr, 4, "out"}})
                     .lower(device::fetch(Device::Type::Cpu), flatAllocate);
    EXPECT(throws<std::runtime_error>([&] { onCpu.record(); }));
}

// A chain of 64 small kernels: what a recording is for.  The replayed result must equal the result
// of the routines enqueued one by one, on every replay, with other work in between.
static void longChainRecorded() {
    using namespace computation;
    constexpr dim_t R = 8, C = 1024, L = 64;
    auto x = Tensor::share(DataType::F32, Shape{R, C});
    auto w = Tensor::share(DataType::F32, Shape{C});
    graph_topo::GraphTopo topo(2, 1);
    std::vector<computation::Node> ops;
    std::vector<computation::Edge> edges{{x, "x"}, {w, "w"}};
    count_t last = 0;
    for (dim_t i = 0; i < L; ++i) {
        last = topo.pushNode({last, 1}, 0, 1).begin_;
        ops.push_back({std::make_unique<RmsNormalization>(1e-5f), "norm" + std::to_string(i)});
        edges.push_back({x, "t" + std::to_string(i)});
    }
    topo.setGlobalOutput(0, last);
    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    auto stream = computation::Graph(std::move(topo), std::move(ops), std::move(edges)).lower(Target::Amd).lower(dev, reusableAllocate);
    // two ranges of the stack are enough for the whole chain
    EXPECT(stream.graph().edges[2].stackOffset == 0 && stream.graph().edges[3].stackOffset == R * C * 4 && stream.graph().edges[4].stackOffset == 0);
    std::mt19937 rng(3);
    std::normal_distribution<float> n01;
    std::vector<float> x_(R * C), w_(C), eager(R * C), replayed(R * C);
    for (auto &v : w_) v = 1.f + 0.1f * n01(rng);
    stream.setData(1, w_.data(), C * 4);
    stream.setData(0, size_t(R * C * 4));
    stream.record();
    bool same = true;
    for (int round = 0; round < 4; ++round) {
        for (auto &v : x_) v = n01(rng);
        stream.getData(0)->copyFromHost(x_.data(), R * C * 4);
        stream.run();
        device::sync(Device::Type::Amd);
        stream.copyData(last, eager.data(), R * C * 4);
        std::vector<float> zeros(R * C, 0.f);
        stream.getData(last)->copyFromHost(zeros.data(), R * C * 4);// eager work between the replays
        stream.replay();
        device::sync(Device::Type::Amd);
        stream.copyData(last, replayed.data(), R * C * 4);
        same &= std::memcmp(eager.data(), replayed.data(), R * C * 4) == 0 && eager[0] != 0.f;
    }
    EXPECT(same);
    auto clock = [] { return std::chrono::steady_clock::now(); };
    auto t0 = clock();
    for (int i = 0; i < 50; ++i) stream.run();
    device::sync(Device::Type::Amd);
    auto t1 = clock();
    for (int i = 0; i < 50; ++i) stream.replay();
    device::sync(Device::Type::Amd);
    auto t2 = clock();
    std::printf("  chain of 64 RmsNormalization [8, 1024]: %.1f us per run enqueued routine by routine, %.1f us replayed\n",
                std::chrono::duration<double, std::micro>(t1 - t0).count() / 50,
                std::chrono::duration<double, std::micro>(t2 - t1).count() / 50);
}

static void executorOnGpu() {
    using namespace python_ffi;
    constexpr dim_t M = 64, K = 256, N = 256;
    auto x = Tensor::share(DataType::F32, Shape{M, K});
    auto xq = Tensor::share(DataType::U8, Shape{M, K});
    auto scale = Tensor::share(DataType::F32, Shape{});
    auto zp = Tensor::share(DataType::U8, Shape{});
    auto [wBlob, wPtr] = kernel::Blob::share(K * N);
    auto w = Tensor::share(DataType::I8, Shape{K, N}, LayoutType::Others, wBlob);
    auto acc = Tensor::share(DataType::I32, Shape{M, N});
    auto y = Tensor::share(DataType::F32, Shape{M, N});
    std::mt19937 rng(5);
    std::vector<int8_t> w_(K * N);
    for (auto &v : w_) v = static_cast<int8_t>(rng());
    std::memcpy(wPtr, w_.data(), w_.size());
    std::vector<float> x_(M * K), out(M * N), ref(M * N);
    std::normal_distribution<float> g(0.f, 1.f);
    for (auto &v : x_) v = g(rng);
    graph_topo::GraphTopo topo(1, 1);
    topo.pushNode({0}, 0, 3);
    topo.pushNode({1, 4, 3}, 1, 1);
    topo.pushNode({5, 2}, 0, 1);
    topo.setGlobalOutput(0, 6);
    std::vector<computation::Node> ops;
    ops.push_back({std::make_unique<computation::DynamicQuantizeLinear>(), "quantise"});
    ops.push_back({std::make_unique<computation::MatMulInteger>(), "matmul"});
    ops.push_back({std::make_unique<computation::DequantizeLinear>(), "dequantise"});
    EXPECT(findDevice("amd", 0)->type() == Device::Type::Amd);
    auto exe = compile(computation::Graph(std::move(topo), std::move(ops),
                                          {{x, "x"}, {xq, "xq"}, {scale, "scale"}, {zp, "zp"}, {w, "W"}, {acc, "acc"}, {y, "y"}}),
                       "hip", "flat");
    exe->setInput(0, x_.data(), x_.size() * 4);
    exe->run();
    exe->getOutput(0, out.data(), out.size() * 4);// the blocking copy waits for the kernels
    std::vector<uint8_t> q(M * K);
    float s;
    uint8_t z;
    oracle_dynamic_quantize_linear(q.data(), &s, &z, x_.data(), x_.size());
    std::vector<int32_t> accRef(M * N);
    oracle_matmul_integer(accRef.data(), q.data(), w_.data(), &z, 0, 1, nullptr, 1, 1, 1, M, K, N, nullptr, nullptr, 1, 1, 8);
    oracle_dequantize_linear(ref.data(), accRef.data(), &s, nullptr, 1, 1, M * N, ORACLE_I32, 1, 1);
    EXPECT(std::memcmp(out.data(), ref.data(), out.size() * 4) == 0);
    auto times = exe->bench(true);
    EXPECT(times.size() == 2);// the dequantisation went into the product
    auto dir = std::filesystem::temp_directory_path() / ("rg_host_trace_gpu_" + std::to_string(::getpid()));
    exe->trace(dir.string(), "npy");
    // node 1 reads xq, W, zp, scale and writes y: the fifth file of that node is y
    auto meta = readFile(dir / "node000001.meta");
    std::string metaText(meta.begin(), meta.end());
    auto at = metaText.find("output\t0\ty\t");
    EXPECT(at != std::string::npos);
    if (at != std::string::npos) {
        auto file = metaText.substr(at + 11, metaText.find('\n', at) - at - 11);
        auto npy = readFile(file);
        EXPECT(npy.size() == 128 + ref.size() * 4 && std::memcmp(npy.data() + 128, ref.data(), ref.size() * 4) == 0);
    }
    std::filesystem::remove_all(dir);
}

static void transposeHip() {
    runtime::Resources res;
    auto &dev = amd();
    auto run = [&](DataType dt, Shape shape, Permutation perm) {
        auto x = Tensor::share(dt, shape);
        Shape outShape;
        for (auto p : perm) outShape.push_back(shape[p]);
        auto y = Tensor::share(dt, outShape);
        auto kernels = TransposeCollector(Device::Type::Amd, perm).filter({*x}, {*y});
        EXPECT(kernels.size() == 1);
        auto routine = kernels[0]->lower(res).routine;
        std::vector<uint8_t> x_(x->bytesSize()), y_(x_.size()), ref(x_.size());
        std::mt19937 rng(8);
        for (auto &v : x_) v = rng();
        auto mx = dev.malloc(x_.size()), my = dev.malloc(x_.size());
        mx->copyFromHost(x_.data());
        void const *inputs[]{*mx};
        void *outputs[]{*my};
        routine(res, nullptr, inputs, outputs);
        my->copyToHost(y_.data());
        oracle_transpose(ref.data(), x_.data(), shape.data(), perm.data(), static_cast<int>(shape.size()), static_cast<uint32_t>(dt.size()));
        EXPECT(y_ == ref);
    };
    run(DataType::F32, {1, 3, 2, 5}, {2, 3, 0, 1});// src/04kernel/test/kernels/transpose/test_cuda.cpp
    run(DataType::FP16, {2, 48, 8, 128}, {0, 2, 1, 3});
    run(DataType::U8, {5, 7, 3}, {2, 0, 1});
    run(DataType::F64, {4, 1, 6}, {2, 1, 0});
}

// Prefill of an attention block with the data in the layout a projection leaves it in
// ([N, seq, heads, D]): RotaryEmbedding -> Transpose to [N, heads, seq, D] -> Attention (tiled kernel,
// caches filled from position 0) -> Transpose back.
static void prefillAttentionStream() {
    using namespace computation;
    constexpr dim_t N = 2, H = 4, Hkv = 2, D = 128, S = 32, CAP = 64;
    constexpr float theta = 10000.f;
    auto qIn = Tensor::share(DataType::FP16, Shape{N, S, H, D}), qT = Tensor::share(DataType::FP16, Shape{N, H, S, D});
    auto kIn = Tensor::share(DataType::FP16, Shape{N, S, Hkv, D}), kT = Tensor::share(DataType::FP16, Shape{N, Hkv, S, D});
    auto pos = Tensor::share(DataType::I64, Shape{N, S}), past = Tensor::share(DataType::I64, Shape{1});
    auto cache = Tensor::share(DataType::FP16, Shape{N, Hkv, CAP, D});
    // edges: 0 q 1 k 2 v 3 pos 4 past | 5 qr | 6 kr | 7 qT | 8 kT | 9 vT | 10 oT 11 kc 12 vc | 13 o
    graph_topo::GraphTopo topo(5, 3);
    topo.pushNode({0, 3}, 0, 1);
    topo.pushNode({1, 3}, 0, 1);
    topo.pushNode({5}, 0, 1);
    topo.pushNode({6}, 0, 1);
    topo.pushNode({2}, 0, 1);
    topo.pushNode({7, 8, 9, 4}, 0, 3);
    topo.pushNode({10}, 0, 1);
    topo.setGlobalOutput(0, 13);
    topo.setGlobalOutput(1, 11);
    topo.setGlobalOutput(2, 12);
    std::vector<computation::Node> ops;
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_q"});
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_k"});
    for (auto name : {"q_heads_first", "k_heads_first", "v_heads_first"})
        ops.push_back({std::make_unique<Transpose>(kernel::Permutation{0, 2, 1, 3}), name});
    ops.push_back({std::make_unique<Attention>(CAP), "attention"});
    ops.push_back({std::make_unique<Transpose>(kernel::Permutation{0, 2, 1, 3}), "o_tokens_first"});
    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    auto stream = computation::Graph(std::move(topo), std::move(ops),
                                     {{qIn, "q"}, {kIn, "k"}, {kIn, "v"}, {pos, "pos"}, {past, "past"}, {qIn, "qr"}, {kIn, "kr"},
                                      {qT, "qT"}, {kT, "kT"}, {kT, "vT"}, {qT, "oT"}, {cache, "k_cache"}, {cache, "v_cache"}, {qIn, "o"}})
                      .lower(Target::Amd)
                      .lower(dev, reusableAllocate);
    std::mt19937 rng(12);
    std::normal_distribution<float> n01;
    auto randomHalf = [&](size_t n) { std::vector<uint16_t> v(n); for (auto &e : v) e = f2h(n01(rng)); return v; };
    auto q_ = randomHalf(qIn->elementsSize()), k_ = randomHalf(kIn->elementsSize()), v_ = randomHalf(kIn->elementsSize());
    std::vector<int64_t> pos_(N * S);
    for (dim_t b = 0; b < N; ++b)
        for (dim_t t = 0; t < S; ++t) pos_[b * S + t] = t;
    int64_t zero = 0;
    stream.setData(0, q_.data(), q_.size() * 2);
    stream.setData(1, k_.data(), k_.size() * 2);
    stream.setData(2, v_.data(), v_.size() * 2);
    stream.setData(3, pos_.data(), pos_.size() * 8);
    stream.setData(4, &zero, 8);
    stream.run();
    device::sync(Device::Type::Amd);
    std::vector<uint16_t> o(q_.size()), kc(cache->elementsSize()), vc(kc.size());
    EXPECT(stream.copyData(13, o.data(), o.size() * 2) && stream.copyData(11, kc.data(), kc.size() * 2) && stream.copyData(12, vc.data(), vc.size() * 2));

    // oracle: rotate (positions 0 .. S-1), then per (batch row, head) causal attention over the new rows
    auto rope = [&](std::vector<uint16_t> const &x, dim_t heads) {
        std::vector<float> xf(x.size()), yf(x.size());
        for (size_t i = 0; i < x.size(); ++i) xf[i] = h2f(x[i]);
        oracle_rope_f32(yf.data(), xf.data(), pos_.data(), 1, N, S, heads, D, theta, 1);
        std::vector<uint16_t> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) y[i] = f2h(yf[i]);
        return y;
    };
    auto qr = rope(q_, H), kr = rope(k_, Hkv);
    bool cacheOk = true, ok = true;
    float const scale = 1.0f / std::sqrt(static_cast<float>(D));
    std::vector<float> scratch(2 * S * S), ref(S * D), qf(S * D), kf(S * D), vf(S * D);
    for (dim_t b = 0; b < N; ++b)
        for (dim_t h = 0; h < H; ++h) {
            dim_t const kh = h / (H / Hkv);
            for (dim_t t = 0; t < S; ++t)
                for (dim_t i = 0; i < D; ++i) {
                    qf[t * D + i] = h2f(qr[((b * S + t) * H + h) * D + i]);
                    // keys as the device wrote them to the cache (rotated within the rotary embedding's tolerance)
                    kf[t * D + i] = h2f(kc[((b * Hkv + kh) * CAP + t) * D + i]);
                    vf[t * D + i] = h2f(vc[((b * Hkv + kh) * CAP + t) * D + i]);
                    cacheOk &= std::fabs(kf[t * D + i] - h2f(kr[((b * S + t) * Hkv + kh) * D + i])) <= 2e-3f;
                    cacheOk &= vc[((b * Hkv + kh) * CAP + t) * D + i] == v_[((b * S + t) * Hkv + kh) * D + i];
                }
            oracle_attention_head_f32(ref.data(), qf.data(), kf.data(), vf.data(), S, 0, D, scale, 1, scratch.data());
            for (dim_t t = 0; t < S; ++t)
                for (dim_t i = 0; i < D; ++i) ok &= std::fabs(h2f(o[((b * S + t) * H + h) * D + i]) - ref[t * D + i]) <= 4e-3f;
        }
    EXPECT(cacheOk);
    EXPECT(ok);
}

// The reference's test shapes (src/04kernel/test/kernels/{split,concat,expand,where}/test_cpu.cpp) through
// build -> lower -> routine on the AMD device, against the oracle's restatement of the CPU kernels
static void dataMoversHip() {
    auto &dev = amd();
    runtime::Resources res;
    std::vector<dim_t> const sizes{1, 9, 3, 7};
    auto joined = Tensor::share(DataType::F32, Shape{2, 3, 1, 20, 7, 7});
    std::vector<Arc<Tensor>> parts;
    TensorRefs refs;
    for (auto n : sizes) parts.push_back(Tensor::share(DataType::F32, Shape{2, 3, 1, n, 7, 7}));
    for (auto const &t : parts) refs.emplace_back(*t);
    SplitInfo info(3, refs);
    std::vector<float> data(joined->elementsSize());
    std::iota(data.begin(), data.end(), 0.f);
    auto dJoined = dev.malloc(joined->bytesSize());
    dJoined->copyFromHost(data.data());
    std::vector<Arc<Device::Blob>> dParts;
    std::vector<std::vector<float>> want, got;
    std::vector<void *> wantPtr, outPtr;
    for (auto const &t : parts) {
        dParts.push_back(dev.malloc(t->bytesSize()));
        want.emplace_back(t->elementsSize());
        got.emplace_back(t->elementsSize(), -1.f);
    }
    for (size_t j = 0; j < parts.size(); ++j) {
        wantPtr.push_back(want[j].data());
        outPtr.push_back(dParts[j]->get());
    }
    {// Split
        auto kernel = SplitHip::build(info);
        EXPECT(kernel != nullptr);
        auto routine = kernel->lower(res).routine;
        void const *inputs[]{dJoined->get()};
        routine(res, nullptr, inputs, outPtr.data());
        oracle_split(wantPtr.data(), data.data(), info.segments.data(), info.segments.size(), info.blockCount, info.sum);
        bool ok = true;
        for (size_t j = 0; j < parts.size(); ++j) {
            dParts[j]->copyToHost(got[j].data());
            ok &= got[j] == want[j];
        }
        EXPECT(ok);
        EXPECT(want[1][0] == 49.f && want[3][7 * 49] == 20 * 49 + 13 * 49);// the reference's own expectation (offsets 0, 1, 10, 13)
    }
    {// Concat of the parts gives the joined tensor back
        auto kernel = ConcatHip::build(info);
        auto routine = kernel->lower(res).routine;
        auto dOut = dev.malloc(joined->bytesSize());
        std::vector<void const *> inputs(outPtr.begin(), outPtr.end());
        void *outputs[]{dOut->get()};
        routine(res, nullptr, inputs.data(), outputs);
        std::vector<float> back(data.size(), -1.f), ref(data.size());
        dOut->copyToHost(back.data());
        std::vector<void const *> hostParts(wantPtr.begin(), wantPtr.end());
        oracle_concat(ref.data(), hostParts.data(), info.segments.data(), info.segments.size(), info.blockCount, info.sum);
        EXPECT(back == ref && back == data);
    }
    {// Expand {3, 4, 1, 6} -> {2, 3, 4, 5, 6}
        auto in = Tensor::share(DataType::F32, Shape{3, 4, 1, 6}), out = Tensor::share(DataType::F32, Shape{2, 3, 4, 5, 6});
        ExpandInfo e(*in, *out);
        auto kernel = ExpandHip::build(e);
        EXPECT(kernel != nullptr);
        auto routine = kernel->lower(res).routine;
        std::vector<float> x(in->elementsSize()), y(out->elementsSize(), -1.f), ref(out->elementsSize());
        std::iota(x.begin(), x.end(), 0.f);
        auto dx = dev.malloc(in->bytesSize()), dy = dev.malloc(out->bytesSize());
        dx->copyFromHost(x.data());
        void const *inputs[]{dx->get()};
        void *outputs[]{dy->get()};
        routine(res, nullptr, inputs, outputs);
        dy->copyToHost(y.data());
        std::vector<uint32_t> si, so;
        for (auto [i, o] : e.strides) { si.push_back(i); so.push_back(o); }
        oracle_expand(ref.data(), x.data(), si.data(), so.data(), static_cast<int>(si.size()), e.blockSize, e.blockCount);
        bool pattern = true;// test_cpu.cpp:27-38: result[i][j][k][m] = 6 j + m
        for (size_t idx = 0; idx < y.size(); ++idx) pattern &= y[idx] == static_cast<float>((idx / 30) % 12 * 6 + idx % 6);
        EXPECT(y == ref && pattern);
    }
    {// Where: c {2, 5}, x {2, 3, 2, 5}, y {3, 2, 5}
        auto c = Tensor::share(DataType::Bool, Shape{2, 5});
        auto x = Tensor::share(DataType::F32, Shape{2, 3, 2, 5}), y = Tensor::share(DataType::F32, Shape{3, 2, 5});
        auto kernel = WhereHip::build({*c, *x, *y});
        EXPECT(kernel != nullptr);
        auto const &b = static_cast<WhereHip const &>(*kernel).broadcaster;
        auto routine = kernel->lower(res).routine;
        std::mt19937 rng(5);
        std::vector<uint8_t> c_(10);
        std::vector<float> x_(60), y_(30), out(60, -1.f), ref(60);
        for (auto &v : c_) v = rng() & 1;
        for (auto &v : x_) v = static_cast<float>(rng() % 100);
        for (auto &v : y_) v = static_cast<float>(100 + rng() % 100);
        auto dc = dev.malloc(10), dx = dev.malloc(240), dy = dev.malloc(120), dout = dev.malloc(240);
        dc->copyFromHost(c_.data());
        dx->copyFromHost(x_.data());
        dy->copyFromHost(y_.data());
        void const *inputs[]{dc->get(), dx->get(), dy->get()};
        void *outputs[]{dout->get()};
        routine(res, nullptr, inputs, outputs);
        dout->copyToHost(out.data());
        oracle_where(ref.data(), c_.data(), x_.data(), y_.data(), b.strides.data(), static_cast<int>(b.strides.size() / 4),
                     b.outputsCount, 4);
        bool direct = true;// numpy semantics written out: c broadcasts over the first two dimensions, y over the first
        for (size_t i = 0; i < 60; ++i) direct &= ref[i] == (c_[i % 10] ? x_[i] : y_[i % 30]);
        EXPECT(out == ref && direct);
    }
}

// A decode step whose projection leaves q, k and v in one tensor: Split -> RotaryEmbedding (q, k) -> Attention,
// lowered for the AMD device and stepped, against the oracle chain
static void fusedQkvDecodeStream() {
    using namespace computation;
    constexpr dim_t N = 2, H = 8, Hkv = 2, D = 128, S = 48;
    constexpr float theta = 10000.f;
    auto qkv = Tensor::share(DataType::FP16, Shape{N, 1, (H + 2 * Hkv) * D});
    auto qFlat = Tensor::share(DataType::FP16, Shape{N, 1, H * D}), kFlat = Tensor::share(DataType::FP16, Shape{N, 1, Hkv * D});
    auto q = Tensor::share(DataType::FP16, Shape{N, 1, H, D}), qa = Tensor::share(DataType::FP16, Shape{N, H, 1, D});
    auto k = Tensor::share(DataType::FP16, Shape{N, 1, Hkv, D}), ka = Tensor::share(DataType::FP16, Shape{N, Hkv, 1, D});
    auto pos = Tensor::share(DataType::I64, Shape{N, 1}), past = Tensor::share(DataType::I64, Shape{N});
    auto cache = Tensor::share(DataType::FP16, Shape{N, Hkv, S, D});
    // edges: 0 qkv 1 pos 2 past | 3 q 4 k 5 v (split) | 6 q4 | 7 k4 | 8 qr | 9 kr | 10 q' | 11 k' | 12 v' | 13 o 14 kc 15 vc
    graph_topo::GraphTopo topo(3, 3);
    topo.pushNode({0}, 0, 3);      // Split
    topo.pushNode({3}, 0, 1);      // Reshape q -> [N, 1, H, D]
    topo.pushNode({4}, 0, 1);      // Reshape k
    topo.pushNode({6, 1}, 0, 1);   // rope q
    topo.pushNode({7, 1}, 0, 1);   // rope k
    topo.pushNode({8}, 0, 1);      // heads first (seq is 1: a reshape)
    topo.pushNode({9}, 0, 1);
    topo.pushNode({5}, 0, 1);
    topo.pushNode({10, 11, 12, 2}, 0, 3);
    for (count_t i = 0; i < 3; ++i) topo.setGlobalOutput(i, 13 + i);
    std::vector<computation::Node> ops;
    ops.push_back({std::make_unique<Split>(2), "split_qkv"});
    ops.push_back({std::make_unique<Reshape>(), "q_heads"});
    ops.push_back({std::make_unique<Reshape>(), "k_heads"});
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_q"});
    ops.push_back({std::make_unique<RotaryEmbedding>(theta), "rope_k"});
    ops.push_back({std::make_unique<Reshape>(), "q_heads_first"});
    ops.push_back({std::make_unique<Reshape>(), "k_heads_first"});
    ops.push_back({std::make_unique<Reshape>(), "v_heads_first"});
    ops.push_back({std::make_unique<Attention>(S), "attention"});
    auto dev = device::init(Device::Type::Amd, 0, "pool=4294967296");
    auto stream = computation::Graph(std::move(topo), std::move(ops),
                                     {{qkv, "qkv"}, {pos, "pos"}, {past, "past"}, {qFlat, "q"}, {kFlat, "k"}, {kFlat, "v"},
                                      {q, "q4"}, {k, "k4"}, {q, "qr"}, {k, "kr"}, {qa, "q'"}, {ka, "k'"}, {ka, "v'"},
                                      {qa, "o"}, {cache, "k_cache"}, {cache, "v_cache"}})
                      .lower(Target::Amd)
                      .lower(dev, reusableAllocate);
    std::mt19937 rng(44);
    std::normal_distribution<float> n01;
    auto randomHalf = [&](size_t n) { std::vector<uint16_t> v(n); for (auto &e : v) e = f2h(n01(rng)); return v; };
    auto kc = randomHalf(cache->elementsSize()), vc = randomHalf(cache->elementsSize());
    stream.getData(14)->copyFromHost(kc.data());
    stream.getData(15)->copyFromHost(vc.data());
    int64_t pastLen[N] = {9, 30};
    float const scale = 1.0f / std::sqrt(static_cast<float>(D));
    for (int step = 0; step < 3; ++step) {
        auto x = randomHalf(qkv->elementsSize());
        stream.setData(0, x.data(), x.size() * 2);
        stream.setData(1, pastLen, sizeof pastLen);
        stream.setData(2, pastLen, sizeof pastLen);
        stream.run();
        device::sync(Device::Type::Amd);
        std::vector<uint16_t> o(N * H * D), kcOut(kc.size()), vcOut(vc.size());
        EXPECT(stream.copyData(13, o.data(), o.size() * 2) && stream.copyData(14, kcOut.data(), kc.size() * 2) &&
               stream.copyData(15, vcOut.data(), vc.size() * 2));
        // the oracle chain: split by hand (rows of q | k | v), rope on up-cast values with one rounding back, attention
        constexpr dim_t row = (H + 2 * Hkv) * D;
        std::vector<float> qf(N * H * D), kf(N * Hkv * D), qr(qf.size()), kr(kf.size());
        for (dim_t b = 0; b < N; ++b) {
            for (dim_t i = 0; i < H * D; ++i) qf[b * H * D + i] = h2f(x[b * row + i]);
            for (dim_t i = 0; i < Hkv * D; ++i) kf[b * Hkv * D + i] = h2f(x[b * row + H * D + i]);
        }
        oracle_rope_f32(qr.data(), qf.data(), pastLen, 1, N, 1, H, D, theta, 1);
        oracle_rope_f32(kr.data(), kf.data(), pastLen, 1, N, 1, Hkv, D, theta, 1);
        bool rowsOk = true;
        for (dim_t b = 0; b < N; ++b)
            for (dim_t h = 0; h < Hkv; ++h) {
                auto const at = ((b * Hkv + h) * S + pastLen[b]) * D;
                for (dim_t i = 0; i < D; ++i) rowsOk &= std::fabs(h2f(kcOut[at + i]) - h2f(f2h(kr[(b * Hkv + h) * D + i]))) <= 2e-3f;
                std::memcpy(&kc[at], &kcOut[at], D * 2);
                std::memcpy(&vc[at], &x[b * row + (H + Hkv) * D + h * D], D * 2);// v rows appended bit for bit
            }
        EXPECT(rowsOk && kcOut == kc && vcOut == vc);
        bool ok = true;
        std::vector<float> scratch(2 * S), ref(D), q1(D);
        for (dim_t b = 0; b < N; ++b)
            for (dim_t h = 0; h < H; ++h) {
                dim_t const len = pastLen[b] + 1, kh = h / (H / Hkv);
                std::vector<float> kk(len * D), vv(len * D);
                for (size_t i = 0; i < len * D; ++i) {
                    kk[i] = h2f(kc[(b * Hkv + kh) * S * D + i]);
                    vv[i] = h2f(vc[(b * Hkv + kh) * S * D + i]);
                }
                for (dim_t i = 0; i < D; ++i) q1[i] = h2f(f2h(qr[(b * H + h) * D + i]));
                oracle_attention_head_f32(ref.data(), q1.data(), kk.data(), vv.data(), 1, pastLen[b], D, scale, 1, scratch.data());
                for (dim_t i = 0; i < D; ++i) ok &= std::fabs(h2f(o[(b * H + h) * D + i]) - ref[i]) <= 4e-3f;
            }
        EXPECT(ok);
        for (auto &p : pastLen) ++p;
    }
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
    // usage: rg_host_tests [cpu|gpu] [case]   (gpu = the cpu cases and those that need the device)
    std::string mode = argc > 1 ? argv[1] : "cpu";
    std::string only = argc > 2 ? argv[2] : "";
    RUN(broadcasterKnownAnswer);
    RUN(shapeDigests);
    RUN(memPoolBestFit);
    RUN(resourcesAndErrors);
    RUN(collectorsSelectOrDecline);
    RUN(graphTopoAndBuilder);
    RUN(offsetCalculatorPlan);
    RUN(allocatorsAndStreamOnCpu);
    RUN(executorOnCpu);
    RUN(transposeInfoDigest);
    RUN(computationGraphLowers);
    RUN(dataMoverDigests);
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
        RUN(transposeHip);
        RUN(dataMoversHip);
        RUN(fusedQkvDecodeStream);
        RUN(quantisedLinearStream);
        RUN(normQuantisedLinearStream);
        RUN(executorOnGpu);
        RUN(decodeAttentionStream);
        RUN(prefillAttentionStream);
        RUN(longChainRecorded);
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
