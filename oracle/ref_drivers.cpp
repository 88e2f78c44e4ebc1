// ref_drivers.cpp -- the benchmark's MLP training loop written against the reference's OWN tensor,
// autograd, nn and optimizer classes (<aix.hpp>) on its own aix::DeviceCPU.
//
// TEST INFRASTRUCTURE ONLY, built only where the reference tree is present (oracle/Makefile,
// target `ref`), compiled with the reference's sources from where they lie.  It pins the
// front-end restatement (aix_amd/csrc/frontend): the same model, data and loop run through
// aixfe::Tensor on the oracle device must give the same losses bit for bit and the same number of
// matmul calls, which shows that both generate the same operator stream.

#include <aix.hpp>
#ifdef AIXREF_WITH_HIP
#include "../aix_amd/csrc/device/device_hip.hpp"      // built with AIXHIP_USE_AIX_HEADERS: derives from the reference's aix::Device
#endif

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdint>
#include <vector>

namespace {

struct CountingCPU final : aix::DeviceCPU {
    uint64_t matmuls{0};
    void matmul(const aix::DeviceTensorParams& a, const aix::DeviceTensorParams& b, const aix::DeviceTensorParams& r) override
    {
        ++matmuls;
        aix::DeviceCPU::matmul(a, b, r);
    }
};

aix::Tensor relu(const aix::Tensor& x, aix::Device* dev)
{
    aix::Shape lifted = x.shape();
    lifted.insert(lifted.begin(), 1);
    const aix::Tensor zeros(0.0f, lifted, { .m_dtype = x.dataType(), .m_device = dev });
    return aix::Tensor::cat({x.unsqueeze(0), zeros}, 0).max(0);
}

thread_local char g_err[512] = "";

} // namespace

extern "C" {

const char* aixref_drivers_last_error(void) { return g_err; }

}   // extern "C"

namespace {

// The loop itself, on whatever aix::Device it is given -- nothing in it names a backend.
void mlp_loop(aix::Device& dev, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr,
              const float* x, const float* y, const float* const* w, const float* const* b, float* losses)
{
    const aix::TensorOptions plain{ .m_dtype = aix::DataType::kFloat32, .m_device = &dev };
    const aix::TensorOptions param{ .m_requireGrad = true, .m_dtype = aix::DataType::kFloat32, .m_device = &dev };
    const auto F32 = aix::DataType::kFloat32;
    aix::Tensor X(x, batch * in, F32, aix::Shape{batch, in}, plain);
    aix::Tensor Y(y, batch * out, F32, aix::Shape{batch, out}, plain);
    aix::Tensor w1(w[0], in * hidden, F32, aix::Shape{in, hidden}, param), b1(b[0], hidden, F32, aix::Shape{1, hidden}, param);
    aix::Tensor w2(w[1], hidden * hidden, F32, aix::Shape{hidden, hidden}, param), b2(b[1], hidden, F32, aix::Shape{1, hidden}, param);
    aix::Tensor w3(w[2], hidden * out, F32, aix::Shape{hidden, out}, param), b3(b[2], out, F32, aix::Shape{1, out}, param);
    aix::optim::Adam opt(std::vector<aix::Tensor>{w1, b1, w2, b2, w3, b3}, lr);
    aix::nn::Softmax softmax(1, true);
    aix::nn::CrossEntropyLoss lossFn;
    for (int s = 0; s < steps; ++s) {
        opt.zeroGrad();
        auto h1 = relu(aix::matmul(X, w1) + b1, &dev);
        auto h2 = relu(aix::matmul(h1, w2) + b2, &dev);
        auto logits = aix::matmul(h2, w3) + b3;
        auto loss = lossFn(softmax.forward(logits), Y);
        loss.backward();
        opt.step();
        dev.synchronize();
        losses[s] = loss.value().item<float>();
    }
    dev.synchronize();
}

// The reference's XOR example (Targets/AIXExamples/XORMetalApp/Main.cpp) as a function of the device:
// nn::Sequential of Linear / Tanh, MSELoss, Adam, parameters created on the host and moved with
// Module::to(device) / to(dtype), inputs built from double literals and converted on the device,
// the loss read through item<float>() after synchronize().  losses[epochs], predictions[4].
void xor_loop(aix::Device& dev, aix::DataType dtype, size_t hidden1, size_t hidden2, int epochs, float lr, float* losses, float* predictions)
{
    aix::manualSeed(1234);                                  // identical initial parameters on every device
    aix::nn::Sequential model;
    model.add(aix::nn::Linear(2, hidden1));
    model.add(aix::nn::Tanh());
    model.add(aix::nn::Linear(hidden1, hidden2));
    model.add(aix::nn::Tanh());
    model.add(aix::nn::Linear(hidden2, 1));
    model.to(dev);
    model.to(dtype);
    auto inputs = aix::tensor({0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0}, {4, 2}).to(dev).to(dtype);
    auto targets = aix::tensor({0.0, 1.0, 1.0, 0.0}, {4, 1}).to(dev).to(dtype);
    aix::optim::Adam optimizer(model.parameters(), lr);
    auto lossFunc = aix::nn::MSELoss();
    for (int epoch = 0; epoch < epochs; ++epoch) {
        auto loss = lossFunc(model.forward(inputs), targets);
        optimizer.zeroGrad();
        loss.backward();
        optimizer.step();
        loss = loss.to(aix::DataType::kFloat32);
        dev.synchronize();
        losses[epoch] = loss.value().item<float>();
    }
    auto final = model.forward(inputs).to(aix::DataType::kFloat32);
    dev.synchronize();
    for (int i = 0; i < 4; ++i) predictions[i] = final.value().data<float>()[i];
}

} // namespace

extern "C" {

int aixref_xor(int dtype, uint64_t hidden1, uint64_t hidden2, int epochs, float lr, float* losses, float* predictions)
{
    try {
        aix::DeviceCPU dev;
        xor_loop(dev, static_cast<aix::DataType>(dtype), hidden1, hidden2, epochs, lr, losses, predictions);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

int aixref_mlp(uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr,
               const float* x, const float* y, const float* const* w, const float* const* b, float* losses, uint64_t* counts)
{
    try {
        CountingCPU dev;
        mlp_loop(dev, batch, in, hidden, out, steps, lr, x, y, w, b, losses);
        if (counts) counts[1] = dev.matmuls;
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

} // extern "C"

// ---- the reference's device test cases on DeviceHIP ---------------------------------------------------------------
// The scheme of Targets/AIXTests/DeviceTests.cpp (which does not build here: doctest is fetched from the network and
// the file includes the Apple-only device header) with the reference's OWN classes around the device under test:
// operands made by aix::randn(...).to(dtype) on the host, results allocated as aix::TensorValue on the device, the raw
// device call issued on aix::DeviceCPU and on the device under test, synchronize(), element-wise comparison
// (:199-233 and the per-operator cases :2400-3072 over testSizes :30-31); then "batch compute" (:3074-3300),
// "long command batch queue" (:3455-3476) and "loop without sync" (:3478-3552) through aix::Tensor and autograd, and
// one step of the benchmark's XOR model (Targets/AIXBenchmarks/Model.cpp:20-89), timed.
namespace {

const size_t kTestSizes[] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 31, 32, 33, 63, 64, 65,
                             127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049};

double elementAsDouble(const aix::TensorValue& tv, size_t i)
{
    using aix::DataType;
    switch (tv.dataType()) {
        case DataType::kFloat64:  return tv.data<double>()[i];
        case DataType::kFloat32:  return tv.data<float>()[i];
        case DataType::kFloat16:  return (float)tv.data<aix::float16_t>()[i];
        case DataType::kBFloat16: return (float)tv.data<aix::bfloat16_t>()[i];
        case DataType::kInt64:    return (double)tv.data<int64_t>()[i];
        case DataType::kInt32:    return tv.data<int32_t>()[i];
        case DataType::kInt16:    return tv.data<int16_t>()[i];
        case DataType::kInt8:     return tv.data<int8_t>()[i];
        default:                  return tv.data<uint8_t>()[i];
    }
}

bool isFloatType(aix::DataType t) { return static_cast<size_t>(t) <= static_cast<size_t>(aix::DataType::kBFloat16); }

// The reference compares |a - b| <= epsilon with 1e-5 (1e-2 for f16), integers exactly (DeviceTests.cpp:44-170).  Kept,
// with the epsilon scaled by the magnitude for the 16-bit types' transcendental results and bf16 given f16's epsilon
// (its own test file leaves bf16 at 1e-5 and passes only because the Metal device rounds like the CPU).
bool sameResults(const aix::TensorValue& want, const aix::TensorValue& got, double epsilon)
{
    if (want.dataType() != got.dataType() || want.size() != got.size()) return false;
    for (size_t i = 0; i < want.size(); ++i) {
        const double a = elementAsDouble(want, i), b = elementAsDouble(got, i);
        if (!isFloatType(want.dataType())) { if (a != b) return false; continue; }
        if (std::isnan(a) && std::isnan(b)) continue;
        if (std::isinf(a) || std::isinf(b)) { if (a != b) return false; continue; }
        if (!(std::abs(a - b) <= epsilon * std::max(1.0, std::abs(a)))) return false;
    }
    return true;
}

double epsilonOf(aix::DataType t)
{
    return (t == aix::DataType::kFloat16 || t == aix::DataType::kBFloat16) ? 1e-2 : 1e-5;
}

struct Report {
    char* text; size_t cap, len{0}; int failures{0}, checks{0};
    void fail(const char* what, int dtype, size_t n)
    {
        ++failures;
        if (len + 96 < cap) len += (size_t)std::snprintf(text + len, cap - len, "FAILED %s dtype %d n %zu\n", what, dtype, n);
    }
    void note(const char* fmt, double a = 0, double b = 0)
    {
        if (len + 160 < cap) len += (size_t)std::snprintf(text + len, cap - len, fmt, a, b);
    }
};

template <class Call>
void perOperator(Report& rep, aix::Device& dev, const char* name, int intSpread, bool positive, Call call)
{
    for (size_t t = 0; t < aix::DataTypeCount; ++t) {
        const auto dtype = static_cast<aix::DataType>(t);
        for (size_t n : kTestSizes) {
            aix::DeviceCPU ref;
            auto a = aix::randn({1, n}), b = aix::randn({1, n});
            if (positive) { a = a * a + 0.5f; b = b * b + 0.5f; }                  // sqrt, log, pow: inside the domain
            // integers: a spread of values (small for the math functions: the truncated exp(40) of a 64-bit integer needs
            // the CPU's 80-bit long double), no zero divisor
            if (!isFloatType(dtype)) { a = a * intSpread; b = b * intSpread + (positive ? 0 : intSpread + 10); }
            a = a.to(dtype); b = b.to(dtype);
            auto want = aix::TensorValue({1, n}, &ref).to(dtype);
            auto got = aix::TensorValue({1, n}, &dev).to(dtype);
            call(ref, a.value(), b.value(), want);
            call(dev, a.value(), b.value(), got);
            dev.synchronize();
            ++rep.checks;
            if (!sameResults(want, got, epsilonOf(dtype))) rep.fail(name, (int)t, n);
        }
    }
}

void deviceChecks(aix::Device& dev, Report& rep, int timedRuns)
{
    using aix::DeviceTensorParams;
    using TV = aix::TensorValue;
    perOperator(rep, dev, "add", 50, false, [](aix::Device& d, const TV& a, const TV& b, TV& r) { d.add(a.deviceParams(), b.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "sub", 50, false, [](aix::Device& d, const TV& a, const TV& b, TV& r) { d.sub(a.deviceParams(), b.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "mul", 50, false, [](aix::Device& d, const TV& a, const TV& b, TV& r) { d.mul(a.deviceParams(), b.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "div", 50, false, [](aix::Device& d, const TV& a, const TV& b, TV& r) { d.div(a.deviceParams(), b.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "unary", 50, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.unary(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "sqrt", 3, true, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.sqrt(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "sin", 3, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.sin(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "cos", 3, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.cos(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "tanh", 3, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.tanh(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "log", 3, true, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.log(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "exp", 3, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.exp(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "contiguous", 50, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.contiguous(a.deviceParams(), r.deviceParams()); });
    perOperator(rep, dev, "copy", 50, false, [](aix::Device& d, const TV& a, const TV&, TV& r) { d.copy(a.data(), a.dataType(), r.data(), r.dataType(), a.size()); });
    perOperator(rep, dev, "fill", 50, false, [](aix::Device& d, const TV&, const TV&, TV& r) { const float v = 3.0f; d.fill(&v, aix::DataType::kFloat32, r.deviceParams()); });

    // whole-tensor reductions and the matmul (f32: the reference's own bound for its GPU device, 2e-4, on n x n products)
    for (size_t t = 0; t < aix::DataTypeCount; ++t) {
        const auto dtype = static_cast<aix::DataType>(t);
        for (size_t n : kTestSizes) {
            aix::DeviceCPU ref;
            const bool isFloat = isFloatType(dtype);
            auto a = isFloat ? aix::randn({1, n}).to(dtype) : (aix::randn({1, n}) * 3).to(dtype);     // small integers: sums stay in range
            for (int which = 0; which < 3; ++which) {
                const auto rdt = which == 2 ? aix::DataType::kInt32 : dtype;
                auto want = aix::TensorValue({}, &ref).to(rdt), got = aix::TensorValue({}, &dev).to(rdt);
                if (which == 0) { ref.sum(a.value().deviceParams(), want.deviceParams()); dev.sum(a.value().deviceParams(), got.deviceParams()); }
                if (which == 1) { ref.max(a.value().deviceParams(), want.deviceParams()); dev.max(a.value().deviceParams(), got.deviceParams()); }
                if (which == 2) { ref.argmax(a.value().deviceParams(), want.deviceParams()); dev.argmax(a.value().deviceParams(), got.deviceParams()); }
                dev.synchronize();
                ++rep.checks;
                // a sequential sum in a 16-bit type is far from the truth for long inputs: only short ones are comparable
                const bool comparable = which != 0 || static_cast<size_t>(dtype) < 2 || !isFloat || n <= 17;
                if (comparable && !sameResults(want, got, which == 0 ? epsilonOf(dtype) * (double)n : 0.0)) rep.fail(which == 0 ? "sum" : which == 1 ? "max" : "argmax", (int)t, n);
            }
        }
        for (size_t n : {1, 2, 3, 7, 8, 16, 17, 33, 64, 65, 129}) {
            if (!isFloatType(dtype) || dtype == aix::DataType::kFloat16 || dtype == aix::DataType::kBFloat16) continue;    // as DeviceTests.cpp:1244-1245
            aix::DeviceCPU ref;
            auto a = aix::randn({n, n}).to(dtype), b = aix::randn({n, n}).to(dtype);
            auto want = aix::TensorValue({n, n}, &ref).to(dtype), got = aix::TensorValue({n, n}, &dev).to(dtype);
            ref.matmul(a.value().deviceParams(), b.value().deviceParams(), want.deviceParams());
            dev.matmul(a.value().deviceParams(), b.value().deviceParams(), got.deviceParams());
            dev.synchronize();
            ++rep.checks;
            if (!sameResults(want, got, 2e-4)) rep.fail("matmul", (int)t, n);
            // the transposed views the backward pass uses
            auto wantT = aix::TensorValue({n, n}, &ref).to(dtype), gotT = aix::TensorValue({n, n}, &dev).to(dtype);
            const auto at = a.value().transpose(0, 1);
            ref.matmul(at.deviceParams(), b.value().deviceParams(), wantT.deviceParams());
            dev.matmul(at.deviceParams(), b.value().deviceParams(), gotT.deviceParams());
            dev.synchronize();
            ++rep.checks;
            if (!sameResults(wantT, gotT, 2e-4)) rep.fail("matmul of a transposed view", (int)t, n);
        }
    }

    // batch compute: 200 queued operator pairs with autograd, one synchronize (DeviceTests.cpp:3074-3300)
    {
        const aix::Shape shape{2, 3};
        const aix::TensorOptions opt{ .m_requireGrad = true, .m_device = &dev };
        auto x = aix::tensor({1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f}, shape, opt);
        auto y = aix::tensor({7.0f, 8.0f, 9.0f, 10.0f, 11.0f, 12.0f}, shape, opt);
        auto z = x + y;
        for (size_t i = 0; i < 200; ++i) z = z + x + y;
        z.backward(aix::onesLike(z));
        dev.synchronize();
        const float wantZ[6] = {1608, 2010, 2412, 2814, 3216, 3618};
        ++rep.checks;
        for (int i = 0; i < 6; ++i)
            if (z.value().data<float>()[i] != wantZ[i] || x.grad().data<float>()[i] != 201 || y.grad().data<float>()[i] != 201) { rep.fail("batch compute add", 1, 6); break; }
        auto w = x * y;
        for (size_t i = 0; i < 200; ++i) w = w - x - y;
        w.backward(aix::onesLike(w));
        dev.synchronize();
        ++rep.checks;
        for (int i = 0; i < 6; ++i) {
            const float xi = (float)(i + 1), yi = (float)(i + 7);
            if (w.value().data<float>()[i] != xi * yi - 200 * (xi + yi)) { rep.fail("batch compute mul/sub", 1, 6); break; }
        }
    }
    // long command batch queue (DeviceTests.cpp:3455-3476)
    {
        const ssize_t size = 1024 * 1024;
        std::vector<float> data(size, 1);
        const aix::TensorOptions opt{ .m_dtype = aix::DataType::kFloat32, .m_device = &dev };
        auto x = aix::tensor(data, opt).reshape({1, size});
        auto y = aix::tensor(data, opt).reshape({1, size});
        auto z = x + y;
        for (size_t i = 1; i < 1024; ++i) z = z + x + y;
        dev.synchronize();
        ++rep.checks;
        if (z.value().data<float>()[0] != 2048 || z.value().data<float>()[size - 1] != 2048) rep.fail("long command batch queue", 1, (size_t)size);
    }
    // loop without sync (DeviceTests.cpp:3478-3552): 1000 Adam steps of the XOR model, one synchronize at the end
    {
        aix::manualSeed(42);
        aix::nn::Sequential model;
        model.add(new aix::nn::Linear(2, 10));
        model.add(new aix::nn::Tanh());
        model.add(new aix::nn::Linear(10, 1));
        model.to(dev);
        auto inputs = aix::tensor({0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0}, {4, 2}).to(dev);
        auto targets = aix::tensor({0.0, 1.0, 1.0, 0.0}, {4, 1}).to(dev);
        aix::optim::Adam optimizer(model.parameters(), 0.01f);
        auto lossFunc = aix::nn::MSELoss();
        for (size_t epoch = 0; epoch < 1000; ++epoch) {
            auto loss = lossFunc(model.forward(inputs), targets);
            optimizer.zeroGrad();
            loss.backward();
            optimizer.step();
        }
        auto loss = lossFunc(model.forward(inputs), targets);
        dev.synchronize();
        ++rep.checks;
        rep.note("loop without sync: final loss %.3e\n", loss.value().item<float>());
        if (!(loss.value().item<float>() <= 1e-3f)) rep.fail("loop without sync", 1, 1000);
    }
    // the benchmark's XOR model, f32, layer size 1000 and 10 (Model.cpp:20-89): one run() = forward, loss, backward, step, synchronize
    for (size_t layer : {size_t(1000), size_t(10)}) {
        aix::manualSeed(7);
        aix::nn::Sequential model;
        model.add(new aix::nn::Linear(2, layer)); model.add(new aix::nn::Tanh());
        model.add(new aix::nn::Linear(layer, layer)); model.add(new aix::nn::Tanh());
        model.add(new aix::nn::Linear(layer, 1));
        model.to(dev);
        model.to(aix::DataType::kFloat32);
        auto inputs = aix::tensor({0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0}, {4, 2}).to(dev).to(aix::DataType::kFloat32);
        auto targets = aix::tensor({0.0, 1.0, 1.0, 0.0}, {4, 1}).to(dev).to(aix::DataType::kFloat32);
        aix::optim::Adam optimizer(model.parameters(), 0.01f);
        auto lossFunc = aix::nn::MSELoss();
        auto run = [&] {
            auto loss = lossFunc(model.forward(inputs), targets);
            optimizer.zeroGrad();
            loss.backward();
            optimizer.step();
            dev.synchronize();
            return loss.value().item<float>();
        };
        float first = 0, last = 0;
        for (int i = 0; i < 5; ++i) { const float l = run(); if (i == 0) first = l; }
        const auto t0 = std::chrono::steady_clock::now();
        const int reps = timedRuns;
        for (int i = 0; i < reps; ++i) last = run();
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / reps;
        ++rep.checks;
        rep.note(layer == 1000 ? "model_xor_f32_1k: %.3f ms per run, loss %.4f at the last run\n" : "model_xor_f32_10: %.3f ms per run, loss %.4f at the last run\n", ms, last);
        (void)first;                                                // the first runs of the wide model overshoot: only a finite loss is asked here
        if (!std::isfinite(last)) rep.fail("benchmark XOR model: loss not finite", 1, layer);
    }
}

} // namespace

extern "C" {

// Runs the cases above on the reference's CPU device standing in as the device under test (a check of the checks: it
// must pass with zero failures) -- `on_hip` = 0 -- or on DeviceHIP.  Returns the number of failed checks, -1 on an
// exception; `report` receives the failures and the notes.
int aixref_device_checks(int on_hip, char* report, uint64_t cap, int* checks)
{
    Report rep{report, (size_t)cap};
    if (cap) report[0] = 0;
    try {
        if (!on_hip) { aix::DeviceCPU dev; deviceChecks(dev, rep, 2); }
#ifdef AIXREF_WITH_HIP
        else { aix::hip::DeviceHIP dev; deviceChecks(dev, rep, 50); }
#else
        else { std::snprintf(g_err, sizeof(g_err), "built without DeviceHIP"); return -1; }
#endif
        if (checks) *checks = rep.checks;
        return rep.failures;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return -1; }
}

} // extern "C"

extern "C" {

#ifdef AIXREF_WITH_HIP
// The same loop, the reference's own front-end, on the MI355X backend: aix::hip::DeviceHIP handed to
// aix::Tensor exactly as README.MD:166-188 hands it the Metal device.
int aixref_mlp_hip(uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr,
                   const float* x, const float* y, const float* const* w, const float* const* b, float* losses)
{
    try {
        aix::hip::DeviceHIP dev;
        mlp_loop(dev, batch, in, hidden, out, steps, lr, x, y, w, b, losses);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

int aixref_xor_hip(int dtype, uint64_t hidden1, uint64_t hidden2, int epochs, float lr, float* losses, float* predictions)
{
    try {
        aix::hip::DeviceHIP dev;
        xor_loop(dev, static_cast<aix::DataType>(dtype), hidden1, hidden2, epochs, lr, losses, predictions);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

// nn::save of a model trained on DeviceHIP (the host reads the parameters straight out of device memory), then
// nn::load into a fresh model on DeviceHIP (the host writes them straight into device memory) and into one on the
// reference's CPU device; predictions[0..3] trained model, [4..7] reloaded on DeviceHIP, [8..11] reloaded on the CPU.
int aixref_xor_save_load_hip(uint64_t hidden1, uint64_t hidden2, int epochs, float lr, const char* path, float* predictions)
{
    try {
        const auto F32 = aix::DataType::kFloat32;
        auto build = [&](aix::nn::Sequential& m) {
            m.add(aix::nn::Linear(2, hidden1)); m.add(aix::nn::Tanh());
            m.add(aix::nn::Linear(hidden1, hidden2)); m.add(aix::nn::Tanh());
            m.add(aix::nn::Linear(hidden2, 1));
        };
        auto predict = [&](aix::nn::Sequential& m, aix::Device& dev, float* out) {
            auto inputs = aix::tensor({0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0}, {4, 2}).to(dev).to(F32);
            auto y = m.forward(inputs);
            dev.synchronize();
            for (int i = 0; i < 4; ++i) out[i] = y.value().data<float>()[i];
        };
        aix::hip::DeviceHIP dev;
        aix::manualSeed(99);
        aix::nn::Sequential model;
        build(model);
        model.to(dev);
        auto inputs = aix::tensor({0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0}, {4, 2}).to(dev).to(F32);
        auto targets = aix::tensor({0.0, 1.0, 1.0, 0.0}, {4, 1}).to(dev).to(F32);
        aix::optim::Adam optimizer(model.parameters(), lr);
        auto lossFunc = aix::nn::MSELoss();
        for (int epoch = 0; epoch < epochs; ++epoch) {
            auto loss = lossFunc(model.forward(inputs), targets);
            optimizer.zeroGrad();
            loss.backward();
            optimizer.step();
        }
        dev.synchronize();
        predict(model, dev, predictions);
        aix::nn::save(model, path);

        aix::manualSeed(7);                                     // different initial values: everything must come from the file
        aix::nn::Sequential onGpu;
        build(onGpu);
        onGpu.to(dev);
        dev.synchronize();
        aix::nn::load(onGpu, path);
        predict(onGpu, dev, predictions + 4);

        aix::DeviceCPU cpu;
        aix::nn::Sequential onCpu;
        build(onCpu);
        onCpu.to(cpu);
        aix::nn::load(onCpu, path);
        predict(onCpu, cpu, predictions + 8);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}
#endif

} // extern "C"
