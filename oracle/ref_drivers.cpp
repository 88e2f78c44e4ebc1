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

#include <cstdio>
#include <cstdint>

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
