// driver.cpp -- native step loops for the benchmark (libaixhip_bench.so).
//
// The benchmark's "step" is one pass of an AIX expression through the device interface, issued
// from C++ through the tensor-value front-end exactly as an AIX program would issue it
// (Targets/AIXBenchmarks/Fuse.cpp:34-38, Tensor.cpp, Device.cpp:626-664 are the models), so that
// interpreter overhead of the Python harness never sits inside the timed region.
// Timing: steady_clock around the K steps bracketed by synchronize(), and HIP events on the
// device's stream around the same region.

#include "../../../include/aixhip.h"
#include "../device/device_hip.hpp"
#include "../frontend/mlp.hpp"
#include "../frontend/transformer.hpp"
#include "../frontend/value.hpp"

#include <chrono>
#include <cstdio>
#include <stdexcept>

using aix::DataType;
using aix::hip::DeviceHIP;
using aixfe::Shape;
using aixfe::Value;

namespace {

thread_local char g_err[512] = "";

struct Timer {
    DeviceHIP* dev;
    aixk_event *e0{nullptr}, *e1{nullptr};
    std::chrono::steady_clock::time_point t0;
    explicit Timer(DeviceHIP* d) : dev(d)
    {
        aixk_event_create(dev->kernelContext(), &e0);
        aixk_event_create(dev->kernelContext(), &e1);
    }
    ~Timer() { aixk_event_destroy(dev->kernelContext(), e0); aixk_event_destroy(dev->kernelContext(), e1); }
    void start()
    {
        dev->synchronize();
        t0 = std::chrono::steady_clock::now();
        aixk_event_record(dev->kernelContext(), e0);
    }
    void stop(double* wall_s, float* gpu_ms, int32_t* enqueue_us = nullptr)
    {
        dev->flush();
        aixk_event_record(dev->kernelContext(), e1);
        if (enqueue_us) *enqueue_us = (int32_t)(std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() * 1e6);
        dev->synchronize();
        *wall_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        aixk_event_elapsed_ms(dev->kernelContext(), e0, e1, gpu_ms);
    }
};

template <class F> int guarded(F&& f)
{
    try { f(); return 0; }
    catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

} // namespace

extern "C" {

typedef struct aixbench_result {
    double wall_s;        // K steps, synchronize to synchronize
    float  gpu_ms;        // same region between two events on the device's stream
    int32_t steps;
    int32_t enqueue_us;   // host time to issue the K steps (before waiting for the device)
} aixbench_result;

const char* aixbench_last_error(void) { return g_err; }

// Config 0: y = tanh(a*b + c) / (1 + exp(-a)) - 0.5*c on f32 [rows, cols]; a, b, c are host arrays.
// One step = the expression + flush; y_out (may be NULL) receives the last result.
int aixbench_fused_chain(aixhip_device* handle, uint64_t rows, uint64_t cols, const float* a, const float* b, const float* c,
                         int steps, int warmup, aixbench_result* res, float* y_out)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        const Shape shape{rows, cols};
        Value A = Value::fromHost(dev, DataType::kFloat32, shape, a);
        Value B = Value::fromHost(dev, DataType::kFloat32, shape, b);
        Value Cc = Value::fromHost(dev, DataType::kFloat32, shape, c);
        Value y;
        auto step = [&] {
            y = (A * B + Cc).tanh() / (1.0f + (-A).exp()) - 0.5f * Cc;
            dev->flush();
        };
        for (int i = 0; i < warmup; ++i) step();
        Timer t(dev);
        t.start();
        for (int i = 0; i < steps; ++i) step();
        t.stop(&res->wall_s, &res->gpu_ms, &res->enqueue_us);
        res->steps = steps;
        if (y_out) dev->copyToHost(y_out, y.data(), rows * cols * sizeof(float));
    });
}

// Config 1 items on f32 x[rows, cols] (and v[cols] for the broadcast add).  `which`:
//   0 sum(1)  1 max(1)  2 argmax(0)  3 sum()  4 x + v (row broadcast)  5 x.transpose(0,1).contiguous()
// out receives the last result (float or int32 as the op defines; may be NULL).
int aixbench_reduce_item(aixhip_device* handle, int which, uint64_t rows, uint64_t cols, const float* x, const float* v,
                         int steps, int warmup, aixbench_result* res, void* out)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        Value X = Value::fromHost(dev, DataType::kFloat32, Shape{rows, cols}, x);
        Value V = v ? Value::fromHost(dev, DataType::kFloat32, Shape{cols}, v) : Value();
        Value r;
        auto step = [&] {
            switch (which) {
                case 0: r = X.sum(1, false); break;
                case 1: r = X.max(1, false); break;
                case 2: r = X.argmax(0, false); break;
                case 3: r = X.sum(); break;
                case 4: r = X + V; break;
                case 5: r = X.transpose(0, 1).contiguous(); break;
                default: throw std::invalid_argument("unknown item");
            }
            dev->flush();
        };
        for (int i = 0; i < warmup; ++i) step();
        Timer t(dev);
        t.start();
        for (int i = 0; i < steps; ++i) step();
        t.stop(&res->wall_s, &res->gpu_ms, &res->enqueue_us);
        res->steps = steps;
        if (out) dev->copyToHost(out, r.data(), r.size() * aix::Device::dataTypeSize(r.dtype()));
    });
}

// Config 2: C = A[M,K] . B[K,N]; element type dtype (1 f32, 2 f16, 3 bf16); a, b are host arrays of
// that type.  layout: 0 NN, 1 NT (b given as [N,K], used through a transposed view), 2 TN (a given
// as [K,M]).  batch > 1: a, b hold `batch` matrices and each step issues `batch` matmuls on
// select(0, i) views, as the interface has no batch dim; layout + 4: ONE matmul on the [batch, ., .] stacks instead
// (the extension of matmul to operands with leading dims).
int aixbench_matmul(aixhip_device* handle, int dtype, uint64_t M, uint64_t N, uint64_t K, int layout, uint64_t batch,
                    const void* a, const void* b, int steps, int warmup, aixbench_result* res, void* out)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        const DataType dt = static_cast<DataType>(dtype);
        const bool stacked = (layout & 4) != 0;
        layout &= 3;
        const Shape sa = layout == 2 ? Shape{batch, K, M} : Shape{batch, M, K};
        const Shape sb = layout == 1 ? Shape{batch, N, K} : Shape{batch, K, N};
        Value A = Value::fromHost(dev, dt, sa, a);
        Value B = Value::fromHost(dev, dt, sb, b);
        std::vector<Value> r(batch);
        auto step = [&] {
            if (stacked) {
                r[0] = (layout == 2 ? A.transpose(1, 2) : A).matmul(layout == 1 ? B.transpose(1, 2) : B);
                dev->flush();
                return;
            }
            for (uint64_t i = 0; i < batch; ++i) {
                Value ai = A.select0(i), bi = B.select0(i);
                if (layout == 2) ai = ai.transpose(0, 1);
                if (layout == 1) bi = bi.transpose(0, 1);
                r[i] = ai.matmul(bi);
            }
            dev->flush();
        };
        for (int i = 0; i < warmup; ++i) step();
        Timer t(dev);
        t.start();
        for (int i = 0; i < steps; ++i) step();
        t.stop(&res->wall_s, &res->gpu_ms, &res->enqueue_us);
        res->steps = steps;
        if (out) dev->copyToHost(out, r[0].data(), M * N * aix::Device::dataTypeSize(dt));
    });
}

// Config 3: MLP training (in -> hidden -> hidden -> out, ReLU, softmax + cross-entropy, Adam) for
// `steps` steps from the given host parameters; losses[steps], step_seconds[steps] (may be NULL).
// single_pass = 0 differentiates as the reference does (once per path), 1 once per node.
int aixbench_mlp(aixhip_device* handle, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
                 const float* x, const float* y, const float* const* w, const float* const* b, float* losses, double* step_seconds)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        const aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        aixfe::runMlp(dev, cfg, host, losses, step_seconds);
    });
}

// The same with the L2 norms of the six parameters' gradients (w1, b1, w2, b2, w3, b3) of the first `norm_steps` steps in
// grad_norms[norm_steps * 6].
int aixbench_mlp_norms(aixhip_device* handle, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
                       const float* x, const float* y, const float* const* w, const float* const* b, float* losses, double* step_seconds,
                       float* grad_norms, int norm_steps)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        const aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        aixfe::runMlp(dev, cfg, host, losses, step_seconds, grad_norms, norm_steps);
    });
}

// A run that captures a step plans with a wide window: the planner's cost is paid once, at the capture, and a window of
// thousands of operators lets runs of equal kernels of a whole layer leave as one launch where the usual 200 operators cut
// them into a dozen (per-head transformer: 879 -> 509 graph nodes, 14.1 -> 12.1 ms per replayed step).  The steps issued
// eagerly before the capture use the same window, so that the capture finds every kernel it needs compiled.
struct WideWindow {
    DeviceHIP* dev;
    aixhip::fuse::FuseConfig kept;
    WideWindow(DeviceHIP* d, bool on) : dev(on ? d : nullptr)
    {
        if (!dev) return;
        kept = dev->fuseConfig();
        aixhip::fuse::FuseConfig wide = kept;
        wide.flushThreshold = std::max<size_t>(kept.flushThreshold, 3000);
        dev->setFuseConfig(wide);
    }
    ~WideWindow() { if (dev) { try { dev->setFuseConfig(kept); } catch (...) {} } }
};

// The whole training step -- zeroGrad, forward, loss, backward, Adam's update -- with Adam in its in-place form
// (frontend/nn.hpp) and, with capture_at >= 0, step `capture_at` captured into a HIP graph and that step and every later one
// enqueued by DeviceHIP::replay; capture_at < 0: every step issued eagerly (the run a captured one is compared with).
int aixbench_mlp_captured(aixhip_device* handle, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
                          int capture_at, const float* x, const float* y, const float* const* w, const float* const* b, float* losses,
                          double* step_seconds, uint64_t* graph_nodes)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        cfg.adamInPlace = 1;
        cfg.captureAt = capture_at;
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        DeviceHIP::StepGraph* graph = nullptr;
        const WideWindow window(dev, capture_at >= 0);
        aixfe::StepCapture capture;
        capture.begin = [&] { dev->beginCapture(); };
        capture.end = [&] { graph = dev->endCapture(); };
        capture.replay = [&] { dev->replay(graph); };
        try { aixfe::runMlp(dev, cfg, host, losses, step_seconds, nullptr, 0, capture_at >= 0 ? &capture : nullptr); }
        catch (...) { if (graph) dev->destroyGraph(graph); throw; }
        if (graph_nodes) *graph_nodes = graph ? dev->graphNodes(graph) : 0;
        if (graph) dev->destroyGraph(graph);
    });
}

// Config 4: decoder-only transformer forward + backward (frontend/transformer.hpp); params in the order of
// aixfe::transformerParamShapes; losses[steps], grad_norms[steps * param_count], step_seconds[steps] (may be NULL).
// stacked_attention = 0: one 2-D matmul per (sequence, head), the reference's interface as it is; 1: matmul on stacks.
int aixbench_transformer(aixhip_device* handle, uint64_t layers, uint64_t d_model, uint64_t heads, uint64_t seq, uint64_t batch,
                         uint64_t vocab, int steps, int stacked_attention, const int32_t* tokens, const float* const* params,
                         float* losses, float* grad_norms, double* step_seconds)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        const aixfe::TransformerConfig cfg{layers, d_model, heads, seq, batch, vocab, steps, stacked_attention};
        aixfe::runTransformer(dev, cfg, tokens, params, losses, grad_norms, step_seconds);
    });
}

// The same with step `capture_at` captured into a HIP graph (DeviceHIP::beginCapture / endCapture) and that step and every
// later one enqueued by DeviceHIP::replay: no front-end, no planner, one launch call per step.  The steps before it run
// as usual (they compile the kernels and grow the workspaces the captured step needs).  *graph_nodes (may be NULL): the
// number of nodes of the graph.
int aixbench_transformer_captured(aixhip_device* handle, uint64_t layers, uint64_t d_model, uint64_t heads, uint64_t seq, uint64_t batch,
                                  uint64_t vocab, int steps, int stacked_attention, int capture_at, const int32_t* tokens, const float* const* params,
                                  float* losses, float* grad_norms, double* step_seconds, uint64_t* graph_nodes)
{
    return guarded([&] {
        DeviceHIP* dev = aix::hip::fromHandle(handle);
        aixfe::TransformerConfig cfg{layers, d_model, heads, seq, batch, vocab, steps, stacked_attention};
        cfg.captureAt = capture_at;
        DeviceHIP::StepGraph* graph = nullptr;
        const WideWindow window(dev, capture_at >= 0);
        aixfe::StepCapture capture;
        capture.begin = [&] { dev->beginCapture(); };
        capture.end = [&] { graph = dev->endCapture(); };
        capture.replay = [&] { dev->replay(graph); };
        try { aixfe::runTransformer(dev, cfg, tokens, params, losses, grad_norms, step_seconds, &capture); }
        catch (...) { if (graph) dev->destroyGraph(graph); throw; }
        if (graph_nodes) *graph_nodes = graph ? dev->graphNodes(graph) : 0;
        if (graph) dev->destroyGraph(graph);
    });
}

} // extern "C"
