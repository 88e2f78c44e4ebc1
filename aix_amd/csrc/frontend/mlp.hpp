// mlp.hpp -- the MLP training loop of the benchmark's fourth configuration, written against
// aix::Device only, so the same code drives the GPU backend and a CPU device:
//   layers in -> hidden -> hidden -> out, ReLU after the first two, Softmax(1, keepDim) +
//   CrossEntropyLoss, Adam(lr); per step: zeroGrad, forward, loss, backward, step, read the loss
// (the loop of Targets/AIXExamples/*/Main.cpp: zeroGrad / forward / loss / backward / step).
#pragma once

#include "nn.hpp"

#include <chrono>
#include <cmath>
#include <stdexcept>

namespace aixfe {

struct MlpConfig {
    uint64_t batch, in, hidden, out;
    int32_t steps;
    float lr;
    int32_t singlePass;       // 0: the reference's path-by-path backward(); 1: Tensor::backwardOnce()
    int32_t adamInPlace{0};   // 1: Adam updates its state where it lies and keeps beta^t in device memory (nn.hpp)
    int32_t captureAt{-1};    // >= 0 (with adamInPlace and a StepCapture): that step is captured, it and every later one is a replay
};

inline bool stepIsCaptured(const StepCapture* capture, const MlpConfig& cfg, int s) { return capture && cfg.captureAt >= 0 && s >= cfg.captureAt; }

struct MlpHost {              // host arrays, f32, row-major
    const float* x;           // [batch, in]
    const float* y;           // [batch, out] one-hot
    const float* w[3];        // [in, hidden], [hidden, hidden], [hidden, out]
    const float* b[3];        // [1, hidden], [1, hidden], [1, out]
};

// Runs cfg.steps steps; losses[s] = loss of step s read after the step's synchronize();
// step_seconds[s] (may be null) = wall time of step s, synchronize to synchronize; grad_norms (may be null) =
// the L2 norms of the gradients of w1, b1, w2, b2, w3, b3 in the first grad_norm_steps steps, six per step, taken
// between backward and the optimizer's update (outside the step's time; steps issued eagerly only).
// With a StepCapture, step cfg.captureAt is captured and it and every later step is a replay of that capture: the whole
// training step -- zeroGrad, forward, loss, backward, Adam's update -- as one enqueue.
inline void runMlp(Device* dev, const MlpConfig& cfg, const MlpHost& h, float* losses, double* step_seconds, float* grad_norms = nullptr,
                   int grad_norm_steps = 0, const StepCapture* capture = nullptr)
{
    const Tensor x = Tensor::fromHost(dev, DataType::kFloat32, Shape{cfg.batch, cfg.in}, h.x);
    const Tensor y = Tensor::fromHost(dev, DataType::kFloat32, Shape{cfg.batch, cfg.out}, h.y);
    Linear l1(dev, cfg.in, cfg.hidden, h.w[0], h.b[0]);
    Linear l2(dev, cfg.hidden, cfg.hidden, h.w[1], h.b[1]);
    Linear l3(dev, cfg.hidden, cfg.out, h.w[2], h.b[2]);
    Adam opt({l1.w, l1.b, l2.w, l2.b, l3.w, l3.b}, cfg.lr, 0.9f, 0.999f, 1e-8f, cfg.adamInPlace != 0);
    const bool capturing = capture && cfg.captureAt >= 0;
    if (capturing && !cfg.adamInPlace) throw std::invalid_argument("runMlp: a captured step needs Adam's in-place form (its constants must not change from step to step)");
    dev->synchronize();
    Tensor loss;                                                  // the captured step's graph of nodes: its tensors are what a replay writes
    Value lossValue;                                              // of the last step issued
    double aside = 0;
    auto issueStep = [&](int s, bool keepGraph) {
        loss = Tensor();                                          // a graph that was kept goes first
        opt.zeroGrad();
        const Tensor logits = l3.forward(relu(l2.forward(relu(l1.forward(x)))));
        loss = crossEntropy(softmax(logits, 1, true), y);
        if (cfg.singlePass) loss.backwardOnce(); else loss.backward();
        if (grad_norms && s < grad_norm_steps && !stepIsCaptured(capture, cfg, s)) {
            const auto n0 = std::chrono::steady_clock::now();
            const Tensor* params[6] = {&l1.w, &l1.b, &l2.w, &l2.b, &l3.w, &l3.b};
            for (int p = 0; p < 6; ++p) grad_norms[s * 6 + p] = params[p]->grad().l2Norm();
            aside = std::chrono::duration<double>(std::chrono::steady_clock::now() - n0).count();
        }
        opt.step();
        lossValue = loss.value();
        if (!keepGraph) loss = Tensor();                          // an eager step lets go of its graph while the GPU still works through the step (see runTransformer)
    };
    for (int s = 0; s < cfg.steps; ++s) {
        const auto t0 = std::chrono::steady_clock::now();
        aside = 0;
        const bool captured = capturing && s >= cfg.captureAt;
        if (captured && s == cfg.captureAt) { capture->begin(); issueStep(s, true); capture->end(); }
        if (captured) capture->replay(); else issueStep(s, false);
        losses[s] = lossValue.item();             // synchronizes
        if (step_seconds) step_seconds[s] = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() - aside;
    }
}

} // namespace aixfe
