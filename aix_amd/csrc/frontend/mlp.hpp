// mlp.hpp -- the MLP training loop of the benchmark's fourth configuration, written against
// aix::Device only, so the same code drives the GPU backend and a CPU device:
//   layers in -> hidden -> hidden -> out, ReLU after the first two, Softmax(1, keepDim) +
//   CrossEntropyLoss, Adam(lr); per step: zeroGrad, forward, loss, backward, step, read the loss
// (the loop of Targets/AIXExamples/*/Main.cpp: zeroGrad / forward / loss / backward / step).
#pragma once

#include "nn.hpp"

#include <chrono>
#include <cmath>

namespace aixfe {

struct MlpConfig {
    uint64_t batch, in, hidden, out;
    int32_t steps;
    float lr;
    int32_t singlePass;       // 0: the reference's path-by-path backward(); 1: Tensor::backwardOnce()
};

struct MlpHost {              // host arrays, f32, row-major
    const float* x;           // [batch, in]
    const float* y;           // [batch, out] one-hot
    const float* w[3];        // [in, hidden], [hidden, hidden], [hidden, out]
    const float* b[3];        // [1, hidden], [1, hidden], [1, out]
};

// Runs cfg.steps steps; losses[s] = loss of step s read after the step's synchronize();
// step_seconds[s] (may be null) = wall time of step s, synchronize to synchronize; grad_norms (may be null) =
// the L2 norms of the gradients of w1, b1, w2, b2, w3, b3 in the first grad_norm_steps steps, six per step, taken
// between backward and the optimizer's update (outside the step's time).
inline void runMlp(Device* dev, const MlpConfig& cfg, const MlpHost& h, float* losses, double* step_seconds, float* grad_norms = nullptr,
                   int grad_norm_steps = 0)
{
    const Tensor x = Tensor::fromHost(dev, DataType::kFloat32, Shape{cfg.batch, cfg.in}, h.x);
    const Tensor y = Tensor::fromHost(dev, DataType::kFloat32, Shape{cfg.batch, cfg.out}, h.y);
    Linear l1(dev, cfg.in, cfg.hidden, h.w[0], h.b[0]);
    Linear l2(dev, cfg.hidden, cfg.hidden, h.w[1], h.b[1]);
    Linear l3(dev, cfg.hidden, cfg.out, h.w[2], h.b[2]);
    Adam opt({l1.w, l1.b, l2.w, l2.b, l3.w, l3.b}, cfg.lr);
    dev->synchronize();
    for (int s = 0; s < cfg.steps; ++s) {
        const auto t0 = std::chrono::steady_clock::now();
        opt.zeroGrad();
        const Tensor logits = l3.forward(relu(l2.forward(relu(l1.forward(x)))));
        const Tensor loss = crossEntropy(softmax(logits, 1, true), y);
        if (cfg.singlePass) loss.backwardOnce(); else loss.backward();
        double aside = 0;
        if (grad_norms && s < grad_norm_steps) {
            const auto n0 = std::chrono::steady_clock::now();
            const Tensor* params[6] = {&l1.w, &l1.b, &l2.w, &l2.b, &l3.w, &l3.b};
            for (int p = 0; p < 6; ++p) grad_norms[s * 6 + p] = params[p]->grad().l2Norm();
            aside = std::chrono::duration<double>(std::chrono::steady_clock::now() - n0).count();
        }
        opt.step();
        losses[s] = loss.value().item();          // synchronizes
        if (step_seconds) step_seconds[s] = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() - aside;
    }
}

} // namespace aixfe
