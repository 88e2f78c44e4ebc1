// nn.hpp -- the few network and optimizer pieces the training drivers use, composed from
// aixfe::Tensor operators the way the reference composes them:
//   Linear            matmul(x, w) + b, b of shape [1, out]       (aixNeuralNetwork.hpp:133-157)
//   Softmax           (x - max(x)).exp() / sum                     (aixNeuralNetwork.hpp:182-197)
//   CrossEntropyLoss  -mean(targets * log(predictions))            (aixNeuralNetwork.hpp:246-254)
//   Adam, SGD                                                       (aixOptimizer.hpp:70-159)
// The reference has no ReLU; relu() below builds it from its cat() and max(dim):
// max over a leading axis of the pair {x, 0}.
#pragma once

#include <functional>

#include "autograd.hpp"

#include <cmath>

namespace aixfe {

struct Linear {
    Tensor w, b;
    Linear() = default;
    // Parameters come from the host so that every device starts from the same numbers.
    Linear(Device* dev, size_t in, size_t out, const float* hostW, const float* hostB)
        : w(Tensor::fromHost(dev, DataType::kFloat32, Shape{in, out}, hostW, true)),
          b(Tensor::fromHost(dev, DataType::kFloat32, Shape{1, out}, hostB, true)) {}
    Tensor forward(const Tensor& x) const { return matmul(x, w) + b; }
};

inline Tensor relu(const Tensor& x)
{
    Shape lifted = x.shape();
    lifted.insert(lifted.begin(), 1);
    const Tensor zeros(0.0f, lifted, x.device(), x.dtype());
    return Tensor::cat({x.unsqueeze(0), zeros}, 0).max(0);
}

inline Tensor softmax(Tensor x, size_t dim, bool keepDim)
{
    x = (x - x.max(dim, keepDim)).exp();
    return x / x.sum(dim, keepDim);
}

inline Tensor crossEntropy(const Tensor& predictions, const Tensor& targets)
{
    return -mean(targets * log(predictions));
}

class SGD {
public:
    SGD(std::vector<Tensor> params, float lr) : m_params(std::move(params)), m_lr(lr) {}
    void zeroGrad() { for (auto& p : m_params) p.zeroGrad(); }
    void step()
    {
        for (auto& p : m_params)
            if (p.isRequireGrad()) p.value() -= p.grad().withScalar(&Device::mul, m_lr);
    }
private:
    std::vector<Tensor> m_params;
    float m_lr;
};

// aixOptimizer.hpp:93-159.  All arithmetic is on values (no autograd); `value op scalar` is the
// value-level form (full-shape fill + binary operator).
// How a device captures a step and enqueues it again (a HIP graph on the GPU backend); none on a device without it.
struct StepCapture {
    std::function<void()> begin, end, replay;
};

// Adam (aixOptimizer.hpp:112-140).  Two forms of the same update:
//  * as the reference writes it: m and v are new tensors every step and the bias corrections 1 - beta^t are scalars the
//    host computes, so every step issues different constants;
//  * inPlace: m and v are updated where they lie and beta^t lives in device memory (a rank-0 tensor multiplied by beta
//    every step), so a step is the same device calls on the same addresses every time -- what a captured step needs
//    (StepCapture).  The arithmetic per element is the same; beta^t is a running f32 product instead of a rounded
//    double power, which moves the corrections by an ulp or two.
class Adam {
public:
    Adam(std::vector<Tensor> params, float lr = 0.001f, float beta1 = 0.9f, float beta2 = 0.999f, float eps = 1e-8f, bool inPlace = false)
        : m_params(std::move(params)), m_lr(lr), m_beta1(beta1), m_beta2(beta2), m_eps(eps), m_inPlace(inPlace)
    {
        for (auto& p : m_params) {
            m_m.push_back(Value::full(p.device(), DataType::kFloat32, p.shape(), 0.0f));
            m_v.push_back(Value::full(p.device(), DataType::kFloat32, p.shape(), 0.0f));
        }
        if (m_inPlace && !m_params.empty()) {
            m_b1t = Value::full(m_params[0].device(), DataType::kFloat32, Shape{}, 1.0f);
            m_b2t = Value::full(m_params[0].device(), DataType::kFloat32, Shape{}, 1.0f);
        }
    }

    void zeroGrad() { for (auto& p : m_params) p.zeroGrad(); }

    void step()
    {
        ++m_t;
        if (m_inPlace) return stepInPlace();
        for (size_t i = 0; i < m_params.size(); ++i) {
            Tensor& p = m_params[i];
            if (!p.isRequireGrad()) continue;
            const Value g = p.grad().to(DataType::kFloat32);
            m_m[i] = m_m[i].withScalar(&Device::mul, m_beta1, true) + g.withScalar(&Device::mul, float(1.0 - m_beta1), true);
            m_v[i] = m_v[i].withScalar(&Device::mul, m_beta2, true) + g.withScalar(&Device::mul, float(1.0 - m_beta2), true) * g;
            const Value mHat = m_m[i].withScalar(&Device::div, float(1.0 - std::pow(m_beta1, m_t)));
            const Value vHat = m_v[i].withScalar(&Device::div, float(1.0 - std::pow(m_beta2, m_t)));
            p.value() -= (mHat.withScalar(&Device::mul, m_lr, true) / vHat.sqrt().withScalar(&Device::add, m_eps)).to(p.dtype());
        }
    }

private:
    void stepInPlace()
    {
        if (m_params.empty()) return;
        Device* dev = m_params[0].device();
        m_b1t *= Value::full(dev, DataType::kFloat32, Shape{}, m_beta1);
        m_b2t *= Value::full(dev, DataType::kFloat32, Shape{}, m_beta2);
        const Value c1 = 1.0f - m_b1t, c2 = 1.0f - m_b2t;                       // rank-0, read by every parameter's update
        for (size_t i = 0; i < m_params.size(); ++i) {
            Tensor& p = m_params[i];
            if (!p.isRequireGrad()) continue;
            const Value g = p.grad().to(DataType::kFloat32);
            m_m[i] *= Value::full(dev, DataType::kFloat32, p.shape(), m_beta1);
            m_m[i] += g.withScalar(&Device::mul, float(1.0 - m_beta1), true);
            m_v[i] *= Value::full(dev, DataType::kFloat32, p.shape(), m_beta2);
            m_v[i] += g.withScalar(&Device::mul, float(1.0 - m_beta2), true) * g;
            const Value mHat = m_m[i] / c1, vHat = m_v[i] / c2;
            p.value() -= (mHat.withScalar(&Device::mul, m_lr, true) / vHat.sqrt().withScalar(&Device::add, m_eps)).to(p.dtype());
        }
    }

    std::vector<Tensor> m_params;
    float m_lr, m_beta1, m_beta2, m_eps;
    bool m_inPlace;
    size_t m_t{0};
    std::vector<Value> m_m, m_v;
    Value m_b1t, m_b2t;
};

} // namespace aixfe
