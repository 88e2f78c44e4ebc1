// transformer.hpp -- forward + backward of a decoder-only transformer composed from aix::Device
// operators only (the benchmark's fifth configuration): token + position embeddings by
// indexSelect, pre-LayerNorm blocks (LayerNorm from mean / var, statistics in f32), causal
// self-attention as loops of 2-D matmuls per (batch, head) with a tril mask and the reference's
// Softmax, GELU MLP (the reference's GeLU formula, aixNeuralNetwork.hpp:200-208), final LayerNorm,
// an output projection and the reference's CrossEntropyLoss on f32 logits.  Parameters are f32
// masters that require gradients; every step casts them to bf16 (to() is differentiable), all
// activations are bf16.
//
// Differentiation uses Tensor::backwardOnce(): the reference's path-by-path recursion is
// exponential in the number of residual branches (2 per block) and cannot run this model.
//
// The interface has no batch dimension, so attention is issued the way an AIX program has to issue
// it: projections as one [tokens, d] matmul each, then row slices per sequence and column slices
// per head (views), 2-D matmuls on those, cat() to put heads and sequences back together.
//
// stackedAttention = 1 uses what this device adds to the interface, matmul on stacks of matrices:
// q, k, v are seen as [batch, heads, seq, d / heads] views (reshape + transpose, no copy), the
// scores of all sequences and heads are one [batch, heads, seq, seq] tensor, and mask, softmax and
// the product with v are one operator each over it.  The arithmetic per element is the same.
#pragma once
#include <functional>

#include "nn.hpp"

#include <chrono>
#include <cmath>

namespace aixfe {

struct TransformerConfig {
    uint64_t layers, dModel, heads, seq, batch, vocab;
    int32_t steps;
    int32_t stackedAttention{0};
    int32_t captureAt{-1};        // >= 0 (and a StepCapture given): that step is captured, it and every later one is a replay
};


// Parameter order (all f32, row-major):
//   wte [vocab, d], wpe [seq, d],
//   per layer: ln1_g [1,d], ln1_b [1,d], wq [d,d], bq [1,d], wk, bk, wv, bv, wo [d,d], bo [1,d],
//              ln2_g, ln2_b, w1 [d,4d], b1 [1,4d], w2 [4d,d], b2 [1,d],
//   lnf_g [1,d], lnf_b [1,d], lm_head [d, vocab]
inline std::vector<Shape> transformerParamShapes(const TransformerConfig& c)
{
    const uint64_t d = c.dModel;
    std::vector<Shape> s{{c.vocab, d}, {c.seq, d}};
    for (uint64_t l = 0; l < c.layers; ++l) {
        const Shape block[] = {{1, d}, {1, d}, {d, d}, {1, d}, {d, d}, {1, d}, {d, d}, {1, d}, {d, d}, {1, d},
                               {1, d}, {1, d}, {d, 4 * d}, {1, 4 * d}, {4 * d, d}, {1, d}};
        s.insert(s.end(), std::begin(block), std::end(block));
    }
    s.push_back({1, d}); s.push_back({1, d}); s.push_back({d, c.vocab});
    return s;
}

inline Tensor layerNorm(const Tensor& x, const Tensor& gamma, const Tensor& beta)
{
    const Tensor xf = x.to(DataType::kFloat32);
    const Tensor centered = xf - xf.mean(1, true);
    const Tensor variance = xf.var(1, false, true);
    return (centered / (variance + 1e-5f).sqrt() * gamma + beta).to(x.dtype());
}

// aixNeuralNetwork.hpp:200-208
inline Tensor gelu(const Tensor& x)
{
    return 0.5f * x * (1.0f + tanh(float(std::sqrt(2.0 / 3.14159265358979323846)) * (x + 0.044715f * x.pow(3.0f))));
}

// losses[s], gradNorms[s * P + p] (L2 norm of parameter p's gradient after step s), step_seconds[s] (may be null).
// tokens: int32 [batch * seq]; params: host arrays in the order above.
inline void runTransformer(Device* dev, const TransformerConfig& c, const int32_t* tokens, const float* const* params,
                           float* losses, float* gradNorms, double* step_seconds, const StepCapture* capture = nullptr)
{
    const DataType F32 = DataType::kFloat32, BF16 = DataType::kBFloat16, I32 = DataType::kInt32;
    const uint64_t T = c.batch * c.seq, d = c.dModel, dh = d / c.heads;
    const auto shapes = transformerParamShapes(c);
    std::vector<Tensor> P;
    for (size_t i = 0; i < shapes.size(); ++i) P.push_back(Tensor::fromHost(dev, F32, shapes[i], params[i], true));

    const Value tok = Value::fromHost(dev, I32, Shape{T}, tokens);
    std::vector<int32_t> posHost(T);
    for (uint64_t i = 0; i < T; ++i) posHost[i] = (int32_t)(i % c.seq);
    const Value pos = Value::fromHost(dev, I32, Shape{T}, posHost.data());
    // one-hot targets: next token within the sequence (the last position predicts the first token)
    std::vector<float> onehot(T * c.vocab, 0.0f);
    for (uint64_t b = 0; b < c.batch; ++b)
        for (uint64_t s = 0; s < c.seq; ++s) onehot[(b * c.seq + s) * c.vocab + (uint64_t)tokens[b * c.seq + (s + 1) % c.seq]] = 1.0f;
    const Tensor target = Tensor::fromHost(dev, F32, Shape{T, c.vocab}, onehot.data());
    onehot.clear(); onehot.shrink_to_fit();
    // additive causal mask: 0 on and below the diagonal, -30000 above (exp underflows to 0 in bf16 and f32)
    std::vector<float> maskHost(c.seq * c.seq);
    for (uint64_t i = 0; i < c.seq; ++i) for (uint64_t j = 0; j < c.seq; ++j) maskHost[i * c.seq + j] = j > i ? -30000.0f : 0.0f;
    const Tensor mask = Tensor(Value::fromHost(dev, F32, Shape{c.seq, c.seq}, maskHost.data()).to(BF16));
    const float scale = 1.0f / std::sqrt((float)dh);
    dev->synchronize();

    Tensor loss;                                                 // the captured step's graph of nodes: its tensors are what a replay writes
    Value lossValue;                                             // of the last step issued
    auto issueStep = [&](bool keepGraph) {
        loss = Tensor();                                         // a graph that was kept goes first
        for (auto& p : P) p.zeroGrad();
        std::vector<Tensor> W;                                   // bf16 working copies
        for (auto& p : P) W.push_back(p.to(BF16));
        size_t at = 0;
        Tensor x = W[0].indexSelect(0, tok) + W[1].indexSelect(0, pos);
        at = 2;
        for (uint64_t l = 0; l < c.layers; ++l, at += 16) {
            const Tensor h = layerNorm(x, P[at + 0], P[at + 1]);
            const Tensor q = matmul(h, W[at + 2]) + W[at + 3];
            const Tensor k = matmul(h, W[at + 4]) + W[at + 5];
            const Tensor v = matmul(h, W[at + 6]) + W[at + 7];
            Tensor attn;
            if (c.stackedAttention) {
                const Shape split{c.batch, c.seq, c.heads, dh};
                const Tensor q4 = q.reshape(split).transpose(1, 2), k4 = k.reshape(split).transpose(1, 2), v4 = v.reshape(split).transpose(1, 2);
                const Tensor scores = matmul(q4, k4.transpose(2, 3)).tril() * scale + mask;         // [batch, heads, seq, seq]; scale and mask fuse
                attn = matmul(softmax(scores, 3, true), v4).transpose(1, 2).reshape(Shape{T, d});
            } else {
                // One 2-D product per (sequence, head), as the interface has it, written stage by stage -- all score products,
                // then every head's mask and softmax, then all mixing products -- so that a device that batches runs of
                // equal-shaped matmul calls finds such runs (the arithmetic per head is the same in any order).
                const uint64_t pairs = c.batch * c.heads;
                std::vector<Tensor> qh(pairs), kh(pairs), vh(pairs), raw(pairs), prob(pairs), mixed(pairs);
                for (uint64_t b = 0; b < c.batch; ++b) {
                    const Tensor qb = q.slice(0, b * c.seq, (b + 1) * c.seq), kb = k.slice(0, b * c.seq, (b + 1) * c.seq),
                                 vb = v.slice(0, b * c.seq, (b + 1) * c.seq);
                    for (uint64_t hd = 0; hd < c.heads; ++hd) {
                        const uint64_t i = b * c.heads + hd;
                        qh[i] = qb.slice(1, hd * dh, (hd + 1) * dh); kh[i] = kb.slice(1, hd * dh, (hd + 1) * dh); vh[i] = vb.slice(1, hd * dh, (hd + 1) * dh);
                    }
                }
                for (uint64_t i = 0; i < pairs; ++i) raw[i] = matmul(qh[i], kh[i].transpose(0, 1));
                for (uint64_t i = 0; i < pairs; ++i) prob[i] = softmax(raw[i].tril() * scale + mask, 1, true);
                for (uint64_t i = 0; i < pairs; ++i) mixed[i] = matmul(prob[i], vh[i]);
                std::vector<Tensor> sequences;
                for (uint64_t b = 0; b < c.batch; ++b)
                    sequences.push_back(Tensor::cat(std::vector<Tensor>(mixed.begin() + (long)(b * c.heads), mixed.begin() + (long)((b + 1) * c.heads)), 1));
                attn = Tensor::cat(sequences, 0);
            }
            x = x + (matmul(attn, W[at + 8]) + W[at + 9]);
            const Tensor h2 = layerNorm(x, P[at + 10], P[at + 11]);
            x = x + (matmul(gelu(matmul(h2, W[at + 12]) + W[at + 13]), W[at + 14]) + W[at + 15]);
        }
        const Tensor xf = layerNorm(x, P[at], P[at + 1]);
        const Tensor logits = matmul(xf, W[at + 2]).to(F32);
        loss = crossEntropy(softmax(logits, 1, true), target);
        loss.backwardOnce();
        lossValue = loss.value();
        // An eager step lets go of its graph here, before the loss is read: the host takes the nodes and their intermediate
        // results apart while the GPU still works through the step (the device keeps a freed block until the work enqueued
        // on it has passed), instead of opening the next step with it while the GPU idles; and results that only the graph
        // held and nothing recorded reads any more are never stored.
        if (!keepGraph) loss = Tensor();
    };
    for (int step = 0; step < c.steps; ++step) {
        const auto t0 = std::chrono::steady_clock::now();
        const bool captured = capture && c.captureAt >= 0 && step >= c.captureAt;
        if (captured && step == c.captureAt) { capture->begin(); issueStep(true); capture->end(); }
        if (captured) capture->replay(); else issueStep(false);
        losses[step] = lossValue.item();                         // synchronizes: forward and backward have run
        if (step_seconds) step_seconds[step] = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        for (size_t i = 0; i < P.size(); ++i) {
            gradNorms[(size_t)step * P.size() + i] = P[i].grad().l2Norm();
        }
    }
}

} // namespace aixfe
