// autograd.hpp -- reverse-mode differentiation over aixfe::Value, generating the op stream the
// reference's autograd generates (Targets/AIXLib/aixCore.hpp:1790-1857, 2014-2309).
//
// What a device sees during backward() depends on how the caller differentiates, so this mirrors
// the reference's scheme rather than a textbook tape:
//   * every result is a node holding its value, its input nodes and one backward function;
//   * backward(seed) on a node calls that function at once, which computes the seeds of the inputs
//     with ordinary Value operators and RECURSES into them -- no topological ordering and no
//     accumulation at interior nodes, so a node reachable along p paths is differentiated p times
//     (softmax + cross-entropy reaches the logits along 4 paths; everything below them runs 4x);
//   * leaves add the seed into their gradient buffer (grad += seed);
//   * binary operators first bring both operands to the common shape with broadcastTo(), which
//     is itself a node whose backward is reduceTo() of the seed;
//   * `tensor op scalar` wraps the scalar in a rank-0 tensor and broadcasts it (:2384-2438).
//   * a node's value is kept for as long as somebody can still read it: a Tensor handle, the node's own backward
//     formula (exp, tanh, sqrt) or a consumer's (mul, div, pow, log, max, matmul read their operands).  Once the last
//     handle is gone and no formula reads it, the storage is released and only shape and type stay -- the sum of a
//     residual branch, a masked score tensor, the pieces of a LayerNorm need not stay in memory (or be written to it at
//     all: a fused kernel stores only what is alive).  The reference keeps every intermediate value alive until the
//     graph dies (aixCore.hpp:1790-1857); the operators issued and their results are the same.
// Only the operators the training drivers need are present.
#pragma once

#include "value.hpp"

#include <algorithm>
#include <atomic>
#include <functional>
#include <unordered_set>
#include <utility>

namespace aixfe {

struct Node;
using NodePtr = std::shared_ptr<Node>;

// aixCore.hpp:1790-1857
struct Node {
    Value value;
    bool requireGrad{false};
    bool retainGrad{false};
    bool isLeaf{true};
    std::vector<NodePtr> inputs;
    size_t dim0{0}, dim1{0}, start{0}, end{0};
    ssize_t diagonal{0};
    bool keepDim{false};
    Value indices;
    std::function<void(Node*, const Value&)> backwardFn;
    int handles{0};                                 // Tensor objects that name this node
    int readers{0};                                 // backward formulas (its own, its consumers') that read `value`
    uint64_t serial{nextSerial()};                  // creation order: a node is always younger than its inputs
    uint64_t visited{0};                            // the last single-pass traversal that reached this node

    Node(Value v, bool req) : value(std::move(v)), requireGrad(req) {}

    void backward(const Value& seed)
    {
        if (accumulating()) {                       // single-pass mode: gather the seed, the driver calls backwardFn once
            pending = pending.defined() ? pending + seed : seed;
            return;
        }
        if (retainGrad) grad() += seed;
        if (requireGrad || retainGrad) backwardFn(this, seed);
    }

    // The seed of a slice of this node: `seed` in the window, zero elsewhere (aixCore.hpp:2228-2233).  Single-pass mode
    // only notes the window; takeSeed() puts all of them together.
    void backwardWindow(const Value& seed, size_t dim, size_t from, size_t to, size_t step)
    {
        if (accumulating()) { windows.push_back({seed, dim, from, to, step}); return; }
        backward(value.sliceSet(seed, dim, from, to, step));
    }

    // Single-pass mode: the sum of everything that reached this node, which then holds nothing.  Windows that do not
    // overlap -- the per-head slices of a projection, the parts a cat() was made of -- are written into ONE tensor of
    // zeros, a sliceSet of the window's size each; a sum of zero-padded tensors, one per window, holds the same numbers.
    Value takeSeed()
    {
        Value seed = std::move(pending);
        pending = Value();
        if (windows.empty()) return seed;
        std::vector<Window> w = std::move(windows);
        windows.clear();
        bool apart = !seed.defined();
        for (size_t k = 0; apart && k < w.size(); ++k) {
            apart = w[k].dim == w[0].dim && w[k].step == 1;
            for (size_t j = 0; apart && j < k; ++j) apart = w[k].to <= w[j].from || w[j].to <= w[k].from;
        }
        if (apart) {
            size_t covered = 0;
            for (const auto& x : w) covered += x.to - x.from;
            // windows that leave nothing out (every head of a projection was used): no zeros to start from
            seed = covered == value.shape()[w[0].dim] ? Value(value.device(), value.dtype(), value.shape())
                                                      : Value::full(value.device(), value.dtype(), value.shape(), 0.0f);
            for (const auto& x : w) seed.sliceSetInPlace(x.seed, x.dim, x.from, x.to, x.step);
            return seed;
        }
        for (const auto& x : w) {
            const Value padded = value.sliceSet(x.seed, x.dim, x.from, x.to, x.step);
            seed = seed.defined() ? seed + padded : padded;
        }
        return seed;
    }

    static bool& accumulating() { static thread_local bool on = false; return on; }
    static uint64_t nextSerial() { static std::atomic<uint64_t> n{0}; return ++n; }
    Value pending;                                  // sum of the seeds received so far (single-pass mode)
    struct Window { Value seed; size_t dim, from, to, step; };
    std::vector<Window> windows;                    // seeds of slices of this node, not yet part of `pending`

    Value& grad()
    {
        if (!m_grad.defined()) {
            m_grad = Value(value.device(), value.dtype(), value.shape());
            m_grad.fill(0.0f);
        }
        return m_grad;
    }

    // readsInputs: bit k set = the formula reads inputs[k]->value; readsOwn: it reads this node's value
    void setBackward(std::vector<NodePtr> in, std::function<void(Node*, const Value&)> fn, unsigned readsInputs = 0, bool readsOwn = false)
    {
        if (requireGrad || retainGrad) {
            inputs = std::move(in); backwardFn = std::move(fn);
            for (size_t k = 0; k < inputs.size(); ++k) if ((readsInputs >> k) & 1u) ++inputs[k]->readers;
            if (readsOwn) ++readers;
        }
    }

    // The last handle is gone: nobody but a backward formula can read the value any more.
    void handleReleased()
    {
        if (--handles == 0 && readers == 0 && !retainGrad && !(isLeaf && requireGrad)) value.releaseStorage();
    }

private:
    Value m_grad;
};

class Tensor {
public:
    Tensor() = default;
    Tensor(const Tensor& o) : m_node(o.m_node) { if (m_node) ++m_node->handles; }
    Tensor(Tensor&& o) noexcept : m_node(std::move(o.m_node)) { o.m_node.reset(); }
    Tensor& operator=(const Tensor& o)
    {
        if (this != &o && m_node != o.m_node) { drop(); m_node = o.m_node; if (m_node) ++m_node->handles; }
        return *this;
    }
    Tensor& operator=(Tensor&& o) noexcept
    {
        if (this != &o) { drop(); m_node = std::move(o.m_node); o.m_node.reset(); }
        return *this;
    }
    ~Tensor() { drop(); }

    // Leaf from an existing value.
    explicit Tensor(Value v, bool requireGrad = false) : m_node(std::make_shared<Node>(std::move(v), requireGrad))
    {
        m_node->backwardFn = defaultBackward;
        m_node->handles = 1;
    }

    // Leaf filled with one number (aixCore.hpp:1907-1913).
    Tensor(float v, const Shape& shape, Device* dev, DataType dt = DataType::kFloat32, bool requireGrad = false)
        : Tensor(Value::full(dev, dt, shape, v), requireGrad) {}

    static Tensor fromHost(Device* dev, DataType dt, const Shape& shape, const void* host, bool requireGrad = false)
    {
        return Tensor(Value::fromHost(dev, dt, shape, host), requireGrad);
    }

    const Value& value() const { return m_node->value; }
    Value& value() { return m_node->value; }
    Value& grad() const { return m_node->grad(); }
    const Shape& shape() const { return m_node->value.shape(); }
    DataType dtype() const { return m_node->value.dtype(); }
    Device* device() const { return m_node->value.device(); }
    bool isRequireGrad() const { return m_node->requireGrad; }
    void zeroGrad() const { m_node->grad().fill(0.0f); }
    const NodePtr& node() const { return m_node; }

    // aixCore.hpp:1923-1933: seed of ones.
    void backward() const
    {
        if (value().size() != 1) throw std::invalid_argument("backward() requires a one-element tensor");
        m_node->backward(Value::full(device(), dtype(), shape(), 1.0f));
    }

    // Single-pass differentiation: nodes are visited youngest first -- the reverse of the order the program created
    // them in, which is a reverse topological order -- and each one is differentiated ONCE with the sum of the seeds
    // that reached it.  A program written stage by stage (all heads' score products, then all their softmaxes, ...) is
    // differentiated stage by stage too, so a device that batches runs of equal calls finds the same runs in the
    // backward pass.  The reference has no such mode (its recursion revisits a node once per path, which is
    // exponential in the number of residual branches of a transformer); the backward formulas are the same ones,
    // only the traversal differs.
    void backwardOnce() const
    {
        if (value().size() != 1) throw std::invalid_argument("backward() requires a one-element tensor");
        // everything the result depends on, marked with this pass's number as it is found
        static thread_local uint64_t pass = 0;
        ++pass;
        std::vector<std::pair<uint64_t, Node*>> order{{0, m_node.get()}};
        m_node->visited = pass;
        for (size_t k = 0; k < order.size(); ++k)
            for (const auto& in : order[k].second->inputs)
                if (in->visited != pass) { in->visited = pass; order.push_back({0, in.get()}); }
        // youngest first; the leaves last of all: nothing waits for them, and a scalar constant's "grad += seed", issued
        // where the constant was created -- in the middle of a formula -- would make the kernel that forms the seed stop there
        for (auto& entry : order) entry.first = (entry.second->inputs.empty() ? 0 : uint64_t(1) << 63) | entry.second->serial;
        std::sort(order.begin(), order.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
        Node::accumulating() = true;
        try {
            m_node->pending = Value::full(device(), dtype(), shape(), 1.0f);
            for (const auto& entry : order) {
                Node* n = entry.second;
                if (!n->pending.defined() && n->windows.empty()) continue;
                const Value seed = n->takeSeed();
                if (n->retainGrad) n->grad() += seed;
                if (n->requireGrad || n->retainGrad) n->backwardFn(n, seed);
            }
        } catch (...) { Node::accumulating() = false; throw; }
        Node::accumulating() = false;
    }

    // ---- shape ------------------------------------------------------------------------------
    // aixCore.hpp:1973-1978
    Tensor reshape(const Shape& s) const
    {
        Tensor r = makeResult(value().reshape(s), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.reshape(n->inputs[0]->value.shape()));
        });
        return r;
    }

    // aixCore.hpp:2004-2010; backward casts the seed back (:2052-2057)
    Tensor to(DataType dt) const
    {
        if (dtype() == dt) return *this;
        Tensor r = makeResult(value().to(dt), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.to(n->inputs[0]->value.dtype()));
        });
        return r;
    }

    // aixCore.hpp:2597-2608; backward scatters the seed into zeros (:2228-2233)
    Tensor slice(size_t dim, size_t start, size_t end, size_t step = 1) const
    {
        Tensor r = makeResult(value().slice(dim, start, end, step), isRequireGrad());
        r.m_node->dim0 = dim; r.m_node->dim1 = step; r.m_node->start = start; r.m_node->end = end;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backwardWindow(seed, n->dim0, n->start, n->end, n->dim1);
        });
        return r;
    }

    // aixCore.hpp:2664-2670
    Tensor tril(ssize_t diagonal = 0) const
    {
        Tensor r = makeResult(value().tril(diagonal), isRequireGrad());
        r.m_node->diagonal = diagonal;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.tril(n->diagonal));
        });
        return r;
    }

    // aixCore.hpp:2680-2700; backward adds the seed's rows into zeros (:2284-2290)
    Tensor indexSelect(size_t dim, const Value& indices) const
    {
        Tensor r = makeResult(value().indexSelect(dim, indices), isRequireGrad(), !m_node->isLeaf);
        r.m_node->dim0 = dim; r.m_node->indices = indices;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            const Value zeros = Value::full(seed.device(), seed.dtype(), n->inputs[0]->value.shape(), 0.0f);
            zeros.indexAddInPlace(n->dim0, n->indices, seed);
            n->inputs[0]->backward(zeros);
        });
        return r;
    }

    Tensor broadcastTo(const Shape& s) const
    {
        if (shape() == s) return *this;
        Tensor r = makeResult(value().broadcastTo(s), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.reduceTo(n->inputs[0]->value.shape()));
        });
        return r;
    }

    Tensor transpose(size_t d0, size_t d1) const
    {
        Tensor r = makeResult(value().transpose(d0, d1), isRequireGrad());
        r.m_node->dim0 = d0; r.m_node->dim1 = d1;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.transpose(n->dim0, n->dim1));
        });
        return r;
    }

    Tensor unsqueeze(size_t dim) const
    {
        Tensor r = makeResult(value().unsqueeze(dim), isRequireGrad());
        r.m_node->dim0 = dim;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.squeeze(n->dim0));
        });
        return r;
    }

    Tensor squeeze(size_t dim) const
    {
        Tensor r = makeResult(value().squeeze(dim), isRequireGrad());
        r.m_node->dim0 = dim;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.unsqueeze(n->dim0));
        });
        return r;
    }

    // aixCore.hpp:2702-2779; catBackwardFunc :2292-2309
    static Tensor cat(const std::vector<Tensor>& parts, size_t dim)
    {
        if (parts.empty()) throw std::invalid_argument("cat: no tensors");
        if (parts.size() == 1) return parts[0];
        bool anyGrad = false, anyNonLeaf = false;
        std::vector<Value> values;
        std::vector<NodePtr> inputs;
        for (const auto& p : parts) {
            anyGrad |= p.isRequireGrad(); anyNonLeaf |= !p.m_node->isLeaf;
            values.push_back(p.value()); inputs.push_back(p.m_node);
        }
        Tensor r = makeResult(Value::cat(values, dim), anyGrad, anyNonLeaf);
        r.m_node->dim0 = dim;
        r.m_node->setBackward(std::move(inputs), [](Node* n, const Value& seed) {
            size_t at = 0;
            for (auto& in : n->inputs) {
                const size_t ext = in->value.shape()[n->dim0];
                if (in->requireGrad || in->retainGrad) in->backward(seed.slice(n->dim0, at, at + ext, 1));
                at += ext;
            }
        });
        return r;
    }

    // ---- arithmetic (aixCore.hpp:2317-2438) -----------------------------------------------------
    Tensor operator+(const Tensor& o) const
    {
        return binary(o, [](const Value& a, const Value& b) { return a + b; }, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2) return;
            if (n->inputs[0] == n->inputs[1]) { n->inputs[0]->backward(seed + seed); return; }
            if (wants(n->inputs[0])) n->inputs[0]->backward(seed);
            if (wants(n->inputs[1])) n->inputs[1]->backward(seed);
        });
    }

    Tensor operator-(const Tensor& o) const
    {
        return binary(o, [](const Value& a, const Value& b) { return a - b; }, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2 || n->inputs[0] == n->inputs[1]) return;
            if (wants(n->inputs[0])) n->inputs[0]->backward(seed);
            if (wants(n->inputs[1])) n->inputs[1]->backward(-seed);
        });
    }

    Tensor operator*(const Tensor& o) const
    {
        return binary(o, [](const Value& a, const Value& b) { return a * b; }, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2) return;
            if (n->inputs[0] == n->inputs[1]) {
                const Value g = n->inputs[0]->value * seed;
                n->inputs[0]->backward(g + g);
                return;
            }
            if (wants(n->inputs[0])) n->inputs[0]->backward(n->inputs[1]->value * seed);
            if (wants(n->inputs[1])) n->inputs[1]->backward(n->inputs[0]->value * seed);
        }, 1);
    }

    Tensor operator/(const Tensor& o) const
    {
        return binary(o, [](const Value& a, const Value& b) { return a / b; }, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2) return;
            if (wants(n->inputs[0])) n->inputs[0]->backward(seed / n->inputs[1]->value);
            if (wants(n->inputs[1]))
                n->inputs[1]->backward(-n->inputs[0]->value * seed / (n->inputs[1]->value * n->inputs[1]->value));
        }, 2);
    }

    Tensor operator-() const
    {
        Tensor r = makeResult(-value(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(-seed);
        });
        return r;
    }

    Tensor operator+(float s) const { return *this + scalar(s, false); }
    Tensor operator-(float s) const { return *this - scalar(s, false); }
    Tensor operator*(float s) const { return *this * scalar(s, false); }
    Tensor operator/(float s) const { return *this / scalar(s, false); }
    friend Tensor operator+(float s, const Tensor& t) { return t.scalar(s, true) + t; }
    friend Tensor operator-(float s, const Tensor& t) { return t.scalar(s, true) - t; }
    friend Tensor operator*(float s, const Tensor& t) { return t.scalar(s, true) * t; }
    friend Tensor operator/(float s, const Tensor& t) { return t.scalar(s, true) / t; }

    // ---- math (aixCore.hpp:2440-2480; backward :2123-2163) ------------------------------------------
    Tensor exp() const
    {
        Tensor r = makeResult(value().exp(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed * n->value);
        }, 0, true);
        return r;
    }

    Tensor log() const
    {
        Tensor r = makeResult(value().log(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed / n->inputs[0]->value);
        }, 1);
        return r;
    }

    Tensor tanh() const
    {
        Tensor r = makeResult(value().tanh(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward((n->value * n->value).withScalar(&Device::sub, 1.0f, true) * seed);
        }, 0, true);
        return r;
    }

    // aixCore.hpp:2533-2540; backward :2165-2176 (only the base is differentiated: the exponent is a constant)
    Tensor pow(float e) const
    {
        const Tensor ex = Tensor(e, Shape{}, device(), dtype()).broadcastTo(shape());
        Tensor r = makeResult(value().pow(ex.value()), isRequireGrad(), !m_node->isLeaf);
        r.m_node->setBackward({m_node, ex.m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2) return;
            if (wants(n->inputs[0]))
                n->inputs[0]->backward(seed * n->inputs[1]->value * n->inputs[0]->value.pow(n->inputs[1]->value.withScalar(&Device::sub, 1.0f)));
        }, 3);
        return r;
    }

    Tensor sqrt() const
    {
        Tensor r = makeResult(value().sqrt(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(n->value.withScalar(&Device::div, 0.5f, true) * seed);
        }, 0, true);
        return r;
    }

    // ---- reductions (aixCore.hpp:2482-2521; backward :2165-2176, 2235-2252) --------------------
    Tensor sum() const
    {
        Tensor r = makeResult(value().sum(), isRequireGrad());
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed.broadcastTo(n->inputs[0]->value.shape()));
        });
        return r;
    }

    Tensor sum(size_t dim, bool keepDim = false) const
    {
        Tensor r = makeResult(value().sum(dim, keepDim), isRequireGrad());
        r.m_node->dim0 = dim; r.m_node->keepDim = keepDim;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            const Shape& orig = n->inputs[0]->value.shape();
            n->inputs[0]->backward(n->keepDim ? seed.broadcastTo(orig) : seed.unsqueeze(n->dim0).broadcastTo(orig));
        });
        return r;
    }

    Tensor mean() const { return sum() / (float)value().size(); }
    Tensor mean(size_t dim, bool keepDim = false) const { return sum(dim, keepDim) / (float)shape()[dim]; }

    // aixCore.hpp:2626-2633
    Tensor var(size_t dim, bool unbiased = true, bool keepDim = false) const
    {
        const Tensor deviation = *this - mean(dim, true);
        const size_t count = unbiased ? shape()[dim] - 1 : shape()[dim];
        const Tensor v = (deviation * deviation).sum(dim, true) / float(count);
        return keepDim ? v : v.squeeze(dim);
    }

    Tensor max(size_t dim, bool keepDim = false) const
    {
        Tensor r = makeResult(value().max(dim, keepDim), isRequireGrad());
        r.m_node->dim0 = dim;
        r.m_node->setBackward({m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.empty()) return;
            n->inputs[0]->backward(seed * n->inputs[0]->value.argmaxIndices(n->dim0));
        }, 1);
        return r;
    }

    // aixCore.hpp:2557-2569; matmulBackwardFunc :2178-2194.  Stacks of matrices (rank above 2) transpose their
    // last two dims.
    Tensor matmul(const Tensor& o) const
    {
        Tensor r = makeResult(value().matmul(o.value()), isRequireGrad() || o.isRequireGrad(), !m_node->isLeaf || !o.m_node->isLeaf);
        r.m_node->setBackward({m_node, o.m_node}, [](Node* n, const Value& seed) {
            if (n->inputs.size() < 2) return;
            const size_t rank = seed.shape().size(), d0 = rank - 2, d1 = rank - 1;
            if (n->inputs[0] == n->inputs[1]) {
                const Value xT = n->inputs[0]->value.transpose(d0, d1);
                n->inputs[0]->backward(seed.matmul(xT) + xT.matmul(seed));
                return;
            }
            if (wants(n->inputs[0])) n->inputs[0]->backward(seed.matmul(n->inputs[1]->value.transpose(d0, d1)));
            if (wants(n->inputs[1])) n->inputs[1]->backward(n->inputs[0]->value.transpose(d0, d1).matmul(seed));
        }, 3);
        return r;
    }

private:
    static bool wants(const NodePtr& n) { return n->requireGrad || n->retainGrad; }

    // aixCore.hpp:2017-2024
    static void defaultBackward(Node* n, const Value& seed)
    {
        if (n->requireGrad && !n->retainGrad) n->grad() += seed;
    }

    // aixCore.hpp:2783-2796
    Tensor makeResult(Value v, bool anyGrad) const { return makeResult(std::move(v), anyGrad, !m_node->isLeaf); }
    static Tensor makeResult(Value v, bool anyGrad, bool anyNonLeaf)
    {
        Tensor r;
        r.m_node = std::make_shared<Node>(std::move(v), anyGrad);
        r.m_node->isLeaf = !anyGrad && !anyNonLeaf;
        r.m_node->backwardFn = defaultBackward;
        r.m_node->handles = 1;
        return r;
    }

    // The scalar operand of `tensor op scalar`: rank-0 tensor seen through a broadcast view.  When
    // the scalar is on the left it inherits requireGrad from the tensor (aixCore.hpp:2408-2438).
    Tensor scalar(float s, bool onLeft) const
    {
        return Tensor(s, Shape{}, device(), dtype(), onLeft && isRequireGrad()).broadcastTo(shape());
    }

    // reads: which operands' values the backward formula reads: 0 none (add, sub), 1 "the other operand of every
    // operand that wants a gradient" (mul), 2 "the divisor if anybody wants a gradient, the dividend if the divisor does" (div)
    template <class Fwd, class Bwd> Tensor binary(const Tensor& o, Fwd fwd, Bwd bwd, int reads = 0) const
    {
        const Shape bc = shape() == o.shape() ? shape() : broadcastShapes(shape(), o.shape());
        const Tensor lhs = broadcastTo(bc), rhs = o.broadcastTo(bc);
        Tensor r = makeResult(fwd(lhs.value(), rhs.value()), isRequireGrad() || o.isRequireGrad(),
                              !lhs.m_node->isLeaf || !rhs.m_node->isLeaf);
        unsigned mask = 0;
        const bool wl = wants(lhs.m_node), wr = wants(rhs.m_node);
        if (reads == 1) mask = lhs.m_node == rhs.m_node ? 1u : (wl ? 2u : 0u) | (wr ? 1u : 0u);
        if (reads == 2) mask = (wl || wr ? 2u : 0u) | (wr ? 1u : 0u);
        r.m_node->setBackward({lhs.m_node, rhs.m_node}, bwd, mask);
        return r;
    }

    void drop() noexcept { if (m_node) { m_node->handleReleased(); m_node.reset(); } }

    NodePtr m_node;
};

inline Tensor matmul(const Tensor& a, const Tensor& b) { return a.matmul(b); }
inline Tensor exp(const Tensor& a) { return a.exp(); }
inline Tensor log(const Tensor& a) { return a.log(); }
inline Tensor tanh(const Tensor& a) { return a.tanh(); }
inline Tensor mean(const Tensor& a) { return a.mean(); }

} // namespace aixfe
