// drivers.cpp -- the benchmark's driver loops run on the CPU oracle (liboracle_drivers.so).
// TEST INFRASTRUCTURE: the same front-end / autograd / optimizer headers that drive the GPU
// backend are compiled here against oracle::OracleDevice, so that a loss trace from the GPU can
// be compared with the CPU-device trace of the identical program.
#include "oracle_device.hpp"
#include "../aix_amd/csrc/frontend/mlp.hpp"
#include "../aix_amd/csrc/frontend/transformer.hpp"

#include <cstdio>
#include <cstring>

namespace aix {
// the two non-inline members of the interface class (the product defines them in its own library)
Device::~Device() = default;
size_t Device::dataTypeSize(DataType dtype) { return cpuref_dtype_size((int)dtype); }
}

namespace { thread_local char g_err[512] = ""; }

extern "C" {

const char* oracle_drivers_last_error(void) { return g_err; }

// Same contract as aixbench_mlp (aix_amd/csrc/bench/driver.cpp); counts[0] = operator calls,
// counts[1] = matmul calls (may be NULL).
int oracle_mlp(int threads, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
               const float* x, const float* y, const float* const* w, const float* const* b, float* losses, double* step_seconds,
               uint64_t* counts)
{
    try {
        oracle::OracleDevice dev(threads);
        const aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        aixfe::runMlp(&dev, cfg, host, losses, step_seconds);
        if (counts) { counts[0] = dev.ops; counts[1] = dev.matmuls; }
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

// The same training loop with Adam in its in-place form (frontend/nn.hpp: state updated where it lies, beta^t in device
// memory), every step issued: what aixbench_mlp_captured's eager and replayed steps are compared with.
int oracle_mlp_in_place(int threads, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
                        const float* x, const float* y, const float* const* w, const float* const* b, float* losses, double* step_seconds)
{
    try {
        oracle::OracleDevice dev(threads);
        aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        cfg.adamInPlace = 1;
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        aixfe::runMlp(&dev, cfg, host, losses, step_seconds);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

// Same contract as aixbench_mlp_norms.
int oracle_mlp_norms(int threads, uint64_t batch, uint64_t in, uint64_t hidden, uint64_t out, int steps, float lr, int single_pass,
                     const float* x, const float* y, const float* const* w, const float* const* b, float* losses, double* step_seconds,
                     float* grad_norms, int norm_steps)
{
    try {
        oracle::OracleDevice dev(threads);
        const aixfe::MlpConfig cfg{batch, in, hidden, out, steps, lr, single_pass};
        const aixfe::MlpHost host{x, y, {w[0], w[1], w[2]}, {b[0], b[1], b[2]}};
        aixfe::runMlp(&dev, cfg, host, losses, step_seconds, grad_norms, norm_steps);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

// Same contract as aixbench_transformer.  threads < 0: -threads threads and the oracle device's wide16 mode (matmul,
// reduceTo and sum of 16-bit tensors add exactly and round once; see oracle_device.hpp).
int oracle_transformer(int threads, uint64_t layers, uint64_t d_model, uint64_t heads, uint64_t seq, uint64_t batch, uint64_t vocab,
                       int steps, int stacked_attention, const int32_t* tokens, const float* const* params, float* losses, float* grad_norms, double* step_seconds)
{
    try {
        oracle::OracleDevice dev(threads < 0 ? -threads : threads, threads < 0);
        const aixfe::TransformerConfig cfg{layers, d_model, heads, seq, batch, vocab, steps, stacked_attention};
        aixfe::runTransformer(&dev, cfg, tokens, params, losses, grad_norms, step_seconds);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

// Gradients of programs that slice a tensor in every way the single-pass traversal distinguishes, once by
// Tensor::backward() (the reference's recursion: one zero-padded tensor per slice, added into the leaf, aixCore.hpp:2228-2233)
// and once by Tensor::backwardOnce() (windows gathered per node).  x is [rows, cols] host data; `which` picks the program;
// grads receives the two gradients of x back to back (recursion first).  Values that are small integers make both exact.
int oracle_slice_gradients(int which, uint64_t rows, uint64_t cols, const float* x, const float* w, float* grads)
{
    try {
        using namespace aixfe;
        oracle::OracleDevice dev(1);
        const DataType F32 = DataType::kFloat32;
        for (int pass = 0; pass < 2; ++pass) {
            Tensor X = Tensor::fromHost(&dev, F32, Shape{rows, cols}, x, true);
            const Tensor W = Tensor::fromHost(&dev, F32, Shape{rows, cols}, w);
            // an interior node, so that the windows are gathered at a node that is not a leaf
            const Tensor h = X * W;
            Tensor loss;
            const uint64_t c2 = cols / 2, c4 = cols / 4, r2 = rows / 2;
            switch (which) {
                case 0:     // windows of one dim that cover it: no zero fill
                    loss = (h.slice(1, 0, c4) * 2.0f).sum() + (h.slice(1, c4, c2) * 3.0f).sum() + (h.slice(1, c2, cols) * 5.0f).sum();
                    break;
                case 1:     // windows of one dim that leave a gap
                    loss = (h.slice(1, 0, c4) * 2.0f).sum() + (h.slice(1, c2, cols) * 5.0f).sum();
                    break;
                case 2:     // windows that overlap
                    loss = (h.slice(1, 0, c2) * 2.0f).sum() + (h.slice(1, c4, cols) * 3.0f).sum();
                    break;
                case 3:     // windows beside a seed that is no window
                    loss = (h.slice(1, 0, c2) * 2.0f).sum() + (h.slice(1, c2, cols) * 3.0f).sum() + (h * h).sum();
                    break;
                case 4:     // windows of different dims
                    loss = (h.slice(1, 0, c2) * 2.0f).sum() + (h.slice(0, r2, rows) * 3.0f).sum();
                    break;
                case 5:     // a strided window beside a plain one
                    loss = (h.slice(0, 0, rows, 2) * 2.0f).sum() + (h.slice(0, 1, rows, 2) * 3.0f).sum();
                    break;
                case 6: {   // slices of slices, put together again by cat (heads of sequences)
                    std::vector<Tensor> seqs;
                    for (uint64_t b = 0; b < 2; ++b) {
                        const Tensor hb = h.slice(0, b * r2, (b + 1) * r2);
                        std::vector<Tensor> heads;
                        for (uint64_t k = 0; k < 4; ++k) heads.push_back(hb.slice(1, k * c4, (k + 1) * c4) * float(k + 1 + 4 * b));
                        seqs.push_back(Tensor::cat(heads, 1));
                    }
                    loss = (Tensor::cat(seqs, 0) * W).sum();
                    break;
                }
                default: throw std::invalid_argument("no such program");
            }
            if (pass == 0) loss.backward(); else loss.backwardOnce();
            const Value g = X.grad();
            dev.synchronize();
            std::memcpy(grads + pass * rows * cols, g.data(), rows * cols * sizeof(float));
        }
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

} // extern "C"
