// drivers.cpp -- the benchmark's driver loops run on the CPU oracle (liboracle_drivers.so).
// TEST INFRASTRUCTURE: the same front-end / autograd / optimizer headers that drive the GPU
// backend are compiled here against oracle::OracleDevice, so that a loss trace from the GPU can
// be compared with the CPU-device trace of the identical program.
#include "oracle_device.hpp"
#include "../aix_amd/csrc/frontend/mlp.hpp"
#include "../aix_amd/csrc/frontend/transformer.hpp"

#include <cstdio>

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

// Same contract as aixbench_transformer.
int oracle_transformer(int threads, uint64_t layers, uint64_t d_model, uint64_t heads, uint64_t seq, uint64_t batch, uint64_t vocab,
                       int steps, int stacked_attention, const int32_t* tokens, const float* const* params, float* losses, float* grad_norms, double* step_seconds)
{
    try {
        oracle::OracleDevice dev(threads);
        const aixfe::TransformerConfig cfg{layers, d_model, heads, seq, batch, vocab, steps, stacked_attention};
        aixfe::runTransformer(&dev, cfg, tokens, params, losses, grad_norms, step_seconds);
        return 0;
    } catch (const std::exception& e) { std::snprintf(g_err, sizeof(g_err), "%s", e.what()); return 1; }
}

} // extern "C"
