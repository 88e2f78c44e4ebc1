"""Synthetic host inputs of the benchmark configurations (the MLP of configs[3], the transformer of configs[4], GEMM
operands): what bench.py, the examples and the tests hand to the device and, for comparison, to a CPU device.
Plain numpy, no GPU and no library needed."""
import numpy as np


def round_to_bf16_bits(x):
    """f32 -> bf16 bit patterns (uint16), round to nearest even, NaN kept NaN (aixFloat16.hpp:698-716)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
    hi = u >> 16
    rest = u & 0xFFFF
    up = (rest > 0x8000) | ((rest == 0x8000) & ((hi & 1) == 1))
    return np.where(nan, hi | 0x40, hi + up.astype(np.uint64)).astype(np.uint16)


def mlp_data(batch, n_in, hidden, n_out, seed_w=0, seed_x=5, seed_y=6):
    """Synthetic inputs of the MLP configuration: X ~ U(0,1), one-hot labels uniform over the
    classes, weights and biases U(-1,1)/sqrt(fan_in); all f32, generated on the host."""
    x = np.random.default_rng(seed_x).random((batch, n_in), dtype=np.float32)
    labels = np.random.default_rng(seed_y).integers(0, n_out, size=batch)
    y = np.zeros((batch, n_out), dtype=np.float32)
    y[np.arange(batch), labels] = 1.0
    rng = np.random.default_rng(seed_w)
    dims = [(n_in, hidden), (hidden, hidden), (hidden, n_out)]
    w = [((rng.random(d, dtype=np.float32) * 2 - 1) / np.float32(np.sqrt(d[0]))).astype(np.float32) for d in dims]
    b = [((rng.random((1, d[1]), dtype=np.float32) * 2 - 1) / np.float32(np.sqrt(d[0]))).astype(np.float32) for d in dims]
    return x, y, w, b


def transformer_param_shapes(layers, d, heads, seq, batch, vocab):
    """Parameter order of aix_amd/csrc/frontend/transformer.hpp."""
    shapes = [(vocab, d), (seq, d)]
    for _ in range(layers):
        shapes += [(1, d), (1, d), (d, d), (1, d), (d, d), (1, d), (d, d), (1, d), (d, d), (1, d),
                   (1, d), (1, d), (d, 4 * d), (1, 4 * d), (4 * d, d), (1, d)]
    shapes += [(1, d), (1, d), (d, vocab)]
    return shapes


def transformer_data(layers, d, heads, seq, batch, vocab, seed_tok=7, seed_w=8):
    """Token ids U[0, vocab), weights N(0, 0.02) (LayerNorm gains 1, all biases 0), f32 on the host."""
    tokens = np.random.default_rng(seed_tok).integers(0, vocab, size=batch * seq).astype(np.int32)
    rng = np.random.default_rng(seed_w)
    params = []
    for shape in transformer_param_shapes(layers, d, heads, seq, batch, vocab):
        if shape[0] == 1:
            params.append(np.zeros(shape, np.float32))
        else:
            params.append((rng.standard_normal(shape) * 0.02).astype(np.float32))
    # LayerNorm gains are the [1, d] arrays at block offsets 0 and 10, and the first of the last three
    gains = [2 + 16 * l + o for l in range(layers) for o in (0, 10)] + [2 + 16 * layers]
    for g in gains:
        params[g][:] = 1.0
    return tokens, params
