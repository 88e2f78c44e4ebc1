"""ctypes binding of the native driver loops (libaixhip_bench.so): whole AIX-style programs
(expression chains, reductions, GEMM sweeps, the MLP training loop) issued from C++ through the
tensor front-end into DeviceHIP, so that no Python sits inside a step."""
import ctypes as C
import os

import numpy as np

from . import device as D
from ._build import library_path

_PF = C.POINTER(C.c_float)
_PPF = C.POINTER(_PF)
_lib = None


class BenchResult(C.Structure):
    _fields_ = [("wall_s", C.c_double), ("gpu_ms", C.c_float), ("steps", C.c_int32), ("enqueue_us", C.c_int32)]


def load():
    """Load libaixhip_bench.so.  Never builds, never falls back."""
    global _lib
    if _lib is None:
        D.load()
        path = library_path("libaixhip_bench.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is not built; run __graft_entry__.build()")
        lib = C.CDLL(path)
        P = C.c_void_p
        lib.aixbench_last_error.restype = C.c_char_p
        lib.aixbench_fused_chain.argtypes = [P, C.c_uint64, C.c_uint64, P, P, P, C.c_int, C.c_int, C.POINTER(BenchResult), P]
        lib.aixbench_reduce_item.argtypes = [P, C.c_int, C.c_uint64, C.c_uint64, P, P, C.c_int, C.c_int, C.POINTER(BenchResult), P]
        lib.aixbench_matmul.argtypes = [P, C.c_int, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_uint64, P, P, C.c_int, C.c_int,
                                        C.POINTER(BenchResult), P]
        lib.aixbench_mlp.argtypes = [P, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_float, C.c_int, _PF, _PF, _PPF, _PPF,
                                     _PF, C.POINTER(C.c_double)]
        _lib = lib
    return _lib


def run(fn, *args):
    lib = load()
    if getattr(lib, fn)(*args) != 0:
        raise RuntimeError(f"{fn}: {lib.aixbench_last_error().decode()}")


def _pointer_array(arrays):
    arr = (_PF * len(arrays))()
    for i, a in enumerate(arrays):
        assert a.dtype == np.float32 and a.flags.c_contiguous
        arr[i] = a.ctypes.data_as(_PF)
    return arr


def mlp(dev, batch, n_in, hidden, n_out, steps, lr, data, single_pass=False, norm_steps=0):
    """Train the MLP (n_in -> hidden -> hidden -> n_out, ReLU, softmax + cross-entropy, Adam) for
    `steps` steps on `dev` from host arrays data = (x, onehot, [w1, w2, w3], [b1, b2, b3]).
    single_pass=True differentiates once per node instead of once per path (the reference's way).
    Returns (loss per step, seconds per step); with norm_steps > 0 also the L2 norms of the gradients of
    w1, b1, w2, b2, w3, b3 in the first norm_steps steps, [norm_steps, 6]."""
    x, y, w, b = data
    losses = np.zeros(steps, dtype=np.float32)
    secs = np.zeros(steps, dtype=np.float64)
    pw, pb = _pointer_array(w), _pointer_array(b)
    if norm_steps:
        lib = load()
        lib.aixbench_mlp_norms.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_float, C.c_int, _PF, _PF, _PPF, _PPF,
                                           _PF, C.POINTER(C.c_double), _PF, C.c_int]
        norms = np.zeros((norm_steps, 6), dtype=np.float32)
        run("aixbench_mlp_norms", dev.handle, batch, n_in, hidden, n_out, steps, lr, int(single_pass), x.ctypes.data_as(_PF), y.ctypes.data_as(_PF),
            pw, pb, losses.ctypes.data_as(_PF), secs.ctypes.data_as(C.POINTER(C.c_double)), norms.ctypes.data_as(_PF), norm_steps)
        return losses, secs, norms
    run("aixbench_mlp", dev.handle, batch, n_in, hidden, n_out, steps, lr, int(single_pass), x.ctypes.data_as(_PF), y.ctypes.data_as(_PF),
        pw, pb, losses.ctypes.data_as(_PF), secs.ctypes.data_as(C.POINTER(C.c_double)))
    return losses, secs


def mlp_captured(dev, batch, n_in, hidden, n_out, steps, lr, data, capture_at, single_pass=False):
    """mlp() with Adam in its in-place form (state updated where it lies, beta^t kept in device memory) and, with
    capture_at >= 0, step `capture_at` -- zeroGrad, forward, loss, backward and the update -- captured into a HIP graph and
    that step and every later one enqueued as a replay of it; capture_at < 0 issues every step eagerly.
    Returns (loss per step, seconds per step, graph nodes)."""
    x, y, w, b = data
    lib = load()
    lib.aixbench_mlp_captured.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_float, C.c_int, C.c_int, _PF, _PF,
                                          _PPF, _PPF, _PF, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]
    losses = np.zeros(steps, dtype=np.float32)
    secs = np.zeros(steps, dtype=np.float64)
    nodes = C.c_uint64(0)
    run("aixbench_mlp_captured", dev.handle, batch, n_in, hidden, n_out, steps, lr, int(single_pass), capture_at, x.ctypes.data_as(_PF),
        y.ctypes.data_as(_PF), _pointer_array(w), _pointer_array(b), losses.ctypes.data_as(_PF), secs.ctypes.data_as(C.POINTER(C.c_double)), C.byref(nodes))
    return losses, secs, int(nodes.value)


def transformer_captured(dev, cfg, steps, data, capture_at, stacked=False):
    """transformer() with step `capture_at` captured into a HIP graph and that step and all later ones enqueued as replays
    of it (one launch call per step, no front-end).  Returns (losses, gradient norms, seconds per step, graph nodes)."""
    tokens, params = data
    lib = load()
    lib.aixbench_transformer_captured.argtypes = [C.c_void_p] + [C.c_uint64] * 6 + [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int32), _PPF, _PF, _PF,
                                                                               C.POINTER(C.c_double), C.POINTER(C.c_uint64)]
    losses = np.zeros(steps, np.float32)
    norms = np.zeros((steps, len(params)), np.float32)
    secs = np.zeros(steps, np.float64)
    nodes = C.c_uint64(0)
    pp = _pointer_array(params)
    run("aixbench_transformer_captured", dev.handle, *cfg, steps, int(stacked), capture_at, tokens.ctypes.data_as(C.POINTER(C.c_int32)), pp,
        losses.ctypes.data_as(_PF), norms.ctypes.data_as(_PF), secs.ctypes.data_as(C.POINTER(C.c_double)), C.byref(nodes))
    return losses, norms, secs, int(nodes.value)


def transformer(dev, cfg, steps, data, stacked=False):
    """Forward + backward of the decoder-only transformer for `steps` steps on `dev`;
    cfg = (layers, d_model, heads, seq, batch, vocab), data = (int32 tokens [batch * seq], list of f32
    parameter arrays in the order of frontend/transformer.hpp).  Returns (losses, gradient norms
    [steps, parameters], seconds per step).  stacked: attention as matmuls on [batch, heads, ...] stacks (one
    operator per layer and step of the attention) instead of one 2-D matmul per sequence and head."""
    tokens, params = data
    lib = load()
    lib.aixbench_transformer.argtypes = [C.c_void_p] + [C.c_uint64] * 6 + [C.c_int, C.c_int, C.POINTER(C.c_int32), _PPF, _PF, _PF, C.POINTER(C.c_double)]
    losses = np.zeros(steps, np.float32)
    norms = np.zeros((steps, len(params)), np.float32)
    secs = np.zeros(steps, np.float64)
    pp = _pointer_array(params)
    run("aixbench_transformer", dev.handle, *cfg, steps, int(stacked), tokens.ctypes.data_as(C.POINTER(C.c_int32)), pp, losses.ctypes.data_as(_PF),
        norms.ctypes.data_as(_PF), secs.ctypes.data_as(C.POINTER(C.c_double)))
    return losses, norms, secs
