"""MLP training (autograd + Adam) on DeviceHIP against the CPU device: the same native driver loop
(aix_amd/csrc/frontend/mlp.hpp) runs once on the GPU backend and once on the oracle device, from
identical host data; the per-step losses are compared.

Tolerances.  The two devices agree operator by operator to the parity bars (exact add/mul/div,
<= 2 ulp exp/log, 1e-5 relative for the f32 matmul and reductions, whose summation order differs).
  * First 5 steps: 1e-5 relative (observed: 5e-7).  A wrong formula anywhere in forward, backward
    or Adam shows here at once (at the 1e-2 level and above); rounding differences have not been
    amplified yet (in the MNIST-shaped case they then grow about 3x per step, on the CPU alone too).
  * Whole trace, small networks: 1e-3 relative over 100 steps (observed: 3e-7).
  * Whole trace, MNIST-shaped network: training on random labels drives the loss from 0.23 to
    below 1e-3 by memorising the batch, and in that regime the trace is sensitive to rounding as
    such: moving 1 % of one weight matrix by ONE ulp changes the CPU device's own trace by up to
    7e-3 relative.  The GPU trace is therefore held to an envelope measured in the same test,
    20 x the deviation of that perturbed CPU run (and never more than 0.1), not to a fixed bar.
The observed deviations are printed."""
import numpy as np
import pytest

from oracle import drivers as OD

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from aix_amd import device as D
    d = D.Device(0)
    yield d
    d.close()


def _compare(dev, shape, steps, threads=16, envelope=False):
    from aix_amd import drivers as GD
    batch, n_in, hidden, n_out = shape
    data = OD.mlp_data(batch, n_in, hidden, n_out)
    want, _, (ops, matmuls) = OD.oracle_mlp(batch, n_in, hidden, n_out, steps, 1e-3, data, threads=threads)
    tol = 1e-3
    if envelope:
        x, y, w, b = data
        nudged = [a.copy() for a in w]
        mask = np.random.default_rng(1).random(nudged[1].shape) < 0.01
        nudged[1][mask] = np.nextafter(nudged[1][mask], np.float32(10))
        other, _, _ = OD.oracle_mlp(batch, n_in, hidden, n_out, steps, 1e-3, (x, y, nudged, b), threads=threads)
        spread = float((np.abs(other.astype(np.float64) - want) / np.abs(want)).max())
        tol = min(0.1, max(1e-3, 20 * spread))
        print(f"CPU trace moves by {spread:.3e} when 1% of W2 moves by one ulp -> tolerance {tol:.3e}")
    got, secs = GD.mlp(dev, batch, n_in, hidden, n_out, steps, 1e-3, data)
    rel = np.abs(got.astype(np.float64) - want) / np.abs(want)
    print(f"MLP {shape} x{steps}: loss {want[0]:.6f} -> {want[-1]:.6f} (cpu), {got[-1]:.6f} (gpu); "
          f"max rel dev {rel.max():.3e} at step {int(rel.argmax())}; first step {rel[0]:.3e}; "
          f"gpu {np.median(secs[1:]) * 1e3:.2f} ms/step; {matmuls // steps} matmuls and {ops // steps} operator calls per step")
    assert np.all(np.isfinite(got))
    assert want[-1] < want[0]
    assert rel[0] <= 1e-5, "first forward pass"
    assert rel[:5].max() <= 1e-5, "first 5 steps"
    assert rel.max() <= tol
    return got, want


def test_small_mlp_100_steps(dev):
    before = dev.batched_launch_stats()
    _compare(dev, (64, 48, 32, 10), 100)
    launches, kernels = (a - b for a, b in zip(dev.batched_launch_stats(), before))
    print(f"launches that carried several kernels: {launches}, kernels carried: {kernels}")
    # Adam's update (aixOptimizer.hpp:112-140) of the six parameters: one launch per step, not six
    assert launches >= 100 and kernels >= 500          # (one parameter's update shares its kernel with the end of backward)


def test_ragged_mlp(dev):
    """Extents that are multiples of nothing: every GEMM tile, vector tail and reduction tail is partial."""
    _compare(dev, (37, 29, 23, 7), 30)


def test_mnist_shaped_mlp_100_steps(dev):
    """784 -> 256 -> 256 -> 10, batch 512: the configuration's layout at a size the CPU finishes in seconds."""
    _compare(dev, (512, 784, 256, 10), 100, envelope=True)


def test_full_size_mlp_against_the_committed_cpu_trace(dev):
    """The configuration at its real size -- 784 -> 2048 -> 2048 -> 10, batch 4096, 100 steps -- against the per-step
    losses of the CPU oracle device committed in tests/golden/mlp_c3_trace.json (tests/golden/make_mlp_c3_trace.py
    wrote it from the same seeded host data; over two hours of CPU time, so it is not rerun here).  The first forward
    pass (step 0): 1e-5 relative, the bar of its matmuls and reductions (observed 3e-7).  Steps 1-4: 1e-4 -- Adam's first
    updates have the size of the learning rate whatever the gradient's size (m / sqrt(v) = +-1 after one step), so a
    gradient entry near zero whose sign differs by rounding moves its weight by twice the learning rate: with 6 million
    weights the loss of the next steps differs at the 1e-5 level (observed 1.0e-5 at step 2), not at that of the
    arithmetic.  Whole trace, step by step: six times the largest deviation that the CPU's own run with 1 % of W2 moved
    by one unit in the last place has shown up to two steps later (at least 2e-4, at most 0.5).  That run leaves the
    fixture the way a GPU run does -- 1e-4 by step 11, 1e-3 by step 16, 0.108 at the bump of the loss around step 65 -- and
    is one sample of that sensitivity, hence the factor: two orders in which the GPU adds up the rows of the bias
    gradients' column sums use 0.35 and 0.55 of the bound at their worst step (deviations of 0.123 at step 65 and 0.086
    at step 63), so the bound is tight where the arithmetic shows and follows the CPU's own sensitivity where the
    trajectory, not the arithmetic, decides."""
    import json
    import os
    from aix_amd import drivers as GD
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mlp_c3_trace.json")) as f:
        fixture = json.load(f)
    batch, n_in, hidden, n_out = fixture["shape"]
    assert (batch, n_in, hidden, n_out) == (4096, 784, 2048, 10) and fixture["steps"] == 100
    want = np.frombuffer(bytes.fromhex("".join(fixture["losses_hex"])), dtype=np.float32).astype(np.float64)
    assert np.array_equal(want, np.array(fixture["losses"]))
    other = np.array(fixture["losses_one_ulp_perturbed"])
    own = np.abs(other - want) / np.abs(want)
    spread = float(own.max())
    so_far = np.maximum.accumulate(own)
    tol = np.minimum(0.5, np.maximum(2e-4, 6 * so_far[np.minimum(np.arange(own.size) + 2, own.size - 1)]))
    data = OD.mlp_data(batch, n_in, hidden, n_out)
    got, secs = GD.mlp(dev, batch, n_in, hidden, n_out, fixture["steps"], fixture["lr"], data)
    rel = np.abs(got.astype(np.float64) - want) / np.abs(want)
    print(f"full-size MLP x100: loss {want[0]:.6f} -> {want[-1]:.6f} (cpu fixture), {got[-1]:.6f} (gpu); max rel dev {rel.max():.3e} at step "
          f"{int(rel.argmax())}; first 5 steps {rel[:5].max():.3e}; CPU's own one-ulp spread {spread:.3e}; largest share of the step's bound {(rel / tol).max():.2f} at step {int((rel / tol).argmax())}; "
          f"gpu {np.median(secs[1:]) * 1e3:.2f} ms/step against {fixture['cpu_seconds_per_step']:.1f} s/step on {fixture['threads']} CPU threads")
    print("relative deviation per step:", " ".join(f"{v:.1e}" for v in rel))
    assert np.all(np.isfinite(got)) and got[-1] < got[0]
    assert rel[0] <= 1e-5, "first forward pass"
    assert rel[:5].max() <= 1e-4, "first 5 steps"
    assert np.all(rel <= tol), f"steps beyond their bound: {np.flatnonzero(rel > tol).tolist()}"


def test_full_size_mlp_early_steps_gradients_and_losses(dev):
    """Where the arithmetic, not the trajectory, decides: the L2 norms of the six parameters' gradients in steps 0-4 of the
    full-size configuration and the losses of steps 0-10, against the CPU oracle device's figures committed in
    tests/golden/mlp_c3_early.json (tests/golden/make_mlp_c3_early.py; its losses equal the 100-step trace bit for bit).
    Gradient norms of steps 0 and 1: 1e-4 relative (observed 1.4e-5 and 2.4e-5: the composed ReLU's mask flips where a
    hidden value is within rounding of zero).  From step 2 on the trajectory shows: Adam's first updates move every weight
    by the learning rate whatever its gradient's size, so gradient entries whose sign differs by rounding put the two
    runs 2 lr apart in those weights, and the gradients -- far more than the loss, which stays within 1e-4 -- feel it:
    observed 4.5e-4, 5.8e-4, 2.4e-3 at steps 2, 3, 4, held to 2e-3, 2e-3, 1e-2.  Losses: steps 0-4 1e-4, steps 5-10 1e-3
    (observed 7e-5; the CPU's own run with 1 % of one weight matrix moved by one unit in the last place is 1e-4 away by
    step 11)."""
    import json
    import os
    from aix_amd import drivers as GD
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mlp_c3_early.json")) as f:
        fixture = json.load(f)
    batch, n_in, hidden, n_out = fixture["shape"]
    steps, want_n = fixture["steps"], np.array(fixture["grad_norms"])
    want_l = np.frombuffer(bytes.fromhex("".join(fixture["losses_hex"])), dtype=np.float32).astype(np.float64)
    assert fixture["losses_equal_mlp_c3_trace"] and steps == 11 and want_n.shape == (5, 6)
    data = OD.mlp_data(batch, n_in, hidden, n_out)
    got_l, _, got_n = GD.mlp(dev, batch, n_in, hidden, n_out, steps, fixture["lr"], data, norm_steps=want_n.shape[0])
    rel_n = np.abs(got_n.astype(np.float64) - want_n) / want_n
    rel_l = np.abs(got_l.astype(np.float64) - want_l) / np.abs(want_l)
    print("gradient norms, relative deviation per step (w1 b1 w2 b2 w3 b3):")
    for s in range(rel_n.shape[0]):
        print(f"   step {s}: " + " ".join(f"{v:.1e}" for v in rel_n[s]))
    print("losses, relative deviation per step:", " ".join(f"{v:.1e}" for v in rel_l))
    assert np.all(rel_n.max(axis=1) <= np.array([1e-4, 1e-4, 2e-3, 2e-3, 1e-2])), rel_n.max(axis=1)
    assert rel_l[:5].max() <= 1e-4 and rel_l[5:].max() <= 1e-3
