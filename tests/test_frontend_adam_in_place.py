"""Adam in its in-place form (aix_amd/csrc/frontend/nn.hpp: moments updated where they lie, beta^t a rank-0 tensor in device
memory multiplied by beta every step) against Adam as the reference writes it (aixOptimizer.hpp:112-140: new moment tensors
every step, bias corrections 1 - beta^t computed by the host in double precision), both on the CPU oracle device.  The
per-element arithmetic is the same; only beta^t differs, a running f32 product against a rounded double power, so the loss
traces start a few ulps apart and drift as any two roundings of one training run do (Adam's first updates have the size of
the learning rate whatever the gradient's size) -- and must, or the captured training step on the GPU (which needs the in-place
form) would train a different network."""
import numpy as np
import pytest

from oracle import drivers as OD


@pytest.mark.parametrize("cfg,single_pass", [((64, 32, 48, 10), False), ((96, 20, 64, 7), True)], ids=str)
def test_in_place_adam_follows_the_reference_form(cfg, single_pass):
    steps = 40
    data = OD.mlp_data(*cfg)
    ref, _, _ = OD.oracle_mlp(*cfg, steps, 1e-3, data, threads=4, single_pass=single_pass)
    got, _ = OD.oracle_mlp_in_place(*cfg, steps, 1e-3, data, threads=4, single_pass=single_pass)
    rel = np.abs(got.astype(np.float64) - ref) / np.abs(ref)
    print("relative deviation of the loss, first / worst step:", rel[0], rel.max())
    assert got[0] == ref[0], "the first loss is computed before any update"
    assert rel[:5].max() <= 2e-6 and rel.max() <= 1e-4
    assert ref[-1] < 0.98 * ref[0], "the network trains"
