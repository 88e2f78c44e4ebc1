"""Attention issued as matmuls on [batch, heads, ...] stacks against attention issued as one 2-D matmul
per (sequence, head), on the CPU device: the two programs apply the same arithmetic to the same
numbers -- the stack only changes how many operator calls carry it -- so the losses and the gradient
norms of every parameter agree (the per-head program adds the heads' zero-padded gradients together,
which is exact), while the number of operator calls collapses."""
import numpy as np
import pytest

from oracle import drivers as OD


@pytest.mark.parametrize("cfg", [(2, 64, 4, 32, 2, 128), (1, 48, 3, 16, 3, 64)], ids=str)
def test_stacked_attention_computes_what_the_per_head_loops_compute(cfg):
    data = OD.transformer_data(*cfg)
    loop_l, loop_n, _ = OD.oracle_transformer(cfg, 1, data, threads=4)
    stack_l, stack_n, _ = OD.oracle_transformer(cfg, 1, data, threads=4, stacked=True)
    assert np.all(np.isfinite(stack_l)) and np.all(np.isfinite(stack_n))
    assert stack_l.view(np.uint32).tolist() == loop_l.view(np.uint32).tolist()
    big = loop_n > 1e-3 * loop_n.max()
    rel = np.abs(stack_n.astype(np.float64) - loop_n)[big] / loop_n[big]
    print(f"{cfg}: loss {stack_l[0]:.6f}; gradient norms max rel dev {rel.max():.2e}")
    assert rel.max() <= 1e-6
