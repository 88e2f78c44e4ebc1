"""Writes tests/golden/transformer_c4_widths.json: loss and the L2 norm of every parameter's gradient of ONE layer of the
transformer configuration at its real widths (d 768, 12 heads, seq 512, vocab 8192, GELU MLP 4x; batch 1) on the CPU
oracle device, from the seeded host data of aix_amd.workloads.transformer_data -- the widths at which the GPU runs its
128 x 192, LDS-direct and grouped-launch GEMM routes, which the reduced models of the tests never reach.

Two runs of the stacked-attention program (the per-(sequence, head) program is the same arithmetic: bit-identical loss
and gradient norms to 1e-6 on the CPU device, tests/test_frontend_stacked_attention.py):
  literal   the CPU device as the reference has it: 16-bit matmul / reduceTo / sum keep their running sum in the element
            type (aixDeviceCPU.cpp:244-253, 336-389), one rounding to 8 bits per addition;
  wide16    those three operators add exactly and round once (oracle/oracle_device.hpp), everything else literal: the
            arithmetic the 2e-2 bar for 16-bit work with f32 accumulation is stated against.
At these widths the two differ by up to 12 % in a gradient norm (sums of 512 to 8192 bf16 terms), so the GPU is held to
the wide16 figures; the literal ones are kept beside them.

About 10 s (wide16) + 150 s (literal) on 8 threads; run from the repository root:
    python tests/golden/make_transformer_c4_widths.py [threads]"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import drivers as OD  # noqa: E402

CFG = (1, 768, 12, 512, 1, 8192)          # layers, d_model, heads, seq, batch, vocab


def main():
    threads = int(sys.argv[1]) if len(sys.argv) > 1 else 8
    data = OD.transformer_data(*CFG)
    runs = {}
    for name, wide in (("wide16", True), ("literal", False)):
        t0 = time.time()
        loss, norms, _ = OD.oracle_transformer(CFG, 1, data, threads=threads, stacked=True, wide16=wide)
        print(f"{name}: {time.time() - t0:.0f} s, loss {loss[0]:.8f}", flush=True)
        runs[name] = {"loss": float(loss[0]), "loss_hex": np.float32(loss[0]).tobytes().hex(), "grad_norms": [float(v) for v in norms[0]]}
    out = {
        "what": "decoder-only transformer forward + backward, 1 layer at the real widths, on the CPU oracle device (stacked attention)",
        "cfg": {"layers": CFG[0], "d_model": CFG[1], "heads": CFG[2], "seq": CFG[3], "batch": CFG[4], "vocab": CFG[5]},
        "data": "aix_amd.workloads.transformer_data(*cfg) (seed_tok 7, seed_w 8)",
        "parameter_shapes": [list(s) for s in OD.transformer_param_shapes(*CFG)],
        "threads": threads,
        **runs,
    }
    with open(os.path.join(HERE, "transformer_c4_widths.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("written", flush=True)


if __name__ == "__main__":
    main()
