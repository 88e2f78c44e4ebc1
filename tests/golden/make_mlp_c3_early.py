"""Writes tests/golden/mlp_c3_early.json: the first steps of the MLP configuration at its full size (784 -> 2048 -> 2048
-> 10, batch 4096, f32, Adam lr 1e-3, seeded host data of aix_amd.workloads.mlp_data) on the CPU oracle device, with what
the per-step losses of tests/golden/mlp_c3_trace.json do not show: the L2 norms of the six parameters' gradients (w1, b1,
w2, b2, w3, b3) in steps 0-4, where the arithmetic of the backward pass -- not the trajectory -- decides, and the losses
of steps 0-10 again (they must equal that trace bit for bit: taking the norms between backward and the update changes
nothing the program computes).

About 38 s per step on 6 threads (11 steps: 7 minutes); run from the repository root:
    python tests/golden/make_mlp_c3_early.py [threads]"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import drivers as OD  # noqa: E402

SHAPE = (4096, 784, 2048, 10)
STEPS, NORM_STEPS = 11, 5
LR = 1e-3


def main():
    threads = int(sys.argv[1]) if len(sys.argv) > 1 else 8
    data = OD.mlp_data(*SHAPE)
    t0 = time.time()
    losses, secs, norms = OD.oracle_mlp(*SHAPE, STEPS, LR, data, threads=threads, norm_steps=NORM_STEPS)
    print(f"{time.time() - t0:.0f} s, loss {losses[0]:.6f} -> {losses[-1]:.6f}", flush=True)
    with open(os.path.join(HERE, "mlp_c3_trace.json")) as f:
        trace = json.load(f)
    same = [np.float32(v).tobytes().hex() for v in losses] == trace["losses_hex"][:STEPS]
    print("losses equal the committed trace bit for bit:", same, flush=True)
    out = {
        "what": "MLP 784-2048-2048-10, batch 4096, f32, Adam lr 1e-3: steps 0-10 on the CPU oracle device, gradient norms of steps 0-4",
        "shape": list(SHAPE), "steps": STEPS, "lr": LR, "threads": threads,
        "losses": [float(v) for v in losses],
        "losses_hex": [np.float32(v).tobytes().hex() for v in losses],
        "losses_equal_mlp_c3_trace": bool(same),
        "grad_norm_order": ["w1", "b1", "w2", "b2", "w3", "b3"],
        "grad_norms": [[float(v) for v in row] for row in norms],
    }
    with open(os.path.join(HERE, "mlp_c3_early.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("written", flush=True)


if __name__ == "__main__":
    main()
