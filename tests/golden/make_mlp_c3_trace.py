"""Writes tests/golden/mlp_c3_trace.json: the per-step losses of the MLP configuration at its full size (784 -> 2048 ->
2048 -> 10, batch 4096, f32, Adam lr 1e-3, 100 steps from the seeded host data of oracle.drivers.mlp_data) on the CPU
oracle device, plus the same run with 1 % of the second weight matrix moved by one unit in the last place -- the
measure of how far rounding alone moves this trace on the CPU, which sets the envelope the GPU trace is held to.

The oracle device runs the product's front-end headers on oracle/cpuref (its f32 matmul is the i-k-j reordering of the
reference's loop nest, bit-identical to it: tests/test_frontend_vs_ref.py, tests/test_oracle_vs_ref.py).  Each of the
two runs takes about 65-80 minutes on 6 threads (38 s per step); run from the repository root:  python tests/golden/make_mlp_c3_trace.py [threads]"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import drivers as OD  # noqa: E402

SHAPE = (4096, 784, 2048, 10)
STEPS = 100
LR = 1e-3


def main():
    threads = int(sys.argv[1]) if len(sys.argv) > 1 else 8
    data = OD.mlp_data(*SHAPE)
    t0 = time.time()
    losses, secs, (ops, matmuls) = OD.oracle_mlp(*SHAPE, STEPS, LR, data, threads=threads)
    print(f"base run: {time.time() - t0:.0f} s, loss {losses[0]:.6f} -> {losses[-1]:.6f}", flush=True)
    x, y, w, b = data
    nudged = [a.copy() for a in w]
    mask = np.random.default_rng(1).random(nudged[1].shape) < 0.01
    nudged[1][mask] = np.nextafter(nudged[1][mask], np.float32(10))
    t0 = time.time()
    other, _, _ = OD.oracle_mlp(*SHAPE, STEPS, LR, (x, y, nudged, b), threads=threads)
    print(f"perturbed run: {time.time() - t0:.0f} s", flush=True)
    out = {
        "what": "MLP 784-2048-2048-10, batch 4096, f32, Adam lr 1e-3, 100 steps on the CPU oracle device",
        "shape": list(SHAPE), "steps": STEPS, "lr": LR, "threads": threads,
        "operator_calls_per_step": ops // STEPS, "matmuls_per_step": matmuls // STEPS,
        "losses": [float(v) for v in losses],
        "losses_hex": [np.float32(v).tobytes().hex() for v in losses],
        "losses_one_ulp_perturbed": [float(v) for v in other],
        "cpu_seconds_per_step": float(np.median(secs)),
    }
    with open(os.path.join(HERE, "mlp_c3_trace.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("written", flush=True)


if __name__ == "__main__":
    main()
