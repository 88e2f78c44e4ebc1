"""A step captured into a HIP graph and replayed (DeviceHIP::beginCapture / endCapture / replay, include/aixhip.h) against
the same step issued operator by operator: a replay must compute exactly what issuing the step again would.  The reference
has no such thing (its GPU device batches dispatches into command buffers, aixDeviceMetal.cpp:1344-1389).  Each graph is
replayed several times with the program's own eager work and synchronisations in between, and every replay is checked."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import devharness as H
from aix_amd import device as D
from oracle import cpuref as O
from oracle import drivers as OD

pytestmark = pytest.mark.gpu
CPU = O.lib()


@pytest.fixture(scope="module")
def dev():
    d = H.Dev()
    yield d
    d.close()


def test_replays_of_a_captured_transformer_step_equal_the_eager_steps(dev):
    """Forward + backward of the decoder-only transformer, both ways of issuing attention: steps 0-1 eager, step 2
    captured, steps 2-6 replays.  The step repeats exactly (gradients are zeroed and accumulated in place), so losses and
    every gradient norm of the replays must equal the eager run's bit for bit (embedding gradients are summed with atomics,
    whose order may differ from run to run: those two norms to 1e-3)."""
    from aix_amd import drivers as GD
    for cfg, stacked in (((2, 64, 4, 32, 2, 128), False), ((2, 64, 4, 32, 2, 128), True), ((1, 128, 4, 128, 3, 512), True)):
        data = OD.transformer_data(*cfg)
        eager_l, eager_n, _ = GD.transformer(dev.dev, cfg, 7, data, stacked=stacked)
        got_l, got_n, secs, nodes = GD.transformer_captured(dev.dev, cfg, 7, data, 2, stacked=stacked)
        print(f"{cfg} stacked={stacked}: {nodes} graph nodes; eager step {secs[1] * 1e3:.2f} ms, replayed step {np.median(secs[3:]) * 1e3:.2f} ms")
        assert nodes > 10
        assert np.array_equal(got_l, eager_l), (got_l, eager_l)
        assert np.array_equal(got_n[:, 2:], eager_n[:, 2:])
        assert np.allclose(got_n[:, :2], eager_n[:, :2], rtol=1e-3, atol=0)


def test_captured_updates_in_place_advance_step_by_step(dev):
    """x <- x * a + b on device tensors, updated in place, captured once and replayed five times with eager work between the
    replays: every replay advances x by one step of the recurrence, bit for bit as the oracle computes it; a block the
    captured work used as a temporary is not handed out while the graph lives."""
    rng = np.random.default_rng(48000)
    shape = [96, 40]
    x, a, b = (T.contiguous_tensor(rng, O.F32, shape) for _ in range(3))
    (px, dx), (_, da), (_, db) = dev.put(x), dev.put(a), dev.put(b)
    tmp_host = T.empty(O.F32, shape)
    want = T.empty(O.F32, shape)
    t = T.empty(O.F32, shape)

    def step_on_oracle():
        assert CPU.binary(O.MUL, C.byref(x.desc()), C.byref(a.desc()), C.byref(t.desc())) == 0
        assert CPU.binary(O.ADD, C.byref(t.desc()), C.byref(b.desc()), C.byref(want.desc())) == 0
        x.storage[...] = want.storage

    def issue():
        pt = dev.raw(tmp_host.storage.nbytes, keep=False)
        dt = H.kdesc(tmp_host, pt)
        dev.dev.call("mul", H.ref(dx), H.ref(da), H.ref(dt))
        dev.dev.call("flush")                               # the product is stored: two kernels, a temporary between them
        dev.dev.call("add", H.ref(dt), H.ref(db), H.ref(dx))
        dev.dev.deallocate(pt)
        return pt

    issue(); step_on_oracle()                               # once uncaptured: kernels compiled
    T.assert_same_bits(dev.fetch(px, x.storage), x.storage, "eager step")
    graph = C.c_void_p()
    dev.dev.call("capture_begin")
    temporary = issue()
    dev.dev.call("capture_end", C.byref(graph))
    T.assert_same_bits(dev.fetch(px, x.storage), x.storage, "nothing of a capture has run")
    others = []
    for k in range(5):
        dev.dev.call("graph_replay", graph)
        step_on_oracle()
        # eager work on other tensors between the replays; its blocks never are the graph's temporary
        p = dev.raw(tmp_host.storage.nbytes, keep=False)
        others.append(p)
        assert p != temporary
        dev.dev.call("mul", H.ref(da), H.ref(db), H.ref(H.kdesc(tmp_host, p)))
        T.assert_same_bits(dev.fetch(px, x.storage), x.storage, f"replay {k}")
    for p in others:
        dev.dev.deallocate(p)
    # what a capture refuses
    dev.dev.call("capture_begin")
    assert dev.dev.status("synchronize") == 2
    extra = C.c_void_p()
    dev.dev.call("capture_end", C.byref(extra))
    dev.dev.call("graph_destroy", extra)
    # a capture given up: nothing of it runs, the device goes on as before, another capture can be opened
    before = dev.fetch(px, x.storage).copy()
    dev.dev.call("capture_begin")
    issue()
    assert dev.dev.status("capture_begin") == 2                 # one open capture per device
    dev.dev.call("capture_abort")
    dev.dev.call("capture_abort")                               # (without an open capture: nothing)
    T.assert_same_bits(dev.fetch(px, x.storage), before, "an abandoned capture has run nothing")
    dev.dev.call("graph_replay", graph)
    step_on_oracle()
    T.assert_same_bits(dev.fetch(px, x.storage), x.storage, "a replay after an abandoned capture")
    assert dev.dev.status("graph_replay", None) == 1            # a null graph is an invalid argument
    dev.dev.call("graph_destroy", graph)
    dev.release()


@pytest.mark.parametrize("cfg,single_pass", [((256, 64, 128, 10), False), ((512, 96, 256, 10), True), ((4096, 784, 2048, 10), False)], ids=str)
def test_replays_of_a_captured_training_step_equal_the_eager_steps(dev, cfg, single_pass):
    """A whole training step of the MLP -- zeroGrad, forward, softmax + cross-entropy, backward, Adam's update -- with
    Adam in its in-place form (its state updated where it lies, beta^t in device memory, so nothing the host computes
    changes from step to step): steps 0-2 eager, step 3 captured, steps 3-7 replays.  The losses must equal, bit for bit,
    those of eight eager steps of the same program, i.e. every replay advanced parameters, Adam's moments and beta^t
    exactly as issuing the step would; and they follow the CPU device running the same program.  The last case is the
    benchmark's full-size network (the three-plane f32 GEMM route, K splits, the workspace the eager steps grew)."""
    from aix_amd import drivers as GD
    steps, at = 8, 3
    data = OD.mlp_data(*cfg)
    eager, _, none = GD.mlp_captured(dev.dev, *cfg, steps, 1e-3, data, -1, single_pass=single_pass)
    got, secs, nodes = GD.mlp_captured(dev.dev, *cfg, steps, 1e-3, data, at, single_pass=single_pass)
    print(f"mlp {cfg}: {nodes} graph nodes; eager step {np.median(secs[1:at]) * 1e3:.2f} ms, replayed step {np.median(secs[at + 1:]) * 1e3:.2f} ms; losses {got}")
    assert none == 0 and nodes > 10
    assert np.all(np.isfinite(got)) and got[-1] < got[0]
    assert np.array_equal(got, eager), (got, eager)
    if cfg[0] * cfg[2] <= 1 << 17:                               # the CPU device finishes these in a second
        want, _ = OD.oracle_mlp_in_place(*cfg, steps, 1e-3, data, threads=8, single_pass=single_pass)
        rel = np.abs(got.astype(np.float64) - want) / np.abs(want)
        print("   against the CPU device, relative:", " ".join(f"{v:.1e}" for v in rel))
        assert rel[0] <= 1e-5 and rel.max() <= 1e-4
