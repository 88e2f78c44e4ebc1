"""The reference's own front-end on the GPU backend.

oracle/_ref/libaixref_hip_drivers.so is built where the reference tree is present: the reference's
aix.hpp (Tensor, autograd, nn::Softmax, nn::CrossEntropyLoss, optim::Adam), its DeviceCPU sources, and
this repository's DeviceHIP host sources compiled against those headers, so that DeviceHIP derives
from the framework's own aix::Device and is handed to aix::Tensor like any other device.  The MLP
training loop then runs unchanged on it; its losses are compared with the same loop on the
reference's CPU device (small case, literal reference arithmetic) and with the restated front-end on
the product build of DeviceHIP (same operator stream, so the same numbers bit for bit)."""
import numpy as np
import pytest

from oracle import cpuref, drivers as OD

MISSING = OD.ref_hip_lib_path() is None or OD.ref_lib() is None
# a tree that was never built next to the reference has no oracle/_ref: skip; a tree that was, and lost it: fail loudly
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(MISSING and not cpuref.ref_expected(), reason="oracle/_ref not built (no reference tree)")]


@pytest.fixture(autouse=True)
def _reference_libraries_are_there():
    assert not MISSING, "this tree was built with the reference present (oracle/ref_built.note) but oracle/_ref/*.so is missing"


def test_reference_tensor_autograd_adam_run_unchanged_on_device_hip():
    shape, steps = (64, 48, 32, 10), 60
    on_gpu = OD.ref_hip_mlp(*shape, steps, 1e-3)
    on_cpu, _ = OD.ref_mlp(*shape, steps, 1e-3, OD.mlp_data(*shape))
    rel = np.abs(on_gpu.astype(np.float64) - on_cpu) / np.abs(on_cpu)
    print(f"reference front-end, {shape} x{steps}: CPU {on_cpu[0]:.6f} -> {on_cpu[-1]:.6f}, DeviceHIP {on_gpu[-1]:.6f}, max rel dev {rel.max():.3e}")
    assert np.all(np.isfinite(on_gpu)) and on_cpu[-1] < on_cpu[0]
    assert rel.max() <= 1e-4


def test_restated_front_end_issues_the_same_stream_on_the_gpu():
    from aix_amd import device as D, drivers as GD
    shape, steps = (128, 784, 64, 10), 25
    via_reference = OD.ref_hip_mlp(*shape, steps, 1e-3)
    dev = D.Device(0)
    try:
        via_restatement, _ = GD.mlp(dev, *shape, steps, 1e-3, OD.mlp_data(*shape))
    finally:
        dev.close()
    assert via_reference.view(np.uint32).tolist() == via_restatement.view(np.uint32).tolist()


@pytest.mark.parametrize("dtype,first,tol", [(1, 12, 2e-4), (2, 3, 5e-2), (3, 3, 1e-1)], ids=["f32", "f16", "bf16"])
def test_reference_xor_example_runs_unchanged_on_device_hip(dtype, first, tol):
    """The reference's XOR example (nn::Sequential of Linear / Tanh, MSELoss, Adam; parameters made on
    the host and moved with Module::to(device) / to(dtype), double literals converted on the device,
    item<float>() after synchronize()) with DeviceHIP in place of its GPU device: the first epochs'
    losses follow the same program on the reference's CPU device, and in f32 both runs learn XOR."""
    hidden1, hidden2, epochs = 64, 32, 400 if dtype == 1 else 6
    cpu_losses, cpu_pred = OD.ref_xor(dtype, hidden1, hidden2, epochs, 0.01)
    gpu_losses, gpu_pred = OD.ref_hip_xor(dtype, hidden1, hidden2, epochs, 0.01)
    rel = np.abs(gpu_losses[:first].astype(np.float64) - cpu_losses[:first]) / np.abs(cpu_losses[:first])
    print(f"XOR dtype {dtype}: CPU {cpu_losses[:4]} ... {cpu_losses[-1]:.3e}; DeviceHIP {gpu_losses[:4]} ... {gpu_losses[-1]:.3e}; max rel dev of the first {first}: {rel.max():.3e}")
    assert np.all(np.isfinite(gpu_losses))
    assert rel.max() <= tol
    if dtype == 1:
        want = np.array([0.0, 1.0, 1.0, 0.0])
        assert cpu_losses[-1] < 1e-3 and gpu_losses[-1] < 1e-3
        assert np.abs(cpu_pred - want).max() < 5e-2 and np.abs(gpu_pred - want).max() < 5e-2


def test_reference_save_and_load_through_device_memory(tmp_path):
    """nn::save reads the parameters of a model trained on DeviceHIP straight out of device memory and
    nn::load writes them straight into it (aixNeuralNetwork.hpp:258-301): a fresh model on DeviceHIP
    loaded from the file predicts bit for bit what the trained one does, one on the reference's CPU
    device the same within f32 rounding of tanh."""
    preds = OD.ref_hip_xor_save_load(64, 32, 300, 0.01, str(tmp_path / "xor.bin"))
    trained, on_gpu, on_cpu = preds
    print("trained", trained, "reloaded on DeviceHIP", on_gpu, "reloaded on the CPU device", on_cpu)
    assert trained.view(np.uint32).tolist() == on_gpu.view(np.uint32).tolist()
    assert np.abs(on_cpu - trained).max() <= 1e-5
    assert np.abs(trained - np.array([0.0, 1.0, 1.0, 0.0])).max() < 5e-2


def test_reference_device_test_cases_on_device_hip():
    """The cases of the reference's device test file -- every operator against its CPU device over the reference's test
    sizes and all nine element types, 200 queued operator pairs with autograd, 1024 chained adds on a million elements,
    1000 Adam steps without a synchronize, the benchmark's XOR model -- written with the reference's own TensorValue /
    Tensor / nn / optim classes (oracle/ref_drivers.cpp: deviceChecks) and run with DeviceHIP as the device under test."""
    failures, checks, report = OD.ref_device_checks(True)
    print(f"{checks} checks, {failures} failures\n{report}")
    assert checks > 5000
    assert failures == 0, report
