"""The C++ host layer (lten::Tensor / FullyConnected / FullyConnected_q / Conv2d / matmul over the C ABI):
its test program replays l-ten's matmul_test and fc_test on the GPU and checks the layer plumbing."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HOST = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "light-tensor_amd", "host")


def test_host_layer_program():
    exe = os.path.join(HOST, "test_host")
    assert os.path.exists(exe), "build with: make -C light-tensor_amd/host"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr[-2000:])
    assert r.returncode == 0
    for name in ("matmul_test", "fc_test", "fc_chain_test", "mlp_step_test", "training_test", "conv_training_test", "fcq_test", "fcq_reload_test", "conv_test", "convq_test", "error_test"):
        assert f"{name} passed" in r.stdout
