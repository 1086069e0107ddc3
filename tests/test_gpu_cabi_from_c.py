"""The C ABI driven by a C++ host program (no Python, no PyTorch in the process): two nano-batches of the SwiGLU
MLP on two HIP streams, checked inside the program against the plain-C restatement of the arithmetic."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HOST_PROGRAM = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi_host", "mlp_two_nano_batches")


def test_mlp_through_the_c_abi_from_a_cpp_host_program():
    if not os.path.exists(HOST_PROGRAM):
        pytest.skip("tests/cabi_host/mlp_two_nano_batches is not built: __graft_entry__.build() makes it")
    print("C++ host program: two nano-batches through the C ABI", flush=True)
    done = subprocess.run([HOST_PROGRAM], capture_output=True, text=True, timeout=120)
    print(done.stdout, done.stderr, flush=True)
    assert done.returncode == 0, (done.returncode, done.stdout, done.stderr)
    assert done.stdout.strip().endswith("ok") and "for gfx950" in done.stdout
