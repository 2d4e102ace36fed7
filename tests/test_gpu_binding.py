"""The reference's own code on the gfx950 backend.

`make -C oracle ref-binding` links the reference's own Tensor / Operator / nn / optim object files (compiled, unchanged,
from the reference's sources) with binding/src: the device dispatcher, the memory layer and the origin::cuda::*
functions of include/origin/mat/origin/cuda/cuda_ops.cuh, all over libodl_hip.so. These tests run, through that build,
(1) the reference's GoogleTest suites (their device instances), (2) the reference's example program, and (3) the API
driver of the other host-layer tests — the same checks against the same fixtures and the CPU oracle, but this time every
class above the Mat interface is the reference's own object code.

The binaries exist only where the reference checkout was present at build time; the build records them, and a recorded
binary that is missing fails the test instead of skipping it."""
import re
import subprocess

import numpy as np
import pytest

import oraclelib as ol
import test_gpu_host_layer as T

pytestmark = pytest.mark.gpu


def _binary(name):
    path = ol.ref_binary(name)  # raises when the build recorded the binary and it is gone
    if path is None:
        pytest.skip("built only where the reference checkout is present (make -C oracle ref-binding)")
    return path


class _Driver:
    """The binding build of the API driver under the entry-point names the host-layer tests use (odl_host_*)."""

    def __init__(self, lib):
        self._lib = lib

    def __getattr__(self, name):
        return getattr(self._lib, name.replace("odl_host_", "odl_bind_"))


@pytest.fixture(scope="module")
def b():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    _binary("libodl_bind_driver.so")
    return _Driver(ol.binding_driver())


@pytest.fixture(scope="module")
def o():
    return ol.oracle()


def test_the_references_unit_tests_pass_with_its_own_classes_on_this_backend():
    exe = _binary("reference_tests_on_binding")
    out = subprocess.run([exe, "--gtest_filter=*CUDA*:TensorCreateTest.*:MultiTypeTensorTest.*:TensorOptionsTest.*",
                          "--gtest_brief=1"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    tail = out.stdout[-3000:]
    print("\n" + "\n".join(tail.splitlines()[-4:]), flush=True)
    assert out.returncode == 0, tail
    ran = int(re.search(r"\[==========\] (\d+) tests from (\d+) test suites ran", out.stdout).group(1))
    passed = int(re.search(r"\[  PASSED  \] (\d+) tests", out.stdout).group(1))
    # 556 cases in 40 suites; one skips itself (a broadcast the reference's own device matmul does not take either)
    assert ran >= 556 and passed >= ran - 1, tail


def test_the_references_example_program_trains_with_its_own_classes_on_this_backend():
    exe = _binary("example_nn_linear_on_binding")
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "cuda:0" in out.stdout
    last = [l for l in out.stdout.splitlines() if l.startswith("iter199")][-1]
    m = re.search(r"loss = ([-0-9.e]+), w = ([-0-9.e]+), b = ([-0-9.e]+)", last)
    # the reference's own integration test accepts |w-2| < 0.1 and |b-5| < 0.1
    # (tests/unit_test/autograd/test_linear_regression.cpp:47-101)
    assert abs(float(m.group(2)) - 2.0) < 0.1 and abs(float(m.group(3)) - 5.0) < 0.1, last


def test_matmul_through_the_references_tensor_and_operator(b, o):
    T.test_tensor_level_matmul_forward_backward(b, o)


@pytest.mark.parametrize("name", sorted(T.CONV_CASES))
def test_conv2d_operator_against_the_reference_fixtures(b, name):
    T.test_conv_operator_matches_reference_fixtures(b, name)


def test_conv2d_on_float64_tensors_through_the_references_operator(b):
    T.test_float64_conv2d_and_its_gradients_through_the_tensor_api(b)


def test_softmax_on_float64_tensors_through_the_references_operator(b):
    T.test_float64_softmax_through_the_tensor_api(b)


@pytest.mark.parametrize("name", sorted(T.POOL_CASES))
def test_max_pool_indices_bit_exact(b, name):
    T.test_max_pool_through_the_mat_interface_bit_exact(b, name)


def test_sum_to_broadcast_and_errors(b):
    T.test_sum_to_broadcast_and_error_codes(b)


def test_softmax_cross_entropy_and_label_errors(b):
    T.test_softmax_ce_operator_and_label_errors(b)


@pytest.mark.parametrize("steps", [1, 2])
def test_mlp_training_step_of_the_references_own_layers_and_adam(b, steps):
    T.test_mlp_training_step_matches_the_reference(b, steps)


def test_cnn_training_step_of_the_references_own_layers_and_sgd(b):
    T.test_cnn_training_step_matches_the_reference(b)


def test_mlp_step_at_benchmark_size_against_the_oracle(b, o):
    T.test_mlp_step_at_benchmark_size_against_the_oracle(b, o)


def test_cnn_step_at_reduced_batch_against_the_oracle(b, o):
    T.test_cnn_step_at_reduced_batch_against_the_oracle(b, o)
