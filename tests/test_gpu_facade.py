"""The C++ host facade (cnet_amd/host/cnet.hpp: upstream's CNet / CFunc API over the device library) on the GPU.

tests/cpp/facade_test.cpp builds nets through the upstream-shaped API, runs them batched on the device and compares
every node plane, loss, argmax and SGD step with the CPU oracle run sample by sample with upstream's step semantics
(the pattern of upstream testE2E / testBatch / testUpdateInputs, tests/gputests.h:378, 1454, 1269).  The driver is
compiled by `make -C cnet_amd/host` (part of __graft_entry__.build()).
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "bin", "facade_test")


def _run(*args, timeout=240, env=None):
    assert os.path.exists(BIN), "tests/bin/facade_test is not built (make -C cnet_amd/host)"
    res = subprocess.run([BIN] + list(args), capture_output=True, text=True, timeout=timeout,
                         env=dict(os.environ, **env) if env else None)
    print(res.stdout[-6000:])
    print(res.stderr[-2000:])
    assert res.returncode == 0, "facade_test %s failed:\n%s" % (" ".join(args), "\n".join(
        l for l in res.stdout.splitlines() if l.startswith("FAIL")))
    return res.stdout


def test_readme_mnist_net_batched_training_step():
    out = _run("mnist")
    assert out.count("PASS") > 40 and "FAIL" not in out


def test_readme_mnist_net_with_the_cpu_forward_operator_installed():
    """Same step with the CPU path's own (slightly inexact) forward DFT operator on the device: agreement tightens from
    ~7e-5 to <1e-5, which pins the remaining difference on the CPU FFT's float twiddle recurrence."""
    out = _run("mnist_cpu_operator")
    assert "FAIL" not in out


def test_residual_stack_with_l2_targets():
    out = _run("resblock")
    assert "FAIL" not in out


def test_per_sample_api_runs_on_the_device():
    out = _run("persample")
    assert "FAIL" not in out


def test_embedding_batch():
    out = _run("embedding")
    assert "FAIL" not in out


def test_token_model_with_one_token_per_sample():
    """The fifth configuration's model at reduced size through the facade: an EmbeddingBatch of batch x seq one-token samples,
    SeqFourierTrans mixing along the sequence, per-token layers, CrossEntropy on the next token, one SGD step; with one
    gradient per value and with both halves of every pair."""
    out = _run("token_model")
    assert "FAIL" not in out and out.count("PASS") >= 26


def test_triang_fourier_crelu_net_with_adam_steps():
    out = _run("adam")
    assert "FAIL" not in out and out.count("PASS") > 30


def test_loss_map_sampling_and_the_gpunet_spellings():
    """getLoss(label)[uid], sample(), findFirstOfType, GpuForward / GpuInfer / GpuBackward(label, was_failure)."""
    out = _run("loss_map")
    assert "FAIL" not in out and out.count("PASS") >= 14


def test_accessors_of_the_cpu_net_and_infer_update():
    """ComplexNet's small members as CNet::cpuNet() hands them out upstream: maxDepth / getFuncAtDepth, getTotalSizeBytes,
    getNoVars, layer_at / front / back, testEqual, and infer() / update(rate, batch) of the per-sample API."""
    out = _run("accessors")
    assert "FAIL" not in out and out.count("PASS") >= 33


def test_upstream_model_files_restore_and_run_on_the_device(tmp_path):
    out = _run("saved_model", os.path.join(ROOT, "tests", "golden"), str(tmp_path))
    assert "FAIL" not in out and out.count("PASS") >= 16


def test_host_batch_pipeline_prefetch_and_graph_replay_give_the_same_bits():
    out = _run("pipeline")
    assert "FAIL" not in out and out.count("PASS") >= 11 and "samples_per_sec_prefetch" in out


def test_host_batch_pipeline_variants_at_batch_1024():
    """The same loop variants at a batch where the products take the block kernels (columns split off, K cut): losses and
    weights must still agree to the bit between all of them."""
    out = _run("pipeline", "1024", "4")
    assert "PASS" in out and "FAIL" not in out


def test_data_input_marked_not_trainable():
    """CNet::setInputTrainable(inp, false): same losses and weights to the bit, the data input keeps what was fed."""
    out = _run("frozen_input")
    assert "PASS" in out and "FAIL" not in out


def test_gradients_of_input_functions_left_with_their_consumers_until_the_update():
    """CNet::deferGathers: two backward passes before an update, a look at the gradients in between, an Adam-style step,
    recorded phases and whole recorded steps give the bits of gathering at once."""
    out = _run("deferred")
    assert "FAIL" not in out and out.count("PASS") >= 4


def test_batches_of_real_samples_send_their_real_plane_only():
    """InputBatch::imagIsZero / CNet::sendZeroPlanes: the imaginary plane of real data is cleared on the device instead of
    travelling; losses, weights and the stepped data input agree to the bit with the zeros sent."""
    out = _run("real_batches")
    assert "FAIL" not in out and out.count("PASS") >= 6


def test_nets_of_the_upstream_gpu_tests():
    out = _run("upstream_nets")
    assert "FAIL" not in out and out.count("PASS") >= 25


def test_error_behaviour():
    out = _run("errors")
    assert "FAIL" not in out


def test_residual_stack_of_8_blocks_reduced_width_against_the_oracle():
    """configs[3] at width 64, batch 16, at a rate that trains (1e-4): every step's per-sample losses, input and weight
    gradients and updated weights against the oracle run sample by sample; the loss must fall at every step."""
    out = _run("stack8", "64", "8", "16", "6", "0.0001", "0", "finite", "learn")
    assert "FAIL" not in out and out.count("PASS") >= 30


def test_residual_stack_at_the_configured_rate_overflows_where_the_cpu_path_does():
    """configs[3] names a learning rate of 0.01.  Eight un-normalised residual blocks amplify the input about 4000 times;
    at that rate the first update throws the weights so far that the second forward pass leaves the finite fp32 numbers,
    on the CPU path itself.  The device must agree with the oracle up to that step and overflow at the same one."""
    out = _run("stack8", "64", "8", "16", "4", "0.01", "0", "overflow")
    assert "FAIL" not in out and "at the same step (1)" in out


def test_residual_stack_full_size_against_the_oracle_and_ten_steps():
    """configs[3] at full size (8 x Linear 2048 -> 2048, batch 2048): the per-sample loss and the dz* reaching the data
    input through all eight blocks for 4 rows of the first step against the oracle, then the stated 10 SGD steps at a rate
    that trains, the loss falling at every step."""
    out = _run("stack8", "2048", "8", "2048", "10", "0.000003", "4", "finite", "learn", timeout=600)
    assert "FAIL" not in out and out.count("PASS") >= 4


def test_three_product_switch_of_the_facade():
    """CNet::threeProductGemm(bool): reaches the kernels (other bits), agrees with four products to 1e-5 over three SGD steps,
    and may be flipped on an allocated net."""
    out = _run("three_products")
    assert "FAIL" not in out and out.count("PASS") >= 8


@pytest.mark.parametrize("scenario", [("pipeline", "1024", "4"), ("resblock",), ("adam",), ("upstream_nets",),
                                      ("stack8", "64", "8", "16", "6", "0.0001", "0", "finite", "learn"),
                                      ("stack8", "2048", "8", "2048", "10", "0.000003", "4", "finite", "learn")],
                         ids=lambda s: "_".join(s[:3]))
def test_scenarios_with_three_real_products_per_complex_product(scenario):
    """The block kernels of the matrix products forming a complex product from three real ones (CNET_CGEMM_3M=1,
    cnet_cgemm_set_products(3)): the same comparisons with the oracle, at the same bounds, as with four."""
    out = _run(*scenario, timeout=600, env={"CNET_CGEMM_3M": "1"})
    assert "FAIL" not in out and "PASS" in out
