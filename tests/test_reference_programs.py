"""The reference's OWN test programs (and its optimizer benchmark), linked against libboat_amd.so instead of libboat.

`make -C oracle reftests` compiles tests/unit/*.c, tests/*.c, benchmarks/*.c and three examples of the reference from where they lie, with the
reference's headers, and links them with this repository's library (outputs in oracle/_ref/reftests, built where the
reference tree exists).  They run here unchanged, in coherent-pointer mode: these programs keep the float* of
boat_tensor_data() across calls (finite differences write weights through it, the optimizer tests read the updated
parameter through it).  Programs that build graphs of their own (test_graph_phase2/3) or need a Windows header
(test_export) are not built.

test_schedulers aborts at its line 56 on the compiled reference too (a Release build of the reference compiles its
asserts out): the scheduler here reproduces the reference's learning rates bit for bit (tests/test_schedulers.py), so
it has to stop at the same assertion.
"""
import os
import subprocess
from pathlib import Path

import pytest


BIN = Path(__file__).resolve().parent.parent / "oracle" / "_ref" / "reftests"

PASSING = {   # program -> a line of its own success report
    "test_autodiff": "Autodiff tests passed!",
    "test_optimizer_adam": "All Adam optimizer tests passed!",
    "test_optimizer_rmsprop": "All RMSprop optimizer tests passed!",
    "test_optimizer_adagrad": "All Adagrad optimizer tests passed!",
    "test_attention_gradient_check": "All gradient checks PASSED",
    "test_conv_gradient_check": "All convolution gradient checks PASSED",
    "test_attention_training": "Training test completed successfully",
    "test_dense_forward": "Test PASSED",
    "test_conv_forward": "Test PASSED",
    "test_layernorm_simple": "Test completed",
    "test_transpose": "All transpose tests PASSED",
    "test_tensor": "Tensor tests passed!",
    "test_basic": "All tests passed!",
    "test_memory": "Memory tests passed!",
    "test_model_graph_integration": "All tests passed!",
    "test_phase1": "All Phase 1 tests PASSED",
    "test_simple": None,
    "test_layer_link": None,
}


def run(name, tmp_path):
    exe = BIN / name
    if not exe.exists():
        pytest.skip(f"{exe} not built (make -C oracle reftests needs the reference tree)")
    env = {k: v for k, v in os.environ.items() if k != "BOAT_HIP_COHERENT_POINTERS"}   # the library's default configuration
    return subprocess.run([str(exe)], cwd=tmp_path, env=env, capture_output=True, text=True, errors="replace", timeout=100)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(PASSING))
def test_reference_program_passes_on_this_library(name, tmp_path):
    proc = run(name, tmp_path)
    assert proc.returncode == 0, (proc.stdout[-1500:], proc.stderr[-1500:])
    if PASSING[name]:
        assert PASSING[name] in proc.stdout, proc.stdout[-1500:]
    assert "FAILED" not in proc.stdout


@pytest.mark.gpu
def test_gradient_check_program_reports_what_it_reports_on_the_reference(tmp_path):
    """tests/unit/test_gradient_check.c compares analytical gradients with float32 central differences at a tolerance
    the differences do not meet: on the compiled reference it passes addition and reports two mismatches for
    multiplication (numerical -0.0160933 / -0.00417233 against analytical -0.0163637 / -0.00411147) and exits 1.  The
    same binary on this library prints the same lines: the analytical values agree to every printed digit."""
    proc = run("test_gradient_check", tmp_path)
    assert proc.returncode == 1
    out = proc.stdout
    addition, multiplication = out.split("Testing multiplication operation gradient...")
    assert "Testing addition operation gradient..." in addition and "  PASSED" in addition and "Mismatch" not in addition
    out = multiplication
    assert "Mismatch for b[1]: analytical=-0.0163637, numerical=-0.0160933" in out
    assert "Mismatch for b[3]: analytical=-0.00411147, numerical=-0.00417233" in out
    assert "FAILED: 2 mismatches" in out


@pytest.mark.gpu
def test_optimizer_benchmark_of_the_reference_reports_the_same_losses(tmp_path):
    """benchmarks/linear_regression.c: 1000 steps each with Adam, Adam + StepLR, RMSprop and Adagrad on synthetic data
    from rand().  It registers boat_variable_grad() before the first backward, when that is still NULL
    (benchmarks/linear_regression.c:304-305), so on the reference every optimizer leaves the loss where it starts,
    1.273380; linked against this library the program reports the same final loss four times."""
    proc = run("linear_regression", tmp_path)
    assert proc.returncode == 0, proc.stderr[-1000:]
    summary = proc.stdout.split("Benchmark Results Summary")[1]
    rows = [line.split() for line in summary.splitlines() if line.startswith(("Adam", "RMSprop", "Adagrad"))]
    assert len(rows) == 4 and all("1.273380" in r for r in rows), summary


@pytest.mark.gpu
def test_scheduler_example_prints_the_learning_rates_it_prints_on_the_reference(tmp_path):
    """examples/scheduler_usage.c (step, cosine and caller-function schedules driving Adam and RMSprop): its
    learning-rate lines on this library are, character for character, the lines it printed on the compiled reference
    (tests/golden/scheduler_usage_lines.txt, written from that run)."""
    proc = run("scheduler_usage", tmp_path)
    assert proc.returncode == 0, proc.stderr[-1000:]
    want = (Path(__file__).resolve().parent / "golden" / "scheduler_usage_lines.txt").read_text().splitlines()
    got = [line for line in proc.stdout.splitlines() if ("learning rate" in line.lower() or "LR" in line)
           and "create called" not in line and "create:" not in line]
    assert got == want and len(want) > 40


@pytest.mark.gpu
def test_relu_example_of_the_reference(tmp_path):
    proc = run("test_relu", tmp_path)
    assert proc.returncode == 0 and "Result data: 0.0 0.0 0.0 0.0 1.0 2.0" in proc.stdout, proc.stdout[-500:]


@pytest.mark.gpu
@pytest.mark.parametrize("coherent", ["1", "0"])
def test_mnist_example_of_the_reference_trains_as_on_the_reference(tmp_path, coherent):
    """examples/mnist/mnist.c, the layer-hook training loop (conv, pool, dense, softmax; forward, backward and update
    per batch, mnist.c:197-246) on a small synthetic set: 80 training and 16 test images whose bright patch tells the
    class (tests/golden/mnist_synthetic.npz, which also holds the lines the program printed on the compiled reference).
    Linked against this library it prints the same accuracy after every epoch and on the test set, in coherent-pointer
    mode and in the default mode alike (the program fetches data pointers anew whenever it needs them)."""
    import re

    import numpy as np

    import boat_cases as bc
    with np.load(Path(__file__).resolve().parent / "golden" / "mnist_synthetic.npz", allow_pickle=False) as z:
        g = {k: z[k] for k in z.files}
    bc.write_mnist_example_files(tmp_path, g["train_images"], g["train_labels"], g["test_images"], g["test_labels"])
    exe = BIN / "mnist"
    if not exe.exists():
        pytest.skip(f"{exe} not built (make -C oracle reftests needs the reference tree)")
    env = dict(os.environ, BOAT_HIP_COHERENT_POINTERS=coherent)
    proc = subprocess.run([str(exe)], cwd=tmp_path, env=env, capture_output=True, text=True, errors="replace", timeout=100)
    assert proc.returncode == 0, proc.stderr[-1000:]
    lines = [re.sub(r"time=[0-9.]+s, ", "", line) for line in proc.stdout.splitlines() if re.match(r"Epoch \d|Test accuracy", line)]
    assert lines == [str(line) for line in g["reference_lines"]] and len(lines) == 6


@pytest.mark.gpu
def test_attention_benchmark_of_the_reference_runs(tmp_path):
    """benchmarks/attention_performance.c (B4 S16 H64, 8 heads, causal; 50 forward and backward passes through
    boat_attention_forward / boat_attention_backward): runs to its report on this library."""
    proc = run("attention_performance", tmp_path)
    assert proc.returncode == 0, proc.stderr[-1000:]
    assert "Forward pass:" in proc.stdout and "Backward pass:" in proc.stdout and "Benchmark completed." in proc.stdout


def test_zz_scheduler_program_stops_where_it_stops_on_the_reference(tmp_path):
    """tests/unit/test_schedulers.c fails a host assert of its own (:56) on the reference as well, before it creates a
    tensor: no GPU is involved, so this test carries no gpu mark."""
    proc = run("test_schedulers", tmp_path)
    assert proc.returncode == -6 and "test_schedulers.c:56" in proc.stderr, (proc.returncode, proc.stderr[-500:])
