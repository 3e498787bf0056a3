"""The C programs of boat_amd/examples, built beside the library, run as a user would run them: separate processes
that link libboat_amd.so and speak only Boat's C API."""
import json
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

LIB_DIR = Path(__file__).resolve().parent.parent / "boat_amd" / "lib"


def run_example(name, *args):
    exe = LIB_DIR / name
    if not exe.exists():
        pytest.fail(f"{exe} is missing: build it first (python -m boat_amd.build)")
    return subprocess.run([str(exe), *map(str, args)], capture_output=True, text=True, timeout=110)


def test_api_tour_every_check_holds_and_nothing_stays_allocated():
    """One pass over tensors, the tape, layer hooks, the model container, losses, optimizers, schedulers, attention and
    convolution from plain C; the program checks its own invariants and frees everything it made."""
    proc = run_example("api_tour")
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    rec = json.loads(lines[0])
    assert rec["failed_check_line"] == 0
    assert rec["host_blocks_allocated"] == rec["host_blocks_freed"] > 0
    assert "device in use 0 B" in lines[-1], lines[-1]


def test_mlp_train_step_program_trains():
    proc = run_example("mlp_train_step", 50, 5)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["steps"] == 50 and rec["loss_last"] < rec["loss_first"]


def test_block_train_step_program_trains():
    """The pre-LN transformer block step of the benchmark as a C program against Boat's API, at a small size."""
    proc = run_example("block_train_step", 4, 1, 2, 128, 256, 4, 512)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["steps"] == 4 and rec["d_model"] == 256 and 0 < rec["loss_last"] < rec["loss_first"]


def test_block_train_step_with_kept_pointers_and_large_tensors():
    """The same program in the default configuration (pointers to the weights, the input and the target stay valid, so
    the library compares and copies their buffers around every call) at a size where those buffers are large enough
    for the helper threads (FFN weights and activations of 8 MiB and more): the losses must be the ones of the run in
    which nothing is kept coherent."""
    import os
    args = ("block_train_step", 3, 1, 8, 512, 1024, 16, 2048)
    exe = LIB_DIR / args[0]
    if not exe.exists():
        pytest.fail(f"{exe} is missing: build it first (python -m boat_amd.build)")
    recs = []
    for mode in ("1", "0"):
        env = dict(os.environ, BOAT_HIP_COHERENT_POINTERS=mode)
        proc = subprocess.run([str(exe), *map(str, args[1:])], capture_output=True, text=True, timeout=110, env=env)
        assert proc.returncode == 0, proc.stderr[-2000:]
        recs.append(json.loads(proc.stdout.strip().splitlines()[-1]))
    assert recs[0]["loss_first"] == recs[1]["loss_first"] and recs[0]["loss_last"] == recs[1]["loss_last"]
    assert 0 < recs[0]["loss_last"] < recs[0]["loss_first"]
