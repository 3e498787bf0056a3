"""Every entry point of Boat's API survives null pointers and zero sizes (run in a child process so that a crash
names the entry point instead of taking the test session down)."""
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu


def test_every_entry_point_survives_null_arguments():
    script = Path(__file__).resolve().parent / "null_args_sweep.py"
    proc = subprocess.run([sys.executable, "-u", str(script)], capture_output=True, text=True, timeout=110)
    lines = proc.stdout.strip().splitlines()
    assert proc.returncode == 0, f"died with {proc.returncode} in or after {lines[-1] if lines else '?'}\n{proc.stderr[-1500:]}"
    assert lines[-1].startswith("SURVIVED") and int(lines[-1].split()[1]) > 150
