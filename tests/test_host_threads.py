"""The helper threads that compare and copy the buffers of tensors whose data pointer the caller holds
(boat_amd/csrc/host/parbytes.c): the C check of tests/c/parbytes_check.c, compiled against that source file alone."""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_parallel_compare_and_copy_agree_with_memcmp_and_memcpy(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    exe = tmp_path / "parbytes_check"
    build = subprocess.run([gcc, "-O2", "-std=c11", "-D_GNU_SOURCE", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}",
                            f"-I{ROOT / 'boat_amd' / 'csrc' / 'host'}", str(ROOT / "tests" / "c" / "parbytes_check.c"),
                            str(ROOT / "boat_amd" / "csrc" / "host" / "parbytes.c"), "-o", str(exe), "-lpthread"],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout + run.stderr
