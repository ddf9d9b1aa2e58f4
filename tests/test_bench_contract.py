"""What the measuring program promises without a GPU: more than one GPU is refused in one line."""

from __future__ import annotations

import subprocess
import sys

from conftest import ROOT


def test_more_than_one_gpu_is_refused_with_one_line_and_status_2():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    assert len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout
