"""What of bench.py's contract can be checked without a GPU: more than one GPU is refused with one line and exit code 2."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_exit_code_2():
    p = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2", "--steps", "4", "--warmup", "1"], capture_output=True,
                       text=True, timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
