"""What bench.py promises to whoever launches it, as far as a machine without a GPU can check."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_one_line_and_exit_code_2():
    """This engine runs on one GPU: for N > 1 bench.py prints one line that says so and exits
    with 2 (before anything touches a GPU)."""
    for n in ("2", "8"):
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", n, "--steps", "3",
                              "--warmup", "1"], capture_output=True, text=True, timeout=120)
        assert run.returncode == 2
        lines = [l for l in run.stdout.splitlines() if l.strip()]
        assert len(lines) == 1 and "one GPU" in lines[0] and f"--gpus {n}" in lines[0]
