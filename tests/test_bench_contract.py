"""The parts of the bench / entry-point contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_entry_points_exist_and_product_never_imports_the_oracle():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry
    assert callable(entry.build) and callable(entry.smoke)
    pkg = os.path.join(ROOT, "mindspeed-rl_amd", "mindspeed_rl_amd")
    for name in os.listdir(pkg):
        if name.endswith(".py"):
            text = open(os.path.join(pkg, name)).read()
            assert "import oracle" not in text and "from oracle" not in text, name
    csrc = os.path.join(ROOT, "mindspeed-rl_amd", "csrc")
    for name in os.listdir(csrc):
        assert "oracle" not in open(os.path.join(csrc, name)).read(), name
