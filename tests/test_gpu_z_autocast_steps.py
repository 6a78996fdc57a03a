"""Training steps of both benchmark networks under float16 autocast (utils_own.py:127-131,156-165), each in a child
process: the float16 convolutions of the vendor library are searched and compiled per shape on first use, and a
crash inside that machinery must fail one test, not end the test run."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "autocast_steps_child.py")


@pytest.mark.parametrize("which", ["tinyconv", "resnet18"])
def test_training_steps_under_fp16_autocast(which):
    print("child process:", which, flush=True)
    proc = subprocess.run([sys.executable, "-u", CHILD, which], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          timeout=300)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), (
        "exit code %d\n--- stdout ---\n%s\n--- stderr ---\n%s" % (proc.returncode, proc.stdout[-3000:], proc.stderr[-6000:]))
