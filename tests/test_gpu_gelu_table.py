"""GPU: the first large gelu calls of a process (fresh interpreter per case, because the table's
state is per process): under stream capture before the table exists, and on two streams at once."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
SCRIPT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gelu_first_calls_script.py")


@pytest.mark.parametrize("mode", ["capture", "streams"])
def test_first_large_gelu_calls_of_a_process(ops, mode):
    done = subprocess.run([sys.executable, SCRIPT, mode], capture_output=True, text=True, timeout=110)
    assert done.returncode == 0 and done.stdout.strip().endswith("OK"), done.stdout + done.stderr
