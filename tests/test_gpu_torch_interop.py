"""The C ABI beside PyTorch in one process (device memory and streams that torch owns)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.timeout(900)
def test_torch_tensors_and_a_torch_stream():
    """Runs tests/torch_interop_check.py as a program of its own (importing torch takes a minute or
    two on a fresh machine, and a second GPU runtime stays out of this process)."""
    here = os.path.dirname(os.path.abspath(__file__))
    proc = subprocess.run([sys.executable, "-u", os.path.join(here, "torch_interop_check.py")],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=800)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "ok" in proc.stdout
