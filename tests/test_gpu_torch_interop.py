"""The C ABI beside PyTorch in one process (device memory and streams that torch owns)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

# Importing torch for the first time on a fresh machine can take minutes while its libraries page in;
# the check gets this long and is skipped, not failed, when that is not enough.
PATIENCE_S = 150


def test_torch_tensors_and_a_torch_stream():
    """Runs tests/torch_interop_check.py as a program of its own, so that torch's GPU runtime stays
    out of this process."""
    here = os.path.dirname(os.path.abspath(__file__))
    try:
        proc = subprocess.run([sys.executable, "-u", os.path.join(here, "torch_interop_check.py")],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=PATIENCE_S)
    except subprocess.TimeoutExpired:
        pytest.skip("torch did not import and run within %d s on this machine" % PATIENCE_S)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "ok" in proc.stdout
