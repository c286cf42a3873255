"""A pool of larger physical chunks than the reference's 2 MiB (`vtkv_pool_set_chunk_bytes`): the HIP
runtime serves at most some 30 000 chunks per process, so caches above 58 GiB need them.  The chunk size
belongs to the process-wide pool, hence the child process."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_a_pool_of_8_mib_chunks_serves_the_same_calls():
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "large_chunks_child.py")
    r = subprocess.run([sys.executable, child], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "large chunks ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
