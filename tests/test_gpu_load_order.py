"""The library loaded BEFORE torch has touched the GPU, in a fresh process.  torch's wheels bring their own HIP runtime and
load it at torch's first device call; a process that ends up with two HIP runtimes has one that finds no device.  The
loader (cudf_amd/_capi.py) therefore loads torch's runtime first; this test runs that order for real."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

PROGRAM = r"""
import numpy as np
from cudf_amd import _capi
_capi.load()                       # first: nothing has initialised the GPU yet
from cudf_amd import nvtext as nv
from cudf_amd.arrow_host import HostStringsColumn
from oracle import pyoracle as orc
host = HostStringsColumn.from_pylist(["the quick brown fox", "", None, "jumps over the lazy dog " * 50])
vocab = HostStringsColumn.from_pylist(["[UNK]", "the", "quick", "fox", "dog", "##s", "jump", "over", "lazy"])
d = nv.DeviceStringsColumn.from_host(host)
a = np.array([3, 5, 7], np.uint32); b = np.array([1, 2, 3], np.uint32)
assert nv.minhash(d, 1, a, b, 4).to_host().equals(orc.minhash(host, 1, a, b, 4))
dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(vocab))
assert nv.wordpiece_tokenize(d, dv, 0).to_host().equals(orc.wordpiece_tokenize(host, orc.Vocabulary(vocab), 0))
maps = {line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line}
assert len(maps) == 1, maps
print("one runtime, results as the oracle's")
"""


def test_library_loaded_before_torch_initialises_the_gpu():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    done = subprocess.run([sys.executable, "-c", PROGRAM], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "one runtime" in done.stdout
