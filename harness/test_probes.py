"""The benchmark's measurement aids on the GPU (run by naming this file: it is not part of the product's test suite):
python -m pytest harness/test_probes.py -m gpu"""
import numpy as np
import pytest

from harness import probes
from shrike_amd import runtime
from tests.helpers import Layer
from tests.test_decode_gpu import DeviceLayer

pytestmark = pytest.mark.gpu


def test_measurement_probes_run_and_check_their_arguments():
    """The empty launch and the read-only kernel that bench.py times beside phase 1 (a library of their own)."""
    gpu = runtime
    gpu.init(0)
    L = Layer(33, 256, 128, 12, 4)
    dl = DeviceLayer(gpu, L)
    lib = probes.load()
    sink = gpu.empty(4).fill(0)
    cells = gpu.empty(4 * 4)
    cells.upload(np.array([dl.cell_of[e] for e in (0, 5, 7, 11)], np.uint32))
    nbytes = (dl.off.down_w_off - dl.off.gate_w_off) // 1024 * 1024
    probes.check(lib.shrike_probe_empty_launch(None, 64, sink.ptr), "probe_empty_launch")
    probes.check(lib.shrike_probe_read(None, dl.pool.bases, dl.pool.stride, cells.ptr, 4, dl.off.gate_w_off, nbytes,
                                       sink.ptr), "probe_read")
    gpu.synchronize()
    assert sink.download(np.uint32, 1)[0] == 0
    assert lib.shrike_probe_read(None, dl.pool.bases, dl.pool.stride, cells.ptr, 4, 0, dl.pool.stride + 1024, sink.ptr) != 0
    assert "leaves the cell" in probes.last_error()
    assert lib.shrike_probe_read(None, dl.pool.bases, dl.pool.stride, cells.ptr, 4, 8, 1024, sink.ptr) != 0
    assert lib.shrike_probe_empty_launch(None, 0, sink.ptr) != 0


def test_issue_probe_runs_and_checks_its_arguments():
    """Matrix and vector instructions side by side: the three forms launch, drain, and leave the sink alone."""
    gpu = runtime
    gpu.init(0)
    lib = probes.load()
    one = gpu.empty(4)
    one.upload(np.ones(1, np.float32))
    sink = gpu.empty(64).fill(0)
    for what in (1, 2, 3):
        for waves in (1, 2, 4):
            probes.check(lib.shrike_probe_issue(None, what, waves, 64, one.ptr, sink.ptr), "probe_issue")
    gpu.synchronize()
    assert not sink.download(np.uint32, 16).any()
    assert lib.shrike_probe_issue(None, 0, 2, 64, one.ptr, sink.ptr) != 0
    assert lib.shrike_probe_issue(None, 3, 3, 64, one.ptr, sink.ptr) != 0
    assert lib.shrike_probe_issue(None, 3, 2, 0, one.ptr, sink.ptr) != 0
    assert lib.shrike_probe_issue(None, 3, 2, 64, None, sink.ptr) != 0
