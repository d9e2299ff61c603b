import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ext():
    from glowq_amd.kernels import load_w4a16_extension

    return load_w4a16_extension()


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "w4a16_golden.npz"))


@pytest.fixture(params=["stream", "qstream", "quad", "classic"])
def small_m_route(request, ext):
    """Runs a test with the stream GEMV serving 1..4 token rows (the other kernels above), with the stream-scheduled 4x4x4
    matrix-core GEMV serving 2..4 token rows, with the 4x4x4 matrix-core GEMV serving 1..16 token rows, and with all
    switched off (wave-dot GEMV for 1..4 rows, skinny MFMA kernel above)."""
    if request.param == "qstream":
        old = ext.set_tuning("qstream_max_m", 4), ext.set_tuning("qstream_shape_rule", 0)
        yield request.param
        ext.set_tuning("qstream_max_m", old[0]), ext.set_tuning("qstream_shape_rule", old[1])
        return
    if request.param == "stream":
        old = ext.set_tuning("stream_max_m", 4), ext.set_tuning("stream_shape_rule", 0), ext.set_tuning("qstream_max_m", 0)
        yield request.param
        ext.set_tuning("stream_max_m", old[0]), ext.set_tuning("stream_shape_rule", old[1]), ext.set_tuning("qstream_max_m", old[2])
        return
    old = ext.set_tuning("quad_max_m", 16 if request.param == "quad" else 0)
    old_min = ext.set_tuning("quad_min_m", 1)
    old_small = ext.set_tuning("small_group_mb", 0)  # no shape-dependent choice between the two at 2..4 rows
    old_stream = ext.set_tuning("stream_max_m", 0)   # the stream GEMV would take the single rows of both modes
    old_qstream = ext.set_tuning("qstream_max_m", 0)
    yield request.param
    ext.set_tuning("qstream_max_m", old_qstream)
    ext.set_tuning("quad_max_m", old)
    ext.set_tuning("quad_min_m", old_min)
    ext.set_tuning("small_group_mb", old_small)
    ext.set_tuning("stream_max_m", old_stream)


@pytest.fixture(autouse=True)
def _fresh_env_knobs():
    """The modules read the W4A16_* switches from a cache: every test starts and ends with the cache in step with the
    environment, and a test that edits the environment re-reads it with `refresh_env_knobs()`."""
    from glowq_amd.linear import refresh_env_knobs

    refresh_env_knobs()
    yield
    refresh_env_knobs()
