"""wait(timeout) of the backend's Work without a GPU: a Work that is not backed by device work
answers isCompleted() "not yet" a given number of times (or for good).  The contract is the
reference's synchronizeInternal (src/utils.h:295-319): in blocking mode wait polls until the work
is complete, and raises "Caught collective operation timeout" once the work has run for longer than
the timeout passed in -- or than the timeout the work was created with when none is passed."""
import datetime
import os
import sys
import time

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "torch-ccl_amd"))


@pytest.fixture(scope="module")
def backend_module():
    import torch_ccl_amd  # noqa: F401  (fails loudly when the extension is not built)
    from torch_ccl_amd import _C
    return _C


def test_wait_raises_at_the_timeout_passed_in(backend_module):
    w = backend_module._pending_work(3, -1, datetime.timedelta(seconds=60))
    t0 = time.monotonic()
    with pytest.raises(RuntimeError, match=r"\[Rank 3\] Caught collective operation timeout:  ran for \d+ milliseconds"):
        w.wait(datetime.timedelta(milliseconds=200))
    waited = time.monotonic() - t0
    assert 0.15 < waited < 5.0, waited  # not before the limit, and nowhere near the 60 s of the work itself
    assert not w.is_completed()


def test_wait_without_a_timeout_uses_the_one_of_the_work(backend_module):
    w = backend_module._pending_work(0, -1, datetime.timedelta(milliseconds=250))
    t0 = time.monotonic()
    with pytest.raises(RuntimeError, match="Caught collective operation timeout"):
        w.wait()
    assert 0.2 < time.monotonic() - t0 < 5.0


def test_wait_returns_when_the_work_completes_in_time(backend_module):
    w = backend_module._pending_work(1, 5000, datetime.timedelta(seconds=60))
    assert not w.is_completed()
    assert w.wait(datetime.timedelta(seconds=30)) is True
    assert w.is_completed()
    assert w.is_success()
