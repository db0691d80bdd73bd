import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def fixture_ids_mask():
    """The two data fixtures the reference ships (bloomz-7b/xinput.ids.bin and
    xinput.mask.bin): int32 little-endian [2, 512]."""
    ids = np.fromfile(os.path.join(GOLDEN, "xinput.ids.bin"), dtype="<i4").reshape(2, 512)
    mask = np.fromfile(os.path.join(GOLDEN, "xinput.mask.bin"), dtype="<i4").reshape(2, 512)
    return ids.astype(np.int32), mask.astype(np.int32)


def assert_close(got, ref, rtol, what="", ledger=None):
    """|got - ref| <= rtol * (|ref| + rms(ref)) elementwise: a relative bound
    with a floor tied to the tensor's own scale, so entries that are zero by
    cancellation do not demand infinite precision.  Works through the arrays in
    slices so that a gigabyte-sized gradient needs no fp64 copy of itself.
    Returns the worst error as a fraction of the bound; `ledger` (a dict)
    records it under `what`, so a test can print how far from the bound it ran."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    got = got.reshape(-1)
    ref = ref.reshape(-1)
    step = 1 << 24
    total = 0.0
    for i in range(0, ref.size, step):
        r = ref[i:i + step].astype(np.float64)
        total += float(np.dot(r, r))
    rms = float(np.sqrt(total / ref.size)) if ref.size else 0.0
    worst = 0.0
    for i in range(0, ref.size, step):
        g = got[i:i + step].astype(np.float64)
        r = ref[i:i + step].astype(np.float64)
        assert np.all(np.isfinite(g)), what + ": non-finite values"
        bound = rtol * (np.abs(r) + rms) + 1e-30
        worst = max(worst, float(np.max(np.abs(g - r) / bound)))
    if ledger is not None:
        ledger[what] = worst
    assert worst <= 1.0, "%s: worst error %.3g x the %.1e bound (rms %.3g)" % (
        what, worst, rtol, rms)
    return worst


def assert_rows_close(got, ref, rtol, what="", ledger=None):
    """Row by row: |got[r] - ref[r]|_2 <= rtol * |ref[r]|_2 -- a relative bound
    with no floor at all, for [rows, cols] tensors with so many entries (the
    tied table's gradient has a billion) that the largest single-entry error
    is an extreme-value statistic which any change of summation order moves by
    tens of percent, while a row's relative error is stable.  Rows whose
    reference is exactly zero must be exactly zero.  Returns / records the worst
    row's error as a fraction of the bound."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape and got.ndim == 2, (what, got.shape, ref.shape)
    worst = 0.0
    step = max(1, (1 << 24) // got.shape[1])
    for i in range(0, ref.shape[0], step):
        g = got[i:i + step].astype(np.float64)
        r = ref[i:i + step].astype(np.float64)
        assert np.all(np.isfinite(g)), what + ": non-finite values"
        norm = np.sqrt((r * r).sum(axis=1))
        err = np.sqrt(((g - r) ** 2).sum(axis=1))
        zero = norm == 0.0
        assert not np.any(err[zero] > 0.0), what + ": a row that must be zero is not"
        if np.any(~zero):
            worst = max(worst, float(np.max(err[~zero] / (rtol * norm[~zero]))))
    if ledger is not None:
        ledger[what] = worst
    assert worst <= 1.0, "%s: worst row error %.3g x the %.1e relative bound" % (what, worst, rtol)
    return worst


def print_ledger(title, ledger, top=6):
    """The largest error / bound ratios a test recorded, worst first."""
    rows = sorted(ledger.items(), key=lambda kv: -kv[1])[:top]
    print("%s: worst error as a fraction of the bound -- %s" % (
        title, ", ".join("%s %.2f" % (k, v) for k, v in rows)), flush=True)


@pytest.fixture(autouse=True)
def _release_device_temporaries(request):
    yield
    if request.node.get_closest_marker("gpu") is not None:
        import gpu_util
        gpu_util.release()


@pytest.fixture(scope="session")
def runtime():
    """Boots the C++ host runtime once per test process: on GPU 0 when one is
    visible, host-only otherwise (creating a "cuda" tensor then panics)."""
    import torch
    from blackriver_amd import host
    if not host.booted():
        host.boot(0 if torch.cuda.is_available() else -1, 1 << 30)
    return host
