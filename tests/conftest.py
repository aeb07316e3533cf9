import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture
def cu_count():
    """Setter that sizes one-block-per-CU grids for n compute units (the device's own count again after the test)."""
    from tyloquant_amd import _lib as L
    yield L.lib().mfq_hip_set_cu_count
    L.lib().mfq_hip_set_cu_count(0)


def rel_l2(a, b):
    import numpy as np
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    n = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / n) if n > 0 else float(np.linalg.norm(a - b))


# BASELINE tolerance for matmul outputs against the fp32 dequant-then-matmul oracle
REL_TOL = 1e-3
ABS_TOL = 1e-2


def check_close(y, ref):
    """rel-L2 <= 1e-3 and max-abs <= 1e-2; the absolute bound is stated for outputs of order one
    (the BASELINE configs), so packed-domain fixtures with larger outputs scale it by their RMS."""
    import numpy as np
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rel = rel_l2(y, ref)
    assert rel < REL_TOL, f"rel-L2 {rel:.3e}"
    bound = ABS_TOL * max(1.0, float(np.sqrt(np.mean(ref * ref))))
    err = float(np.abs(y - ref).max())
    assert err < bound, f"max-abs {err:.3e} (bound {bound:.3e})"
