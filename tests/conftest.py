import os
import sys

import pytest

# the library reads its environment switches once per process; the tests flip them between calls
os.environ.setdefault("ZMI_ENV_LIVE", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def zo():
    """The CPU oracle (built on first use)."""
    from oracle import build, oracle
    build.build(force=False)
    return oracle


@pytest.fixture(autouse=True)
def _fresh_weight_cache(request):
    """The packed-weight cache is keyed by weight address (as the reference's is)
    and is_weights_const promises that address keeps its contents.  Tests free
    and reallocate weights at recycled addresses, so each GPU test starts with
    an empty cache."""
    yield
    if request.node.get_closest_marker("gpu") is not None:
        from zendnn_amd import capi
        capi.load().zmi_clear_weight_cache()


@pytest.fixture(params=["decode", "smallm"])
def small_m_kernel(request):
    """Problems of 17 .. 128 rows run on the decode kernel (16-row groups) when K fits its LDS and
    on the small-M kernel otherwise; tests that use this fixture run once on each."""
    old = os.environ.get("ZMI_DECODE_MAX_M")
    if request.param == "smallm":
        os.environ["ZMI_DECODE_MAX_M"] = "16"
    else:
        os.environ.pop("ZMI_DECODE_MAX_M", None)
    yield request.param
    if old is None:
        os.environ.pop("ZMI_DECODE_MAX_M", None)
    else:
        os.environ["ZMI_DECODE_MAX_M"] = old
