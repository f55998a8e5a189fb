import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_lib
    oracle_lib.lib()
    return oracle_lib


@pytest.fixture(scope="session")
def aclnn():
    from ops_cv_amd import aclnn as a
    a.load_library()
    return a


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: the HIP path has no CPU fallback")
    return torch.device("cuda:0")


OPTION_NAMES = ("gs_variant", "resize_variant", "nearest_variant", "reference_cores", "reference_ub_bytes",
                "grid_sampler2d_rule", "gs3d_grad_variant")


@pytest.fixture(autouse=True)
def _library_options_restored():
    """The library's process-wide options (opscvSetOption) are put back after every test that changed them."""
    try:
        from ops_cv_amd import aclnn as a
        a.load_library()
    except Exception:  # the library is not built: the tests that need it fail on their own
        yield
        return
    saved = {n: a.get_option(n) for n in OPTION_NAMES}
    yield
    for n, v in saved.items():
        a.set_option(n, v)
