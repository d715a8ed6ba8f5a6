import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _conv_mode_fixture(mode):
    @pytest.fixture
    def fixture():
        """Runs the test with nn.SpatialConvolutionMM on one route, then restores the library's mode."""
        import mcw_cppamp_torch_amd as pkg
        lib = pkg._lib.lib
        before = lib.thgpu_conv_get_mode()
        assert lib.thgpu_conv_set_mode(mode) == 0
        yield
        assert lib.thgpu_conv_set_mode(before) == 0
    return fixture


columns_route = _conv_mode_fixture(0)    # im2col / GEMM / col2im: finput and fgradInput hold columns
gathered_route = _conv_mode_fixture(2)   # gathered GEMMs wherever the shape fits


@pytest.fixture
def switches():
    """Sets testing switches of the library (thgpu_debug_set) for one test; the library's own choices are restored
    afterwards.  Usage: switches("gemm_tile", "128x128")."""
    import mcw_cppamp_torch_amd as pkg
    lib = pkg._lib.lib
    used = []

    def set_switch(name, value):
        used.append(name)
        rc = lib.thgpu_debug_set(name.encode(), None if value is None else str(value).encode())
        assert rc == 0, lib.thgpu_last_error()

    yield set_switch
    for name in used:
        assert lib.thgpu_debug_set(name.encode(), None) == 0
