import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session", autouse=True)
def _oracle_built():
    from oracle import oracle
    oracle.build()


@pytest.fixture(autouse=True)
def _default_kernel_policies(request):
    """The library's kernel-family switches are process-global: whatever a GPU test sets, the next test starts from the
    defaults again, also when the test failed half way."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    from llm_metal_amd import lib
    L = lib.load()
    L.hip_gemm_force_large_m(0)
    L.hip_gemm_large_m_split(1)
    L.hip_gemm_large_m_block(0)
    L.hip_gemm_ring(1)
    L.hip_gemm_ring_wide(1)
    L.hip_gemm_half_planes(1)
    L.hip_attention_flash(-1)
    L.hip_attention_backward_one_launch(1)
    L.hip_gemm_image_budget_mb(65536)
