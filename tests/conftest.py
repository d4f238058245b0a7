import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "flux2.c_amd"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: CPU test that takes minutes (opt in with FLUX_SLOW=1)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle as O
    O.enable_blas()
    return O


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


@pytest.fixture(autouse=True, scope="module")
def _default_switches(request):
    """The switches of include/flux_hip_debug.h are process-wide: every GPU test module starts from the
    defaults, whatever an earlier module (or a failed assertion in it) left behind."""
    mark = getattr(request.module, "pytestmark", None)
    marks = list(mark) if isinstance(mark, (list, tuple)) else [mark] if mark is not None else []
    if not any(getattr(m, "name", "") == "gpu" for m in marks):
        yield
        return
    import fluxhip
    L = fluxhip.lib()

    def restore():
        L.flux_hip_linear_force_tile(-1)
        L.flux_hip_linear_tile_mask(0)
        L.flux_hip_linear_enable_splitk(1)
        L.flux_hip_linear_force_split(0)
        L.flux_hip_linear_persistent(1)
        L.flux_hip_linear_ring(1)
        L.flux_hip_attention_force_variant(-1)
        L.flux_hip_set_batched_cfg(1)
        L.flux_hip_set_fused_qkv_mlp(1)
        L.flux_hip_vae_set_attention_chunk(0)
        L.flux_hip_linear_probe(-1)
    restore()
    yield
    restore()
