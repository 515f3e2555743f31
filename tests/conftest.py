"""Shared test plumbing: marker registration, package import, oracle import, GPU library handle."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_terminal_summary(terminalreporter):
    """The largest unscaled max-abs and rel-L2 each GPU parity test saw in its check() calls."""
    log = getattr(sys.modules.get("test_gpu_kernels"), "PARITY_LOG", None)
    if not log:
        return
    terminalreporter.write_sep("-", "parity: largest max-abs / rel-L2 per test (unscaled)")
    for test, (max_abs, rel, n) in log.items():
        terminalreporter.write_line(f"{max_abs:.3e}  {rel:.3e}  {n:4d} checks  {test}")


@pytest.fixture(scope="session")
def pkg():
    """The product package (its directory name has a hyphen, so it is imported through the entry module)."""
    import __graft_entry__ as entry

    return entry.import_package()


@pytest.fixture(scope="session")
def oracle():
    from oracle import raven_oracle

    return raven_oracle


@pytest.fixture(scope="session")
def lib(pkg):
    """The loaded C-ABI library; GPU tests fail (not skip) when it is missing."""
    return pkg.hip.load()


# defaults of the launch-shape knobs the tests change (raven_set_tuning); results never depend on them
TUNING_DEFAULTS = {"linear_ks": 0, "gemm_four_tiles": 1, "attn_wide": 0, "gemm_tiled_min_rows": 33, "gemm_tiled_variant": 0, "gemm_tiled_split_tail": 1, "prefill_waves": 0, "gemm_ragged": 1, "norm_early": -1, "fuse_sums_norm": 1, "attn_prefetch": 1, "fuse_qkv_rope": 1, "pad_chunk_rows": 1, "pad_decode_rows": 1, "attn_nosplit_pairs": 165, "attn_nosplit_len": 1536}


@pytest.fixture
def tuned(pkg):
    """tuned(key=value, ...) sets knobs for the rest of the test; all of them are back at their defaults afterwards, also
    when the test fails."""
    touched = set()

    def set_knobs(**knobs):
        for key, value in knobs.items():
            touched.add(key)
            pkg.hip.set_tuning(key, value)

    try:
        yield set_knobs
    finally:
        for key in touched:
            pkg.hip.set_tuning(key, TUNING_DEFAULTS[key])
