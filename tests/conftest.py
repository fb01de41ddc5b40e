"""Shared test plumbing: the `gpu` marker, import paths for the host binding (dlspm-esimd_amd/dlspm_hip.py)
and the CPU oracle (oracle/oracle.py), and small helpers to build seeded problems."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("dlspm-esimd_amd", "oracle"):
    p = os.path.join(ROOT, sub)
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc

    orc.lib()  # builds oracle/libdlspm_oracle.so with gcc on first use if it is missing
    return orc


@pytest.fixture(scope="session")
def dl():
    import dlspm_hip

    return dlspm_hip


@pytest.fixture(autouse=True)
def _rules_after_every_test():
    """Tests that override the launch rules (dl.set_tuning) must not leak the override into the next test."""
    yield
    import dlspm_hip

    if dlspm_hip._lib is not None:
        dlspm_hip.set_tuning()


def random_csr(rng, M, K, kind="uniform", density=0.1):
    """Seeded CSR pattern with ascending unique columns. kind: uniform | skewed | empty_rows | full | empty."""
    if kind == "uniform":
        lens = rng.binomial(K, density, size=M)
    elif kind == "skewed":
        lens = np.minimum(K, np.round(np.exp(rng.normal(np.log(max(density * K, 1.0)), 1.0, size=M))).astype(np.int64))
    elif kind == "empty_rows":
        lens = rng.binomial(K, density, size=M) * (rng.random(M) < 0.5)
    elif kind == "full":
        lens = np.full(M, K)
    elif kind == "empty":
        lens = np.zeros(M, dtype=np.int64)
    else:
        raise ValueError(kind)
    lens = np.clip(lens, 0, K).astype(np.int64)
    ro = np.zeros(M + 1, dtype=np.int32)
    ro[1:] = np.cumsum(lens)
    ci = np.empty(int(ro[-1]), dtype=np.int32)
    for i in range(M):
        k = int(lens[i])
        if k:
            ci[ro[i]:ro[i + 1]] = np.sort(rng.choice(K, size=k, replace=False))
    return ro, ci
