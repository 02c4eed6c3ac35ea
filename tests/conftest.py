import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_package():
    """Import the product package (its directory name has a hyphen)."""
    if "legion_ibp_amd" in sys.modules:
        return sys.modules["legion_ibp_amd"]
    path = os.path.join(ROOT, "legion-ibp_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("legion_ibp_amd", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["legion_ibp_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lmi():
    return load_package()


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    binding.lib()
    return binding


def random_graph(rng, n_nodes, mean_deg, hubs=0, hub_deg=0, zero_frac=0.1):
    """Random multigraph CSR with a few zero-degree nodes and optional hubs."""
    deg = rng.poisson(mean_deg, n_nodes).astype(np.int64)
    deg[rng.random(n_nodes) < zero_frac] = 0
    if hubs:
        deg[rng.choice(n_nodes, hubs, replace=False)] = hub_deg
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n_nodes, int(indptr[-1])).astype(np.int32)
    return indptr, indices


def load_ipc_service():
    """Import the trainer-side consumer module of the product package."""
    name = "legion_ibp_amd_ipc_service"
    if name in sys.modules:
        return sys.modules[name]
    path = os.path.join(ROOT, "legion-ibp_amd", "ipc_service.py")
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod
