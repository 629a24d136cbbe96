"""Shared fixtures.  `-m "not gpu"` tests cover the oracle, the host logic and the C-ABI's
symbol table; `-m gpu` tests are the parity tests proper and call through the C ABI."""
import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP path through the C ABI)")


def load_package():
    """The package directory is named `light-tensor_amd`; import it as light_tensor_amd."""
    if "light_tensor_amd" in sys.modules:
        return sys.modules["light_tensor_amd"]
    pkg_dir = os.path.join(ROOT, "light-tensor_amd")
    spec = importlib.util.spec_from_file_location("light_tensor_amd", os.path.join(pkg_dir, "__init__.py"),
                                                  submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["light_tensor_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def lt():
    return load_package()


@pytest.fixture(scope="session")
def wl(lt):
    from light_tensor_amd import workloads
    return workloads


@pytest.fixture(scope="session")
def ob():
    from oracle import bindings
    bindings.oracle()
    return bindings


@pytest.fixture(scope="session")
def gpu(lt):
    """Initialised HIP library on device 0; a missing library or device is a failure, not a skip."""
    lt.init(0)
    yield lt
    lt.set_option("qgemm_tile", 0)
    lt.set_option("qskinny", 0)


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before any GPU work starts, so a run that dies still says where
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


GOLDEN = os.path.join(ROOT, "tests", "golden")


def golden_path(name):
    return os.path.join(GOLDEN, name)


def exact_acc(A, B, zpA, zpB):
    """sum_k (A-zpA)(B-zpB) for A[M,K], B[N,K], exact: every product and sum fits a double."""
    return ((A.astype(np.float64) - float(zpA)) @ (B.astype(np.float64) - float(zpB)).T).astype(np.int64)


def requant_numpy(acc, mult, zp):
    """The five-step requantize of l-ten/math_fns.cpp:1474 on arrays (|s| < 2^31 assumed)."""
    s = (acc.astype(np.float32) * np.float32(mult)).astype(np.float32) + np.float32(zp)
    return (np.trunc(s.astype(np.float32)).astype(np.int64) & 0xFF).astype(np.uint8)


def rel_err(got, want):
    """The fp32 error measure used throughout: max |got - want| / max(|want|, rms(want)).
    Outputs smaller than the typical output magnitude (cancellation) are measured against that
    magnitude; no fp32 summation order can promise a relative bound on them."""
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    floor = max(float(np.sqrt(np.mean(want * want))), 1e-30)
    return float((np.abs(got - want) / np.maximum(np.abs(want), floor)).max()) if want.size else 0.0
