import importlib
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu on the GPU box")


# The parity bound of the path: max relative error 1e-4 for floating point, bit-exact for
# indices. "Relative" is |got - want| / max(|want|, rms(want)): an element much smaller than
# the tensor's typical magnitude (a sum that happens to cancel) is measured against that
# magnitude, not against itself.
REL_TOL = 1e-4


def rel_err(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if got.size == 0:
        return 0.0
    scale = np.maximum(np.abs(want), np.sqrt(np.mean(want * want)) + 1e-30)
    return float(np.max(np.abs(got - want) / scale))


# The plain element-wise figure, reported beside the gate: |got - want| / max(|want|, floor)
# with the absolute floor ELEMENTWISE_FLOOR * rms(want) (without a floor an element that is
# exactly zero in the reference makes the figure infinite).
ELEMENTWISE_FLOOR = 1e-3


def elementwise_rel_err(got, want, floor=ELEMENTWISE_FLOOR):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    if got.size == 0:
        return 0.0
    scale = np.maximum(np.abs(want), floor * np.sqrt(np.mean(want * want)) + 1e-300)
    return float(np.max(np.abs(got - want) / scale))


# Every comparison of a run leaves its figures here; a GPU run writes the maxima per test to
# gpurun_out/parity_summary.json when the session ends (passing runs included).
_PARITY_LOG = {}
_CURRENT_TEST = [""]


@pytest.fixture(autouse=True)
def _name_the_running_test(request):
    _CURRENT_TEST[0] = request.node.nodeid
    yield
    _CURRENT_TEST[0] = ""


def pytest_sessionfinish(session, exitstatus):
    if not _PARITY_LOG:
        return
    out_dir = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        worst = max(_PARITY_LOG.values(), key=lambda r: r["gate_max"])
        worst_plain = max(_PARITY_LOG.values(), key=lambda r: r["elementwise_max"])
        with open(os.path.join(out_dir, "parity_summary.json"), "w") as f:
            json.dump({"gate": "|got-want| / max(|want|, rms(want))", "tolerance": REL_TOL,
                       "elementwise": f"|got-want| / max(|want|, {ELEMENTWISE_FLOOR:g}*rms(want))",
                       "comparisons": sum(r["comparisons"] for r in _PARITY_LOG.values()),
                       "worst_gate": {"test": worst["test"], "what": worst["gate_what"], "value": worst["gate_max"]},
                       "worst_elementwise": {"test": worst_plain["test"], "what": worst_plain["elementwise_what"],
                                             "value": worst_plain["elementwise_max"]},
                       "tests": sorted(_PARITY_LOG.values(), key=lambda r: -r["elementwise_max"])}, f, indent=1)
    except OSError:
        pass


def assert_close(got, want, tol=REL_TOL, what=""):
    e = rel_err(got, want)
    plain = elementwise_rel_err(got, want)
    rec = _PARITY_LOG.setdefault(_CURRENT_TEST[0], {"test": _CURRENT_TEST[0], "comparisons": 0, "gate_max": 0.0,
                                                    "gate_what": "", "elementwise_max": 0.0,
                                                    "elementwise_what": "", "tolerance_max": 0.0})
    rec["comparisons"] += 1
    rec["tolerance_max"] = max(rec["tolerance_max"], tol)
    if e >= rec["gate_max"]:
        rec["gate_max"], rec["gate_what"] = e, what
    if plain >= rec["elementwise_max"]:
        rec["elementwise_max"], rec["elementwise_what"] = plain, what
    assert e <= tol, (f"{what}: relative error {e:.3e} > {tol:g} (plain element-wise, floor "
                      f"{ELEMENTWISE_FLOOR:g}*rms: {elementwise_rel_err(got, want):.3e})")


@pytest.fixture(scope="session")
def O():
    """The CPU oracle (test infrastructure)."""
    from oracle import oracle
    oracle.oracle_lib()
    return oracle


@pytest.fixture(scope="session")
def W():
    return importlib.import_module("tiny-cnn_amd.workloads")


@pytest.fixture(scope="session")
def T():
    """The product binding, device initialised (GPU tests only)."""
    mod = importlib.import_module("tiny-cnn_amd")
    mod.init(0)
    return mod


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(GOLDEN, "reference_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def layer_grads():
    return np.load(os.path.join(GOLDEN, "layer_grads.npz"))


@pytest.fixture(scope="session")
def act_golden():
    return np.load(os.path.join(GOLDEN, "activations.npz"))


@pytest.fixture(scope="session")
def norm_golden():
    return np.load(os.path.join(GOLDEN, "norm.npz"))


@pytest.fixture(scope="session")
def net_steps():
    return np.load(os.path.join(GOLDEN, "net_steps.npz"))


def load_net_params(net_like, params, setter):
    for (i, which, a) in params:
        setter(net_like, i, which, a)


def input_checksum(x, t, params):
    return float(sum(np.asarray(a, np.float64).sum() for a in [x, t] + [p for _, _, p in params]))
