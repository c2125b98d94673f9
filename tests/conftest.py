import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def _load_build():
    """``torchex_amd/_build.py`` loaded by path: importing the package itself needs the
    shared objects this module creates."""
    import importlib.util
    path = os.path.join(ROOT, "torchex_amd", "_build.py")
    spec = importlib.util.spec_from_file_location("_torchex_amd_build", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # a fresh checkout carries no shared objects: build the missing ones once
    _load_build().ensure_built()
    from oracle import c_oracle
    c_oracle.lib()


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this machine")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


_SPECIAL = {"NZ": -0.0, "NI": -np.inf, "PI": np.inf, "NAN": np.nan,
            "NFLTMAX": -float(np.finfo(np.float32).max)}


def _decode(x):
    if isinstance(x, list):
        return [_decode(v) for v in x]
    if isinstance(x, str):
        return _SPECIAL[x]
    return x


def load_hand_cases():
    with open(os.path.join(GOLDEN, "hand_cases.json")) as f:
        raw = json.load(f)["cases"]
    cases = []
    for c in raw:
        d = {"name": c["name"], "inv": np.array(c["inv"], dtype=np.int32)}
        for k, v in c.items():
            if k in ("name", "inv"):
                continue
            dt = np.int32 if k in ("arg", "arg_ref") else np.float32
            d[k] = np.array(_decode(v), dtype=dt)
        cases.append(d)
    return cases


def load_reference_counts():
    with open(os.path.join(GOLDEN, "reference_test_counts.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def hand_cases():
    return load_hand_cases()


@pytest.fixture(scope="session")
def reference_counts():
    return load_reference_counts()
