import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden.npz"))


@pytest.fixture(scope="session")
def golden_12d():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_12d.npz"))


@pytest.fixture(scope="session")
def golden_i32():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_i32.npz"))


@pytest.fixture(scope="session")
def golden_64():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_64.npz"))


@pytest.fixture(scope="session")
def digests():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "zfp_digests.json")) as fh:
        return json.load(fh)


def golden_cases(g):
    """Yield (name, rate, maxbits, field, stream_bytes, decoded) for every fixture."""
    import numpy as np

    names = sorted({k.split("/")[0] for k in g.files})
    for n in names:
        f = g[n + "/in"]
        for k in sorted(g.files):
            if k.startswith(n + "/r") and k.endswith("/stream"):
                rate = float(k.split("/")[1][1:])
                maxbits = int(np.floor(4 ** f.ndim * rate + 0.5))   # bits per block of 4^d values
                yield n, rate, maxbits, f, g[k], g[k[: -len("stream")] + "dec"]
