"""pytest configuration: import path for the in-tree package and the `gpu` marker."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "jax-js_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


# JAXHIP_SEED_SHIFT=<n> adds n to every integer seed the tests hand to numpy.random.default_rng: the same tests on
# other random data (shapes a test draws from its generator change with it).  Unset or 0: the committed data.
_SHIFT = int(os.environ.get("JAXHIP_SEED_SHIFT", "0"))
if _SHIFT:
    import numpy as _np

    _default_rng = _np.random.default_rng
    _np.random.default_rng = lambda seed=None: _default_rng(seed + _SHIFT if isinstance(seed, int) else seed)
