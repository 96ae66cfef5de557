"""The golden fixtures are the oracle's output, frozen: the oracle must still reproduce them exactly
(inputs bit for bit, expected outputs to fp64 round-off)."""
import glob
import importlib.util
import os

import numpy as np

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _generator():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_fixture_is_reproduced_by_the_oracle():
    gen = _generator()
    seen = set()
    for name, inputs, expected in gen.cases():
        f = np.load(os.path.join(HERE, name + ".npz"))
        seen.add(name + ".npz")
        for k, v in inputs.items():
            assert np.array_equal(f["in_" + k], gen.store(v)), (name, k)
        for k, v in expected.items():
            a, b = f["out_" + k], v.detach().double().numpy()
            assert a.shape == b.shape and np.allclose(a, b, rtol=1e-10, atol=1e-12 * max(1.0, float(np.abs(a).max()))), (name, k)
    assert seen == {os.path.basename(p) for p in glob.glob(os.path.join(HERE, "*.npz"))}
