"""The caller side against a float64 torch shadow, on the CPU: random programs of softmax, maxima, mean / variance,
LayerNorm, RMS, Linear, in-place tensor updates, attention and wide Concats (tests/fuzz_models.py) run through the
oracle -- so through adhip.core's graph nodes, their backward rules and the command stream they emit -- and compared
with the same computation written with torch's own functions, which shares no code with them.  A front-end mistake
(a wrong backward rule, a reduction along the wrong dim, a broadcast that lands on the wrong axis) is invisible to a
device-against-oracle comparison, because both execute the same commands; this is where it shows."""
import math

import numpy as np
import pytest

from oracle.interp import OracleDevice


@pytest.mark.parametrize("scale,seed", [(1, s) for s in range(40)] + [(4, s) for s in range(10)] + [(16, 0), (16, 1)])
def test_caller_side_matches_float64_shadow(scale, seed):
    from fuzz_models import random_model_program, shadow_model_program
    oracle = OracleDevice()
    ref = random_model_program(oracle, seed, scale)
    exact = shadow_model_program(seed, scale)
    assert len(ref) >= 4 and "target" in ref
    tol = 1e-5 * math.sqrt(oracle.max_terms) * 2
    largest = max(float(np.max(np.abs(x))) for x in exact.values())
    compared = 0
    for k, rv in ref.items():
        if k not in exact:
            continue  # the gradient of a leaf that the shadow holds as a constant
        assert list(exact[k].shape) == rv.dim, (k, exact[k].shape, rv.dim)
        e = exact[k].ravel()
        err = float(np.max(np.abs(np.asarray(rv.data, np.float64) - e)))
        assert err <= tol * max(float(np.max(np.abs(e))), 1e-3 * largest), (scale, seed, k, err)
        compared += 1
    assert compared >= 4


def test_every_building_block_is_drawn():
    """Over the seeds the tests use, each kind of operation of the generator produces a value at least once (a kind
    that silently never applies would test nothing)."""
    from adhip import ir as IR
    from adhip.core import ValueData
    from adhip.device import Device
    from fuzz_models import random_model_program

    class Capture(Device):
        def execute(self, proc, deps):
            self.proc = proc

        def get_tensor(self, id):
            return ValueData([1], np.zeros(1, np.float32), id, False)

    seen = set()
    for seed in range(40):
        dev = Capture()
        random_model_program(dev, seed, 4)
        seen |= {type(c).__name__ for c in dev.proc.walk()}
    assert {"Max", "Sum", "DotProduct", "Concat", "ElwAddEq", "ElwMultiplyEq", "Exp2", "Sqrt", "Recip", "Sin", "Broadcast", "Permute"} <= seen
