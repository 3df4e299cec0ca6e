"""Seeded random problems through the AUTO regime: row counts across every regime boundary, K that
is not a multiple of the weight tile, N that is not a multiple of any output tile, every group size
family, both weight widths and activation types, optional inputs drawn independently.  Each case is
checked against the float64 oracle at the usual 1e-2 bar (global and per-column norm).  The shapes
are small enough for the CPU oracle; what they add to the hand-picked cases of the other files is the
combinations nobody thought of."""
import numpy as np
import pytest

from _util import parity_err, random_problem, run_product

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.choice([4, 8]))
    group = int(rng.choice([0, 64, 128, 128, 192, 256]))
    dtype = str(rng.choice(["bf16", "fp16"]))
    m = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 24, 33, 64, 65, 100, 129, 200, 257, 300, 520]))
    tiles = int(rng.integers(1, 10))
    k = 64 * tiles if group in (0, 64) else (128 * tiles if group == 128 else 64 * max(tiles, group // 64))
    if group in (64, 128) and k % group:
        k += group - k % group
    n = 16 * int(rng.integers(1, 60))
    zero = bool(rng.integers(0, 2)) and group != 0
    return dict(M=m, K=k, N=n, bits=bits, group=group, dtype=dtype, zero=zero, bias=bool(rng.integers(0, 2)),
                pqs=bool(rng.integers(0, 2)), seed=seed)


@pytest.mark.parametrize("seed", range(48))
def test_random_problem_auto_regime(pkg, oracle, dev, seed):
    c = _case(seed)
    p = random_problem(oracle, c["M"], c["K"], c["N"], c["bits"], c["group"], c["dtype"], zero=c["zero"],
                       bias=c["bias"], pqs=c["pqs"], seed=c["seed"])
    out = run_product(pkg, oracle, dev, p, 0)
    assert np.isfinite(out).all(), c
    err = parity_err(oracle, out, p)
    assert err < TOL, (c, err, (pkg._lib.lib.woq_last_launch() or b"").decode())
