"""The C oracle against the committed golden fixtures (float64 library-routine outputs)."""
import glob
import os

import numpy as np
import pytest

from oracle import oracle_bwd, oracle_fwd

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def rel(a, b):
    return np.abs(a.astype(np.float64) - b).max() / max(np.abs(b).max(), 1e-30)


def test_fixtures_present():
    assert len(GOLDEN) >= 3


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_matches_golden(path):
    z = np.load(path)
    W, Himg, scale = int(z["WIDTH"]), int(z["HEIGHT"]), float(z["sm_scale"])
    out, _ = oracle_fwd(z["q"], z["k"], z["v"], z["coords"], W, Himg, scale)
    dq, dk, dv = oracle_bwd(z["q"], z["k"], z["v"], z["coords"], z["dout"], W, Himg, scale)
    assert rel(out, z["out"]) < 1e-5
    assert rel(dq, z["dq"]) < 1e-5
    assert rel(dk, z["dk"]) < 1e-5
    assert rel(dv, z["dv"]) < 1e-5
