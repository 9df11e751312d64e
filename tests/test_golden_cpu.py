"""The committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py) against
the oracle's independent routes: autograd through the closed form in fp64, and the tiled
restatement.  A change of the oracle that alters any stored answer fails here."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import attention_oracle as O

GOLDEN = sorted((Path(__file__).parent / "golden").glob("*.npz"))


def load(path):
    z = np.load(path, allow_pickle=False)
    d = {k: z[k] for k in z.files}
    d["keep"] = np.unpackbits(d["keep"], axis=-1, count=int(d["keep_shape"][-1])).astype(bool)
    return d


@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: p.stem)
def test_fixture_matches_oracle_routes(path):
    d = load(path)
    q, k, v, do = (torch.from_numpy(d[n]).double() for n in ("q", "k", "v", "do"))
    causal, doc = bool(d["causal"]), bool(d["doc"])
    eq = torch.from_numpy(d["eq"]) if doc else None
    ek = torch.from_numpy(d["ek"]) if doc else None
    M, N = q.shape[2], k.shape[2]
    mode = int(doc)
    if "block" in d:   # block mask: the map travels in the place of eq
        eq, mode = torch.from_numpy(d["block"]), 2
        d["eq"] = d["block"]
    keep = np.broadcast_to(O.keep_mask(M, N, causal, d.get("eq"), d.get("ek"), mode), d["keep"].shape)
    assert np.array_equal(keep, d["keep"])
    o, lse, dq, dk, dv = O.attention_autograd(q, k, v, do, causal, None, eq, ek, mode, dtype=torch.float64)
    for name, got in (("o", o), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert np.allclose(got.numpy(), d[name], atol=1e-10), name
    if "block" not in d:   # the tiled restatement knows the reference's two score modes
        Ot, L2, dQ, dK, dV = O.attention_tiled(d["q"], d["k"], d["v"], d["do"], causal, 1 / np.sqrt(q.shape[-1]),
                                               d.get("eq"), d.get("ek"), int(doc), 8, 16)
        assert np.allclose(Ot, d["o"], atol=1e-10) and np.allclose(dK, d["dk"], atol=1e-10)
        assert np.allclose(dQ, d["dq"], atol=1e-10) and np.allclose(dV, d["dv"], atol=1e-10)
