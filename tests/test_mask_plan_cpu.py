"""Properties of the mask plan (host restatement in tests/_plan_ref.py; the device plan is
compared with it in the GPU tests): the permutation is a stable partition, and a tile pair the
kernels skip never holds a kept element (soundness); tiles declared all-kept really are."""
import numpy as np
from hypothesis import given, settings, strategies as st

from oracle import attention_oracle as O
from tests import _plan_ref as P


@st.composite
def id_case(draw):
    M = draw(st.integers(1, 300))
    N = draw(st.integers(M, 400)) if draw(st.booleans()) else draw(st.integers(1, 400))
    seed = draw(st.integers(0, 2**31 - 1))
    style = draw(st.sampled_from(["packed", "random", "allglobal", "alllocal"]))
    rng = np.random.default_rng(seed)

    def ids(L):
        if style == "packed":
            x = -(np.cumsum(rng.random(L) < 0.05) + 1)
            x[rng.random(L) < 0.1] = 0
        elif style == "random":
            x = rng.integers(-4, 3, L)
        elif style == "allglobal":
            x = rng.integers(0, 3, L)
        else:
            x = -(np.cumsum(rng.random(L) < 0.1) + 1)
        return x.astype(np.int64)
    return M, N, ids(M), ids(N)


@settings(max_examples=60, deadline=None)
@given(id_case(), st.booleans())
def test_plan_is_sound(case, causal):
    M, N, eq, ek = case
    if causal and N < M:
        causal = False
    gap = max(0, N - M)
    perm, hdr, qs = P.plan_q(eq, M)
    ks = P.plan_k(ek, N)
    keep = O.keep_mask(M, N, causal, eq[None, None], ek[None, None], 1)[0, 0]
    # stable partition covering every row exactly once
    rows = perm[perm >= 0]
    assert sorted(rows.tolist()) == list(range(M))
    assert (np.diff(perm[:hdr["nL"]]) > 0).all() and (np.diff(perm[hdr["nLp"]:hdr["nLp"] + hdr["nG"]]) > 0).all()
    assert (eq[perm[:hdr["nL"]]] < 0).all() and (eq[perm[hdr["nLp"]:hdr["nLp"] + hdr["nG"]]] >= 0).all()
    assert hdr["nT128"] * 128 <= len(perm)
    for t, q in enumerate(qs):
        r = perm[t * 64:(t + 1) * 64]
        r = r[r >= 0]
        for kt, k in enumerate(ks):
            sub = keep[np.ix_(r, np.arange(kt * 64, min(N, (kt + 1) * 64)))] if len(r) else np.zeros((0, 1), bool)
            if not P.visits(q, k, kt, causal, gap):
                assert not sub.any(), "a skipped tile pair holds a kept element"
            elif P.all_keep(q, k) and len(r):
                # the doc test passes everywhere; only causal / tail masking may remove elements
                doc_only = O.keep_mask(M, N, False, eq[None, None], ek[None, None], 1)[0, 0]
                assert doc_only[np.ix_(r, np.arange(kt * 64, min(N, (kt + 1) * 64)))].all()


@settings(max_examples=40, deadline=None)
@given(id_case(), st.integers(0, 2**31 - 1))
def test_plan_is_sound_with_per_row_positions(case, seed):
    """The same soundness property when every row carries its own causal position (arbitrary, not
    even monotonic; -1 = the row sees nothing): summaries hold the smallest / largest position."""
    M, N, eq, ek = case
    rng = np.random.default_rng(seed)
    pos = rng.integers(-1, N + 3, M)
    perm, hdr, qs = P.plan_q(eq, M, pos)
    ks = P.plan_k(ek, N)
    keep = O.keep_mask(M, N, True, eq[None, None], ek[None, None], 1, qpos=pos[None])[0, 0]
    for t, q in enumerate(qs):
        r = perm[t * 64:(t + 1) * 64]
        r = r[r >= 0]
        for kt, k in enumerate(ks):
            if len(r) and not P.visits(q, k, kt, True, 0):
                assert not keep[np.ix_(r, np.arange(kt * 64, min(N, (kt + 1) * 64)))].any(), "a skipped tile pair holds a kept element"
