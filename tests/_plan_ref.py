"""Host restatement of the device mask plan (csrc/fa_aux.hip) for the tests:
permutation (local rows first, then global rows), per-64 summaries of both sides,
and the tile-pair visit predicate the kernels apply."""
import numpy as np

SUM = 64
INT_MAX, INT_MIN = 2**31 - 1, -2**31


def plan_q(eq, M, pos=None):
    """eq: int array [M]; pos: key position of every row's diagonal (default: the row index, to which
    visits() adds the causal gap; the device plan stores gap + row, or the caller's per-row positions).
    Returns perm [Pp], header dict, summaries list of dicts (rmin / rmax over the positions)."""
    pos = np.arange(M) if pos is None else np.asarray(pos)
    Pp = (M + 255) // 256 * 256 + 256
    local = np.nonzero(eq < 0)[0]
    glob = np.nonzero(eq >= 0)[0]
    nL, nG = len(local), len(glob)
    nLp = (nL + 255) // 256 * 256
    perm = np.full(Pp, -1, np.int64)
    perm[:nL] = local
    perm[nLp:nLp + nG] = glob
    sums = []
    for t in range(Pp // SUM):
        rows = perm[t * SUM:(t + 1) * SUM]
        rows = rows[rows >= 0]
        ids = eq[rows]
        loc = ids[ids < 0]
        sums.append(dict(lo=int(loc.min()) if len(loc) else INT_MAX, hi=int(loc.max()) if len(loc) else INT_MIN,
                         glob=int((ids >= 0).any()), rmin=int(pos[rows].min()) if len(rows) else INT_MAX,
                         rmax=int(pos[rows].max()) if len(rows) else -1, nvalid=len(rows)))
    hdr = dict(nL=nL, nG=nG, nLp=nLp, nT128=(nLp + (nG + 127) // 128 * 128) // 128)
    return perm, hdr, sums


def first_local_key_tile(qsums, ksums, causal, gap):
    """Header field k0: the first key tile that any summary entry of local rows visits (INT_MAX: none)."""
    k0 = INT_MAX
    for s in qsums:
        if s["nvalid"] and not s["glob"]:
            cand = [kt for kt, k_ in enumerate(ksums) if visits(s, k_, kt, causal, gap)]
            if cand:
                k0 = min(k0, cand[0])
    return k0


def plan_k(ek, N):
    sums = []
    for t in range((N + SUM - 1) // SUM):
        ids = ek[t * SUM:min(N, (t + 1) * SUM)]
        sums.append(dict(lo=int(ids.min()), hi=int(ids.max())))
    return sums


def may_keep(q, k):
    return bool(q["glob"]) or (q["lo"] <= k["hi"] and k["lo"] <= q["hi"])


def all_keep(q, k):
    return q["lo"] > q["hi"] or (q["lo"] == q["hi"] and k["lo"] == k["hi"] and q["lo"] == k["lo"])


def visits(qs, ks, kt, causal, gap):
    """Does the kernel visit (query summary qs, key tile index kt with summary ks)?"""
    if qs["nvalid"] == 0:
        return False
    if causal and kt * SUM > gap + qs["rmax"]:
        return False
    return may_keep(qs, ks)
