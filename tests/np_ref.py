"""Independent float32 numpy statements of the path's arithmetic, used to pin the
C oracle on small inputs.  Written from the behavioural description of the
reference (sequential left-to-right f32 accumulation, separately rounded multiply
and add, strict '<', first index wins), vectorised over (row, centroid) pairs
instead of looping over them, so that an indexing or ordering mistake in the C
oracle does not repeat here.
"""
import numpy as np

F = np.float32


def dist_matrix(metric, X, Cb):
    """All-pairs distances, (n, k) float32. metric in {'sq','euclid','cos','l1'}."""
    X = np.asarray(X, F)
    Cb = np.asarray(Cb, F)
    n, d = X.shape
    k = Cb.shape[0]
    if metric in ("sq", "euclid"):
        acc = np.zeros((n, k), F)
        for t in range(d):
            diff = X[:, t:t + 1] - Cb[None, :, t]
            acc = acc + diff * diff
        return np.sqrt(acc) if metric == "euclid" else acc
    if metric == "l1":
        acc = np.zeros((n, k), F)
        for t in range(d):
            acc = acc + np.abs(X[:, t:t + 1] - Cb[None, :, t])
        return acc
    if metric == "cos":
        dot = np.zeros((n, k), F)
        sa = np.zeros((n, 1), F)
        sb = np.zeros((1, k), F)
        for t in range(d):
            dot = dot + X[:, t:t + 1] * Cb[None, :, t]
            sa = sa + X[:, t:t + 1] * X[:, t:t + 1]
            sb = sb + Cb[None, :, t] * Cb[None, :, t]
        na, nb = np.sqrt(sa), np.sqrt(sb)
        den = na * nb
        with np.errstate(divide="ignore", invalid="ignore"):
            out = F(1.0) - dot / den
        out = np.where((na == 0) | (nb == 0), F(1.0), out).astype(F)
        return out
    raise ValueError(metric)


def argmin_first(Dm):
    """First index of the row minimum under strict '<' scanning (NaN never wins
    unless it sits at index 0)."""
    n, k = Dm.shape
    best = np.zeros(n, np.int64)
    bd = Dm[:, 0].copy()
    for j in range(1, k):
        upd = Dm[:, j] < bd
        best = np.where(upd, j, best)
        bd = np.where(upd, Dm[:, j], bd)
    return best


def mean_seq(rows):
    rows = np.asarray(rows, F)
    acc = np.zeros(rows.shape[1], F)
    for r in rows:
        acc = acc + r
    return acc / F(np.float64(rows.shape[0]))


def mean_tree(rows, leaf=1024):
    """The fixed midpoint tree used above 1024 members."""
    rows = np.asarray(rows, F)
    c = rows.shape[0]
    depth = 0
    while c > (leaf << depth):
        depth += 1

    def rec(lo, hi, dep):
        if dep == 0:
            acc = np.zeros(rows.shape[1], F)
            for r in rows[lo:hi]:
                acc = acc + r
            return acc
        mid = lo + (hi - lo) // 2
        return rec(lo, mid, dep - 1) + rec(mid, hi, dep - 1)

    return rec(0, c, depth) / F(np.float64(c))


def mean_parts(X, rows, part=4096, seq_max=1024):
    """The order used inside lbg_quantize: sequential up to 1024 members; above, per part of
    4096 consecutive row indices a sequential sum from 0, parts added in order from 0."""
    X = np.asarray(X, F)
    rows = np.asarray(rows, np.int64)
    c = len(rows)
    if c <= seq_max:
        return mean_seq(X[rows])
    acc = np.zeros(X.shape[1], F)
    for q in range((X.shape[0] + part - 1) // part):
        sel = rows[(rows >= q * part) & (rows < (q + 1) * part)]
        sub = np.zeros(X.shape[1], F)
        for r in sel:
            sub = sub + X[r]
        acc = acc + sub
    return acc / F(np.float64(c))


def lbg(X, k, max_iters, init_idx, reseed_stream):
    X = np.asarray(X, F)
    n = X.shape[0]
    cen = X[np.asarray(init_idx, np.int64)].copy()
    assign = np.zeros(n, np.int64)
    used = 0
    iters = 0
    for _ in range(max_iters):
        new = argmin_first(dist_matrix("sq", X, cen))
        changed = bool(np.any(new != assign))
        assign = new
        for j in range(k):
            mem = np.flatnonzero(assign == j)
            if len(mem):
                cen[j] = mean_parts(X, mem)
            else:
                cen[j] = X[int(reseed_stream[used])]
                used += 1
        iters += 1
        if not changed:
            break
    return cen, assign, iters, used
