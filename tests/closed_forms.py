"""Brute-force closed forms of the attention patterns, one query row at a time, in fp64.

Independent of oracle/t5_basic.py's blocked evaluation: each row's live keys and
bias buckets are enumerated from the index formulas, the softmax is done in
numpy.  Only for tiny inputs.
"""
import math

import numpy as np


def bucket(rel, bidirectional=True, nb=32, md=128):
    out = 0
    if bidirectional:
        nb //= 2
        if rel > 0:
            out += nb
        d = abs(rel)
    else:
        d = max(-rel, 0)
    me = nb // 2
    if d < me:
        return out + d
    x = math.log(d / me) / math.log(md / me) * (nb - me)
    r = round(x)
    if abs(x - r) < 1e-9:
        x = r
    return out + min(me + int(x), nb - 1)


def _row(qrow, keys, vals, biases):
    """softmax(q.k + bias) @ v for one query row; keys/vals lists of vectors."""
    if not keys:
        return np.zeros_like(qrow)
    K = np.stack(keys).astype(np.float64)
    V = np.stack(vals).astype(np.float64)
    s = K @ qrow.astype(np.float64) + np.asarray(biases, dtype=np.float64)
    s -= s.max()
    p = np.exp(s)
    return (p / p.sum()) @ V


def dense(q, k, v, table, causal=False, sm_scale=1.0, nb=32, md=128):
    """q (H,M,D), k/v (H,N,D), table (nb,H) or None.  rel = j - (i + N - M); causal: j <= i + N - M."""
    H, M, D = q.shape
    N = k.shape[1]
    out = np.zeros((H, M, D))
    for h in range(H):
        for i in range(M):
            ip = i + N - M
            js = [j for j in range(N) if (not causal or j <= ip)]
            bs = [0.0 if table is None else table[bucket(j - ip, not causal, nb, md), h] for j in js]
            out[h, i] = _row(q[h, i] * sm_scale, [k[h, j] for j in js], [v[h, j] for j in js], bs)
    return out


def local(q, k, v, table, Bl, nb=32, md=128):
    """keys {j: |j-i| < Bl}, bias T[b(j-i)]."""
    H, L, D = q.shape
    out = np.zeros((H, L, D))
    for h in range(H):
        for i in range(L):
            js = [j for j in range(L) if abs(j - i) < Bl]
            bs = [0.0 if table is None else table[bucket(j - i, True, nb, md), h] for j in js]
            out[h, i] = _row(q[h, i], [k[h, j] for j in js], [v[h, j] for j in js], bs)
    return out


def block(q, k, v, table, Bl, G, nb=32, md=128):
    """Reference-faithful block attention with G global tokens (all-ones mask).

    i < G: all keys, bias T[b(j-i)].  i >= G, blk=i//Bl, r=i%Bl: key list
    [G global tokens | Bl tokens of the own block (zero vectors past L)];
    list column c has bias T[b(c-(G+r))]; in block 0 columns [Bl, Bl+G) are dead.
    """
    H, L, D = q.shape
    out = np.zeros((H, L, D))
    if L < Bl:
        return dense(q, k, v, table, False, 1.0, nb, md)
    zero = np.zeros(D)
    for h in range(H):
        for i in range(L):
            if i < G:
                js = list(range(L))
                bs = [0.0 if table is None else table[bucket(j - i, True, nb, md), h] for j in js]
                out[h, i] = _row(q[h, i], [k[h, j] for j in js], [v[h, j] for j in js], bs)
                continue
            blk, r = divmod(i, Bl)
            ks, vs, bs = [], [], []
            for c in range(G + Bl):
                if blk == 0 and c >= Bl:
                    continue
                tok = c if c < G else blk * Bl + (c - G)
                ks.append(k[h, tok] if tok < L else zero)
                vs.append(v[h, tok] if tok < L else zero)
                bs.append(0.0 if table is None else table[bucket(c - (G + r), True, nb, md), h])
            out[h, i] = _row(q[h, i], ks, vs, bs)
    return out


def tglobal(q, k, v, sk, sv, table, Bl, gbs, nb=32, md=128):
    """local(Bl) keys plus side tokens g in [0, L//gbs) with bias T[b(g - i//gbs)] (L % gbs == 0)."""
    H, L, D = q.shape
    Gn = sk.shape[1]
    out = np.zeros((H, L, D))
    for h in range(H):
        for i in range(L):
            js = [j for j in range(L) if abs(j - i) < Bl]
            ks = [k[h, j] for j in js] + [sk[h, g] for g in range(Gn)]
            vs = [v[h, j] for j in js] + [sv[h, g] for g in range(Gn)]
            bs = [0.0 if table is None else table[bucket(j - i, True, nb, md), h] for j in js]
            bs += [0.0 if table is None else table[bucket(g - i // gbs, True, nb, md), h] for g in range(Gn)]
            out[h, i] = _row(q[h, i], ks, vs, bs)
    return out
