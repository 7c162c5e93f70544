"""float64 numpy restatements used as independent references at sizes the C oracle would take minutes for.

attention_slice: one (batch, head) slice of causal attention, forward and backward, written from the textbook formulas
(softmax(Q K^T scale + mask) V; dV = P^T dO; dP = dO V^T; dS = P (dP - rowsum(P dP)); dQ = scale dS K; dK = scale dS^T Q).
It is itself pinned against the C oracle on small shapes by tests/test_oracle_math.py.
"""
import numpy as np


def attention_slice(q, k, v, go, scale, old_len=0):
    """q, go: [newLen, hd]; k, v: [totalLen, hd] -> O, m, l, dQ, dK, dV in float64."""
    q, k, v, go = (np.asarray(t, np.float64) for t in (q, k, v, go))
    new_len, total = q.shape[0], k.shape[0]
    s = (q @ k.T) * scale
    visible = np.arange(total)[None, :] <= old_len + np.arange(new_len)[:, None]
    s = np.where(visible, s, -np.inf)
    m = s.max(-1)
    p = np.exp(s - m[:, None])
    l = p.sum(-1)
    p /= l[:, None]
    o = p @ v
    dv = p.T @ go
    dp = go @ v.T
    ds = p * (dp - (p * dp).sum(-1, keepdims=True))
    dq = (ds @ k) * scale
    dk = (ds.T @ q) * scale
    return o, m, l, dq, dk, dv
