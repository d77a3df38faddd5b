"""Independent numpy statement of GQA attention, written from the mathematics
(float64 softmax over explicitly gathered heads), sharing no code with the C
oracle.  Used only to pin the oracle."""
import numpy as np


def attention_rows(q, k, v, start, scale, gate=None, window=0, kv_valid=None):
    """q [rows][H][D], k/v [positions][KH][D]; row r sees keys [first, min(kv_valid, start+r+1))."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    rows, H, D = q.shape
    KH = k.shape[1]
    group = H // KH
    kv_valid = k.shape[0] if kv_valid is None else kv_valid
    out = np.zeros((rows, H, D))
    for r in range(rows):
        last = min(kv_valid, start + r + 1)
        first = max(0, start + r + 1 - window) if window else 0
        if last <= first:
            continue
        for h in range(H):
            kh = h // group
            scores = (k[first:last, kh, :] @ q[r, h, :]) * scale
            w = np.exp(scores - scores.max())
            w /= w.sum()
            out[r, h, :] = w @ v[first:last, kh, :]
    if gate is not None:
        out = out / (1.0 + np.exp(-np.asarray(gate, dtype=np.float64)))
    return out
