"""Independent numpy (float64, matrix-form) statements of the memory rules.

Written from the update equations, not from the oracle's C loops, so that a
transcription slip in the oracle (dropped term, wrong sign, transposed operand)
shows up as a disagreement.  Used only by the CPU tests that pin the oracle.

Straight-through pieces (error clip, M-norm projection) are modelled as
*frozen additive offsets*: the forward uses e + off_e[t] and M + off_m[t] with
offsets recorded at the base point, which has exactly the identity Jacobian the
reference's backward assumes (core/kernels/error_clip.cuh:5,
m_norm_project.cuh:7).
"""
import numpy as np


def _clip(e, clip):
    if clip <= 0:
        return e
    n = np.sqrt(np.sum(e * e))
    return e * (clip / n) if n > clip else e


def _mnorm(m, mx):
    if mx <= 0 or mx >= 1e30:
        return m
    n = np.sqrt(np.sum(m * m))
    return m * (mx / n) if n > mx else m


def titans_forward(k, v, q, alpha, theta, eta, m0, s0, error_clip=0.0, m_norm_max=0.0,
                   offsets=None, record=False, momentum=True):
    """Exact per-token rule.  momentum=False is the Delta rule (eta, s0 ignored).
    offsets=(off_e [s,d], off_m [s,d,d]) replaces clip/projection by constants.
    Returns y, M trajectory, S trajectory (and the offsets when record=True)."""
    s, d = k.shape
    M = np.array(m0, np.float64)
    S = np.array(s0, np.float64) if momentum else np.zeros((d, d))
    Ms, Ss, ys = [M.copy()], [S.copy()], []
    off_e = np.zeros((s, d))
    off_m = np.zeros((s, d, d))
    for t in range(s):
        e_raw = M @ k[t] - v[t]
        if offsets is None:
            e = _clip(e_raw, error_clip)
            off_e[t] = e - e_raw
        else:
            e = e_raw + offsets[0][t]
        g = -theta[t] * np.outer(e, k[t])
        if momentum:
            S = eta[t] * S + g
            M_raw = (1.0 - alpha[t]) * M + S
        else:
            M_raw = (1.0 - alpha[t]) * M + g
        if offsets is None:
            M = _mnorm(M_raw, m_norm_max)
            off_m[t] = M - M_raw
        else:
            M = M_raw + offsets[1][t]
        ys.append(M @ q[t])
        Ms.append(M.copy())
        Ss.append(S.copy())
    out = (np.array(ys[0:]) if ys else np.zeros((0, d)), np.array(Ms), np.array(Ss))
    if record:
        return out + ((off_e, off_m),)
    return out


def chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, C, error_clip=0.0, m_norm_max=0.0,
                      offsets=None, record=False, momentum=True):
    """Frozen-M0 rule: errors of a chunk use the chunk-start M."""
    s, d = k.shape
    M = np.array(m0, np.float64)
    S = np.array(s0, np.float64) if momentum else np.zeros((d, d))
    Mb, Sb, ys = [M.copy()], [S.copy()], []
    off_e = np.zeros((s, d))
    off_m = np.zeros((s, d, d))
    for c0 in range(0, s, C):
        c1 = min(c0 + C, s)
        M0 = M.copy()
        E_raw = k[c0:c1] @ M0.T - v[c0:c1]
        for t in range(c0, c1):
            if offsets is None:
                e = _clip(E_raw[t - c0], error_clip)
                off_e[t] = e - E_raw[t - c0]
            else:
                e = E_raw[t - c0] + offsets[0][t]
            g = -theta[t] * np.outer(e, k[t])
            if momentum:
                S = eta[t] * S + g
                M_raw = (1.0 - alpha[t]) * M + S
            else:
                M_raw = (1.0 - alpha[t]) * M + g
            if offsets is None:
                M = _mnorm(M_raw, m_norm_max)
                off_m[t] = M - M_raw
            else:
                M = M_raw + offsets[1][t]
            ys.append(M @ q[t])
        Mb.append(M.copy())
        Sb.append(S.copy())
    out = (np.array(ys), np.array(Mb), np.array(Sb))
    if record:
        return out + ((off_e, off_m),)
    return out


def fd_grads(loss_fn, params, eps=1e-6):
    """Central finite differences of a scalar loss w.r.t. each array in params."""
    grads = {}
    for name, arr in params.items():
        g = np.zeros_like(arr)
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            old = arr[idx]
            arr[idx] = old + eps
            lp = loss_fn()
            arr[idx] = old - eps
            lm = loss_fn()
            arr[idx] = old
            g[idx] = (lp - lm) / (2 * eps)
        grads[name] = g
    return grads
