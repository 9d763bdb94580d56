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


# ── the exact Titans rule in chunk-parallel matrix form ─────────────────────
# The rule is linear in (M, S).  Inside a chunk that starts at (M0, S0), with the per-token state after token t
#   M_(t+1) = a_t M0 + beta_t S0 + sum_(j<=t) W[t][j] u_j k_j^T,   S_(t+1) = h_t S0 + sum_(j<=t) Ws[t][j] u_j k_j^T
# (a, beta, h, W = -theta_j c[t][j], Ws = -theta_j bb[j][t]: the coefficients of the frozen-M0 chunkwise rule), the
# exact errors u_t = M_t k_t - v_t obey a unit lower triangular system
#   (I - Lam) U = R,   Lam[t][j] = W[t-1][j] (k_j . k_t)  (j < t),   R = am.(K M0^T) + bm.(K S0^T) - V
# with am, bm the vectors a, beta shifted by one token (am_0 = 1, bm_0 = 0).  Everything else is the frozen rule
# with its errors replaced by U.  A third statement of the rule beside the oracle's loops and titans_forward above:
# a slip in either shows up as a disagreement, and the gradients below are checked against the oracle's backward.
def _chunk_coefficients(alpha, theta, eta):
    L = len(alpha)
    keep = 1.0 - alpha
    a, h, beta = np.zeros(L), np.zeros(L), np.zeros(L)
    pa, ph, pb = 1.0, 1.0, 0.0
    for t in range(L):
        pa, ph = pa * keep[t], ph * eta[t]
        pb = keep[t] * pb + ph
        a[t], h[t], beta[t] = pa, ph, pb
    c, bb = np.zeros((L, L)), np.zeros((L, L))   # c[t][j], bb[j][t]
    for j in range(L):
        b, cc = 1.0, 1.0
        for t in range(j, L):
            if t > j:
                b *= eta[t]
                cc = keep[t] * cc + b
            c[t, j], bb[j, t] = cc, b
    return a, beta, h, c, bb


def titans_exact_chunk_forward(k, v, q, alpha, theta, eta, m0, s0, C):
    """y [s,d] and the states at chunk boundaries ([nc+1,d,d] each), from one triangular solve per chunk."""
    s, d = k.shape
    M, S = np.array(m0, np.float64), np.array(s0, np.float64)
    Mb, Sb, ys = [M.copy()], [S.copy()], []
    for c0 in range(0, s, C):
        sl = slice(c0, min(c0 + C, s))
        K, V, Q = k[sl], v[sl], q[sl]
        L = len(K)
        a, beta, h, c, bb = _chunk_coefficients(alpha[sl], theta[sl], eta[sl])
        W = -theta[sl][None, :] * c                                  # [t][j], zero above the diagonal
        am, bm = np.concatenate([[1.0], a[:-1]]), np.concatenate([[0.0], beta[:-1]])
        G = K @ K.T
        Lam = np.zeros((L, L))
        Lam[1:, :] = np.tril(W[:-1, :] * G[1:, :], 0)[:, :]          # row t uses W[t-1][j], j <= t-1
        R = am[:, None] * (K @ M.T) + bm[:, None] * (K @ S.T) - V
        U = np.linalg.solve(np.eye(L) - Lam, R)
        ys.append(a[:, None] * (Q @ M.T) + beta[:, None] * (Q @ S.T) + (W * (Q @ K.T)) @ U)
        wM, wS = W[L - 1], -theta[sl] * bb[:, L - 1]
        M, S = (a[-1] * M + beta[-1] * S + U.T @ (wM[:, None] * K), h[-1] * S + U.T @ (wS[:, None] * K))
        Mb.append(M.copy())
        Sb.append(S.copy())
    return np.concatenate(ys), np.array(Mb), np.array(Sb)


def titans_exact_chunk_backward(k, v, q, alpha, theta, eta, m_bound, s_bound, d_y, C):
    """Gradients of sum(y * d_y) from the chunk-boundary states: per chunk two triangular solves (one transposed),
    a reverse scan over the chunks for the state adjoints, and the coefficient recurrences differentiated in
    reverse for the gates.  Returns the oracle's dictionary (d_m, d_s: gradients of the initial states)."""
    s, d = k.shape
    g = {n: np.zeros((s, d)) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(s) for n in ("d_alpha", "d_theta", "d_eta")})
    dM, dS = np.zeros((d, d)), np.zeros((d, d))
    starts = list(range(0, s, C))
    for ci in reversed(range(len(starts))):
        c0 = starts[ci]
        sl = slice(c0, min(c0 + C, s))
        K, V, Q, dY = k[sl], v[sl], q[sl], d_y[sl]
        L = len(K)
        al, th, et = alpha[sl], theta[sl], eta[sl]
        keep = 1.0 - al
        M0, S0 = m_bound[ci], s_bound[ci]
        a, beta, h, c, bb = _chunk_coefficients(al, th, et)
        W = -th[None, :] * c
        am, bm = np.concatenate([[1.0], a[:-1]]), np.concatenate([[0.0], beta[:-1]])
        G, P = K @ K.T, Q @ K.T
        Lam = np.zeros((L, L))
        Lam[1:, :] = np.tril(W[:-1, :] * G[1:, :], 0)
        T = np.linalg.inv(np.eye(L) - Lam)
        KM, KS = K @ M0.T, K @ S0.T
        U = T @ (am[:, None] * KM + bm[:, None] * KS - V)
        wM, wS = W[L - 1], -th * bb[:, L - 1]
        # adjoints of the errors, of the right-hand side and of the triangular matrix
        dU = (W * P).T @ dY + wM[:, None] * (K @ dM.T) + wS[:, None] * (K @ dS.T)
        dR = T.T @ dU
        dLam = np.tril(dR @ U.T, -1)
        dYU = np.tril(dY @ U.T, 0)
        dP = W * dYU
        dG = np.zeros((L, L))
        dG[1:, :] = W[:-1, :] * dLam[1:, :]
        g["d_v"][sl] = -dR
        g["d_q"][sl] = a[:, None] * (dY @ M0) + beta[:, None] * (dY @ S0) + dP @ K
        g["d_k"][sl] = (dP.T @ Q + wM[:, None] * (U @ dM) + wS[:, None] * (U @ dS) + am[:, None] * (dR @ M0)
                        + bm[:, None] * (dR @ S0) + (dG + dG.T) @ K)
        # gradients of the coefficients
        dW = dYU * P
        dW[:-1, :] += dLam[1:, :] * G[1:, :]
        dW[L - 1] += np.sum((U @ dM) * K, 1)
        dwS = np.sum((U @ dS) * K, 1)
        da = np.sum(dY * (Q @ M0.T), 1)
        db = np.sum(dY * (Q @ S0.T), 1)
        dam, dbm = np.sum(dR * KM, 1), np.sum(dR * KS, 1)
        da[:-1] += dam[1:]
        db[:-1] += dbm[1:]
        da[-1] += np.sum(dM * M0)
        db[-1] += np.sum(dM * S0)
        dh = np.zeros(L)
        dh[-1] = np.sum(dS * S0)
        # W = -theta_j c[t][j], wS = -theta_j bb[j][L-1]
        dth = -np.sum(dW * c, 0) - dwS * bb[:, L - 1]
        dc = -th[None, :] * dW
        dbb = np.zeros((L, L))
        dbb[:, L - 1] = -th * dwS
        dkeep, deta = np.zeros(L), np.zeros(L)
        for j in range(L):      # reverse of: b *= eta_t; cc = keep_t cc + b   (t = j+1 .. L-1)
            gcc, gb = 0.0, 0.0
            for t in range(L - 1, j, -1):
                gcc += dc[t, j]
                gb += dbb[j, t]
                dkeep[t] += gcc * c[t - 1, j]
                gb += gcc
                gcc *= keep[t]
                deta[t] += gb * bb[j, t - 1]
                gb *= et[t]
        ga, gh, gbt = 0.0, 0.0, 0.0   # reverse of: a *= keep_t; h *= eta_t; beta = keep_t beta + h
        for t in range(L - 1, -1, -1):
            ga += da[t]
            gh += dh[t]
            gbt += db[t]
            pa = a[t - 1] if t else 1.0
            ph = h[t - 1] if t else 1.0
            pb = beta[t - 1] if t else 0.0
            dkeep[t] += gbt * pb + ga * pa
            gh += gbt
            gbt *= keep[t]
            deta[t] += gh * ph
            ga *= keep[t]
            gh *= et[t]
        g["d_alpha"][sl] = -dkeep
        g["d_theta"][sl] = dth
        g["d_eta"][sl] = deta
        # adjoints of the chunk-start states
        dM, dS = (a[-1] * dM + (a[:, None] * dY).T @ Q + (am[:, None] * dR).T @ K,
                  beta[-1] * dM + h[-1] * dS + (beta[:, None] * dY).T @ Q + (bm[:, None] * dR).T @ K)
    g["d_m"], g["d_s"] = dM, dS
    return g
