"""Pins the oracle of the HOPE self-referential memory (oracle/selfref.inc):
an independent numpy implementation of the forward, structural properties the
reference tests (C=1 equals the per-token rule; self-generated targets read the
FROZEN snapshot; remainder chunks), and central finite differences of the
double-precision forward for the input and all six initial memories.  CPU only."""
import numpy as np
import pytest

from oracle import pyoracle as orc


def _sigmoid(x):
    return 1.0 if x >= 15 else 0.0 if x <= -15 else 1 / (1 + np.exp(-x))


def _softplus(x):
    return x if x >= 15 else 0.0 if x <= -15 else np.log1p(np.exp(x))


def np_selfref_forward(mems, x, C, self_gen):
    """From the update equations (HOPE Eqs 84, 88, 90-93): projections read the
    current memories, errors the chunk-start snapshot, y reads M_mem before its update."""
    M = [np.array(m, np.float64) for m in mems]
    s, d = x.shape
    ys = []
    for t in range(s):
        if t % C == 0:
            F = [m.copy() for m in M]
        k, v, q, er, ar = (M[c] @ x[t] for c in range(5))
        alpha, theta = _sigmoid(ar.mean()), _softplus(er.mean())
        ys.append(M[5] @ q)
        for c in range(6):
            target = F[c] @ v if self_gen else v
            e = F[c] @ k - target
            M[c] = (1 - alpha) * M[c] - theta * np.outer(e, k)
    return np.array(ys), np.array(M)


def _case(s, d, seed, scale=0.3):
    r = np.random.default_rng(seed)
    mems = scale * r.standard_normal((6, d, d))
    mems[3] += 0.3   # eta: keep theta away from 0
    x = r.standard_normal((s, d)) / np.sqrt(d)
    dy = r.standard_normal((s, d))
    return mems, x, dy


@pytest.mark.parametrize("C", [1, 3, 4, 16])
@pytest.mark.parametrize("self_gen", [True, False])
def test_forward_matches_numpy(C, self_gen):
    mems, x, _ = _case(10, 5, 1)
    y, mf, _ = orc.selfref_forward(mems, x, C, self_gen)
    yn, mn = np_selfref_forward(mems, x, C, self_gen)
    assert np.allclose(y, yn, rtol=1e-10, atol=1e-12) and np.allclose(mf, mn, rtol=1e-10, atol=1e-12)
    y32, m32, _ = orc.selfref_forward(mems.astype(np.float32), x.astype(np.float32), C, self_gen)
    assert np.abs(y32 - yn).max() < 1e-4 * max(1.0, np.abs(yn).max())


def test_chunk_size_one_is_the_sequential_rule():
    """chunkwise_self_ref.rs:661-716: with C=1 the frozen snapshot is the current state,
    so each memory follows the plain DGD step M <- (1-a)M - th (M k - target) k^T."""
    mems, x, _ = _case(6, 4, 2)
    y, mf, c = orc.selfref_forward(mems, x, 1, False)
    M = [m.copy() for m in mems]
    for t in range(6):
        k, v = M[0] @ x[t], M[1] @ x[t]
        a, th = c["alpha"][t], c["theta"][t]
        M = [(1 - a) * m - th * np.outer(m @ k - v, k) for m in M]
    assert np.allclose(mf, np.array(M), rtol=1e-10)
    assert np.allclose(c["traj"][:, 0], mems) and np.allclose(c["frozen"][:, :, :, :], c["traj"][:, :-1].transpose(1, 0, 2, 3))


def test_self_generated_targets_use_the_frozen_snapshot():
    """chunkwise_self_ref.rs:974-1015."""
    mems, x, _ = _case(8, 4, 3)
    _, _, c = orc.selfref_forward(mems, x, 4, True)
    for t in (1, 2, 3, 5, 7):
        ci = t // 4
        for comp in range(6):
            assert np.allclose(c["v_hat"][comp, t], c["frozen"][ci, comp] @ c["v"][t], rtol=1e-12)
            assert not np.allclose(c["v_hat"][comp, t], c["traj"][comp, t] @ c["v"][t], rtol=1e-6)


@pytest.mark.parametrize("s,C", [(7, 3), (8, 4), (5, 8), (6, 1)])
@pytest.mark.parametrize("self_gen", [True, False])
def test_backward_matches_finite_differences(s, C, self_gen):
    d = 4
    mems, x, dy = _case(s, d, 4 + s)
    _, _, cache = orc.selfref_forward(mems, x, C, self_gen)
    d_emb, d_mems = orc.selfref_backward(cache, dy)

    def loss(m, xx):
        y, _ = np_selfref_forward(m, xx, C, self_gen)
        return float((y * dy).sum())

    eps = 1e-6
    fd_x = np.zeros_like(x)
    for idx in np.ndindex(*x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += eps; xm[idx] -= eps
        fd_x[idx] = (loss(mems, xp) - loss(mems, xm)) / (2 * eps)
    fd_m = np.zeros_like(mems)
    for idx in np.ndindex(*mems.shape):
        mp, mm = mems.copy(), mems.copy()
        mp[idx] += eps; mm[idx] -= eps
        fd_m[idx] = (loss(mp, x) - loss(mm, x)) / (2 * eps)
    assert np.abs(d_emb - fd_x).max() < 2e-6 * max(1.0, np.abs(fd_x).max())
    for c in range(6):
        assert np.abs(d_mems[c] - fd_m[c]).max() < 2e-6 * max(1.0, np.abs(fd_m).max()), c


def test_float_backward_tracks_double():
    mems, x, dy = _case(24, 8, 9)
    _, _, c64 = orc.selfref_forward(mems, x, 8, True)
    e64, m64 = orc.selfref_backward(c64, dy)
    f = np.float32
    _, _, c32 = orc.selfref_forward(mems.astype(f), x.astype(f), 8, True)
    e32, m32 = orc.selfref_backward(c32, dy.astype(f))
    assert np.abs(e32 - e64).max() < 1e-4 * max(1.0, np.abs(e64).max())
    assert np.abs(m32 - m64).max() < 1e-4 * max(1.0, np.abs(m64).max())
