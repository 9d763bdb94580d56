"""Helpers shared by the GPU parity tests: seeded synthetic inputs with the
distributions of the benchmark configurations, upload/download, and the
norm-relative error the tolerances are stated in."""
import numpy as np
import torch

REL_TOL_F32 = 1e-4   # fp32 paths: max|a-b| / max|b|
REL_TOL_BF16 = 2e-2  # bf16-input / fp32-accumulate paths


def rule_inputs(B, s, d, seed, gates="sigmoid", m0_scale=0.0, momentum=True):
    """k,q ~ N(0,1) L2-normalised per token; v ~ N(0,1); gates sigmoid(N(0,1));
    M0 = S0 = m0_scale * N(0,1); dY ~ N(0,1).  All float32 numpy."""
    r = np.random.default_rng(seed)
    f = np.float32
    k = r.standard_normal((B, s, d))
    q = r.standard_normal((B, s, d))
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    q /= np.linalg.norm(q, axis=-1, keepdims=True)
    v = r.standard_normal((B, s, d))
    sig = lambda x: 1.0 / (1.0 + np.exp(-x))
    if gates == "sigmoid":
        alpha, theta, eta = (sig(r.standard_normal((B, s))) for _ in range(3))
    else:  # the constants of the reference's CUDA tests
        alpha = np.full((B, s), 0.05)
        theta = np.full((B, s), 0.01)
        eta = np.full((B, s), 0.9)
    m0 = m0_scale * r.standard_normal((B, d, d))
    s0 = m0_scale * r.standard_normal((B, d, d))
    dy = r.standard_normal((B, s, d))
    out = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, eta=eta, m0=m0, s0=s0, dy=dy)
    return {n: np.ascontiguousarray(x, f) for n, x in out.items()}


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def zeros(*shape):
    return torch.zeros(*shape, dtype=torch.float32, device="cuda")


def rel_err(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), "non-finite values in kernel output"
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def l2_rel_err(got, want):
    """||got - want||_2 / ||want||_2: a tensor whose small entries are all wrong fails this one even
    when a few large entries keep the max-norm figure low."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.sqrt(np.sum((got - want) ** 2)) / max(np.sqrt(np.sum(want ** 2)), 1e-30))


def assert_close(name, got, want, tol=REL_TOL_F32):
    """Both figures must hold: max|a-b| / max|b| and ||a-b||_2 / ||b||_2."""
    e = rel_err(got, want)
    assert e <= tol, f"{name}: rel err {e:.3e} > {tol:.0e}"
    e2 = l2_rel_err(got, want)
    assert e2 <= tol, f"{name}: L2-relative err {e2:.3e} > {tol:.0e}"
    return e


def assert_abs(name, got, want, tol):
    """The reference's own check: max abs difference (cuda_test_utils.rs:17-40)."""
    got, want = np.asarray(got), np.asarray(want)
    assert np.isfinite(got).all()
    diff = float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max()) if got.size else 0.0
    assert diff < tol, f"{name}: max diff {diff:.3e} >= {tol:.0e}"
