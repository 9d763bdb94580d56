"""Pins the CPU oracle of the memory rules (oracle/nlh_oracle.c) without the
reference: reference-held known answers, closed forms, an independent numpy
matrix-form implementation, and finite differences of the double-precision
forward for every gradient.  CPU only.
"""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import np_rules as npr


def _inputs(s, d, seed, dt=np.float64, momentum=True, gate_lo=0.05, gate_hi=0.95):
    r = np.random.default_rng(seed)
    k = r.standard_normal((s, d))
    q = r.standard_normal((s, d))
    k /= np.linalg.norm(k, axis=1, keepdims=True)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    v = r.standard_normal((s, d))
    sig = lambda x: 1 / (1 + np.exp(-x))
    alpha = np.clip(sig(r.standard_normal(s)), gate_lo, gate_hi)
    theta = np.clip(sig(r.standard_normal(s)), gate_lo, gate_hi)
    eta = np.clip(sig(r.standard_normal(s)), gate_lo, gate_hi)
    m0 = 0.3 * r.standard_normal((d, d))
    s0 = 0.3 * r.standard_normal((d, d))
    dy = r.standard_normal((s, d))
    return [np.ascontiguousarray(x, dt) for x in (k, v, q, alpha, theta, eta, m0, s0, dy)]


# ── reference-held known answers ───────────────────────────────────────────
def test_kat_dgd_step_basic():
    """core/tests/test_dgd.rs:20-50: M=I, k=e0, v=0.5, alpha=0.1, theta=0.5."""
    d = 4
    for dt in (np.float32, np.float64):
        k = np.array([[1, 0, 0, 0]], dt)
        v = np.full((1, d), 0.5, dt)
        q = np.zeros((1, d), dt)
        y, ms = orc.delta_forward(k, v, q, np.array([0.1], dt), np.array([0.5], dt), np.eye(d, dtype=dt))
        m = ms[1]
        assert abs(m[0, 0] - 0.65) < 1e-6 and abs(m[1, 0] - 0.25) < 1e-6 and abs(m[1, 1] - 0.9) < 1e-6
        # error = [0.5,-0.5,-0.5,-0.5] is visible through column 0: M[:,0] = 0.9*I[:,0] - 0.5*e
        e = (0.9 * np.eye(d)[:, 0] - m[:, 0]) / 0.5
        assert np.allclose(e, [0.5, -0.5, -0.5, -0.5], atol=1e-6)


def test_kat_zero_gates_leave_m_unchanged():
    """core/tests/test_dgd.rs:54-72."""
    d = 4
    k = np.array([[1, 2, 3, 4]], np.float32)
    v = np.full((1, d), 0.5, np.float32)
    _, ms = orc.delta_forward(k, v, k, np.zeros(1, np.float32), np.zeros(1, np.float32),
                              np.eye(d, dtype=np.float32))
    assert np.abs(ms[1] - np.eye(d)).max() < 1e-10


def test_simple_rng_matches_xorshift64_in_python_ints():
    """tensor.rs:380-408 restated with Python big-int arithmetic."""
    for seed in (0, 1, 100, 1300, 2**63 + 12345):
        s = max(seed, 1)
        want = []
        for _ in range(16):
            s ^= (s << 13) & (2**64 - 1)
            s ^= s >> 7
            s ^= (s << 17) & (2**64 - 1)
            u = np.float32(s / float(2**64 - 1))
            want.append((np.float32(2.0) * u - np.float32(1.0)) * np.float32(0.1))
        got = orc.simple_rng_uniform(16, seed, 0.1)
        assert np.array_equal(got, np.array(want, np.float32))
    big = orc.simple_rng_uniform(20000, 42, 0.1)
    assert np.abs(big).max() <= 0.1 and abs(big.mean()) < 2e-3


def test_checkpoint_count_table():
    """core/src/gpu_forward.rs:2885-2897 and test_gradient_checkpoint.rs:285."""
    assert orc.checkpoint_count(8, 4) == 3
    assert orc.checkpoint_count(8, 1) == 9
    assert orc.checkpoint_count(7, 4) == 3      # 0, after t=3, final
    assert orc.checkpoint_count(8, 8) == 2
    assert orc.checkpoint_count(8, 16) == 2
    assert orc.checkpoint_count(2048, 64) == 33


# ── closed forms ───────────────────────────────────────────────────────────
def test_theta_zero_is_pure_decay():
    s, d = 9, 5
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 1)
    theta[:] = 0
    y, ms = orc.delta_forward(k, v, q, alpha, theta, m0)
    decay = np.cumprod(1 - alpha)
    for t in range(s):
        assert np.allclose(ms[t + 1], decay[t] * m0, rtol=1e-12)
        assert np.allclose(y[t], decay[t] * m0 @ q[t], rtol=1e-12)


def test_one_step_stores_value_exactly():
    """alpha=0, eta=0, theta=1, |k|=1, M0=0: M1 k = v."""
    d = 6
    k, v, q, *_ = _inputs(1, d, 2)
    z = np.zeros((d, d))
    one, zero = np.ones(1), np.zeros(1)
    _, ms, _ = orc.titans_forward(k, v, k, zero, one, zero, z, z)
    assert np.allclose(ms[1] @ k[0], v[0], atol=1e-12)
    y, _ = orc.delta_forward(k, v, k, zero, one, z)
    assert np.allclose(y[0], v[0], atol=1e-12)


def test_eta_zero_titans_is_delta():
    s, d = 10, 6
    for dt in (np.float32, np.float64):
        k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 3, dt)
        yt, mt, st = orc.titans_forward(k, v, q, alpha, theta, np.zeros(s, dt), m0, s0)
        yd, md = orc.delta_forward(k, v, q, alpha, theta, m0)
        assert np.allclose(yt, yd, rtol=1e-6, atol=1e-6) and np.allclose(mt, md, rtol=1e-6, atol=1e-6)


def test_hand_computed_clip_d2():
    """d=2, M0=0, v=(3,4): e=(-3,-4), |e|=5 > clip=1 -> e=(-0.6,-0.8);
    k=(1,0), theta=0.5 -> M1 = [[0.3,0],[0.4,0]]."""
    k = np.array([[1.0, 0.0]])
    v = np.array([[3.0, 4.0]])
    _, ms = orc.delta_forward(k, v, k, np.zeros(1), np.array([0.5]), np.zeros((2, 2)), error_clip=1.0)
    assert np.allclose(ms[1], [[0.3, 0.0], [0.4, 0.0]], atol=1e-12)
    # m-norm projection: |M1|_F = 0.5 -> max 0.25 halves it
    y, ms = orc.delta_forward(k, v, k, np.zeros(1), np.array([0.5]), np.zeros((2, 2)),
                              error_clip=1.0, m_norm_max=0.25)
    assert np.allclose(ms[1], [[0.15, 0.0], [0.2, 0.0]], atol=1e-12)
    assert np.allclose(y[0], [0.15, 0.2], atol=1e-12)


def test_clip_and_mnorm_invariants_and_noop():
    s, d = 24, 8
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 4)
    y0, m_a, s_a = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0)
    # no-ops: clip<=0, m_norm_max >= f32::MAX or <= 0
    for kw in (dict(error_clip=0.0), dict(error_clip=-1.0), dict(m_norm_max=orc.F32_MAX),
               dict(m_norm_max=0.0), dict(error_clip=1e9, m_norm_max=1e9)):
        y1, m_b, _ = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0, **kw)
        assert np.array_equal(y0, y1) and np.array_equal(m_a, m_b)
    y2, m_c, _ = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0, error_clip=0.5, m_norm_max=0.7)
    assert not np.allclose(y0, y2)
    assert np.all(np.sqrt((m_c[1:] ** 2).sum((1, 2))) <= 0.7 * (1 + 1e-12))


# ── independent numpy matrix form ──────────────────────────────────────────
@pytest.mark.parametrize("clip,mx", [(0.0, 0.0), (0.6, 0.0), (0.0, 1.2), (0.6, 1.2)])
def test_forward_matches_numpy_matrix_form(clip, mx):
    s, d = 20, 7
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 5)
    mxo = mx if mx > 0 else orc.F32_MAX
    y, ms, ss = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mxo)
    yn, mn, sn = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mx)
    assert np.allclose(y, yn, rtol=1e-10, atol=1e-12)
    assert np.allclose(ms, mn, rtol=1e-10, atol=1e-12) and np.allclose(ss, sn, rtol=1e-10, atol=1e-12)
    yd, md = orc.delta_forward(k, v, q, alpha, theta, m0, clip, mxo)
    ydn, mdn, _ = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mx, momentum=False)
    assert np.allclose(yd, ydn, rtol=1e-10, atol=1e-12) and np.allclose(md, mdn, rtol=1e-10, atol=1e-12)
    # float oracle tracks the double one
    f = [x.astype(np.float32) for x in (k, v, q, alpha, theta, eta, m0, s0)]
    y32, m32, s32 = orc.titans_forward(*f, clip, mxo)
    assert np.abs(y32 - yn).max() < 2e-5 * max(1.0, np.abs(yn).max())


# ── gradients: finite differences of the double-precision forward ──────────
def _check_grads(fd, an, names, rtol=2e-6):
    for n in names:
        scale = max(np.abs(fd[n]).max(), 1e-3)
        err = np.abs(fd[n] - an[n]).max() / scale
        assert err < rtol, f"{n}: rel err {err:.3e}"


@pytest.mark.parametrize("clip,mx", [(0.0, 0.0), (0.5, 0.0), (0.5, 1.0)])
def test_titans_backward_matches_finite_differences(clip, mx):
    s, d = 7, 4
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 6)
    mxo = mx if mx > 0 else orc.F32_MAX
    _, ms, ss, offs = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mx, record=True)
    if clip > 0:
        assert np.abs(offs[0]).max() > 0, "clip must be active in this case"
    if mx > 0:
        assert np.abs(offs[1]).max() > 0, "projection must be active in this case"
    P = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, eta=eta, m0=m0, s0=s0)

    def loss():
        y, _, _ = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, offsets=offs)
        return float((y * dy).sum())

    fd = npr.fd_grads(loss, P)
    _, mo, so = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mxo)
    g = orc.titans_backward(k, v, q, alpha, theta, eta, mo, so, dy, clip)
    an = dict(k=g["d_k"], v=g["d_v"], q=g["d_q"], alpha=g["d_alpha"], theta=g["d_theta"],
              eta=g["d_eta"], m0=g["d_m"], s0=g["d_s"])
    _check_grads(fd, an, P.keys())


@pytest.mark.parametrize("clip,mx", [(0.0, 0.0), (0.5, 1.0)])
def test_delta_backward_matches_finite_differences(clip, mx):
    s, d = 7, 4
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 7)
    mxo = mx if mx > 0 else orc.F32_MAX
    _, ms, _, offs = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mx, record=True,
                                        momentum=False)
    P = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, m0=m0)

    def loss():
        y, _, _ = npr.titans_forward(k, v, q, alpha, theta, eta, m0, s0, offsets=offs, momentum=False)
        return float((y * dy).sum())

    fd = npr.fd_grads(loss, P)
    _, mo = orc.delta_forward(k, v, q, alpha, theta, m0, clip, mxo)
    g = orc.delta_backward(k, v, q, alpha, theta, mo, dy, clip)
    an = dict(k=g["d_k"], v=g["d_v"], q=g["d_q"], alpha=g["d_alpha"], theta=g["d_theta"], m0=g["d_m"])
    _check_grads(fd, an, P.keys())


def test_float_backward_tracks_double_backward():
    s, d = 32, 8
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 8)
    _, ms, ss = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0)
    g64 = orc.titans_backward(k, v, q, alpha, theta, eta, ms, ss, dy)
    f = [x.astype(np.float32) for x in (k, v, q, alpha, theta, eta, m0, s0, dy)]
    _, ms32, ss32 = orc.titans_forward(*f[:8])
    g32 = orc.titans_backward(*f[:6], ms32, ss32, f[8])
    for n in g64:
        assert np.abs(g32[n] - g64[n]).max() < 1e-4 * max(1.0, np.abs(g64[n]).max()), n


def test_batched_backward_sums_initial_state_grads_over_batch():
    B, s, d = 3, 6, 4
    r = np.random.default_rng(9)
    chains = [[x.astype(np.float32) for x in _inputs(s, d, 90 + b)] for b in range(B)]
    st = lambda i: np.stack([c[i] for c in chains])
    k, v, q, al, th, et, m0, s0, dy = [st(i) for i in range(9)]
    y, ms, ss = orc.titans_forward_batch(k, v, q, al, th, et, m0, s0)
    g = orc.titans_backward_batch(k, v, q, al, th, et, ms, ss, dy)
    dm = np.zeros((d, d), np.float32)
    ds = np.zeros((d, d), np.float32)
    for b in range(B):
        y1, m1, s1 = orc.titans_forward(*[c for c in chains[b][:8]])
        assert np.array_equal(y1, y[b])
        g1 = orc.titans_backward(*chains[b][:6], m1, s1, chains[b][8])
        assert np.array_equal(g1["d_k"], g["d_k"][b]) and np.array_equal(g1["d_eta"], g["d_eta"][b])
        dm += g1["d_m"]
        ds += g1["d_s"]
    assert np.array_equal(dm, g["d_m_initial"]) and np.array_equal(ds, g["d_s_initial"])
    yd, md = orc.delta_forward_batch(k, v, q, al, th, m0)
    gd = orc.delta_backward_batch(k, v, q, al, th, md, dy)
    dm = sum(orc.delta_backward(*chains[b][:5], md[b], chains[b][8])["d_m"] for b in range(B))
    assert np.allclose(dm, gd["d_m_initial"], atol=1e-6)


# ── checkpoint / segment schedule ──────────────────────────────────────────
@pytest.mark.parametrize("C", [1, 4, 8, 64, 5])
@pytest.mark.parametrize("has_s", [True, False])
def test_checkpointed_equals_full_trajectory(C, has_s):
    """core/tests/test_gradient_checkpoint.rs:140-280: ckpt == full for
    C in {1, 4, 8, >= s, non-divisor}."""
    s, d = 19, 6
    k, v, q, alpha, theta, eta, m0, s0, dy = [x.astype(np.float32) for x in _inputs(s, d, 10)]
    clip, mx = 0.8, 2.0
    if has_s:
        y, ms, ss = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0, clip, mx)
        g = orc.titans_backward(k, v, q, alpha, theta, eta, ms, ss, dy, clip)
    else:
        y, ms = orc.delta_forward(k, v, q, alpha, theta, m0, clip, mx)
        ss = None
        g = orc.delta_backward(k, v, q, alpha, theta, ms, dy, clip)
    yc, mc, sc = orc.forward_ckpt(k, v, q, alpha, theta, eta, m0, s0, C, has_s, clip, mx)
    assert np.array_equal(y, yc)
    slots = [0] + [t + 1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s]
    assert mc.shape[0] == len(slots)
    assert np.array_equal(mc, ms[slots])
    if has_s:
        assert np.array_equal(sc, ss[slots])
    gc = orc.backward_ckpt(k, v, q, alpha, theta, eta, mc, sc, dy, C, has_s, clip, mx)
    for n in g:
        assert np.array_equal(g[n], gc[n]), n


def test_segment_backward_composes():
    s, d = 12, 5
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 11)
    _, ms, ss = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0)
    full = orc.titans_backward(k, v, q, alpha, theta, eta, ms, ss, dy)
    hi = orc.titans_backward(k, v, q, alpha, theta, eta, ms[7:], ss[7:], dy, t_lo=7, t_hi=12)
    lo = orc.titans_backward(k, v, q, alpha, theta, eta, ms[:8], ss[:8], dy, t_lo=0, t_hi=7,
                             d_m_seed=hi["d_m"], d_s_seed=hi["d_s"])
    assert np.allclose(lo["d_m"], full["d_m"], rtol=1e-12) and np.allclose(lo["d_s"], full["d_s"], rtol=1e-12)
    assert np.allclose(hi["d_k"][7:], full["d_k"][7:], rtol=1e-12)
    assert np.allclose(lo["d_k"][:7], full["d_k"][:7], rtol=1e-12)
    assert np.all(hi["d_k"][:7] == 0), "a segment call writes only its own tokens"


# ── frozen-M0 chunkwise ────────────────────────────────────────────────────
@pytest.mark.parametrize("has_s", [True, False])
def test_chunkwise_c1_equals_exact(has_s):
    """core/src/gpu_forward.rs:4193-4338: chunk size 1 is the per-token rule."""
    s, d = 14, 6
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 12)
    yc, mc, sc = orc.chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, 1, has_s)
    if has_s:
        y, ms, ss = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0)
        assert np.allclose(sc, ss, rtol=1e-12)
        g = orc.titans_backward(k, v, q, alpha, theta, eta, ms, ss, dy)
    else:
        y, ms = orc.delta_forward(k, v, q, alpha, theta, m0)
        g = orc.delta_backward(k, v, q, alpha, theta, ms, dy)
    assert np.allclose(yc, y, rtol=1e-12) and np.allclose(mc, ms, rtol=1e-12)
    gc = orc.chunkwise_backward(k, v, q, alpha, theta, eta, mc, sc, dy, 1, has_s)
    for n in g:
        assert np.allclose(g[n], gc[n], rtol=1e-10, atol=1e-12), n


def test_chunkwise_differs_from_exact_for_c_gt_1():
    s, d = 16, 6
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 13)
    yc, _, _ = orc.chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, 4)
    y, _, _ = orc.titans_forward(k, v, q, alpha, theta, eta, m0, s0)
    assert np.allclose(yc[0], y[0]) and not np.allclose(yc, y)


@pytest.mark.parametrize("C", [3, 4, 16])
@pytest.mark.parametrize("has_s", [True, False])
@pytest.mark.parametrize("clip,mx", [(0.0, 0.0), (0.5, 1.0)])
def test_chunkwise_matches_numpy_and_finite_differences(C, has_s, clip, mx):
    s, d = 10, 4
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, 14)
    mxo = mx if mx > 0 else orc.F32_MAX
    yn, mbn, sbn, offs = npr.chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, C, clip, mx,
                                               record=True, momentum=has_s)
    y, mc, sc = orc.chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, C, has_s, clip, mxo)
    assert np.allclose(y, yn, rtol=1e-10, atol=1e-12) and np.allclose(mc, mbn, rtol=1e-10, atol=1e-12)
    if has_s:
        assert np.allclose(sc, sbn, rtol=1e-10, atol=1e-12)
    P = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, m0=m0)
    if has_s:
        P.update(eta=eta, s0=s0)

    def loss():
        yy, _, _ = npr.chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, C, offsets=offs,
                                         momentum=has_s)
        return float((yy * dy).sum())

    fd = npr.fd_grads(loss, P)
    g = orc.chunkwise_backward(k, v, q, alpha, theta, eta, mc, sc, dy, C, has_s, clip, mxo)
    an = dict(k=g["d_k"], v=g["d_v"], q=g["d_q"], alpha=g["d_alpha"], theta=g["d_theta"],
              eta=g["d_eta"], m0=g["d_m"], s0=g["d_s"])
    _check_grads(fd, an, P.keys())


@pytest.mark.parametrize("s,d,C", [(37, 6, 8), (64, 8, 64), (130, 4, 64), (9, 5, 1), (20, 3, 7)])
@pytest.mark.parametrize("saturate", [False, True])
def test_exact_rule_matches_its_chunk_parallel_matrix_form(s, d, C, saturate):
    """The exact Titans rule restated per chunk as one unit lower triangular solve (np_rules.titans_exact_chunk_*):
    a different algorithm from the oracle's token loops (dispatch.rs:1226-1563), so agreement of the outputs, the
    boundary states and every gradient in float64 pins both.  saturate: alpha = 1 and eta = 0 at some tokens
    (no division anywhere, so the gradients stay finite and equal)."""
    r = np.random.default_rng(1000 + s + d + C)
    k, v, q, dy = (r.standard_normal((s, d)) * 0.5 for _ in range(4))
    al, th, et = r.uniform(0.05, 0.4, s), r.uniform(0.05, 0.5, s), r.uniform(0.3, 0.95, s)
    if saturate:
        al[s // 3], et[s // 2], al[s - 1], et[0] = 1.0, 0.0, 1.0, 0.0
    m0, s0 = r.standard_normal((d, d)) * 0.3, r.standard_normal((d, d)) * 0.3
    y, mb, sb = npr.titans_exact_chunk_forward(k, v, q, al, th, et, m0, s0, C)
    yo, mo, so = orc.titans_forward(k, v, q, al, th, et, m0, s0)
    bounds = list(range(0, s, C)) + [s]
    assert np.abs(y - yo).max() < 1e-12
    assert np.abs(mb - mo[bounds]).max() < 1e-12 and np.abs(sb - so[bounds]).max() < 1e-12
    g = npr.titans_exact_chunk_backward(k, v, q, al, th, et, mb, sb, dy, C)
    go = orc.titans_backward(k, v, q, al, th, et, mo, so, dy)
    for n in go:
        assert np.abs(g[n] - go[n]).max() <= 1e-11 * max(1.0, np.abs(go[n]).max()), n
