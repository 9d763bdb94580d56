"""Pins oracle/blocks.py (the opaque VJP blocks of the Delta rule and Titans LMM: projections, row L2
norm, gates with their feedback into k and v, the token recurrence, the clamp masks) without the
reference: central finite differences of the float64 block forward for the input and for every
parameter, hand cases for the straight-through clamp masks, and the flat-buffer round trip."""
import numpy as np
import pytest

from oracle import blocks as B


def _loss(kind, p, emb, w, **kw):
    y, _ = B.rule_step(kind, p, emb, round_weights=False, **kw)
    return float((y * w).sum())


@pytest.mark.parametrize("kind", ["delta", "titans"])
def test_block_backward_matches_finite_differences(kind):
    s, d = 7, 6
    rs = np.random.default_rng(11)
    p = B.init_params(d, 3, np.float64)
    emb = rs.standard_normal((s, d)) * 0.7
    w = rs.standard_normal((s, d))
    m0 = rs.standard_normal((d, d)) * 0.2
    kw = dict(m0=m0, s0=(rs.standard_normal((d, d)) * 0.1 if kind == "titans" else None))
    y, c = B.rule_step(kind, p, emb, round_weights=False, **kw)
    grads, d_emb = B.rule_step_backward(kind, p, c, w, emb, round_weights=False)
    eps = 1e-6

    def fd(arr, idx):
        old = arr[idx]
        arr[idx] = old + eps
        lp = _loss(kind, p, emb, w, **kw)
        arr[idx] = old - eps
        lm = _loss(kind, p, emb, w, **kw)
        arr[idx] = old
        return (lp - lm) / (2 * eps)
    for idx in [(0, 0), (3, 2), (6, 5), (2, 4)]:
        assert abs(fd(emb, idx) - d_emb[idx]) < 1e-6 * max(1.0, abs(d_emb[idx])), ("embedded", idx)
    names = list(B.FIELDS) if kind == "titans" else [n for n in B.FIELDS if "eta" not in n]
    for n in names:
        arr = p[n]
        for idx in ([(0, 0), (2, 5), (5, 1)] if arr.ndim == 2 else [(0,), (arr.size - 1,), (arr.size // 2,)]):
            if arr.ndim == 1 and idx[0] >= arr.size:
                continue
            g = grads[n][idx]
            assert abs(fd(arr, idx) - g) < 2e-6 * max(1.0, abs(g)), (n, idx, fd(arr, idx), g)
    if kind == "delta":
        assert not np.any(grads["w_eta"]) and not np.any(grads["b_eta"])


def test_projections_read_the_bf16_copy_of_the_matrices():
    d, s = 8, 5
    p = B.init_params(d, 5)
    emb = np.random.default_rng(2).standard_normal((s, d)).astype(np.float32)
    y_r, _ = B.rule_step("delta", p, emb)
    p2 = dict(p)
    for n in ("w_k_mem", "w_v_mem", "w_q_mem"):
        p2[n] = B.bf16_round(p[n])
        assert np.abs(p2[n] - p[n]).max() > 0
    y_2, _ = B.rule_step("delta", p2, emb, round_weights=False)
    np.testing.assert_array_equal(y_r, y_2)


def test_clamp_masks_follow_each_rule():
    """Delta (delta_rule.rs:566-569): theta masked where the CLAMPED value sits on a bound, alpha never.
    Titans (titans_lmm.rs:1707-1719): alpha and theta masked where the UNCLAMPED value is outside."""
    d, s = 6, 9
    emb = np.random.default_rng(4).standard_normal((s, d)).astype(np.float64)
    w = np.ones((s, d))
    for kind in ("delta", "titans"):
        p = B.init_params(d, 7, np.float64)
        lim = dict(alpha_lim=(0.2, 0.6), theta_lim=(0.05, 0.4))
        y, c = B.rule_step(kind, p, emb, round_weights=False, **lim)
        at_bound = (c["theta"] <= 0.05) | (c["theta"] >= 0.4)
        assert at_bound.any() and not at_bound.all(), "the case must clamp some tokens and not others"
        g_on, _ = B.rule_step_backward(kind, p, c, w, emb, round_weights=False, **lim)
        # with every theta on a bound the theta parameters get no gradient at all
        lim_all = dict(alpha_lim=(0.2, 0.6), theta_lim=(0.3, 0.3))
        y2, c2 = B.rule_step(kind, p, emb, round_weights=False, **lim_all)
        g_all, _ = B.rule_step_backward(kind, p, c2, w, emb, round_weights=False, **lim_all)
        assert not np.any(g_all["w_theta"]) and not np.any(g_all["b_theta"])
        assert np.any(g_on["w_theta"])
        # alpha pinned everywhere: Titans masks it, Delta passes the sigmoid slope through
        lim_a = dict(alpha_lim=(0.5, 0.5), theta_lim=(0.0, B.F32_MAX))
        y3, c3 = B.rule_step(kind, p, emb, round_weights=False, **lim_a)
        g_a, _ = B.rule_step_backward(kind, p, c3, w, emb, round_weights=False, **lim_a)
        assert np.any(g_a["w_alpha"]) == (kind == "delta")


def test_flat_parameter_buffer_round_trip_and_saved_layout():
    d, s = 8, 4
    p = B.init_params(d, 9)
    flat = B.params_to_flat(p)
    assert flat.size == 3 * d * d + 6 * d + 3
    q = B.params_from_flat(flat, d)
    for n in B.FIELDS:
        np.testing.assert_array_equal(np.asarray(q[n]).reshape(-1), np.asarray(p[n]).reshape(-1))
    assert B.params_to_flat(p, flat.size + 9).size == flat.size + 9
    emb = np.random.default_rng(1).standard_normal((s, d)).astype(np.float32)
    for kind, n_saved, meta_len in (("delta", 17, 12), ("titans", 20, 16)):
        y, c = B.rule_step(kind, p, emb)
        saved = B.saved_buffers(kind, p, c, emb)
        assert len(saved) == n_saved and saved[0].size == meta_len
        assert saved[0][0] == s and saved[0][1] == d and saved[0][2] == 2.0 and saved[0][-1] == 0.0
        assert saved[3].size == (s + 1) * d * d and saved[2].size == s * d
