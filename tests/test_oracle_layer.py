"""Pins the CPU oracle of the pieces around the memory rules (AdamW, clip,
pulse, gates, L2 normalisation, bf16, sliding-window attention) with
reference-held known answers, library routines (torch on CPU as a generic
routine) and finite differences.  CPU only."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc


# ── AdamW ──────────────────────────────────────────────────────────────────
def test_adamw_first_step_closed_form():
    """Step 1 with zero moments: m_hat = g, v_hat = g^2 -> w -= lr*(g/(|g|+eps) + wd*w)."""
    w = np.array([1.0, -2.0, 0.5], np.float32)
    g = np.array([0.3, -0.1, 2.0], np.float32)
    m, v = np.zeros(3, np.float32), np.zeros(3, np.float32)
    w0 = w.copy()
    b1, b2, lr, wd, eps = 0.9, 0.95, 3e-4, 0.1, 1e-8
    orc.adamw_step(w, g, m, v, lr, b1, b2, eps, 1 / (1 - b1), 1 / (1 - b2), wd)
    want = w0 - lr * (g / (np.abs(g) + eps) + wd * w0)
    assert np.allclose(w, want, rtol=1e-6)
    assert np.allclose(m, (1 - b1) * g, rtol=1e-6) and np.allclose(v, (1 - b2) * g * g, rtol=1e-6)


def test_adamw_matches_torch_over_several_steps():
    r = np.random.default_rng(0)
    w = r.standard_normal(257).astype(np.float32)
    m, v = np.zeros_like(w), np.zeros_like(w)
    b1, b2, lr, wd, eps = 0.9, 0.95, 3e-3, 0.1, 1e-8
    tw = torch.tensor(w.copy(), requires_grad=True)
    opt = torch.optim.AdamW([tw], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    for step in range(1, 6):
        g = r.standard_normal(257).astype(np.float32)
        orc.adamw_step(w, g, m, v, lr, b1, b2, eps, 1 / (1 - b1 ** step), 1 / (1 - b2 ** step), wd)
        tw.grad = torch.tensor(g)
        opt.step()
        # torch divides by (sqrt(v)/sqrt(bc2) + eps): same placement of eps
        assert np.allclose(w, tw.detach().numpy(), rtol=2e-5, atol=2e-6), step


def test_per_level_step_counters_under_scripted_pulses():
    """core/src/adamw.rs:437-500: a level's bias correction uses how often THAT
    level fired; a frozen level changes neither its moments nor its counter."""
    chunk = [1, 2, 4]
    steps = [0, 0, 0]
    for gstep in range(8):
        act = orc.pulse(gstep, chunk)
        for l, a in enumerate(act):
            steps[l] += int(a)
    assert steps == [8, 4, 2]


def test_grad_norm_clip():
    g = [np.full(4, 3.0, np.float32), np.full(9, 4.0 / 1.5, np.float32)]
    # norm^2 = 4*9 + 9*(64/9) = 36 + 64 = 100
    n, s = orc.grad_norm_clip(g, 1.0)
    assert abs(n - 10.0) < 1e-5 and abs(s - 0.1) < 1e-7
    n, s = orc.grad_norm_clip(g, 20.0)
    assert s == 1.0
    n, s = orc.grad_norm_clip(g, 0.0)
    assert s == 1.0


# ── Conductor ──────────────────────────────────────────────────────────────
def test_pulse_truth_tables():
    """core/src/conductor.rs:268-300: k=2, chunk_sizes [1,8]."""
    for step in range(17):
        assert orc.pulse(step, [1, 8]) == [True, step % 8 == 0]
    # core/src/conductor.rs:387-427: k=4 [1,8,64,512]
    for step, want in [(0, [1, 1, 1, 1]), (1, [1, 0, 0, 0]), (8, [1, 1, 0, 0]), (64, [1, 1, 1, 0]),
                       (512, [1, 1, 1, 1]), (520, [1, 1, 0, 0])]:
        assert orc.pulse(step, [1, 8, 64, 512]) == [bool(x) for x in want]
    # seq_len >= chunk size keeps a level active every step (conductor.rs:136-144)
    assert orc.pulse(3, [1, 8, 64, 512], seq_len=64) == [True, True, True, False]
    assert orc.pulse(3, [1, 8, 64, 512], seq_len=4096) == [True] * 4


# ── gates, normalisation, bf16 ─────────────────────────────────────────────
def test_gate_compute_and_backward_against_numpy_and_fd():
    r = np.random.default_rng(1)
    T, D = 13, 6
    k, v = r.standard_normal((T, D)).astype(np.float32), r.standard_normal((T, D)).astype(np.float32)
    w = (0.3 * r.standard_normal(2 * D)).astype(np.float32)
    b = 0.2
    z = k @ w[:D] + v @ w[D:] + b
    assert np.allclose(orc.gate_compute(k, v, w, b, 0), 1 / (1 + np.exp(-z)), rtol=1e-5)
    assert np.allclose(orc.gate_compute(k, v, w, b, 1), np.log1p(np.exp(z)), rtol=1e-5)
    assert orc.gate_compute(k * 100, v, np.ones(2 * D, np.float32), 500.0, 1).max() > 20  # identity branch
    # backward: loss = sum_t c_t * gate_t for each gate; d_w = sum_t c_t gate'(z_t) x_t
    c = r.standard_normal((3, T)).astype(np.float32)
    alpha, theta, eta = (orc.gate_compute(k, v, w, b, a) for a in (0, 1, 0))
    g = orc.gate_backward(c[0], alpha, c[1], theta, c[2], eta, k, v)
    x = np.concatenate([k, v], 1).astype(np.float64)
    sig = 1 / (1 + np.exp(-z.astype(np.float64)))
    assert np.allclose(g["d_w_alpha"], (c[0] * sig * (1 - sig)) @ x, rtol=1e-4, atol=1e-5)
    assert np.allclose(g["d_w_theta"], (c[1] * sig) @ x, rtol=1e-4, atol=1e-5)  # softplus' = sigmoid
    assert np.allclose(g["d_w_eta"], (c[2] * sig * (1 - sig)) @ x, rtol=1e-4, atol=1e-5)
    assert np.allclose(g["d_b_theta"], (c[1] * sig).sum(), rtol=1e-4)


def test_l2_normalize_and_backward():
    r = np.random.default_rng(2)
    x = r.standard_normal((5, 9)).astype(np.float32)
    xn, norms = orc.l2_normalize_rows(x)
    assert np.allclose(np.linalg.norm(xn, axis=1), 1.0, atol=1e-6)
    assert np.allclose(norms, np.linalg.norm(x, axis=1), rtol=1e-6)
    g = r.standard_normal((5, 9)).astype(np.float32)
    d_in = orc.l2_normalize_backward(g, xn, norms)
    xd = x.astype(np.float64)
    fd = np.zeros_like(xd)
    eps = 1e-6
    for i in range(5):
        for j in range(9):
            for sgn in (1, -1):
                y = xd.copy(); y[i, j] += sgn * eps
                fd[i, j] += sgn * ((y / np.linalg.norm(y, axis=1, keepdims=True)) * g).sum() / (2 * eps)
    assert np.allclose(d_in, fd, rtol=1e-3, atol=1e-4)
    # zero row: forward divides by eps, backward multiplies by 1/eps
    z = np.zeros((1, 4), np.float32)
    zn, zno = orc.l2_normalize_rows(z)
    assert zno[0] == 0 and np.all(zn == 0)
    assert np.allclose(orc.l2_normalize_backward(np.ones((1, 4), np.float32), zn, zno), 1e8)


def test_bf16_round_trip_matches_torch():
    r = np.random.default_rng(3)
    x = np.concatenate([r.standard_normal(4000) * 10 ** r.uniform(-6, 6, 4000),
                        [0.0, -0.0, 1.0, 1.00390625, 1.0 + 2 ** -8, 3.0e38]]).astype(np.float32)
    b = orc.f32_to_bf16(x)
    t = torch.tensor(x).to(torch.bfloat16)
    assert np.array_equal(b, t.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(orc.bf16_to_f32(b), t.float().numpy())


# ── sliding-window attention ───────────────────────────────────────────────
def _bf(x):
    return orc.f32_to_bf16(np.asarray(x, np.float32))


def test_swa_known_answers():
    """core/src/swa.rs:286-344."""
    q = _bf([[[1.0, 0.0, 0.0, 1.0]]]); v = _bf([[[0.5, 0.3, 0.1, 0.7]]])
    out, aw = orc.swa_forward(q, q, v, 1, 1)
    assert np.allclose(orc.bf16_to_f32(out), orc.bf16_to_f32(v))       # window 1 copies V
    qq = _bf(np.tile([1.0, 0.0], (1, 4, 1)))
    vv = _bf([[[10.0, 0], [20.0, 0], [30.0, 0], [40.0, 0]]])
    out, aw = orc.swa_forward(qq, qq, vv, 2, 1)
    assert abs(orc.bf16_to_f32(out)[0, 3, 0] - 35.0) < 0.2             # uniform average of V[2:4]
    q3 = _bf([[[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]]]); v3 = _bf([[[1.0, 0.0], [0.0, 1.0], [0.5, 0.5]]])
    out, aw = orc.swa_forward(q3, q3, v3, 3, 1)
    o = orc.bf16_to_f32(out)
    assert abs(o[0, 0, 0] - 1.0) < 1e-2 and abs(o[0, 0, 1]) < 1e-2     # causal: position 0 sees itself
    w = orc.bf16_to_f32(aw)
    assert np.allclose(w.sum(-1), 1.0, atol=2e-2)


@pytest.mark.parametrize("n_persistent", [0, 3])
def test_swa_forward_matches_torch_sdpa_with_band_mask(n_persistent):
    r = np.random.default_rng(4)
    B, s, H, hd, ws = 2, 19, 2, 8, 5
    q, k, v = (_bf(r.standard_normal((B, s, H * hd))) for _ in range(3))
    out, aw = orc.swa_forward(q, k, v, ws, H, n_persistent)
    tq, tk, tv = (torch.tensor(orc.bf16_to_f32(a)).view(B, s, H, hd).transpose(1, 2) for a in (q, k, v))
    i = torch.arange(s)[:, None]; j = torch.arange(s)[None, :]
    mask = (j <= i) & ((j > i - ws) | (j < n_persistent))
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask)
    ref = ref.transpose(1, 2).reshape(B, s, H * hd).numpy()
    assert np.abs(orc.bf16_to_f32(out) - ref).max() < 2e-2


def test_swa_backward_matches_finite_differences():
    r = np.random.default_rng(5)
    B, s, H, hd, ws, npers = 1, 7, 2, 4, 3, 2
    q, k, v = (_bf(r.standard_normal((B, s, H * hd))) for _ in range(3))
    go = r.standard_normal((B, s, H * hd)).astype(np.float32)
    out, aw = orc.swa_forward(q, k, v, ws, H, npers)
    dq, dk, dv = orc.swa_backward(q, k, v, aw, go, ws, H, npers)

    def f64_forward(qf, kf, vf):
        o = np.zeros((B, s, H * hd))
        for b in range(B):
            for h in range(H):
                sl = slice(h * hd, (h + 1) * hd)
                for t in range(s):
                    keys = [j for j in range(t + 1) if j > t - ws or j < npers]
                    sc = np.array([qf[b, t, sl] @ kf[b, j, sl] for j in keys]) / np.sqrt(hd)
                    w = np.exp(sc - sc.max()); w /= w.sum()
                    o[b, t, sl] = sum(wi * vf[b, j, sl] for wi, j in zip(w, keys))
        return o

    base = [orc.bf16_to_f32(a).astype(np.float64) for a in (q, k, v)]
    eps = 1e-5
    for idx, got in ((0, dq), (1, dk), (2, dv)):
        fd = np.zeros_like(base[idx])
        it = np.nditer(base[idx], flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            old = base[idx][i]
            base[idx][i] = old + eps; lp = (f64_forward(*base) * go).sum()
            base[idx][i] = old - eps; lm = (f64_forward(*base) * go).sum()
            base[idx][i] = old
            fd[i] = (lp - lm) / (2 * eps)
        # the backward runs on bf16-rounded weights: 2e-2 of the gradient scale
        assert np.abs(got - fd).max() < 2e-2 * max(1.0, np.abs(fd).max()), idx
