"""CPU checks of the oracle's composed functions (fused forward, error subtract-and-clip,
single-token decode attention) against properties and library routines."""
import numpy as np
import torch

from oracle import pyoracle as orc


def test_error_subtract_clip_properties():
    r = np.random.default_rng(0)
    pred, v = r.standard_normal((50, 24)).astype(np.float32), r.standard_normal((50, 24)).astype(np.float32)
    raw = pred - v
    assert np.array_equal(orc.error_subtract_clip(pred, v, 0.0), raw)
    clip = float(np.median(np.linalg.norm(raw, axis=1)))
    e = orc.error_subtract_clip(pred, v, clip)
    n_raw, n = np.linalg.norm(raw, axis=1), np.linalg.norm(e, axis=1)
    under = n_raw <= clip
    assert under.any() and (~under).any()
    assert np.array_equal(e[under], raw[under])
    assert np.allclose(n[~under], clip, rtol=1e-6)
    cos = np.sum(e[~under] * raw[~under], axis=1) / (n[~under] * n_raw[~under])
    assert np.allclose(cos, 1.0, atol=1e-6)


def test_fused_forward_reduces_to_the_plain_rule_for_constant_gates():
    r = np.random.default_rng(1)
    f = np.float32
    s, d = 12, 8
    k, v, q = (r.standard_normal((s, d)).astype(f) for _ in range(3))
    zero = np.zeros(2 * d, f)
    m0, s0 = np.zeros((d, d), f), np.zeros((d, d), f)
    o = orc.fused_forward(k, v, q, zero, -1.0, zero, 0.5, zero, 2.0, (0.0, 1.0), (0.0, 10.0), m0, s0)
    sig = lambda x: 1 / (1 + np.exp(-x))
    assert np.allclose(np.linalg.norm(o["k"], axis=1), 1, atol=1e-6)
    assert np.allclose(o["k_norms"], np.linalg.norm(k, axis=1), rtol=1e-6)
    assert np.allclose(o["alpha"], sig(-1.0), rtol=1e-6) and np.allclose(o["eta"], sig(2.0), rtol=1e-6)
    assert np.allclose(o["theta"], np.log1p(np.exp(0.5)), rtol=1e-6)
    kn, qn = k / np.linalg.norm(k, axis=1, keepdims=True), q / np.linalg.norm(q, axis=1, keepdims=True)
    y, _, _ = orc.titans_forward(kn.astype(f), v, qn.astype(f), o["alpha"], o["theta"], o["eta"], m0, s0)
    assert np.allclose(o["y"], y, rtol=1e-5, atol=1e-6)
    # clamps
    o2 = orc.fused_forward(k, v, q, zero, -1.0, zero, 0.5, None, 0.0, (0.4, 0.5), (0.1, 0.2), m0, s0)
    assert np.all(o2["alpha"] == f(0.4)) and np.all(o2["theta"] == f(0.2))


def test_single_token_decode_matches_sdpa():
    r = np.random.default_rng(2)
    H, hd, L, window = 2, 16, 21, 8
    td = H * hd
    bits = lambda x: torch.from_numpy(x.astype(np.float32)).to(torch.bfloat16).view(torch.uint16).numpy()
    q, kc, vc = bits(r.standard_normal(td)), bits(r.standard_normal((L, td))), bits(r.standard_normal((L, td)))
    got = orc.bf16_to_f32(orc.swa_single_token(q, kc, vc, window, H, 0))
    qf = torch.from_numpy(orc.bf16_to_f32(q)).view(1, H, 1, hd)
    kf = torch.from_numpy(orc.bf16_to_f32(kc)).view(L, H, hd).permute(1, 0, 2)[None, :, L - window:]
    vf = torch.from_numpy(orc.bf16_to_f32(vc)).view(L, H, hd).permute(1, 0, 2)[None, :, L - window:]
    want = torch.nn.functional.scaled_dot_product_attention(qf, kf, vf).reshape(td).numpy()
    assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max()


def _close(a, b, tol):
    return np.abs(np.asarray(a, np.float64) - b).max() <= tol * max(np.abs(b).max(), 1e-30)


def test_phase2_oracle_chained_equals_chunkwise_oracle():
    """The numpy phase-2 restatement, fed errors = M0 k - v chunk by chunk, is the chunkwise rule."""
    r = np.random.default_rng(3)
    f = np.float32
    s, d, C = 22, 6, 8
    k, v, q, dy = (r.standard_normal((s, d)).astype(f) for _ in range(4))
    sg = lambda x: (1 / (1 + np.exp(-x))).astype(f)
    al, th, et = (sg(r.standard_normal(s)) for _ in range(3))
    m0, s0 = (0.2 * r.standard_normal((d, d)).astype(f) for _ in range(2))
    for has_s in (True, False):
        y, mc, sc = orc.chunkwise_forward(k, v, q, al, th, et, m0, s0 if has_s else 0 * s0, 8, has_s)
        g = orc.chunkwise_backward(k, v, q, al, th, et, mc, sc, dy, 8, has_s)
        nc = (s + C - 1) // C
        m, sm = m0.copy(), (s0.copy() if has_s else None)
        errs = []
        for ci in range(nc):
            sl = slice(ci * C, min(s, ci * C + C))
            e = orc.error_subtract_clip(k[sl] @ m.T, v[sl], 0.0)
            errs.append(e)
            yy, m, sm = orc.phase2_forward(k[sl], q[sl], al[sl], th[sl], et[sl] if has_s else None, e, m, sm)
            assert _close(yy, y[sl], 1e-5) and _close(m, mc[ci + 1], 1e-5)
        dm, ds = np.zeros((d, d)), np.zeros((d, d))
        for ci in range(nc - 1, -1, -1):
            sl = slice(ci * C, min(s, ci * C + C))
            o = orc.phase2_backward(k[sl], q[sl], al[sl], th[sl], et[sl] if has_s else None, errs[ci], mc[ci],
                                    sc[ci], dy[sl], dm, ds)
            dm, ds = o["d_m"], o["d_s"]
            for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta") + (("d_eta",) if has_s else ()):
                assert _close(o[n], g[n][sl], 1e-4), n
        assert _close(dm, g["d_m"], 1e-4)
