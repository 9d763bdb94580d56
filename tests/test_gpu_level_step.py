"""The level step behind the C ABI (level_project_forward_bf16_rocm, titans_levels_{forward,backward}_bf16_rocm,
linear_{forward,backward}_bf16_rocm, cms_combine_gate_bf16x1_rocm), driven through ctypes only: no GEMM is
issued from Python.  Checker: the float64 glue of oracle/memory_level.py (row normalisation, gates, head split,
accumulate_projection_grads) around the C oracle's chunkwise rule, on the operands the contract names: x and the
weights rounded once to bf16, k / v / q rounded to bf16 after the normalisation.  Tolerances: quantities that
are rounded to bf16 at most one bf16 step (2^-8 relative); fp32 by-products 1e-4; gradients the bf16 bar 2e-2
(measured values are printed)."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd.ffi import lib
from oracle import memory_level as OL
from oracle import pyoracle as orc
from tests.gpu_util import dev, host, rel_err, l2_rel_err

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(BF).to(torch.float32).numpy().astype(np.float64)


def make_inputs(bs, s, nh, levels, n_extra, seed):
    d = nh * 64
    r = np.random.default_rng(seed)
    x = (r.standard_normal((bs * s, d)) / np.sqrt(d) * 4).astype(np.float32)
    lim = np.sqrt(6.0 / (2 * d))
    w_extra = r.uniform(-lim, lim, (n_extra * d, d)).astype(np.float32)
    w_levels = r.uniform(-lim, lim, (levels * 3 * d, d)).astype(np.float32)
    gates = []
    for _ in range(levels):
        gates.append(dict(w_alpha=r.uniform(-.3, .3, 2 * d).astype(np.float32), b_alpha=np.array([-1.0], np.float32),
                          w_theta=r.uniform(-.3, .3, 2 * d).astype(np.float32), b_theta=np.array([-2.0], np.float32),
                          w_eta=r.uniform(-.3, .3, 2 * d).astype(np.float32), b_eta=np.array([1.0], np.float32)))
    return x, w_extra, w_levels, gates


GATE_NAMES = ("w_alpha", "b_alpha", "w_theta", "b_theta", "w_eta", "b_eta")


def ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def reference_projections(x, w_extra, w_levels, gates, bs, s, nh, levels, n_extra):
    """float64 glue on bf16-rounded x and weights."""
    d = nh * 64
    xb = bf16_round(x)
    extra = [xb @ bf16_round(w_extra[e * d:(e + 1) * d]).T for e in range(n_extra)]
    out = []
    for lv in range(levels):
        wk, wv, wq = (bf16_round(w_levels[(3 * lv + i) * d:(3 * lv + i + 1) * d]) for i in range(3))
        k, kn = OL.l2_normalize(xb @ wk.T)
        q, qn = OL.l2_normalize(xb @ wq.T)
        v = xb @ wv.T
        g = {n: gates[lv][n].astype(np.float64) for n in GATE_NAMES}
        al = OL.gate(k, v, g["w_alpha"], g["b_alpha"], 0)
        th = OL.gate(k, v, g["w_theta"], g["b_theta"], 1)
        et = OL.gate(k, v, g["w_eta"], g["b_eta"], 0)
        out.append(dict(k=k, v=v, q=q, k_norms=kn, q_norms=qn, alpha=al, theta=th, eta=et))
    return xb, extra, out


class Step:
    """Device buffers of one call of the level step."""

    def __init__(self, bs, s, nh, levels, n_extra, chunk):
        d, hd = nh * 64, 64
        n, B = bs * s, bs * nh
        L = max(levels, 1)
        new = lambda *sh, dt=torch.float32: torch.empty(*sh, dtype=dt, device="cuda")
        self.extra = [new(n, d, dt=BF) for _ in range(n_extra)]
        self.xb = new(n, d, dt=BF)
        self.kh, self.vh, self.qh = (new(L * B, s, hd, dt=BF) for _ in range(3))
        self.ah, self.th, self.eh = (new(L * B, s) for _ in range(3))
        self.k_norms, self.q_norms, self.alpha, self.theta, self.eta = (new(L, n) for _ in range(5))
        nc = (s + chunk - 1) // chunk
        self.mc, self.sc = new(L * B, nc + 1, hd * hd), new(L * B, nc + 1, hd * hd)
        self.y = new(L, bs, s, d)


@pytest.mark.parametrize("bs,s,nh,levels,n_extra", [(2, 96, 4, 2, 3), (1, 200, 8, 3, 3), (3, 50, 8, 1, 0), (1, 130, 8, 0, 2)])
def test_projection_kernel_matches_the_float64_glue(bs, s, nh, levels, n_extra):
    d, n, B = nh * 64, bs * s, bs * nh
    x, w_extra, w_levels, gates = make_inputs(bs, s, nh, levels, n_extra, seed=bs * 1000 + s)
    st = Step(bs, s, nh, levels, n_extra, 64)
    tx, twe, twl = dev(x), dev(w_extra if n_extra else np.zeros((1, d), np.float32)), dev(w_levels if levels else np.zeros((1, d), np.float32))
    tg = [[dev(g[nm]) for nm in GATE_NAMES] for g in gates]
    lib.level_project_forward_bf16_rocm(
        tx.data_ptr(), twe.data_ptr(), n_extra, ptr_array(st.extra), twl.data_ptr(), ptr_array([t for g in tg for t in g]),
        st.xb.data_ptr(), st.kh.data_ptr(), st.vh.data_ptr(), st.qh.data_ptr(), st.ah.data_ptr(), st.th.data_ptr(),
        st.eh.data_ptr(), st.k_norms.data_ptr(), st.q_norms.data_ptr(), st.alpha.data_ptr(), st.theta.data_ptr(),
        st.eta.data_ptr(), bs, s, nh, 64, levels, 1e-8)
    torch.cuda.synchronize()
    xb, extra, ref = reference_projections(x, w_extra, w_levels, gates, bs, s, nh, levels, n_extra)
    assert np.array_equal(host(st.xb.float()).astype(np.float64), xb), "x_bf16 is x rounded to nearest even"
    step = 2.0 ** -8
    worst = {}
    for e in range(n_extra):
        worst[f"extra{e}"] = rel_err(host(st.extra[e].float()), extra[e])
        assert worst[f"extra{e}"] <= step
    for lv in range(levels):
        r = ref[lv]
        sl = slice(lv * B, (lv + 1) * B)
        for name, got in (("k", st.kh), ("v", st.vh), ("q", st.qh)):
            want = OL.to_heads(r[name], bs, s, nh, 64)
            e = rel_err(host(got[sl].float()), want)
            worst[f"L{lv}.{name}"] = e
            assert e <= step, (name, e)
            assert l2_rel_err(host(got[sl].float()), want) <= step
        for name, got in (("k_norms", st.k_norms), ("q_norms", st.q_norms), ("alpha", st.alpha), ("theta", st.theta),
                          ("eta", st.eta)):
            e = rel_err(host(got[lv]), r[name])
            worst[f"L{lv}.{name}"] = e
            assert e <= 1e-4, (name, e)
        for name, got in (("alpha", st.ah), ("theta", st.th), ("eta", st.eh)):
            want = OL.gates_to_heads(host(getattr(st, name)[lv]), bs, s, nh)
            assert np.array_equal(host(got[sl]), want), "per-head gate copies equal the token-major gates"
    print({k: f"{v:.1e}" for k, v in worst.items()}, flush=True)


@pytest.mark.parametrize("bs,s,nh,levels,chunk", [(2, 96, 4, 2, 32), (1, 200, 8, 3, 64)])
def test_levels_forward_and_backward_through_the_c_abi(bs, s, nh, levels, chunk):
    d, hd, n, B, n_extra = nh * 64, 64, bs * s, bs * nh, 3
    x, w_extra, w_levels, gates = make_inputs(bs, s, nh, levels, n_extra, seed=7 + s)
    r = np.random.default_rng(s)
    st = Step(bs, s, nh, levels, n_extra, chunk)
    tx, twe, twl = dev(x), dev(w_extra), dev(w_levels)
    tg = [[dev(g[nm]) for nm in GATE_NAMES] for g in gates]
    m0 = (0.05 * r.standard_normal((levels * B, hd * hd))).astype(np.float32)
    s0 = (0.05 * r.standard_normal((levels * B, hd * hd))).astype(np.float32)
    m_ctx, s_ctx = dev(m0), dev(s0)
    lib.titans_levels_forward_bf16_rocm(
        tx.data_ptr(), twe.data_ptr(), n_extra, ptr_array(st.extra), twl.data_ptr(), ptr_array([t for g in tg for t in g]),
        m_ctx.data_ptr(), s_ctx.data_ptr(), st.xb.data_ptr(), st.kh.data_ptr(), st.vh.data_ptr(), st.qh.data_ptr(),
        st.ah.data_ptr(), st.th.data_ptr(), st.eh.data_ptr(), st.k_norms.data_ptr(), st.q_norms.data_ptr(),
        st.alpha.data_ptr(), st.theta.data_ptr(), st.eta.data_ptr(), st.mc.data_ptr(), st.sc.data_ptr(), st.y.data_ptr(),
        bs, s, nh, hd, levels, chunk, 1e-8)
    torch.cuda.synchronize()
    f32 = np.float32
    kh, vh, qh = (host(t.float()) for t in (st.kh, st.vh, st.qh))
    ah, th, eh = host(st.ah), host(st.th), host(st.eh)
    nc = (s + chunk - 1) // chunk
    # the rule on the operands the projection kernel wrote (those are checked in the test above)
    y_ref = np.zeros((levels * B, s, hd), f32)
    mcs, scs = np.zeros((levels * B, nc + 1, hd, hd), f32), np.zeros((levels * B, nc + 1, hd, hd), f32)
    for c in range(levels * B):
        y_ref[c], mcs[c], scs[c] = orc.chunkwise_forward(kh[c], vh[c], qh[c], ah[c], th[c], eh[c], m0[c].reshape(hd, hd),
                                                         s0[c].reshape(hd, hd), chunk)
    y_tok = np.stack([OL.from_heads(y_ref[lv * B:(lv + 1) * B], bs, s, nh, hd).reshape(bs, s, d) for lv in range(levels)])
    e_y = rel_err(host(st.y), y_tok)
    assert e_y <= 1e-3, e_y
    assert rel_err(host(st.mc), mcs.reshape(levels * B, nc + 1, -1)) <= 1e-3
    assert np.array_equal(host(m_ctx), host(st.mc[:, -1])) and np.array_equal(host(s_ctx), host(st.sc[:, -1])), \
        "the context memories carry the final chunk states"

    # backward
    d_y = r.standard_normal((bs, s, d)).astype(f32)
    d_extra = [r.standard_normal((n, d)).astype(f32) for _ in range(n_extra)]
    t_dy, t_de = dev(d_y), [dev(a) for a in d_extra]
    d_x = torch.empty(n, d, device="cuda")
    d_we, d_wl = torch.empty(n_extra * d, d, device="cuda"), torch.empty(levels * 3 * d, d, device="cuda")
    d_g = [[torch.empty_like(t) for t in g] for g in tg]
    dm, ds = torch.zeros(hd, hd, device="cuda"), torch.zeros(hd, hd, device="cuda")
    lib.titans_levels_backward_bf16_rocm(
        st.xb.data_ptr(), twe.data_ptr(), n_extra, ptr_array(t_de), twl.data_ptr(), st.kh.data_ptr(), st.vh.data_ptr(),
        st.qh.data_ptr(), st.ah.data_ptr(), st.th.data_ptr(), st.eh.data_ptr(), st.k_norms.data_ptr(),
        st.q_norms.data_ptr(), st.alpha.data_ptr(), st.theta.data_ptr(), st.eta.data_ptr(), st.mc.data_ptr(),
        st.sc.data_ptr(), t_dy.data_ptr(), d_x.data_ptr(), d_we.data_ptr(), d_wl.data_ptr(),
        ptr_array([t for g in d_g for t in g]), dm.data_ptr(), ds.data_ptr(), bs, s, nh, hd, levels, chunk, 1e-8)
    torch.cuda.synchronize()
    # reference: the C oracle's rule backward per chain, then accumulate_projection_grads in float64
    xb = host(st.xb.float()).astype(np.float64).reshape(bs, s, d)
    dyh = OL.to_heads(d_y.reshape(n, d), bs, s, nh, hd)
    dx_ref = np.zeros((bs, s, d))
    dm_ref = np.zeros((hd, hd))
    worst = {}
    mc_h, sc_h = host(st.mc).reshape(levels * B, nc + 1, hd, hd), host(st.sc).reshape(levels * B, nc + 1, hd, hd)
    for lv in range(levels):
        gs = []
        for b in range(B):
            c = lv * B + b
            gs.append(orc.chunkwise_backward(kh[c], vh[c], qh[c], ah[c], th[c], eh[c], mc_h[c], sc_h[c], dyh[b], chunk))
            dm_ref += gs[-1]["d_m"]
        stack = lambda nm: np.stack([g[nm] for g in gs]).astype(np.float64)
        dk, dv, dq = (OL.from_heads(stack(nm), bs, s, nh, hd) for nm in ("d_k", "d_v", "d_q"))
        da, dt, de = (OL.gates_from_heads(stack(nm), bs, s, nh) for nm in ("d_alpha", "d_theta", "d_eta"))
        cache = dict(k=OL.from_heads(kh[lv * B:(lv + 1) * B].astype(np.float64), bs, s, nh, hd),
                     v=OL.from_heads(vh[lv * B:(lv + 1) * B].astype(np.float64), bs, s, nh, hd),
                     q=OL.from_heads(qh[lv * B:(lv + 1) * B].astype(np.float64), bs, s, nh, hd),
                     k_norms=host(st.k_norms[lv]).astype(np.float64), q_norms=host(st.q_norms[lv]).astype(np.float64),
                     alpha=host(st.alpha[lv]).astype(np.float64), theta=host(st.theta[lv]).astype(np.float64),
                     eta=host(st.eta[lv]).astype(np.float64))
        p = {nm: bf16_round(w_levels[(3 * lv + i) * d:(3 * lv + i + 1) * d]) for i, nm in enumerate(("w_k", "w_v", "w_q"))}
        g, dx = OL.projection_grads(p, xb, cache, dk, dv, dq, da, dt, de)
        dx_ref += dx
        for i, nm in enumerate(("w_k", "w_v", "w_q")):
            worst[f"L{lv}.d_{nm}"] = rel_err(host(d_wl[(3 * lv + i) * d:(3 * lv + i + 1) * d]), g[nm])
        for i, nm in enumerate(GATE_NAMES):
            if nm.startswith("b_"):
                # one scalar, a sum over all tokens of signed terms that can nearly cancel: measured against the size
                # of the sums it belongs to (the matching weight-vector gradient) when its own value is smaller
                scale = max(abs(float(g[nm][0])), float(np.linalg.norm(g["w_" + nm[2:]])))
                worst[f"L{lv}.d_{nm}"] = abs(float(host(d_g[lv][i])[0]) - float(g[nm][0])) / scale
            else:
                worst[f"L{lv}.d_{nm}"] = rel_err(host(d_g[lv][i]), g[nm])
    x2 = xb.reshape(n, d)
    for e in range(n_extra):
        gq = bf16_round(d_extra[e])
        dx_ref += (gq @ bf16_round(w_extra[e * d:(e + 1) * d])).reshape(bs, s, d)
        worst[f"d_w_extra{e}"] = rel_err(host(d_we[e * d:(e + 1) * d]), gq.T @ x2)
    worst["d_x"] = rel_err(host(d_x).reshape(bs, s, d), dx_ref)
    worst["d_m_initial"] = rel_err(host(dm), dm_ref)
    print({k: f"{v:.1e}" for k, v in worst.items()}, flush=True)
    assert max(worst.values()) <= 2e-2, worst


def test_linear_pair_and_combine_gate():
    n, d_in, d_out, k = 300, 256, 512, 3
    r = np.random.default_rng(5)
    a = r.standard_normal((n, d_in)).astype(np.float32)
    w = (r.standard_normal((d_out, d_in)) / 16).astype(np.float32)
    g = r.standard_normal((n, d_out)).astype(np.float32)
    ta = dev(a).to(BF)
    tw, tg = dev(w), dev(g)
    out, d_a, d_w = (torch.empty(*sh, device="cuda") for sh in ((n, d_out), (n, d_in), (d_out, d_in)))
    lib.linear_forward_bf16_rocm(ta.data_ptr(), tw.data_ptr(), out.data_ptr(), n, d_in, d_out)
    lib.linear_backward_bf16_rocm(tg.data_ptr(), ta.data_ptr(), tw.data_ptr(), d_a.data_ptr(), d_w.data_ptr(), n, d_in, d_out)
    torch.cuda.synchronize()
    ab, wb, gb = bf16_round(a), bf16_round(w), bf16_round(g)
    assert rel_err(host(out), ab @ wb.T) <= 1e-5
    assert rel_err(host(d_a), gb @ wb) <= 1e-5
    assert rel_err(host(d_w), gb.T @ ab) <= 1e-5
    # combine + gate with the gated product leaving as bf16
    ys = [r.standard_normal((n, d_in)).astype(np.float32) for _ in range(k)]
    attn = r.standard_normal((n, d_in)).astype(np.float32)
    t_ys, t_attn = [dev(y) for y in ys], dev(attn).to(BF)
    gate, gated = torch.empty(n, d_in, device="cuda"), torch.empty(n, d_in, dtype=BF, device="cuda")
    lib.cms_combine_gate_bf16x1_rocm(ptr_array(t_ys), k, t_attn.data_ptr(), gate.data_ptr(), gated.data_ptr(), n * d_in)
    torch.cuda.synchronize()
    want_gate = OL.sigmoid(sum(y.astype(np.float64) for y in ys) / np.sqrt(k))
    assert rel_err(host(gate), want_gate) <= 1e-6
    assert rel_err(host(gated.float()), bf16_round(attn) * want_gate) <= 2.0 ** -8


def test_layer_with_single_bf16_projections_matches_autograd():
    """The whole layer on the path that issues no GEMM from Python, against the float64 autograd restatement:
    all levels active, then with a frozen level (sequence shorter than its period)."""
    from tests.test_gpu_mag_layer import run_case
    import nl_hecate_amd.mag_layer as ML
    orig = ML.MagLayer.__init__

    def init_bf16(self, *a, **kw):
        kw["precision"] = "bf16"
        orig(self, *a, **kw)
    ML.MagLayer.__init__ = init_bf16
    try:
        w = run_case(bs=2, s=200, d=256, nh=4, k=2, window=64, periods=[1, 8], rule="chunkwise", chunk=32, seed=17,
                     bias_scale=True)
        print("active:", {n: f"{e:.1e}" for n, e in w.items()}, flush=True)
        assert max(w.values()) < 2e-2, w
        w = run_case(bs=1, s=40, d=256, nh=4, k=3, window=16, periods=[1, 8, 64], rule="chunkwise", chunk=16, seed=19,
                     steps=2, bias_scale=True)
        print("with a frozen level:", {n: f"{e:.1e}" for n, e in w.items()}, flush=True)
        assert max(w.values()) < 2e-2, w
    finally:
        ML.MagLayer.__init__ = orig
