"""TEST INFRASTRUCTURE ONLY — one CMS memory level end to end on the CPU.

The composition the reference's host code makes around its rule kernels, for the matrix memories:
gpu_memory_forward (core/src/gpu_forward.rs:1197-1705: projections, L2 normalisation of k and q, gate
projections and clamps, per-head layout, the rule, carry of the final memory with its Frobenius clamp) and
gpu_memory_backward (core/src/gpu_backward.rs:459-1200) with accumulate_projection_grads (:2047-2117).
The rules themselves are the C oracle's (oracle/rules.inc through pyoracle); the glue is written here in
numpy in the dtype of the inputs, so the whole level also runs in float64 and its backward can be checked
against finite differences of its forward.  tests/test_oracle_memory_level.py pins the glue against the C
oracle's float32 glue (orc_gate_compute, orc_l2_normalize_*, orc_gate_backward) and the backward against
central differences of the float64 forward.

cfg: any object with the attributes of nl_hecate_amd.memory_level.LevelConfig.
p: dict of numpy arrays w_k, w_v, w_q [d, d], w_alpha, w_theta, w_eta [2d], b_alpha, b_theta, b_eta [1].
"""
import numpy as np

from . import model_glue as glue
from . import pyoracle as orc

F32_MAX = 3.4028234663852886e38
EPS = 1e-8


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x):
    """core/kernels/elementwise.cu:47: identity above 20."""
    return np.where(x > 20.0, x, np.log1p(np.exp(np.minimum(x, 20.0))))


def l2_normalize(x):
    """core/kernels/elementwise.cu l2_normalize_rows: x / max(|x|, eps), norms before normalisation."""
    n = np.sqrt((x * x).sum(-1))
    return x / np.maximum(n, EPS)[:, None], n


def l2_normalize_backward(d_out, x_norm, norms):
    """d_in = (d_out - x_norm (x_norm . d_out)) / norm for norm >= eps, d_out / eps below it."""
    dot = (d_out * x_norm).sum(-1, keepdims=True)
    big = (d_out - x_norm * dot) / np.maximum(norms, EPS)[:, None]
    return np.where((norms >= EPS)[:, None], big, d_out / EPS)


def gate(k, v, w, b, act):
    d = k.shape[1]
    z = k @ w[:d] + v @ w[d:] + b[0]
    return sigmoid(z) if act == 0 else softplus(z)


def to_heads(x, bs, s, nh, hd):
    """[bs*s, nh*hd] -> [bs*nh, s, hd] (reshape_to_per_head, gpu_forward.rs:1133)."""
    return np.ascontiguousarray(x.reshape(bs, s, nh, hd).transpose(0, 2, 1, 3).reshape(bs * nh, s, hd))


def from_heads(x, bs, s, nh, hd):
    return np.ascontiguousarray(x.reshape(bs, nh, s, hd).transpose(0, 2, 1, 3).reshape(bs * s, nh * hd))


def gates_to_heads(g, bs, s, nh):
    """[bs*s] -> [bs*nh, s] (broadcast_gates, gpu_forward.rs:1161)."""
    return np.ascontiguousarray(np.repeat(g.reshape(bs, 1, s), nh, axis=1).reshape(bs * nh, s))


def gates_from_heads(g, bs, s, nh):
    return g.reshape(bs, nh, s).sum(1).reshape(bs * s)


def frobenius_clamp(m, m_norm_max):
    """m_norm_clamp_batch_f32_cuda: each [hd, hd] block scaled back onto the ball; off for max <= 0 or >= 1e30."""
    if not 0 < m_norm_max < 1e30:
        return m
    out = m.copy()
    for i in range(out.shape[0]):
        n = np.sqrt((out[i] * out[i]).sum())
        if n > m_norm_max:
            out[i] *= m_norm_max / n
    return out


def _clamped(cfg):
    return (cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0), (cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX)


def level_forward(p, cfg, x, m0, gates=None):
    """x [bs, s, d], m0 [bs*nh, hd, hd] -> y [bs, s, d], cache, carried memory [bs*nh, hd, hd].
    gates: (alpha, theta, eta) to use instead of the computed ones (the reference's backward sends no gradient
    from the gates into k and v, so a finite-difference check of the k, v, q path holds them fixed)."""
    bs, s, d = x.shape
    nh, hd = cfg.num_heads, cfg.head_dim
    dt = x.dtype
    x2 = x.reshape(bs * s, d)
    if cfg.memory_rule == "swiglu":   # stateless MLP level (gpu_forward.rs:1705-1727)
        y, gate_b, up_b, fused, sig = glue.swiglu_forward(x2, p["gate_proj"], p["up_proj"], p["down_proj"])
        return y.reshape(bs, s, d).astype(dt), dict(gate=gate_b, up=up_b, fused=fused, sig=sig), m0
    k_raw, v, q_raw = x2 @ p["w_k"].T, x2 @ p["w_v"].T, x2 @ p["w_q"].T
    k, k_norms = l2_normalize(k_raw)
    q, q_norms = l2_normalize(q_raw)
    alpha = gate(k, v, p["w_alpha"], p["b_alpha"], 0)
    theta = gate(k, v, p["w_theta"], p["b_theta"], 1)
    ca, ct = _clamped(cfg)
    if ca:
        alpha = np.clip(alpha, cfg.alpha_floor, cfg.alpha_ceil)
    if ct:
        theta = np.clip(theta, cfg.theta_floor, cfg.theta_ceil)
    rule = cfg.memory_rule
    eta = gate(k, v, p["w_eta"], p["b_eta"], 0) if rule == "titans" else None
    if gates is not None:
        alpha, theta, eta = gates
    base = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, eta=eta, k_norms=k_norms, q_norms=q_norms)
    if rule in ("moneta", "yaad"):
        # an MLP memory at model width, one sequence; m0 = (W1 [dh, d], W2 [d, dh]) (gpu_forward.rs:1729-1852)
        assert bs == 1
        w1, w2 = m0
        dh = cfg.d_hidden
        if rule == "yaad":
            y, w1s, w2s = orc.miras_mlp_forward(1, k, v, q, alpha, theta, w1, w2, dh, cfg.delta, cfg.lambda_local,
                                                cfg.lambda_2, boundary=(w1, w2))
            bnd = (w1, w2)
        else:
            y, w1s, w2s = orc.miras_mlp_forward(0, k, v, q, alpha, theta, w1, w2, dh, cfg.lp_p, cfg.sign_sharpness,
                                                cfg.lambda_2, cfg.lq_q)
            bnd = None
        return y.reshape(1, s, d).astype(dt), dict(base, w1_states=w1s, w2_states=w2s, boundary=bnd), (w1s[s], w2s[s])
    kh, vh, qh = (to_heads(t, bs, s, nh, hd) for t in (k, v, q))
    ah, th = gates_to_heads(alpha, bs, s, nh), gates_to_heads(theta, bs, s, nh)
    eh = gates_to_heads(eta, bs, s, nh) if eta is not None else None
    B = bs * nh
    z = np.zeros((hd, hd), dt)
    clip = cfg.error_clip
    # DGD: the Delta update without the per-token projection (core/kernels/dgd_forward.cu:6-11)
    mx = F32_MAX if rule == "dgd" else cfg.m_norm_max
    C = cfg.checkpoint_interval
    ys, ms, ss = [], [], []
    mlp_mem = rule == "titans" and getattr(cfg, "memory_layers", 1) == 2
    for b in range(B):
        if mlp_mem:   # per head, the memory a packed two-layer MLP (gpu_forward.rs:1473-1510); no carried clamp
            d_h = cfg.memory_expansion_factor * hd
            act = {"gelu": 0, "silu": 1, "relu": 2}[cfg.memory_activation]
            y, m, sst = orc.titans_mlp_forward(kh[b], vh[b], qh[b], ah[b], th[b], eh[b], m0[b], np.zeros_like(m0[b]),
                                               d_h, act, mx)
        elif C is not None:
            if rule == "hebbian":
                y, m = orc.hebbian_forward(kh[b], vh[b], qh[b], ah[b], m0[b], checkpoint_interval=C)
                sst = None
            else:
                y, m, sst = orc.forward_ckpt(kh[b], vh[b], qh[b], ah[b], th[b], None if eh is None else eh[b], m0[b],
                                             z, C, has_s=rule == "titans", error_clip=clip, m_norm_max=mx)
        elif cfg.proxy and rule in ("delta", "titans"):
            cs = cfg.chunk_size or s
            y, m, sst = orc.chunkwise_forward(kh[b], vh[b], qh[b], ah[b], th[b], None if eh is None else eh[b], m0[b],
                                              z, cs, has_s=rule == "titans", error_clip=clip, m_norm_max=mx)
        elif rule == "titans":
            y, m, sst = orc.titans_forward(kh[b], vh[b], qh[b], ah[b], th[b], eh[b], m0[b], z, clip, mx)
        elif rule == "hebbian":
            y, m = orc.hebbian_forward(kh[b], vh[b], qh[b], ah[b], m0[b])
            sst = None
        else:
            y, m = orc.delta_forward(kh[b], vh[b], qh[b], ah[b], th[b], m0[b], clip, mx)
            sst = None
        ys.append(y); ms.append(m); ss.append(sst)
    y = from_heads(np.stack(ys), bs, s, nh, hd).reshape(bs, s, d)
    m_states = np.stack(ms)
    carried = m_states[:, -1] if mlp_mem else frobenius_clamp(m_states[:, -1], cfg.m_norm_max)
    cache = dict(base, m_states=m_states, s_states=None if ss[0] is None else np.stack(ss))
    return y.astype(dt), cache, carried


def level_backward(p, cfg, cache, d_y, x):
    """-> (grads: dict like p, d_x [bs, s, d])."""
    bs, s, d = x.shape
    nh, hd = cfg.num_heads, cfg.head_dim
    dt = x.dtype
    rule = cfg.memory_rule
    c = cache
    if rule == "swiglu":
        d_x, dg, du, dd = glue.swiglu_backward(d_y.reshape(bs * s, d), x.reshape(bs * s, d), p["gate_proj"],
                                               p["up_proj"], p["down_proj"], c["fused"], c["gate"], c["up"], c["sig"])
        return dict(gate_proj=dg, up_proj=du, down_proj=dd), d_x.reshape(bs, s, d)
    if rule in ("moneta", "yaad"):
        mode = 1 if rule == "yaad" else 0
        p1, p2 = (cfg.delta, cfg.lambda_local) if mode else (cfg.lp_p, cfg.sign_sharpness)
        g = orc.miras_mlp_backward(mode, c["k"], c["v"], c["q"], c["alpha"], c["theta"], c["w1_states"],
                                   c["w2_states"], d_y.reshape(s, d), cfg.d_hidden, p1, p2, cfg.lambda_2, c["boundary"])
        d_alpha, d_theta = g["d_alpha"], g["d_theta"]
        ca, ct = _clamped(cfg)
        if ca:
            d_alpha = np.where((c["alpha"] <= cfg.alpha_floor) | (c["alpha"] >= cfg.alpha_ceil), 0.0, d_alpha)
        if ct:
            d_theta = np.where((c["theta"] <= cfg.theta_floor) | (c["theta"] >= cfg.theta_ceil), 0.0, d_theta)
        return projection_grads(p, x, c, g["d_k"], g["d_v"], g["d_q"], d_alpha, d_theta, None)
    mlp_mem = rule == "titans" and getattr(cfg, "memory_layers", 1) == 2
    kh, vh, qh = (to_heads(c[n], bs, s, nh, hd) for n in ("k", "v", "q"))
    dyh = to_heads(d_y.reshape(bs * s, d), bs, s, nh, hd)
    ah, th = gates_to_heads(c["alpha"], bs, s, nh), gates_to_heads(c["theta"], bs, s, nh)
    eh = gates_to_heads(c["eta"], bs, s, nh) if c["eta"] is not None else None
    B = bs * nh
    clip = cfg.error_clip
    mx = F32_MAX if rule == "dgd" else cfg.m_norm_max
    C = cfg.checkpoint_interval
    gs = []
    for b in range(B):
        m = c["m_states"][b]
        sst = None if c["s_states"] is None else c["s_states"][b]
        if mlp_mem:
            d_h = cfg.memory_expansion_factor * hd
            act = {"gelu": 0, "silu": 1, "relu": 2}[cfg.memory_activation]
            g = orc.titans_mlp_backward(kh[b], vh[b], qh[b], ah[b], th[b], eh[b], m, sst, dyh[b], d_h, act)
        elif C is not None:
            if rule == "hebbian":
                # replay each segment from its checkpoint, then the segment backward
                # (hebbian_backward_checkpointed, gpu_backward.rs:1967-2035)
                g = None
                seed = None
                t_ends = list(range(0, s, C))
                for ci in reversed(range(len(t_ends))):
                    t0, t1 = t_ends[ci], min(t_ends[ci] + C, s)
                    _, traj = orc.hebbian_forward(kh[b][t0:t1], vh[b][t0:t1], qh[b][t0:t1], ah[b][t0:t1], m[ci])
                    gi = orc.hebbian_backward(kh[b], vh[b], qh[b], ah[b], traj, dyh[b], t0, t1, seed)
                    seed = gi["d_m"]
                    if g is None:
                        g = gi
                    else:
                        for n in ("d_k", "d_v", "d_q", "d_alpha"):
                            g[n] = g[n] + gi[n]
            else:
                g = orc.backward_ckpt(kh[b], vh[b], qh[b], ah[b], th[b], None if eh is None else eh[b], m, sst,
                                      dyh[b], C, has_s=rule == "titans", error_clip=clip, m_norm_max=mx)
        elif cfg.proxy and rule in ("delta", "titans"):
            cs = cfg.chunk_size or s
            g = orc.chunkwise_backward(kh[b], vh[b], qh[b], ah[b], th[b], None if eh is None else eh[b], m, sst,
                                       dyh[b], cs, has_s=rule == "titans", error_clip=clip, m_norm_max=mx)
        elif rule == "titans":
            g = orc.titans_backward(kh[b], vh[b], qh[b], ah[b], th[b], eh[b], m, sst, dyh[b], clip)
        elif rule == "hebbian":
            g = orc.hebbian_backward(kh[b], vh[b], qh[b], ah[b], m, dyh[b])
        else:
            g = orc.delta_backward(kh[b], vh[b], qh[b], ah[b], th[b], m, dyh[b], clip)
        gs.append(g)
    stack = lambda n: np.stack([g[n] for g in gs])
    d_k, d_v, d_q = (from_heads(stack(n), bs, s, nh, hd) for n in ("d_k", "d_v", "d_q"))
    d_alpha = gates_from_heads(stack("d_alpha"), bs, s, nh)
    has_theta, has_eta = rule != "hebbian", rule == "titans"
    d_theta = gates_from_heads(stack("d_theta"), bs, s, nh) if has_theta else None
    d_eta = gates_from_heads(stack("d_eta"), bs, s, nh) if has_eta else None
    # straight-through clamps: no gradient where the gate sits on a bound (theta_clamp_mask_cuda)
    ca, ct = _clamped(cfg)
    if ca:
        d_alpha = np.where((c["alpha"] <= cfg.alpha_floor) | (c["alpha"] >= cfg.alpha_ceil), 0.0, d_alpha)
    if ct and has_theta:
        d_theta = np.where((c["theta"] <= cfg.theta_floor) | (c["theta"] >= cfg.theta_ceil), 0.0, d_theta)
    return projection_grads(p, x, c, d_k, d_v, d_q, d_alpha, d_theta, d_eta)


def projection_grads(p, x, c, d_k, d_v, d_q, d_alpha, d_theta, d_eta):
    """accumulate_projection_grads (gpu_backward.rs:2047-2117).  As there, the gate gradients reach the gate
    weights only: the gates' own inputs k, v receive no gradient from them."""
    bs, s, d = x.shape
    x2 = x.reshape(bs * s, d)
    d_k_raw = l2_normalize_backward(d_k, c["k"], c["k_norms"])
    d_q_raw = l2_normalize_backward(d_q, c["q"], c["q_norms"])
    g = dict(w_k=d_k_raw.T @ x2, w_v=d_v.T @ x2, w_q=d_q_raw.T @ x2)
    d_x = d_k_raw @ p["w_k"] + d_v @ p["w_v"] + d_q_raw @ p["w_q"]
    kv = np.concatenate([c["k"], c["v"]], axis=1)
    pre = d_alpha * c["alpha"] * (1.0 - c["alpha"])
    g["w_alpha"], g["b_alpha"] = pre @ kv, np.array([pre.sum()])
    z2, z1 = np.zeros(2 * d, x.dtype), np.zeros(1, x.dtype)
    if d_theta is not None:
        pre = d_theta * (1.0 - np.exp(-c["theta"]))
        g["w_theta"], g["b_theta"] = pre @ kv, np.array([pre.sum()])
    else:
        g["w_theta"], g["b_theta"] = z2, z1
    if d_eta is not None:
        pre = d_eta * c["eta"] * (1.0 - c["eta"])
        g["w_eta"], g["b_eta"] = pre @ kv, np.array([pre.sum()])
    else:
        g["w_eta"], g["b_eta"] = z2, z1
    return g, d_x.reshape(bs, s, d)


# ── TNT: shards of local chunks around a global memory (gpu_forward.rs:1878-2293, gpu_backward.rs:1201-1632) ──
GLOBAL_RETENTION = 0.95


def _pad(t, n, padded):
    """[nh, n, ...] -> [nh, padded, ...], zeros behind."""
    out = np.zeros((t.shape[0], padded) + t.shape[2:], t.dtype)
    out[:, :n] = t
    return out


def tnt_forward(p, cfg, x, m0, cg, cl, gates=None):
    """x [s, d], m0 [nh, hd, hd] (global memory per head) -> y [s, d], cache (list of per-shard dicts), final
    global memory.  gates: per-shard list of (alpha, theta, eta) to use instead of the computed ones."""
    s, d = x.shape
    nh, hd = cfg.num_heads, cfg.head_dim
    dt = x.dtype
    titans = cfg.memory_rule == "titans"
    m_glob = m0.copy()
    y_full = np.zeros((s, d), dt)
    shards = []
    for si, t0 in enumerate(range(0, s, cg)):
        t1 = min(t0 + cg, s)
        n = t1 - t0
        n_batch = -(-n // cl)
        padded = n_batch * cl
        xs = x[t0:t1]
        k, k_norms = l2_normalize(xs @ p["w_k"].T)
        q, q_norms = l2_normalize(xs @ p["w_q"].T)
        v = xs @ p["w_v"].T
        alpha = gate(k, v, p["w_alpha"], p["b_alpha"], 0)
        theta = gate(k, v, p["w_theta"], p["b_theta"], 1)
        ca, ct = _clamped(cfg)
        if ca:
            alpha = np.clip(alpha, cfg.alpha_floor, cfg.alpha_ceil)
        if ct:
            theta = np.clip(theta, cfg.theta_floor, cfg.theta_ceil)
        eta = gate(k, v, p["w_eta"], p["b_eta"], 0) if titans else None
        if gates is not None:
            alpha, theta, eta = gates[si]
        kh, vh, qh = (_pad(to_heads(t, 1, n, nh, hd), n, padded) for t in (k, v, q))
        ah, th = (_pad(gates_to_heads(g, 1, n, nh), n, padded) for g in (alpha, theta))
        eh = _pad(gates_to_heads(eta, 1, n, nh), n, padded) if titans else None
        y_local = np.zeros((nh, padded, hd), dt)
        ms, ss = [], []
        z = np.zeros((hd, hd), dt)
        for h in range(nh):
            for b in range(n_batch):
                sl = slice(b * cl, (b + 1) * cl)
                if titans:
                    y, m, sst = orc.titans_forward(kh[h, sl], vh[h, sl], qh[h, sl], ah[h, sl], th[h, sl], eh[h, sl],
                                                   m_glob[h], z, cfg.error_clip, cfg.m_norm_max)
                    ss.append(sst)
                else:
                    y, m = orc.delta_forward(kh[h, sl], vh[h, sl], qh[h, sl], ah[h, sl], th[h, sl], m_glob[h],
                                             cfg.error_clip, cfg.m_norm_max)
                y_local[h, sl] = y
                ms.append(m)
        y_full[t0:t1] = from_heads(y_local, 1, padded, nh, hd)[:n]
        mean = y_local[:, :n].sum(1) / dt.type(n)          # [nh, hd]: key and value summary alike
        m_glob = dt.type(GLOBAL_RETENTION) * m_glob + np.einsum("hi,hj->hij", mean, mean)
        m_glob = frobenius_clamp(m_glob, cfg.m_norm_max)
        shards.append(dict(t0=t0, n=n, n_batch=n_batch, padded=padded, k=k, v=v, q=q, k_norms=k_norms, q_norms=q_norms,
                           alpha=alpha, theta=theta, eta=eta, kh=kh, vh=vh, qh=qh, ah=ah, th=th, eh=eh,
                           m_states=np.stack(ms), s_states=np.stack(ss) if titans else None, summary=mean))
    return y_full, shards, m_glob


def tnt_backward(p, cfg, shards, d_y, x, cl, first_retained=0, per_head_memory_gradient=False):
    """-> (grads, d_x).  The rule's backward returns the gradient of the initial memory summed over the chains of
    a call; as in the reference (gpu_backward.rs:1408-1418) the whole sum is added to head 0's global memory
    gradient — the gradient itself for one head.  per_head_memory_gradient: every chain's gradient goes to its own
    head's global memory instead, which is the gradient of the forward for any number of heads."""
    s, d = x.shape
    nh, hd = cfg.num_heads, cfg.head_dim
    dt = x.dtype
    titans = cfg.memory_rule == "titans"
    d_k_tot, d_v_tot, d_q_tot = np.zeros((s, d), dt), np.zeros((s, d), dt), np.zeros((s, d), dt)
    g = {n: np.zeros(2 * d, dt) for n in ("w_alpha", "w_theta", "w_eta")}
    g.update({n: np.zeros(1, dt) for n in ("b_alpha", "b_theta", "b_eta")})
    d_m_carry = np.zeros((nh, hd, hd), dt)
    for si in reversed(range(len(shards))):
        c = shards[si]
        n, n_batch, padded, t0 = c["n"], c["n_batch"], c["padded"], c["t0"]
        mean = c["summary"]
        d_m_old = dt.type(GLOBAL_RETENTION) * d_m_carry
        d_k_sum = np.einsum("hij,hi->hj", d_m_carry, mean)      # M_new = a M + v_sum k_sum^T
        d_v_sum = np.einsum("hij,hj->hi", d_m_carry, mean)
        if si < first_retained:
            d_m_carry = d_m_old
            continue
        d_local = np.repeat(((d_k_sum + d_v_sum) / dt.type(n))[:, None, :], n, axis=1)   # [nh, n, hd]
        d_y_comb = d_y[t0:t0 + n] + from_heads(d_local, 1, n, nh, hd)
        dyh = _pad(to_heads(d_y_comb, 1, n, nh, hd), n, padded)
        dk, dv, dq = (np.zeros((nh, padded, hd), dt) for _ in range(3))
        da, dth, de = (np.zeros((nh, padded), dt) for _ in range(3))
        d_m_sum = np.zeros((hd, hd), dt)
        d_m_head = np.zeros((nh, hd, hd), dt)
        for h in range(nh):
            for b in range(n_batch):
                sl = slice(b * cl, (b + 1) * cl)
                i = h * n_batch + b
                m_i = c["m_states"][i]
                s_i = c["s_states"][i] if titans else None
                if cfg.proxy:   # a proxy level keeps the final states only; they stand in for every state
                    m_i = np.ascontiguousarray(np.broadcast_to(m_i[-1], m_i.shape))
                    s_i = np.ascontiguousarray(np.broadcast_to(s_i[-1], s_i.shape)) if titans else None
                if titans:
                    gi = orc.titans_backward(c["kh"][h, sl], c["vh"][h, sl], c["qh"][h, sl], c["ah"][h, sl], c["th"][h, sl],
                                             c["eh"][h, sl], m_i, s_i, dyh[h, sl], cfg.error_clip)
                    de[h, sl] = gi["d_eta"]
                else:
                    gi = orc.delta_backward(c["kh"][h, sl], c["vh"][h, sl], c["qh"][h, sl], c["ah"][h, sl], c["th"][h, sl],
                                            m_i, dyh[h, sl], cfg.error_clip)
                dk[h, sl], dv[h, sl], dq[h, sl] = gi["d_k"], gi["d_v"], gi["d_q"]
                da[h, sl], dth[h, sl] = gi["d_alpha"], gi["d_theta"]
                d_m_sum += gi["d_m"]
                d_m_head[h] += gi["d_m"]
        if not cfg.proxy:
            if per_head_memory_gradient:
                d_m_old += d_m_head
            else:
                d_m_old[0] += d_m_sum
        ca, ct = _clamped(cfg)
        if ca:
            da = np.where((c["ah"] <= cfg.alpha_floor) | (c["ah"] >= cfg.alpha_ceil), 0.0, da)
        if ct:
            dth = np.where((c["th"] <= cfg.theta_floor) | (c["th"] >= cfg.theta_ceil), 0.0, dth)
        dk_dm, dv_dm, dq_dm = (from_heads(t, 1, padded, nh, hd)[:n] for t in (dk, dv, dq))
        da_dm, dth_dm, de_dm = (t.sum(0)[:n] for t in (da, dth, de))
        d_k_tot[t0:t0 + n] += l2_normalize_backward(dk_dm, c["k"], c["k_norms"])
        d_v_tot[t0:t0 + n] += dv_dm
        d_q_tot[t0:t0 + n] += l2_normalize_backward(dq_dm, c["q"], c["q_norms"])
        kv = np.concatenate([c["k"], c["v"]], axis=1)
        pre = da_dm * c["alpha"] * (1.0 - c["alpha"])
        g["w_alpha"] += pre @ kv; g["b_alpha"] += pre.sum()
        pre = dth_dm * (1.0 - np.exp(-c["theta"]))
        g["w_theta"] += pre @ kv; g["b_theta"] += pre.sum()
        if titans:
            pre = de_dm * c["eta"] * (1.0 - c["eta"])
            g["w_eta"] += pre @ kv; g["b_eta"] += pre.sum()
        d_m_carry = d_m_old
    g["w_k"], g["w_v"], g["w_q"] = d_k_tot.T @ x, d_v_tot.T @ x, d_q_tot.T @ x
    d_x = d_k_tot @ p["w_k"] + d_v_tot @ p["w_v"] + d_q_tot @ p["w_q"]
    return g, d_x
