"""TEST INFRASTRUCTURE ONLY — the reference's whole training step on the CPU: gpu_cms_forward
(core/src/gpu_forward.rs:760-1117) and gpu_cms_backward (core/src/gpu_backward.rs:143-455) composed from the
oracle's pieces: embedding / LayerNorm / cross-entropy of oracle/model_glue.py, the attention of pyoracle (bf16
storage, as the reference runs it) or a plain float attention written here (for float64 finite differences),
and the level step of oracle/memory_level.py (TNT levels when a parallel configuration is given).
tests/test_oracle_cms_model.py pins the float attention against the bf16 one and the composed backward against
central differences of the float64 forward.

p: dict with w_embed [v, d], w_q, w_k, w_v, w_o [d, d], w_unembed [d, v], levels (list of level dicts) and, for
the residual variant, ln_attn_gamma / ln_attn_beta / ln_mem_gamma / ln_mem_beta [d].
cfg: object with d_model, vocab_size, num_heads, head_dim, window_size, seq_len, n_persistent, residual, levels,
parallel (None or an object with tnt_global_chunk_size, tnt_local_chunk_size).
memories: per level [bs*nh, hd, hd].
"""
import numpy as np

from . import memory_level as ML
from . import model_glue as G
from . import pyoracle as orc

LN_EPS = 1e-5


def swa_mask(s, window, n_p):
    """Query t sees the prefix keys [0, min(t+1, n_p)) and the local keys [max(t+1-window, n_p), t]."""
    m = np.zeros((s, s), bool)
    for t in range(s):
        m[t, :min(t + 1, n_p)] = True
        m[t, max(t + 1 - window, n_p):t + 1] = True
    return m


def swa_float_forward(q, k, v, window, nh, n_p):
    """q, k, v [s, nh*hd] in any float type -> out [s, nh*hd], weights [nh, s, s]."""
    s, d = q.shape
    hd = d // nh
    mask = swa_mask(s, window, n_p)
    out = np.zeros_like(q)
    w = np.zeros((nh, s, s), q.dtype)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        sc = q[:, sl] @ k[:, sl].T / np.sqrt(q.dtype.type(hd))
        sc = np.where(mask, sc, -np.inf)
        e = np.exp(sc - sc.max(1, keepdims=True))
        w[h] = e / e.sum(1, keepdims=True)
        out[:, sl] = w[h] @ v[:, sl]
    return out, w


def swa_float_backward(q, k, v, w, d_out, nh):
    s, d = q.shape
    hd = d // nh
    dq, dk, dv = np.zeros_like(q), np.zeros_like(q), np.zeros_like(q)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        dw = d_out[:, sl] @ v[:, sl].T
        ds = w[h] * (dw - (w[h] * dw).sum(1, keepdims=True)) / np.sqrt(q.dtype.type(hd))
        dq[:, sl] = ds @ k[:, sl]
        dk[:, sl] = ds.T @ q[:, sl]
        dv[:, sl] = w[h].T @ d_out[:, sl]
    return dq, dk, dv


def _tnt(cfg, lcfg, bs):
    return cfg.parallel is not None and bs == 1 and lcfg.memory_rule in ("titans", "delta")


def forward(p, cfg, input_ids, target_ids, active, memories, quantize=True, gates=None):
    """-> (loss, cache, memories after the step).  quantize: bf16 attention storage as the reference; False: the
    float attention in the dtype of the parameters.  gates: per level, gate values to hold fixed (see
    memory_level.level_forward)."""
    s, d, v, nh, hd = cfg.seq_len, cfg.d_model, cfg.vocab_size, cfg.num_heads, cfg.head_dim
    ids, tgt = np.asarray(input_ids), np.asarray(target_ids)
    bs = len(ids) // s
    n = bs * s
    dt = p["w_embed"].dtype
    emb = G.embedding_gather(p["w_embed"], ids)
    c = dict(ids=ids, tgt=tgt, emb=emb, bs=bs, active=list(active), quantize=quantize)
    src = emb
    if cfg.residual:
        c["ln_attn_out"], c["ln_attn_mean"], c["ln_attn_rstd"] = G.layer_norm_forward(emb, p["ln_attn_gamma"],
                                                                                      p["ln_attn_beta"], LN_EPS)
        src = c["ln_attn_out"]
    q, k, vv = src @ p["w_q"].T, src @ p["w_k"].T, src @ p["w_v"].T
    attn = np.zeros((n, d), dt)
    if quantize:
        qb, kb, vb = (orc.f32_to_bf16(t.astype(np.float32)).reshape(bs, s, d) for t in (q, k, vv))
        out, aw = orc.swa_forward(qb, kb, vb, cfg.window_size, nh, cfg.n_persistent)
        attn = orc.bf16_to_f32(out).reshape(n, d).astype(dt)
        c.update(qb=qb, kb=kb, vb=vb, aw=aw)
    else:
        c["w"] = []
        for b in range(bs):
            r = slice(b * s, (b + 1) * s)
            attn[r], w = swa_float_forward(q[r], k[r], vv[r], cfg.window_size, nh, cfg.n_persistent)
            c["w"].append(w)
        c.update(q=q, k=k, v=vv)
    c["attn"] = attn
    mem_in = emb
    if cfg.residual:
        c["res_attn"] = emb + attn
        c["ln_mem_out"], c["ln_mem_mean"], c["ln_mem_rstd"] = G.layer_norm_forward(c["res_attn"], p["ln_mem_gamma"],
                                                                                   p["ln_mem_beta"], LN_EPS)
        mem_in = c["ln_mem_out"]
    c["mem_in"] = mem_in
    ys, caches, new_mem = [], [], []
    for lv, lcfg in enumerate(cfg.levels):
        gl = None if gates is None else gates[lv]
        if active[lv] or lcfg.memory_rule == "swiglu":
            if _tnt(cfg, lcfg, bs):
                y, lc, m = ML.tnt_forward(p["levels"][lv], lcfg, mem_in, memories[lv], cfg.parallel.tnt_global_chunk_size,
                                          cfg.parallel.tnt_local_chunk_size, gl)
            else:
                y, lc, m = ML.level_forward(p["levels"][lv], lcfg, mem_in.reshape(bs, s, d), memories[lv], gl)
                y = y.reshape(n, d)
        elif getattr(lcfg, "memory_layers", 1) == 2 and lcfg.memory_rule == "titans":
            raise RuntimeError(f"Frozen TitansLMM MLP level unsupported (level {lv})")   # gpu_forward.rs:32-39
        elif lcfg.memory_rule in ("moneta", "yaad"):   # frozen_mlp_fallback (gpu_forward.rs:45-57, 1010-1012): zeros
            y, lc, m = np.zeros((n, d), dt), None, memories[lv]
        else:   # gpu_memory_read_only: y = M_h q_h with the projection q as it comes, batch slot 0's memories
            qr = (mem_in @ p["levels"][lv]["w_q"].T).reshape(n, nh, hd)
            y = np.einsum("hij,nhj->nhi", memories[lv][:nh], qr).reshape(n, d)
            lc, m = None, memories[lv]
        ys.append(y.astype(dt)); caches.append(lc); new_mem.append(m)
    comb = np.sum(ys, axis=0)
    if len(ys) > 2:
        comb = comb * dt.type(1.0 / np.sqrt(len(ys)))
    c.update(level_caches=caches, comb=comb)
    if cfg.residual:
        c["res_final"] = c["res_attn"] + comb
        proj = c["res_final"] @ p["w_o"].T
    else:
        c["gate"] = ML.sigmoid(comb)
        c["gated"] = attn * c["gate"]
        proj = c["gated"] @ p["w_o"].T
    c["proj"] = proj
    c["logits"] = proj @ p["w_unembed"]
    valid = int(((tgt >= 0) & (tgt < v)).sum())
    loss = G.cross_entropy_forward(c["logits"], tgt) / valid if valid else 0.0
    return float(loss), c, new_mem


def backward(p, cfg, c):
    """-> dict of gradients: w_embed, w_q, w_k, w_v, w_o, w_unembed, (ln_*), levels (list of dicts or None)."""
    s, d, v, nh = cfg.seq_len, cfg.d_model, cfg.vocab_size, cfg.num_heads
    bs = c["bs"]
    n = bs * s
    tgt = c["tgt"]
    valid = int(((tgt >= 0) & (tgt < v)).sum())
    d_logits = G.cross_entropy_backward(c["logits"], tgt, 1.0 / (valid if valid else 1))
    g = dict(w_unembed=c["proj"].T @ d_logits)
    d_proj = d_logits @ p["w_unembed"].T
    d_gated = d_proj @ p["w_o"]
    g["w_o"] = d_proj.T @ (c["res_final"] if cfg.residual else c["gated"])
    if cfg.residual:
        d_comb, d_attn = d_gated.copy(), d_gated.copy()
    else:
        d_attn = d_gated * c["gate"]
        d_comb = d_gated * c["attn"] * c["gate"] * (1.0 - c["gate"])
    k_lv = len(cfg.levels)
    if k_lv > 2:
        d_comb = d_comb / np.sqrt(d_comb.dtype.type(k_lv))
    d_mem_in = np.zeros((n, d), d_comb.dtype)
    g["levels"] = []
    for lv, lcfg in enumerate(cfg.levels):
        lc = c["level_caches"][lv]
        if lc is None:   # frozen: no gradient in this path
            g["levels"].append(None)
            continue
        if _tnt(cfg, lcfg, bs):
            gl, dx = ML.tnt_backward(p["levels"][lv], lcfg, lc, d_comb, c["mem_in"], cfg.parallel.tnt_local_chunk_size)
        else:
            gl, dx = ML.level_backward(p["levels"][lv], lcfg, lc, d_comb.reshape(bs, s, d), c["mem_in"].reshape(bs, s, d))
            dx = dx.reshape(n, d)
        g["levels"].append(gl)
        d_mem_in += dx
    if cfg.residual:
        d_res, g["ln_mem_gamma"], g["ln_mem_beta"] = G.layer_norm_backward(d_mem_in, c["res_attn"], p["ln_mem_gamma"],
                                                                           c["ln_mem_mean"], c["ln_mem_rstd"])
        d_attn = d_attn + d_res
    dq, dk, dv = (np.zeros((n, d), d_attn.dtype) for _ in range(3))
    if c["quantize"]:
        a, b_, c_ = orc.swa_backward(c["qb"], c["kb"], c["vb"], c["aw"], d_attn.reshape(bs, s, d).astype(np.float32),
                                     cfg.window_size, nh, cfg.n_persistent)
        dq, dk, dv = (t.reshape(n, d) for t in (a, b_, c_))
    else:
        for b in range(bs):
            r = slice(b * s, (b + 1) * s)
            dq[r], dk[r], dv[r] = swa_float_backward(c["q"][r], c["k"][r], c["v"][r], c["w"][b], d_attn[r], nh)
    src = c["ln_attn_out"] if cfg.residual else c["emb"]
    d_src = dq @ p["w_q"] + dk @ p["w_k"] + dv @ p["w_v"]
    g["w_q"], g["w_k"], g["w_v"] = dq.T @ src, dk.T @ src, dv.T @ src
    if cfg.residual:
        d_emb, g["ln_attn_gamma"], g["ln_attn_beta"] = G.layer_norm_backward(d_src, c["emb"], p["ln_attn_gamma"],
                                                                             c["ln_attn_mean"], c["ln_attn_rstd"])
        d_emb = d_emb + d_attn
    else:
        d_emb = d_src + d_mem_in
    g["w_embed"] = G.embedding_scatter_add(d_emb, c["ids"], np.zeros_like(p["w_embed"]))
    return g
