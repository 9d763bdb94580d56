"""TEST INFRASTRUCTURE ONLY: CPU restatement of the opaque VJP blocks of the Wengert tape for the
Delta rule and the Titans LMM in their default configuration (L2 attentional bias, identity
feature map, no Conv1D, linear memory, EMA momentum): the rule structs' full-sequence `step`
(projections, row L2 norm, gates, token recurrence) and `step_backward`, with the saved-buffer
layouts of the tape adapters.  numpy, float32 or float64 by the dtype of `embedded`; the token
recurrence itself is the C oracle's (pyoracle.delta_* / titans_*).

Follows, line by line:
  core/src/delta_rule.rs:278-412 (step), :414-640 (step_backward)
  core/src/titans_lmm.rs:1314-1533 (step), :1535-1762 (step_backward), :515-567 (projection_backward)
  core/src/tensor.rs:202-207 (sigmoid, clamped at +-15), :222-227 (softplus), :296-351 (row L2 norm)
  core/src/opaque_adapters.rs:93-113 (flat parameter order), :290-304 and :386-401 (saved layouts),
  :1004-1068 (frozen read), core/src/tape.rs:141-150 (backward signature)
Pinned by tests/test_oracle_blocks.py: finite differences of the float64 forward for every input and
parameter (clamps inactive), hand cases for the clamp masks.
"""
import numpy as np

from . import pyoracle as orc

F32_MAX = orc.F32_MAX


def sigmoid(x):
    x = np.asarray(x)
    out = 1.0 / (1.0 + np.exp(-np.clip(x, -15.0, 15.0)))
    return np.where(x >= 15.0, 1.0, np.where(x <= -15.0, 0.0, out)).astype(x.dtype)


def softplus(x):
    x = np.asarray(x)
    out = np.log1p(np.exp(np.clip(x, -15.0, 15.0)))
    return np.where(x >= 15.0, x, np.where(x <= -15.0, 0.0, out)).astype(x.dtype)


def bf16_round(w):
    """The projections read the bf16 copy of the three matrices (core/src/bf16.rs:108-112 as_f32 of the
    stored copy; round to nearest even, tensor.rs:37-42); gradients go to the fp32 master."""
    return orc.bf16_to_f32(orc.f32_to_bf16(np.ascontiguousarray(w, np.float32))).astype(w.dtype).reshape(w.shape)


def l2_normalize_rows(x, eps=1e-8):
    norms = np.sqrt((x * x).sum(axis=1))
    return x / np.maximum(norms, eps)[:, None], norms


def l2_normalize_rows_backward(d_out, x_norm, norms, eps=1e-8):
    dot = (d_out * x_norm).sum(axis=1, keepdims=True)
    sphere = (d_out - x_norm * dot) / np.where(norms >= eps, norms, 1.0)[:, None]
    return np.where((norms >= eps)[:, None], sphere, d_out / eps)


# ── flat parameter buffer (opaque_adapters.rs:93-113, mandatory fields only) ──
FIELDS = ("w_k_mem", "w_v_mem", "w_q_mem", "w_alpha", "b_alpha", "w_theta", "b_theta", "w_eta", "b_eta")


def field_sizes(d):
    return {"w_k_mem": d * d, "w_v_mem": d * d, "w_q_mem": d * d, "w_alpha": 2 * d, "b_alpha": 1,
            "w_theta": 2 * d, "b_theta": 1, "w_eta": 2 * d, "b_eta": 1}


def params_from_flat(flat, d):
    out, off = {}, 0
    for n, sz in field_sizes(d).items():
        out[n] = flat[off:off + sz]
        off += sz
    for n in ("w_k_mem", "w_v_mem", "w_q_mem"):
        out[n] = out[n].reshape(d, d)
    return out


def params_to_flat(p, total_len=None):
    flat = np.concatenate([np.asarray(p[n]).reshape(-1) for n in FIELDS])
    if total_len is not None and total_len > flat.size:   # level_params_grads_to_flat_padded
        flat = np.concatenate([flat, np.zeros(total_len - flat.size, flat.dtype)])
    return flat


def init_params(d, seed, dtype=np.float32):
    rs = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: ((rs.random((d, d)) * 2 - 1) * lim) for n in ("w_k_mem", "w_v_mem", "w_q_mem")}
    for g, b in (("alpha", -2.0), ("theta", -1.0), ("eta", 1.5)):
        p["w_" + g] = rs.standard_normal(2 * d) * 0.3
        p["b_" + g] = np.array([b])
    return {n: np.ascontiguousarray(v, dtype) for n, v in p.items()}


# ── the block: forward ──
def rule_step(kind, p, embedded, m0=None, s0=None, alpha_lim=(0.0, 1.0), theta_lim=(0.0, F32_MAX),
              round_weights=True):
    """-> (y [s,d], cache dict with the rule cache's fields).  kind: "delta" | "titans".
    round_weights=False keeps the matrices as given (finite-difference checks perturb them)."""
    dt = embedded.dtype
    s, d = embedded.shape
    rw = bf16_round if round_weights else (lambda w: w)
    k = embedded @ rw(p["w_k_mem"]).T
    v = embedded @ rw(p["w_v_mem"]).T
    q = embedded @ rw(p["w_q_mem"]).T
    k, k_norms = l2_normalize_rows(k)
    q, q_norms = l2_normalize_rows(q)
    concat = np.concatenate([k, v], axis=1)
    c = dict(k_mem=k, v_mem=v, q_mem=q, concat_kv=concat, k_mem_norms=k_norms, q_mem_norms=q_norms)
    c["alpha_pre"] = concat @ p["w_alpha"] + p["b_alpha"][0]
    c["alpha"] = np.clip(sigmoid(c["alpha_pre"]), alpha_lim[0], alpha_lim[1])
    c["theta_pre"] = concat @ p["w_theta"] + p["b_theta"][0]
    c["theta"] = np.clip(softplus(c["theta_pre"]), theta_lim[0], theta_lim[1])
    m0 = np.zeros((d, d), dt) if m0 is None else m0
    args = [np.ascontiguousarray(a, dt) for a in (k, v, q, c["alpha"], c["theta"])]
    if kind == "titans":
        c["eta_pre"] = concat @ p["w_eta"] + p["b_eta"][0]
        c["eta"] = sigmoid(c["eta_pre"])
        s0 = np.zeros((d, d), dt) if s0 is None else s0
        y, ms, ss = orc.titans_forward(*args, np.ascontiguousarray(c["eta"], dt), np.ascontiguousarray(m0, dt),
                                       np.ascontiguousarray(s0, dt))
        c["s_states"] = ss
    else:
        y, ms = orc.delta_forward(*args, np.ascontiguousarray(m0, dt))
    c["m_states"] = ms
    c["error"] = np.einsum("tij,tj->ti", ms[:-1], k) - v            # e_t = M_t k_t - v_t
    c["grad_outer"] = np.einsum("ti,tj->tij", c["error"], k)        # outer(e_t, k_t)
    c["y"] = y
    for n in c:
        c[n] = np.ascontiguousarray(c[n], dt)
    return y, c


# ── the block: backward ──
def rule_step_backward(kind, p, c, d_y, embedded, alpha_lim=(0.0, 1.0), theta_lim=(0.0, F32_MAX),
                       round_weights=True):
    """-> (parameter gradients dict, d_embedded)."""
    dt = embedded.dtype
    rw = bf16_round if round_weights else (lambda w: w)
    s, d = embedded.shape
    a = [c[n] for n in ("k_mem", "v_mem", "q_mem", "alpha", "theta")]
    if kind == "titans":
        g = orc.titans_backward(*a, c["eta"], c["m_states"], c["s_states"], np.ascontiguousarray(d_y, dt))
    else:
        g = orc.delta_backward(*a, c["m_states"], np.ascontiguousarray(d_y, dt))
    d_k, d_v, d_q = g["d_k"].copy(), g["d_v"].copy(), g["d_q"].copy()
    # gates; the straight-through clamp masks differ between the two rules
    d_alpha_pre = g["d_alpha"] * c["alpha"] * (1.0 - c["alpha"])
    if kind == "titans":   # titans_lmm.rs:1707-1719: masks on the unclamped gate values
        a_raw, t_raw = sigmoid(c["alpha_pre"]), softplus(c["theta_pre"])
        d_alpha_pre = d_alpha_pre * ~((a_raw <= alpha_lim[0]) | (a_raw >= alpha_lim[1]))
    else:                  # delta_rule.rs:566-569: theta mask on the clamped value, none for alpha
        t_raw = c["theta"]
    d_theta_pre = g["d_theta"] * sigmoid(c["theta_pre"]) * ~((t_raw <= theta_lim[0]) | (t_raw >= theta_lim[1]))
    grads = {n: np.zeros_like(np.asarray(v), dtype=dt) for n, v in p.items()}
    pre = {"alpha": d_alpha_pre, "theta": d_theta_pre}
    if kind == "titans":
        pre["eta"] = g["d_eta"] * c["eta"] * (1.0 - c["eta"])
    for name, dp in pre.items():
        grads["w_" + name] = dp @ c["concat_kv"]
        grads["b_" + name] = np.array([dp.sum()], dt)
        d_k += np.outer(dp, p["w_" + name][:d])       # concat backward: the gates read k and v
        d_v += np.outer(dp, p["w_" + name][d:])
    d_k = l2_normalize_rows_backward(d_k, c["k_mem"], c["k_mem_norms"])
    d_q = l2_normalize_rows_backward(d_q, c["q_mem"], c["q_mem_norms"])
    grads["w_k_mem"] = d_k.T @ embedded
    grads["w_v_mem"] = d_v.T @ embedded
    grads["w_q_mem"] = d_q.T @ embedded
    d_emb = d_k @ rw(p["w_k_mem"]) + d_v @ rw(p["w_v_mem"]) + d_q @ rw(p["w_q_mem"])
    return {n: np.ascontiguousarray(v, dt) for n, v in grads.items()}, np.ascontiguousarray(d_emb, dt)


# ── saved buffers of the tape adapters ──
DELTA_CACHE = ("m_states", "k_mem", "v_mem", "q_mem", "concat_kv", "alpha_pre", "alpha", "theta_pre", "theta",
               "error", "grad_outer", "y", "k_mem_norms", "q_mem_norms")
TITANS_CACHE = ("m_states", "s_states", "k_mem", "v_mem", "q_mem", "concat_kv", "alpha_pre", "alpha", "theta_pre",
                "theta", "eta_pre", "eta", "error", "grad_outer", "y", "k_mem_norms", "q_mem_norms")


def saved_buffers(kind, p, c, embedded, alpha_lim=(0.0, 1.0), theta_lim=(0.0, F32_MAX)):
    """The `saved` list of the opaque block in the newest recording format (float32 arrays).
    Delta meta (opaque_adapters.rs:1199, :1170-1172): [seq_len, d, bias = 2 (L2, moneta.rs:1233-1245),
    sign_sharpness, theta_floor, theta_ceil, fm_kind = 0 (identity), fm_sigma, 1 (norms present), alpha_floor,
    alpha_ceil, kernel_size = 0].
    Titans meta (:1279): [seq_len, d, bias, sign_sharpness, momentum_kind = 1 (EMA), theta_floor, theta_ceil,
    fm_kind, fm_sigma, 1 (norms present), alpha_floor, alpha_ceil, memory_layers = 1, expansion, activation,
    kernel_size = 0]."""
    f = np.float32
    s, d = embedded.shape
    if kind == "delta":
        meta = [s, d, 2.0, 10.0, theta_lim[0], theta_lim[1], 0.0, 1.0, 1.0, alpha_lim[0], alpha_lim[1], 0.0]
        names = DELTA_CACHE
    else:
        meta = [s, d, 2.0, 10.0, 1.0, theta_lim[0], theta_lim[1], 0.0, 1.0, 1.0, alpha_lim[0], alpha_lim[1], 1.0, 4.0,
                0.0, 0.0]
        names = TITANS_CACHE
    saved = [np.array(meta, f), params_to_flat(p).astype(f), np.ascontiguousarray(embedded, f).reshape(-1)]
    saved += [np.ascontiguousarray(c[n], f).reshape(-1) for n in names]
    return saved


def frozen_read_backward(m_frozen, d_y):
    """opaque_adapters.rs:1009-1068 with the identity feature map: d_q[t] = M^T d_y[t]."""
    return d_y @ m_frozen
