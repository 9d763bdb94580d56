"""TEST INFRASTRUCTURE ONLY — numpy restatement of the reference's kernels around the memory path
(LayerNorm, embedding, transpose copy, cross-entropy, TNT helpers, 1-D pooling, M3 helpers).  Each function
cites the reference lines it follows and computes in the dtype of its inputs (float32 = the arithmetic the
reference runs, float64 for pinning).  Only tests/, the smoke check and bench.py's CPU baseline may import it.
Pinned by tests/test_oracle_model_glue.py: torch's library routines and autograd in float64, and for the M3
helpers the known answers that the reference's own tests hold (core/tests/test_m3.rs), kept as
tests/golden/m3_known_answers.json.
"""
import numpy as np


# core/kernels/layer_norm.cu:27-77
def layer_norm_forward(x, gamma, beta, eps):
    d = x.shape[1]
    mean = x.sum(1) / d
    var = (x * x).sum(1) / d - mean * mean
    rstd = 1.0 / np.sqrt(var + x.dtype.type(eps))
    out = gamma * ((x - mean[:, None]) * rstd[:, None]) + beta
    return out.astype(x.dtype), mean.astype(x.dtype), rstd.astype(x.dtype)


# core/kernels/layer_norm.cu:81-136 (d_gamma, d_beta: sums over rows, added to the caller's buffers)
def layer_norm_backward(d_out, x, gamma, mean, rstd):
    d = x.shape[1]
    xh = (x - mean[:, None]) * rstd[:, None]
    dg = d_out * gamma
    s1, s2 = dg.sum(1, keepdims=True), (dg * xh).sum(1, keepdims=True)
    d_x = rstd[:, None] * (1.0 / d) * (d * dg - s1 - xh * s2)
    return d_x.astype(x.dtype), (d_out * xh).sum(0).astype(x.dtype), d_out.sum(0).astype(x.dtype)


# core/kernels/embedding.cu:23-38, 44-60, 68-80
def embedding_gather(w, ids):
    return w[ids]


def embedding_scatter_add(d_embedded, ids, d_embed):
    out = d_embed.copy()
    for t, tok in enumerate(ids):   # position order
        out[tok] += d_embedded[t]
    return out


def transpose_copy(src):
    return np.ascontiguousarray(src.T)


# core/kernels/cross_entropy.cu:29-84 (sum of the rows' NLL; invalid targets skipped), :101-160
def cross_entropy_forward(logits, targets):
    vocab = logits.shape[1]
    loss = logits.dtype.type(0)
    for t, tgt in enumerate(targets):
        if tgt < 0 or tgt >= vocab:
            continue
        row = logits[t]
        mx = row.max()
        loss += -(row[tgt] - mx - np.log(np.exp(row - mx).sum()))
    return loss


def cross_entropy_backward(logits, targets, inv_count):
    vocab = logits.shape[1]
    out = np.zeros_like(logits)
    for t, tgt in enumerate(targets):
        if tgt < 0 or tgt >= vocab:
            continue
        row = logits[t]
        e = np.exp(row - row.max())
        g = e / e.sum()
        g[tgt] -= 1.0
        out[t] = g * logits.dtype.type(inv_count)
    return out


# core/kernels/tnt_forward.cu:26-40, 62-79, 101-114; tnt_backward.cu:27-48, 69-82, 103-113
def tnt_broadcast_m(m, n_local):
    return np.tile(m.reshape(1, -1), (n_local, 1))


def tnt_shard_summary_mean(local_y):
    mean = local_y.sum(0) / local_y.dtype.type(local_y.shape[0])
    return mean, mean.copy()


def tnt_global_update(m, k_sum, v_sum, alpha):
    return m.dtype.type(alpha) * m + np.outer(v_sum, k_sum)


def tnt_global_update_backward(d_m_new, k_sum, v_sum, alpha, d_k_sum, d_v_sum):
    return (d_m_new.dtype.type(alpha) * d_m_new, d_k_sum + d_m_new.T @ v_sum, d_v_sum + d_m_new @ k_sum)


def tnt_shard_summary_mean_backward(d_k_sum, d_v_sum, d_local_y):
    return d_local_y + (d_k_sum + d_v_sum) / d_local_y.dtype.type(d_local_y.shape[0])


# core/kernels/pool_ops.cu (groups of C tokens; tokens past the last full group take no part)
def mean_pool_1d(x, C):
    bs, s, d = x.shape
    sf = s // C
    return x[:, :sf * C].reshape(bs, sf, C, d).sum(2) / x.dtype.type(C)


def repeat_upsample_1d(x, s, C, out):
    sf = s // C
    out = out.copy()
    out[:, :sf * C] = np.repeat(x, C, axis=1)
    return out


def mean_pool_1d_backward(d_out, d_x, C):
    return d_x + _expand(d_out, d_x.shape[1], C) / d_x.dtype.type(C)


def _expand(g, s, C):
    bs, sf, d = g.shape
    out = np.zeros((bs, s, d), g.dtype)
    out[:, :sf * C] = np.repeat(g, C, axis=1)
    return out


def repeat_upsample_1d_backward(d_out, C):
    bs, s, d = d_out.shape
    sf = s // C
    return d_out[:, :sf * C].reshape(bs, sf, C, d).sum(2)


# core/kernels/m3_optimizer.cu:24-42, 66-80, 103-114, 204-215
def m3_ema_update(m1, m2, v, g, b1, b2, b3, update_m2):
    f = g.dtype.type
    m1n = f(b1) * m1 + (f(1) - f(b1)) * g
    vn = f(b2) * v + (f(1) - f(b2)) * g * g
    m2n = f(b3) * m2 + (f(1) - f(b3)) * g if update_m2 else m2.copy()
    return m1n, m2n, vn


def m3_apply_1d(w, m1, m2, v, lr, alpha, eps, bc2):
    f = w.dtype.type
    return w - f(lr) * (m1 + f(alpha) * m2) / (np.sqrt(v / f(bc2)) + f(eps))


def m3_apply_2d(w, o1, o2, lr, alpha):
    f = w.dtype.type
    return w - f(lr) * (o1 + f(alpha) * o2)


def m3_ns_poly(x, y, z, a, b, c):
    f = x.dtype.type
    return f(a) * x + f(b) * y + f(c) * z


# core/kernels/swiglu_forward.cu:144-158, 301-355; swiglu_backward.cu:174-197, 411-500
def swiglu_forward(x, gate_proj, up_proj, down_proj):
    gate, up = x @ gate_proj.T, x @ up_proj.T
    sig = 1.0 / (1.0 + np.exp(-gate))
    fused = gate * sig * up
    return fused @ down_proj.T, gate, up, fused, sig


def swiglu_backward(d_y, x, gate_proj, up_proj, down_proj, fused, gate, up, sig):
    d_fused = d_y @ down_proj
    d_down = d_y.T @ fused
    d_gate = d_fused * up * (sig * (1.0 + gate * (1.0 - sig)))
    d_up = d_fused * gate * sig
    return d_gate @ gate_proj + d_up @ up_proj, d_gate.T @ x, d_up.T @ x, d_down
