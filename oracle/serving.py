"""TEST INFRASTRUCTURE ONLY — the cached generation path on the CPU: what gpu_prefill_forward
(core/src/gpu_forward.rs:3160-3312) and gpu_single_token_forward (:3377-3492) compute, composed from the
oracle's attention (pyoracle.swa_forward / swa_single_token), the level step of oracle/memory_level.py and
numpy matmuls.  float32 throughout, bf16 where the reference stores bf16 (q, k, v of the attention branch and
its output).  tests/test_oracle_serving.py pins the step-by-step form against the whole-sequence form.

p: dict with w_embed [v, d], w_q, w_k, w_v, w_o [d, d], w_unembed [d, v], levels: list of level dicts
(oracle/memory_level.py).  cfg: object with d_model, num_heads, head_dim, window_size, n_persistent and
levels (a list of level configs).  memories: list of [nh, hd, hd] arrays, one per level (batch 1)."""
import numpy as np

from . import memory_level as ML
from . import pyoracle as orc

f32 = np.float32


def _read_only(lp, emb, m, nh, hd):
    """gpu_memory_read_only (:2906-2950): y = M_h q_h with the projection q as it comes (not normalised)."""
    q = (emb @ lp["w_q"].T).astype(f32)
    s = q.shape[0]
    y = np.einsum("hij,shj->shi", m.astype(f32), q.reshape(s, nh, hd))
    return y.reshape(s, nh * hd).astype(f32)


def _levels(p, cfg, emb, active, memories):
    ys, new = [], []
    for lv, lcfg in enumerate(cfg.levels):
        if active[lv]:
            y, _, carried = ML.level_forward(p["levels"][lv], lcfg, emb[None], memories[lv])
            ys.append(y[0].astype(f32))
            new.append(carried.astype(f32))
        else:
            # frozen (gpu_forward.rs:3255-3265): the matrix read; zeros for MONETA / YAAD (frozen_mlp_fallback, :45-57);
            # refused for the two-layer Titans memory (panic_if_frozen_titans_mlp, :32-39)
            if getattr(lcfg, "memory_layers", 1) == 2 and lcfg.memory_rule == "titans":
                raise RuntimeError(f"Frozen TitansLMM MLP level unsupported (level {lv})")
            if lcfg.memory_rule in ("moneta", "yaad"):
                ys.append(np.zeros((emb.shape[0], cfg.num_heads * cfg.head_dim), f32))
            else:
                ys.append(_read_only(p["levels"][lv], emb, memories[lv], cfg.num_heads, cfg.head_dim))
            new.append(memories[lv])
    return ys, new


def _head(p, cfg, ys, attn):
    k = len(ys)
    comb = np.sum(ys, axis=0, dtype=f32)
    if k > 2:
        comb = comb * f32(1.0 / np.sqrt(k))
    gated = attn * ML.sigmoid(comb).astype(f32)
    return (gated @ p["w_o"].T) @ p["w_unembed"]


def forward_all(p, cfg, ids, active, memories):
    """The whole sequence at once -> (logits [s, v], memories after it, k bf16 bits [s, d], v bf16 bits)."""
    emb = p["w_embed"][np.asarray(ids)].astype(f32)
    q, k, v = (orc.f32_to_bf16((emb @ p[n].T).astype(f32)) for n in ("w_q", "w_k", "w_v"))
    out, _ = orc.swa_forward(q[None], k[None], v[None], cfg.window_size, cfg.num_heads, cfg.n_persistent)
    attn = orc.bf16_to_f32(out[0])
    ys, new = _levels(p, cfg, emb, active, memories)
    return _head(p, cfg, ys, attn), new, k, v


def single_token(p, cfg, token_id, active, memories, k_cache, v_cache):
    """One decode step on caches [n, d] of bf16 bits -> (logits [v], memories, caches with the token appended)."""
    emb = p["w_embed"][[token_id]].astype(f32)
    q, k, v = (orc.f32_to_bf16((emb @ p[n].T).astype(f32)) for n in ("w_q", "w_k", "w_v"))
    k_cache, v_cache = np.concatenate([k_cache, k]), np.concatenate([v_cache, v])
    out = orc.swa_single_token(q[0], k_cache, v_cache, cfg.window_size, cfg.num_heads, cfg.n_persistent)
    attn = orc.bf16_to_f32(out)[None]
    ys, new = _levels(p, cfg, emb, active, memories)
    return _head(p, cfg, ys, attn)[0], new, k_cache, v_cache
