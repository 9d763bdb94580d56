"""Host mirror of the reference's TNT level on device buffers: gpu_tnt_forward
(core/src/gpu_forward.rs:1878-2293) and the TNT arm of gpu_memory_backward
(core/src/gpu_backward.rs:1201-1632).

The sequence is cut into shards of `tnt_global_chunk_size` tokens.  Inside a shard every local chunk of
`tnt_local_chunk_size` tokens runs the Delta or Titans rule as a chain of its own, all of them started from
the shard's global memory (chains = heads x local chunks, the last chunk padded with zero tokens and zero
gates, which leave a memory as it is).  The shard's outputs are mean-pooled per head into a key and a value
summary, and the global memory takes one outer-product step M <- 0.95 M + v_sum k_sum^T before the next shard.
The backward walks the shards in reverse: through the global step, the summary, into the shard's outputs,
through the chains, and from the chains' initial memories back into the global memory.

Same order of operations, cached tensors and argument checks as the reference, each step a call into
libnl_hecate_rocm.so (the rule kernels, the tnt_* helpers, the glue) or a torch matmul / copy in the place of
cuBLAS / cudaMemcpy.  One property of the reference is kept on purpose: the rule's backward returns the
gradient of the initial memory summed over all chains of the call, and the reference adds that sum to the
first head's global memory gradient (gpu_backward.rs:1408-1418: its per-chain loop finds every other slot
empty).  With one head this is the gradient; with several heads the other heads' share lands on head 0.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import dispatch as D
from .memory_level import (F32_MAX, GpuMemoryCache, LevelConfig, LevelGrads, _gate_heads, _heads, _new, _sum_heads,
                           _tokens, _zeros)

GLOBAL_RETENTION = 0.95   # the constant of tnt_global_update_f32_cuda's call sites (gpu_forward.rs:2262)


@dataclass
class ParallelConfig:
    """The two fields of crate::parallel::ParallelConfig this path reads."""
    tnt_global_chunk_size: int
    tnt_local_chunk_size: int


@dataclass
class TntCache:
    """GpuMemoryCache::TNT: inner caches of the retained shards (a rolling window: the oldest are dropped),
    summaries of every shard."""
    shard_inner_caches: List[GpuMemoryCache]
    k_summaries: List[torch.Tensor]      # [d] = heads x head_dim each
    v_summaries: List[torch.Tensor]
    global_chunk_size: int
    local_chunk_size: int
    total_shards: int
    first_retained_shard: int
    kind: str = "TNT"

    def dgd_delta_norm(self, s, d, batch_size, num_heads):
        """gpu_forward.rs:414-428: the largest value over the retained shards' inner caches (slot 0 of each)."""
        return max((c.dgd_delta_norm(self.local_chunk_size, d, 1, num_heads) for c in self.shard_inner_caches),
                   default=0.0)


def _pad_heads(t, nh, shard_len, padded_len):
    """[nh, shard_len, ...] -> [nh, padded_len, ...] with zeros behind each head's tokens."""
    if shard_len == padded_len:
        return t
    out = torch.zeros((nh, padded_len) + tuple(t.shape[2:]), dtype=t.dtype, device=t.device)
    out[:, :shard_len].copy_(t.view((nh, shard_len) + tuple(t.shape[2:])))
    return out


def gpu_tnt_forward(level_params, cfg: LevelConfig, embedded, context_m, s, d, batch_size, parallel_cfg: ParallelConfig,
                    max_retained: Optional[int] = None):
    """embedded [s, d]; context_m [nh, hd*hd]: the global memory per head, updated shard by shard.
    max_retained: MAGConfig::retained_shards(global chunk) — how many shards keep their inner caches for the
    backward (None: all).  Returns (y [s, d], TntCache)."""
    lp = level_params
    if batch_size != 1:
        raise ValueError("TNT forward requires batch_size=1 (the inner batch holds the local memories)")
    if cfg.memory_rule not in ("titans", "delta"):
        raise ValueError(f"TNT forward only supports titans and delta, got {cfg.memory_rule}")
    nh = cfg.num_heads
    hd = d // nh
    dd = hd * hd
    if context_m.numel() < nh * dd:
        raise ValueError(f"context_m layout mismatch: expected >= {nh * dd}, got {context_m.numel()}")
    cg, cl = parallel_cfg.tnt_global_chunk_size, parallel_cfg.tnt_local_chunk_size
    assert 1 <= cl <= cg
    num_shards = (s + cg - 1) // cg
    mx, clip = cfg.m_norm_max, cfg.error_clip
    titans = cfg.memory_rule == "titans"
    y_full = _zeros(s, d)
    keep = num_shards if max_retained is None else max(1, max_retained)
    caches, k_summaries, v_summaries, dropped = [], [], [], 0
    ctx = context_m.view(-1)
    for shard_idx in range(num_shards):
        t0 = shard_idx * cg
        t1 = min(t0 + cg, s)
        n = t1 - t0
        n_batch = (n + cl - 1) // cl
        kb, padded = n_batch * nh, n_batch * cl
        # 1: every local memory starts from its head's global memory
        m_broadcast = _new(nh, n_batch, dd)
        rc = D.call("broadcast_fill_f32_cuda", m_broadcast, ctx[:nh * dd], dd, n_batch, nh)
        assert rc == 0, f"broadcast_fill_f32_cuda failed (rc={rc})"
        # 2, 3: projections, normalisation and gates of the shard's tokens at model width
        emb = embedded[t0:t1]
        k_mem, v_mem, q_mem = emb @ lp.w_k.t(), emb @ lp.w_v.t(), emb @ lp.w_q.t()
        # norms padded to the padded length: the backward walks the padded rows (zero rows, zero gradients)
        k_norms, q_norms = _zeros(padded), _zeros(padded)
        D.call("l2_normalize_rows_f32_cuda", k_mem, k_norms, n, d, 1e-8)
        D.call("l2_normalize_rows_f32_cuda", q_mem, q_norms, n, d, 1e-8)
        alpha, theta = _new(n), _new(n)
        eta = None
        if titans:
            eta = _new(n)
            D.call("gate_compute_cuda", k_mem, v_mem, lp.w_eta, lp.b_eta, eta, n, d, 0)
        D.call("gate_compute_cuda", k_mem, v_mem, lp.w_alpha, lp.b_alpha, alpha, n, d, 0)
        D.call("gate_compute_cuda", k_mem, v_mem, lp.w_theta, lp.b_theta, theta, n, d, 1)
        if cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0:
            D.call("clamp_f32_cuda", alpha, n, cfg.alpha_floor, cfg.alpha_ceil)
        if cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX:
            D.call("clamp_f32_cuda", theta, n, cfg.theta_floor, cfg.theta_ceil)
        # per head, padded to whole local chunks: [nh, padded, hd] = [nh * n_batch, cl, hd]
        k_b, v_b, q_b = (_pad_heads(_heads(cfg, t, 1, n), nh, n, padded) for t in (k_mem, v_mem, q_mem))
        a_b, t_b = (_pad_heads(_gate_heads(cfg, g, 1, n), nh, n, padded) for g in (alpha, theta))
        e_b = _pad_heads(_gate_heads(cfg, eta, 1, n), nh, n, padded) if titans else None
        # 5: the rule on all local chains at once
        y_local = _new(nh, padded, hd)
        m_states = _new(kb, cl + 1, dd)
        s_states = None
        if titans:
            s_states = _new(kb, cl + 1, dd)
            D.titans_forward_dd(k_b, v_b, q_b, a_b, t_b, e_b, m_broadcast, _zeros(kb, dd), m_states, s_states, y_local,
                                cl, hd, kb, cl, dd, clip, mx)
        else:
            D.call("delta_forward_f32_cuda", k_b, v_b, q_b, a_b, t_b, m_broadcast, m_states, y_local, cl, hd, kb, cl,
                   dd, clip, mx)
        if cfg.proxy:   # only the final states are kept
            m_states = m_states[:, cl].contiguous()
            s_states = s_states[:, cl].contiguous() if titans else None
        inner = GpuMemoryCache("Titans" if titans else "Delta", k_mem=k_b, v_mem=v_b, q_mem=q_b, alpha=a_b, theta=t_b,
                               eta=e_b, m_states=m_states, s_states=s_states, k_norms=k_norms, q_norms=q_norms,
                               proxy=cfg.proxy)
        # 6: outputs back at model width
        y_full[t0:t1].copy_(_tokens(cfg, y_local, 1, padded)[:n])
        # 7: per-head mean of the shard's outputs as key and value summary
        k_sum, v_sum = _zeros(d), _zeros(d)
        for h in range(nh):
            h_y = y_local[h, :n].contiguous()
            D.call("tnt_shard_summary_mean_f32_cuda", h_y, k_sum[h * hd:], v_sum[h * hd:], n, hd)
        # 8: one outer-product step of each head's global memory, then its norm bound
        for h in range(nh):
            D.call("tnt_global_update_f32_cuda", ctx[h * dd:], k_sum[h * hd:], v_sum[h * hd:], hd, GLOBAL_RETENTION)
        D.call("m_norm_clamp_batch_f32_cuda", ctx, hd, nh, mx)
        caches.append(inner)
        k_summaries.append(k_sum)
        v_summaries.append(v_sum)
        while len(caches) > keep:
            caches.pop(0)
            dropped += 1
    return y_full, TntCache(caches, k_summaries, v_summaries, cg, cl, num_shards, dropped)


def gpu_tnt_backward(level_params, cfg: LevelConfig, cache: TntCache, d_y, embedded, level_grads: LevelGrads, s, d,
                     batch_size, per_head_memory_gradient=False):
    """d_y, embedded [s, d].  Adds the gate gradients of every retained shard into level_grads (zero them first),
    writes the projection gradients, returns d_embedded [s, d].  Shards whose inner caches were dropped pass
    the global memory's gradient on and contribute nothing else.
    per_head_memory_gradient=False is the reference's behaviour (the local chains' initial-memory gradients, summed
    over all chains by the rule's backward, land on head 0: see the module text); True sends every chain's gradient
    to its own head's global memory (the rule's segment backward over the whole chain returns it per chain), which
    is the gradient of the forward for any number of heads."""
    lp, c, g = level_params, cache, level_grads
    if batch_size != 1:
        raise ValueError("TNT backward currently supports batch_size=1 only")
    nh = cfg.num_heads
    hd = d // nh
    dd = hd * hd
    cg, cl, n_total, first_ret = c.global_chunk_size, c.local_chunk_size, c.total_shards, c.first_retained_shard
    assert n_total > 0 and first_ret < n_total
    assert len(c.shard_inner_caches) == n_total - first_ret
    assert len(c.k_summaries) == n_total and len(c.v_summaries) == n_total
    clip = cfg.error_clip
    d_k_total, d_v_total, d_q_total = _zeros(s, d), _zeros(s, d), _zeros(s, d)
    d_m_carry = _zeros(nh * dd)
    for shard_idx in reversed(range(n_total)):
        t0 = shard_idx * cg
        t1 = min(t0 + cg, s)
        n = t1 - t0
        n_batch = (n + cl - 1) // cl
        kb, padded = n_batch * nh, n_batch * cl
        # 1: through the global memory's step, head by head
        d_m_old, d_k_sum, d_v_sum = _zeros(nh * dd), _zeros(d), _zeros(d)
        for h in range(nh):
            D.call("tnt_global_update_backward_f32_cuda", d_m_carry[h * dd:], c.k_summaries[shard_idx][h * hd:],
                   c.v_summaries[shard_idx][h * hd:], d_m_old[h * dd:], d_k_sum[h * hd:], d_v_sum[h * hd:], hd,
                   GLOBAL_RETENTION)
        if shard_idx < first_ret:
            d_m_carry = d_m_old
            continue
        inner = c.shard_inner_caches[shard_idx - first_ret]
        titans = inner.kind == "Titans"
        # 2: through the summaries into the shard's outputs
        d_local_y = _zeros(nh, n, hd)
        for h in range(nh):
            D.call("tnt_shard_summary_mean_backward_f32_cuda", d_k_sum[h * hd:], d_v_sum[h * hd:],
                   d_local_y.view(-1)[h * n * hd:], n, hd)
        d_local_y_dm = _tokens(cfg, d_local_y, 1, n)
        # 3, 4: plus the upstream gradient, per head, padded
        d_y_combined = _new(n, d)
        D.call("tnt_combine_gradients_f32_cuda", d_y[t0:t1], d_local_y_dm, d_y_combined, n * d)
        d_y_b = _pad_heads(_heads(cfg, d_y_combined, 1, n), nh, n, padded)
        # 5: the rule's backward on all local chains
        tokens = nh * padded
        dk, dv, dq = _zeros(tokens, hd), _zeros(tokens, hd), _zeros(tokens, hd)
        da, dth, de = _zeros(tokens), _zeros(tokens), _zeros(tokens)
        d_m_initial = _zeros(kb, dd)
        m_bw, s_bw = inner.m_states, inner.s_states
        if inner.proxy:   # the final state stands in for every state of the chain
            m_bw = _new(kb, cl + 1, dd)
            rc = D.call("broadcast_fill_f32_cuda", m_bw, inner.m_states, dd, cl + 1, kb)
            assert rc == 0, f"broadcast_fill M failed (rc={rc})"
            if titans:
                s_bw = _new(kb, cl + 1, dd)
                rc = D.call("broadcast_fill_f32_cuda", s_bw, inner.s_states, dd, cl + 1, kb)
                assert rc == 0, f"broadcast_fill S failed (rc={rc})"
        if per_head_memory_gradient:   # the segment form over the whole chain: d_m_out is per chain
            seed = _zeros(kb, dd)
            if titans:
                D.titans_backward_dd_segment(inner.k_mem, inner.v_mem, inner.q_mem, inner.alpha, inner.theta, inner.eta,
                                             m_bw, s_bw, d_y_b, seed, seed, dk, dv, dq, da, dth, de, d_m_initial,
                                             _zeros(kb, dd), 0, cl, hd, kb, cl, clip)
            else:
                D.delta_backward_dd_segment(inner.k_mem, inner.v_mem, inner.q_mem, inner.alpha, inner.theta, m_bw, d_y_b,
                                            seed, dk, dv, dq, da, dth, d_m_initial, 0, cl, hd, kb, cl, clip)
        elif titans:
            D.titans_backward_dd(inner.k_mem, inner.v_mem, inner.q_mem, inner.alpha, inner.theta, inner.eta, m_bw, s_bw,
                                 d_y_b, dk, dv, dq, da, dth, de, d_m_initial, _zeros(kb, dd), cl, hd, kb, clip)
        else:
            D.call("delta_backward_f32_cuda", inner.k_mem, inner.v_mem, inner.q_mem, inner.alpha, inner.theta, m_bw,
                   d_y_b, dk, dv, dq, da, dth, d_m_initial, cl, hd, kb, clip)
        if not inner.proxy:   # chain b belongs to head b / n_batch (see the module text for what arrives where)
            for b in range(kb):
                D.call("saxpy_cuda", 1.0, d_m_initial.view(-1)[b * dd:], d_m_old[(b // n_batch) * dd:], dd)
        if cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0:
            D.call("theta_clamp_mask_cuda", inner.alpha, da, tokens, cfg.alpha_floor, cfg.alpha_ceil)
        if cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX:
            D.call("theta_clamp_mask_cuda", inner.theta, dth, tokens, cfg.theta_floor, cfg.theta_ceil)
        # back to model width over the padded rows
        dk_dm, dv_dm, dq_dm = (_tokens(cfg, t, 1, padded) for t in (dk, dv, dq))
        da_dm, dth_dm = _sum_heads(cfg, da, 1, padded), _sum_heads(cfg, dth, 1, padded)
        de_dm = _sum_heads(cfg, de, 1, padded) if titans else None
        k_dm, v_dm, q_dm = (_tokens(cfg, t, 1, padded) for t in (inner.k_mem, inner.v_mem, inner.q_mem))
        # head 0's copy of the gates (all heads hold the same values)
        a_dm, t_dm = inner.alpha.view(-1)[:padded], inner.theta.view(-1)[:padded]
        e_dm = inner.eta.view(-1)[:padded] if titans else None
        d_k_raw, d_q_raw = _new(padded, d), _new(padded, d)
        D.call("l2_normalize_backward_f32_cuda", dk_dm, k_dm, inner.k_norms, d_k_raw, padded, d, 1e-8)
        D.call("l2_normalize_backward_f32_cuda", dq_dm, q_dm, inner.q_norms, d_q_raw, padded, d, 1e-8)
        # 6: the shard's rows of the full-sequence totals
        for src, dst in ((d_k_raw, d_k_total), (dv_dm, d_v_total), (d_q_raw, d_q_total)):
            D.call("saxpy_cuda", 1.0, src, dst.view(-1)[t0 * d:], n * d)
        # 7: gate weights and biases, added over the shards
        tmp = LevelGrads.zeros(d)
        z = da_dm
        D.call("gate_backward_cuda", da_dm, a_dm, dth_dm, t_dm, de_dm if titans else z, e_dm if titans else z, k_dm,
               v_dm, tmp.d_w_alpha, tmp.d_b_alpha, tmp.d_w_theta, tmp.d_b_theta, tmp.d_w_eta, tmp.d_b_eta, padded, d, 1,
               int(titans))
        names = ["alpha", "theta"] + (["eta"] if titans else [])
        for nm in names:
            D.call("saxpy_cuda", 1.0, getattr(tmp, "d_w_" + nm), getattr(g, "d_w_" + nm), 2 * d)
            D.call("saxpy_cuda", 1.0, getattr(tmp, "d_b_" + nm), getattr(g, "d_b_" + nm), 1)
        d_m_carry = d_m_old
    torch.mm(d_k_total.t(), embedded, out=g.d_w_k_mem)
    torch.mm(d_v_total.t(), embedded, out=g.d_w_v_mem)
    torch.mm(d_q_total.t(), embedded, out=g.d_w_q_mem)
    d_embedded = d_k_total @ lp.w_k
    d_embedded.addmm_(d_v_total, lp.w_v)
    d_embedded.addmm_(d_q_total, lp.w_q)
    return d_embedded
