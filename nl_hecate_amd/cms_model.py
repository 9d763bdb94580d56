"""Host mirror of the reference's whole training step on device buffers: gpu_cms_forward
(core/src/gpu_forward.rs:760-1117), gpu_cms_backward (core/src/gpu_backward.rs:143-455),
gpu_weight_update (:2203-2236) and gpu_sync_embed_weights (:2239-2251).

Forward: embedding gather, (with `residual`) LayerNorm, q/k/v projections, bf16 sliding-window attention,
(residual: skip connection + second LayerNorm), every CMS level — an active level through the level step of
memory_level.py (or the TNT level of tnt.py when a parallel configuration is set), a frozen one as a read of its
memory — sum of the levels (times 1/sqrt(k) for k > 2), sigmoid gate on the attention output (residual: sum
instead), output projection, unembedding, cross-entropy over the valid targets.  Backward: the same chain in
reverse down to the embedding table's scatter-add.  As in the reference, a frozen level passes no gradient in
this path (its read-only backward is called without the memory, gpu_backward.rs:312-322).

This is the plain caller, one library call or torch matmul per reference call, for every rule the level step
covers; the tuned layer step (split-bf16 GEMMs, stacked levels, fused glue, captured graphs, AdamW) is
mag_layer.py.  The reference's CUDA-graph capture / replay inside gpu_cms_forward is not mirrored here.
"""
import ctypes
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import dispatch as D
from .cms import ContextState, Pulse
from .ffi import lib
from .memory_level import LevelConfig, LevelGrads, gpu_memory_backward, gpu_memory_forward
from .serving import GpuMAGParams, frozen_level_output
from .tnt import ParallelConfig, gpu_tnt_backward, gpu_tnt_forward

LN_EPS = 1e-5


def _new(*shape, dtype=torch.float32):
    return torch.empty(*shape, dtype=dtype, device="cuda")


def _zeros(*shape, dtype=torch.float32):
    return torch.zeros(*shape, dtype=dtype, device="cuda")


@dataclass
class ModelConfig:
    """What the training step reads from MAGConfig."""
    d_model: int
    vocab_size: int
    num_heads: int
    head_dim: int
    window_size: int
    seq_len: int
    levels: List[LevelConfig]
    n_persistent: int = 0
    residual: bool = False
    parallel: Optional[ParallelConfig] = None     # set: TNT levels (batch 1, titans / delta)
    tnt_retained_shards: Optional[int] = None

    @property
    def k(self):
        return len(self.levels)


@dataclass
class LayerNormParams:
    """ln_attn_* / ln_mem_* of the residual variant."""
    ln_attn_gamma: torch.Tensor
    ln_attn_beta: torch.Tensor
    ln_mem_gamma: torch.Tensor
    ln_mem_beta: torch.Tensor


@dataclass
class GpuMAGGrads:
    d_w_embed: torch.Tensor
    d_w_q: torch.Tensor
    d_w_k: torch.Tensor
    d_w_v: torch.Tensor
    d_w_o: torch.Tensor
    d_w_unembed: torch.Tensor
    d_ln_attn_gamma: torch.Tensor
    d_ln_attn_beta: torch.Tensor
    d_ln_mem_gamma: torch.Tensor
    d_ln_mem_beta: torch.Tensor
    levels: List[LevelGrads]
    level_output_gnorms: List[float]


def _uses_tnt(cfg, level, bs):
    return cfg.parallel is not None and bs == 1 and cfg.levels[level].memory_rule in ("titans", "delta")


def gpu_cms_forward(params: GpuMAGParams, cfg: ModelConfig, input_ids, target_ids, pulse: Pulse, context: ContextState,
                    ln: Optional[LayerNormParams] = None):
    """input_ids, target_ids: batch_size * seq_len token ids (targets outside [0, vocab) are skipped by the loss).
    Returns (mean loss over the valid targets, cache for gpu_cms_backward)."""
    s, d, v, nh, hd, ws = cfg.seq_len, cfg.d_model, cfg.vocab_size, cfg.num_heads, cfg.head_dim, cfg.window_size
    assert s > 0 and d == nh * hd
    assert len(input_ids) >= s, "input_ids too short"
    bs = len(input_ids) // s
    assert len(input_ids) == bs * s, "input_ids must be a multiple of seq_len"
    assert len(target_ids) == bs * s, "target_ids must match input_ids length"
    if cfg.residual and ln is None:
        raise ValueError("residual=True needs the LayerNorm parameters")
    n = bs * s
    ids = torch.tensor([int(t) for t in input_ids], dtype=torch.int32).cuda()
    tgt_host = [int(t) for t in target_ids]
    tgt = torch.tensor(tgt_host, dtype=torch.int32).cuda()
    embedded = _new(n, d)
    D.call("embedding_gather_cuda", params.w_embed, ids, embedded, n, d)
    c = dict(input_ids=ids, target_ids=tgt, target_host=tgt_host, embedded=embedded, pulse=pulse, bs=bs)
    qkv_source = embedded
    if cfg.residual:
        c["ln_attn_out"], c["ln_attn_mean"], c["ln_attn_rstd"] = _new(n, d), _new(n), _new(n)
        D.call("layer_norm_forward_cuda", embedded, ln.ln_attn_gamma, ln.ln_attn_beta, c["ln_attn_out"],
               c["ln_attn_mean"], c["ln_attn_rstd"], n, d, LN_EPS)
        qkv_source = c["ln_attn_out"]
    q_f32, k_f32, v_f32 = (qkv_source @ w.t() for w in (params.w_q, params.w_k, params.w_v))
    bf = lambda: _new(n, d, dtype=torch.bfloat16)
    c["q_bf16"], c["k_bf16"], c["v_bf16"], attn_out_bf16 = bf(), bf(), bf(), bf()
    for src, dst in ((q_f32, c["q_bf16"]), (k_f32, c["k_bf16"]), (v_f32, c["v_bf16"])):
        D.call("f32_to_bf16_cuda", src, dst, n * d)
    c["attn_weights_bf16"] = _new(bs, nh, s, cfg.n_persistent + ws, dtype=torch.bfloat16)
    D.call("swa_forward_f32_cuda", c["q_bf16"], c["k_bf16"], c["v_bf16"], attn_out_bf16, c["attn_weights_bf16"], s, nh,
           hd, ws, bs, cfg.n_persistent)
    c["attn_out"] = _new(n, d)
    D.call("bf16_to_f32_cuda", attn_out_bf16, c["attn_out"], n * d)
    mem_input = embedded
    if cfg.residual:
        c["residual_after_attn"] = embedded + c["attn_out"]
        c["ln_mem_out"], c["ln_mem_mean"], c["ln_mem_rstd"] = _new(n, d), _new(n), _new(n)
        D.call("layer_norm_forward_cuda", c["residual_after_attn"], ln.ln_mem_gamma, ln.ln_mem_beta, c["ln_mem_out"],
               c["ln_mem_mean"], c["ln_mem_rstd"], n, d, LN_EPS)
        mem_input = c["ln_mem_out"]
    ys, caches = [], []
    for level in range(cfg.k):
        lcfg = cfg.levels[level]
        if pulse.active_levels[level] or lcfg.memory_rule == "swiglu":
            if _uses_tnt(cfg, level, bs):
                y, mc = gpu_tnt_forward(params.levels[level], lcfg, mem_input, context.memory[level], s, d, bs,
                                        cfg.parallel, cfg.tnt_retained_shards)
            else:
                y, mc = gpu_memory_forward(params.levels[level], lcfg, mem_input, context.memory[level], s, d, bs)
        else:
            # the matrix read; zeros for MONETA / YAAD, an error for the two-layer Titans memory (gpu_forward.rs:1008-1024)
            y, mc = frozen_level_output(lcfg, params.levels[level], mem_input, context.memory[level], n, nh, hd, level), None
        ys.append(y)
        caches.append(mc)
    c["memory_caches"], c["y_per_level"] = caches, ys
    c["y_combined"], c["gate"], c["gated_out"] = _new(n, d), _new(n, d), _new(n, d)
    if cfg.residual:
        comb = torch.stack(ys).sum(0)
        if cfg.k > 2:
            comb = comb * (1.0 / cfg.k ** 0.5)
        c["y_combined"] = comb
        c["residual_final"] = c["residual_after_attn"] + comb
        c["projected"] = c["residual_final"] @ params.w_o.t()
        c["gated_out"] = c["attn_out"].clone()
    else:
        ptrs = (ctypes.c_void_p * len(ys))(*[y.data_ptr() for y in ys])
        lib.cms_combine_gate_rocm(ptrs, len(ys), c["attn_out"].data_ptr(), c["y_combined"].data_ptr(),
                                  c["gate"].data_ptr(), c["gated_out"].data_ptr(), n * d)
        c["projected"] = c["gated_out"] @ params.w_o.t()
    c["logits"] = c["projected"] @ params.w_unembed
    loss_gpu = _zeros(1)
    D.call("cross_entropy_forward_cuda", c["logits"], tgt, loss_gpu, n, v)
    valid = sum(1 for t in tgt_host if 0 <= t < v)
    loss = float(loss_gpu.item()) / valid if valid > 0 else 0.0
    return loss, c


def gpu_cms_backward(params: GpuMAGParams, cfg: ModelConfig, cache, collect_output_gnorms=False,
                     ln: Optional[LayerNormParams] = None) -> GpuMAGGrads:
    c = cache
    s, d, v, nh, hd, ws, bs = cfg.seq_len, cfg.d_model, cfg.vocab_size, cfg.num_heads, cfg.head_dim, cfg.window_size, c["bs"]
    n = bs * s
    inter = lambda lv: cfg.levels[lv].intermediate_size if cfg.levels[lv].memory_rule == "swiglu" else 0
    g = GpuMAGGrads(_zeros(v, d), _zeros(d, d), _zeros(d, d), _zeros(d, d), _zeros(d, d), _zeros(d, v), _zeros(d),
                    _zeros(d), _zeros(d), _zeros(d), [LevelGrads.zeros(d, intermediate=inter(lv)) for lv in range(cfg.k)],
                    [0.0] * cfg.k)
    valid = sum(1 for t in c["target_host"] if 0 <= t < v)
    d_logits = _zeros(n, v)
    D.call("cross_entropy_backward_cuda", c["logits"], c["target_ids"], d_logits, n, v, 1.0 / (valid if valid > 0 else 1))
    d_projected = d_logits @ params.w_unembed.t()
    torch.mm(c["projected"].t(), d_logits, out=g.d_w_unembed)
    d_gated_out = d_projected @ params.w_o
    torch.mm(d_projected.t(), c["residual_final"] if cfg.residual else c["gated_out"], out=g.d_w_o)
    if cfg.residual:
        d_y_combined, d_attn_out = d_gated_out.clone(), d_gated_out.clone()
    else:
        d_attn_out, d_gate, d_y_combined = _new(n, d), _new(n, d), _new(n, d)
        D.call("gating_backward_cuda", d_gated_out, c["attn_out"], c["gate"], d_attn_out, d_gate, n * d)
        D.call("sigmoid_backward_cuda", d_gate, c["gate"], d_y_combined, n * d)
    if cfg.k > 2:
        D.call("saxpy_cuda", 1.0 / cfg.k ** 0.5 - 1.0, d_y_combined, d_y_combined, n * d)   # y += (c - 1) y
    if collect_output_gnorms:
        norm = float(torch.linalg.vector_norm(d_y_combined.double()).item())
        for level in range(cfg.k):
            if c["pulse"].active_levels[level]:
                g.level_output_gnorms[level] = norm
    mem_input = c["ln_mem_out"] if cfg.residual else c["embedded"]
    d_mem_input = _zeros(n, d)
    for level in range(cfg.k):
        mc = c["memory_caches"][level]
        if mc is None:   # frozen: no gradient in this path (the read-only backward is called without the memory)
            continue
        if mc.kind == "TNT":
            d_emb = gpu_tnt_backward(params.levels[level], cfg.levels[level], mc, d_y_combined, mem_input,
                                     g.levels[level], s, d, bs)
        else:
            d_emb = gpu_memory_backward(params.levels[level], cfg.levels[level], mc, d_y_combined, mem_input,
                                        g.levels[level], s, d, bs)
        D.call("saxpy_cuda", 1.0, d_emb, d_mem_input, n * d)
    if cfg.residual:
        d_res = _new(n, d)
        D.call("layer_norm_backward_cuda", d_mem_input, c["residual_after_attn"], ln.ln_mem_gamma, c["ln_mem_mean"],
               c["ln_mem_rstd"], d_res, g.d_ln_mem_gamma, g.d_ln_mem_beta, n, d)
        D.call("saxpy_cuda", 1.0, d_res, d_attn_out, n * d)
    d_q, d_k, d_v = _new(n, d), _zeros(n, d), _zeros(n, d)
    D.call("swa_backward_f32_cuda", c["q_bf16"], c["k_bf16"], c["v_bf16"], c["attn_weights_bf16"], d_attn_out, d_q, d_k,
           d_v, s, nh, hd, ws, bs, cfg.n_persistent)
    qkv_source = c["ln_attn_out"] if cfg.residual else c["embedded"]
    d_qkv_source = d_q @ params.w_q
    d_qkv_source.addmm_(d_k, params.w_k)
    d_qkv_source.addmm_(d_v, params.w_v)
    torch.mm(d_q.t(), qkv_source, out=g.d_w_q)
    torch.mm(d_k.t(), qkv_source, out=g.d_w_k)
    torch.mm(d_v.t(), qkv_source, out=g.d_w_v)
    if cfg.residual:
        d_embedded = _new(n, d)
        D.call("layer_norm_backward_cuda", d_qkv_source, c["embedded"], ln.ln_attn_gamma, c["ln_attn_mean"],
               c["ln_attn_rstd"], d_embedded, g.d_ln_attn_gamma, g.d_ln_attn_beta, n, d)
        D.call("saxpy_cuda", 1.0, d_attn_out, d_embedded, n * d)
    else:
        d_embedded = d_qkv_source
        D.call("saxpy_cuda", 1.0, d_mem_input, d_embedded, n * d)
    D.call("embedding_scatter_add_cuda", d_embedded, c["input_ids"], g.d_w_embed, n, d)
    return g


def gpu_weight_update(params: GpuMAGParams, grads: GpuMAGGrads, lr):
    """Plain SGD on every tensor: p <- p - lr * g (gpu_backward.rs:2203-2236)."""
    pairs = [(grads.d_w_embed, params.w_embed), (grads.d_w_q, params.w_q), (grads.d_w_k, params.w_k),
             (grads.d_w_v, params.w_v), (grads.d_w_o, params.w_o), (grads.d_w_unembed, params.w_unembed)]
    for lg, lp in zip(grads.levels, params.levels):
        if hasattr(lp, "gate_proj"):
            pairs += [(lg.d_gate_proj, lp.gate_proj), (lg.d_up_proj, lp.up_proj), (lg.d_down_proj, lp.down_proj)]
            continue
        pairs += [(lg.d_w_k_mem, lp.w_k), (lg.d_w_v_mem, lp.w_v), (lg.d_w_q_mem, lp.w_q), (lg.d_w_alpha, lp.w_alpha),
                  (lg.d_b_alpha, lp.b_alpha), (lg.d_w_theta, lp.w_theta), (lg.d_b_theta, lp.b_theta),
                  (lg.d_w_eta, lp.w_eta), (lg.d_b_eta, lp.b_eta)]
    for gr, p in pairs:
        D.call("saxpy_cuda", -float(lr), gr, p, p.numel())


def gpu_sync_embed_weights(params: GpuMAGParams, d, vocab):
    """Tied weights: w_embed [vocab, d] <- transpose of w_unembed [d, vocab] (gpu_backward.rs:2239-2251)."""
    D.call("transpose_copy_cuda", params.w_unembed, params.w_embed, d, vocab)
