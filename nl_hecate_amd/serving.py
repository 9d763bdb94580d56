"""Host mirror of the reference's cached generation path on device buffers:
GpuKVCache (core/src/gpu_forward.rs:2979-3147), gpu_prefill_forward (:3160-3312), DecodeWorkspace
(:3321-3362) and gpu_single_token_forward (:3377-3492).

Prefill runs the full forward over the prompt, fills the bf16 K/V cache and returns the logits of the
last position; a decode step embeds one token, appends its K and V, attends over the cache
(swa_single_token_cuda), runs every memory level with seq_len = 1 on the carried context memory
(active levels: the level step of memory_level.py; frozen levels: a read of the memory), combines the
levels, gates the attention output, projects and unembeds.  Every step is a call into
libnl_hecate_rocm.so or a torch matmul in the place of the reference's cuBLAS calls; the only transfers are
the token ids in and the logits out, as in the reference.
"""
import ctypes
from dataclasses import dataclass, field
from typing import List

import torch

from . import dispatch as D
from .cms import ContextState, Pulse
from .ffi import lib
from .mag_layer import MemoryLevelParams
from .memory_level import LevelConfig, gpu_memory_forward


def _new(*shape, dtype=torch.float32):
    return torch.empty(*shape, dtype=dtype, device="cuda")


def _zeros(*shape, dtype=torch.float32):
    return torch.zeros(*shape, dtype=dtype, device="cuda")


@dataclass
class GpuMAGParams:
    """The tensors the generation path reads (GpuMAGParams: swa block + levels)."""
    w_embed: torch.Tensor      # [vocab, d]
    w_q: torch.Tensor          # [d, d]
    w_k: torch.Tensor
    w_v: torch.Tensor
    w_o: torch.Tensor
    w_unembed: torch.Tensor    # [d, vocab]
    levels: List[MemoryLevelParams] = field(default_factory=list)


@dataclass
class ServeConfig:
    """What the two functions read from MAGConfig."""
    d_model: int
    vocab_size: int
    num_heads: int
    head_dim: int
    window_size: int
    seq_len: int                    # prompt length of a prefill
    levels: List[LevelConfig]       # one per CMS level (cfg.k = len(levels))
    n_persistent: int = 0
    decode_tokens: int = 2048       # prefill sizes the cache for the prompt plus this many decode tokens
    residual: bool = False          # the reference's cached-generation path refuses residual = true (:3175, :3392)

    @property
    def k(self):
        return len(self.levels)


class GpuKVCache:
    """bf16 K and V of every position so far, [max_len, d] each, with a conversion scratch sized once."""

    def __init__(self, max_len, d, scratch_tokens):
        self.k_cache_bf16 = _zeros(max_len, d, dtype=torch.bfloat16)
        self.v_cache_bf16 = _zeros(max_len, d, dtype=torch.bfloat16)
        self.len, self.max_len, self.d = 0, max_len, d
        self._scratch_k = _zeros(scratch_tokens * d, dtype=torch.bfloat16)
        self._scratch_v = _zeros(scratch_tokens * d, dtype=torch.bfloat16)

    def append_f32(self, k_f32, v_f32, n_tokens):
        """:3017-3053: convert into the scratch, copy behind the filled positions."""
        if self.len + n_tokens > self.max_len:
            raise OverflowError(f"KV cache overflow: {self.len} + {n_tokens} > {self.max_len}")
        total = n_tokens * self.d
        if total > self._scratch_k.numel():
            raise ValueError(f"append_f32: n_tokens*d={total} exceeds scratch buffer size {self._scratch_k.numel()}")
        D.call("f32_to_bf16_cuda", k_f32, self._scratch_k, total)
        D.call("f32_to_bf16_cuda", v_f32, self._scratch_v, total)
        self.k_cache_bf16.view(-1)[self.len * self.d:self.len * self.d + total].copy_(self._scratch_k[:total])
        self.v_cache_bf16.view(-1)[self.len * self.d:self.len * self.d + total].copy_(self._scratch_v[:total])
        self.len += n_tokens

    def _project_persistent(self, persistent_tokens, w_k, w_v, n_persistent, d):
        if d != self.d:
            raise ValueError(f"persistent tokens: caller d={d} != cache d={self.d}")
        npd = n_persistent * d
        if persistent_tokens.numel() < npd:
            raise ValueError(f"persistent_tokens has {persistent_tokens.numel()} < n_persistent*d={npd} elements")
        p = persistent_tokens.reshape(-1)[:npd].view(n_persistent, d)
        pk, pv = (p @ w_k.t()).contiguous(), (p @ w_v.t()).contiguous()
        D.call("f32_to_bf16_cuda", pk, self.k_cache_bf16, npd)
        D.call("f32_to_bf16_cuda", pv, self.v_cache_bf16, npd)

    def prepopulate_persistent(self, persistent_tokens, w_k, w_v, n_persistent, d):
        """:3055-3099: positions [0, n_persistent) = projections of the persistent tokens; empty cache only."""
        if n_persistent == 0:
            return
        if n_persistent > self.max_len:
            raise OverflowError(f"KV cache too small for {n_persistent} persistent tokens")
        if self.len != 0:
            raise RuntimeError("prepopulate_persistent must be called on an empty cache")
        self._project_persistent(persistent_tokens, w_k, w_v, n_persistent, d)
        self.len = n_persistent

    def refresh_persistent(self, persistent_tokens, w_k, w_v, n_persistent, d):
        """:3101-3141: the same projection after an optimizer step; the length does not change."""
        if n_persistent == 0:
            return
        if self.len < n_persistent:
            raise RuntimeError(f"cache len {self.len} < n_persistent {n_persistent}")
        self._project_persistent(persistent_tokens, w_k, w_v, n_persistent, d)

    def reset(self):
        self.len = 0


class DecodeWorkspace:
    """Buffers of one decode step, allocated once (:3321-3362)."""

    def __init__(self, d, v):
        self.d_input = _zeros(1, dtype=torch.int32)
        self.embedded = _zeros(1, d)
        self.q_bf16 = _zeros(1, d, dtype=torch.bfloat16)
        self.attn_out_bf16 = _zeros(1, d, dtype=torch.bfloat16)
        self.attn_out = _zeros(1, d)
        self.y_combined, self.gate, self.gated_out = _zeros(1, d), _zeros(1, d), _zeros(1, d)
        self.logits_gpu = _zeros(1, v)


def _memory_read_only(lp, embedded, memory, n, nh, hd):
    """gpu_memory_read_only (:2906-2950): y = M_h q per head with the raw projection q and the memories of the
    first batch slot."""
    q = (embedded @ lp.w_q.t()).contiguous()
    y = _new(n, nh * hd)
    D.call("memory_read_only_f32_rocm", q, memory[:nh].contiguous(), y, n, nh, hd)
    return y


def frozen_level_output(lcfg, lp, embedded, memory, n, nh, hd, level):
    """What a frozen level contributes (gpu_forward.rs:1008-1024, 3255-3265, 3449-3459): the read y = M_h q for a
    matrix memory; zeros for MONETA / YAAD, whose context memory is the flat [W1 | W2] block that the matrix read
    cannot interpret (frozen_mlp_fallback, :45-57); an error for the two-layer Titans memory
    (panic_if_frozen_titans_mlp, :32-39)."""
    if lcfg.is_mlp_mem:
        raise RuntimeError(f"Frozen TitansLMM MLP level unsupported (level {level}): read-only MLP kernel not implemented")
    if lcfg.memory_rule in ("moneta", "yaad"):
        return _zeros(n, nh * hd)
    return _memory_read_only(lp, embedded, memory, n, nh, hd)


def _levels(params, cfg, embedded, pulse, context, s):
    ys = []
    for level in range(cfg.k):
        if pulse.active_levels[level]:
            y, _cache = gpu_memory_forward(params.levels[level], cfg.levels[level], embedded, context.memory[level], s,
                                           cfg.d_model, 1)
        else:
            y = frozen_level_output(cfg.levels[level], params.levels[level], embedded, context.memory[level], s,
                                    cfg.num_heads, cfg.head_dim, level)
        ys.append(y)
    return ys


def _combine_gate(ys, attn_out, y_combined, gate, gated, n):
    """Sum of the levels (times 1/sqrt(k) for k > 2), sigmoid gate on the attention output (:3275-3293)."""
    ptrs = (ctypes.c_void_p * len(ys))(*[y.data_ptr() for y in ys])
    lib.cms_combine_gate_rocm(ptrs, len(ys), attn_out.data_ptr(), y_combined.data_ptr(), gate.data_ptr(),
                              gated.data_ptr(), n)


def gpu_prefill_forward(params: GpuMAGParams, cfg: ServeConfig, input_ids, pulse: Pulse, context: ContextState):
    """-> (logits of the last prompt position [vocab] on the host, GpuKVCache holding the prompt)."""
    s, d, nh, hd = cfg.seq_len, cfg.d_model, cfg.num_heads, cfg.head_dim
    assert d == nh * hd
    assert not cfg.residual, "gpu_prefill_forward: residual=true is not served by the cached-generation path"
    assert len(input_ids) >= s
    ids = torch.tensor([int(t) for t in input_ids[:s]], dtype=torch.int32).cuda()
    embedded = _new(s, d)
    D.call("embedding_gather_cuda", params.w_embed, ids, embedded, s, d)
    q_f32, k_f32, v_f32 = (embedded @ w.t() for w in (params.w_q, params.w_k, params.w_v))
    kv_cache = GpuKVCache(s + cfg.decode_tokens, d, s)
    kv_cache.append_f32(k_f32, v_f32, s)
    q_bf16 = _new(s, d, dtype=torch.bfloat16)
    D.call("f32_to_bf16_cuda", q_f32, q_bf16, s * d)
    attn_out_bf16 = _new(s, d, dtype=torch.bfloat16)
    attn_weights = _new(nh, s, cfg.n_persistent + cfg.window_size, dtype=torch.bfloat16)
    k_bf16 = kv_cache.k_cache_bf16[:s].contiguous()
    v_bf16 = kv_cache.v_cache_bf16[:s].contiguous()
    D.call("swa_forward_f32_cuda", q_bf16, k_bf16, v_bf16, attn_out_bf16, attn_weights, s, nh, hd, cfg.window_size,
           1, cfg.n_persistent)
    attn_out = _new(s, d)
    D.call("bf16_to_f32_cuda", attn_out_bf16, attn_out, s * d)
    ys = _levels(params, cfg, embedded, pulse, context, s)
    y_combined, gate, gated = _new(s, d), _new(s, d), _new(s, d)
    _combine_gate(ys, attn_out, y_combined, gate, gated, s * d)
    projected = gated @ params.w_o.t()
    logits = projected[s - 1:s] @ params.w_unembed
    return logits[0].cpu().numpy(), kv_cache


def gpu_single_token_forward(params: GpuMAGParams, cfg: ServeConfig, token_id, pulse: Pulse, context: ContextState,
                             kv_cache: GpuKVCache, ws: DecodeWorkspace):
    """One decode step -> logits [vocab] on the host."""
    d, v, nh, hd = cfg.d_model, cfg.vocab_size, cfg.num_heads, cfg.head_dim
    assert not cfg.residual, "gpu_single_token_forward: residual=true is not served by the cached-generation path"
    if not 0 <= token_id < v:
        raise ValueError(f"token_id {token_id} >= vocab_size {v}")
    if kv_cache.len == 0:
        raise RuntimeError("KV cache must be populated via prefill first")
    if kv_cache.len >= kv_cache.max_len:
        raise OverflowError(f"KV cache full: {kv_cache.len} >= {kv_cache.max_len}")
    ws.d_input.copy_(torch.tensor([token_id], dtype=torch.int32))
    D.call("embedding_gather_cuda", params.w_embed, ws.d_input, ws.embedded, 1, d)
    q_f32, k_f32, v_f32 = (ws.embedded @ w.t() for w in (params.w_q, params.w_k, params.w_v))
    kv_cache.append_f32(k_f32, v_f32, 1)
    D.call("f32_to_bf16_cuda", q_f32, ws.q_bf16, d)
    D.call("swa_single_token_cuda", ws.q_bf16, kv_cache.k_cache_bf16, kv_cache.v_cache_bf16, ws.attn_out_bf16,
           kv_cache.len, nh, hd, cfg.window_size, cfg.n_persistent)
    D.call("bf16_to_f32_cuda", ws.attn_out_bf16, ws.attn_out, d)
    ys = _levels(params, cfg, ws.embedded, pulse, context, 1)
    _combine_gate(ys, ws.attn_out, ws.y_combined, ws.gate, ws.gated_out, d)
    projected = ws.gated_out @ params.w_o.t()
    torch.mm(projected, params.w_unembed, out=ws.logits_gpu)
    return ws.logits_gpu[0].cpu().numpy()
