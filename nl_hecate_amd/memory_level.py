"""Host mirror of the reference's per-level memory step on device buffers:
gpu_memory_forward (core/src/gpu_forward.rs:1197-1705), gpu_memory_backward
(core/src/gpu_backward.rs:459-1200), accumulate_projection_grads (:2047-2117) and the
GpuMemoryCache variants of the matrix memories (gpu_forward.rs:129-312):

    Delta, Titans, Hebbian, DGD                  full trajectory  [bs*nh, s+1, hd*hd]
    DeltaCkpt, TitansCkpt, HebbianCkpt, DGDCkpt  checkpoints      [bs*nh, n_ckpt, hd*hd]
    DeltaChunkwise, TitansChunkwise              chunk states     [bs*nh, n_chunks+1, hd*hd]
    TitansMlp                                    packed MLP state [bs*nh, s+1, 2*hd*dh + dh + hd] per head
    Mlp (MONETA, YAAD)                           W1 / W2 trajectories [s+1, dh*d], [s+1, d*dh], batch 1
    SwiGlu                                       the stateless MLP's four activation buffers

Same order of operations and the same cached tensors as the reference: projections of the input,
L2 normalisation of k and q, gate projections with their clamps, per-head layout, the rule, the final
memory carried into `context_m` under its Frobenius clamp; backward: the rule's backward per head, gate
gradients summed over heads and masked where a gate sat on a clamp bound, back to token layout,
normalisation backward, projection and gate weight gradients, d_embedded.  Tensors are float32 CUDA
tensors (torch stands in for GpuBuf); every step is a call into libnl_hecate_rocm.so or a torch matmul
for the projections (cublas_matmul_*_dd in the reference) — nothing is computed on the host.

Where the reference loops single-chain kernels over heads and refuses batch_size > 1 (checkpointed
variants, gpu_forward.rs:1608-1703), the batched entry points of the library take every chain at once
and any batch size.
"""
from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from . import dispatch as D
from .mag_layer import MemoryLevelParams

F32_MAX = 3.4028234663852886e38
RULES = ("delta", "titans", "hebbian", "dgd", "moneta", "yaad", "swiglu")
ACTIVATIONS = {"gelu": 0, "silu": 1, "relu": 2}   # MemoryActivation -> the kernels' activation id


@dataclass
class LevelConfig:
    """What gpu_memory_forward / gpu_memory_backward read from MAGConfig for one level."""
    memory_rule: str                            # MemoryRuleKind: "delta", "titans", "hebbian", "dgd"
    num_heads: int                              # cfg.swa.num_heads
    head_dim: int                               # cfg.swa.head_dim
    checkpoint_interval: Optional[int] = None   # effective_checkpoint_interval(level)
    proxy: bool = False                         # tape_strategy_for_level(level) == Proxy: frozen-M0 chunkwise
    chunk_size: Optional[int] = None            # chunk_sizes[level]; seq_len when unset
    alpha_floor: float = 0.0
    alpha_ceil: float = 1.0
    theta_floor: float = 0.0
    theta_ceil: float = F32_MAX
    error_clip: float = 0.0                     # error_clip_for_level(level); 0 = off
    m_norm_max: float = F32_MAX                 # max_m_norm(level)
    memory_layers: int = 1                      # 2 with "titans": the memory is a two-layer MLP per head
    memory_expansion_factor: int = 4            # its hidden size = factor * head_dim
    memory_activation: str = "gelu"             # "gelu", "silu", "relu"
    d_hidden: int = 0                           # MONETA / YAAD hidden size
    lp_p: float = 2.0                           # MONETA
    sign_sharpness: float = 10.0
    lambda_2: float = 0.0                       # MONETA and YAAD
    lq_q: float = 2.0
    delta: float = 1.0                          # YAAD: Huber threshold
    lambda_local: float = 0.0
    intermediate_size: int = 0                  # SwiGLU

    def __post_init__(self):
        if self.memory_rule not in RULES:
            raise ValueError(f"memory_rule {self.memory_rule!r}: expected one of {RULES}")
        if self.checkpoint_interval is not None and self.checkpoint_interval < 1:
            raise ValueError("checkpoint_interval must be > 0")
        if self.memory_activation not in ACTIVATIONS:
            raise ValueError(f"memory_activation {self.memory_activation!r}: expected one of {tuple(ACTIVATIONS)}")

    @property
    def is_mlp_mem(self):
        return self.memory_layers == 2 and self.memory_rule == "titans"


@dataclass
class GpuMemoryCache:
    """One of the reference's enum variants; `kind` is the variant's name."""
    kind: str
    k_mem: Optional[torch.Tensor] = None      # [bs*s, d] normalised
    v_mem: Optional[torch.Tensor] = None
    q_mem: Optional[torch.Tensor] = None      # [bs*s, d] normalised
    alpha: Optional[torch.Tensor] = None      # [bs*s]
    k_norms: Optional[torch.Tensor] = None
    q_norms: Optional[torch.Tensor] = None
    m_states: Optional[torch.Tensor] = None   # trajectory, checkpoints or chunk states (see the module text)
    theta: Optional[torch.Tensor] = None
    eta: Optional[torch.Tensor] = None
    s_states: Optional[torch.Tensor] = None
    checkpoint_interval: Optional[int] = None
    chunk_size: Optional[int] = None
    num_chunks: Optional[int] = None
    proxy: bool = False
    d_hidden: Optional[int] = None            # TitansMlp
    activation: Optional[int] = None
    w1_states: Optional[torch.Tensor] = None  # Mlp
    w2_states: Optional[torch.Tensor] = None
    w1_boundary: Optional[torch.Tensor] = None   # YAAD only: the memory at the start of the call
    w2_boundary: Optional[torch.Tensor] = None
    gate_buf: Optional[torch.Tensor] = None   # SwiGlu
    up_buf: Optional[torch.Tensor] = None
    fused_buf: Optional[torch.Tensor] = None
    cache_buf: Optional[torch.Tensor] = None

    def dgd_delta_norm(self, s, d, batch_size, num_heads):
        """|M k - v|_2 of the last token against the memory that token was written into
        (gpu_forward.rs:328-437): 0 for several heads, for Hebbian, and without tokens."""
        if num_heads > 1 or s == 0 or self.kind.startswith("Hebbian") or self.kind in ("TitansMlp", "Mlp", "SwiGlu"):
            return 0.0
        if self.proxy:   # only final states are kept (the TNT inner caches of a proxy level)
            return 0.0
        assert batch_size <= 1, "dgd_delta_norm reads batch slot 0 only"
        if self.kind.endswith("Chunkwise"):
            if not self.num_chunks:
                return 0.0
            slot = self.num_chunks - 1
        elif self.kind.endswith("Ckpt"):
            c = self.checkpoint_interval
            n_ckpt = (s + c - 1) // c + 1
            slot = n_ckpt - 2 if n_ckpt >= 2 else 0
        else:
            slot = s - 1
        out = torch.zeros(1, device=self.k_mem.device)
        D.call("dgd_delta_norm_cuda", self.m_states[0, slot].contiguous(), self.k_mem.reshape(-1, d)[s - 1].contiguous(),
               self.v_mem.reshape(-1, d)[s - 1].contiguous(), out, d)
        return float(out.item())

    def alpha_stats(self, alpha_floor):
        """gpu_forward.rs:440-503."""
        return None if self.alpha is None else GateStats.from_slice(self.alpha.cpu().numpy(), alpha_floor, True)

    def eta_stats(self):
        """gpu_forward.rs:505-564: only the Titans variants have a momentum gate."""
        return None if self.eta is None else GateStats.from_slice(self.eta.cpu().numpy(), 0.0, True)

    def theta_stats(self, theta_ceil):
        """gpu_forward.rs:566-623 (ThetaStats: the bound is a ceiling)."""
        return None if self.theta is None else GateStats.from_slice(self.theta.cpu().numpy(), theta_ceil, False)


@dataclass
class GateStats:
    """Distribution of one gate over the tokens of a forward pass (GateStats / ThetaStats,
    gpu_forward.rs:626-752): interpolated quantiles and the fraction of tokens on the configured bound."""
    count: int
    min: float
    max: float
    mean: float
    median: float
    p95: float
    p99: float
    frac_at_bound: float

    @staticmethod
    def from_slice(values, bound, bound_is_floor):
        v = np.sort(np.asarray(values, np.float32).ravel())
        n = v.size
        assert n > 0
        def quantile(p):
            rank = p * (n - 1.0)
            lo = int(np.floor(rank))
            hi = min(lo + 1, n - 1)
            frac = rank - lo
            return float(np.float32(float(v[lo]) * (1.0 - frac) + float(v[hi]) * frac))
        if bound_is_floor and bound > 0.0:
            at = int((v <= np.float32(bound * (1.0 + 1e-4))).sum())
        elif not bound_is_floor and bound < F32_MAX:
            at = int((v >= np.float32(bound * (1.0 - 1e-4))).sum())
        else:
            at = 0
        return GateStats(n, float(v[0]), float(v[-1]), float(v.sum(dtype=np.float32) / np.float32(n)),
                         quantile(0.5), quantile(0.95), quantile(0.99), at / n)


@dataclass
class LevelGrads:
    """GpuLevelGrads: gradients of one level's outer-loop parameters (overwritten by a backward)."""
    d_w_k_mem: torch.Tensor
    d_w_v_mem: torch.Tensor
    d_w_q_mem: torch.Tensor
    d_w_alpha: torch.Tensor
    d_b_alpha: torch.Tensor
    d_w_theta: torch.Tensor
    d_b_theta: torch.Tensor
    d_w_eta: torch.Tensor
    d_b_eta: torch.Tensor
    d_gate_proj: Optional[torch.Tensor] = None   # SwiGLU levels ([inter, d], [inter, d], [d, inter])
    d_up_proj: Optional[torch.Tensor] = None
    d_down_proj: Optional[torch.Tensor] = None

    @staticmethod
    def zeros(d, device="cuda", intermediate=0):
        z = lambda *sh: torch.zeros(*sh, dtype=torch.float32, device=device)
        g = LevelGrads(z(d, d), z(d, d), z(d, d), z(2 * d), z(1), z(2 * d), z(1), z(2 * d), z(1))
        if intermediate:
            g.d_gate_proj, g.d_up_proj, g.d_down_proj = z(intermediate, d), z(intermediate, d), z(d, intermediate)
        return g


@dataclass
class SwiGluLevelParams:
    """The parameters a SwiGLU level reads (GpuMemoryLevelParams gate_proj / up_proj / down_proj)."""
    gate_proj: torch.Tensor    # [intermediate, d]
    up_proj: torch.Tensor      # [intermediate, d]
    down_proj: torch.Tensor    # [d, intermediate]


def checkpoint_count(seq_len, c):
    """gpu_forward.rs:2885-2897: M_0, one slot per C-token boundary, the final state."""
    assert c > 0, "checkpoint_interval must be > 0"
    return 1 + sum(1 for t in range(seq_len) if (t + 1) % c == 0 or t + 1 == seq_len)


def segment_boundaries(seq_len, c):
    """gpu_backward.rs:1770-1782 -> [(t_start, t_end, ckpt_idx)]."""
    assert c > 0, "checkpoint_interval must be > 0"
    return [(t, min(t + c, seq_len), i) for i, t in enumerate(range(0, seq_len, c))]


def _new(*shape):
    return torch.empty(*shape, dtype=torch.float32, device="cuda")


def _zeros(*shape):
    return torch.zeros(*shape, dtype=torch.float32, device="cuda")


def _heads(cfg, t, bs, s):
    out = _new(bs * cfg.num_heads, s, cfg.head_dim)
    D.call("transpose_heads_f32_cuda", t, out, bs, s, cfg.num_heads, cfg.head_dim, 1)
    return out


def _tokens(cfg, t, bs, s):
    out = _new(bs * s, cfg.num_heads * cfg.head_dim)
    D.call("transpose_heads_f32_cuda", t, out, bs, s, cfg.num_heads, cfg.head_dim, 0)
    return out


def _gate_heads(cfg, g, bs, s):
    out = _new(bs * cfg.num_heads, s)
    D.call("broadcast_heads_f32_cuda", g, out, bs, s, cfg.num_heads)
    return out


def _sum_heads(cfg, g, bs, s):
    out = _new(bs * s)
    D.call("sum_heads_f32_cuda", g, out, bs, s, cfg.num_heads)
    return out


def gpu_memory_forward(level_params: MemoryLevelParams, cfg: LevelConfig, embedded, context_m, s, d, batch_size):
    """embedded [bs*s, d]; context_m [bs*nh, hd*hd]: the level's carried memory per (batch, head), read as the
    initial state and overwritten with the final one.  Returns (y [bs*s, d], GpuMemoryCache)."""
    lp, bs, nh, hd = level_params, batch_size, cfg.num_heads, cfg.head_dim
    assert nh * hd == d, "num_heads * head_dim must equal d"
    n, B, dd = bs * s, bs * nh, hd * hd
    assert tuple(embedded.shape) == (n, d)
    rule = cfg.memory_rule
    if rule == "swiglu":   # stateless: no projections, no memory (gpu_forward.rs:1705-1727)
        inter = cfg.intermediate_size
        bufs = [_new(n, inter) for _ in range(4)]
        y = _new(n, d)
        D.call("swiglu_forward_f32_cuda_dd", embedded, lp.gate_proj, lp.up_proj, lp.down_proj, y, *bufs, n, d, inter)
        return y, GpuMemoryCache("SwiGlu", gate_buf=bufs[0], up_buf=bufs[1], fused_buf=bufs[2], cache_buf=bufs[3])
    if cfg.is_mlp_mem and (cfg.checkpoint_interval is not None or cfg.proxy):
        raise ValueError("MLP memory (memory_layers >= 2) supports neither checkpointing nor the proxy strategy")
    if rule in ("moneta", "yaad"):
        if cfg.checkpoint_interval is not None:
            raise ValueError(f"checkpointed forward is not supported for {rule}: use checkpoint_interval=None")
        if bs != 1:
            raise ValueError(f"{rule} forward with batch_size > 1 is not supported")
    elif not cfg.is_mlp_mem:
        assert tuple(context_m.shape) == (B, dd)
    k_mem, v_mem, q_mem = embedded @ lp.w_k.t(), embedded @ lp.w_v.t(), embedded @ lp.w_q.t()
    k_norms, q_norms = _new(n), _new(n)
    D.call("l2_normalize_rows_f32_cuda", k_mem, k_norms, n, d, 1e-8)
    D.call("l2_normalize_rows_f32_cuda", q_mem, q_norms, n, d, 1e-8)
    alpha, theta = _new(n), _new(n)
    D.call("gate_compute_cuda", k_mem, v_mem, lp.w_alpha, lp.b_alpha, alpha, n, d, 0)
    D.call("gate_compute_cuda", k_mem, v_mem, lp.w_theta, lp.b_theta, theta, n, d, 1)
    if cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0:
        D.call("clamp_f32_cuda", alpha, n, cfg.alpha_floor, cfg.alpha_ceil)
    if cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX:
        D.call("clamp_f32_cuda", theta, n, cfg.theta_floor, cfg.theta_ceil)
    common = dict(k_mem=k_mem, v_mem=v_mem, q_mem=q_mem, alpha=alpha, k_norms=k_norms, q_norms=q_norms)
    if rule in ("moneta", "yaad"):
        return _mlp_forward(cfg, context_m, theta, common, s, d)
    kh, vh, qh = (_heads(cfg, t, bs, s) for t in (k_mem, v_mem, q_mem))
    ah, th = _gate_heads(cfg, alpha, bs, s), _gate_heads(cfg, theta, bs, s)
    eta = eh = None
    if rule == "titans":   # compute_eta, gpu_forward.rs:2866
        eta = _new(n)
        D.call("gate_compute_cuda", k_mem, v_mem, lp.w_eta, lp.b_eta, eta, n, d, 0)
        eh = _gate_heads(cfg, eta, bs, s)
    yh = _new(B, s, hd)
    clip, mx, C = cfg.error_clip, cfg.m_norm_max, cfg.checkpoint_interval
    s_states = None
    if cfg.is_mlp_mem:
        # the memory of a head is {W1, b1, W2, b2} packed; the kernel projects per token, so the carried state
        # needs no clamp afterwards (gpu_forward.rs:1473-1510)
        d_h = cfg.memory_expansion_factor * hd
        n_state = 2 * hd * d_h + d_h + hd
        assert tuple(context_m.shape) == (B, n_state)
        act = ACTIVATIONS[cfg.memory_activation]
        m_states, s_states = _new(B, s + 1, n_state), _new(B, s + 1, n_state)
        D.call("titans_mlp_forward_f32_cuda", kh, vh, qh, ah, th, eh, context_m, _zeros(B, n_state), m_states, s_states,
               yh, s, hd, d_h, B, s * hd, (s + 1) * n_state, act, mx)
        context_m.copy_(m_states[:, -1])
        cache = GpuMemoryCache("TitansMlp", theta=theta, eta=eta, m_states=m_states, s_states=s_states, d_hidden=d_h,
                               activation=act, **common)
        return _tokens(cfg, yh, bs, s), cache
    if C is not None:
        n_ck = checkpoint_count(s, C)
        m_states = _new(B, n_ck, dd)
        if rule == "titans":
            s_states = _new(B, n_ck, dd)
            D.call("titans_forward_ckpt_batched_f32_rocm", kh, vh, qh, ah, th, eh, context_m, _zeros(B, dd), m_states,
                   s_states, yh, s, hd, B, C, clip, mx)
        elif rule == "hebbian":
            flat = lambda t: t.view(-1)
            for b in range(B):   # single-chain entry point, as the reference calls it (gpu_forward.rs:1669)
                D.call("hebbian_forward_ckpt_f32_cuda", flat(kh)[b * s * hd:], flat(vh)[b * s * hd:],
                       flat(qh)[b * s * hd:], flat(ah)[b * s:], flat(context_m)[b * dd:],
                       flat(m_states)[b * n_ck * dd:], flat(yh)[b * s * hd:], s, hd, C)
        else:   # DGD: Delta without the per-token projection (core/kernels/dgd_forward.cu:6-11)
            D.call("delta_forward_ckpt_batched_f32_rocm", kh, vh, qh, ah, th, context_m, m_states, yh, s, hd, B, C,
                   clip, F32_MAX if rule == "dgd" else mx)
        kind = {"delta": "DeltaCkpt", "titans": "TitansCkpt", "hebbian": "HebbianCkpt", "dgd": "DGDCkpt"}[rule]
        cache = GpuMemoryCache(kind, theta=None if rule == "hebbian" else theta, eta=eta, m_states=m_states,
                               s_states=s_states, checkpoint_interval=C, **common)
    elif cfg.proxy and rule in ("delta", "titans"):
        cs = cfg.chunk_size or s
        nc = (s + cs - 1) // cs
        m_states = _new(B, nc + 1, dd)
        if rule == "titans":
            s_states = _new(B, nc + 1, dd)
            D.call("titans_chunkwise_forward_f32_cuda", kh, vh, qh, ah, th, eh, context_m, _zeros(B, dd), m_states,
                   s_states, yh, s, hd, B, cs, clip, mx)
        else:
            D.call("delta_chunkwise_forward_f32_cuda", kh, vh, qh, ah, th, context_m, m_states, yh, s, hd, B, cs,
                   clip, mx)
        cache = GpuMemoryCache("TitansChunkwise" if rule == "titans" else "DeltaChunkwise", theta=theta, eta=eta,
                               m_states=m_states, s_states=s_states, chunk_size=cs, num_chunks=nc, **common)
    else:
        m_states = _new(B, s + 1, dd)
        if rule == "titans":
            s_states = _new(B, s + 1, dd)
            D.titans_forward_dd(kh, vh, qh, ah, th, eh, context_m, _zeros(B, dd), m_states, s_states, yh, s, hd, B,
                                s, dd, clip, mx)
        elif rule == "hebbian":
            D.call("hebbian_forward_f32_cuda", kh, vh, qh, ah, context_m, m_states, yh, s, hd, B, s, dd)
        elif rule == "dgd":
            D.call("dgd_forward_f32_cuda", kh, vh, qh, ah, th, context_m, m_states, yh, s, hd, B, s, dd, clip)
        else:
            D.call("delta_forward_f32_cuda", kh, vh, qh, ah, th, context_m, m_states, yh, s, hd, B, s, dd, clip, mx)
        kind = {"delta": "Delta", "titans": "Titans", "hebbian": "Hebbian", "dgd": "DGD"}[rule]
        cache = GpuMemoryCache(kind, theta=None if rule == "hebbian" else theta, eta=eta, m_states=m_states,
                               s_states=s_states, **common)
    # copy_final_m_batch + m_norm_clamp_batch_f32_cuda (gpu_forward.rs:2824, :1431)
    context_m.copy_(m_states[:, -1])
    D.call("m_norm_clamp_batch_f32_cuda", context_m, hd, B, mx)
    return _tokens(cfg, yh, bs, s), cache


def _mlp_forward(cfg, context_m, theta, common, s, d):
    """MONETA / YAAD: an MLP memory at model width, one sequence; context_m = [W1 (dh x d) | W2 (d x dh)]
    (gpu_forward.rs:1729-1852)."""
    dh = cfg.d_hidden
    w1_size, w2_size = dh * d, d * dh
    flat = context_m.view(-1)
    if flat.numel() < w1_size + w2_size:
        raise ValueError(f"{cfg.memory_rule}: context_m too small ({flat.numel()} elements) for [W1|W2] = "
                         f"{w1_size + w2_size} (d_hidden={dh}, d={d})")
    w1, w2 = flat[:w1_size], flat[w1_size:w1_size + w2_size]
    w1_states, w2_states, y = _new(s + 1, w1_size), _new(s + 1, w2_size), _new(s, d)
    c = common
    b1 = b2 = None
    if cfg.memory_rule == "yaad":   # the memory at the start of the call anchors the local retention
        b1, b2 = w1.clone(), w2.clone()
        D.call("mlp_forward_huber_f32_cuda", c["k_mem"], c["v_mem"], c["q_mem"], c["alpha"], theta, w1, w2, b1, b2,
               w1_states, w2_states, y, s, d, dh, cfg.delta, cfg.lambda_local, cfg.lambda_2)
    else:
        D.call("mlp_forward_lp_f32_cuda", c["k_mem"], c["v_mem"], c["q_mem"], c["alpha"], theta, w1, w2, w1_states,
               w2_states, y, s, d, dh, cfg.lp_p, cfg.sign_sharpness, cfg.lambda_2, cfg.lq_q)
    w1.copy_(w1_states[s])
    w2.copy_(w2_states[s])
    return y, GpuMemoryCache("Mlp", theta=theta, w1_states=w1_states, w2_states=w2_states, w1_boundary=b1,
                             w2_boundary=b2, **common)


def gpu_memory_backward(level_params: MemoryLevelParams, cfg: LevelConfig, mem_cache: GpuMemoryCache, d_y, embedded,
                        level_grads: LevelGrads, s, d, batch_size):
    """d_y, embedded [bs*s, d].  Writes the level's parameter gradients into level_grads and returns
    d_embedded [bs*s, d]."""
    c, bs, nh, hd = mem_cache, batch_size, cfg.num_heads, cfg.head_dim
    n, B, dd = bs * s, bs * nh, hd * hd
    kind = c.kind
    if kind == "SwiGlu":   # direct weight gradients, d_x returned (gpu_backward.rs:1736-1760)
        inter = cfg.intermediate_size
        d_x = _new(n, d)
        D.call("swiglu_backward_f32_cuda_dd", d_y, embedded, level_params.gate_proj, level_params.up_proj,
               level_params.down_proj, c.fused_buf, c.gate_buf, c.up_buf, c.cache_buf, d_x, level_grads.d_gate_proj,
               level_grads.d_up_proj, level_grads.d_down_proj, n, d, inter)
        return d_x
    if kind == "Mlp":
        return _mlp_backward(level_params, cfg, c, d_y, embedded, level_grads, s, d, bs)
    has_theta, has_eta = not kind.startswith("Hebbian"), kind.startswith("Titans")
    dyh = _heads(cfg, d_y, bs, s)
    kh, vh, qh = (_heads(cfg, t, bs, s) for t in (c.k_mem, c.v_mem, c.q_mem))
    ah = _gate_heads(cfg, c.alpha, bs, s)
    th = _gate_heads(cfg, c.theta, bs, s) if has_theta else None
    eh = _gate_heads(cfg, c.eta, bs, s) if has_eta else None
    dkh, dvh, dqh = _zeros(B, s, hd), _zeros(B, s, hd), _zeros(B, s, hd)
    dah, dth, deh = _zeros(B, s), _zeros(B, s), _zeros(B, s)
    d_m0, d_s0 = _zeros(dd), _zeros(dd)
    clip, mx = cfg.error_clip, cfg.m_norm_max
    if kind in ("Delta", "DGD"):
        D.call("delta_backward_f32_cuda", kh, vh, qh, ah, th, c.m_states, dyh, dkh, dvh, dqh, dah, dth, d_m0, s, hd,
               B, clip)
    elif kind == "Titans":
        D.titans_backward_dd(kh, vh, qh, ah, th, eh, c.m_states, c.s_states, dyh, dkh, dvh, dqh, dah, dth, deh, d_m0,
                             d_s0, s, hd, B, clip)
    elif kind == "DeltaChunkwise":
        D.call("delta_chunkwise_backward_f32_cuda", kh, vh, qh, ah, th, c.m_states, dyh, dkh, dvh, dqh, dah, dth,
               d_m0, s, hd, B, c.chunk_size, clip, mx)
    elif kind == "TitansChunkwise":
        D.call("titans_chunkwise_backward_f32_cuda", kh, vh, qh, ah, th, eh, c.m_states, c.s_states, dyh, dkh, dvh,
               dqh, dah, dth, deh, d_m0, d_s0, s, hd, B, c.chunk_size, clip, mx)
    elif kind == "Hebbian":
        flat = lambda t: t.view(-1)
        for b in range(B):   # single-chain entry point, one call per head (gpu_backward.rs:913-930)
            D.call("hebbian_backward_f32_cuda", flat(kh)[b * s * hd:], flat(vh)[b * s * hd:], flat(qh)[b * s * hd:],
                   flat(ah)[b * s:], flat(c.m_states)[b * (s + 1) * dd:], flat(dyh)[b * s * hd:],
                   flat(dkh)[b * s * hd:], flat(dvh)[b * s * hd:], flat(dqh)[b * s * hd:], flat(dah)[b * s:], d_m0,
                   s, hd)
    elif kind in ("DeltaCkpt", "DGDCkpt"):
        # one call walks the segments in reverse (the host loop delta_backward_checkpointed, gpu_backward.rs:1791);
        # the DGD replay leaves the projection off as its forward did (:1156-1161)
        D.call("delta_backward_ckpt_f32_rocm", kh, vh, qh, ah, th, c.m_states, dyh, dkh, dvh, dqh, dah, dth, d_m0, s,
               hd, B, c.checkpoint_interval, clip, F32_MAX if kind == "DGDCkpt" else mx)
    elif kind == "TitansMlp":
        n_state = c.m_states.shape[-1]
        D.call("titans_mlp_backward_f32_cuda", kh, vh, qh, ah, th, eh, c.m_states, c.s_states, dyh, dkh, dvh, dqh, dah,
               dth, deh, _zeros(n_state), _zeros(n_state), s, hd, c.d_hidden, B, s * hd, (s + 1) * n_state,
               c.activation, mx)
    elif kind == "TitansCkpt":
        D.call("titans_backward_ckpt_f32_rocm", kh, vh, qh, ah, th, eh, c.m_states, c.s_states, dyh, dkh, dvh, dqh,
               dah, dth, deh, d_m0, d_s0, s, hd, B, c.checkpoint_interval, clip, mx)
    elif kind == "HebbianCkpt":
        _hebbian_backward_checkpointed(kh, vh, qh, ah, c.m_states, dyh, dkh, dvh, dqh, dah, s, hd,
                                       c.checkpoint_interval, B)
    else:
        raise ValueError(f"gpu_memory_backward: unsupported cache variant {kind}")
    d_alpha = _sum_heads(cfg, dah, bs, s)
    d_theta = _sum_heads(cfg, dth, bs, s) if has_theta else None
    d_eta = _sum_heads(cfg, deh, bs, s) if has_eta else None
    # straight-through clamps: no gradient where the gate sat on a bound
    if cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0:
        D.call("theta_clamp_mask_cuda", c.alpha, d_alpha, n, cfg.alpha_floor, cfg.alpha_ceil)
    if has_theta and (cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX):
        D.call("theta_clamp_mask_cuda", c.theta, d_theta, n, cfg.theta_floor, cfg.theta_ceil)
    d_k, d_v, d_q = (_tokens(cfg, t, bs, s) for t in (dkh, dvh, dqh))
    return accumulate_projection_grads(level_params, embedded, c, d_k, d_v, d_q, d_alpha, d_theta, d_eta, level_grads,
                                       s, d, bs)


def _mlp_backward(level_params, cfg, c, d_y, embedded, level_grads, s, d, bs):
    """MONETA (L2 retention only: lq_q = 2) / YAAD backward at model width, one sequence
    (gpu_backward.rs:1635-1733).  As in the reference the gradients of the initial W1, W2 are computed and
    not used."""
    if bs != 1:
        raise ValueError("MLP memory backward with batch_size > 1 is not supported")
    dh = cfg.d_hidden
    d_k, d_v, d_q = _zeros(s, d), _zeros(s, d), _zeros(s, d)
    d_alpha, d_theta = _zeros(s), _zeros(s)
    d_w1, d_w2 = _zeros(dh * d), _zeros(d * dh)
    if (c.w1_boundary is None) != (c.w2_boundary is None):
        raise ValueError("MLP backward: W1 and W2 boundaries must both be present (YAAD) or both absent (MONETA)")
    if c.w1_boundary is not None:
        D.call("mlp_backward_huber_f32_cuda", c.k_mem, c.v_mem, c.q_mem, c.alpha, c.theta, c.w1_states, c.w2_states,
               c.w1_boundary, c.w2_boundary, d_y, d_k, d_v, d_q, d_alpha, d_theta, d_w1, d_w2, s, d, dh, cfg.delta,
               cfg.lambda_local, cfg.lambda_2)
    else:
        if abs(cfg.lq_q - 2.0) >= 1e-6:
            raise ValueError(f"MONETA backward only supports lq_q=2.0 (L2 retention); got {cfg.lq_q}")
        D.call("mlp_backward_lp_f32_cuda", c.k_mem, c.v_mem, c.q_mem, c.alpha, c.theta, c.w1_states, c.w2_states, d_y,
               d_k, d_v, d_q, d_alpha, d_theta, d_w1, d_w2, s, d, dh, cfg.lp_p, cfg.sign_sharpness, cfg.lambda_2,
               cfg.lq_q)
    if cfg.alpha_floor > 0.0 or cfg.alpha_ceil < 1.0:
        D.call("theta_clamp_mask_cuda", c.alpha, d_alpha, s, cfg.alpha_floor, cfg.alpha_ceil)
    if cfg.theta_floor > 0.0 or cfg.theta_ceil < F32_MAX:
        D.call("theta_clamp_mask_cuda", c.theta, d_theta, s, cfg.theta_floor, cfg.theta_ceil)
    return accumulate_projection_grads(level_params, embedded, c, d_k, d_v, d_q, d_alpha, d_theta, None, level_grads, s,
                                       d, 1)


def _hebbian_backward_checkpointed(kh, vh, qh, ah, m_ckpt, dyh, dkh, dvh, dqh, dah, s, hd, c, B):
    """hebbian_backward_checkpointed (gpu_backward.rs:1967-2035): per segment, last first, replay the
    trajectory of every chain from its checkpoint, then the batched segment backward seeded with the
    state gradient of the segment after it."""
    dd = hd * hd
    n_ck = checkpoint_count(s, c)
    seg_max = min(c, s)
    local_m, local_y = _new(B, seg_max + 1, dd), _new(B, seg_max, hd)
    seed, out = _zeros(B, dd), _zeros(B, dd)
    flat = lambda t: t.view(-1)
    for t0, t1, ci in reversed(segment_boundaries(s, c)):
        seg = t1 - t0
        lm = local_m if seg == seg_max else _new(B, seg + 1, dd)
        ly = local_y if seg == seg_max else _new(B, seg, hd)
        D.call("hebbian_forward_f32_cuda", flat(kh)[t0 * hd:], flat(vh)[t0 * hd:], flat(qh)[t0 * hd:], flat(ah)[t0:],
               flat(m_ckpt)[ci * dd:], lm, ly, seg, hd, B, s, n_ck * dd)
        out.zero_()
        D.call("hebbian_backward_segment_f32_cuda", kh, vh, qh, ah, lm, dyh, seed, dkh, dvh, dqh, dah, out, t0, t1, hd,
               B, s)
        seed.copy_(out)


def accumulate_projection_grads(level_params, embedded, cache, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta,
                                level_grads, s, d, batch_size):
    """gpu_backward.rs:2047-2117.  As in the reference the gate gradients reach the gate weights and biases
    only; k_mem and v_mem receive nothing through the gates."""
    lp, c, g = level_params, cache, level_grads
    n = batch_size * s
    d_k_raw, d_q_raw = _new(n, d), _new(n, d)
    D.call("l2_normalize_backward_f32_cuda", d_k_mem, c.k_mem, c.k_norms, d_k_raw, n, d, 1e-8)
    D.call("l2_normalize_backward_f32_cuda", d_q_mem, c.q_mem, c.q_norms, d_q_raw, n, d, 1e-8)
    torch.mm(d_k_raw.t(), embedded, out=g.d_w_k_mem)
    torch.mm(d_v_mem.t(), embedded, out=g.d_w_v_mem)
    torch.mm(d_q_raw.t(), embedded, out=g.d_w_q_mem)
    d_embedded = d_k_raw @ lp.w_k
    d_embedded.addmm_(d_v_mem, lp.w_v)
    d_embedded.addmm_(d_q_raw, lp.w_q)
    z = d_alpha   # placeholder for the absent gates: not read when the has_* flag is 0
    D.call("gate_backward_cuda", d_alpha, c.alpha, d_theta if d_theta is not None else z,
           c.theta if c.theta is not None else z, d_eta if d_eta is not None else z,
           c.eta if c.eta is not None else z, c.k_mem, c.v_mem, g.d_w_alpha, g.d_b_alpha, g.d_w_theta, g.d_b_theta,
           g.d_w_eta, g.d_b_eta, n, d, int(d_theta is not None), int(d_eta is not None))
    return d_embedded
