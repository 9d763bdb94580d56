"""Host mirror of the HOPE self-referential chunkwise step
(core/src/chunkwise_self_ref.rs:52 chunkwise_self_ref_step, :336
chunkwise_self_ref_step_backward), batched over independent chains and running
on the GPU library.  Tensors are float32 CUDA tensors; the six memories are one
[batch, 6, d, d] block in the reference's component order
(m_k, m_v, m_q, m_eta, m_alpha, m_mem)."""
from dataclasses import dataclass

import torch

from . import dispatch as D

COMPONENTS = ("m_k", "m_v", "m_q", "m_eta", "m_alpha", "m_mem")


@dataclass
class ChunkwiseSelfRefCache:
    """What the backward needs (the reference's ChunkwiseSelfRefCache, :20-30, without
    the per-token memory histories: the kernels rebuild those chunk by chunk)."""
    embedded: torch.Tensor
    k_mem: torch.Tensor
    v_mem: torch.Tensor
    q_mem: torch.Tensor
    alpha: torch.Tensor
    theta: torch.Tensor
    alpha_mean: torch.Tensor
    eta_mean: torch.Tensor
    frozen_snapshots: torch.Tensor   # [batch, num_chunks, 6, d, d]
    chunk_size: int
    num_chunks: int
    self_generated_values: bool


def _check(t, shape, name):
    if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous float32 CUDA tensor")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: shape {tuple(t.shape)} != {tuple(shape)}")


def chunkwise_self_ref_step(mems, embedded, chunk_size, self_generated_values=False):
    """mems [batch, 6, d, d] is updated in place (the reference mutates its state);
    embedded [batch, seq_len, d].  Returns (y [batch, seq_len, d], cache)."""
    if chunk_size < 1:
        raise ValueError("chunk_size must be >= 1")
    B, s, d = embedded.shape
    _check(mems, (B, 6, d, d), "mems")
    _check(embedded, (B, s, d), "embedded")
    nc = (s + chunk_size - 1) // chunk_size
    new = lambda *sh: torch.empty(*sh, dtype=torch.float32, device=embedded.device)
    y = new(B, s, d)
    c = ChunkwiseSelfRefCache(embedded, new(B, s, d), new(B, s, d), new(B, s, d), new(B, s), new(B, s),
                              new(B, s), new(B, s), new(B, nc, 6, d, d), chunk_size, nc,
                              bool(self_generated_values))
    D.call("selfref_chunkwise_forward_f32_rocm", mems, embedded, y, c.k_mem, c.v_mem, c.q_mem, c.alpha,
           c.theta, c.alpha_mean, c.eta_mean, c.frozen_snapshots, s, d, B, chunk_size,
           int(c.self_generated_values))
    return y, c


def chunkwise_self_ref_step_backward(cache, d_y):
    """Returns (d_embedded [batch, seq_len, d], d_mems [batch, 6, d, d]): the gradient
    w.r.t. the input and w.r.t. each chain's initial memories (SelfRefParamGrads)."""
    c = cache
    B, s, d = c.embedded.shape
    _check(d_y, (B, s, d), "d_y")
    d_emb = torch.empty_like(c.embedded)
    d_mems = torch.empty(B, 6, d, d, dtype=torch.float32, device=d_y.device)
    D.call("selfref_chunkwise_backward_f32_rocm", c.embedded, d_y, c.k_mem, c.v_mem, c.q_mem, c.alpha,
           c.theta, c.alpha_mean, c.eta_mean, c.frozen_snapshots, d_emb, d_mems, s, d, B, c.chunk_size,
           int(c.self_generated_values))
    return d_emb, d_mems
