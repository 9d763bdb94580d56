"""Device-pointer dispatch layer: the host-side mirror of the reference's
`*_dd` functions (core/src/dispatch.rs:2093-3404) for the memory-rule path.

Same names, argument order and argument meaning as the reference; buffers are
torch CUDA tensors standing in for `GpuBuf<f32>` (torch is plumbing: device
memory and streams).  Every function forwards to the C ABI of
libnl_hecate_rocm.so; nothing here computes.
"""
import torch

from .ffi import lib


def _ptr(t, dtype=torch.float32):
    if t is None:
        return None
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"expected a torch tensor, got {type(t)}")
    if not t.is_cuda:
        raise ValueError("device buffer expected (tensor is on the CPU)")
    if t.dtype != dtype:
        raise ValueError(f"expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError("buffers must be contiguous")
    return t.data_ptr()


def call(name, *args):
    """Call a C-ABI entry point; tensors become device pointers."""
    conv = []
    for a in args:
        if isinstance(a, torch.Tensor):
            dt = a.dtype if a.dtype in (torch.uint16, torch.bfloat16, torch.int32) else torch.float32
            conv.append(_ptr(a, dt))
        else:
            conv.append(a)
    return getattr(lib, name)(*conv)


def cuda_sync():
    """dispatch.rs:3288 cuda_sync."""
    torch.cuda.synchronize()


def check_forward_strides(seq_len, d, batch_size, input_stride, m_stride):
    """dispatch.rs:2245-2260."""
    assert batch_size > 0, "batch_size must be > 0"
    assert input_stride >= seq_len, f"input_stride ({input_stride}) must be >= seq_len ({seq_len})"
    assert m_stride >= d * d, f"m_stride ({m_stride}) must be >= d*d ({d * d})"
    for v in (seq_len, d, batch_size, input_stride, m_stride):
        assert v <= 2**31 - 1, "argument exceeds i32"


# ── Titans LMM ──────────────────────────────────────────────────────────────
def titans_forward_dd(k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial,
                      m_states, s_states, y, seq_len, d, batch_size, input_stride, m_stride,
                      error_clip, m_norm_max):
    """dispatch.rs:2311."""
    check_forward_strides(seq_len, d, batch_size, input_stride, m_stride)
    call("titans_forward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial,
         m_states, s_states, y, seq_len, d, batch_size, input_stride, m_stride, error_clip, m_norm_max)


def titans_backward_dd(k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y,
                       d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial,
                       seq_len, d, batch_size, error_clip):
    """dispatch.rs:2337."""
    call("titans_backward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y,
         d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial,
         seq_len, d, batch_size, error_clip)


def titans_forward_dd_ckpt(k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial,
                           m_states, s_states, y, seq_len, d, checkpoint_interval, error_clip,
                           m_norm_max):
    """dispatch.rs:3061 (one chain)."""
    call("titans_forward_ckpt_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial,
         m_states, s_states, y, seq_len, d, checkpoint_interval, error_clip, m_norm_max)


def titans_backward_dd_segment(k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y,
                               d_m_seed, d_s_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta,
                               d_m_out, d_s_out, t_start, t_end, d, batch_size, seq_len, error_clip):
    """dispatch.rs:3155."""
    assert t_start < t_end, f"segment t_start={t_start} must be < t_end={t_end}"
    assert t_end <= seq_len, f"segment t_end={t_end} must be <= seq_len={seq_len}"
    assert d > 0, "d must be > 0"
    for name, b in (("d_m_seed", d_m_seed), ("d_m_out", d_m_out), ("d_s_seed", d_s_seed),
                    ("d_s_out", d_s_out)):
        assert b.numel() >= batch_size * d * d, f"{name} too small"
    call("titans_backward_segment_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, eta, m_states,
         s_states, d_y, d_m_seed, d_s_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta,
         d_m_out, d_s_out, t_start, t_end, d, batch_size, seq_len, error_clip)


# ── Hebbian rule ────────────────────────────────────────────────────────────
def hebbian_forward_dd(k_mem, v_mem, q_mem, alpha, m_initial, m_states, y,
                       seq_len, d, batch_size, input_stride, m_stride):
    """dispatch.rs:2947."""
    check_forward_strides(seq_len, d, batch_size, input_stride, m_stride)
    call("hebbian_forward_f32_cuda", k_mem, v_mem, q_mem, alpha, m_initial, m_states, y,
         seq_len, d, batch_size, input_stride, m_stride)


def hebbian_backward_dd(k_mem, v_mem, q_mem, alpha, m_states, d_y,
                        d_k_mem, d_v_mem, d_q_mem, d_alpha, d_m_initial, seq_len, d):
    """dispatch.rs:2969 (one chain)."""
    call("hebbian_backward_f32_cuda", k_mem, v_mem, q_mem, alpha, m_states, d_y,
         d_k_mem, d_v_mem, d_q_mem, d_alpha, d_m_initial, seq_len, d)


def hebbian_forward_dd_ckpt(k_mem, v_mem, q_mem, alpha, m_initial, m_states, y,
                            seq_len, d, checkpoint_interval):
    """dispatch.rs:3083 (one chain)."""
    call("hebbian_forward_ckpt_f32_cuda", k_mem, v_mem, q_mem, alpha, m_initial, m_states, y,
         seq_len, d, checkpoint_interval)


def hebbian_backward_dd_segment(k_mem, v_mem, q_mem, alpha, m_states, d_y, d_m_seed,
                                d_k_mem, d_v_mem, d_q_mem, d_alpha, d_m_out,
                                t_start, t_end, d, batch_size, seq_len):
    """dispatch.rs:3190."""
    assert t_start < t_end and t_end <= seq_len and d > 0
    call("hebbian_backward_segment_f32_cuda", k_mem, v_mem, q_mem, alpha, m_states, d_y, d_m_seed,
         d_k_mem, d_v_mem, d_q_mem, d_alpha, d_m_out, t_start, t_end, d, batch_size, seq_len)


# ── Delta rule ──────────────────────────────────────────────────────────────
def delta_forward_dd(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
                     seq_len, d, batch_size, input_stride, m_stride, error_clip, m_norm_max):
    """dispatch.rs:2264."""
    check_forward_strides(seq_len, d, batch_size, input_stride, m_stride)
    call("delta_forward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
         seq_len, d, batch_size, input_stride, m_stride, error_clip, m_norm_max)


def delta_backward_dd(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
                      d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_initial,
                      seq_len, d, batch_size, error_clip):
    """dispatch.rs:2289."""
    call("delta_backward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
         d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_initial, seq_len, d, batch_size, error_clip)


def delta_forward_dd_ckpt(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
                          seq_len, d, checkpoint_interval, error_clip, m_norm_max):
    """dispatch.rs:3039 (one chain)."""
    call("delta_forward_ckpt_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
         seq_len, d, checkpoint_interval, error_clip, m_norm_max)


def delta_backward_dd_segment(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y, d_m_seed,
                              d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_out,
                              t_start, t_end, d, batch_size, seq_len, error_clip):
    """dispatch.rs:3123."""
    assert t_start < t_end and t_end <= seq_len and d > 0
    call("delta_backward_segment_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
         d_m_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_out,
         t_start, t_end, d, batch_size, seq_len, error_clip)


# ── DGD ─────────────────────────────────────────────────────────────────────
def dgd_forward_dd(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
                   seq_len, d, batch_size, input_stride, m_stride, error_clip):
    """dispatch.rs:2990."""
    check_forward_strides(seq_len, d, batch_size, input_stride, m_stride)
    call("dgd_forward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
         seq_len, d, batch_size, input_stride, m_stride, error_clip)


def dgd_backward_dd(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
                    d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_initial, seq_len, d, error_clip):
    """dispatch.rs:3013 (single chain)."""
    call("dgd_backward_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
         d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_initial, seq_len, d, error_clip)


def dgd_forward_dd_ckpt(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
                        seq_len, d, checkpoint_interval, error_clip):
    """dispatch.rs:3102."""
    call("dgd_forward_ckpt_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y,
         seq_len, d, checkpoint_interval, error_clip)


def dgd_backward_dd_segment(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y, d_m_seed,
                            d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_out,
                            t_start, t_end, d, batch_size, seq_len, error_clip):
    """dispatch.rs:3219."""
    assert t_start < t_end and t_end <= seq_len and d > 0
    call("dgd_backward_segment_f32_cuda", k_mem, v_mem, q_mem, alpha, theta, m_states, d_y,
         d_m_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_m_out,
         t_start, t_end, d, batch_size, seq_len, error_clip)
