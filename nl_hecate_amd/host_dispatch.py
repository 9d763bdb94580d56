"""Host-slice dispatch layer: the mirror of the reference's `*_dispatch` functions
(core/src/dispatch.rs:378-460, 746-895, 1083-1224), the entry points the rule
structs and the opaque VJP blocks of the Wengert tape call with CPU slices.

Same names, argument order and in/out convention as the reference: inputs and
pre-allocated outputs are float32 numpy arrays, outputs are written in place.
Every function forwards to the C ABI (`nlh_*_dispatch`), which stages one chain
on the device; nothing here computes, and there is no CPU path.
"""
import ctypes

import numpy as np

from .ffi import lib


def _hp(a, writable=False):
    if not isinstance(a, np.ndarray):
        raise TypeError(f"expected a numpy array, got {type(a)}")
    if a.dtype != np.float32:
        raise ValueError(f"expected float32, got {a.dtype}")
    if not a.flags["C_CONTIGUOUS"]:
        raise ValueError("slices must be contiguous")
    if writable and not a.flags["WRITEABLE"]:
        raise ValueError("output slice is read-only")
    return a.ctypes.data_as(ctypes.c_void_p)


def _need(a, n, name):
    assert a.size == n, f"{name}: expected {n} elements, got {a.size}"


def delta_forward_dispatch(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y, seq_len, d,
                           error_clip, m_norm_max):
    """dispatch.rs:746. m_states [(seq_len+1)*d*d] and y [seq_len*d] are written."""
    _need(m_states, (seq_len + 1) * d * d, "m_states"); _need(y, seq_len * d, "y")
    lib.nlh_delta_forward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(m_initial),
                                   _hp(m_states, True), _hp(y, True), seq_len, d, error_clip, m_norm_max)


def delta_backward_dispatch(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y, d_k_mem, d_v_mem, d_q_mem,
                            d_alpha, d_theta, d_m_initial, seq_len, d, error_clip):
    """dispatch.rs:775."""
    _need(m_states, (seq_len + 1) * d * d, "m_states"); _need(d_m_initial, d * d, "d_m_initial")
    lib.nlh_delta_backward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(m_states),
                                    _hp(d_y), _hp(d_k_mem, True), _hp(d_v_mem, True), _hp(d_q_mem, True),
                                    _hp(d_alpha, True), _hp(d_theta, True), _hp(d_m_initial, True), seq_len, d,
                                    error_clip)


def titans_forward_dispatch(k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial, m_states, s_states, y,
                            seq_len, d, error_clip, m_norm_max):
    """dispatch.rs:810."""
    _need(m_states, (seq_len + 1) * d * d, "m_states"); _need(s_states, (seq_len + 1) * d * d, "s_states")
    lib.nlh_titans_forward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(eta),
                                    _hp(m_initial), _hp(s_initial), _hp(m_states, True), _hp(s_states, True),
                                    _hp(y, True), seq_len, d, error_clip, m_norm_max)


def titans_backward_dispatch(k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y, d_k_mem, d_v_mem,
                             d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial, seq_len, d, error_clip):
    """dispatch.rs:842."""
    _need(m_states, (seq_len + 1) * d * d, "m_states"); _need(s_states, (seq_len + 1) * d * d, "s_states")
    lib.nlh_titans_backward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(eta),
                                     _hp(m_states), _hp(s_states), _hp(d_y), _hp(d_k_mem, True), _hp(d_v_mem, True),
                                     _hp(d_q_mem, True), _hp(d_alpha, True), _hp(d_theta, True), _hp(d_eta, True),
                                     _hp(d_m_initial, True), _hp(d_s_initial, True), seq_len, d, error_clip)


def hebbian_forward_dispatch(k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, d, m_norm_max):
    """dispatch.rs:1083. A finite positive m_norm_max is refused (the reference runs it on the CPU)."""
    _need(m_states, (seq_len + 1) * d * d, "m_states")
    lib.nlh_hebbian_forward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(m_initial),
                                     _hp(m_states, True), _hp(y, True), seq_len, d, m_norm_max)


def hebbian_backward_dispatch(k_mem, v_mem, q_mem, alpha, m_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                              d_m_initial, seq_len, d):
    """dispatch.rs:1110."""
    _need(m_states, (seq_len + 1) * d * d, "m_states")
    lib.nlh_hebbian_backward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(m_states), _hp(d_y),
                                      _hp(d_k_mem, True), _hp(d_v_mem, True), _hp(d_q_mem, True), _hp(d_alpha, True),
                                      _hp(d_m_initial, True), seq_len, d)


def dgd_forward_dispatch(k_mem, v_mem, q_mem, alpha, theta, m_initial, m_states, y, seq_len, d, error_clip):
    """dispatch.rs:1153."""
    _need(m_states, (seq_len + 1) * d * d, "m_states")
    lib.nlh_dgd_forward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(m_initial),
                                 _hp(m_states, True), _hp(y, True), seq_len, d, error_clip)


def dgd_backward_dispatch(k_mem, v_mem, q_mem, alpha, theta, m_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                          d_theta, d_m_initial, seq_len, d, error_clip):
    """dispatch.rs:1182."""
    _need(m_states, (seq_len + 1) * d * d, "m_states")
    lib.nlh_dgd_backward_dispatch(_hp(k_mem), _hp(v_mem), _hp(q_mem), _hp(alpha), _hp(theta), _hp(m_states),
                                  _hp(d_y), _hp(d_k_mem, True), _hp(d_v_mem, True), _hp(d_q_mem, True),
                                  _hp(d_alpha, True), _hp(d_theta, True), _hp(d_m_initial, True), seq_len, d,
                                  error_clip)


def swa_forward_dispatch(q, k, v, out, attn_weights, seq_len, num_heads, head_dim, window_size):
    """dispatch.rs:378. Slices are float32; the device computes on their bf16 roundings."""
    _need(out, seq_len * num_heads * head_dim, "out")
    _need(attn_weights, num_heads * seq_len * window_size, "attn_weights")
    lib.nlh_swa_forward_dispatch(_hp(q), _hp(k), _hp(v), _hp(out, True), _hp(attn_weights, True), seq_len,
                                 num_heads, head_dim, window_size)


def swa_backward_dispatch(q, k, v, attn_weights, d_attn_out, d_q, d_k, d_v, seq_len, num_heads, head_dim,
                          window_size):
    """dispatch.rs:408. d_q, d_k, d_v are not zeroed here: the caller pre-zeroes them."""
    _need(attn_weights, num_heads * seq_len * window_size, "attn_weights")
    lib.nlh_swa_backward_dispatch(_hp(q), _hp(k), _hp(v), _hp(attn_weights), _hp(d_attn_out), _hp(d_q, True),
                                  _hp(d_k, True), _hp(d_v, True), seq_len, num_heads, head_dim, window_size)
