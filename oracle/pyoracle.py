"""TEST INFRASTRUCTURE ONLY: numpy front-end of the CPU oracle (liboracle.so).

Only the test-suite, ``__graft_entry__.smoke()`` and the CPU-baseline leg of
``bench.py`` may import this module.  The product path (``nl_hecate_amd``)
never does: it fails loudly when the HIP library is missing.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

F32_MAX = float(np.finfo(np.float32).max)


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _arg(x, real):
    """numpy array -> pointer; python scalar -> c scalar (ints stay ints)."""
    if isinstance(x, np.ndarray):
        assert x.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
        return x.ctypes.data_as(ctypes.c_void_p)
    if x is None:
        return ctypes.c_void_p(0)
    if isinstance(x, (int, np.integer)):
        return ctypes.c_int(int(x))
    return real(float(x))


def _call(name, *args, real=ctypes.c_float, restype=None):
    fn = getattr(lib(), name)
    fn.restype = restype
    return fn(*[_arg(a, real) for a in args])


def _np(real):
    return np.float32 if real is ctypes.c_float else np.float64


def _sfx(dtype):
    return ("_f32", ctypes.c_float) if np.dtype(dtype) == np.float32 else ("_f64", ctypes.c_double)


def _c(x, dt):
    return np.ascontiguousarray(x, dtype=dt)


# ── utilities ───────────────────────────────────────────────────────────────
def simple_rng_uniform(n, seed, scale=0.1):
    """SimpleRng::fill_uniform (core/src/tensor.rs:380-408); rand_buf of the
    reference's CUDA tests is this with scale 0.1."""
    out = np.empty(n, np.float32)
    f = lib().orc_simple_rng_fill_uniform
    f.restype = None
    f(ctypes.c_uint64(seed), ctypes.c_float(scale), out.ctypes.data_as(ctypes.c_void_p),
      ctypes.c_int64(n))
    return out


def checkpoint_count(seq_len, c):
    return _call("orc_checkpoint_count", seq_len, c, restype=ctypes.c_int)


# ── single-chain rules (float32 or float64 by input dtype) ─────────────────
def titans_forward(k, v, q, alpha, theta, eta, m0, s0, error_clip=0.0, m_norm_max=F32_MAX):
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    m_states = np.zeros((s + 1, d, d), dt)
    s_states = np.zeros((s + 1, d, d), dt)
    y = np.zeros((s, d), dt)
    _call("orc_titans_forward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt),
          _c(eta, dt), _c(m0, dt), _c(s0, dt), m_states, s_states, y, s, d,
          float(error_clip), float(m_norm_max), real=real)
    return y, m_states, s_states


def delta_forward(k, v, q, alpha, theta, m0, error_clip=0.0, m_norm_max=F32_MAX):
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    m_states = np.zeros((s + 1, d, d), dt)
    y = np.zeros((s, d), dt)
    _call("orc_delta_forward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt),
          _c(m0, dt), m_states, y, s, d, float(error_clip), float(m_norm_max), real=real)
    return y, m_states


def titans_backward(k, v, q, alpha, theta, eta, m_states, s_states, d_y, error_clip=0.0,
                    t_lo=0, t_hi=None, d_m_seed=None, d_s_seed=None):
    """Full backward (defaults) or segment backward over [t_lo, t_hi) with a
    segment-local trajectory and seeds.  Returns dict of gradients; d_m/d_s are
    the state gradients flowing into token t_lo."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    t_hi = s if t_hi is None else t_hi
    g = {n: np.zeros((s, d), dt) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(s, dt) for n in ("d_alpha", "d_theta", "d_eta")})
    g["d_m"] = np.zeros((d, d), dt) if d_m_seed is None else _c(d_m_seed, dt).copy()
    g["d_s"] = np.zeros((d, d), dt) if d_s_seed is None else _c(d_s_seed, dt).copy()
    _call("orc_titans_backward_range" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt),
          _c(theta, dt), _c(eta, dt), _c(m_states, dt), _c(s_states, dt), _c(d_y, dt),
          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], g["d_m"], g["d_s"],
          t_lo, t_hi, d, float(error_clip), real=real)
    return g


def delta_backward(k, v, q, alpha, theta, m_states, d_y, error_clip=0.0,
                   t_lo=0, t_hi=None, d_m_seed=None):
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    t_hi = s if t_hi is None else t_hi
    g = {n: np.zeros((s, d), dt) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(s, dt) for n in ("d_alpha", "d_theta")})
    g["d_m"] = np.zeros((d, d), dt) if d_m_seed is None else _c(d_m_seed, dt).copy()
    _call("orc_delta_backward_range" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt),
          _c(theta, dt), _c(m_states, dt), _c(d_y, dt),
          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_m"],
          t_lo, t_hi, d, float(error_clip), real=real)
    return g


def chunkwise_forward(k, v, q, alpha, theta, eta, m0, s0, chunk_size, has_s=True,
                      error_clip=0.0, m_norm_max=F32_MAX):
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    nc = (s + chunk_size - 1) // chunk_size
    mc = np.zeros((nc + 1, d, d), dt)
    sc = np.zeros((nc + 1, d, d), dt)
    y = np.zeros((s, d), dt)
    eta = np.zeros(s, dt) if eta is None else eta
    s0 = np.zeros((d, d), dt) if s0 is None else s0
    _call("orc_chunkwise_forward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt),
          _c(theta, dt), _c(eta, dt), _c(m0, dt), _c(s0, dt), mc, sc, y, s, d, chunk_size,
          int(has_s), float(error_clip), float(m_norm_max), real=real)
    return y, mc, sc


def chunkwise_backward(k, v, q, alpha, theta, eta, mc, sc, d_y, chunk_size, has_s=True,
                       error_clip=0.0, m_norm_max=F32_MAX):
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    g = {n: np.zeros((s, d), dt) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(s, dt) for n in ("d_alpha", "d_theta", "d_eta")})
    g["d_m"] = np.zeros((d, d), dt)
    g["d_s"] = np.zeros((d, d), dt)
    eta = np.zeros(s, dt) if eta is None else eta
    sc = np.zeros_like(mc) if sc is None else sc
    _call("orc_chunkwise_backward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt),
          _c(theta, dt), _c(eta, dt), _c(mc, dt), _c(sc, dt), _c(d_y, dt),
          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], g["d_m"], g["d_s"],
          s, d, chunk_size, int(has_s), float(error_clip), float(m_norm_max), real=real)
    return g


# ── batched float32 entry points with the kernels' layout contract ─────────
def titans_forward_batch(k, v, q, alpha, theta, eta, m0, s0, error_clip=0.0, m_norm_max=F32_MAX):
    """k,v,q [B,s,d]; gates [B,s]; m0,s0 [B,d,d] -> y [B,s,d], m_states, s_states [B,s+1,d,d]."""
    f = np.float32
    B, s, d = k.shape
    ms = np.zeros((B, s + 1, d, d), f)
    ss = np.zeros((B, s + 1, d, d), f)
    y = np.zeros((B, s, d), f)
    _call("orc_titans_forward_batch_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(eta, f), _c(m0, f), _c(s0, f), ms, ss, y, s, d, B, s, d * d,
          float(error_clip), float(m_norm_max))
    return y, ms, ss


def delta_forward_batch(k, v, q, alpha, theta, m0, error_clip=0.0, m_norm_max=F32_MAX):
    f = np.float32
    B, s, d = k.shape
    ms = np.zeros((B, s + 1, d, d), f)
    y = np.zeros((B, s, d), f)
    _call("orc_delta_forward_batch_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(m0, f), ms, y, s, d, B, s, d * d, float(error_clip), float(m_norm_max))
    return y, ms


def titans_backward_batch(k, v, q, alpha, theta, eta, m_states, s_states, d_y, error_clip=0.0):
    f = np.float32
    B, s, d = k.shape
    g = {n: np.zeros((B, s, d), f) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros((B, s), f) for n in ("d_alpha", "d_theta", "d_eta")})
    g["d_m_initial"] = np.zeros((d, d), f)
    g["d_s_initial"] = np.zeros((d, d), f)
    _call("orc_titans_backward_batch_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(eta, f), _c(m_states, f), _c(s_states, f), _c(d_y, f),
          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
          g["d_m_initial"], g["d_s_initial"], s, d, B, float(error_clip))
    return g


def delta_backward_batch(k, v, q, alpha, theta, m_states, d_y, error_clip=0.0):
    f = np.float32
    B, s, d = k.shape
    g = {n: np.zeros((B, s, d), f) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros((B, s), f) for n in ("d_alpha", "d_theta")})
    g["d_m_initial"] = np.zeros((d, d), f)
    _call("orc_delta_backward_batch_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(m_states, f), _c(d_y, f), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"],
          g["d_m_initial"], s, d, B, float(error_clip))
    return g


def forward_ckpt(k, v, q, alpha, theta, eta, m0, s0, C, has_s=True, error_clip=0.0,
                 m_norm_max=F32_MAX):
    """One chain, float32.  Returns y [s,d], m_ckpt, s_ckpt [n_ckpt,d,d]."""
    f = np.float32
    s, d = k.shape
    n = checkpoint_count(s, C)
    mc = np.zeros((n, d, d), f)
    sc = np.zeros((n, d, d), f)
    y = np.zeros((s, d), f)
    eta = np.zeros(s, f) if eta is None else eta
    s0 = np.zeros((d, d), f) if s0 is None else s0
    _call("orc_forward_ckpt_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(eta, f), _c(m0, f), _c(s0, f), mc, sc, y, s, d, C, int(has_s),
          float(error_clip), float(m_norm_max))
    return y, mc, sc


def backward_ckpt(k, v, q, alpha, theta, eta, mc, sc, d_y, C, has_s=True, error_clip=0.0,
                  m_norm_max=F32_MAX):
    f = np.float32
    s, d = k.shape
    g = {n: np.zeros((s, d), f) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(s, f) for n in ("d_alpha", "d_theta", "d_eta")})
    g["d_m"] = np.zeros((d, d), f)
    g["d_s"] = np.zeros((d, d), f)
    eta = np.zeros(s, f) if eta is None else eta
    sc = np.zeros_like(mc) if sc is None else sc
    _call("orc_backward_ckpt_f32", _c(k, f), _c(v, f), _c(q, f), _c(alpha, f), _c(theta, f),
          _c(eta, f), _c(mc, f), _c(sc, f), _c(d_y, f),
          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], g["d_m"], g["d_s"],
          s, d, C, int(has_s), float(error_clip), float(m_norm_max))
    return g
