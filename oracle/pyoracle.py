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


def hebbian_forward(k, v, q, alpha, m0, m_norm_max=F32_MAX, checkpoint_interval=0):
    """rust_hebbian_forward (core/src/dispatch.rs:1566-1601); with checkpoint_interval > 0 m_states holds
    M_0 and the states after every C-th token and the last one (hebbian_forward.cu:212-268)."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    n = s + 1 if checkpoint_interval <= 0 else checkpoint_count(s, checkpoint_interval)
    m_states = np.zeros((n, d, d), dt)
    y = np.zeros((s, d), dt)
    _call("orc_hebbian_forward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(m0, dt),
          m_states, y, s, d, float(m_norm_max), int(checkpoint_interval), real=real)
    return y, m_states


def hebbian_backward(k, v, q, alpha, m_states, d_y, t_lo=0, t_hi=None, d_m_seed=None):
    """rust_hebbian_backward (core/src/dispatch.rs:1604-1660); segment form as in delta_backward."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    t_hi = s if t_hi is None else t_hi
    g = {n: np.zeros((s, d), dt) for n in ("d_k", "d_v", "d_q")}
    g["d_alpha"] = np.zeros(s, dt)
    g["d_m"] = np.zeros((d, d), dt) if d_m_seed is None else _c(d_m_seed, dt).copy()
    _call("orc_hebbian_backward_range" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt),
          _c(m_states, dt), _c(d_y, dt), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_m"],
          t_lo, t_hi, d, real=real)
    return g


def mlp_state_size(d, dh):
    """packed [W1 (dh x d) | b1 (dh) | W2 (d x dh) | b2 (d)]"""
    return 2 * dh * d + dh + d


def titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act=0, m_norm_max=F32_MAX, actp_fix=None):
    """core/kernels/titans_mlp_forward.cu:115-330, one chain.  actp_fix [s, dh]: values used in place of
    act'(pre) in the inner gradient (for tests that freeze them)."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    n = mlp_state_size(d, dh)
    m_states, s_states, y = np.zeros((s + 1, n), dt), np.zeros((s + 1, n), dt), np.zeros((s, d), dt)
    _call("orc_titans_mlp_forward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt), _c(eta, dt),
          _c(m0, dt), _c(s0, dt), m_states, s_states, y, s, d, int(dh), int(act), float(m_norm_max),
          None if actp_fix is None else _c(actp_fix, dt), real=real)
    return y, m_states, s_states


def titans_mlp_backward(k, v, q, alpha, theta, eta, m_states, s_states, d_y, dh, act=0):
    """core/kernels/titans_mlp_backward.cu:100-560, one chain; d_m / d_s: gradients of the initial state."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    n = mlp_state_size(d, dh)
    g = {nm: np.zeros((s, d), dt) for nm in ("d_k", "d_v", "d_q")}
    g.update({nm: np.zeros(s, dt) for nm in ("d_alpha", "d_theta", "d_eta")})
    g["d_m"], g["d_s"] = np.zeros(n, dt), np.zeros(n, dt)
    _call("orc_titans_mlp_backward" + sfx, _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt), _c(eta, dt),
          _c(m_states, dt), _c(s_states, dt), _c(d_y, dt), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"],
          g["d_eta"], g["d_m"], g["d_s"], s, d, int(dh), int(act), real=real)
    return g


def miras_mlp_forward(mode, k, v, q, alpha, theta, w1, w2, dh, p1, p2, lambda_2, lq_q=2.0, boundary=None,
                      slope_fix=None):
    """MONETA (mode 0: p1 = lp_p, p2 = sign_sharpness) / YAAD (mode 1: p1 = huber_delta, p2 = lambda_local,
    boundary = (w1_boundary, w2_boundary)) forward, core/kernels/moneta_forward.cu:100-430, one chain."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    w1s, w2s, y = np.zeros((s + 1, dh, d), dt), np.zeros((s + 1, d, dh), dt), np.zeros((s, d), dt)
    b1, b2 = (None, None) if boundary is None else (_c(boundary[0], dt), _c(boundary[1], dt))
    _call("orc_miras_mlp_forward" + sfx, int(mode), _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt),
          _c(w1, dt), _c(w2, dt), b1, b2, w1s, w2s, y, s, d, int(dh), float(p1), float(p2), float(lambda_2),
          float(lq_q), None if slope_fix is None else _c(slope_fix, dt), real=real)
    return y, w1s, w2s


def miras_mlp_backward(mode, k, v, q, alpha, theta, w1s, w2s, d_y, dh, p1, p2, lambda_2, boundary=None,
                       d_k0=None, d_v0=None):
    """core/kernels/moneta_backward.cu:96-520 (q = 2); d_k / d_v start from d_k0 / d_v0 (accumulate contract)."""
    dt = k.dtype
    sfx, real = _sfx(dt)
    s, d = k.shape
    g = dict(d_k=np.zeros((s, d), dt) if d_k0 is None else _c(d_k0, dt).copy(),
             d_v=np.zeros((s, d), dt) if d_v0 is None else _c(d_v0, dt).copy(), d_q=np.zeros((s, d), dt),
             d_alpha=np.zeros(s, dt), d_theta=np.zeros(s, dt), d_w1=np.zeros((dh, d), dt), d_w2=np.zeros((d, dh), dt))
    b1, b2 = (None, None) if boundary is None else (_c(boundary[0], dt), _c(boundary[1], dt))
    _call("orc_miras_mlp_backward" + sfx, int(mode), _c(k, dt), _c(v, dt), _c(q, dt), _c(alpha, dt), _c(theta, dt),
          _c(w1s, dt), _c(w2s, dt), b1, b2, _c(d_y, dt), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"],
          g["d_w1"], g["d_w2"], s, d, int(dh), float(p1), float(p2), float(lambda_2), real=real)
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


# ── pieces around the memory rules (nlh_oracle_layer.c) ────────────────────
def adamw_step(params, grads, m, v, lr, beta1, beta2, eps, bc1_inv, bc2_inv, weight_decay):
    """In place on float32 arrays (core/src/adamw.rs:102-126)."""
    f = lib().orc_adamw_step
    f.restype = None
    for a in (params, grads, m, v):
        assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    f(p(params), p(grads), p(m), p(v), ctypes.c_int64(params.size), *[ctypes.c_float(x) for x in
      (lr, beta1, beta2, eps, bc1_inv, bc2_inv, weight_decay)])


def grad_norm_clip(grads, max_grad_norm):
    """-> (norm, scale) over a list of float32 arrays (core/src/adamw.rs:203-262)."""
    n = len(grads)
    ptrs = (ctypes.c_void_p * n)(*[g.ctypes.data for g in grads])
    sizes = (ctypes.c_int64 * n)(*[g.size for g in grads])
    scale = ctypes.c_float(0)
    f = lib().orc_grad_norm_clip
    f.restype = ctypes.c_float
    norm = f(ptrs, sizes, ctypes.c_int(n), ctypes.c_float(max_grad_norm), ctypes.byref(scale))
    return float(norm), float(scale.value)


def pulse(step, chunk_sizes, seq_len=0):
    k = len(chunk_sizes)
    cs = (ctypes.c_int64 * k)(*chunk_sizes)
    out = (ctypes.c_int * k)()
    f = lib().orc_pulse
    f.restype = None
    f(ctypes.c_int64(step), cs, ctypes.c_int(k), ctypes.c_int64(seq_len), out)
    return [bool(x) for x in out]


def gate_compute(k, v, w, bias, activation):
    f = np.float32
    n, d = k.shape
    out = np.zeros(n, f)
    _call("orc_gate_compute", _c(k, f), _c(v, f), _c(w, f), float(bias), out, n, d, int(activation))
    return out


def gate_backward(d_alpha, alpha, d_theta, theta, d_eta, eta, k, v, has_theta=True, has_eta=True):
    f = np.float32
    T, D = k.shape
    o = {n: np.zeros(2 * D, f) for n in ("d_w_alpha", "d_w_theta", "d_w_eta")}
    o.update({n: np.zeros(1, f) for n in ("d_b_alpha", "d_b_theta", "d_b_eta")})
    z = np.zeros(T, f)
    _call("orc_gate_backward", _c(d_alpha, f), _c(alpha, f),
          _c(d_theta if has_theta else z, f), _c(theta if has_theta else z, f),
          _c(d_eta if has_eta else z, f), _c(eta if has_eta else z, f), _c(k, f), _c(v, f),
          o["d_w_alpha"], o["d_b_alpha"], o["d_w_theta"], o["d_b_theta"], o["d_w_eta"], o["d_b_eta"],
          T, D, int(has_theta), int(has_eta))
    return o


def l2_normalize_rows(x, eps=1e-8):
    f = np.float32
    x = _c(x, f).copy()
    n, d = x.shape
    norms = np.zeros(n, f)
    _call("orc_l2_normalize_rows", x, norms, n, d, float(eps))
    return x, norms


def l2_normalize_backward(d_out, x_norm, norms, eps=1e-8):
    f = np.float32
    n, d = d_out.shape
    d_in = np.zeros((n, d), f)
    _call("orc_l2_normalize_backward", _c(d_out, f), _c(x_norm, f), _c(norms, f), d_in, n, d, float(eps))
    return d_in


def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.zeros(x.shape, np.uint16)
    fn = lib().orc_f32_to_bf16
    fn.restype = None
    fn(x.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(x.size))
    return out


def bf16_to_f32(x):
    x = _c(x, np.uint16)
    out = np.zeros(x.shape, np.float32)
    fn = lib().orc_bf16_to_f32
    fn.restype = None
    fn(x.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(x.size))
    return out


def swa_forward(q, k, v, window, num_heads, n_persistent=0):
    """q,k,v uint16 (bf16 bits) [B, s, H*hd] -> out uint16, attn_weights uint16 [B,H,s,np+window]."""
    B, s, td = q.shape
    hd = td // num_heads
    out = np.zeros((B, s, td), np.uint16)
    aw = np.zeros((B, num_heads, s, n_persistent + window), np.uint16)
    _call("orc_swa_forward", _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16), out, aw,
          s, num_heads, hd, window, B, n_persistent)
    return out, aw


def swa_backward(q, k, v, aw, d_out, window, num_heads, n_persistent=0):
    B, s, td = q.shape
    hd = td // num_heads
    f = np.float32
    dq, dk, dv = np.zeros((B, s, td), f), np.zeros((B, s, td), f), np.zeros((B, s, td), f)
    _call("orc_swa_backward", _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16), _c(aw, np.uint16),
          _c(d_out, f), dq, dk, dv, s, num_heads, hd, window, B, n_persistent)
    return dq, dk, dv


# ── HOPE self-referential memory (selfref.inc) ─────────────────────────────
def selfref_forward(mems, embedded, chunk_size, self_gen=True):
    """mems [6,d,d] (k,v,q,eta,alpha,mem), embedded [s,d]; float32 or float64.
    Returns y [s,d], final memories [6,d,d] and the cache dict for the backward."""
    dt = embedded.dtype
    sfx, real = _sfx(dt)
    s, d = embedded.shape
    nc = (s + chunk_size - 1) // chunk_size
    m = _c(mems, dt).copy()
    c = dict(k=np.zeros((s, d), dt), v=np.zeros((s, d), dt), q=np.zeros((s, d), dt),
             alpha=np.zeros(s, dt), theta=np.zeros(s, dt), alpha_mean=np.zeros(s, dt),
             eta_mean=np.zeros(s, dt), traj=np.zeros((6, s + 1, d, d), dt),
             frozen=np.zeros((nc, 6, d, d), dt), v_hat=np.zeros((6, s, d), dt),
             embedded=_c(embedded, dt), chunk_size=chunk_size, self_gen=self_gen)
    y = np.zeros((s, d), dt)
    _call("orc_selfref_forward" + sfx, m, c["embedded"], y, c["k"], c["v"], c["q"], c["alpha"],
          c["theta"], c["alpha_mean"], c["eta_mean"], c["traj"], c["frozen"], c["v_hat"],
          s, d, chunk_size, int(self_gen), real=real)
    return y, m, c


def selfref_backward(cache, d_y):
    dt = d_y.dtype
    sfx, real = _sfx(dt)
    s, d = d_y.shape
    c = cache
    d_emb = np.zeros((s, d), dt)
    d_mems = np.zeros((6, d, d), dt)
    _call("orc_selfref_backward" + sfx, c["embedded"], _c(d_y, dt), c["k"], c["v"], c["q"], c["alpha"],
          c["theta"], c["alpha_mean"], c["eta_mean"], c["traj"], c["frozen"], c["v_hat"],
          d_emb, d_mems, s, d, c["chunk_size"], int(c["self_gen"]), real=real)
    return d_emb, d_mems


# ── compositions the reference ships as single kernels ─────────────────────
def error_subtract_clip(pred, v, error_clip):
    """core/kernels/error_subtract_clip.cu:18-70: e = pred - v per row; rows with |e|_2 > clip
    are scaled to clip (float32 arithmetic, clip <= 0: off)."""
    f = np.float32
    e = (_c(pred, f) - _c(v, f)).astype(f)
    if error_clip > 0:
        for r in range(e.shape[0]):
            n = np.sqrt(np.sum(e[r] * e[r], dtype=f), dtype=f)
            if n > f(error_clip):
                e[r] = e[r] * (f(error_clip) / n)
    return e


def fused_forward(k, v, q, w_alpha, b_alpha, w_theta, b_theta, w_eta, b_eta, alpha_lim, theta_lim, m0, s0,
                  error_clip=0.0, m_norm_max=F32_MAX):
    """One chain of core/kernels/titans_forward.cu:569-760 (w_eta None: dgd_forward.cu's fused form):
    normalise k, q rows (norm floor 1e-8), gates from normalised k and raw v, clamp alpha / theta,
    then the exact recurrence.  Returns a dict of everything the kernel writes."""
    f = np.float32
    kn, knorm = l2_normalize_rows(k)
    qn, qnorm = l2_normalize_rows(q)
    alpha = np.clip(gate_compute(kn, v, w_alpha, b_alpha, 0), f(alpha_lim[0]), f(alpha_lim[1])).astype(f)
    theta = np.clip(gate_compute(kn, v, w_theta, b_theta, 1), f(theta_lim[0]), f(theta_lim[1])).astype(f)
    out = dict(k=kn, q=qn, k_norms=knorm, q_norms=qnorm, alpha=alpha, theta=theta)
    if w_eta is not None:
        eta = gate_compute(kn, v, w_eta, b_eta, 0)
        y, ms, ss = titans_forward(kn, _c(v, f), qn, alpha, theta, eta, m0, s0, error_clip, m_norm_max)
        out.update(eta=eta, y=y, m_states=ms, s_states=ss)
    else:
        y, ms = delta_forward(kn, _c(v, f), qn, alpha, theta, m0, error_clip, F32_MAX)  # DGD: no projection
        out.update(y=y, m_states=ms)
    return out


def swa_single_token(q, k_cache, v_cache, window, num_heads, n_persistent=0):
    """core/kernels/swa_forward.cu:187-291: the full kernel's output row for query position
    cache_len-1 (q uint16 [H*hd], caches uint16 [cache_len, H*hd])."""
    cache_len, td = k_cache.shape
    qf = np.zeros((1, cache_len, td), np.uint16)
    qf[0, -1] = q
    out, _ = swa_forward(qf, k_cache[None], v_cache[None], window, num_heads, n_persistent)
    return out[0, -1]


# ── phase-2 kernels of the split chunkwise path (errors supplied) ───────────
def _project(m, m_norm_max):
    f = np.float32
    if 0 < m_norm_max < 1e30:
        n = np.sqrt(np.sum(m * m, dtype=f), dtype=f)
        if n > f(m_norm_max):
            m = (m * (f(m_norm_max) / n)).astype(f)
    return m


def phase2_forward(k, q, alpha, theta, eta, errors, m, s, m_norm_max=F32_MAX):
    """One chain, one chunk (core/kernels/titans_phase2_forward.cu:107-139; eta None: the Delta
    kernel): S' = eta S - theta e k^T, M' = (1-alpha) M + S', project, y = M' q.
    Returns y [C,d], final M, final S."""
    f = np.float32
    m, s = _c(m, f).copy(), (None if eta is None else _c(s, f).copy())
    ys = []
    for t in range(k.shape[0]):
        upd = (-f(theta[t]) * np.outer(errors[t], k[t])).astype(f)
        if eta is None:
            m = ((f(1) - f(alpha[t])) * m + upd).astype(f)
        else:
            s = (f(eta[t]) * s + upd).astype(f)
            m = ((f(1) - f(alpha[t])) * m + s).astype(f)
        m = _project(m, m_norm_max)
        ys.append((m @ q[t]).astype(f))
    return np.array(ys, f), m, s


def phase2_backward(k, q, alpha, theta, eta, errors, m0, s0, d_y, d_m, d_s, m_norm_max=F32_MAX):
    """One chain, one chunk (core/kernels/titans_phase2_backward.cu:88-285; eta None: Delta).
    d_m / d_s: adjoints carried in from later chunks.  Returns the per-token gradients, the
    updated d_m / d_s and d_m0 (the error path onto the chunk-start matrix)."""
    f = np.float64   # float64 yardstick: the kernel's float32 sums are compared at 1e-4
    C, d = k.shape
    has_s = eta is not None
    ms, ss = [np.asarray(m0, f)], [np.asarray(s0, f) if has_s else None]
    for t in range(C):
        upd = -theta[t] * np.outer(errors[t], k[t])
        if has_s:
            ss.append(eta[t] * ss[-1] + upd)
            mn = (1 - alpha[t]) * ms[-1] + ss[-1]
        else:
            mn = (1 - alpha[t]) * ms[-1] + upd
        if 0 < m_norm_max < 1e30:
            n = np.linalg.norm(mn)
            if n > m_norm_max:
                mn = mn * (m_norm_max / n)
        ms.append(mn)
    dm, ds = np.asarray(d_m, f).copy(), (np.asarray(d_s, f).copy() if has_s else None)
    dm0 = np.zeros((d, d), f)
    g = {n: np.zeros((C, d), f) for n in ("d_k", "d_v", "d_q")}
    g.update({n: np.zeros(C, f) for n in ("d_alpha", "d_theta", "d_eta")})
    for t in range(C - 1, -1, -1):
        dm += np.outer(d_y[t], q[t])
        g["d_q"][t] = ms[t + 1].T @ d_y[t]
        if has_s:
            ds += dm
            G = ds
        else:
            G = dm
        g["d_alpha"][t] = -(ms[t] * dm).sum()
        if has_s:
            g["d_eta"][t] = (ss[t] * ds).sum()
        g["d_theta"][t] = -(np.outer(errors[t], k[t]) * G).sum()
        d_err = -theta[t] * (G @ k[t])
        g["d_k"][t] = -theta[t] * (G.T @ errors[t]) + ms[0].T @ d_err
        g["d_v"][t] = -d_err
        dm0 += np.outer(d_err, k[t])
        dm = (1 - alpha[t]) * dm
        if has_s:
            ds = eta[t] * ds
    g.update(d_m=dm + dm0, d_s=ds, d_m0=dm0)
    return g
