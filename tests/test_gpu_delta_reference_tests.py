"""The reference's Delta-rule CUDA tests (core/tests/test_cuda_delta.rs) through the GPU library with the
reference's recipes (rand_buf seeds, alpha = 0.05, theta = 0.01) and its absolute bounds, against the CPU oracle
(the Rust loops those tests restate are the oracle's, oracle/rules.inc).  The two "full pipeline" cases need the
model's projection stage and are covered by the level step (tests/test_gpu_memory_level.py)."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_abs, dev, host, zeros

pytestmark = pytest.mark.gpu
f32 = np.float32
rb = orc.simple_rng_uniform


def recipe(s, d, seeds):
    k, v, q = (rb(s * d, sd).reshape(s, d) for sd in seeds)
    return k, v, q, np.full(s, 0.05, f32), np.full(s, 0.01, f32)


def gpu_forward(k, v, q, al, th, m0):
    s, d = k.shape
    ms, y = zeros(s + 1, d, d), zeros(s, d)
    D.delta_forward_dd(dev(k), dev(v), dev(q), dev(al), dev(th), dev(m0), ms, y, s, d, 1, s, d * d, 0.0, orc.F32_MAX)
    torch.cuda.synchronize()
    return host(y), host(ms)


@pytest.mark.parametrize("s,d,seeds,m0_seed,tol", [
    (16, 8, (100, 200, 300), None, 1e-5),      # :116 test_cuda_delta_forward_matches_rust
    (1, 4, (800, 900, 1000), None, 1e-5),      # :303 test_cuda_delta_forward_seq_len_1
    (8, 8, (1100, 1200, 1300), 1400, 1e-5),    # :331 test_cuda_delta_forward_nonzero_initial
    (8, 16, (2900, 3000, 3100), None, 1e-4),   # :622 test_cuda_delta_forward_d16
    (4, 128, (5000, 5100, 5200), None, 1e-4),  # :650 test_cuda_delta_forward_large_d
])
def test_forward_recipes(s, d, seeds, m0_seed, tol):
    k, v, q, al, th = recipe(s, d, seeds)
    m0 = np.zeros((d, d), f32) if m0_seed is None else rb(d * d, m0_seed).reshape(d, d)
    y, ms = gpu_forward(k, v, q, al, th, m0)
    yo, mo = orc.delta_forward(k, v, q, al, th, m0)
    assert_abs("y", y, yo, tol)
    assert_abs("m_states", ms, mo, tol)
    assert np.linalg.norm(ms[-1]) > 1e-6


@pytest.mark.parametrize("s,d,seeds,dy_seed", [(12, 8, (400, 500, 600), 700),      # :174 backward_matches_rust
                                               (1, 4, (1600, 1700, 1800), 1900),   # :407 backward_seq_len_1
                                               (12, 8, (2000, 2100, 2200), 2300)])  # :550 backward_nonzero (recipe of its kind)
def test_backward_recipes(s, d, seeds, dy_seed):
    k, v, q, al, th = recipe(s, d, seeds)
    dy = rb(s * d, dy_seed).reshape(s, d)
    _, mo = orc.delta_forward(k, v, q, al, th, np.zeros((d, d), f32))
    want = orc.delta_backward(k, v, q, al, th, mo, dy)
    g = dict(d_k=zeros(s, d), d_v=zeros(s, d), d_q=zeros(s, d), d_alpha=zeros(s), d_theta=zeros(s), d_m=zeros(d, d))
    D.delta_backward_dd(dev(k), dev(v), dev(q), dev(al), dev(th), dev(mo), dev(dy), g["d_k"], g["d_v"], g["d_q"],
                        g["d_alpha"], g["d_theta"], g["d_m"], s, d, 1, 0.0)
    torch.cuda.synchronize()
    for n in g:
        assert_abs(n, host(g[n]), want[n], 1e-4)
    assert np.linalg.norm(host(g["d_k"])) > 0 and np.linalg.norm(host(g["d_m"])) > 0


def test_forward_deterministic():
    """:592 test_cuda_delta_forward_deterministic: two runs, equal bits."""
    k, v, q, al, th = recipe(12, 8, (2600, 2700, 2800))
    m0 = np.zeros((8, 8), f32)
    y1, m1 = gpu_forward(k, v, q, al, th, m0)
    y2, m2 = gpu_forward(k, v, q, al, th, m0)
    assert np.array_equal(y1, y2) and np.array_equal(m1, m2)
