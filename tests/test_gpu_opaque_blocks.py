"""The opaque VJP blocks of the tape through the C ABI (nlh_opaque_backward) against the CPU
restatement of the reference's adapters (oracle/blocks.py, pinned by finite differences): saved buffers
in the reference's order and newest recording format, results ADDED into non-zero d_inputs (the tape's
accumulate, tape.rs:839-866).  Tolerance: relative 1e-4 (fp32 path; the attention block 2e-2: its
operands travel as bf16, dispatch.rs:463-490).  The host-side refusals need no GPU."""
import numpy as np
import pytest

from nl_hecate_amd import opaque as OP
from oracle import blocks as B
from oracle import pyoracle as orc
from tests.gpu_util import assert_close

f32 = np.float32


def _block_case(kind, s, d, seed, alpha_lim=(0.0, 1.0), theta_lim=(0.0, B.F32_MAX), extra_flat=0):
    rs = np.random.default_rng(seed)
    p = B.init_params(d, seed)
    emb = (rs.standard_normal((s, d)) * 0.7).astype(f32)
    m0 = (rs.standard_normal((d, d)) * 0.2).astype(f32)
    s0 = (rs.standard_normal((d, d)) * 0.1).astype(f32) if kind == "titans" else None
    y, c = B.rule_step(kind, p, emb, m0, s0, alpha_lim, theta_lim)
    d_y = rs.standard_normal((s, d)).astype(f32)
    grads, d_emb = B.rule_step_backward(kind, p, c, d_y, emb, alpha_lim, theta_lim)
    saved = B.saved_buffers(kind, p, c, emb, alpha_lim, theta_lim)
    if extra_flat:   # a flat buffer with learned-frequency fields behind the mandatory ones
        saved[1] = np.concatenate([saved[1], rs.standard_normal(extra_flat).astype(f32)])
    flat_len = saved[1].size
    # the tape's buffers already hold gradients from other consumers
    start = [rs.standard_normal(s * d).astype(f32), rs.standard_normal(flat_len).astype(f32)]
    d_inputs = [a.copy() for a in start]
    OP.opaque_backward(OP.TITANS_LMM if kind == "titans" else OP.DELTA_RULE, [d_y.reshape(-1)], saved, d_inputs)
    assert_close(f"{kind} d_embedded", d_inputs[0] - start[0], d_emb.reshape(-1))
    got = B.params_from_flat(d_inputs[1] - start[1], d)
    for n in B.FIELDS:
        want = np.asarray(grads[n]).reshape(-1)
        if np.any(want):
            assert_close(f"{kind} d_{n}", np.asarray(got[n]).reshape(-1), want)
        else:
            assert not np.any(got[n]), f"{kind} d_{n} must stay untouched"
    if extra_flat:
        np.testing.assert_array_equal(d_inputs[1][-extra_flat:], start[1][-extra_flat:])


@pytest.mark.gpu
@pytest.mark.parametrize("kind,s,d", [("delta", 12, 8), ("titans", 12, 8), ("delta", 40, 32), ("titans", 33, 16),
                                      ("titans", 70, 64)])
def test_rule_blocks_add_their_gradients_into_the_tape_buffers(kind, s, d):
    _block_case(kind, s, d, seed=100 + s + d)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["delta", "titans"])
def test_rule_blocks_with_active_clamps_and_a_longer_flat_buffer(kind):
    """Clamp bounds inside the gates' range: some tokens sit on a bound (masked by the rule's own
    straight-through convention), others do not."""
    _block_case(kind, 24, 16, seed=7, alpha_lim=(0.1, 0.3), theta_lim=(0.05, 0.4), extra_flat=17)


@pytest.mark.gpu
def test_dgd_block():
    s, d = 20, 16
    rs = np.random.default_rng(3)
    k, v, q, dy = (rs.standard_normal((s, d)).astype(f32) for _ in range(4))
    k /= np.linalg.norm(k, axis=1, keepdims=True)
    al, th = (1 / (1 + np.exp(-rs.standard_normal(s)))).astype(f32), (0.3 / (1 + np.exp(-rs.standard_normal(s)))).astype(f32)
    m0 = (rs.standard_normal((d, d)) * 0.2).astype(f32)
    y, ms = orc.delta_forward(k, v, q, al, th, m0)
    g = orc.delta_backward(k, v, q, al, th, ms, dy)
    saved = [np.array([s, d, 0.0], f32), k.reshape(-1), v.reshape(-1), q.reshape(-1), al, th, ms.reshape(-1)]
    start = [rs.standard_normal(n).astype(f32) for n in (s * d, s * d, s * d, s, s, d * d)]
    d_inputs = [a.copy() for a in start]
    OP.opaque_backward(OP.DGD, [dy.reshape(-1)], saved, d_inputs)
    for i, n in enumerate(("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_m")):
        assert_close(n, d_inputs[i] - start[i], g[n].reshape(-1))


@pytest.mark.gpu
def test_swa_block():
    s, nh, hd, ws = 48, 2, 16, 8
    rs = np.random.default_rng(5)
    q, k, v, do = (rs.standard_normal((1, s, nh * hd)).astype(f32) for _ in range(4))
    bits = lambda a: orc.f32_to_bf16(a)
    out, aw = orc.swa_forward(bits(q), bits(k), bits(v), ws, nh, 0)
    dq, dk, dv = orc.swa_backward(bits(q), bits(k), bits(v), aw, do, ws, nh, 0)
    saved = [np.array([s, nh, hd, ws], f32), q.reshape(-1), k.reshape(-1), v.reshape(-1),
             orc.bf16_to_f32(aw).reshape(-1).astype(f32)]
    start = [rs.standard_normal(s * nh * hd).astype(f32) for _ in range(3)]
    d_inputs = [a.copy() for a in start]
    OP.opaque_backward(OP.SWA, [do.reshape(-1)], saved, d_inputs)
    for i, (n, want) in enumerate((("d_q", dq), ("d_k", dk), ("d_v", dv))):
        assert_close(n, d_inputs[i] - start[i], np.asarray(want).reshape(-1), 2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("key", [OP.FROZEN_DELTA_RULE, OP.FROZEN_TITANS_LMM])
def test_frozen_read_block(key):
    s, d = 30, 24
    rs = np.random.default_rng(8)
    m = rs.standard_normal((d, d)).astype(f32)
    dy = rs.standard_normal((s, d)).astype(f32)
    start = rs.standard_normal(s * d).astype(f32)
    d_inputs = [start.copy()]
    OP.opaque_backward(key, [dy.reshape(-1)], [np.array([s, d], f32), m.reshape(-1)], d_inputs)
    assert_close("d_q", d_inputs[0] - start, B.frozen_read_backward(m, dy).reshape(-1))


def test_unsupported_configurations_and_bad_layouts_are_refused_with_a_message():
    s, d = 4, 8
    p = B.init_params(d, 1)
    emb = np.zeros((s, d), f32)
    y, c = B.rule_step("delta", p, emb)
    saved = B.saved_buffers("delta", p, c, emb)
    d_in = [np.zeros(s * d, f32), np.zeros(saved[1].size, f32)]
    dy = [np.zeros(s * d, f32)]
    bad = [a.copy() for a in saved]
    bad[0][6] = 1.0                       # random-Fourier feature map
    with pytest.raises(OP.OpaqueBlockError, match="identity feature map"):
        OP.opaque_backward(OP.DELTA_RULE, dy, bad, d_in)
    bad = [a.copy() for a in saved]
    bad[0][2] = 1.0                       # L1 attentional bias
    with pytest.raises(OP.OpaqueBlockError, match="L2 bias"):
        OP.opaque_backward(OP.DELTA_RULE, dy, bad, d_in)
    with pytest.raises(OP.OpaqueBlockError, match="m_states"):
        OP.opaque_backward(OP.DELTA_RULE, dy, saved[:3] + [saved[3][:-1]] + saved[4:], d_in)
    with pytest.raises(OP.OpaqueBlockError, match="older recording format"):
        OP.opaque_backward(OP.DELTA_RULE, dy, [saved[0][:7].copy()] + saved[1:], d_in)
    with pytest.raises(OP.OpaqueBlockError, match="no GPU adapter"):
        OP.opaque_backward(3, dy, saved, d_in)       # Moneta
    ys, cs = B.rule_step("titans", p, emb)
    st = B.saved_buffers("titans", p, cs, emb)
    st[0][4] = 2.0                        # DeltaMomentum
    with pytest.raises(OP.OpaqueBlockError, match="EMA momentum"):
        OP.opaque_backward(OP.TITANS_LMM, dy, st, d_in)
    assert not np.any(d_in[0]) and not np.any(d_in[1]), "a refused call writes nothing"
