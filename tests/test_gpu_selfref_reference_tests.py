"""The reference's own test module of the chunkwise self-referential step (core/src/chunkwise_self_ref.rs:622-1085),
run through the GPU library at the reference's size d = 4 with the reference's input recipes (identity-scaled
memories, a ramp as the input).  `self_ref_step`, the reference's sequential form, is the chunkwise rule at C = 1
(its first two tests assert exactly that), so the CPU oracle at C = 1 stands for it."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import selfref as SR
from oracle import pyoracle as orc
from tests.gpu_util import dev, host

pytestmark = pytest.mark.gpu
f32 = np.float32
D = 4


def make_state(scale, m_mem=None, **over):
    """make_state / make_m_mem (:628-644): [6, d, d] = m_k, m_v, m_q, m_eta, m_alpha scaled identities, m_mem."""
    mems = np.zeros((6, D, D), f32)
    for c in range(5):
        mems[c] = np.eye(D, dtype=f32) * scale
    mems[5] = np.eye(D, dtype=f32) * (scale if m_mem is None else m_mem)
    for name, val in over.items():
        mems[SR.COMPONENTS.index(name)] = np.eye(D, dtype=f32) * val
    return mems


def make_embedded(seq_len):
    """:646-648"""
    return (np.arange(seq_len * D, dtype=f32) * f32(0.1) + f32(0.05)).reshape(seq_len, D)


def gpu_step(mems, emb, C, sg):
    m = dev(mems[None].copy())
    y, cache = SR.chunkwise_self_ref_step(m, dev(emb[None]), C, sg)
    torch.cuda.synchronize()
    return host(y)[0], host(m)[0], cache


def gpu_backward(cache, d_y):
    de, dm = SR.chunkwise_self_ref_step_backward(cache, dev(d_y[None]))
    torch.cuda.synchronize()
    return host(de)[0], host(dm)[0]


def sequential(mems, emb, sg):
    y, mf, _ = orc.selfref_forward(mems.copy(), emb, 1, sg)
    return y, mf


@pytest.mark.parametrize("sg", [False, True])
def test_c1_matches_sequential(sg):
    """:660-716 test_c1_matches_sequential, test_c1_self_gen_matches_sequential"""
    mems, emb = make_state(0.1), make_embedded(4)
    y_seq, m_seq = sequential(mems, emb, sg)
    y, m, _ = gpu_step(mems, emb, 1, sg)
    assert np.abs(y - y_seq).max() < 1e-5 * max(1.0, np.abs(y_seq).max())
    assert np.abs(m - m_seq.reshape(m.shape)).max() < 1e-5 * max(1.0, np.abs(m_seq).max())


def test_c2_and_c4_forward_finite():
    """:718-743 test_c2_forward_finite, test_c4_forward_finite (7 tokens: a remainder chunk)"""
    y, _, cache = gpu_step(make_state(0.1), make_embedded(4), 2, False)
    assert np.isfinite(y).all() and cache.num_chunks == 2 and cache.chunk_size == 2
    y, _, cache = gpu_step(make_state(0.1), make_embedded(7), 4, False)
    assert np.isfinite(y).all() and cache.num_chunks == 2


def test_backward_shapes_and_finite():
    """:746-782 test_backward_shapes, test_backward_finite"""
    y, _, cache = gpu_step(make_state(0.1), make_embedded(4), 2, False)
    d_emb, d_mems = gpu_backward(cache, y)
    assert d_emb.shape == (4, D) and d_mems.shape == (6, D, D)
    assert np.isfinite(d_emb).all() and np.isfinite(d_mems).all()


def test_backward_nonzero():
    """:784-805"""
    y, _, cache = gpu_step(make_state(0.1, m_eta=0.5, m_alpha=0.5), make_embedded(4), 2, False)
    d_emb, d_mems = gpu_backward(cache, y)
    assert (d_emb ** 2).sum() > 1e-10
    assert (d_mems[0] ** 2).sum() > 0.0 and (d_mems[5] ** 2).sum() > 0.0


def _loss(y):
    return float((y.astype(np.float64) ** 2).sum() / 2.0)


@pytest.mark.parametrize("C", [1, 2])
def test_fd_check_embedded(C):
    """:809-843 test_c1_fd_check_embedded and :880-916 test_c2_fd_check_embedded: forward differences of the
    float32 forward, eps 1e-3, relative 5 % on the entries above 1e-4 (the reference's own bar)."""
    seq_len, eps = (2 if C == 1 else 4), f32(1e-3)
    mems, emb = make_state(0.1), make_embedded(seq_len)
    y, _, cache = gpu_step(mems, emb, C, False)
    d_emb, _ = gpu_backward(cache, y)
    loss0, worst = _loss(y), 0.0
    for idx in range(emb.size):
        pert = emb.copy()
        pert.reshape(-1)[idx] += eps
        fd = (_loss(gpu_step(mems, pert, C, False)[0]) - loss0) / float(eps)
        ana = float(d_emb.reshape(-1)[idx])
        if abs(ana) > 1e-4:
            worst = max(worst, abs(fd - ana) / max(abs(fd), abs(ana), 1e-8))
    assert worst < 0.05, worst


def test_c1_fd_check_initial_mk():
    """:845-878: the gradient w.r.t. the initial M_k."""
    seq_len, eps = 2, f32(1e-3)
    mems, emb = make_state(0.1), make_embedded(seq_len)
    y, _, cache = gpu_step(mems, emb, 1, False)
    _, d_mems = gpu_backward(cache, y)
    loss0, worst = _loss(y), 0.0
    for idx in range(D * D):
        pert = mems.copy()
        pert[0].reshape(-1)[idx] += eps
        fd = (_loss(gpu_step(pert, emb, 1, False)[0]) - loss0) / float(eps)
        ana = float(d_mems[0].reshape(-1)[idx])
        if abs(ana) > 1e-4:
            worst = max(worst, abs(fd - ana) / max(abs(fd), abs(ana), 1e-8))
    assert worst < 0.05, worst


def test_c2_approx_bounded_and_quality_degrades_with_c():
    """:918-971 test_c2_approx_bounded, test_quality_degrades_with_c"""
    mems, emb = make_state(0.1), make_embedded(4)
    y_seq, _ = sequential(mems, emb, False)
    y_c2 = gpu_step(mems, emb, 2, False)[0]
    assert np.abs(y_seq - y_c2).sum() / max(np.abs(y_seq).sum(), 1e-8) < 0.5
    emb = make_embedded(8)
    y_ref, _ = sequential(mems, emb, False)
    diff2 = np.abs(y_ref - gpu_step(mems, emb, 2, False)[0]).sum()
    diff4 = np.abs(y_ref - gpu_step(mems, emb, 4, False)[0]).sum()
    assert diff2 <= diff4 + 1e-6


def test_self_gen_uses_frozen_snapshot():
    """:973-1014.  The library's cache does not hold the self-generated targets; what the test establishes —
    both tokens of a chunk see the chunk-start memories — is checked on what they determine: the snapshot is
    the initial state, and the memories after the chunk are those of the oracle, whose targets are F v_t with
    the frozen F (oracle/selfref.inc), not those of the per-token rule."""
    mems, emb = make_state(0.2, m_k=0.3, m_eta=1.0, m_alpha=1.0), make_embedded(2)
    y, m, cache = gpu_step(mems, emb, 2, True)
    assert cache.num_chunks == 1
    assert np.array_equal(host(cache.frozen_snapshots)[0, 0].reshape(6, D, D), mems)
    _, m_frozen, _ = orc.selfref_forward(mems.copy(), emb, 2, True)
    _, m_current = sequential(mems, emb, True)
    assert np.abs(m - m_frozen.reshape(m.shape)).max() < 1e-5 * np.abs(m_frozen).max()
    assert np.abs(m_frozen - m_current).max() > 1e-4, "the two target choices must differ for the test to mean anything"


def test_outer_loop_convergence():
    """:1016-1057: 100 gradient steps on the initial memories, C = 2, lr 0.01: the loss must not grow by 10 %."""
    mems, emb, lr = make_state(0.1), make_embedded(4), f32(0.01)
    first = last = None
    for step in range(100):
        y, _, cache = gpu_step(mems, emb, 2, False)
        last = _loss(y)
        first = last if step == 0 else first
        _, d_mems = gpu_backward(cache, y)
        mems = (mems - lr * d_mems).astype(f32)
    assert last <= first * 1.1, (first, last)


def test_remainder_chunk():
    """:1059-1083"""
    y, _, cache = gpu_step(make_state(0.1), make_embedded(7), 4, False)
    assert y.shape == (7, D) and cache.num_chunks == 2 and np.isfinite(y).all()
    d_emb, d_mems = gpu_backward(cache, y)
    assert d_emb.shape == (7, D) and np.isfinite(d_emb).all() and np.isfinite(d_mems[0]).all()
