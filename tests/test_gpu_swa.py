"""GPU parity of sliding-window attention (bf16 storage, f32 math) against the
CPU oracle.  bf16 path: relative 2e-2; with identical stored weights the
backward agrees to fp32 round-off (1e-4).  The reference's own bounds are
absolute 1e-2 forward / 5e-2 backward (core/tests/test_cuda_swa.rs:100,325)."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, zeros, REL_TOL_BF16

pytestmark = pytest.mark.gpu


def _case(B, s, H, hd, seed):
    r = np.random.default_rng(seed)
    q, k, v = (orc.f32_to_bf16(r.standard_normal((B, s, H * hd)).astype(np.float32)) for _ in range(3))
    go = r.standard_normal((B, s, H * hd)).astype(np.float32)
    return q, k, v, go


def _u16(a):
    return torch.from_numpy(a.view(np.int16)).cuda().view(torch.uint16)


def gpu_forward(q, k, v, ws, H, npers):
    B, s, td = q.shape
    out = torch.zeros(B, s, td, dtype=torch.uint16, device="cuda")
    aw = torch.full((B, H, s, npers + ws), 0x7fc0, dtype=torch.uint16, device="cuda")  # NaN canary
    D.call("swa_forward_f32_cuda", _u16(q), _u16(k), _u16(v), out, aw, s, H, td // H, ws, B, npers)
    torch.cuda.synchronize()
    return out.cpu().numpy(), aw.cpu().numpy()


def gpu_backward(q, k, v, aw, go, ws, H, npers):
    B, s, td = q.shape
    dq, dk, dv = zeros(B, s, td), zeros(B, s, td), zeros(B, s, td)
    D.call("swa_backward_f32_cuda", _u16(q), _u16(k), _u16(v), _u16(aw), dev(go), dq, dk, dv,
           s, H, td // H, ws, B, npers)
    torch.cuda.synchronize()
    return host(dq), host(dk), host(dv)


@pytest.mark.parametrize("B,s,H,hd,ws,npers", [(2, 40, 2, 64, 16, 0), (1, 70, 3, 32, 64, 0),
                                               (2, 33, 2, 64, 8, 5), (1, 20, 1, 8, 32, 0),
                                               (1, 600, 2, 64, 512, 0), (1, 50, 2, 24, 7, 3),
                                               (2, 200, 2, 64, 101, 0), (1, 1100, 1, 64, 300, 0),
                                               (2, 600, 4, 32, 512, 0), (1, 200, 2, 32, 101, 0), (3, 130, 2, 32, 64, 0),
                                               (1, 1100, 1, 32, 300, 0), (1, 2, 1, 32, 2, 0)])
def test_swa_forward_backward_parity(B, s, H, hd, ws, npers):
    q, k, v, go = _case(B, s, H, hd, 100 + s + ws)
    out, aw = gpu_forward(q, k, v, ws, H, npers)
    oo, awo = orc.swa_forward(q, k, v, ws, H, npers)
    assert_close("out", orc.bf16_to_f32(out), orc.bf16_to_f32(oo), REL_TOL_BF16)
    w, wo = orc.bf16_to_f32(aw), orc.bf16_to_f32(awo)
    assert np.abs(w - wo).max() < 1e-2, "test_cuda_swa.rs:100 bound"
    assert np.all(w[wo == 0] == 0), "unused slots are written as zero"
    assert np.allclose(w.sum(-1), 1.0, atol=2e-2)
    # backward on identical stored weights: fp32 round-off only
    dq, dk, dv = gpu_backward(q, k, v, awo, go, ws, H, npers)
    oq, ok, ov = orc.swa_backward(q, k, v, awo, go, ws, H, npers)
    assert_close("d_q", dq, oq, 1e-4)
    assert_close("d_k", dk, ok, 1e-4)
    assert_close("d_v", dv, ov, 1e-4)
    # end to end (GPU weights): bf16 tolerance
    dq2, dk2, dv2 = gpu_backward(q, k, v, aw, go, ws, H, npers)
    assert_close("d_q e2e", dq2, oq, REL_TOL_BF16)
    assert_close("d_k e2e", dk2, ok, REL_TOL_BF16)
    assert_close("d_v e2e", dv2, ov, REL_TOL_BF16)


def test_swa_known_answers_on_gpu():
    """core/src/swa.rs:286-344: window 1 copies V; identical keys average V."""
    bf = lambda x: orc.f32_to_bf16(np.asarray(x, np.float32))
    q = bf(np.tile([1.0, 0, 0, 0, 0, 0, 0, 0], (1, 4, 1)))
    vals = np.zeros((1, 4, 8), np.float32)
    vals[0, :, 0] = [10, 20, 30, 40]
    out, aw = gpu_forward(q, q, bf(vals), 1, 1, 0)
    assert np.array_equal(orc.bf16_to_f32(out), vals)
    out, aw = gpu_forward(q, q, bf(vals), 2, 1, 0)
    assert abs(orc.bf16_to_f32(out)[0, 3, 0] - 35.0) < 0.2


def test_swa_backward_accumulates_dk_dv_and_overwrites_dq():
    q, k, v, go = _case(1, 30, 2, 16, 7)
    out, aw = gpu_forward(q, k, v, 8, 2, 0)
    B, s, td = q.shape
    dq = torch.full((B, s, td), 5.0, device="cuda")
    dk = torch.full((B, s, td), 1.0, device="cuda")
    dv = torch.full((B, s, td), 2.0, device="cuda")
    D.call("swa_backward_f32_cuda", _u16(q), _u16(k), _u16(v), _u16(aw), dev(go), dq, dk, dv, s, 2, 16, 8, B, 0)
    torch.cuda.synchronize()
    oq, ok, ov = orc.swa_backward(q, k, v, aw, go, 8, 2, 0)
    assert_close("d_q", host(dq), oq, 1e-4)
    assert_close("d_k", host(dk) - 1.0, ok, 1e-4)
    assert_close("d_v", host(dv) - 2.0, ov, 1e-4)


@pytest.mark.parametrize("hd", [64, 32])
@pytest.mark.parametrize("B,s,H,ws", [(2, 40, 2, 16), (1, 600, 2, 512), (2, 200, 2, 101), (1, 1100, 1, 300),
                                      (1, 2, 1, 2), (8, 130, 2, 64), (1, 64, 1, 64), (1, 65, 3, 2)])
def test_swa_without_weight_tensor(B, s, H, ws, hd):
    """The pair that keeps per-query softmax statistics instead of the weight tensor: output against the
    weight-storing forward and the oracle, statistics against the oracle's scores, gradients against the weight-storing
    backward (same rounding of the weights: fp32 round-off) and the oracle (bf16 tolerance)."""
    q, k, v, go = _case(B, s, H, hd, 300 + s + ws)
    out_w, aw = gpu_forward(q, k, v, ws, H, 0)
    out = torch.zeros(B, s, H * hd, dtype=torch.uint16, device="cuda")
    stats = torch.full((B, H, s, 2), float("nan"), device="cuda")
    D.call("swa_forward_lse_bf16_rocm", _u16(q), _u16(k), _u16(v), out, stats, s, H, hd, ws, B)
    torch.cuda.synchronize()
    # blocked softmax with a running maximum: the output agrees with the weight-storing forward to bf16 rounding
    # (its weights are rounded before the product with V, here the unnormalised ones are) and with the oracle
    assert_close("out vs stored weights", orc.bf16_to_f32(out.cpu().numpy()), orc.bf16_to_f32(out_w), REL_TOL_BF16)
    assert_close("out", orc.bf16_to_f32(out.cpu().numpy()), orc.bf16_to_f32(orc.swa_forward(q, k, v, ws, H, 0)[0]),
                 REL_TOL_BF16)
    # statistics from the scores in float64
    qf, kf = (orc.bf16_to_f32(a).astype(np.float64).reshape(B, s, H, hd) for a in (q, k))
    st = host(stats)
    for b in range(B):
        for h in range(H):
            sc = qf[b, :, h] @ kf[b, :, h].T / np.sqrt(hd)
            for t in range(0, s, max(1, s // 37)):
                row = sc[t, max(t + 1 - ws, 0):t + 1]
                assert abs(st[b, h, t, 0] - row.max() * np.log2(np.e)) < 1e-3 * max(1.0, abs(row.max()))
                assert abs(st[b, h, t, 1] * np.exp(row - row.max()).sum() - 1.0) < 1e-4
    dq, dk, dv = zeros(B, s, H * hd), zeros(B, s, H * hd), zeros(B, s, H * hd)
    D.call("swa_backward_lse_bf16_rocm", _u16(q), _u16(k), _u16(v), stats, dev(go), dq, dk, dv, s, H, hd, ws, B)
    torch.cuda.synchronize()
    wq, wk, wv = gpu_backward(q, k, v, aw, go, ws, H, 0)
    # a weight rebuilt from a score that differs in its last bit may round to the neighbouring bf16
    assert_close("d_q vs stored weights", host(dq), wq, 2e-3)
    assert_close("d_k vs stored weights", host(dk), wk, 2e-3)
    assert_close("d_v vs stored weights", host(dv), wv, 2e-3)
    oo, awo = orc.swa_forward(q, k, v, ws, H, 0)
    oq, ok, ov = orc.swa_backward(q, k, v, awo, go, ws, H, 0)
    assert_close("d_q", host(dq), oq, REL_TOL_BF16)
    assert_close("d_k", host(dk), ok, REL_TOL_BF16)
    assert_close("d_v", host(dv), ov, REL_TOL_BF16)
    # d_k and d_v are accumulated into, d_q is overwritten: a second call doubles the first two only
    q1, k1, v1 = host(dq), host(dk), host(dv)
    D.call("swa_backward_lse_bf16_rocm", _u16(q), _u16(k), _u16(v), stats, dev(go), dq, dk, dv, s, H, hd, ws, B)
    torch.cuda.synchronize()
    assert np.array_equal(host(dq), q1)
    assert np.array_equal(host(dk), 2 * k1) and np.array_equal(host(dv), 2 * v1)


@pytest.mark.parametrize("B,s,H,hd,ws", [(2, 200, 2, 64, 101), (1, 130, 4, 32, 64), (1, 600, 2, 64, 512)])
def test_swa_backward_into_bf16_columns(B, s, H, hd, ws):
    """The statistics backward that writes its gradients as bf16 into columns of a wider matrix: the same numbers as the
    fp32 outputs rounded to bf16, bit for bit (the sums are the same, the rounding happens at the store); columns
    between and around the three blocks are left alone."""
    from nl_hecate_amd.ffi import lib
    q, k, v, go = _case(B, s, H, hd, 900 + s + ws)
    td = H * hd
    out = torch.zeros(B, s, td, dtype=torch.uint16, device="cuda")
    stats = torch.zeros(B, H, s, 2, device="cuda")
    D.call("swa_forward_lse_bf16_rocm", _u16(q), _u16(k), _u16(v), out, stats, s, H, hd, ws, B)
    dq, dk, dv = zeros(B, s, td), zeros(B, s, td), zeros(B, s, td)
    god = dev(go)
    D.call("swa_backward_lse_bf16_rocm", _u16(q), _u16(k), _u16(v), stats, god, dq, dk, dv, s, H, hd, ws, B)
    ld = 3 * td + 24
    G = _u16(np.full((B * s, ld), 0x7fc1, dtype=np.uint16))   # a NaN pattern: untouched columns keep it
    qd, kd, vd = _u16(q), _u16(k), _u16(v)
    base = G.data_ptr()
    lib.swa_backward_lse_bf16_cols_rocm(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), stats.data_ptr(), god.data_ptr(),
                                        base + 2 * 8, base + 2 * (8 + td), base + 2 * (16 + 2 * td), ld, s, H, hd, ws, B)
    torch.cuda.synchronize()
    Gh = G.cpu().numpy()
    want = lambda t: t.reshape(B * s, td).to(torch.bfloat16).view(torch.uint16).cpu().numpy()
    assert np.array_equal(Gh[:, 8:8 + td], want(dq))
    assert np.array_equal(Gh[:, 8 + td:8 + 2 * td], want(dk))
    assert np.array_equal(Gh[:, 16 + 2 * td:16 + 3 * td], want(dv))
    for lo, hi in ((0, 8), (8 + 2 * td, 16 + 2 * td), (16 + 3 * td, ld)):
        assert np.all(Gh[:, lo:hi] == 0x7fc1)


def test_swa_without_weight_tensor_rejects_other_shapes():
    from nl_hecate_amd.ffi import lib
    z = torch.zeros(1, 8, 16, dtype=torch.uint16, device="cuda")
    st = torch.zeros(1, 1, 8, 2, device="cuda")
    lib.nlh_set_error_mode(1)
    try:
        lib.nlh_clear_error()
        D.call("swa_forward_lse_bf16_rocm", z, z, z, z, st, 8, 1, 16, 4, 1)
        assert b"head_dim 64" in lib.nlh_last_error()
        lib.nlh_clear_error()
        g = torch.zeros(1, 8, 16, device="cuda")
        D.call("swa_backward_lse_bf16_rocm", z, z, z, st, g, g, g, g, 8, 1, 16, 4, 1)
        assert b"head_dim 64" in lib.nlh_last_error()
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)
