"""GPU parity of the entry points the reference ships as fused kernels and this library
composes or adds late: fused forwards (normalise + gates + recurrence), the per-row error
subtract-and-clip, and single-token decode attention.  fp32: relative 1e-4; the bf16 decode
output may differ from the oracle by one bf16 ulp (the softmax is summed in another order)."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
F32_MAX = orc.F32_MAX


@pytest.mark.parametrize("rows,d,clip", [(37, 64, 0.0), (37, 64, 3.0), (5, 100, 1.5), (200, 16, 0.7)])
def test_error_subtract_clip(rows, d, clip):
    r = np.random.default_rng(rows + d)
    pred, v = r.standard_normal((rows, d)).astype(np.float32), r.standard_normal((rows, d)).astype(np.float32)
    want = orc.error_subtract_clip(pred, v, clip)
    p = dev(pred)
    D.call("error_subtract_clip_f32_cuda", p, dev(v), rows, d, clip)
    torch.cuda.synchronize()
    assert_close("errors", host(p), want, 1e-6)
    if clip > 0:
        assert np.linalg.norm(host(p), axis=1).max() <= clip * (1 + 1e-5)


@pytest.mark.parametrize("titans", [True, False])
@pytest.mark.parametrize("B,s,d", [(3, 40, 64), (2, 33, 32), (2, 16, 16)])
def test_fused_forward(titans, B, s, d):
    r = np.random.default_rng(B * s + d + titans)
    f = np.float32
    k, v, q = (r.standard_normal((B, s, d)).astype(f) * 1.7 for _ in range(3))
    wa, wt, we = (0.3 * r.standard_normal(2 * d).astype(f) for _ in range(3))
    ba, bt, be = -1.0, -2.0, 1.0
    alim, tlim = (0.05, 0.9), (0.01, 0.6)
    m0 = 0.1 * r.standard_normal((B, d, d)).astype(f)
    s0 = 0.1 * r.standard_normal((B, d, d)).astype(f)
    want = [orc.fused_forward(k[b], v[b], q[b], wa, ba, wt, bt, we if titans else None, be, alim, tlim, m0[b],
                              s0[b]) for b in range(B)]
    kd, vd, qd = dev(k), dev(v), dev(q)
    bias = lambda x: dev(np.array([x], f))
    ms, ss, y = zeros(B, s + 1, d, d), zeros(B, s + 1, d, d), zeros(B, s, d)
    al, th, et, kn, qn = (zeros(B * s) for _ in range(5))
    if titans:
        D.call("titans_fused_forward_f32_cuda", kd, vd, qd, dev(wa), bias(ba), dev(wt), bias(bt), dev(we),
               bias(be), alim[0], alim[1], tlim[0], tlim[1], dev(m0), dev(s0), ms, ss, y, al, th, et, kn, qn,
               s, d, B, 0.0, F32_MAX)
    else:
        D.call("dgd_fused_forward_f32_cuda", kd, vd, qd, dev(wa), bias(ba), dev(wt), bias(bt), alim[0], alim[1],
               tlim[0], tlim[1], dev(m0), ms, y, al, th, kn, qn, s, d, B, 0.0)
    torch.cuda.synchronize()
    st = lambda n: np.stack([w[n] for w in want])
    assert_close("k normalised in place", host(kd), st("k"), 1e-6)
    assert_close("q normalised in place", host(qd), st("q"), 1e-6)
    assert_close("k_norms", host(kn).reshape(B, s), st("k_norms"), 1e-6)
    assert_close("alpha", host(al).reshape(B, s), st("alpha"), 1e-5)
    assert_close("theta", host(th).reshape(B, s), st("theta"), 1e-5)
    assert host(al).min() >= alim[0] and host(al).max() <= alim[1]
    assert host(th).min() >= tlim[0] and host(th).max() <= tlim[1]
    assert_close("y", host(y), st("y"))
    assert_close("m_states", host(ms), st("m_states"))
    if titans:
        assert_close("eta", host(et).reshape(B, s), st("eta"), 1e-5)
        assert_close("s_states", host(ss), st("s_states"))


def _bf16_bits(x):
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.uint16).numpy()


@pytest.mark.parametrize("cache_len,H,hd,window,n_p", [(1, 2, 64, 8, 0), (5, 2, 64, 8, 0), (40, 4, 64, 16, 0),
                                                       (40, 4, 32, 16, 4), (3, 2, 64, 16, 4), (600, 8, 64, 512, 0),
                                                       (600, 2, 128, 512, 16)])
def test_swa_single_token(cache_len, H, hd, window, n_p):
    r = np.random.default_rng(cache_len + H + hd)
    td = H * hd
    q = _bf16_bits(r.standard_normal(td).astype(np.float32))
    kc = _bf16_bits(r.standard_normal((cache_len, td)).astype(np.float32))
    vc = _bf16_bits(r.standard_normal((cache_len, td)).astype(np.float32))
    want = orc.swa_single_token(q, kc, vc, window, H, n_p)
    out = torch.zeros(td, dtype=torch.uint16, device="cuda")
    D.call("swa_single_token_cuda", torch.from_numpy(q).cuda(), torch.from_numpy(kc).cuda(),
           torch.from_numpy(vc).cuda(), out, cache_len, H, hd, window, n_p)
    torch.cuda.synchronize()
    got_f, want_f = orc.bf16_to_f32(out.cpu().numpy()), orc.bf16_to_f32(want)
    assert_close("decode output", got_f, want_f, 2e-2)
    assert np.mean(out.cpu().numpy() == want) > 0.9   # bit-identical except for rounding ties
