"""Second opinion on the yardstick of the layer tests: tests/torch_mag_reference.py (PyTorch autograd, float64 state;
what tests/test_gpu_mag_layer.py and the full-size configs[4] test compare the GPU layer against) is a restatement
written for this build, so its forward conventions are pinned here against the oracle's composition of the same
layer (oracle/cms_model.py: oracle attention with bf16 storage, the level step of oracle/memory_level.py around the C
oracle's rules, combine with 1 / sqrt(k) for k > 2, sigmoid gate, W_o), on one small shape per rule: the exact
Titans rule, the frozen-M0 chunkwise rule, and a frozen (read-only) level."""
import types

import numpy as np
import pytest
import torch

from oracle import cms_model as CM
from tests import torch_mag_reference as R
from tests.test_oracle_memory_level import cfg_of, params

f64 = np.float64


@pytest.mark.parametrize("rule,chunk,active,k", [("exact", None, [True, True], 2), ("chunkwise", 4, [True, True, True], 3),
                                                 ("exact", None, [True, False], 2)])
def test_torch_layer_forward_equals_the_oracle_composition(rule, chunk, active, k):
    nh, hd, s, bs, window, v = 2, 4, 12, 2, 5, 17
    d = nh * hd
    r = np.random.default_rng(7 + k)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: r.uniform(-lim, lim, (d, d)).astype(f64) for n in ("w_q", "w_k", "w_v", "w_o")}
    p["w_embed"] = (r.standard_normal((v, d)) / np.sqrt(d) * 2).astype(f64)
    p["w_unembed"] = np.eye(d, v).astype(f64)
    p["levels"] = [params(d, 30 + i, f64) for i in range(k)]
    kw = dict(proxy=True, chunk_size=chunk) if rule == "chunkwise" else {}
    cfg = types.SimpleNamespace(d_model=d, vocab_size=v, num_heads=nh, head_dim=hd, window_size=window, seq_len=s,
                                n_persistent=0, residual=False, parallel=None,
                                levels=[cfg_of("titans", nh, hd, **kw) for _ in range(k)])
    ids = r.integers(0, v, bs * s)
    mem0 = [(0.2 * r.standard_normal((bs * nh, hd, hd))).astype(f64) for _ in range(k)]
    _, c, _ = CM.forward(p, cfg, ids, ids, active, mem0, quantize=True)
    want = c["proj"].reshape(bs, s, d)
    # the same layer in the torch restatement: x = the embedded tokens, zero initial momentum as the level step has it
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    P = dict(w_q=t(p["w_q"]), w_k=t(p["w_k"]), w_v=t(p["w_v"]), w_o=t(p["w_o"]),
             levels=[{n: t(a) for n, a in L.items()} for L in p["levels"]])
    x = t(p["w_embed"][ids].reshape(bs, s, d))
    m_states = [t(m.reshape(bs * nh, hd * hd)) for m in mem0]
    s_states = [torch.zeros(bs * nh, hd * hd, dtype=torch.float64) for _ in range(k)]
    out, _ = R.forward(P, x, nh, window, active, m_states, s_states, rule, chunk, bf16_mem=False)
    got = out.detach().numpy()
    # the attention branch is stored as bf16 on both sides (q, k, v and the output rounded once): a projection that
    # lands on a rounding boundary can round apart, which moves an output by one bf16 step of the attention value
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 2.0 ** -7, err
    # and without that storage the two agree to rounding: the float attention of the oracle against torch's own
    _, cf, _ = CM.forward(p, cfg, ids, ids, active, mem0, quantize=False)
    saved = R._bf16_st
    R._bf16_st = lambda z: z
    try:
        out_f, _ = R.forward(P, x, nh, window, active, m_states, s_states, rule, chunk, bf16_mem=False)
    finally:
        R._bf16_st = saved
    assert np.abs(out_f.detach().numpy() - cf["proj"].reshape(bs, s, d)).max() <= 1e-10 * max(1.0, np.abs(want).max())
