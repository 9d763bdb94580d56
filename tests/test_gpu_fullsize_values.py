"""Value checks at the FULL size of every BASELINE configuration, against the CPU oracle (the chains
are independent, so the oracle runs them on a thread pool: the whole of configs[2] takes a few seconds
on the host cores of a GPU box).  Every output and every gradient of every chain is compared, in the
max norm and in the L2 norm, at the tolerance of the path: 1e-4 for fp32 paths, for the bf16-token
path 1e-3 on the forward and 1e-2 on the backward (stated bar 2e-2).

  configs[1]  exact Titans, 64 chains x 2048 tokens, checkpoints every 64, fused checkpointed backward
  configs[2]  chunkwise Titans on bf16 tokens, 128 chains x 4096 tokens, chunk 64, all gradients
  configs[3]  HOPE self-referential memory, 64 chains x 2048 tokens launched together, 8 of them compared
  configs[4]  the full layer, batch 8 x 4096 tokens, d = 512, k = 4 levels at periods [1, 8, 64, 512],
              window 512: one training step, eager and replayed from a HIP graph (bit-equal), finite;
              the same layer on batch 1 x 1024 tokens against the float64 autograd restatement
"""
import math
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from nl_hecate_amd import selfref as SR
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu
F32_MAX = orc.F32_MAX


def _threads():
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(1, min(n, 16))


def _pool_map(fn, n):
    with ThreadPoolExecutor(_threads()) as pool:
        return list(pool.map(fn, range(n)))


def test_config1_exact_titans_full_size_against_the_oracle():
    B, s, d, C = 64, 2048, 64, 64
    x = rule_inputs(B, s, d, 0xC1)
    n = orc.checkpoint_count(s, C)
    print(f"configs[1]: {B} chains x {s} tokens, {n} checkpoints", flush=True)
    mc, sc, y = zeros(B, n, d, d), zeros(B, n, d, d), zeros(B, s, d)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s), d_theta=zeros(B, s),
             d_eta=zeros(B, s), d_m=zeros(d, d), d_s=zeros(d, d))
    dx = {k_: dev(v) for k_, v in x.items()}
    D.call("titans_forward_ckpt_batched_f32_rocm", dx["k"], dx["v"], dx["q"], dx["alpha"], dx["theta"], dx["eta"],
           dx["m0"], dx["s0"], mc, sc, y, s, d, B, C, 0.0, F32_MAX)
    D.call("titans_backward_ckpt_f32_rocm", dx["k"], dx["v"], dx["q"], dx["alpha"], dx["theta"], dx["eta"], mc, sc,
           dx["dy"], *g.values(), s, d, B, C, 0.0, F32_MAX)
    # the library's choice at this shape is the chunk-parallel matrix form; the fused sequential kernel once more
    g2 = {n_: torch.zeros_like(t) for n_, t in g.items()}
    prev = lib.nlh_exact_backward_form(2)
    try:
        D.call("titans_backward_ckpt_f32_rocm", dx["k"], dx["v"], dx["q"], dx["alpha"], dx["theta"], dx["eta"], mc, sc,
               dx["dy"], *g2.values(), s, d, B, C, 0.0, F32_MAX)
    finally:
        lib.nlh_exact_backward_form(prev)
    torch.cuda.synchronize()

    def chain(b):
        a = [x[n_][b] for n_ in ("k", "v", "q", "alpha", "theta", "eta")]
        yo, mco, sco = orc.forward_ckpt(*a, x["m0"][b], x["s0"][b], C)
        return yo, mco, sco, orc.backward_ckpt(*a, mco, sco, x["dy"][b], C)
    want = _pool_map(chain, B)
    assert_close("y", host(y), np.stack([w[0] for w in want]))
    assert_close("m_ckpt", host(mc), np.stack([w[1] for w in want]))
    assert_close("s_ckpt", host(sc), np.stack([w[2] for w in want]))
    for n_ in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
        assert_close(n_, host(g[n_]), np.stack([w[3][n_] for w in want]))
    for n_ in ("d_m", "d_s"):   # summed over the batch
        assert_close(n_, host(g[n_]), np.sum([w[3][n_].astype(np.float64) for w in want], axis=0))
    for n_ in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
        assert_close(n_ + " (fused kernel)", host(g2[n_]), np.stack([w[3][n_] for w in want]))
    for n_ in ("d_m", "d_s"):
        assert_close(n_ + " (fused kernel)", host(g2[n_]), np.sum([w[3][n_].astype(np.float64) for w in want], axis=0))


def test_config2_chunkwise_bf16_full_size_against_the_oracle():
    B, s, d, C = 128, 4096, 64, 64
    nc = s // C
    x = rule_inputs(B, s, d, 0xC2)
    bf = {n_: torch.from_numpy(x[n_]).to(torch.bfloat16) for n_ in ("k", "v", "q")}
    for n_ in bf:   # the oracle sees the same (exactly representable) tokens
        x[n_] = bf[n_].float().numpy()
    print(f"configs[2]: {B} chains x {s} tokens, chunk {C}", flush=True)
    mc, sc, y = zeros(B, nc + 1, d, d), zeros(B, nc + 1, d, d), zeros(B, s, d)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s), d_theta=zeros(B, s),
             d_eta=zeros(B, s), d_m=zeros(d, d), d_s=zeros(d, d))
    kq = [bf[n_].cuda() for n_ in ("k", "v", "q")]
    gates = [dev(x[n_]) for n_ in ("alpha", "theta", "eta")]
    D.call("titans_chunkwise_forward_bf16_rocm", *kq, *gates, dev(x["m0"]), dev(x["s0"]), mc, sc, y, s, d, B, C)
    D.call("titans_chunkwise_backward_bf16_rocm", *kq, *gates, mc, sc, dev(x["dy"]), *g.values(), s, d, B, C)
    torch.cuda.synchronize()

    def chain(b):
        a = [x[n_][b] for n_ in ("k", "v", "q", "alpha", "theta", "eta")]
        yo, mco, sco = orc.chunkwise_forward(*a, x["m0"][b], x["s0"][b], C, True)
        return yo, mco, sco, orc.chunkwise_backward(*a, mco, sco, x["dy"][b], C, True)
    want = _pool_map(chain, B)
    assert_close("y", host(y), np.stack([w[0] for w in want]), 1e-3)
    assert_close("m_chunk_states", host(mc), np.stack([w[1] for w in want]), 1e-3)
    assert_close("s_chunk_states", host(sc), np.stack([w[2] for w in want]), 1e-3)
    errs = {}
    for n_ in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
        errs[n_] = assert_close(n_, host(g[n_]), np.stack([w[3][n_] for w in want]), 1e-2)
    for n_ in ("d_m", "d_s"):
        errs[n_] = assert_close(n_, host(g[n_]), np.sum([w[3][n_].astype(np.float64) for w in want], axis=0), 1e-2)
    print("configs[2] backward errors:", {k_: f"{v:.1e}" for k_, v in errs.items()}, flush=True)


def hope_inputs(B, s, d, seed):
    """All six memories live (a zero M_mem stays zero with self-generated values) and a decay gate that
    starts near 1e-3 (M_alpha, M_eta carry a rank-1 term against the mean of x), so that the memories
    survive more than a hundred tokens; the gate feedback of the rule collapses every chain eventually,
    whatever the start, and the chunks after that hold exact zeros on both sides."""
    rs = np.random.default_rng(seed)
    lim = math.sqrt(6.0 / (2 * d))
    u = np.ones(d, np.float32) / np.sqrt(d)
    mems = ((rs.random((B, 6, d, d)) * 2 - 1) * lim).astype(np.float32)
    mems[:, 4] += -13.0 * np.outer(np.ones(d), u).astype(np.float32)
    mems[:, 3] += -6.0 * np.outer(np.ones(d), u).astype(np.float32)
    x = (rs.standard_normal((B, s, d)) / np.sqrt(8 * d) + 0.5 * u).astype(np.float32)
    dy = rs.standard_normal((B, s, d)).astype(np.float32)
    return mems, x, dy


def _assert_chunks_close(name, got, want, C, tol):
    """Per 64-token chunk: relative to the chunk's own size while it carries data (a chain's memories
    decay, so a whole-array norm would only see the first chunks), absolutely small once it is dead."""
    top = np.abs(want).max()
    for c0 in range(0, want.shape[0], C):
        w, gt = want[c0:c0 + C], got[c0:c0 + C]
        if np.abs(w).max() > 1e-6 * top:
            assert_close(f"{name} tokens {c0}..", gt, w, tol)
        else:
            assert np.abs(gt).max() <= 1e-5 * top, f"{name} tokens {c0}..: {np.abs(gt).max():.3e} where the oracle is dead"


def test_config3_hope_full_size_against_the_oracle():
    B, s, d, C = 64, 2048, 64, 64
    n_cmp = 8
    mems, x, dy = hope_inputs(B, s, d, 0xC3)
    print(f"configs[3]: {B} chains x {s} tokens launched, {n_cmp} compared", flush=True)
    m = dev(mems)
    y, cache = SR.chunkwise_self_ref_step(m, dev(x), C, True)
    d_emb, d_mems = SR.chunkwise_self_ref_step_backward(cache, dev(dy))
    torch.cuda.synchronize()
    pick = [0, 7, 8, 21, 33, 46, 55, 63][:n_cmp]

    def chain(i):
        b = pick[i]
        yo, mo, c = orc.selfref_forward(mems[b].copy(), x[b], C, True)
        de, dm = orc.selfref_backward(c, dy[b])
        return yo, mo, c["k"], c["alpha"], c["theta"], c["frozen"], de, dm
    want = _pool_map(chain, n_cmp)
    alive = []
    for i, b in enumerate(pick):
        yo, mo, ko, ao, to, fo, de, dm = want[i]
        alive.append(int(np.abs(yo).max(axis=1).nonzero()[0].max()) + 1)
        _assert_chunks_close(f"y[{b}]", host(y)[b], yo, C, 1e-4)
        _assert_chunks_close(f"k_cache[{b}]", host(cache.k_mem)[b], ko, C, 1e-4)
        _assert_chunks_close(f"d_emb[{b}]", host(d_emb)[b], de, C, 1e-4)
        assert_close(f"alpha[{b}]", host(cache.alpha)[b], ao)
        assert_close(f"theta[{b}]", host(cache.theta)[b], to)
        assert_close(f"frozen[{b}]", host(cache.frozen_snapshots)[b], fo)
        assert_close(f"final memories[{b}]", host(m)[b], mo)
        for mi in range(6):
            assert_close(f"d_mems[{b}][{mi}]", host(d_mems)[b, mi], dm[mi])
    print("configs[3]: tokens with non-zero output per compared chain:", alive, flush=True)
    assert min(alive) > 2 * C, "the compared chains must carry data over several chunks"


def test_config4_full_layer_step_graph_equals_eager_and_is_finite():
    from nl_hecate_amd.mag_layer import MagLayer, MagTrainer
    bs, s, d, heads, k, window = 8, 4096, 512, 8, 4, 512
    print("configs[4]: full layer, batch 8 x 4096, k = 4", flush=True)
    mk = lambda: MagLayer(d, heads, k, window, [1, 8, 64, 512], rule="chunkwise", chunk=64, seed=0xC4)
    eager, graphed = MagTrainer(mk()), MagTrainer(mk())
    g = torch.Generator(device="cpu").manual_seed(0xC5)
    for step in range(2):
        x = (torch.randn(bs, s, d, generator=g) / math.sqrt(d)).cuda()
        d_out = torch.randn(bs, s, d, generator=g).cuda()
        out_e = eager.step(x, lambda out: d_out).clone()
        out_g = graphed.step_graphed(x, d_out).clone()
        torch.cuda.synchronize()
        assert torch.isfinite(out_e).all()
        assert torch.equal(out_g, out_e), f"step {step}: replayed output differs from the eager one"
        for a, b in zip(graphed.grads.tensors(), eager.grads.tensors()):
            assert torch.isfinite(b).all() and torch.equal(a, b)
        for a, b in zip(graphed.layer.p.tensors(), eager.layer.p.tensors()):
            assert torch.isfinite(b).all() and torch.equal(a, b)
        for a, b in zip(graphed.layer.m_state, eager.layer.m_state):
            assert torch.equal(a, b)
    assert all(eager.opt.level_step(lv) == 2 for lv in range(k)), "seq 4096 >= every period: all levels fire"


def test_config4_layer_against_autograd_at_k4_periods_up_to_512():
    """Same layer (d = 512, 8 heads, k = 4, periods [1, 8, 64, 512], window 512, chunkwise rule) on one
    sequence of 1024 tokens against the float64 autograd restatement: output, d_x and every parameter
    gradient of all four levels.  Gate bias gradients (one scalar each, a sum over 1024 tokens that can
    nearly cancel) are measured against the size of the matching weight-vector gradient."""
    from tests.test_gpu_mag_layer import run_case
    w = run_case(bs=1, s=1024, d=512, nh=8, k=4, window=512, periods=[1, 8, 64, 512], rule="chunkwise", chunk=64,
                 seed=0xC6, bias_scale=True)
    print({n: f"{e:.1e}" for n, e in w.items()}, flush=True)
    assert max(w.values()) < 2e-2, w


def test_config4_layer_behind_the_c_abi_at_full_sequence_length_against_autograd():
    """The same layer on the path that issues every projection through the library (precision "bf16": x and the weights
    rounded once to bf16, fp32 accumulation; titans_levels_{forward,backward}_bf16_rocm) on one sequence of the
    configuration's full 4096 tokens (64 chunks per chain, every level's period inside the sequence) against the float64
    autograd restatement: output, d_x and every parameter gradient at the bf16 bar."""
    import nl_hecate_amd.mag_layer as ML
    from tests.test_gpu_mag_layer import run_case
    orig = ML.MagLayer.__init__

    def init_bf16(self, *a, **kw):
        kw["precision"] = "bf16"
        orig(self, *a, **kw)
    ML.MagLayer.__init__ = init_bf16
    try:
        print("configs[4]: layer behind the C ABI, 1 x 4096 tokens, k = 4", flush=True)
        w = run_case(bs=1, s=4096, d=512, nh=8, k=4, window=512, periods=[1, 8, 64, 512], rule="chunkwise", chunk=64,
                     seed=0xC7, bias_scale=True)
    finally:
        ML.MagLayer.__init__ = orig
    print({n: f"{e:.1e}" for n, e in w.items()}, flush=True)
    assert max(w.values()) < 2e-2, w
