"""GPU parity of the whole training step on device buffers (nl_hecate_amd.cms_model: the host mirror of the
reference's gpu_cms_forward / gpu_cms_backward / gpu_weight_update) against its CPU composition
(oracle/cms_model.py, bf16 attention storage as the reference runs it), and the reference's own GPU-resident and
TNT tests (core/tests/test_gpu_resident.rs, test_cuda_tnt.rs: loss parity at 5 %, the loss falling over five
SGD steps, k = 2, finiteness) with its data recipe (token t -> t % vocab, target t + 1)."""
import types

import numpy as np
import pytest
import torch

from nl_hecate_amd import cms_model as GM
from nl_hecate_amd.cms import ContextState, Pulse
from nl_hecate_amd.mag_layer import MemoryLevelParams
from nl_hecate_amd.memory_level import LevelConfig
from nl_hecate_amd.serving import GpuMAGParams
from nl_hecate_amd.tnt import ParallelConfig
from oracle import cms_model as CM
from tests.gpu_util import assert_close, dev, host
from tests.test_gpu_memory_level import NAMES
from tests.test_oracle_cms_model import model

pytestmark = pytest.mark.gpu
f32 = np.float32
LN = ("ln_attn_gamma", "ln_attn_beta", "ln_mem_gamma", "ln_mem_beta")


def make_test_data(s, v, bs=1):
    """test_gpu_resident.rs:68-72"""
    return [t % v for t in range(s)] * bs, [t % v for t in range(1, s + 1)] * bs


def gpu_model(p):
    lv = [MemoryLevelParams(*[dev(l[n]) for n in NAMES]) for l in p["levels"]]
    gp = GpuMAGParams(dev(p["w_embed"]), dev(p["w_q"]), dev(p["w_k"]), dev(p["w_v"]), dev(p["w_o"]), dev(p["w_unembed"]), lv)
    ln = GM.LayerNormParams(*[dev(p[n]) for n in LN]) if "ln_attn_gamma" in p else None
    return gp, ln


def setup(rule, k, nh, hd, v, s, window, bs=1, n_p=0, residual=False, parallel=None, seed=7, **kw):
    d = nh * hd
    lcfgs = [LevelConfig(rule, nh, hd, **kw) for _ in range(k)]
    cfg = GM.ModelConfig(d, v, nh, hd, window, s, lcfgs, n_persistent=n_p, residual=residual,
                         parallel=None if parallel is None else ParallelConfig(*parallel))
    ocfg = types.SimpleNamespace(d_model=d, vocab_size=v, num_heads=nh, head_dim=hd, window_size=window, seq_len=s,
                                 n_persistent=n_p, residual=residual, levels=lcfgs,
                                 parallel=None if parallel is None else types.SimpleNamespace(
                                     tnt_global_chunk_size=parallel[0], tnt_local_chunk_size=parallel[1]))
    p = model(d, v, k, seed, f32, residual=residual)
    r = np.random.default_rng(seed + 1)
    mem = [(0.2 * r.standard_normal((bs * nh, hd, hd))).astype(f32) for _ in range(k)]
    return cfg, ocfg, p, mem


def compare(cfg, ocfg, p, mem, ids, tgt, active):
    k, nh, hd = cfg.k, cfg.num_heads, cfg.head_dim
    gp, ln = gpu_model(p)
    ctx = ContextState([dev(m.reshape(m.shape[0], hd * hd)) for m in mem])
    pulse = Pulse(0, list(active))
    loss, cache = GM.gpu_cms_forward(gp, cfg, ids, tgt, pulse, ctx, ln)
    grads = GM.gpu_cms_backward(gp, cfg, cache, True, ln)
    torch.cuda.synchronize()
    loss_o, c_o, mem_o = CM.forward(p, ocfg, ids, tgt, active, mem)
    g_o = CM.backward(p, ocfg, c_o)
    assert abs(loss - loss_o) <= 2e-3 * abs(loss_o), (loss, loss_o)
    assert_close("logits", host(cache["logits"]), c_o["logits"], 2e-2)
    for lv in range(k):
        assert_close(f"memory[{lv}]", host(ctx.memory[lv]).reshape(mem_o[lv].shape), mem_o[lv], 1e-4)
    # gradients: the attention branch stores bf16, and a bf16 rounding of q, k, v that falls the other way
    # (fp32 GEMMs in another summation order) moves them: the bf16 bar
    for n in ("w_embed", "w_q", "w_k", "w_v", "w_o", "w_unembed"):
        assert_close("d_" + n, host(getattr(grads, "d_" + n)), g_o[n], 2e-2)
    if cfg.residual:
        for n in LN:
            assert_close("d_" + n, host(getattr(grads, "d_" + n)), g_o[n], 2e-2)
    for lv in range(k):
        gl = g_o["levels"][lv]
        lg = grads.levels[lv]
        if gl is None:
            assert float(lg.d_w_k_mem.abs().max()) == 0.0 and float(lg.d_w_alpha.abs().max()) == 0.0
            assert grads.level_output_gnorms[lv] == 0.0
            continue
        assert grads.level_output_gnorms[lv] > 0.0
        for n in ("w_k", "w_v", "w_q"):
            assert_close(f"level {lv} d_{n}", host(getattr(lg, f"d_{n}_mem")), gl[n], 2e-2)
        for n in ("w_alpha", "b_alpha", "w_theta", "b_theta"):
            assert_close(f"level {lv} d_{n}", host(getattr(lg, "d_" + n)), gl[n], 2e-2)
    return loss, loss_o


CASES = [  # rule, k, active, nh, hd, v, s, window, bs, n_p, residual, parallel, extra level settings
    ("delta", 1, [True], 2, 8, 17, 16, 8, 1, 0, False, None, {}),
    ("titans", 3, [True, True, False], 2, 8, 17, 12, 5, 2, 2, False, None, {}),
    ("hebbian", 2, [True, True], 1, 16, 11, 10, 4, 1, 0, False, None, {}),
    ("titans", 2, [True, False], 2, 8, 17, 12, 6, 1, 0, True, None, {}),
    ("delta", 2, [True, True], 2, 8, 17, 14, 7, 1, 0, False, (6, 3), {}),
    ("titans", 1, [True], 1, 16, 13, 12, 12, 1, 0, False, (4, 4), {}),
    ("titans", 2, [True, True], 2, 8, 17, 16, 8, 2, 0, False, None, dict(proxy=True, chunk_size=4)),
    ("delta", 1, [True], 2, 8, 17, 16, 8, 1, 0, False, None, dict(checkpoint_interval=4, alpha_floor=0.2, alpha_ceil=0.3)),
]


@pytest.mark.parametrize("rule,k,active,nh,hd,v,s,window,bs,n_p,residual,parallel,kw", CASES)
def test_forward_and_backward_match_the_composition(rule, k, active, nh, hd, v, s, window, bs, n_p, residual, parallel, kw):
    cfg, ocfg, p, mem = setup(rule, k, nh, hd, v, s, window, bs, n_p, residual, parallel, seed=20 + k + s, **kw)
    r = np.random.default_rng(5)
    ids, tgt = r.integers(0, v, bs * s), r.integers(0, v, bs * s)
    tgt[1] = -1
    compare(cfg, ocfg, p, mem, list(ids), list(tgt), active)


@pytest.mark.parametrize("rule", ["delta", "titans", "hebbian"])
def test_reference_forward_parity(rule):
    """test_gpu_resident.rs:79-122: the loss within 5 % of the CPU forward (here: the float attention composition,
    no bf16 anywhere, which is what the reference's CPU model runs)."""
    nh, hd, v, s = 2, 4, 16, 8
    cfg, ocfg, p, mem = setup(rule, 1, nh, hd, v, s, s, seed=42)
    mem = [np.zeros_like(mem[0])]
    ids, tgt = make_test_data(s, v)
    gp, _ = gpu_model(p)
    ctx = ContextState([dev(mem[0].reshape(nh, hd * hd))])
    loss, _ = GM.gpu_cms_forward(gp, cfg, ids, tgt, Pulse(0, [True]), ctx)
    loss_cpu, _, _ = CM.forward({n: (a.astype(np.float64) if isinstance(a, np.ndarray) else
                                      [{m: b.astype(np.float64) for m, b in l.items()} for l in a]) for n, a in p.items()},
                                ocfg, ids, tgt, [True], [mem[0].astype(np.float64)], quantize=False)
    assert abs(loss - loss_cpu) / max(abs(loss_cpu), 1e-8) < 0.05, (loss, loss_cpu)


@pytest.mark.parametrize("parallel", [None, (4, 2)])
def test_multistep_loss_decrease(parallel):
    """test_gpu_resident.rs:124-146 and test_cuda_tnt.rs:153-180: five SGD steps at lr 0.01, the loss falls."""
    nh, hd, v, s = 2, 4, 16, 8
    cfg, _, p, mem = setup("delta", 1, nh, hd, v, s, s, parallel=parallel, seed=42)
    ids, tgt = make_test_data(s, v)
    gp, _ = gpu_model(p)
    ctx = ContextState([dev(np.zeros((nh, hd * hd), f32))])
    losses = []
    for _ in range(5):
        loss, cache = GM.gpu_cms_forward(gp, cfg, ids, tgt, Pulse(0, [True]), ctx)
        grads = GM.gpu_cms_backward(gp, cfg, cache)
        GM.gpu_weight_update(gp, grads, 0.01)
        losses.append(loss)
    assert all(np.isfinite(losses)) and losses[4] < losses[0], losses


@pytest.mark.parametrize("parallel", [None, (4, 2)])
def test_k2_forward(parallel):
    """test_gpu_resident.rs:149-170, test_cuda_tnt.rs:183-202: two levels, both firing, a finite positive loss."""
    nh, hd, v, s = 2, 4, 16, 8
    cfg, _, p, mem = setup("delta", 2, nh, hd, v, s, 8, parallel=parallel, seed=42)
    ids, tgt = make_test_data(s, v)
    gp, _ = gpu_model(p)
    ctx = ContextState([dev(np.zeros((nh, hd * hd), f32)) for _ in range(2)])
    loss, _ = GM.gpu_cms_forward(gp, cfg, ids, tgt, Pulse(0, [True, True]), ctx)
    assert np.isfinite(loss) and loss > 0.0


def test_sync_embed_weights_and_argument_checks():
    nh, hd, v, s = 1, 8, 11, 6
    cfg, _, p, mem = setup("delta", 1, nh, hd, v, s, 4)
    gp, _ = gpu_model(p)
    GM.gpu_sync_embed_weights(gp, 8, v)
    assert np.array_equal(host(gp.w_embed), p["w_unembed"].T)
    ctx = ContextState([dev(mem[0].reshape(nh, 64))])
    with pytest.raises(AssertionError):
        GM.gpu_cms_forward(gp, cfg, [0] * 7, [0] * 7, Pulse(0, [True]), ctx)
    cfg.residual = True
    with pytest.raises(ValueError):
        GM.gpu_cms_forward(gp, cfg, [0] * 6, [0] * 6, Pulse(0, [True]), ctx)
