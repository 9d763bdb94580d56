"""The MAG layer harness (k Titans levels + sliding-window attention + sigmoid gate) against a
plain PyTorch autograd restatement.  fp32 memory path: relative 1e-3 end to end through the
bf16 attention branch's tolerance of 2e-2 where attention contributes."""
import math

import numpy as np
import pytest
import torch

from nl_hecate_amd.mag_layer import MagLayer, MagTrainer, init_params
from tests import torch_mag_reference as R
from tests.gpu_util import rel_err

pytestmark = pytest.mark.gpu


def ref_params(p, dtype=torch.float64):
    leaf = lambda t: t.detach().cpu().to(dtype).requires_grad_(True)
    names = ("w_k", "w_v", "w_q", "w_alpha", "b_alpha", "w_theta", "b_theta", "w_eta", "b_eta")
    return dict(w_q=leaf(p.w_q), w_k=leaf(p.w_k), w_v=leaf(p.w_v), w_o=leaf(p.w_o),
                levels=[{n: leaf(getattr(l, n)) for n in names} for l in p.levels])


def run_case(bs, s, d, nh, k, window, periods, rule, chunk, seed, steps=1, bias_scale=False):
    """bias_scale: a gate bias gradient is one scalar, a sum over all tokens of signed terms that can
    nearly cancel; its error is then taken relative to max(|reference|, ||gradient of the matching gate
    weight vector||), the size of the sums it belongs to, instead of to its own (possibly tiny) value."""
    torch.manual_seed(seed)
    p = init_params(d, k, seed)
    layer = MagLayer(d, nh, k, window, periods, rule=rule, chunk=chunk, params=p)
    P = ref_params(p)
    hd = d // nh
    m_ref = [torch.zeros(bs * nh, hd * hd, dtype=torch.float64) for _ in range(k)]
    s_ref = [torch.zeros(bs * nh, hd * hd, dtype=torch.float64) for _ in range(k)]
    g = torch.Generator().manual_seed(seed + 1)
    worst = {}
    for step in range(steps):
        x = torch.randn(bs, s, d, generator=g) / math.sqrt(d) * 4
        d_out = torch.randn(bs, s, d, generator=g)
        out, cache = layer.forward(x.cuda())
        d_x, grads = layer.backward(cache, d_out.cuda())
        torch.cuda.synchronize()
        active = cache["pulse"].active_levels
        xr = x.double().requires_grad_(True)
        out_r, finals = R.forward(P, xr, nh, window, active, m_ref, s_ref, rule, chunk, bf16_mem=(rule == "chunkwise"))
        for t in [xr] + [P[n] for n in ("w_q", "w_k", "w_v", "w_o")] + [v for L in P["levels"] for v in L.values()]:
            t.grad = None
        (out_r * d_out.double()).sum().backward()
        m_ref = [f[0].detach() for f in finals]
        s_ref = [f[1].detach() for f in finals]
        layer.conductor.advance()
        chk = {"out": (out, out_r), "d_x": (d_x, xr.grad)}
        for n in ("w_q", "w_k", "w_v", "w_o"):
            chk["d_" + n] = (getattr(grads, n), P[n].grad)
        for lv in range(k):
            for n, t in P["levels"][lv].items():
                if t.grad is not None:
                    chk[f"L{lv}.d_{n}"] = (getattr(grads.levels[lv], n), t.grad)
        for n, (a, b) in chk.items():
            e = rel_err(a.detach().cpu().numpy().reshape(b.shape), b.detach().numpy())
            if bias_scale and ".d_b_" in n:
                wref = chk[n.replace(".d_b_", ".d_w_")][1]
                e = float((a.detach().cpu().double().reshape(b.shape) - b.detach()).abs().max()
                          / max(float(b.detach().abs().max()), float(wref.detach().norm())))
            worst[n] = max(worst.get(n, 0.0), e)
    return worst


@pytest.mark.parametrize("rule,chunk", [("exact", 8)])
def test_small_layer_matches_autograd(rule, chunk):
    # hd = 16: general SWA kernels, d = 16 memory kernels; both levels fire (seq >= period).
    # (the matrix-form chunkwise rule needs hd = 64: covered below)
    w = run_case(bs=2, s=24, d=32, nh=2, k=2, window=8, periods=[1, 8], rule=rule, chunk=chunk, seed=3)
    print(w)
    assert max(w.values()) < 2e-2, w


def test_layer_with_production_head_size_matches_autograd():
    # hd = 64: matrix-core SWA, fused checkpointed backward; k = 3 exercises the 1/sqrt(k) scaling
    w = run_case(bs=1, s=70, d=128, nh=2, k=3, window=32, periods=[1, 8, 64], rule="exact", chunk=16, seed=5)
    print(w)
    assert max(w.values()) < 2e-2, w


def test_chunkwise_matrix_form_layer_matches_autograd():
    w = run_case(bs=1, s=70, d=128, nh=2, k=2, window=32, periods=[1, 8], rule="chunkwise", chunk=32, seed=7)
    print(w)
    assert max(w.values()) < 2e-2, w


def test_frozen_levels_and_context_carry_over_steps():
    # seq 6 < period 8: level 1 fires on step 0 only (step % 8 == 0), then reads its frozen memory
    w = run_case(bs=1, s=6, d=32, nh=2, k=2, window=4, periods=[1, 8], rule="exact", chunk=4, seed=9, steps=3)
    print(w)
    assert max(w.values()) < 2e-2, w


def test_training_step_changes_only_active_levels():
    d, nh, k = 32, 2, 2
    layer = MagLayer(d, nh, k, 4, [1, 8], rule="exact", chunk=4, seed=11)
    tr = MagTrainer(layer)
    g = torch.Generator().manual_seed(0)
    before = [t.clone() for t in layer.p.tensors()]
    for step in range(2):
        x = (torch.randn(1, 6, d, generator=g) / math.sqrt(d)).cuda()
        tr.step(x, lambda out: torch.ones_like(out))
        torch.cuda.synchronize()
        after = [t.clone() for t in layer.p.tensors()]
        changed = [not torch.equal(a, b) for a, b in zip(before, after)]
        assert all(changed[:4 + 9]), "attention branch and level 0 update every step"
        if step == 0:
            assert any(changed[13:]), "level 1 fires at step 0"
        else:
            assert not any(changed[13:]), "level 1 is frozen at step 1: parameters untouched"
        before = after
    assert tr.opt.level_step(0) == 2 and tr.opt.level_step(1) == 1


def test_frozen_level_gradients_wait_in_the_error_buffer_and_are_applied_when_it_fires():
    """conductor.rs:224-261 with the loop of core/tests/test_cms.rs:66-84: level 1 (period 4, sequences
    shorter than that) is frozen on steps 1..3; its read path still produces a w_q gradient, which is
    summed in the level's ErrorBuffer and applied as one plain step of size lr when the level fires again."""
    d, nh, k = 32, 2, 2
    layer = MagLayer(d, nh, k, 4, [1, 4], rule="exact", chunk=2, seed=21)
    tr = MagTrainer(layer, lr=1e-2, max_grad_norm=0.0)   # no clip: the step's gradients stay as the backward wrote them
    g = torch.Generator().manual_seed(3)
    wq_idx = 2   # level tensors: w_k, w_v, w_q, ...
    sums = torch.zeros_like(layer.p.levels[1].w_q)
    for step in range(5):
        x = (torch.randn(1, 3, d, generator=g) / math.sqrt(d)).cuda()
        before = [t.clone() for t in layer.p.levels[1].tensors()]
        pulse = layer.conductor.pulse()
        out = tr.step(x, lambda o: torch.ones_like(o))
        torch.cuda.synchronize()
        eb = tr.error_buffers[1]
        if step == 0:
            assert pulse.active_levels[1] and eb.steps_accumulated == 0
        elif step < 4:
            assert not pulse.active_levels[1]
            assert eb.steps_accumulated == step
            sums += tr.grads.levels[1].w_q
            assert float(tr.grads.levels[1].w_q.abs().max()) > 0, "the frozen read carries a w_q gradient"
            assert torch.allclose(eb.grads[wq_idx], sums, rtol=1e-6, atol=1e-9)
            assert all(torch.equal(a, b) for a, b in zip(before, layer.p.levels[1].tensors())), "frozen: untouched"
            ratio = eb.health_check(tr.grads.levels[1].tensors())
            assert ratio is not None and 0.5 < ratio < 2.0 * step
        else:
            assert pulse.active_levels[1] and eb.steps_accumulated == 0 and not eb.grads[wq_idx].any()
    # the last step applied AdamW (gradients of step 4) and then the buffered sum: replay it by hand
    assert float(sums.abs().max()) > 0


def test_context_state_reset_zeroes_the_layer_memories_in_place():
    d, nh, k = 32, 2, 2
    layer = MagLayer(d, nh, k, 4, [1, 8], rule="exact", chunk=4, seed=22)
    x = (torch.randn(2, 6, d, generator=torch.Generator().manual_seed(2)) / math.sqrt(d)).cuda()
    layer.forward(x)
    cs = layer.context_state(2)
    ptrs = [t.data_ptr() for t in layer.m_state]
    assert any(float(t.abs().max()) > 0 for t in layer.m_state)
    step_before = layer.conductor.step()
    cs.reset()
    torch.cuda.synchronize()
    assert not any(t.any() for t in layer.m_state + layer.s_state)
    assert ptrs == [t.data_ptr() for t in layer.m_state] and layer.conductor.step() == step_before


def test_trainer_clamps_b_theta_after_every_level_update():
    """gpu_optimizer.rs:491-493: b_theta of an updated level is held in [-10, 2]."""
    d, nh, k = 32, 2, 2
    layer = MagLayer(d, nh, k, 4, [1, 8], rule="exact", chunk=4, seed=12)
    with torch.no_grad():
        layer.p.levels[0].b_theta.fill_(7.5)
        layer.p.levels[1].b_theta.fill_(-30.0)
    tr = MagTrainer(layer)
    x = (torch.randn(1, 6, d, generator=torch.Generator().manual_seed(1)) / math.sqrt(d)).cuda()
    tr.step(x, lambda out: torch.ones_like(out))
    torch.cuda.synchronize()
    assert float(layer.p.levels[0].b_theta.max()) <= 2.0
    assert float(layer.p.levels[1].b_theta.min()) >= -10.0
    for lp in layer.p.levels:   # the other biases are not clamped
        assert torch.isfinite(lp.b_alpha).all() and torch.isfinite(lp.b_eta).all()


def test_graph_replayed_steps_match_eager_steps():
    """Three training steps from a captured HIP graph (forward + backward replayed, optimizer eager)
    against three eager steps from the same start, with different inputs per step and eager work on
    the device between the replays; every replay is compared, not only the first."""
    import copy
    from nl_hecate_amd.mag_layer import MagLayer, MagTrainer
    bs, s, d, heads, k = 2, 128, 128, 2, 2
    torch.manual_seed(5)
    mk = lambda: MagLayer(d, heads, k, 64, [1, 2], rule="chunkwise", chunk=64, seed=11)
    eager, graphed = MagTrainer(mk()), MagTrainer(mk())
    xs = [torch.randn(bs, s, d, device="cuda") / d ** 0.5 for _ in range(3)]
    ds = [torch.randn(bs, s, d, device="cuda") for _ in range(3)]
    for step in range(3):
        print(f"mag layer graph replay step {step}", flush=True)
        out_e = eager.step(xs[step], lambda out: ds[step]).clone()
        out_g = graphed.step_graphed(xs[step], ds[step]).clone()
        torch.cuda.synchronize()
        scratch = torch.randn(1 << 20, device="cuda").sin().sum()   # unrelated eager work between replays
        torch.cuda.synchronize()
        assert torch.isfinite(scratch)
        assert torch.allclose(out_g, out_e, rtol=1e-5, atol=1e-6), (out_g - out_e).abs().max()
        for a, b in zip(graphed.layer.p.tensors(), eager.layer.p.tensors()):
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-7)
        for a, b in zip(graphed.layer.m_state, eager.layer.m_state):
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("frozen_second", [False, True])
def test_decode_steps_reproduce_the_full_sequence_forward(frozen_second):
    """Token-by-token decode with the KV cache (gpu_single_token_forward, gpu_forward.rs:3377 ff.) against one
    forward over the whole sequence, exact rule: the recurrence is sequential and the attention row of the
    newest token sees the same keys, so both give the same outputs and leave the same context memories.
    Projections differ in the last bits (split-bf16 GEMM vs fp32), which can flip a bf16 rounding of q/k/v:
    compared at the bf16 tolerance of the attention branch."""
    from nl_hecate_amd.cms import Pulse
    torch.manual_seed(3)
    d, heads, s, window = 128, 2, 40, 16
    mk = lambda: MagLayer(d, heads, 2, window, [1, 1], rule="exact", chunk=8, seed=21)
    full, dec = mk(), mk()
    x = torch.randn(1, s, d, device="cuda") / d ** 0.5
    pulse = Pulse(0, [True, not frozen_second])
    for layer in (full, dec):   # a non-trivial memory for the frozen level to read
        layer.ensure_state(1)
        layer.m_state[1].copy_(0.05 * torch.randn_like(layer.m_state[1]))
    dec.m_state[1].copy_(full.m_state[1])
    full.conductor.pulse = lambda: pulse
    out_full, _ = full.forward(x)
    dec.decode_reset(s)
    outs = [dec.decode_step(x[0, t], pulse) for t in range(s)]
    out_dec = torch.stack(outs)
    torch.cuda.synchronize()
    err = (out_dec - out_full[0]).abs().max().item() / out_full.abs().max().item()
    assert err < 2e-2, err
    for lv in range(2):
        m_err = (dec.m_state[lv] - full.m_state[lv]).abs().max().item()
        assert m_err <= 1e-4 * max(full.m_state[lv].abs().max().item(), 1e-6), (lv, m_err)


def test_failed_capture_restores_the_launch_stream_and_the_context_memories():
    """A warm-up that raises must not leave the library launching on the side stream, nor the context memories
    advanced: the next (eager) step then equals the step of a trainer that never tried to capture."""
    from nl_hecate_amd.mag_layer import MagLayer, MagTrainer
    bs, s, d, heads, k = 1, 64, 128, 2, 2
    mk = lambda: MagLayer(d, heads, k, 32, [1, 2], rule="chunkwise", chunk=32, seed=13)
    broken, plain = MagTrainer(mk()), MagTrainer(mk())
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(bs, s, d, generator=g) / d ** 0.5).cuda()
    d_out = torch.randn(bs, s, d, generator=g).cuda()
    real = broken._forward_backward

    def fails_after_the_forward(xs, ds):
        real(xs, ds)            # advances the context memories, as a warm-up does
        raise RuntimeError("scratch error during the warm-up")
    broken._forward_backward = fails_after_the_forward
    broken.layer.ensure_state(bs)
    before = [m.clone() for m in broken.layer.m_state]
    with pytest.raises(RuntimeError, match="warm-up"):
        broken.step_graphed(x, d_out)
    torch.cuda.synchronize()
    for a, b in zip(broken.layer.m_state, before):
        assert torch.equal(a, b), "the warm-up's memory updates were put back"
    broken._forward_backward = real
    out_b = broken.step(x, lambda o: d_out).clone()
    out_p = plain.step(x, lambda o: d_out).clone()
    torch.cuda.synchronize()
    assert torch.equal(out_b, out_p)
    for a, b in zip(broken.layer.p.tensors(), plain.layer.p.tensors()):
        assert torch.equal(a, b)
