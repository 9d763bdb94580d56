"""Seeded sweeps over shapes that the hand-picked cases of the other GPU tests do not list: every entry-point
family of the memory path against the CPU oracle at lengths, chunk sizes, windows and batch sizes drawn from a
fixed random stream (ragged last chunks, chunk sizes that are no power of two, windows around the kernels' stage
sizes, more chains than compute units' worth of one size class).  The comparisons and tolerances are those of the
tests whose helpers are used; a gradient that is exactly zero in the oracle (one key in the window) is compared
absolutely."""
import random

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests import test_gpu_chunkwise_mm as cw
from tests import test_gpu_hebbian as heb
from tests import test_gpu_memory_rules as rules
from tests import test_gpu_swa as swa
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros, REL_TOL_BF16

pytestmark = pytest.mark.gpu

CHUNKS = [1, 2, 3, 5, 8, 13, 16, 17, 31, 32, 33, 47, 48, 63, 64]


def _chunked_shape(rnd):
    C = rnd.choice(CHUNKS)
    s = max(4, C * rnd.randint(1, 9) - rnd.choice([0, 0, 1, C // 2, C - 1]))
    return rnd.choice([1, 2, 3, 5, 8, 17]), s, C


@pytest.mark.parametrize("seed", [11, 12])
def test_titans_chunkwise_pair(seed):
    rnd = random.Random(seed)
    for it in range(25):
        B, s, C = _chunked_shape(rnd)
        bf16 = rnd.random() < 0.8
        print(f"titans chunkwise seed={seed} case={it} B={B} s={s} C={C} bf16={bf16}", flush=True)
        cw.test_forward_matches_oracle(B, s, C, bf16)
        cw.test_backward_matches_oracle(B, s, C, bf16)


def test_delta_chunkwise_pair():
    rnd = random.Random(21)
    for it in range(25):
        B, s, C = _chunked_shape(rnd)
        bf16 = rnd.random() < 0.8
        cw.test_delta_matrix_form_matches_oracle(B, s, C, bf16)


def _close_or_zero(name, got, want, tol):
    if np.abs(want).max() < 1e-12:
        assert np.abs(got).max() < 1e-4, f"{name}: expected zero, got {np.abs(got).max():.3e}"
    else:
        assert_close(name, got, want, tol)


def test_sliding_window_attention_pairs():
    rnd = random.Random(31)
    hd = 64
    for it in range(40):
        H, B = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 3])
        s = rnd.choice([3, 15, 16, 17, 63, 64, 65, 127, 128, 129, 191, 200, 255, 256, 257, 383, 400, 513, 640, 700])
        ws = rnd.choice([1, 2, 3, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 448,
                         511, 512])
        print(f"swa case={it} B={B} s={s} H={H} ws={ws}", flush=True)
        q, k, v, go = swa._case(B, s, H, hd, 5000 + it)
        out_w, aw = swa.gpu_forward(q, k, v, ws, H, 0)
        oo, awo = orc.swa_forward(q, k, v, ws, H, 0)
        assert_close("out (weights stored)", orc.bf16_to_f32(out_w), orc.bf16_to_f32(oo), REL_TOL_BF16)
        w, wo = orc.bf16_to_f32(aw), orc.bf16_to_f32(awo)
        assert np.abs(w - wo).max() < 1e-2
        assert np.all(w[wo == 0] == 0)
        oq, ok, ov = orc.swa_backward(q, k, v, awo, go, ws, H, 0)
        dq, dk, dv = swa.gpu_backward(q, k, v, awo, go, ws, H, 0)
        for n, a, b in (("d_q", dq, oq), ("d_k", dk, ok), ("d_v", dv, ov)):
            _close_or_zero(n + " (weights stored)", a, b, 3e-4)
        out = torch.zeros(B, s, H * hd, dtype=torch.uint16, device="cuda")
        stats = torch.full((B, H, s, 2), float("nan"), device="cuda")
        D.call("swa_forward_lse_bf16_rocm", swa._u16(q), swa._u16(k), swa._u16(v), out, stats, s, H, hd, ws, B)
        gq, gk, gv = zeros(B, s, H * hd), zeros(B, s, H * hd), zeros(B, s, H * hd)
        D.call("swa_backward_lse_bf16_rocm", swa._u16(q), swa._u16(k), swa._u16(v), stats, dev(go), gq, gk, gv,
               s, H, hd, ws, B)
        torch.cuda.synchronize()
        assert_close("out (statistics)", orc.bf16_to_f32(out.cpu().numpy()), orc.bf16_to_f32(oo), REL_TOL_BF16)
        assert np.isfinite(host(stats)).all()
        for n, a, b in (("d_q", gq, oq), ("d_k", gk, ok), ("d_v", gv, ov)):
            _close_or_zero(n + " (statistics)", host(a), b, REL_TOL_BF16)


def test_hebbian_forward_and_segment_backward():
    rnd = random.Random(41)
    for it in range(30):
        d = rnd.choice([8, 16, 32, 64, 64, 64, 128, 12, 24])
        B = rnd.choice([1, 2, 3, 7, 20])
        s = rnd.choice([1, 2, 7, 8, 9, 63, 64, 65, 127, 128, 129, 130, 191, 192, 193, 300, 511])
        s = min(s, 130) if d == 128 else s
        print(f"hebbian case={it} B={B} s={s} d={d}", flush=True)
        x = rule_inputs(B, s, d, 7000 + it, m0_scale=0.3)
        y, ms = heb.gpu_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
        yo, mo = heb.oracle_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
        assert_close("y", y, yo)
        assert_close("m_states", ms, mo)
        seed = 0.1 * np.random.default_rng(5).standard_normal((B, d, d)).astype(np.float32)
        g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s), d_m=zeros(B, d, d))
        D.hebbian_backward_dd_segment(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(mo), dev(x["dy"]),
                                      dev(seed), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_m"], 0, s, d, B, s)
        torch.cuda.synchronize()
        for b in range(B):
            want = orc.hebbian_backward(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], mo[b], x["dy"][b],
                                        d_m_seed=seed[b])
            for n in want:
                assert_close(f"{n}[{b}]", host(g[n])[b], want[n])


def test_exact_rules_full_and_checkpointed():
    rnd = random.Random(51)
    for it in range(40):
        d = rnd.choice([8, 16, 32, 64, 64, 64, 128, 4, 12, 24, 48])
        B = rnd.choice([1, 2, 3, 7, 33, 70])
        s = rnd.choice([1, 2, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 129, 200])
        if d == 128:
            s, B = min(s, 65), min(B, 7)
        C = rnd.choice([1, 2, 5, 8, 16, 33, 64, 64, 64, 100, 200])
        entry = rnd.choice(["", "_replay"])
        print(f"exact rules case={it} B={B} s={s} d={d} C={C} entry={entry!r}", flush=True)
        x = rule_inputs(B, s, d, 9000 + it, m0_scale=0.2)
        if it % 2 == 0:
            y, ms, ss = rules.gpu_titans_forward(x)
            yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                                  x["m0"], x["s0"])
            assert_close("y", y, yo)
            assert_close("m_states", ms, mo)
            assert_close("s_states", ss, so)
            g = rules.gpu_titans_backward(x, mo, so)
            go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], mo, so, x["dy"])
            for n in go:
                assert_close(n, g[n], go[n])
        else:
            for has_s in (True, False):
                g = rules._gpu_ckpt_fwd_bwd(x, C, has_s, entry)
                go = rules._oracle_ckpt_grads(x, C, has_s)
                for n in g:
                    assert_close(f"{n} has_s={has_s}", g[n], go[n])


def test_layer_steps_against_the_autograd_reference():
    """Whole layer steps (levels, gate, attention branch, projections) at drawn configurations against the float64
    autograd model of tests/torch_mag_reference.py, tolerance and bias scaling as in tests/test_gpu_mag_layer.py."""
    from tests import test_gpu_mag_layer as layer
    rnd = random.Random(61)
    for it in range(14):
        rule = rnd.choice(["exact", "chunkwise", "chunkwise"])
        nh = rnd.choice([1, 2, 3])
        hd = 64 if rule == "chunkwise" else rnd.choice([16, 32, 64])
        k = rnd.choice([1, 2, 3, 4])
        periods = ([1, 2, 4, 8] if rnd.random() < 0.5 else [1, 8, 64, 512])[:k]
        bs, s = rnd.choice([1, 2, 3]), rnd.choice([5, 16, 33, 64, 70, 100, 129])
        window = rnd.choice([4, 8, 32, 50, 64, 128])   # one key in the window makes d_w_q exactly zero: not drawn
        chunk = rnd.choice([4, 8, 16, 32, 64]) if rule == "chunkwise" else rnd.choice([4, 8, 16, 64])
        steps = rnd.choice([1, 1, 2, 3])
        print(f"layer case={it} bs={bs} s={s} d={nh * hd} nh={nh} k={k} window={window} periods={periods} rule={rule} "
              f"chunk={chunk} steps={steps}", flush=True)
        w = layer.run_case(bs=bs, s=s, d=nh * hd, nh=nh, k=k, window=window, periods=periods, rule=rule, chunk=chunk,
                           seed=100 + it, steps=steps, bias_scale=True)
        assert max(w.values()) < 2e-2, {n: f"{e:.1e}" for n, e in w.items() if e > 5e-3}
