"""Pins oracle/serving.py: decoding token by token over a growing cache gives the logits of one pass over the
whole sequence when the memory rule carries no state besides M (Delta rule, full trajectory) — the attention
row of the newest token sees the same keys and the recurrence is sequential either way."""
import types

import numpy as np
import pytest

from oracle import serving as SV
from tests.test_oracle_memory_level import cfg_of, params

f32 = np.float32


def model(d, v, k, seed):
    r = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: r.uniform(-lim, lim, (d, d)).astype(f32) for n in ("w_q", "w_k", "w_v", "w_o")}
    p["w_embed"] = (r.standard_normal((v, d)) / np.sqrt(d)).astype(f32)
    p["w_unembed"] = (r.standard_normal((d, v)) / np.sqrt(d)).astype(f32)
    p["levels"] = [params(d, seed + 10 + i, f32) for i in range(k)]
    return p


@pytest.mark.parametrize("k,active,n_persistent", [(1, [True], 0), (2, [True, False], 0), (3, [True, True, False], 2)])
def test_decode_steps_equal_the_whole_sequence(k, active, n_persistent):
    nh, hd, v, s, extra, window = 2, 4, 11, 9, 5, 4
    d = nh * hd
    p = model(d, v, k, 40 + k)
    cfg = types.SimpleNamespace(d_model=d, num_heads=nh, head_dim=hd, window_size=window, n_persistent=n_persistent,
                                levels=[cfg_of("delta", nh, hd) for _ in range(k)])
    r = np.random.default_rng(9)
    ids = r.integers(0, v, s + extra)
    mem0 = [(0.2 * r.standard_normal((nh, hd, hd))).astype(f32) for _ in range(k)]
    want, mem_all, _, _ = SV.forward_all(p, cfg, ids, active, mem0)
    logits, mem, kc, vc = SV.forward_all(p, cfg, ids[:s], active, mem0)
    assert np.allclose(logits, want[:s], rtol=1e-5, atol=1e-6)
    for i in range(extra):
        step, mem, kc, vc = SV.single_token(p, cfg, int(ids[s + i]), active, mem, kc, vc)
        assert np.allclose(step, want[s + i], rtol=2e-2, atol=2e-3 * np.abs(want).max()), i
    for a, b in zip(mem, mem_all):
        assert np.allclose(a, b, rtol=1e-4, atol=1e-6)


def test_frozen_mlp_memory_levels_contribute_zeros_or_are_refused():
    """gpu_forward.rs:32-57: a frozen MONETA / YAAD level adds nothing (the model answers as if the level were not
    there, up to the 1 / sqrt(k) scaling that only k > 2 applies); a frozen two-layer Titans memory is an error."""
    nh, hd, v, s, window = 2, 4, 11, 7, 4
    d = nh * hd
    p = model(d, v, 2, 51)
    r = np.random.default_rng(3)
    ids = r.integers(0, v, s)
    mem0 = [(0.2 * r.standard_normal((nh, hd, hd))).astype(f32), r.standard_normal(64).astype(f32)]
    mk = lambda levels: types.SimpleNamespace(d_model=d, num_heads=nh, head_dim=hd, window_size=window, n_persistent=0,
                                               levels=levels)
    moneta = types.SimpleNamespace(memory_rule="moneta", memory_layers=1)
    with_frozen, _, _, _ = SV.forward_all(p, mk([cfg_of("delta", nh, hd), moneta]), ids, [True, False], mem0)
    p1 = dict(p, levels=p["levels"][:1])
    alone, _, _, _ = SV.forward_all(p1, mk([cfg_of("delta", nh, hd)]), ids, [True], mem0[:1])
    assert np.array_equal(with_frozen, alone)
    mlp = types.SimpleNamespace(memory_rule="titans", memory_layers=2)
    with pytest.raises(RuntimeError):
        SV.forward_all(p, mk([cfg_of("delta", nh, hd), mlp]), ids, [True, False], mem0)
