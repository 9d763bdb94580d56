"""Conductor / Pulse host logic through the C ABI (no GPU needed): the
reference's truth tables (core/src/conductor.rs:268-300, 387-427) and the
bitmask cases of core/tests/test_cuda_graph.rs:137-200."""
import pytest

from nl_hecate_amd.cms import Conductor, Pulse, RestoreError
from oracle import pyoracle as orc


def test_k2_pulse_pattern_and_advance():
    c = Conductor(2, [1, 8])
    for step in range(17):
        p = c.pulse()
        assert p.global_step == step
        assert p.active_levels == [True, step % 8 == 0]
        assert c.pulse() == p, "pulse() does not advance"
        c.advance()
    assert c.step() == 17


def test_k4_pattern_matches_oracle_for_many_steps():
    cs = [1, 8, 64, 512]
    c = Conductor(4, cs)
    for step in range(1030):
        assert c.pulse().active_levels == orc.pulse(step, cs)
        c.advance()


def test_seq_len_keeps_levels_active():
    c = Conductor(4, [1, 8, 64, 512])
    c.set_seq_len(64)
    c.advance(); c.advance(); c.advance()
    assert c.pulse().active_levels == [True, True, True, False]
    c.set_seq_len(4096)
    assert c.pulse().active_levels == [True] * 4


def test_bitmask_cases():
    assert Pulse(0, [True, False, False, False]).bitmask() == 0b0001
    assert Pulse(0, [True, True, False, False]).bitmask() == 0b0011
    assert Pulse(0, [True, False, True, True]).bitmask() == 0b1101
    assert Pulse(0, [True] * 4).bitmask() == 0b1111
    c = Conductor(4, [1, 2, 4, 8])
    seen = set()
    for _ in range(16):
        seen.add(c.pulse().bitmask())
        c.advance()
    assert all(m & 1 for m in seen), "level 0 always fires: only odd masks are reachable"


def test_restore_checks_config_and_pulse_id():
    c = Conductor(2, [1, 8])
    c.restore(2, [1, 8], 40, 40)
    assert c.step() == 40
    with pytest.raises(RestoreError, match="ConfigMismatch"):
        c.restore(2, [1, 4], 40, 40)
    with pytest.raises(RestoreError, match="ConfigMismatch"):
        c.restore(3, [1, 8, 64], 40, 40)
    with pytest.raises(RestoreError, match="PulseMismatch"):
        c.restore(2, [1, 8], 40, 41)
    assert c.step() == 40


def test_constructor_validates():
    with pytest.raises(AssertionError):
        Conductor(2, [1])
    with pytest.raises(AssertionError):
        Conductor(1, [0])
