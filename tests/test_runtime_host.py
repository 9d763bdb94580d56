"""Host-side runtime logic that needs no GPU: the scratch-arena generation counter, the graph cache
that follows it, and error recording that does not leak from one call into the next."""
from nl_hecate_amd.ffi import lib
from nl_hecate_amd.mag_layer import GraphCache


def test_release_workspace_bumps_the_arena_generation():
    g0 = lib.nlh_workspace_generation()
    lib.nlh_release_workspace()
    g1 = lib.nlh_workspace_generation()
    lib.nlh_release_workspace()
    assert g1 > g0 and lib.nlh_workspace_generation() > g1


def test_graph_cache_drops_graphs_of_an_older_generation():
    gen = [7]
    c = GraphCache(lambda: gen[0])
    assert c.get("a") is None
    c.put("a", "graph-a")
    c.put("b", "graph-b")
    assert c.get("a") == "graph-a" and c.get("b") == "graph-b" and len(c) == 2
    gen[0] = 8                      # a slot was reallocated: every cached address is dead
    assert c.get("a") is None and c.get("b") is None and len(c) == 0
    c.put("a", "graph-a2")          # captured under generation 8
    assert c.get("a") == "graph-a2"
    gen[0] = 9                      # the capture's own warm-up grew a slot before put(): put() re-reads
    c.put("b", "graph-b2")
    assert c.get("a") is None and c.get("b") == "graph-b2"


def test_recorded_error_keeps_its_message_until_cleared_and_counts_per_call():
    lib.nlh_set_error_mode(1)
    try:
        lib.nlh_clear_error()
        assert lib.nlh_last_error() == b""
        lib.titans_backward_noalloc_f32_rocm(*([None] * 17), 8, 64, 100000, 0.0)
        first = lib.nlh_last_error()
        assert b"fixed buffer" in first
        # a later argument error replaces the message: the entry point ran its own checks
        lib.titans_backward_noalloc_f32_rocm(*([None] * 17), 8, 48, 2, 0.0)
        assert b"d=48" in lib.nlh_last_error()
        lib.nlh_clear_error()
        assert lib.nlh_last_error() == b""
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)
